// Host-side planner entry points: diagnose() reports and a replay of the
// thread -> byte assignment of every object, run with the same GridState /
// HaloGeom code the device uses.
#include "common.hpp"
#include "../../include/hipDMA.h"

namespace {

struct MapWriter {
  int* map;               // NULL: only the extents are recorded
  size_t len;
  long long src_origin, dst_origin;
  int doubles;
  bool out_of_range;
  bool any = false;
  long long src_min = 0, src_end = 0, dst_min = 0, dst_end = 0;
  void move(long long src_off, long long dst_off, int nbytes)
  {
    if (nbytes <= 0) return;
    if (!any) { src_min = src_off; src_end = src_off + nbytes; dst_min = dst_off; dst_end = dst_off + nbytes; any = true; }
    if (src_off < src_min) src_min = src_off;
    if (src_off + nbytes > src_end) src_end = src_off + nbytes;
    if (dst_off < dst_min) dst_min = dst_off;
    if (dst_off + nbytes > dst_end) dst_end = dst_off + nbytes;
    if (map == nullptr) return;
    for (int b = 0; b < nbytes; ++b) {
      const long long d = dst_origin + dst_off + b;
      if (d < 0 || (size_t)d >= len) { out_of_range = true; return; }
      if (map[d] != -1) ++doubles;
      map[d] = (int)(src_origin + src_off + b);
    }
  }
};

int replay_sequential(const cudadma_plan_query_t& q, MapWriter& w, int* steps)
{
  const int a = q.alignment, t = q.dma_threads, max_lds = q.bytes_per_thread / a;
  const hipdma::SequentialPlan p(a, q.bytes_per_thread, q.bytes_per_elmt, t);
  for (int tid = 0; tid < t; ++tid)
    for (int step = 0; step < p.total_steps; ++step)
      for (int k = 0; k < max_lds; ++k) {
        const int off = hipdma::SequentialPlan::chunk_offset(a, max_lds, t, tid, step, k);
        const int rem = q.bytes_per_elmt - off;
        if (step < p.full_steps || rem >= a) w.move(off, off, a);
        else if (rem > 0) w.move(off, off, rem);
      }
  *steps = p.total_steps;
  return 0;
}

int replay_grid(const cudadma_plan_query_t& q, MapWriter& w, int* steps)
{
  const int a = q.alignment, max_lds = q.bytes_per_thread / a;
  const bool gather = q.pattern == CUDADMA_PATTERN_GATHER, scatter = q.pattern == CUDADMA_PATTERN_SCATTER;
  const int e = q.bytes_per_elmt;
  for (int tid = 0; tid < q.dma_threads; ++tid) {
    hipdma::detail::GridState g;
    g.init(a, max_lds, e, q.num_elmts, q.dma_threads, tid);
    hipdma::detail::GridCursor c = g.begin();
    for (int r = 0; r < g.steps * max_lds; ++r) {
      if (g.live(r, c)) {
        if (c.row < 0 || c.row >= q.num_elmts || c.col < 0 || c.col >= g.LPE) return CUDADMA_ERANGE;
        long long so, dd;
        if (gather) {
          const int dense = q.dst_stride > e ? q.dst_stride : e;
          so = (long long)q.index[c.row] * e + c.col * a;
          dd = (long long)c.row * dense + c.col * a;
        } else if (scatter) {
          const int dense = q.src_stride > e ? q.src_stride : e;
          so = (long long)c.row * dense + c.col * a;
          dd = (long long)q.index[c.row] * e + c.col * a;
        } else {
          so = (long long)c.row * q.src_stride + c.col * a;
          dd = (long long)c.row * q.dst_stride + c.col * a;
        }
        w.move(so, dd, g.chunk_bytes(a, c));
      }
      g.advance(c);
    }
    *steps = g.steps;
  }
  return 0;
}

template<int A, int ES, int R, bool C>
int replay_halo_t(const cudadma_plan_query_t& q, MapWriter& w, int* steps)
{
  if ((2 * R * ES) % A != 0) return CUDADMA_EINVAL;
  hipdma::detail::HaloGeom<A, ES, R, C> g;
  g.init(q.dimx, q.dimy, q.pitch, q.dst_pitch);
  const int max_lds = q.bytes_per_thread / A;
  const int nsteps = hipdma::detail::ceil_div(hipdma::detail::ceil_div(g.total, q.dma_threads), max_lds);
  for (int tid = 0; tid < q.dma_threads; ++tid)
    for (int r = 0; r < nsteps * max_lds; ++r) {
      const hipdma::detail::HaloSlot s = g.decode(tid + r * q.dma_threads);
      if (s.live) w.move(s.src_off, s.dst_off, s.nbytes);
    }
  *steps = nsteps;
  return 0;
}

template<int A, int ES, int R>
int replay_halo_c(const cudadma_plan_query_t& q, MapWriter& w, int* steps)
{ return q.corners ? replay_halo_t<A, ES, R, true>(q, w, steps) : replay_halo_t<A, ES, R, false>(q, w, steps); }

template<int A, int ES>
int replay_halo_r(const cudadma_plan_query_t& q, MapWriter& w, int* steps)
{
  switch (q.radius) {
    case 1: return replay_halo_c<A, ES, 1>(q, w, steps);
    case 2: return replay_halo_c<A, ES, 2>(q, w, steps);
    case 3: return replay_halo_c<A, ES, 3>(q, w, steps);
    case 4: return replay_halo_c<A, ES, 4>(q, w, steps);
    case 5: return replay_halo_c<A, ES, 5>(q, w, steps);
    case 6: return replay_halo_c<A, ES, 6>(q, w, steps);
    case 7: return replay_halo_c<A, ES, 7>(q, w, steps);
    case 8: return replay_halo_c<A, ES, 8>(q, w, steps);
    default: return CUDADMA_EINVAL;
  }
}

template<int A>
int replay_halo_es(const cudadma_plan_query_t& q, MapWriter& w, int* steps)
{
  switch (q.bytes_per_elmt) {
    case 4: return replay_halo_r<A, 4>(q, w, steps);
    case 8: return replay_halo_r<A, 8>(q, w, steps);
    case 16: return replay_halo_r<A, 16>(q, w, steps);
    default: return CUDADMA_EINVAL;
  }
}

}  // namespace

// Replays the query into `w`; shared by cudadma_plan_map and cudadma_plan_extents.
static int replay(const cudadma_plan_query_t* q, MapWriter& w, int* steps_out)
{
  CUDADMA_REQUIRE(q->alignment == 4 || q->alignment == 8 || q->alignment == 16, "ALIGNMENT must be 4, 8 or 16");
  CUDADMA_REQUIRE(q->bytes_per_thread >= q->alignment && (q->bytes_per_thread % q->alignment) == 0,
                  "BYTES_PER_THREAD must be a positive multiple of ALIGNMENT");
  CUDADMA_REQUIRE(q->dma_threads > 0, "DMA_THREADS must be positive");
  CUDADMA_REQUIRE(q->bytes_per_elmt >= 0 && (q->bytes_per_elmt % 4) == 0, "sizes are multiples of 4 bytes");
  if (q->pattern == CUDADMA_PATTERN_HALO)
    CUDADMA_REQUIRE(q->dimx > 0 && q->dimy > 0 && q->pitch >= q->dimx + 2 * q->radius &&
                    (q->dst_pitch == 0 || q->dst_pitch >= q->dimx + 2 * q->radius),
                    "halo: dimx, dimy positive, both pitches at least dimx + 2*radius");
  int steps = 0, rc = 0;
  switch (q->pattern) {
    case CUDADMA_PATTERN_SEQUENTIAL: rc = replay_sequential(*q, w, &steps); break;
    case CUDADMA_PATTERN_GATHER:
    case CUDADMA_PATTERN_SCATTER:
      CUDADMA_REQUIRE(q->index != nullptr, "gather / scatter need index");
      /* fall through */
    case CUDADMA_PATTERN_STRIDED: rc = replay_grid(*q, w, &steps); break;
    case CUDADMA_PATTERN_HALO:
      rc = q->alignment == 4 ? replay_halo_es<4>(*q, w, &steps)
         : q->alignment == 8 ? replay_halo_es<8>(*q, w, &steps) : replay_halo_es<16>(*q, w, &steps);
      break;
    default: rc = CUDADMA_EINVAL; break;
  }
  if (rc != 0) {
    cudadma_host::set_error("plan replay rejected the query (pattern %d)", q->pattern);
    return rc;
  }
  if (steps_out != nullptr) *steps_out = steps;
  return CUDADMA_OK;
}

extern "C" int cudadma_plan_map(const cudadma_plan_query_t* q, long long src_origin, long long dst_origin,
                                int* map, size_t map_len, int* steps_out)
{
  CUDADMA_REQUIRE(q != nullptr && map != nullptr, "NULL argument");
  for (size_t i = 0; i < map_len; ++i) map[i] = -1;
  MapWriter w{map, map_len, src_origin, dst_origin, 0, false};
  const int rc = replay(q, w, steps_out);
  if (rc != 0) return rc;
  if (w.out_of_range) {
    cudadma_host::set_error("plan replay: a thread steps outside the %zu-byte destination window", map_len);
    return CUDADMA_ERANGE;
  }
  return w.doubles;
}

extern "C" int cudadma_plan_extents(const cudadma_plan_query_t* q, long long extents[4])
{
  CUDADMA_REQUIRE(q != nullptr && extents != nullptr, "NULL argument");
  MapWriter w{nullptr, 0, 0, 0, 0, false};
  const int rc = replay(q, w, nullptr);
  if (rc != 0) return rc;
  extents[0] = w.src_min; extents[1] = w.src_end; extents[2] = w.dst_min; extents[3] = w.dst_end;
  return CUDADMA_OK;
}

extern "C" int cudadma_diagnose(int pattern, int alignment, int bytes_per_thread, int bytes_per_elmt,
                                int dma_threads, int num_elmts, int full_template, int verbose)
{
  CUDADMA_REQUIRE(alignment == 4 || alignment == 8 || alignment == 16, "ALIGNMENT must be 4, 8 or 16");
  CUDADMA_REQUIRE(bytes_per_thread >= alignment && dma_threads > 0, "bad BYTES_PER_THREAD / DMA_THREADS");
  switch (pattern) {
    case CUDADMA_PATTERN_SEQUENTIAL:
      CudaDMASequential<true, 0, 0, 0, 0>::diagnose(alignment, bytes_per_thread, bytes_per_elmt, dma_threads,
                                                     full_template != 0, verbose != 0);
      return CUDADMA_OK;
    case CUDADMA_PATTERN_STRIDED:
      CudaDMAStrided<true, 0, 0, 0, 0, 0>::diagnose(alignment, bytes_per_thread, bytes_per_elmt, dma_threads,
                                                     num_elmts, full_template != 0, verbose != 0);
      return CUDADMA_OK;
    case CUDADMA_PATTERN_GATHER:
      CudaDMAIndirect<true, true, 0, 0, 0, 0, 0>::diagnose(alignment, bytes_per_thread, bytes_per_elmt, dma_threads,
                                                            num_elmts, full_template != 0, verbose != 0);
      return CUDADMA_OK;
    case CUDADMA_PATTERN_SCATTER:
      CudaDMAIndirect<false, true, 0, 0, 0, 0, 0>::diagnose(alignment, bytes_per_thread, bytes_per_elmt, dma_threads,
                                                             num_elmts, full_template != 0, verbose != 0);
      return CUDADMA_OK;
    default:
      cudadma_host::set_error("no diagnose() for pattern %d", pattern);
      return CUDADMA_EINVAL;
  }
}
