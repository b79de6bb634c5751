// Case registry and C entry points of the known-answer harness.
#include "harness.hpp"
#include <algorithm>
#include <vector>

namespace harness {

static std::vector<Entry>& registry()
{
  static std::vector<Entry> r;
  return r;
}

// Called from static initialisers only (the Registrar objects), before any entry point can run.
void register_case(const cudadma_case_t& desc, launch_fn fn, int order)
{
  registry().push_back(Entry{desc, fn, order});
}

// Static initialisers of different translation units run in no fixed order:
// give the cases a stable numbering (pattern, then order of appearance in its list).
// Sorted once, on the first call of an entry point (the initialisation of a local static
// is thread-safe); the registry does not change afterwards.
static const std::vector<Entry>& sorted()
{
  static const bool once = [] {
    std::vector<Entry>& r = registry();
    std::stable_sort(r.begin(), r.end(), [](const Entry& x, const Entry& y) {
      if (x.desc.pattern != y.desc.pattern) return x.desc.pattern < y.desc.pattern;
      return x.order < y.order;
    });
    return true;
  }();
  (void)once;
  return registry();
}

}  // namespace harness

extern "C" int cudadma_num_cases(void) { return (int)harness::sorted().size(); }

extern "C" int cudadma_get_case(int case_id, cudadma_case_t* out)
{
  const auto& r = harness::sorted();
  if (case_id < 0 || case_id >= (int)r.size() || out == nullptr) {
    cudadma_host::set_error("case %d out of range [0,%d)", case_id, (int)r.size());
    return CUDADMA_ERANGE;
  }
  *out = r[case_id].desc;
  return CUDADMA_OK;
}

extern "C" int cudadma_run_case(int case_id, const cudadma_run_t* run, void* stream)
{
  const auto& r = harness::sorted();
  if (case_id < 0 || case_id >= (int)r.size()) {
    cudadma_host::set_error("case %d out of range [0,%d)", case_id, (int)r.size());
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(run != nullptr, "run is NULL");
  // the case as it runs: the compiled description with the run-time values of this call
  cudadma_case_t d = r[case_id].desc;
  {
    const bool halo = d.pattern == CUDADMA_PATTERN_HALO;
    const bool rows = d.pattern == CUDADMA_PATTERN_STRIDED || d.pattern == CUDADMA_PATTERN_GATHER ||
                      d.pattern == CUDADMA_PATTERN_SCATTER;
    if (run->rt_bytes_per_elmt != 0) {
      CUDADMA_REQUIRE(!halo && d.level == 1, "bytes_per_elmt is a compile-time parameter of case %d", case_id);
      CUDADMA_REQUIRE(run->rt_bytes_per_elmt > 0 && (run->rt_bytes_per_elmt % 4) == 0,
                      "rt_bytes_per_elmt %d must be a positive multiple of 4", run->rt_bytes_per_elmt);
      d.bytes_per_elmt = run->rt_bytes_per_elmt;
    }
    if (run->rt_dma_threads != 0) {
      CUDADMA_REQUIRE(halo ? d.level <= 1 : d.level <= 2, "dma_threads is a compile-time parameter of case %d", case_id);
      CUDADMA_REQUIRE(run->rt_dma_threads > 0 && (run->rt_dma_threads % 64) == 0 &&
                      run->rt_dma_threads + (d.warp_specialized ? harness::kComputeThreads : 0) <= 1024,
                      "rt_dma_threads %d must be a multiple of 64 that fits a workgroup of 1024", run->rt_dma_threads);
      d.dma_threads = run->rt_dma_threads;
    }
    if (run->rt_num_elmts != 0) {
      CUDADMA_REQUIRE(rows && d.level <= 3, "num_elmts is not a run-time parameter of case %d", case_id);
      CUDADMA_REQUIRE(run->rt_num_elmts > 0, "rt_num_elmts must be positive");
      d.num_elmts = run->rt_num_elmts;
    }
    if (run->rt_dimx != 0 || run->rt_dimy != 0) {
      CUDADMA_REQUIRE(halo && d.level <= 2, "dimx / dimy are not run-time parameters of case %d", case_id);
      CUDADMA_REQUIRE(run->rt_dimx >= 0 && run->rt_dimy >= 0, "rt_dimx / rt_dimy must not be negative");
      if (run->rt_dimx != 0) d.dimx = run->rt_dimx;
      if (run->rt_dimy != 0) d.dimy = run->rt_dimy;
    }
  }
  CUDADMA_REQUIRE(run->d_in != nullptr && run->d_out != nullptr, "d_in / d_out must not be NULL");
  CUDADMA_REQUIRE(run->lds_bytes > 0 && run->lds_bytes <= 64 * 1024 - 256 && (run->lds_bytes % 16) == 0,
                  "lds_bytes %d must be a positive multiple of 16 below 64 KiB", run->lds_bytes);
  CUDADMA_REQUIRE(run->reps >= 1, "reps must be >= 1");
  CUDADMA_REQUIRE(run->call_style >= CUDADMA_CALL_UNQUALIFIED && run->call_style <= CUDADMA_CALL_LDS_DIRECT_SWIZZLE,
                  "unknown call_style %d", run->call_style);
  const bool swizzled = run->call_style == CUDADMA_CALL_LDS_SWIZZLE || run->call_style == CUDADMA_CALL_LDS_DIRECT_SWIZZLE;
  const bool direct = run->call_style == CUDADMA_CALL_LDS_DIRECT || run->call_style == CUDADMA_CALL_LDS_DIRECT_SWIZZLE;
  if (swizzled) {
    CUDADMA_REQUIRE(d.pattern == CUDADMA_PATTERN_STRIDED, "swizzled LDS rows are a CudaDMAStrided layout");
    CUDADMA_REQUIRE((d.bytes_per_elmt % d.alignment) == 0, "swizzled rows must be whole chunks (%d bytes per row, chunks of %d)",
                    d.bytes_per_elmt, d.alignment);
  }
  if (d.pattern == CUDADMA_PATTERN_HALO) {
    // the origins, not the buffer starts, carry the alignment
    const int src_origin = run->src_offset_bytes + (d.radius * run->pitch + d.radius) * d.bytes_per_elmt;
    const int dst_origin = run->dst_offset_bytes + (d.radius * (d.dimx + 2 * d.radius) + d.radius) * d.bytes_per_elmt;
    CUDADMA_REQUIRE((src_origin % d.alignment) == 0 && (dst_origin % d.alignment) == 0 &&
                    ((run->pitch * d.bytes_per_elmt) % d.alignment) == 0 && (run->rep_src_bytes % d.alignment) == 0,
                    "halo origins and pitch must keep the ALIGNMENT (%d) the case was compiled for", d.alignment);
    CUDADMA_REQUIRE(run->pitch >= d.dimx + 2 * d.radius, "pitch %d is narrower than the padded tile", run->pitch);
  } else {
    CUDADMA_REQUIRE((run->src_offset_bytes % d.alignment) == 0 && (run->dst_offset_bytes % d.alignment) == 0 &&
                    (run->rep_src_bytes % d.alignment) == 0,
                    "offsets must keep the ALIGNMENT (%d) the case was compiled for", d.alignment);
  }
  CUDADMA_REQUIRE(cudadma_host::aligned_to(run->d_in, 16) && cudadma_host::aligned_to(run->d_out, 16),
                  "d_in and d_out must be 16-byte aligned");
  if (d.pattern == CUDADMA_PATTERN_GATHER || d.pattern == CUDADMA_PATTERN_SCATTER)
    CUDADMA_REQUIRE(run->d_index != nullptr, "gather / scatter need d_index");
  if (d.pattern == CUDADMA_PATTERN_STRIDED)
    CUDADMA_REQUIRE((run->src_stride % d.alignment) == 0 && (run->dst_stride % d.alignment) == 0,
                    "strides must be multiples of ALIGNMENT");
  if (d.pattern == CUDADMA_PATTERN_HALO)
    CUDADMA_REQUIRE(!direct, "the halo object has no direct path");
  if (d.pattern == CUDADMA_PATTERN_SCATTER)
    CUDADMA_REQUIRE(!direct, "scatter has no direct path");
  if (direct)
    CUDADMA_REQUIRE(d.alignment == 16 || d.alignment == 4, "the direct path moves 4 or 16 bytes per lane");
  if (run->reverse) {
    CUDADMA_REQUIRE(run->call_style == CUDADMA_CALL_UNQUALIFIED,
                    "LDS -> global transfers go through the unqualified (generic-pointer) calls");
    CUDADMA_REQUIRE(run->out_bytes > 0 && (run->out_bytes % 16) == 0, "out_bytes must be a positive multiple of 16");
    CUDADMA_REQUIRE((run->rep_src_bytes % 4) == 0, "rep_src_bytes must be a multiple of 4");
  }

  harness::Args a;
  a.in = (const char*)run->d_in;
  a.out = (char*)run->d_out;
  a.index = run->d_index;
  a.lds_bytes = run->lds_bytes;
  a.src_offset = run->src_offset_bytes;
  a.dst_offset = run->dst_offset_bytes;
  a.src_stride = run->src_stride;
  a.dst_stride = run->dst_stride;
  a.pitch = run->pitch;
  a.call_style = run->call_style;
  a.two_phase = run->two_phase;
  a.reps = run->reps;
  a.rep_src_bytes = run->rep_src_bytes;
  a.rep_index_elmts = run->rep_index_elmts;
  a.reverse = run->reverse ? 1 : 0;
  a.out_bytes = run->out_bytes;
  a.bytes_per_elmt = d.bytes_per_elmt;
  a.dma_threads = d.dma_threads;
  a.num_elmts = d.num_elmts;
  a.dimx = d.dimx;
  a.dimy = d.dimy;
  return r[case_id].launch(a, (hipStream_t)stream);
}
