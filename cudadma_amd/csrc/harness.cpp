// Case registry and C entry points of the known-answer harness.
#include "harness.hpp"
#include <algorithm>
#include <vector>

extern "C" int cudadma_plan_extents(const cudadma_plan_query_t* q, long long extents[4]);

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
  CUDADMA_REQUIRE(run->call_style >= CUDADMA_CALL_UNQUALIFIED && run->call_style < CUDADMA_CALL_STYLES,
                  "unknown call_style %d", run->call_style);
  const bool swizzled = run->call_style == CUDADMA_CALL_LDS_SWIZZLE || run->call_style == CUDADMA_CALL_LDS_DIRECT_SWIZZLE;
  const bool direct = run->call_style == CUDADMA_CALL_LDS_DIRECT || run->call_style == CUDADMA_CALL_LDS_DIRECT_SWIZZLE ||
                      run->call_style == CUDADMA_CALL_LDS_DIRECT_SC1 || run->call_style == CUDADMA_CALL_LDS_DIRECT_NT;
  if (run->call_style == CUDADMA_CALL_INDEX_AHEAD)
    CUDADMA_REQUIRE(d.pattern == CUDADMA_PATTERN_GATHER || d.pattern == CUDADMA_PATTERN_SCATTER,
                    "the index-ahead call style belongs to the gather and scatter cases");
  const bool generic_source = run->call_style == CUDADMA_CALL_UNQUALIFIED || run->call_style == CUDADMA_CALL_INDEX_AHEAD ||
                              (run->call_style >= CUDADMA_CALL_QG_GLOBAL_CS && run->call_style <= CUDADMA_CALL_QG_VOLATILE_WB);
  if (swizzled) {
    CUDADMA_REQUIRE(d.pattern == CUDADMA_PATTERN_STRIDED, "swizzled LDS rows are a CudaDMAStrided layout");
    CUDADMA_REQUIRE((d.bytes_per_elmt % d.alignment) == 0, "swizzled rows must be whole chunks (%d bytes per row, chunks of %d)",
                    d.bytes_per_elmt, d.alignment);
  }
  const int halo_dst_pitch = run->dst_pitch > 0 ? run->dst_pitch : d.dimx + 2 * d.radius;
  if (d.pattern == CUDADMA_PATTERN_HALO) {
    CUDADMA_REQUIRE(run->dst_pitch >= 0 && halo_dst_pitch >= d.dimx + 2 * d.radius &&
                    ((halo_dst_pitch * d.bytes_per_elmt) % d.alignment) == 0,
                    "dst_pitch %d must be at least dimx + 2*radius cells and a multiple of ALIGNMENT in bytes", run->dst_pitch);
    // the origins, not the buffer starts, carry the alignment
    const int src_origin = run->src_offset_bytes + (d.radius * run->pitch + d.radius) * d.bytes_per_elmt;
    const int dst_origin = run->dst_offset_bytes + (d.radius * halo_dst_pitch + d.radius) * d.bytes_per_elmt;
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
  if (d.pattern == CUDADMA_PATTERN_HALO) {
    CUDADMA_REQUIRE(!direct, "the halo object has no direct path");
    CUDADMA_REQUIRE(run->dst_pitch == 0 || d.level >= 1, "the older cudaDMAHalo interface has no destination pitch");
  } else {
    CUDADMA_REQUIRE(run->dst_pitch == 0, "dst_pitch is a halo parameter");
  }
  if (d.pattern == CUDADMA_PATTERN_SCATTER)
    CUDADMA_REQUIRE(!direct, "scatter has no direct path");
  if (direct)
    CUDADMA_REQUIRE(d.alignment == 16 || d.alignment == 4, "the direct path moves 4 or 16 bytes per lane");
  if (run->reverse) {
    CUDADMA_REQUIRE(generic_source, "LDS -> global transfers go through the calls that take a generic source pointer");
    CUDADMA_REQUIRE(run->out_bytes > 0 && (run->out_bytes % 16) == 0, "out_bytes must be a positive multiple of 16");
    CUDADMA_REQUIRE((run->rep_src_bytes % 4) == 0, "rep_src_bytes must be a multiple of 4");
  }

  // ---- every byte the transfer touches must lie inside the caller's buffers and the LDS window ----
  {
    const bool indexed = d.pattern == CUDADMA_PATTERN_GATHER || d.pattern == CUDADMA_PATTERN_SCATTER;
    const size_t per_rep_out = run->reverse ? (size_t)run->out_bytes : (size_t)run->lds_bytes;
    if (run->out_capacity < (size_t)run->reps * per_rep_out) {
      cudadma_host::set_error("out_capacity %zu is smaller than reps * %zu bytes", run->out_capacity, per_rep_out);
      return CUDADMA_ERANGE;
    }
    CUDADMA_REQUIRE(run->rep_src_bytes >= 0 && run->rep_index_elmts >= 0 && run->src_offset_bytes >= 0 &&
                    run->dst_offset_bytes >= 0, "offsets and per-repetition advances must not be negative");
    std::vector<int> host_index;
    if (indexed && d.num_elmts > 0) {
      const long long need = (long long)(run->reps - 1) * run->rep_index_elmts + d.num_elmts;
      if (run->index_elmts < need) {
        cudadma_host::set_error("index_elmts %d is smaller than the %lld indices the repetitions read", run->index_elmts, need);
        return CUDADMA_ERANGE;
      }
      host_index.resize((size_t)need);
      CUDADMA_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
      CUDADMA_HIP_CHECK(hipMemcpy(host_index.data(), run->d_index, (size_t)need * sizeof(int), hipMemcpyDeviceToHost));
    }
    cudadma_plan_query_t q{};
    q.pattern = d.pattern; q.alignment = d.alignment; q.bytes_per_thread = d.bytes_per_thread;
    q.bytes_per_elmt = d.bytes_per_elmt; q.dma_threads = d.dma_threads; q.num_elmts = d.num_elmts;
    q.src_stride = run->src_stride; q.dst_stride = run->dst_stride;
    q.radius = d.radius; q.corners = d.corners; q.dimx = d.pattern == CUDADMA_PATTERN_HALO ? d.dimx : 0; q.dimy = d.dimy;
    q.pitch = run->pitch; q.dst_pitch = run->dst_pitch;
    long long src_origin = run->src_offset_bytes, dst_origin = run->dst_offset_bytes;
    if (d.pattern == CUDADMA_PATTERN_HALO) {
      src_origin += (long long)(d.radius * run->pitch + d.radius) * d.bytes_per_elmt;
      dst_origin += (long long)(d.radius * halo_dst_pitch + d.radius) * d.bytes_per_elmt;
    }
    for (int rep = 0; rep < run->reps; ++rep) {
      q.index = indexed && !host_index.empty() ? host_index.data() + (size_t)rep * run->rep_index_elmts : nullptr;
      long long ext[4] = {0, 0, 0, 0};
      if (!(indexed && d.num_elmts == 0)) {
        const int rc = cudadma_plan_extents(&q, ext);
        if (rc != 0) return rc;
      }
      // forward: source in d_in (advancing per repetition), destination in the LDS window;
      // reverse: the LDS image comes from d_in, the object reads LDS and writes its window of d_out
      const long long src_lo = src_origin + ext[0] + (run->reverse ? 0 : (long long)rep * run->rep_src_bytes);
      const long long src_hi = src_origin + ext[1] + (run->reverse ? 0 : (long long)rep * run->rep_src_bytes);
      const long long dst_lo = dst_origin + ext[2], dst_hi = dst_origin + ext[3];
      const long long src_cap = run->reverse ? (long long)run->lds_bytes : (long long)run->in_bytes;
      const long long dst_cap = run->reverse ? (long long)run->out_bytes : (long long)run->lds_bytes;
      if (ext[1] > ext[0] && (src_lo < 0 || src_hi > src_cap)) {
        cudadma_host::set_error("repetition %d reads bytes [%lld, %lld) of a %lld-byte %s", rep, src_lo, src_hi, src_cap,
                                run->reverse ? "LDS window" : "input buffer (in_bytes)");
        return CUDADMA_ERANGE;
      }
      if (ext[3] > ext[2] && (dst_lo < 0 || dst_hi > dst_cap)) {
        cudadma_host::set_error("repetition %d writes bytes [%lld, %lld) of a %lld-byte %s", rep, dst_lo, dst_hi, dst_cap,
                                run->reverse ? "output window (out_bytes)" : "LDS window");
        return CUDADMA_ERANGE;
      }
      if (run->reverse && (size_t)rep * run->rep_src_bytes + (size_t)run->lds_bytes > run->in_bytes) {
        cudadma_host::set_error("repetition %d loads its LDS image from beyond in_bytes", rep);
        return CUDADMA_ERANGE;
      }
    }
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
  a.dst_pitch = run->dst_pitch;
  return r[case_id].launch(a, (hipStream_t)stream);
}
