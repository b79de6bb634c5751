// Variant tables, the occupancy knob and grid sizing shared by the workloads.
#include "workloads.hpp"
#include <atomic>
#include <cstring>

namespace workloads {

static std::atomic<int> g_wg_per_cu{0};

int device_cus()
{
  // queried once (thread-safe initialisation of a local static); 256 if the query fails
  static const int cus = [] {
    const int n = cudadma_device_cus();
    return n > 0 ? n : 256;
  }();
  return cus;
}

int persistent_grid(long long work_items, int default_wg_per_cu)
{
  const int knob = g_wg_per_cu.load();
  const long long want = (long long)device_cus() * (knob > 0 ? knob : default_wg_per_cu);
  return (int)(work_items < want ? work_items : want);
}

struct Knob {
  const char* name;
  std::atomic<int> value;
};
static Knob g_knobs[] = {{"transpose_band", {0}}, {"transpose_workgroups", {0}}, {"transpose_split", {0}}, {"stencil_zchunk", {0}}, {"stencil_xcd_remap", {0}}, {"stencil_ring", {0}}, {"probe_piece_bytes", {0}}, {"probe_xcd_group", {0}}, {"transpose_wide_order", {0}}, {"transpose_wide_dma", {0}}};

static Knob* find_knob(const char* name)
{
  for (Knob& k : g_knobs)
    if (name != nullptr && std::strcmp(k.name, name) == 0) return &k;
  return nullptr;
}

int tuning(const char* name, int fallback)
{
  Knob* k = find_knob(name);
  const int v = k != nullptr ? k->value.load() : 0;
  return v > 0 ? v : fallback;
}

static const VariantInfo kSequential[] = {
  {"manual double buffer: one DMA group of 2 wavefronts, two objects, two-phase calls, registers -> ds_write_b128, four "
   "workgroups per compute unit; for more than 96 MiB (a working set beyond the Infinity Cache) variant 5 instead"},
  {"single buffer: one object, execute_dma"},
  {"double buffer: two DMA groups of 1 wavefront, one object each"},
  {"manual double buffer with STORE_LDS_DIRECT (global_load_lds_dwordx4, no VGPR staging)"},
  {"no DMA object: every wavefront copies global -> LDS -> global between workgroup barriers"},
  {"single buffer (the next tile waits in the DMA wavefronts' registers), two workgroups per compute unit, streaming "
   "loads and non-temporal stores: the shape for buffers beyond the Infinity Cache"},
  {"variant 5 with a contiguous run of tiles per workgroup instead of every n-th tile"},
};
static const VariantInfo kStrided[] = {
  {"the library's choice: variant 10 at its default split (three DMA wavefronts, one compute wavefront, one LDS tile, "
   "the next tile in the DMA wavefronts' registers)"},
  {"single buffer: one object and one LDS tile, execute_dma (the next tile waits in the DMA wavefronts' registers); one "
   "workgroup per compute unit, tiles walked down the columns, streaming loads (LOAD_CACHE_STREAMING), the consumer "
   "transposes 4 x 4 words inside each quad and writes non-temporal dwordx4: the fastest shape"},
  {"manual double buffer, unpadded LDS rows (256 B): shows the bank-conflict cost"},
  {"double buffer: two DMA groups of 1 wavefront, one CudaDMAStrided object and one padded LDS tile each"},
  {"not warp-specialised: all four wavefronts move the tile and write it out, next tile requested two-phase"},
  {"two DMA groups, unpadded 256 B LDS rows filled by global_load_lds_dwordx4 with XOR-swizzled chunks "
   "(STORE_LDS_DIRECT_SWIZZLE): no VGPR staging, no padding, no bank conflicts"},
  {"two DMA groups, unpadded 256 B LDS rows with XOR-swizzled chunks written from registers (STORE_LDS_SWIZZLE)"},
  {"as variant 11, but the compute lanes transpose 4 x 4 words inside each quad (quad-permute moves) and write "
   "dwordx4: one store covers four output rows of 256 contiguous bytes instead of one"},
  {"one DMA wavefront and one compute wavefront per workgroup, two objects of a whole tile each on the DMA "
   "wavefront, two LDS tiles; dword stores"},
  {"as variant 8 with the quad transposition and dwordx4 stores of variant 7"},
  {"variant 1 with the split of the workgroup as a knob (\"transpose_split\" = 100 x DMA wavefronts + 10 x compute "
   "wavefronts + tiles requested ahead; default 311: three DMA wavefronts, one compute wavefront, one tile ahead, "
   "the fastest of the 22 splits compiled; with 3 + 1 wavefronts the last digit 3 to 7 asks for the tile in halves "
   "or quarters, 0.75 to 1.75 tiles in flight, and 8 for the next tile requested as soon as the loads of the current "
   "one have returned): one LDS tile guarded by a sync-only object, one or two CudaDMAStrided "
   "objects without a handshake of their own on the DMA wavefronts; the kernel the benchmark reports"},
  {"manual double buffer in LDS: one DMA group of 2 wavefronts, two CudaDMAStrided objects and two LDS tiles with padded "
   "rows (272 B), four workgroups per compute unit"},
#ifdef HIPDMA_SWEEP_VARIANTS
  {"output rows written 1 KiB at a time: the DMA side of variant 10 (tiles of 64 rows x 256 B, one LDS tile, one tile of loads "
   "in flight), the compute wavefront gathers four tiles that lie side by side in the output in a second LDS buffer, "
   "transposed, and writes 64 rows of 1 KiB with one store instruction per row (knobs transpose_wide_order, transpose_wide_dma)"},
  {"variant 12 with two LDS tiles on the DMA side (still one tile of loads in flight)"},
#else
  {""}, {""},
#endif
  {"double buffer in LDS with one object: two LDS tiles with a guard each, filled in turn by one CudaDMAStrided object on "
   "three DMA wavefronts, the next tile in their registers (one tile of loads in flight), one compute wavefront, one "
   "workgroup per compute unit"},
};
static const VariantInfo kGather[] = {
  {"the library's choice: variant 6 (two objects, index words requested one transfer ahead)"},
  {"single buffer: one object, execute_dma"},
  {"manual double buffer: one DMA group of 2 wavefronts, two CudaDMAIndirect objects, each transfer fetches its own index words"},
  {"manual 4-stage buffering: four objects, each transfer fetches its own index words"},
  {"four objects, the index words of each object's next tile requested one turn of the ring ahead (prefetch_index)"},
  {"three objects, index words requested ahead"},
  {"two objects, index words requested ahead; three workgroups per compute unit (four for tables beyond 1 GiB)"},
};
static const VariantInfo kHalo[] = {
  {"warp-specialised, 4 cells per thread as one dwordx4: 1 DMA wavefront keeps the rings of 7 planes in flight in 8 "
   "CudaDMAHalo objects and lands one per plane (execute_dma_no_sync style); one s_barrier per plane orders the ring, "
   "the interior exchange and the reuse of the 4 LDS planes"},
  {"as variant 0 plus the empty/full handshake (cudaDMACustom guards on the 4 LDS planes) next to the s_barrier"},
  {"as variant 1 but the compute wavefronts meet in an LDS-counter GroupBarrier and the DMA wavefront runs free"},
  {"not warp-specialised, dwordx4 cells: every thread computes, half of them also carry a ring chunk requested one "
   "plane ahead; one LDS plane, two s_barriers per plane"},
#ifdef HIPDMA_SWEEP_VARIANTS
  {"warp-specialised, one cell per dword load (first version kept for comparison)"},
#else
  {""},
#endif
#ifdef HIPDMA_SWEEP_VARIANTS
  {"not warp-specialised, one cell per dword load"},
#else
  {""},
#endif
  {"variant 0 with tiles of 64 x 16 cells (rows of 256 B; nx a multiple of 64, ny of 16): 2 to 8 % faster at 512^3, not "
   "the tile the benchmark configuration names"},
  {"variant 1 with tiles of 64 x 16 cells"},
};

static const VariantInfo kGemm[] = {
  {"the largest workgroup tile that divides the problem and gives every compute unit a tile: variant 9, 3 or 2, else "
   "variant 1"},
  {"warp-specialised: two DMA wavefronts per operand with two CudaDMAStrided objects each (two LDS stages, tile two K "
   "steps ahead in flight), four compute wavefronts with v_mfma_f32_32x32x16_bf16, B fragments through "
   "ds_read_b64_tr_b16; 128 x 128 workgroup tile, 64 x 64 per compute wavefront, two workgroups per compute unit"},
  {"same structure, 128 x 256 workgroup tile, 64 x 128 per compute wavefront, one workgroup per compute unit"},
  {"same structure, 256 x 128 workgroup tile, 128 x 64 per compute wavefront, one workgroup per compute unit"},
#ifdef HIPDMA_SWEEP_VARIANTS
  {"256 x 128 workgroup tile with the tiles brought in by global_load_lds_dwordx4 (STORE_LDS_DIRECT_SWIZZLE): three "
   "unpadded swizzled LDS stages, two transfers in flight per DMA wavefront, no ds_write"},
#else
  {""},
#endif
#ifdef HIPDMA_SWEEP_VARIANTS
  {"256 x 256 workgroup tile (m and n multiples of 256): eight compute wavefronts of 128 x 64, two per SIMD, next to the "
   "four DMA wavefronts; twelve wavefronts leave 168 registers each"},
#else
  {""},
#endif
#ifdef HIPDMA_SWEEP_VARIANTS
  {"256 x 256 workgroup tile, K step 32, four unpadded swizzled LDS stages filled by global_load_lds_dwordx4 "
   "(three transfers in flight per DMA wavefront), eight compute wavefronts"},
#else
  {""},
#endif
  {"variant 6 with A transfers of two K steps (256 rows x 128 B, whole cache lines) into two 32 KB buffers with guards "
   "of their own; B keeps four stages of one K step"},
#ifdef HIPDMA_SWEEP_VARIANTS
  {"not warp-specialised: 256 x 256 tile, four wavefronts that each issue their share of the direct-to-LDS loads and "
   "multiply a 128 x 128 block; one s_barrier per K step"},
#else
  {""},
#endif
  {"variant 8 with A transfers of two K steps (rows of 128 B, whole cache lines) into a ring of three buffers: with the "
   "four B stages all of the 160 KB of LDS"},
};

static const VariantInfo kScatter[] = {
  {"manual 4-stage buffering, LDS -> global: the compute wavefronts fill four LDS tiles of 32 records, one DMA group of "
   "2 wavefronts drains them with one CudaDMAIndirect<false> object, a cudaDMACustom guard per tile"},
  {"single buffer: one LDS tile, one guard"},
  {"manual double buffer: two LDS tiles, two guards"},
  {"not warp-specialised: all four wavefronts fill the tile, meet, and all four scatter it"},
};

static const VariantInfo* table(int workload, int* count)
{
  switch (workload) {
    case CUDADMA_WORKLOAD_SEQUENTIAL: *count = sizeof(kSequential) / sizeof(VariantInfo); return kSequential;
    case CUDADMA_WORKLOAD_STRIDED:    *count = sizeof(kStrided) / sizeof(VariantInfo);    return kStrided;
    case CUDADMA_WORKLOAD_GATHER:     *count = sizeof(kGather) / sizeof(VariantInfo);     return kGather;
    case CUDADMA_WORKLOAD_HALO:       *count = sizeof(kHalo) / sizeof(VariantInfo);       return kHalo;
    case CUDADMA_WORKLOAD_GEMM:       *count = sizeof(kGemm) / sizeof(VariantInfo);       return kGemm;
    case CUDADMA_WORKLOAD_SCATTER:    *count = sizeof(kScatter) / sizeof(VariantInfo);    return kScatter;
    default: *count = 0; return nullptr;
  }
}

}  // namespace workloads

extern "C" int cudadma_num_variants(int workload)
{
  int n = 0;
  workloads::table(workload, &n);
  return n;
}

extern "C" const char* cudadma_variant_name(int workload, int variant)
{
  int n = 0;
  const workloads::VariantInfo* t = workloads::table(workload, &n);
  return (t != nullptr && variant >= 0 && variant < n) ? t[variant].name : "";
}

extern "C" int cudadma_set_tuning(const char* name, int value)
{
  workloads::Knob* k = workloads::find_knob(name);
  if (k == nullptr) {
    cudadma_host::set_error("unknown tuning knob '%s'", name != nullptr ? name : "(null)");
    return CUDADMA_EINVAL;
  }
  return k->value.exchange(value < 0 ? 0 : value);
}

extern "C" int cudadma_set_workgroups_per_cu(int value)
{
  return workloads::g_wg_per_cu.exchange(value < 0 ? 0 : value);
}
