// Known-answer cases for the first-generation class names (cudaDMASequential,
// cudaDMAStrided, cudaDMAIndirect of include/cudaDMA.h:644-3580): every constructor
// form of the adapters in hipdma/v1.hpp moves one transfer into an LDS window that
// was filled with a sentinel, and the whole window is copied out for comparison.
#include "common.hpp"
#include "../../include/cudadma_amd_harness.h"
#include "../../include/cudaDMA.h"
#include "status_word.hpp"

namespace {

constexpr int kWindow = 16 * 1024;
constexpr int kCompute = 64;
constexpr unsigned kSentinel = 0xA5A5A5A5u;

struct Args {
  const char* in;
  const int* index;
  char* out;
};

// One transfer by a warp-specialised object: compute threads [0, 64), DMA threads after them.
template<typename DMA, typename... Src>
__device__ __forceinline__ void ws_transfer(DMA& dma, char* window, Src... src)
{
  if (dma.owns_this_thread()) {
    dma.execute_dma(src..., window);
  } else {
    dma.start_async_dma();
    dma.wait_for_dma_finish();
  }
}

template<int ID> struct Case;

#define V1_CASE(ID, PATTERN, WS, E, N, SRC_STRIDE, DST_STRIDE, DMA_THREADS_, TEXT, ...)                 \
  template<> struct Case<ID> {                                                                         \
    static constexpr cudadma_v1_case_t info = {PATTERN, WS, E, N, SRC_STRIDE, DST_STRIDE, DMA_THREADS_, \
                                               (WS ? kCompute : 0) + DMA_THREADS_, kWindow};           \
    static constexpr const char* text = TEXT;                                                          \
    static __device__ __forceinline__ void run(const Args& a, char* window) { __VA_ARGS__ }            \
  };

// ---- cudaDMASequential ----
V1_CASE(0, CUDADMA_PATTERN_SEQUENTIAL, 1, 4096, 1, 0, 0, 64,
        "cudaDMASequential<true,16,4096,64>(dmaID, num_compute, start)",
        cudaDMASequential<true, 16, 4096, 64> dma(1, kCompute, kCompute);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(1, CUDADMA_PATTERN_SEQUENTIAL, 0, 4100, 1, 0, 0, 128,
        "cudaDMASequential<false,4,4100,128>()",
        cudaDMASequential<false, 4, 4100, 128> dma;
        dma.execute_dma(a.in, window);)
V1_CASE(2, CUDADMA_PATTERN_SEQUENTIAL, 1, 1000, 1, 0, 0, 128,
        "cudaDMASequential<true,8>(dmaID, dma_threads, num_compute, start, bytes)",
        cudaDMASequential<true, 8> dma(2, 128, kCompute, kCompute, 1000);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(3, CUDADMA_PATTERN_SEQUENTIAL, 0, 2052, 1, 0, 0, 64,
        "cudaDMASequential<false,4>(bytes)",
        cudaDMASequential<false, 4> dma(2052);
        dma.execute_dma(a.in, window);)
V1_CASE(4, CUDADMA_PATTERN_SEQUENTIAL, 1, 3072, 1, 0, 0, 128,
        "cudaDMASequential<true,16,3072>(dmaID, dma_threads, num_compute, start)",
        cudaDMASequential<true, 16, 3072> dma(3, 128, kCompute, kCompute);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(5, CUDADMA_PATTERN_SEQUENTIAL, 0, 512, 1, 0, 0, 64,
        "cudaDMASequential<false,16,512>()",
        cudaDMASequential<false, 16, 512> dma;
        dma.execute_dma(a.in, window);)
// ---- cudaDMAStrided: one stride argument strides the source and packs the destination ----
V1_CASE(6, CUDADMA_PATTERN_STRIDED, 1, 256, 16, 1024, 256, 64,
        "cudaDMAStrided<true,16,256,64,16>(dmaID, num_compute, start, el_stride): destination packed",
        cudaDMAStrided<true, 16, 256, 64, 16> dma(1, kCompute, kCompute, 1024);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(7, CUDADMA_PATTERN_STRIDED, 1, 256, 16, 1024, 272, 64,
        "cudaDMAStrided<true,16,256,64,16>(dmaID, num_compute, start, src_stride, dst_stride)",
        cudaDMAStrided<true, 16, 256, 64, 16> dma(1, kCompute, kCompute, 1024, 272);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(8, CUDADMA_PATTERN_STRIDED, 0, 132, 9, 400, 132, 128,
        "cudaDMAStrided<false,4>(bytes_per_elmt, num_elmts, el_stride): destination packed",
        cudaDMAStrided<false, 4> dma(132, 9, 400);
        dma.execute_dma(a.in, window);)
V1_CASE(9, CUDADMA_PATTERN_STRIDED, 0, 132, 9, 400, 136, 128,
        "cudaDMAStrided<false,4>(bytes_per_elmt, num_elmts, src_stride, dst_stride)",
        cudaDMAStrided<false, 4> dma(132, 9, 400, 136);
        dma.execute_dma(a.in, window);)
V1_CASE(10, CUDADMA_PATTERN_STRIDED, 1, 2048, 5, 2560, 2048, 128,
        "cudaDMAStrided<true,8>(dmaID, dma_threads, num_compute, start, bytes_per_elmt, num_elmts, el_stride)",
        cudaDMAStrided<true, 8> dma(4, 128, kCompute, kCompute, 2048, 5, 2560);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(11, CUDADMA_PATTERN_STRIDED, 1, 64, 40, 96, 64, 64,
        "cudaDMAStrided<true,16,64>(dmaID, dma_threads, num_compute, start, num_elmts, el_stride)",
        cudaDMAStrided<true, 16, 64> dma(5, 64, kCompute, kCompute, 40, 96);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(12, CUDADMA_PATTERN_STRIDED, 1, 64, 40, 96, 80, 128,
        "cudaDMAStrided<true,16,64,128>(dmaID, num_compute, start, num_elmts, src_stride, dst_stride)",
        cudaDMAStrided<true, 16, 64, 128> dma(6, kCompute, kCompute, 40, 96, 80);
        ws_transfer(dma, window, (const void*)a.in);)
V1_CASE(13, CUDADMA_PATTERN_STRIDED, 0, 96, 33, 128, 96, 64,
        "cudaDMAStrided<false,8,96>(num_elmts, el_stride)",
        cudaDMAStrided<false, 8, 96> dma(33, 128);
        dma.execute_dma(a.in, window);)
V1_CASE(14, CUDADMA_PATTERN_STRIDED, 0, 96, 33, 128, 96, 64,
        "cudaDMAStrided<false,8,96,64>(num_elmts, el_stride)",
        cudaDMAStrided<false, 8, 96, 64> dma(33, 128);
        dma.execute_dma(a.in, window);)
V1_CASE(15, CUDADMA_PATTERN_STRIDED, 0, 48, 12, 64, 48, 64,
        "cudaDMAStrided<false,16,48,64,12>(el_stride)",
        cudaDMAStrided<false, 16, 48, 64, 12> dma(64);
        dma.execute_dma(a.in, window);)
// ---- cudaDMAIndirect: element i of the dense side pairs with element index[i] of the sparse side ----
V1_CASE(16, CUDADMA_PATTERN_GATHER, 1, 128, 32, 0, 128, 64,
        "cudaDMAIndirect<true,true,16,128,64,32>(dmaID, num_compute, start)",
        cudaDMAIndirect<true, true, 16, 128, 64, 32> dma(1, kCompute, kCompute);
        ws_transfer(dma, window, a.index, (const void*)a.in);)
V1_CASE(17, CUDADMA_PATTERN_GATHER, 0, 128, 32, 0, 128, 64,
        "cudaDMAIndirect<true,false,16,128,64,32>()",
        cudaDMAIndirect<true, false, 16, 128, 64, 32> dma;
        dma.execute_dma(a.index, a.in, window);)
V1_CASE(18, CUDADMA_PATTERN_GATHER, 1, 36, 50, 0, 36, 128,
        "cudaDMAIndirect<true,true,4>(dmaID, dma_threads, num_compute, start, bytes_per_elmt, num_elmts)",
        cudaDMAIndirect<true, true, 4> dma(2, 128, kCompute, kCompute, 36, 50);
        ws_transfer(dma, window, a.index, (const void*)a.in);)
V1_CASE(19, CUDADMA_PATTERN_SCATTER, 0, 64, 20, 64, 0, 64,
        "cudaDMAIndirect<false,false,16>(bytes_per_elmt, num_elmts)",
        cudaDMAIndirect<false, false, 16> dma(64, 20);
        dma.execute_dma(a.index, a.in, window);)
V1_CASE(20, CUDADMA_PATTERN_SCATTER, 1, 256, 10, 256, 0, 64,
        "cudaDMAIndirect<false,true,8,256>(dmaID, dma_threads, num_compute, start, num_elmts)",
        cudaDMAIndirect<false, true, 8, 256> dma(3, 64, kCompute, kCompute, 10);
        ws_transfer(dma, window, a.index, (const void*)a.in);)
V1_CASE(21, CUDADMA_PATTERN_GATHER, 1, 512, 7, 0, 512, 128,
        "cudaDMAIndirect<true,true,16,512,128>(dmaID, num_compute, start, num_elmts)",
        cudaDMAIndirect<true, true, 16, 512, 128> dma(4, kCompute, kCompute, 7);
        ws_transfer(dma, window, a.index, (const void*)a.in);)
V1_CASE(22, CUDADMA_PATTERN_GATHER, 0, 512, 7, 0, 512, 128,
        "cudaDMAIndirect<true,false,16,512>(num_elmts)",
        cudaDMAIndirect<true, false, 16, 512> dma(7);
        dma.execute_dma(a.index, a.in, window);)
constexpr int kNumCases = 23;

template<int ID>
__global__ void v1_case_kernel(Args a)
{
  __shared__ __attribute__((aligned(16))) char window[kWindow];
  for (int i = threadIdx.x * 4; i < kWindow; i += blockDim.x * 4) *reinterpret_cast<unsigned*>(window + i) = kSentinel;
  __syncthreads();
  Case<ID>::run(a, window);
  __syncthreads();
  for (int i = threadIdx.x * 4; i < kWindow; i += blockDim.x * 4)
    *reinterpret_cast<unsigned*>(a.out + i) = *reinterpret_cast<const unsigned*>(window + i);
}

template<int ID>
int dispatch(int id, cudadma_v1_case_t* info, const char** text, const Args* a, hipStream_t s)
{
  if (id == ID) {
    if (info != nullptr) *info = Case<ID>::info;
    if (text != nullptr) *text = Case<ID>::text;
    if (a != nullptr) hipLaunchKernelGGL(v1_case_kernel<ID>, dim3(1), dim3(Case<ID>::info.block_threads), 0, s, *a);
    return CUDADMA_OK;
  }
  if constexpr (ID + 1 < kNumCases) return dispatch<ID + 1>(id, info, text, a, s);
  return CUDADMA_ERANGE;
}

}  // namespace

extern "C" int cudadma_v1_num_cases(void) { return kNumCases; }

extern "C" int cudadma_v1_get_case(int id, cudadma_v1_case_t* out)
{
  CUDADMA_REQUIRE(out != nullptr, "out is NULL");
  const int rc = dispatch<0>(id, out, nullptr, nullptr, nullptr);
  if (rc != CUDADMA_OK) cudadma_host::set_error("no first-generation case %d", id);
  return rc;
}

extern "C" const char* cudadma_v1_case_text(int id)
{
  const char* text = nullptr;
  return dispatch<0>(id, nullptr, &text, nullptr, nullptr) == CUDADMA_OK ? text : nullptr;
}

extern "C" int cudadma_v1_run_case(int id, const void* d_in, const int* d_index, void* d_out, void* stream)
{
  cudadma_v1_case_t info;
  if (dispatch<0>(id, &info, nullptr, nullptr, nullptr) != CUDADMA_OK) {
    cudadma_host::set_error("no first-generation case %d", id);
    return CUDADMA_ERANGE;
  }
  CUDADMA_REQUIRE(d_in != nullptr && d_out != nullptr, "NULL pointer");
  CUDADMA_REQUIRE(cudadma_host::aligned_to(d_in, 16) && cudadma_host::aligned_to(d_out, 4), "d_in must be 16-byte aligned");
  const bool indirect = info.pattern == CUDADMA_PATTERN_GATHER || info.pattern == CUDADMA_PATTERN_SCATTER;
  CUDADMA_REQUIRE(!indirect || d_index != nullptr, "this case needs an index array");
  const Args a = {(const char*)d_in, d_index, (char*)d_out};
  dispatch<0>(id, nullptr, nullptr, &a, (hipStream_t)stream);
  CUDADMA_HIP_CHECK(hipGetLastError());
  return CUDADMA_OK;
}
