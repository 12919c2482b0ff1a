// Device self-test of the instruction-level assumptions the split kernel is built on:
//  * lane_ops.hpp: max / sum over lanes l, l^16, l^32, l^48 with v_permlane16/32_swap equal the
//    same reductions with __shfl_xor;
//  * ds_read_b64_tr_b16: within a 16-lane group, result lane i element r is source lane
//    (4r + i/4) element (i%4), the mapping the transposed V reads are addressed for.
//  * v_mfma_f32_32x32x16_f16: A lane l holds row l%32, k = 8(l/32)..+7; B lane l holds column l%32,
//    k = 8(l/32)..+7; accumulator register i of lane l is element (8(i/4) + 4(l/32) + i%4, l%32):
//    the layouts the tall-box path of the split kernel is written for.
// All were established on the hardware; a compiler or driver that breaks one of them shows up
// here instead of as wrong attention outputs.
#include <hip/hip_runtime.h>

#include "capi_error.hpp"
#include "hip/lane_ops.hpp"
#include "pat_amd.h"

namespace pat {
namespace {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ void selftest_kernel(int* failures) {
  __shared__ __attribute__((aligned(16))) short tile[64 * 4];
  const int lane = threadIdx.x;
  int bad = 0;
  // ---- lane reductions -------------------------------------------------------------------
  const float x = (float)((lane * 37) % 64) + 0.25f * (float)(lane & 3);
  float m = fmaxf(x, __shfl_xor(x, 16));
  m = fmaxf(m, __shfl_xor(m, 32));
  float s = x + __shfl_xor(x, 16);
  s = s + __shfl_xor(s, 32);
  bad += max_xor32(max_xor16(x)) != m;
  bad += sum_xor32(sum_xor16(x)) != s;
  bad += max_xor16(x) != fmaxf(x, __shfl_xor(x, 16));
  bad += max_xor32(x) != fmaxf(x, __shfl_xor(x, 32));
  // ---- transposed LDS read ---------------------------------------------------------------
  // lane l holds 4 shorts l*4 .. l*4+3 at byte offset l*8; every lane reads back its own 8 bytes
  // through the transposing read
#pragma unroll
  for (int e = 0; e < 4; ++e) tile[lane * 4 + e] = (short)(lane * 4 + e);
  __syncthreads();
  const s16x4 got = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4*)(tile + lane * 4));
  const int grp = lane & ~15, i = lane & 15;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int src_lane = grp + 4 * r + i / 4;
    bad += got[r] != (short)(src_lane * 4 + (i % 4));
  }
  // ---- 32x32x16 MFMA operand and accumulator layouts ----------------------------------------
  {
    auto A = [](int m, int k) { return (float)((m * 3 + k * 5) % 7 - 3); };
    auto B = [](int k, int c) { return (float)((k * 2 + c) % 5 - 2); };
    const int half = lane >> 5, idx = lane & 31;
    f16x8 a, b;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      a[j] = (_Float16)A(idx, 8 * half + j);
      b[j] = (_Float16)B(8 * half + j, idx);
    }
    f32x16 c;
#pragma unroll
    for (int r = 0; r < 16; ++r) c[r] = 0.f;
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = 8 * (r / 4) + 4 * half + r % 4;
      float want = 0.f;
      for (int k = 0; k < 16; ++k) want += A(m, k) * B(k, idx);
      bad += c[r] != want;
    }
  }
  if (bad) atomicAdd(failures, bad);
}

}  // namespace
}  // namespace pat

extern "C" int pat_selftest_device(void* hip_stream, int32_t* failures) {
  using namespace pat;
  if (failures == nullptr) return fail(PAT_ERR_INVALID, "failures must not be NULL");
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  int* dev = nullptr;
  hipError_t e = hipMalloc(&dev, sizeof(int));
  if (e != hipSuccess) return fail(PAT_ERR_HIP, std::string("hipMalloc: ") + hipGetErrorString(e));
  int host = 0;
  e = hipMemcpyAsync(dev, &host, sizeof(int), hipMemcpyHostToDevice, stream);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(selftest_kernel, dim3(1), dim3(64), 0, stream, dev);
    e = hipGetLastError();
  }
  if (e == hipSuccess) e = hipMemcpyAsync(&host, dev, sizeof(int), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  hipFree(dev);
  if (e != hipSuccess) return fail(PAT_ERR_HIP, std::string("self-test: ") + hipGetErrorString(e));
  *failures = host;
  return PAT_OK;
}
