// Merge kernel for gfx950: combines the partial outputs of one (sequence, query head)
// into the final attention row.
//
// Contract (the reference's gather_kernel, csrc/pat_fwd_kernel.h:314-467): with
// partial results (O_i, LSE_i), LSE = M + ln(sum_i e^(LSE_i - M)), M = max_i LSE_i and
// out = sum_i e^(LSE_i - LSE) * O_i, cast to the output type; the final LSE is natural
// log of the scaled-logit sum.
//
// One wave64 per (sequence, head). The row's slot LSEs are read once, up to 4 per lane,
// and stay in registers (slots no workgroup filled hold -inf and get weight 0); then each
// lane accumulates head_dim/64 columns over the filled slots, whose rows are fetched in
// batches of 16 independent loads. That is a chain of three memory round trips (split count,
// LSEs, partial rows), which is what the kernel's run time consists of; launches with up to 8
// slots per row make it one: slot addresses do not depend on the split count, so everything is
// requested at once and what turns out unused is dropped (measured: 0.3-0.8 us less per launch;
// with 16 rows requested blindly the extra registers and reads cost what the round trips save).
#include <hip/hip_runtime.h>

#include "fwd_params.hpp"

namespace pat {

#ifndef PAT_MERGE_PAIRS_MIN
#define PAT_MERGE_PAIRS_MIN 16384   // rows from which a half-wave takes a row (launches of up to 8 slots per row)
#endif

// (the leading scalar arguments repeat the fields of `p` that the first two memory reads need:
// they are preloaded into SGPRs with the wave, the rest of `p` arrives by load meanwhile)
template <typename T, int D>
__global__ void __launch_bounds__(256) pat_merge_kernel(const int32_t* __restrict__ num_split_per_seq,
                                                        const float* __restrict__ lse_part, const int num_slots,
                                                        const int chunks_per_rank, const int max_split, const int batch,
                                                        const int heads, const int kv_heads, const MergeParams p) {
  constexpr int CPL = D / 64;   // columns per lane
  constexpr int kRegs = 4;      // LSE registers per lane: up to 256 slots stay in registers
  constexpr int kBatch = 16;    // partial rows fetched together
  constexpr int kSpec = 8;      // launches with up to this many slots per row fetch every slot's row at once
  const int lane = threadIdx.x & 63;
  // Which (sequence, head) is this wave's? Workgroups are dealt to the 8 XCDs round-robin, and the
  // split kernel's launch order put every partial row of kv head h through the L2 of XCD h mod 8
  // (where most of it still sits): with a multiple of 8 kv heads, workgroup b serves heads of the kv
  // heads = b mod 8, so the rows are found in its own L2. A matter of speed only.
  int s, hq;
  if (kv_heads % 8 == 0) {
    const int xcd = blockIdx.x & 7;
    const int per_seq = heads >> 3;                       // heads of one sequence served by one XCD
    const int64_t u = (int64_t)(blockIdx.x >> 3) * 4 + (threadIdx.x >> 6);
    if (u >= (int64_t)batch * per_seq) return;
    s = (int)(u / per_seq);
    const int local = (int)(u - (int64_t)s * per_seq);      // kv head (xcd + 8 i), head g of its group
    const int group = heads / kv_heads;
    hq = (xcd + 8 * (local / group)) * group + local % group;
  } else {
    const int64_t u = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= (int64_t)batch * heads) return;
    s = (int)(u / heads);
    hq = (int)(u % heads);
  }
  const int64_t pair = (int64_t)s * heads + hq;
  const float ninf = -__builtin_inff();

  const float* __restrict__ lse = lse_part + pair * num_slots;
  const float* __restrict__ op = p.o_part + pair * (int64_t)num_slots * D;
  if (num_slots <= kSpec) {
    // Few slots: nothing here depends on the split count but which slots count, so the count, the
    // slot LSEs and every slot's row are requested together (one round trip instead of three);
    // rows of slots that turn out empty or beyond the count are dropped unread.
    int ns = num_split_per_seq[s];
    float l = (lane < num_slots) ? lse[lane] : ninf;
    float v[kSpec][CPL];
#pragma unroll
    for (int b = 0; b < kSpec; ++b) {
      if (b < num_slots) {
        const float* row = op + (int64_t)b * D + lane * CPL;
        if (CPL == 2) {
          const float2 t = *(const float2*)row;
          v[b][0] = t.x;
          v[b][CPL - 1] = t.y;
        } else {
          v[b][0] = row[0];
        }
      }
    }
    ns = ns < 0 ? 0 : (ns > max_split ? max_split : ns);
    const int nsl = ns * chunks_per_rank;
    if (lane >= nsl) l = ninf;
    float mx = l;
#pragma unroll
    for (int off = kSpec / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    mx = __shfl(mx, 0);
    float e = (l > ninf) ? __expf(l - mx) : 0.f;
    float sum = e;
#pragma unroll
    for (int off = kSpec / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    sum = __shfl(sum, 0);
    const float total = (sum > 0.f) ? mx + logf(sum) : ninf;
    const float w_mine = (l > ninf) ? __expf(l - total) : 0.f;
    float acc[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[c] = 0.f;
#pragma unroll
    for (int b = 0; b < kSpec; ++b) {
      const float w = __shfl(w_mine, b);
      if (b < num_slots && w > 0.f) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) acc[c] += w * v[b][c];
      }
    }
    T* dst = (T*)p.out + (int64_t)s * p.o_stride_b + (int64_t)hq * p.o_stride_h + lane * CPL;
#pragma unroll
    for (int c = 0; c < CPL; ++c) dst[c] = (T)acc[c];
    if (p.lse_out != nullptr && lane == 0) p.lse_out[pair] = total;
    return;
  }
  int nsplit = num_split_per_seq[s];
  nsplit = nsplit < 0 ? 0 : (nsplit > max_split ? max_split : nsplit);
  const int nslots = nsplit * chunks_per_rank;  // slots are box-major

  // slot LSEs -> registers (slots past 256 are re-read below; no plan of the default buckets
  // gets there: 32 splits x 64 chunks would)
  float mine[kRegs];
  float mx = ninf;
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    const int i = r * 64 + lane;
    mine[r] = (i < nslots) ? lse[i] : ninf;
    mx = fmaxf(mx, mine[r]);
  }
  for (int i = kRegs * 64 + lane; i < nslots; i += 64) mx = fmaxf(mx, lse[i]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  float sum = 0.f;
  if (mx > ninf) {
#pragma unroll
    for (int r = 0; r < kRegs; ++r) sum += __expf(mine[r] - mx);   // exp(-inf) = 0
    for (int i = kRegs * 64 + lane; i < nslots; i += 64) sum += __expf(lse[i] - mx);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  const float total = (sum > 0.f) ? mx + logf(sum) : ninf;

  float acc[CPL];
#pragma unroll
  for (int c = 0; c < CPL; ++c) acc[c] = 0.f;

  // weighted sum of the filled slots of one 64-slot group
  auto accumulate = [&](int base, float w_mine) {
    unsigned long long live = __ballot(w_mine > 0.f);
    while (live) {
      int js[kBatch];
      float v[kBatch][CPL];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        js[b] = live ? __builtin_ctzll(live) : -1;
        live &= live - 1;   // 0 stays 0
      }
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        if (js[b] >= 0) {
          const float* row = op + (int64_t)(base + js[b]) * D + lane * CPL;
          if (CPL == 2) {
            const float2 t = *(const float2*)row;
            v[b][0] = t.x;
            v[b][CPL - 1] = t.y;
          } else {
            v[b][0] = row[0];
          }
        }
      }
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        if (js[b] >= 0) {
          const float w = __shfl(w_mine, js[b]);
#pragma unroll
          for (int c = 0; c < CPL; ++c) acc[c] += w * v[b][c];
        }
      }
    }
  };
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    if (r * 64 >= nslots) break;
    accumulate(r * 64, (mine[r] > ninf) ? __expf(mine[r] - total) : 0.f);
  }
  for (int base = kRegs * 64; base < nslots; base += 64) {
    const int i = base + lane;
    const float l = (i < nslots) ? lse[i] : ninf;
    accumulate(base, (l > ninf) ? __expf(l - total) : 0.f);
  }

  T* dst = (T*)p.out + (int64_t)s * p.o_stride_b + (int64_t)hq * p.o_stride_h + lane * CPL;
#pragma unroll
  for (int c = 0; c < CPL; ++c) dst[c] = (T)acc[c];
  if (p.lse_out != nullptr && lane == 0) p.lse_out[pair] = total;
}

// Launches with up to 8 slots per row and many rows (tens of thousands: hundreds of requests x
// 32-64 heads) are bound by the number of waves, each of which lives for one round trip: there a
// half-wave takes a (sequence, head), 16 bytes of a partial row per lane, which halves the waves and
// the load instructions per byte. Same arithmetic in the same order as the kernel above.
template <typename T, int D>
__global__ void __launch_bounds__(256) pat_merge_pairs_kernel(const int32_t* __restrict__ num_split_per_seq,
                                                              const float* __restrict__ lse_part, const int num_slots,
                                                              const int chunks_per_rank, const int max_split, const int batch,
                                                              const int heads, const int kv_heads, const MergeParams p) {
  constexpr int CPL = D / 32;   // columns per lane
  constexpr int kSpec = 8;
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5, l32 = lane & 31;
  const int slot_in_wg = (int)(threadIdx.x >> 6) * 2 + half;   // 8 rows per workgroup
  int s, hq;
  bool live;
  if (kv_heads % 8 == 0) {
    const int xcd = blockIdx.x & 7;
    const int per_seq = heads >> 3;
    int64_t u = (int64_t)(blockIdx.x >> 3) * 8 + slot_in_wg;
    const int64_t n = (int64_t)batch * per_seq;
    live = u < n;
    if (!live) u = n - 1;          // (an idle half repeats the last row's reads and stores nothing)
    s = (int)(u / per_seq);
    const int local = (int)(u - (int64_t)s * per_seq);
    const int group = heads / kv_heads;
    hq = (xcd + 8 * (local / group)) * group + local % group;
  } else {
    int64_t u = (int64_t)blockIdx.x * 8 + slot_in_wg;
    const int64_t n = (int64_t)batch * heads;
    live = u < n;
    if (!live) u = n - 1;
    s = (int)(u / heads);
    hq = (int)(u % heads);
  }
  const int64_t pair = (int64_t)s * heads + hq;
  const float ninf = -__builtin_inff();
  const float* __restrict__ lse = lse_part + pair * num_slots;
  const float* __restrict__ op = p.o_part + pair * (int64_t)num_slots * D;
  int ns = num_split_per_seq[s];
  float l = (l32 < num_slots) ? lse[l32] : ninf;
  float v[kSpec][CPL];
#pragma unroll
  for (int b = 0; b < kSpec; ++b) {
    if (b < num_slots) {
      const float* row = op + (int64_t)b * D + l32 * CPL;
      if (CPL == 4) {
        const float4 t = *(const float4*)row;
        v[b][0] = t.x; v[b][1] = t.y; v[b][CPL - 2] = t.z; v[b][CPL - 1] = t.w;
      } else {
        const float2 t = *(const float2*)row;
        v[b][0] = t.x; v[b][CPL - 1] = t.y;
      }
    }
  }
  ns = ns < 0 ? 0 : (ns > max_split ? max_split : ns);
  const int nsl = ns * chunks_per_rank;
  if (l32 >= nsl) l = ninf;
  float mx = l;
#pragma unroll
  for (int off = kSpec / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  mx = __shfl(mx, half * 32);
  float e = (l > ninf) ? __expf(l - mx) : 0.f;
  float sum = e;
#pragma unroll
  for (int off = kSpec / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  sum = __shfl(sum, half * 32);
  const float total = (sum > 0.f) ? mx + logf(sum) : ninf;
  const float w_mine = (l > ninf) ? __expf(l - total) : 0.f;
  float acc[CPL];
#pragma unroll
  for (int c = 0; c < CPL; ++c) acc[c] = 0.f;
#pragma unroll
  for (int b = 0; b < kSpec; ++b) {
    const float w = __shfl(w_mine, half * 32 + b);
    if (b < num_slots && w > 0.f) {
#pragma unroll
      for (int c = 0; c < CPL; ++c) acc[c] += w * v[b][c];
    }
  }
  if (!live) return;
  T* dst = (T*)p.out + (int64_t)s * p.o_stride_b + (int64_t)hq * p.o_stride_h + l32 * CPL;
#pragma unroll
  for (int c = 0; c < CPL; ++c) dst[c] = (T)acc[c];
  if (p.lse_out != nullptr && l32 == 0) p.lse_out[pair] = total;
}

// Host launcher: one wave per (sequence, query head), four per workgroup; a half-wave each in large launches
// of few slots.
hipError_t launch_merge(bool bf16, int head_dim, hipStream_t stream, const MergeParams& params) {
  const int64_t pairs = (int64_t)params.batch * params.heads;
  void (*fn)(const int32_t*, const float*, int, int, int, int, int, int, const MergeParams);
  int per_wg = 4;
  if (params.num_slots <= 8 && pairs >= PAT_MERGE_PAIRS_MIN) {
    per_wg = 8;
    if (bf16) fn = head_dim == 64 ? pat_merge_pairs_kernel<__bf16, 64> : pat_merge_pairs_kernel<__bf16, 128>;
    else fn = head_dim == 64 ? pat_merge_pairs_kernel<_Float16, 64> : pat_merge_pairs_kernel<_Float16, 128>;
  } else {
    if (bf16) fn = head_dim == 64 ? pat_merge_kernel<__bf16, 64> : pat_merge_kernel<__bf16, 128>;
    else fn = head_dim == 64 ? pat_merge_kernel<_Float16, 64> : pat_merge_kernel<_Float16, 128>;
  }
  // (a multiple of 8 kv heads: 8 interleaved lists of pairs, one per XCD, each rounded up to whole workgroups)
  const int64_t wgs = params.kv_heads % 8 == 0 ? 8 * ((pairs / 8 + per_wg - 1) / per_wg) : (pairs + per_wg - 1) / per_wg;
  const dim3 grid((unsigned)wgs), block(256);
  hipLaunchKernelGGL(fn, grid, block, 0, stream, params.num_split_per_seq, params.lse_part, params.num_slots,
                     params.chunks_per_rank, params.max_split, params.batch, params.heads, params.kv_heads, params);
  return hipGetLastError();
}

}  // namespace pat
