// Split-KV forward kernel for gfx950 (MI355X): one workgroup streams one chunk of one
// packed box's KV for one kv-head and writes a normalised partial output + LSE.
//
// Functional contract (what the reference's pat_fwd_splitkv_kernel computes,
// csrc/pat_fwd_kernel.h:25-299): rows r = g + G*j of a box are (sequence
// q_table[j], query head h*G + g); every row attends to the same kv tokens, found
// through the box's block table; the partial result is softmax(q.K^T*scale).V over
// those tokens plus LSE = max + ln(sum) (csrc/softmax.h:169-188).
//
// Mapping to the hardware (this kernel's own design):
//  * a workgroup = 4 wave64 working on one (box, kv-head, chunk) in one of two ways:
//      - boxes of up to 16 rows: each wave owns every 4th 32-token step of the chunk and
//        runs an independent online softmax; the 4 states are combined through LDS;
//      - boxes of 17..64 rows: wave w owns rows 16w..16w+15 over the whole chunk (the
//        waves re-read the same K/V lines through L1), no combine needed.
//    Either way one (box, head, chunk) yields one partial row set, every wave carries a
//    single 16-row tile of state, and one launch covers all buckets.
//  * S^T = K.Q^T on v_mfma_f32_16x16x32: K rows are the MFMA A operand, so a lane
//    loads 16 contiguous bytes of one token straight from HBM into operand layout
//    (no LDS for K). The accumulator layout of S^T is the B-operand layout of
//    O^T = V^T.P^T, so P never moves between lanes.
//  * V must be contracted along tokens but is contiguous along head_dim: each wave
//    stages its 32 x D tile in a private, padded LDS region (16-byte writes) and
//    reads it back transposed with ds_read_b64_tr_b16.
//  * all softmax state of a row lives in the 4 lanes {n, n+16, n+32, n+48}.
#include <hip/hip_runtime.h>

#include "fwd_params.hpp"

namespace pat {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define PAT_LDS __attribute__((address_space(3)))

template <typename T> struct Elem;
template <> struct Elem<_Float16> {
  using vec8 = f16x8;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Elem<__bf16> {
  using vec8 = bf16x8;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float neg_inf() { return -__builtin_inff(); }

template <typename T, int D>
__global__ void __launch_bounds__(kThreads) pat_split_kernel(const SplitParams p) {
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  constexpr int KK = D / 32;             // MFMA k-steps across head_dim in S^T = K.Q^T
  constexpr int DB = D / 16;             // 16-wide head_dim blocks of O^T
  constexpr int NV = D / 16;             // 16-byte V loads per lane per 32-token step
  constexpr int CPR = D / 8;             // 16-byte pieces per token row
  constexpr int RS = D * 2 + 32;         // padded LDS row stride of the V tile, bytes
  constexpr int VSTAGE = kStepTokens * RS;
  constexpr int OROW = D + 4;            // padded row of the combine buffer, floats
  constexpr int COMBINE = kWaves * 16 * OROW * 4;
  constexpr int SMEM = (kWaves * VSTAGE > COMBINE) ? kWaves * VSTAGE : COMBINE;

  __shared__ __attribute__((aligned(16))) char smem[SMEM];
  __shared__ int s_pages[kMaxChunkPages];
  __shared__ float s_m[kWaves][16];
  __shared__ float s_l[kWaves][16];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int g = lane >> 4;   // lane group 0..3
  const int n = lane & 15;   // index inside the group

  // ---- which (bucket, box, chunk, kv-head) is this workgroup? -----------------
  const int wg = blockIdx.x;
  int bi = 0;
  for (int i = 1; i < p.num_buckets; ++i)
    if (wg >= p.bucket[i].wg_begin) bi = i;
  const BucketDev& bk = p.bucket[bi];
  int local = wg - bk.wg_begin;
  const int head = local % p.kv_heads;
  local /= p.kv_heads;
  const int chunk = local % bk.chunks;
  const int box = local / bk.chunks;
  if (box >= bk.num_boxes) return;

  const int G = p.group;
  const int rank = bk.rank[box];
  int nseq = bk.num_seqs[box];
  nseq = nseq < 0 ? 0 : (nseq > bk.max_seqs ? bk.max_seqs : nseq);
  int R = nseq * G;
  if (R > 64) R = 64;
  const bool tall = bk.row_tiles > 1;            // rows split across waves instead of KV steps
  const int row0 = tall ? wave * 16 : 0;         // first row of this wave's tile
  int kv = bk.kv[box];
  const int kv_cap = bk.max_blocks * p.page_size;
  kv = kv < 0 ? 0 : (kv > kv_cap ? kv_cap : kv);
  const int t_begin = chunk * bk.chunk_tokens;
  const int* __restrict__ qt = bk.q_table + (int64_t)box * bk.q_stride;
  // Partial-slot ordinal of this box per sequence: the plan's own rank, or - when the caller
  // supplies it - the box's ordinal among the boxes of that sequence (always collision-free).
  const int* __restrict__ qs = bk.q_slot ? bk.q_slot + (int64_t)box * bk.q_stride : nullptr;
  auto slot_base = [&](int j) -> int {
    const int ord = qs ? qs[j] : rank;
    return ((unsigned)ord < (unsigned)p.max_split) ? ord * p.chunks_per_rank : -1;
  };

  // ---- slots of this rank nobody will fill are marked empty (-inf) -------------
  {
    const bool empty = t_begin >= kv;
    const int first = empty ? chunk : chunk + 1;
    const int last = (chunk == bk.chunks - 1) ? p.chunks_per_rank : chunk + 1;  // exclusive
    const int nmark = last - first;
    for (int idx = tid; idx < R * nmark; idx += kThreads) {
      const int r = idx / nmark, c = first + idx % nmark;
      const int s = qt[r / G];
      const int sb = slot_base(r / G);
      if ((unsigned)s < (unsigned)p.batch && sb >= 0) {
        const int hq = head * G + r % G;
        p.lse_part[((int64_t)s * p.heads + hq) * p.num_slots + sb + c] = neg_inf();
      }
    }
    if (empty) return;
  }
  const int t_end = (kv < t_begin + bk.chunk_tokens) ? kv : t_begin + bk.chunk_tokens;

  // ---- page ids of the chunk -> LDS ---------------------------------------------
  const int page = p.page_size;
  {
    const int* __restrict__ bt = bk.block_table + (int64_t)box * bk.bt_stride;
    const int first_page = t_begin / page;
    const int npages = (t_end - t_begin + page - 1) / page;
    for (int i = tid; i < npages; i += kThreads) {
      int pg = bt[first_page + i];
      pg = pg < 0 ? 0 : (pg >= p.num_pages ? p.num_pages - 1 : pg);
      s_pages[i] = pg;
    }
  }

  // ---- Q rows as MFMA B operand (lane (g, n): row row0 + n, dims kk*32 + g*8 .. +7) ----
  vec8 qreg[KK];
  {
    const int r = row0 + n;
    int s = -1;
    if (r < R) s = qt[r / G];
    const bool ok = (unsigned)s < (unsigned)p.batch;
    const T* qrow = (const T*)p.q + (ok ? ((int64_t)s * p.q_stride_b + (int64_t)(head * G + r % G) * p.q_stride_h) : 0);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      u32x4 raw = u32x4{0u, 0u, 0u, 0u};
      if (ok) raw = *(const u32x4*)(qrow + kk * 32 + g * 8);
      qreg[kk] = __builtin_bit_cast(vec8, raw);
    }
  }
  __syncthreads();  // s_pages visible

  const int nsteps = (t_end - t_begin + kStepTokens - 1) / kStepTokens;
  // KV steps of this wave: every 4th one (short boxes) or all of them (tall boxes, where a
  // wave whose rows are all padding has nothing to do)
  const int st_first = tall ? ((row0 < R) ? 0 : nsteps) : wave;
  const int st_stride = tall ? 1 : kWaves;
  const bool pow2 = (page & (page - 1)) == 0;
  const int pshift = 31 - __builtin_clz(page);
  const T* __restrict__ kbase = (const T*)p.k + (int64_t)head * p.k_stride_h;
  const T* __restrict__ vbase = (const T*)p.v + (int64_t)head * p.v_stride_h;

  // address of token (chunk-relative index rel) in K or V
  auto token_ptr = [&](const T* base, int64_t stride_page, int64_t stride_slot, int rel) {
    int pidx, sl;
    if (pow2) { pidx = rel >> pshift; sl = rel & (page - 1); }
    else { pidx = rel / page; sl = rel - pidx * page; }
    return base + (int64_t)s_pages[pidx] * stride_page + (int64_t)sl * stride_slot;
  };
  const int last_rel = t_end - t_begin - 1;

  u32x4 kraw[2][KK], vraw[NV];
  auto load_step = [&](int st) {
    const int rel0 = st * kStepTokens;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      int rel = rel0 + a * 16 + n;
      rel = rel > last_rel ? last_rel : rel;
      const T* row = token_ptr(kbase, p.k_stride_page, p.k_stride_slot, rel) + g * 8;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kraw[a][kk] = *(const u32x4*)(row + kk * 32);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int piece = j * 64 + lane;
      int rel = rel0 + piece / CPR;
      rel = rel > last_rel ? last_rel : rel;
      const T* row = token_ptr(vbase, p.v_stride_page, p.v_stride_slot, rel);
      vraw[j] = *(const u32x4*)(row + (piece % CPR) * 8);
    }
  };

  float m_run = neg_inf(), l_run = 0.f;
  f32x4 acc_o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc_o[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  char* vstage = smem + wave * VSTAGE;
  if (st_first < nsteps) load_step(st_first);

  for (int st = st_first; st < nsteps; st += st_stride) {
    // current tile -> registers of this iteration; start fetching the next one
    u32x4 kcur[2][KK], vcur[NV];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) kcur[a][kk] = kraw[a][kk];
#pragma unroll
    for (int j = 0; j < NV; ++j) vcur[j] = vraw[j];
    if (st + st_stride < nsteps) load_step(st + st_stride);

    // V tile -> this wave's LDS region, row-major with padded rows
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int piece = j * 64 + lane;
      *(PAT_LDS u32x4*)((PAT_LDS char*)vstage + (piece / CPR) * RS + (piece % CPR) * 16) = vcur[j];
    }

    // S^T = K.Q^T for the two 16-token halves of the step
    f32x4 sc[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
        acc = E::mfma(__builtin_bit_cast(vec8, kcur[a][kk]), qreg[kk], acc);
      sc[a] = acc * p.scale_log2;
    }
    const int t0 = t_begin + st * kStepTokens;
    if (t0 + kStepTokens > t_end) {
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (t0 + a * 16 + g * 4 + i >= t_end) sc[a][i] = neg_inf();
    }

    // online softmax; the row's running max is shared by its 4 lanes, the sum stays per lane
    float mx = fmaxf(fmaxf(fmaxf(sc[0][0], sc[0][1]), fmaxf(sc[0][2], sc[0][3])),
                     fmaxf(fmaxf(sc[1][0], sc[1][1]), fmaxf(sc[1][2], sc[1][3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    float psum = 0.f;
    vec8 pv;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e = fast_exp2(sc[a][i] - m_new);
        psum += e;
        pv[a * 4 + i] = (T)e;
      }
    l_run = l_run * alpha + psum;

    // O^T += V^T.P^T. V^T operand: lane (g, n) of d-block db gets 8 tokens of column db*16 + n:
    // tokens g*4..g*4+3 of each 16-token half, matching the accumulator layout of S^T.
    {
      const int rrow = g * 4 + (n >> 2);
      const PAT_LDS char* src = (const PAT_LDS char*)vstage + rrow * RS + (n & 3) * 8;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PAT_LDS s16x4*)(src + db * 32));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PAT_LDS s16x4*)(src + 16 * RS + db * 32));
        s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        acc_o[db] = acc_o[db] * alpha;
        acc_o[db] = E::mfma(__builtin_bit_cast(vec8, both), pv, acc_o[db]);
      }
    }
  }

  // the row's sum over all of this wave's tokens
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);

  if (tall) {
    // ---- tall box: this wave holds the finished rows row0..row0+15 of the chunk -----------
    const int r = row0 + n;
    if (r < R) {
      const int s = qt[r / G];
      const int sb = slot_base(r / G);
      if ((unsigned)s < (unsigned)p.batch && sb >= 0) {
        const int hq = head * G + r % G;
        const int64_t prow = ((int64_t)s * p.heads + hq) * p.num_slots + sb + chunk;
        const float inv = 1.f / l_run;
        float* dst = p.o_part + prow * D + g * 4;
#pragma unroll
        for (int db = 0; db < DB; ++db) *(f32x4*)(dst + db * 16) = acc_o[db] * inv;
        if (g == 0) p.lse_part[prow] = (m_run + __builtin_amdgcn_logf(l_run)) * 0.6931471805599453f;
      }
    }
    return;
  }

  // ---- short box: combine the 4 waves' states through LDS and write the partial -------------
  float* cbuf = (float*)smem;
  const int crow = tid >> 4;                 // row this thread finalises
  const int ccol = (tid & 15) * (D / 16);    // its first column
  __syncthreads();  // every wave is done with its V staging region
  if (g == 0) { s_m[wave][n] = m_run; s_l[wave][n] = l_run; }
#pragma unroll
  for (int db = 0; db < DB; ++db)
    *(f32x4*)(cbuf + (wave * 16 + n) * OROW + db * 16 + g * 4) = acc_o[db];
  __syncthreads();

  if (crow < R) {
    float mw[kWaves], mmax = neg_inf();
#pragma unroll
    for (int w = 0; w < kWaves; ++w) { mw[w] = s_m[w][crow]; mmax = fmaxf(mmax, mw[w]); }
    float wsum = 0.f, wgt[kWaves];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      wgt[w] = fast_exp2(mw[w] - mmax);   // a wave without steps has m = -inf -> weight 0
      wsum += wgt[w] * s_l[w][crow];
    }
    const float inv = 1.f / wsum;
    const int s = qt[crow / G];
    const int sb = slot_base(crow / G);
    if ((unsigned)s < (unsigned)p.batch && sb >= 0) {
      const int hq = head * G + crow % G;
      const int64_t prow = ((int64_t)s * p.heads + hq) * p.num_slots + sb + chunk;
      float* dst = p.o_part + prow * D + ccol;
#pragma unroll
      for (int c = 0; c < D / 16; c += 4) {
        f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kWaves; ++w)
          o += *(const f32x4*)(cbuf + (w * 16 + crow) * OROW + ccol + c) * wgt[w];
        *(f32x4*)(dst + c) = o * inv;
      }
      if ((tid & 15) == 0)
        p.lse_part[prow] = (mmax + __builtin_amdgcn_logf(wsum)) * 0.6931471805599453f;
    }
  }
}

// Host launcher: picks the instance for (element type, head_dim).
hipError_t launch_split(bool bf16, int head_dim, unsigned workgroups, hipStream_t stream,
                        const SplitParams& params) {
  void (*fn)(const SplitParams);
  if (bf16) fn = head_dim == 64 ? pat_split_kernel<__bf16, 64> : pat_split_kernel<__bf16, 128>;
  else fn = head_dim == 64 ? pat_split_kernel<_Float16, 64> : pat_split_kernel<_Float16, 128>;
  hipLaunchKernelGGL(fn, dim3(workgroups), dim3(kThreads), 0, stream, params);
  return hipGetLastError();
}

}  // namespace pat
