// Split-KV forward kernel for gfx950 (MI355X): one workgroup streams one chunk of one
// packed box's KV for one kv-head and one 16-row tile of the box, and writes a normalised
// partial output + LSE per row.
//
// Functional contract (what the reference's pat_fwd_splitkv_kernel computes,
// csrc/pat_fwd_kernel.h:25-299): rows r = g + G*j of a box are (sequence
// q_table[j], query head h*G + g); every row attends to the same kv tokens, found
// through the box's block table; the partial result is softmax(q.K^T*scale).V over
// those tokens plus LSE = max + ln(sum) (csrc/softmax.h:169-188).
//
// Mapping to the hardware (this kernel's own design):
//  * work item = (box, kv-head, KV chunk), one workgroup of 4 wave64 each, launched as a flat
//    list with the kv-head fastest: workgroups are dealt to the 8 XCDs round-robin, so with 8
//    kv-heads XCD x serves head x and boxes that share KV pages (the boxes of one prefix node)
//    find them in that XCD's L2. Inside a bucket the list is chunk-major. What a workgroup is to do
//    it reads from its launch record (fwd_params.hpp), written once per plan by the record kernel.
//  * buckets of very short boxes: one workgroup serves 4 kv heads, one per wave, each wave
//    walking its head's steps alone (no combine).
//  * boxes of up to 16 rows (one MFMA row tile): each wave owns every 4th 32-token step of
//    the chunk on wave-private tiles and runs an independent online softmax; the 4 states are
//    combined through LDS at the end. K rows are the MFMA A operand of S^T = K.Q^T, so a lane
//    loads 16 contiguous bytes of one token straight from HBM into operand layout (no LDS).
//  * boxes of 17..64 rows: 32-row tiles on v_mfma_f32_32x32x16. All waves walk the chunk in
//    super-steps of 64 tokens whose K and V tiles are fetched once per workgroup (coalesced
//    256-byte rows, two super-steps ahead in registers) into a two-stage LDS buffer; wave w works on
//    rows 32(w&1).. and on tokens 32(w>>1).. of every super-step, so the two wave pairs run
//    independent online softmaxes over alternate 32-token steps and are combined through LDS at the
//    end. Per row and token that is half the MFMA, operand-read and softmax instructions of
//    16-row tiles.
//  * S^T on v_mfma_f32_16x16x32 (32x32x16 for tall boxes); its accumulator layout is the B-operand
//    layout of O^T = V^T.P^T, so P never moves between lanes.
//  * V must be contracted along tokens but is contiguous along head_dim: V tiles sit row-major
//    in padded LDS rows and are read back transposed with ds_read_b64_tr_b16.
//  * all softmax state of a row lives in the 4 lanes {n, n+16, n+32, n+48}.
//  * the chunk's page ids live in two VGPRs per wave (lane i holds page i) and are
//    broadcast with v_readlane; with the launch record the prologue is two dependent memory
//    round trips: {record: header, sequence ids, slots, page ids} -> {K, V, Q}.
#include <hip/hip_runtime.h>

#include <mutex>
#include <type_traits>

#include "fwd_params.hpp"
#include "lane_ops.hpp"

namespace pat {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
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
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Elem<__bf16> {
  using vec8 = bf16x8;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float neg_inf() { return -__builtin_inff(); }

// Tuning knob: steps a wave keeps in flight on wave-private tiles (measured on MI355X: deeper rings
// lose more to registers and to late-arriving first tiles than they gain).
#ifndef PAT_DEPTH
#define PAT_DEPTH 1
#endif

// Two forms of the tall path (boxes of 17..64 rows), one kernel instance each:
//  TALLK 32: 32-row tiles on 32x32x16 MFMAs, 64-token super-steps; the faster walk of a tall box
//            (a lone workgroup: 1.1-1.3 us per 64 tokens), at the price of 64 accumulator registers
//            and 75 KB of LDS: 2 workgroups per CU at head_dim 128;
//  TALLK 16: a 16-row tile per wave on 16x16x32 MFMAs, 32-token steps, three steps ahead in registers
//            (1.7 us per 64 tokens), in the register and LDS budget of the <= 16-row path: 3 per CU.
// The host picks per launch: 32 where the tall boxes are what the launch waits for, 16 where the
// <= 16-row boxes are and the third resident workgroup per CU is worth more (pat_fwd_tuning.tall_rows).
__host__ __device__ constexpr int split_occupancy(int head_dim, int tallk) {
  return (head_dim == 128 && tallk == 32) ? 2 : 3;
}

// LDS bytes of one workgroup (dynamic: more than the 64 KB a static allocation may have).
__host__ __device__ constexpr int split_smem_bytes(int D, int tallk) {
  const int wave_private = kWaves * kStepTokens * (D * 2 + 32);     // 4 private V tiles
  const int combine = kWaves * 16 * (D + 4) * 4;                     // short boxes: the waves' states
  const int tall = tallk == 32 ? 2 * (2 * kStepTokens) * ((D * 2 + 16) + (D * 2 + 64))   // two stages of 64 K rows + 64 V rows
                               : 2 * kStepTokens * ((D * 2 + 16) + (D * 2 + 32));        // two stages of 32 K rows + 32 V rows
  int m = wave_private > combine ? wave_private : combine;
  return m > tall ? m : tall;
}

// DIRECT instances serve launches in which every row has one partial slot: they store `out`.
template <typename T, int D, bool DIRECT, int TALLK>
__global__ void __launch_bounds__(kThreads, split_occupancy(D, TALLK)) pat_split_kernel(const char* __restrict__ records, const int record_stride,
                                                                             const int record_max_seqs, const SplitParams p) {
  using E = Elem<T>;
  using vec8 = typename E::vec8;
  constexpr int KK = D / 32;             // MFMA k-steps across head_dim in S^T = K.Q^T (16x16x32 tiles)
  constexpr int DB = D / 16;             // 16-wide head_dim blocks of O^T (16x16x32 tiles)
  constexpr int NV = D / 16;             // 16-byte V loads per lane per step (wave-private tiles)
  constexpr int DEPTH = PAT_DEPTH;       // wave-private tiles: steps kept in flight per wave
  constexpr int CPR = D / 8;             // 16-byte pieces per token row
  constexpr int TPL = 64 / CPR;          // tokens covered by one wave-wide load instruction
  constexpr int RSV = D * 2 + 32;        // LDS row stride of a wave-private V tile (conflict-free transposed reads)
  constexpr int VSTAGE = kStepTokens * RSV;            // one wave's private V tile
  constexpr int OROW = D + 4;            // padded row of the combine buffer, floats
  constexpr int WSTAGE = VSTAGE;                       // one wave's private staging (V only)

  extern __shared__ __attribute__((aligned(16))) char smem[];
  __shared__ float s_m[kWaves * 16];
  __shared__ float s_l[kWaves * 16];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int g = lane >> 4;   // 16-row tiles: lane group 0..3
  const int n = lane & 15;   //               index inside the group
  const int h2 = lane >> 5;  // 32-row tiles: lane half
  const int n32 = lane & 31; //               index inside the half

  // ---- this workgroup's launch record: one round trip for everything the plan says about it ---
  // (header, sequence ids and partial-result slots of its rows, page ids of its piece: checked,
  // clamped and laid out by the record kernel once per plan). The launch is a flat list of
  // workgroups; consecutive ones serve consecutive kv heads of one piece (workgroups are dealt to
  // the 8 XCDs round-robin, so with 8 kv heads XCD x serves head x and the boxes that share KV
  // pages find them in that XCD's L2), and inside a bucket the list is chunk-major.
  // (the grid is padded to whole slices of kGridX only beyond 2^20 workgroups; the padding has
  // records too, empty ones, so nothing here waits for a bound from the kernel arguments)
  const unsigned wg_id = blockIdx.y * (unsigned)kGridX + blockIdx.x;
  const char* __restrict__ rec = records + (size_t)wg_id * (unsigned)record_stride;
  const int4 rh0 = *(const int4*)rec;
  const int4 rh1 = *(const int4*)(rec + 16);
  // The piece's length, twice: as a scalar for the loops of the tall path, and laundered
  // into a vector register for the wave-private path. With loop bounds it can prove uniform the
  // compiler schedules the wave-private loops for 50 more registers; with vector bounds in the
  // tall path its per-step branches turn into masked execution of both sides.
  int ntok_v = rh0.x;
  asm volatile("" : "+v"(ntok_v));
  const int ntok = ntok_v;
  const int ntok_u = __builtin_amdgcn_readfirstlane(rh0.x);
  const int R = __builtin_amdgcn_readfirstlane(rh0.y);
  const int mode = __builtin_amdgcn_readfirstlane(rh0.z);
  const bool head_per_wave = (mode & kRecordModeHeadPerWave) != 0;
  // Boxes of up to 16 rows: the 4 waves split the piece's steps, each on wave-private tiles (or,
  // with a kv head per wave, each wave walks all steps of its own head).
  // Taller boxes: wave w owns rows 32(w&1).. and tokens 32(w>>1).. of every 64-token super-step,
  // on tiles shared through LDS.
  const bool tall = (mode & 0xff) > 1;
  // (both uniform, and known to be: branches on them are scalar branches)
  const int rt = __builtin_amdgcn_readfirstlane(wave & 1);   // tall boxes: this wave's 32-row tile
  const int ph = __builtin_amdgcn_readfirstlane(wave >> 1);  //             and which half of a super-step it works on
  // (uniform over the wave: kept in a scalar register so that address arithmetic stays scalar)
  const int head = __builtin_amdgcn_readfirstlane(rh0.w + (head_per_wave ? (int)(threadIdx.x >> 6) : 0));
  const int fill_begin = __builtin_amdgcn_readfirstlane(rh1.x);
  const int fill_end = __builtin_amdgcn_readfirstlane(rh1.y);
  const int G = p.group;                       // 1, 2, 4 or 8 (checked on the host)
  const int gshift = 31 - __builtin_clz(G);
  const int page = p.page_size;
  // this lane's row: sequence id and partial-result slot (-1: no such row)
  const int my_row = tall ? (TALLK == 32 ? rt * 32 + n32 : wave * 16 + n) : n;
  const int my_j = my_row >> gshift;
  const bool j_ok = (my_row < R) && my_j < record_max_seqs;
  const int* __restrict__ rows_tab = (const int*)(rec + sizeof(RecordHead));
  const int my_seq = j_ok ? rows_tab[my_j] : -1;
  const int my_sl = j_ok ? rows_tab[record_max_seqs + my_j] : -1;
  // page ids of the piece: lane i of every wave holds pages i and 64 + i (the record kernel
  // filled all kMaxChunkPages-or-fewer entries it reserved, so no bound is checked here)
  const int* __restrict__ pages_tab = rows_tab + 2 * record_max_seqs;
  const int npages = (ntok + page - 1) / page;
  const int pg0 = (lane < npages) ? pages_tab[lane] : 0;
  const int pg1 = (64 + lane < npages) ? pages_tab[64 + lane] : 0;

  const bool has_rows = !tall || (TALLK == 32 ? rt * 32 : wave * 16) < R;   // false: a wave that only helps loading shared tiles
  const bool row_ok = my_seq >= 0 && my_sl >= 0;
  const int my_hq = head * G + (my_row & (G - 1));
  // partial slot of (my row, this piece); -1: the row is not to be written
  const int my_slot0 = row_ok ? (my_seq * p.heads + my_hq) * p.num_slots + my_sl : -1;
  // the one lane per row that writes what exists once per row (LSE, empty-slot marks)
  const bool row_lead = tall ? (TALLK == 32 ? (ph == 0 && h2 == 0) : g == 0) : ((head_per_wave || wave == 0) && g == 0);

  // ---- where a finished row goes ---------------------------------------------------------
  // Normally into its partial slot (fp32, merged by the second kernel). A launch in which every
  // row has exactly one slot (no sequence in two boxes, no box in two chunks) has nothing to
  // merge: its rows go straight to `out` in the output type (the reference does the same when
  // max_split_per_seq is 1, csrc/api.h:230-238). A row's slot index is then its (sequence, head)
  // pair.
  constexpr bool direct = DIRECT;
  auto row_out = [&](int slot0) -> T* {
    const int s_ = slot0 / p.heads;
    return (T*)p.out + (int64_t)s_ * p.o_stride_b + (int64_t)(slot0 - s_ * p.heads) * p.o_stride_h;
  };
  auto put4 = [&](float* part, T* out, f32x4 v) {
    if (direct) {
      typedef T tx4 __attribute__((ext_vector_type(4)));
      *(tx4*)out = tx4{(T)v[0], (T)v[1], (T)v[2], (T)v[3]};
    } else {
      *(f32x4*)part = v;
    }
  };
  auto put_lse = [&](int64_t prow, float lse) {
    if (!direct) p.lse_part[prow] = lse;
    else if (p.lse_out != nullptr) p.lse_out[prow] = lse;
  };

  // ---- slots of these rows that no workgroup will fill are marked empty (-inf) -----------
  {
    const bool empty = ntok <= 0;
    const bool marker = row_lead && my_slot0 >= 0;
    if (direct) {
      // (one piece per box: only a box without tokens gets here; its rows are zero, LSE -inf)
      if (empty && marker) {
        T* o = row_out(my_slot0);
        for (int c = 0; c < D; c += 4) put4(nullptr, o + c, f32x4{0.f, 0.f, 0.f, 0.f});
        put_lse(my_slot0, neg_inf());
      }
    } else if (marker)
      for (int c = fill_begin; c < fill_end; ++c) p.lse_part[my_slot0 + c] = neg_inf();
    if (empty) return;
  }
  const int t_begin = 0, t_end = ntok;   // token positions are piece-relative from here on
  const int last_rel = ntok - 1;
  const int nsteps = (ntok + kStepTokens - 1) / kStepTokens;

  // ---- addressing ---------------------------------------------------------------------------
  // A 16-token half of a step never straddles a page, so its rows share one base address that is
  // uniform over the wave (page id broadcast with v_readlane, 64-bit arithmetic on the scalar
  // unit) and every lane adds a 32-bit byte offset that does not change from step to step.
  const int hpp = page >> 4;                                   // halves per page
  const int hshift = ((hpp & (hpp - 1)) == 0) ? 31 - __builtin_clz(hpp) : -1;
  const int64_t ksp = p.k_stride_page * (int64_t)sizeof(T), kss = p.k_stride_slot * (int64_t)sizeof(T);
  const int64_t vsp = p.v_stride_page * (int64_t)sizeof(T), vss = p.v_stride_slot * (int64_t)sizeof(T);
  const char* __restrict__ kbase = (const char*)p.k + (int64_t)head * p.k_stride_h * (int64_t)sizeof(T);
  const char* __restrict__ vbase = (const char*)p.v + (int64_t)head * p.v_stride_h * (int64_t)sizeof(T);

  // base address of half h (chunk-relative, uniform, h * 16 <= last_rel)
  auto half_base = [&](const char* base, int64_t sp, int64_t ss, int h) -> const char* {
    int pidx, s16;
    if (hshift >= 0) { pidx = h >> hshift; s16 = h & (hpp - 1); }
    else { pidx = (int)__umulhi((unsigned)h, p.hpp_magic); s16 = h - pidx * hpp; }
    const int pg = __builtin_amdgcn_readlane(pidx < 64 ? pg0 : pg1, pidx & 63);
    return base + (int64_t)pg * sp + (int64_t)(s16 * 16) * ss;
  };
  // per-lane address of token tok (chunk-relative; clamped to the last valid token, whose score
  // is masked and whose probability is 0 wherever it stands in for a token past the end). Only
  // the last, partial step of a chunk takes this slower route.
  auto lane_row = [&](const char* base, int64_t sp, int64_t ss, int tok) -> const char* {
    tok = tok > last_rel ? last_rel : tok;
    const int h = tok >> 4;
    int pidx, s16;
    if (hshift >= 0) { pidx = h >> hshift; s16 = h & (hpp - 1); }
    else { pidx = (int)__umulhi((unsigned)h, p.hpp_magic); s16 = h - pidx * hpp; }
    const int pg = __shfl(pidx < 64 ? pg0 : pg1, pidx & 63);
    return base + (int64_t)pg * sp + (int64_t)(s16 * 16 + (tok & 15)) * ss;
  };

  // Half h of the chunk as the loads see it (uniform over the wave): the half that holds its rows
  // and, in `lim`, the last row of that half that exists. Rows past the end of the chunk re-read
  // the chunk's last token (their scores are masked and their probabilities are 0); a half that
  // lies wholly past the end stands in for the half of that token.
  auto half_geom = [&](int h, int& lim) -> int {
    const int left = last_rel - h * 16;
    lim = left < 0 ? (last_rel & 15) : (left > 15 ? 15 : left);
    return left < 0 ? (last_rel >> 4) : h;
  };

  // Q rows as MFMA B operand of the 16x16x32 tiles (lane (g, n): row n, dims kk*32 + g*8 .. +7)
  vec8 qreg[KK];
  auto load_q = [&]() {
    const bool ok = my_seq >= 0;
    const T* qrow = (const T*)p.q + (ok ? ((int64_t)my_seq * p.q_stride_b + (int64_t)my_hq * p.q_stride_h) : 0);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      u32x4 raw = u32x4{0u, 0u, 0u, 0u};
      if (ok) raw = *(const u32x4*)(qrow + kk * 32 + g * 8);
      qreg[kk] = __builtin_bit_cast(vec8, raw);
    }
  };

  float m_run = neg_inf(), l_run = 0.f;
  f32x4 acc_o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc_o[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  // One 32-token step of online-softmax attention for this wave's 16 rows. k_op(a, kk) yields the
  // K operand of half a / k-step kk; vtile is a row-major V tile in LDS with row stride RSV.
  // after_scores() runs once the K operands have been consumed: the caller refills their
  // registers there, so the next step's K is in flight during the softmax and the PV product.
  auto attend = [&](auto k_op, const PAT_LDS char* vtile, int t0, auto after_scores) {
    f32x4 sc[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) acc = E::mfma(k_op(a, kk), qreg[kk], acc);
      sc[a] = acc * p.scale_log2;
    }
    after_scores();
    if (t0 + kStepTokens > t_end) {
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (t0 + a * 16 + g * 4 + i >= t_end) sc[a][i] = neg_inf();
    }
    // the row's running max is shared by its 4 lanes, the sum stays per lane until the end
    float mx = fmaxf(fmaxf(fmaxf(sc[0][0], sc[0][1]), fmaxf(sc[0][2], sc[0][3])),
                     fmaxf(fmaxf(sc[1][0], sc[1][1]), fmaxf(sc[1][2], sc[1][3])));
    mx = max_xor32(max_xor16(mx));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = fast_exp2(m_run - m_new);
    // once the running maxima have settled no row of the wave needs its accumulator rescaled
    const bool rescale = __builtin_amdgcn_ballot_w64(m_new != m_run) != 0;
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
    if (rescale) {
      asm volatile("" ::: "memory");   // a real branch: if-converted, the skipped multiplies come back as selects
#pragma unroll
      for (int db = 0; db < DB; ++db) acc_o[db] = acc_o[db] * alpha;
    }
    // O^T += V^T.P^T. V^T operand: lane (g, n) of d-block db gets 8 tokens of column db*16 + n:
    // tokens g*4..g*4+3 of each 16-token half, matching the accumulator layout of S^T.
    const PAT_LDS char* src = vtile + (g * 4 + (n >> 2)) * RSV + (n & 3) * 8;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PAT_LDS s16x4*)(src + db * 32));
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PAT_LDS s16x4*)(src + 16 * RSV + db * 32));
      s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      acc_o[db] = E::mfma(__builtin_bit_cast(vec8, both), pv, acc_o[db]);
    }
  };

  if (tall) {
    if constexpr (TALLK == 16) {
    constexpr int NP = D / 64;             // 16-byte K (and V) loads per thread per step
    constexpr int PF = 3;                  // steps kept in flight per workgroup (a 4th costs the registers that let the operand
                                           // reads of a step run ahead of its MFMAs: lone tall workgroups 6 % slower per step)
    constexpr int RSK = D * 2 + 16;        // LDS row stride of a K tile (conflict-free 16-byte row reads)
    constexpr int SHARED = kStepTokens * (RSK + RSV);    // one K + V stage
    static_assert(2 * SHARED <= split_smem_bytes(D, 16), "LDS size");
    const int nsteps_u = (ntok_u + kStepTokens - 1) / kStepTokens;
    // ============ tall box, 16-row tile per wave: 32-token tiles shared through LDS ============
    // Each step's K and V tile is fetched once per workgroup: thread t loads pieces t, t + 256 ..
    // of the tile (16 lanes cover one 256-byte row), PF steps ahead, and drops them into one of
    // two LDS stages; after a barrier every wave runs its own 16 rows against the stage.
    u32x4 kst[PF][NP], vst[PF][NP];
    int tok_in[NP];
    unsigned koff[NP], voff[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      tok_in[i] = (i * kThreads + tid) / CPR;                 // token of the step, 0..31
      const unsigned col = ((i * kThreads + tid) % CPR) * 16;
      koff[i] = (unsigned)((tok_in[i] & 15) * kss) + col;
      voff[i] = (unsigned)((tok_in[i] & 15) * vss) + col;
    }
    // Steps are fetched in order, so the half a wave reads next is tracked on the scalar unit
    // (page of the chunk, 16-token slot in the page, byte offset of the slot) instead of being
    // derived from the step number every time: a few scalar adds per half. Page strides are
    // below 4 GiB (checked on the host): page id x stride is one 32 x 32 -> 64 bit multiply.
    int f_page = 0, f_slot = 0;
    unsigned f_koff = 0, f_voff = 0;
    const unsigned ksp32 = (unsigned)ksp, vsp32 = (unsigned)vsp, k16 = (unsigned)(16 * kss), v16 = (unsigned)(16 * vss);
    auto next_half = [&]() {
      ++f_slot; f_koff += k16; f_voff += v16;
      if (f_slot == hpp) { f_slot = 0; f_koff = 0; f_voff = 0; ++f_page; }
    };
    // D = 64: one load per step and thread, waves 2 and 3 read the step's second half
    if (NP == 1 && __builtin_amdgcn_readfirstlane(wave >> 1)) next_half();
    auto fetch = [&](int st, u32x4 (&kd)[NP], u32x4 (&vd)[NP]) {
      if ((st + 1) * kStepTokens <= ntok_u) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
          const unsigned pg = (unsigned)__builtin_amdgcn_readlane(f_page < 64 ? pg0 : pg1, f_page & 63);
          kd[i] = *(const u32x4*)(kbase + ((uint64_t)pg * ksp32 + f_koff) + koff[i]);
          vd[i] = *(const u32x4*)(vbase + ((uint64_t)pg * vsp32 + f_voff) + voff[i]);
          next_half();
        }
        if (NP == 1) next_half();
      } else {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
          const unsigned col = ((i * kThreads + tid) % CPR) * 16;
          kd[i] = *(const u32x4*)(lane_row(kbase, ksp, kss, st * kStepTokens + tok_in[i]) + col);
          vd[i] = *(const u32x4*)(lane_row(vbase, vsp, vss, st * kStepTokens + tok_in[i]) + col);
        }
      }
    };
#pragma unroll
    for (int s = 0; s < PF; ++s)
      if (s < nsteps_u) fetch(s, kst[s], vst[s]);
    load_q();
    for (int st0 = 0; st0 < nsteps_u; st0 += PF) {
#pragma unroll
      for (int s = 0; s < PF; ++s) {
        const int st = st0 + s;
        if (st >= nsteps_u) break;
        PAT_LDS char* stage = (PAT_LDS char*)smem + (st & 1) * SHARED;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
          const int tok_in = (i * kThreads + tid) / CPR;
          const int col16 = ((i * kThreads + tid) % CPR) * 16;
          *(PAT_LDS u32x4*)(stage + tok_in * RSK + col16) = kst[s][i];
          *(PAT_LDS u32x4*)(stage + kStepTokens * RSK + tok_in * RSV + col16) = vst[s][i];
        }
        if (st + PF < nsteps_u) fetch(st + PF, kst[s], vst[s]);
        __syncthreads();
        if (has_rows)
          attend([&](int a, int kk) { return *(const PAT_LDS vec8*)(stage + (a * 16 + n) * RSK + (kk * 32 + g * 8) * 2); },
                 stage + kStepTokens * RSK, t_begin + st * kStepTokens, []() {});
      }
    }
    l_run = sum_xor32(sum_xor16(l_run));
    if (my_slot0 >= 0) {
      const int64_t prow = (int64_t)my_slot0;
      const float inv = 1.f / l_run;
      float* dst = p.o_part + prow * D + g * 4;
      T* o = direct ? row_out(my_slot0) + g * 4 : nullptr;
#pragma unroll
      for (int db = 0; db < DB; ++db) put4(dst + db * 16, o + db * 16, acc_o[db] * inv);
      if (g == 0) put_lse(prow, (m_run + __builtin_amdgcn_logf(l_run)) * 0.6931471805599453f);
    }
    } else {
    // ====================== tall box: 32-row tiles, K/V shared through LDS ======================
    // The chunk is walked in super-steps of 64 tokens. Thread t loads pieces t, t + 256 .. of a
    // super-step's K and V tiles (16 lanes cover one 256-byte row), PF2 super-steps ahead in
    // registers, and drops them into one of two LDS stages; after a barrier the wave pair ph = 0
    // runs tokens 0..31 of the stage and the pair ph = 1 tokens 32..63, each wave on its 32 rows.
    //   S^T = K.Q^T on 32x32x16 tiles: A = K (lane: token n32, dims 16kk + 8h2 ..+7, a 16-byte
    //   LDS read), B = Q^T in registers; the accumulator holds, in lane (n32, h2), row n32's scores
    //   for tokens 8b + 4h2 + r (register 4b + r).
    //   O^T += V^T.P^T: B = P^T straight from those registers - k index 8h2 + j of MFMA t stands
    //   for token 16t + 8(j>>2) + 4h2 + (j&3), any order does as long as V^T uses the same - and
    //   A = V^T read transposed from LDS (two 4-token groups per lane and MFMA). The row's softmax
    //   state lives in the two lanes n32 and n32 + 32.
    constexpr int KK2 = D / 16;            // MFMA k-steps across head_dim in S^T
    constexpr int DB2 = D / 32;            // 32-wide head_dim blocks of O^T
    constexpr int NP2 = D / 32;            // 16-byte K (and V) loads per thread and super-step
    constexpr int PF2 = 1;                 // super-steps in flight in registers beside the one in LDS (2: no faster, 34 more registers)
    constexpr int SST = 2 * kStepTokens;   // tokens per super-step
    constexpr int RSK2 = D * 2 + 16;       // LDS row stride of a K tile (conflict-free 16-byte row reads)
    constexpr int RSV2 = D * 2 + 64;       // LDS row stride of a V tile (conflict-free transposed reads)
    constexpr int STAGE2 = SST * (RSK2 + RSV2);
    constexpr int TPR = kThreads / CPR;    // tokens one load round of the workgroup covers: 16 (D 128) or 32 (D 64)
    static_assert(2 * STAGE2 <= split_smem_bytes(D, 32), "LDS size");
    static_assert(2 * (D / 8) * 64 * 16 <= 2 * STAGE2, "the exchange buffer of the epilogue fits the stages");
    const int nss_u = (ntok_u + SST - 1) / SST;
    const float sc_abs = __builtin_fabsf(p.scale_log2);

    // Q^T operand (lane (n32, h2): row n32, dims 16kk + 8h2 ..+7). A negative softmax scale is
    // folded into Q's sign (exact), so that the row maximum can be taken over the raw scores.
    vec8 q2[KK2];
    {
      const bool ok = my_seq >= 0;
      const T* qrow = (const T*)p.q + (ok ? ((int64_t)my_seq * p.q_stride_b + (int64_t)my_hq * p.q_stride_h) : 0);
      const unsigned flip = p.scale_log2 < 0.f ? 0x80008000u : 0u;
#pragma unroll
      for (int kk = 0; kk < KK2; ++kk) {
        u32x4 raw = u32x4{0u, 0u, 0u, 0u};
        if (ok) raw = *(const u32x4*)(qrow + kk * 16 + h2 * 8);
        raw = raw ^ u32x4{flip, flip, flip, flip};
        q2[kk] = __builtin_bit_cast(vec8, raw);
      }
    }
    f32x16 acc2[DB2];
#pragma unroll
    for (int db = 0; db < DB2; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc2[db][i] = 0.f;

    u32x4 kst[PF2][NP2], vst[PF2][NP2];
    const int tok_r = tid / CPR;                        // this thread's token within a load round
    const unsigned col16 = (unsigned)(tid % CPR) * 16u;
    const unsigned koff = (unsigned)((tok_r & 15) * kss) + col16;
    const unsigned voff = (unsigned)((tok_r & 15) * vss) + col16;
    // Where the next half (16 tokens) of the chunk lies. Fast route (pages of 16 tokens, K and V
    // laid out alike - two tensors of one shape or the two halves of one; the usual case): half h is
    // page h, its id comes out of the page registers with one v_readlane, the page's byte offset is
    // one 32 x 32 -> 64 bit scalar multiply (page strides are below 4 GiB, checked on the host), V's
    // address is K's plus the distance between the two caches, and the loads take the scalar address
    // plus a 32-bit lane offset that never changes. General route: the half is tracked on the scalar
    // unit (page of the chunk, slot in the page, byte offset of the slot), K and V apart.
    int f_page = 0, f_slot = 0;
    unsigned f_koff = 0, f_voff = 0;
    const unsigned ksp32 = (unsigned)ksp, vsp32 = (unsigned)vsp, k16 = (unsigned)(16 * kss), v16 = (unsigned)(16 * vss);
    // (pages of 32, 64 or 128 tokens take the same route with the half's place inside its page added)
    const int fast_route = (ksp == vsp && kss == vss) ? (hpp == 1 ? 1 : (hshift > 0 ? 2 : 0)) : 0;
    const int64_t kv_delta = vbase - kbase;
    auto next_half = [&]() {
      ++f_slot; f_koff += k16; f_voff += v16;
      if (f_slot == hpp) { f_slot = 0; f_koff = 0; f_voff = 0; ++f_page; }
    };
    // D = 64: a load round covers two halves, waves 2 and 3 read the second one
    const int wave_half = TPR == 32 ? __builtin_amdgcn_readfirstlane(wave >> 1) : 0;
    if (wave_half) next_half();
    auto fetch = [&](auto fast, int ss, u32x4 (&kd)[NP2], u32x4 (&vd)[NP2]) {
      if ((ss + 1) * SST <= ntok_u) {
        if (decltype(fast)::value == 1) {
          const int h0 = ss * (SST / 16) + wave_half;         // this wave's first half (= page) of the super-step
          const int pgsel = h0 < 64 ? pg0 : pg1;              // (a super-step's 4 pages lie in one register)
          // (kept out of loop-invariant hoisting: next to the scalar base the 32-bit offset becomes the
          // load's own offset operand instead of a 64-bit vector add per load)
          unsigned ko = koff, vo = voff;
          asm volatile("" : "+v"(ko), "+v"(vo));
#pragma unroll
          for (int i = 0; i < NP2; ++i) {
            const unsigned pg = (unsigned)__builtin_amdgcn_readlane(pgsel, (h0 + i * (TPR / 16)) & 63);
            const char* ka = kbase + (uint64_t)pg * ksp32;
            kd[i] = *(const u32x4*)(ka + ko);
            vd[i] = *(const u32x4*)(ka + kv_delta + vo);
          }
        } else if (decltype(fast)::value == 2) {
          const int h0 = ss * (SST / 16) + wave_half;         // this wave's first half of the super-step
          const int pgsel = (h0 >> hshift) < 64 ? pg0 : pg1;  // (a super-step's pages lie in one register)
          unsigned ko = koff, vo = voff;
          asm volatile("" : "+v"(ko), "+v"(vo));
#pragma unroll
          for (int i = 0; i < NP2; ++i) {
            const int hh = h0 + i * (TPR / 16);
            const unsigned pg = (unsigned)__builtin_amdgcn_readlane(pgsel, (hh >> hshift) & 63);
            const char* ka = kbase + ((uint64_t)pg * ksp32 + (unsigned)(hh & (hpp - 1)) * k16);
            kd[i] = *(const u32x4*)(ka + ko);
            vd[i] = *(const u32x4*)(ka + kv_delta + vo);
          }
        } else {
#pragma unroll
          for (int i = 0; i < NP2; ++i) {
            const unsigned pg = (unsigned)__builtin_amdgcn_readlane(f_page < 64 ? pg0 : pg1, f_page & 63);
            kd[i] = *(const u32x4*)(kbase + ((uint64_t)pg * ksp32 + f_koff) + koff);
            vd[i] = *(const u32x4*)(vbase + ((uint64_t)pg * vsp32 + f_voff) + voff);
            next_half();
            if (TPR == 32) next_half();
          }
        }
      } else {
        // the chunk's last, partial super-step: per-lane addresses, clamped to the last token
#pragma unroll
        for (int i = 0; i < NP2; ++i) {
          kd[i] = *(const u32x4*)(lane_row(kbase, ksp, kss, ss * SST + i * TPR + tok_r) + col16);
          vd[i] = *(const u32x4*)(lane_row(vbase, vsp, vss, ss * SST + i * TPR + tok_r) + col16);
        }
      }
    };

    // LDS offsets of this lane's operand reads inside a stage
    const unsigned k_rd = (unsigned)((ph * 32 + n32) * RSK2 + h2 * 16);
    const unsigned v_rd = (unsigned)(SST * RSK2 + (ph * 32 + h2 * 4 + (n >> 2)) * RSV2 + (g & 1) * 32 + (n & 3) * 8);

    // One 32-token step of online-softmax attention for this wave's 32 rows against a stage.
    auto attend32 = [&](const PAT_LDS char* stage, int t0) {
      // every K operand of the step is requested before the first MFMA waits for one (left alone, the
      // compiler reads each operand right ahead of its use and exposes the LDS latency KK2 times)
      vec8 kop[KK2];
#pragma unroll
      for (int kk = 0; kk < KK2; ++kk) kop[kk] = *(const PAT_LDS vec8*)(stage + k_rd + kk * 32);
      __builtin_amdgcn_sched_barrier(0);
      f32x16 s;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
      for (int kk = 0; kk < KK2; ++kk) s = E::mfma32(kop[kk], q2[kk], s);
      // The rows' reference maxima move only when some row's maximum has left a window of kLazy
      // (base-2 exponent units) above its reference: probabilities then reach 2^kLazy at most, which
      // fp32 sums and 16-bit P hold as well as values below 1, and the accumulator is rescaled a few
      // times per chunk instead of at nearly every step (with 32 rows per wave some row's maximum
      // moves at almost every step).
      constexpr float kLazy = 8.f;
      float e[16];
      float mx;
      const bool full = t0 + kStepTokens <= ntok_u;
      if (full) {
        mx = s[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[i]);
        mx = max_xor32(mx) * sc_abs;
      } else {
        // the chunk's last step: tokens past its end are masked
        mx = neg_inf();
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int tok = t0 + (i >> 2) * 8 + h2 * 4 + (i & 3);
          e[i] = tok < ntok_u ? s[i] * sc_abs : neg_inf();
          mx = fmaxf(mx, e[i]);
        }
        mx = max_xor32(mx);
      }
      if (__builtin_amdgcn_ballot_w64(mx > m_run + kLazy) != 0) {
        asm volatile("" ::: "memory");   // a real branch: if-converted, the skipped multiplies come back as selects
        const float m_new = fmaxf(m_run, mx);
        const float alpha = fast_exp2(m_run - m_new);   // (first step: m_run = -inf, alpha = 0)
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < DB2; ++db) acc2[db] = acc2[db] * alpha;
      }
      if (full) {
#pragma unroll
        for (int i = 0; i < 16; ++i) e[i] = fast_exp2(__builtin_fmaf(s[i], sc_abs, -m_run));
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) e[i] = fast_exp2(e[i] - m_run);
      }
      float psum = 0.f;
      vec8 pv[2];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        psum += e[i];
        pv[i >> 3][i & 7] = (T)e[i];
      }
      l_run += psum;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int db = 0; db < DB2; ++db) {
          const PAT_LDS char* src = stage + v_rd + t * 16 * RSV2 + db * 64;
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PAT_LDS s16x4*)src);
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((PAT_LDS s16x4*)(src + 8 * RSV2));
          s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          acc2[db] = E::mfma32(__builtin_bit_cast(vec8, both), pv[t], acc2[db]);
        }
    };

    // LDS offsets of this thread's tile writes inside a stage (round i: + i * TPR rows)
    const unsigned k_wr = (unsigned)(tok_r * RSK2) + col16;
    const unsigned v_wr = (unsigned)(SST * RSK2 + tok_r * RSV2) + col16;
    auto walk = [&](auto same) {
#pragma unroll
      for (int s = 0; s < PF2; ++s)
        if (s < nss_u) fetch(same, s, kst[s], vst[s]);
      for (int ss0 = 0; ss0 < nss_u; ss0 += PF2) {
#pragma unroll
        for (int s = 0; s < PF2; ++s) {
          const int ss = ss0 + s;
          if (ss >= nss_u) break;
          PAT_LDS char* stage = (PAT_LDS char*)smem + (ss & 1) * STAGE2;
          PAT_LDS char* kw = stage + k_wr;
          PAT_LDS char* vw = stage + v_wr;
#pragma unroll
          for (int i = 0; i < NP2; ++i) {
            *(PAT_LDS u32x4*)(kw + i * TPR * RSK2) = kst[s][i];
            *(PAT_LDS u32x4*)(vw + i * TPR * RSV2) = vst[s][i];
          }
          if (ss + PF2 < nss_u) fetch(same, ss + PF2, kst[s], vst[s]);
          __syncthreads();
          if (has_rows && ss * SST + ph * kStepTokens < ntok_u) attend32(stage, ss * SST + ph * kStepTokens);
        }
      }
    };
    if (fast_route == 1) walk(std::integral_constant<int, 1>{});
    else if (fast_route == 2) walk(std::integral_constant<int, 2>{});
    else walk(std::integral_constant<int, 0>{});
    // ---- the two wave pairs' states of the same rows are combined through LDS ----------------
    l_run = sum_xor32(l_run);
    float* xbuf = (float*)smem;                 // [rt][DB2 * 4 pieces][64 lanes] x 16 bytes
    __syncthreads();                            // every wave is done with the stages
    if (ph == 1 && has_rows) {
#pragma unroll
      for (int db = 0; db < DB2; ++db)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          *(f32x4*)(xbuf + (((rt * DB2 + db) * 4 + b) * 64 + lane) * 4) =
              f32x4{acc2[db][4 * b], acc2[db][4 * b + 1], acc2[db][4 * b + 2], acc2[db][4 * b + 3]};
      if (h2 == 0) { s_m[rt * 32 + n32] = m_run; s_l[rt * 32 + n32] = l_run; }
    }
    __syncthreads();
    if (ph == 0 && has_rows && my_slot0 >= 0) {
      const float m1 = s_m[rt * 32 + n32], l1 = s_l[rt * 32 + n32];   // (a pair without steps: -inf, 0)
      const float mm = fmaxf(m_run, m1);
      const float w0 = fast_exp2(m_run - mm), w1 = fast_exp2(m1 - mm);
      const float lsum = l_run * w0 + l1 * w1;
      const float a0 = w0 / lsum, a1 = w1 / lsum;
      const int64_t prow = (int64_t)my_slot0;
      float* dst = p.o_part + prow * D + h2 * 4;
      T* o = direct ? row_out(my_slot0) + h2 * 4 : nullptr;
#pragma unroll
      for (int db = 0; db < DB2; ++db)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const f32x4 x = *(const f32x4*)(xbuf + (((rt * DB2 + db) * 4 + b) * 64 + lane) * 4);
          const f32x4 mine = f32x4{acc2[db][4 * b], acc2[db][4 * b + 1], acc2[db][4 * b + 2], acc2[db][4 * b + 3]};
          put4(dst + db * 32 + b * 8, o + db * 32 + b * 8, mine * a0 + x * a1);
        }
      if (h2 == 0) put_lse(prow, (mm + __builtin_amdgcn_logf(lsum)) * 0.6931471805599453f);
    }
    }   // TALLK
  } else {
    // ====================== short box: KV steps split over the 4 waves ========================
    // Each wave keeps DEPTH of its steps in flight in a ring of register buffers: when a step has
    // been consumed its buffer is refilled with the step DEPTH rounds ahead. The chunk is short
    // (a few steps per wave), so most of a workgroup's bytes are requested before the first
    // arrives: the kernel's run time is then set by bandwidth, not by a chain of round trips.
    load_q();
    // K rows go straight into MFMA operand layout (16 rows x 64 bytes per load instruction); V rows
    // are fetched TPL whole rows per instruction and staged in this wave's LDS region. (Staging K
    // the same way and reading operands back from LDS was measured: no faster, twice the LDS.)
    PAT_LDS char* vstage = (PAT_LDS char*)smem + wave * WSTAGE;
    const unsigned koff = (unsigned)(n * kss) + g * 16;                          // K: row n of a half, dims g*8..
    const unsigned voff = (unsigned)((lane / CPR) * vss) + (lane % CPR) * 16;    // V: TPL rows per instruction
    u32x4 kring[DEPTH][2][KK], vring[DEPTH][NV];
    auto fetch_v = [&](int st, u32x4 (&vd)[NV]) {
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        int lim;
        const int h = half_geom(__builtin_amdgcn_readfirstlane(st * 2 + a), lim);
        const char* vb = half_base(vbase, vsp, vss, h);
#pragma unroll
        for (int j = 0; j < NV / 2; ++j) {
          unsigned vo = voff + (unsigned)(j * TPL) * (unsigned)vss;
          if (lim < 15 && j * TPL + lane / CPR > lim) vo = (unsigned)(lim * vss) + (lane % CPR) * 16;
          vd[a * (NV / 2) + j] = *(const u32x4*)(vb + vo);
        }
      }
    };
    auto fetch_k = [&](int st, u32x4 (&kd)[2][KK]) {
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        int lim;
        const int h = half_geom(__builtin_amdgcn_readfirstlane(st * 2 + a), lim);
        const char* kb = half_base(kbase, ksp, kss, h);
        unsigned ko = koff;
        if (lim < 15 && n > lim) ko = (unsigned)(lim * kss) + g * 16;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) kd[a][kk] = *(const u32x4*)(kb + ko + kk * 64);
      }
    };
    // steps of this wave: every kWaves-th one of the chunk, or, with a kv head per wave, all of them
    const int step0 = head_per_wave ? 0 : wave;
    const int stride = head_per_wave ? 1 : kWaves;
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (step0 + d * stride < nsteps) {
        fetch_v(step0 + d * stride, vring[d]);
        fetch_k(step0 + d * stride, kring[d]);
      }
    for (int st0 = step0; st0 < nsteps; st0 += DEPTH * stride) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int st = st0 + d * stride;
        if (st >= nsteps) break;
        const int nxt = st + DEPTH * stride;
        const bool more = nxt < nsteps;
        // V tile -> this wave's LDS region, row-major with padded rows; its registers are free
        // again at once and take the ring's next V tile
#pragma unroll
        for (int j = 0; j < NV; ++j)
          *(PAT_LDS u32x4*)(vstage + (j * TPL + lane / CPR) * RSV + (lane % CPR) * 16) = vring[d][j];
        if (more) fetch_v(nxt, vring[d]);
        // the K registers are refilled as soon as the score MFMAs have read them
        attend([&](int a, int kk) { return __builtin_bit_cast(vec8, kring[d][a][kk]); }, vstage,
               t_begin + st * kStepTokens, [&]() { if (more) fetch_k(nxt, kring[d]); });
      }
    }
    l_run = sum_xor32(sum_xor16(l_run));

    if (head_per_wave) {
      // the wave has seen the whole chunk of its head: its rows go out as they are
      if (my_slot0 >= 0) {
        const int64_t prow = (int64_t)my_slot0;
        const float inv = 1.f / l_run;
        float* dst = p.o_part + prow * D + g * 4;
        T* o = direct ? row_out(my_slot0) + g * 4 : nullptr;
#pragma unroll
        for (int db = 0; db < DB; ++db) put4(dst + db * 16, o + db * 16, acc_o[db] * inv);
        if (g == 0) put_lse(prow, (m_run + __builtin_amdgcn_logf(l_run)) * 0.6931471805599453f);
      }
    } else {
    // combine the 4 waves' states through LDS and write the partial
    float* cbuf = (float*)smem;
    const int crow = tid >> 4;                 // row this thread finalises
    const int ccol = (tid & 15) * (D / 16);    // its first column
    __syncthreads();  // every wave is done with its staging region
    if (g == 0) { s_m[wave * 16 + n] = m_run; s_l[wave * 16 + n] = l_run; }
#pragma unroll
    for (int db = 0; db < DB; ++db)
      *(f32x4*)(cbuf + (wave * 16 + n) * OROW + db * 16 + g * 4) = acc_o[db];
    __syncthreads();

    // the slot of row crow sits in lane crow of every wave
    const int cslot0 = __shfl(my_slot0, crow);
    if (cslot0 >= 0) {
      float mw[kWaves], mmax = neg_inf();
#pragma unroll
      for (int w = 0; w < kWaves; ++w) { mw[w] = s_m[w * 16 + crow]; mmax = fmaxf(mmax, mw[w]); }
      float wsum = 0.f, wgt[kWaves];
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        wgt[w] = fast_exp2(mw[w] - mmax);   // a wave without steps has m = -inf -> weight 0
        wsum += wgt[w] * s_l[w * 16 + crow];
      }
      const float inv = 1.f / wsum;
      const int64_t prow = (int64_t)cslot0;
      float* dst = p.o_part + prow * D + ccol;
      T* od = direct ? row_out(cslot0) + ccol : nullptr;
#pragma unroll
      for (int c = 0; c < D / 16; c += 4) {
        f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kWaves; ++w)
          o += *(const f32x4*)(cbuf + (w * 16 + crow) * OROW + ccol + c) * wgt[w];
        put4(dst + c, od + c, o * inv);
      }
      if ((tid & 15) == 0)
        put_lse(prow, (mmax + __builtin_amdgcn_logf(wsum)) * 0.6931471805599453f);
    }
    }   // combine
  }
}

// Host launcher: picks the instance for (element type, head_dim, single-slot launch, form of the tall path).
typedef void (*SplitFn)(const char*, int, int, const SplitParams);
template <bool DIRECT, int TALLK>
static SplitFn split_instance(bool bf16, int head_dim) {
  if (bf16) return head_dim == 64 ? pat_split_kernel<__bf16, 64, DIRECT, TALLK> : pat_split_kernel<__bf16, 128, DIRECT, TALLK>;
  return head_dim == 64 ? pat_split_kernel<_Float16, 64, DIRECT, TALLK> : pat_split_kernel<_Float16, 128, DIRECT, TALLK>;
}

hipError_t launch_split(bool bf16, int head_dim, hipStream_t stream, const SplitParams& params) {
  const bool t32 = params.tall_rows != 16;
  SplitFn fn = params.direct ? (t32 ? split_instance<true, 32>(bf16, head_dim) : split_instance<true, 16>(bf16, head_dim))
                             : (t32 ? split_instance<false, 32>(bf16, head_dim) : split_instance<false, 16>(bf16, head_dim));
  const unsigned lds = (unsigned)split_smem_bytes(head_dim, t32 ? 32 : 16);
  // more dynamic LDS than the default limit of a kernel: raised once per instance and device
  {
    static std::mutex mutex;
    static bool raised[64][16] = {{false}};
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    const int inst = (t32 ? 8 : 0) + (bf16 ? 4 : 0) + (head_dim == 128 ? 2 : 0) + (params.direct ? 1 : 0);
    std::lock_guard<std::mutex> lock(mutex);
    if (dev >= 0 && dev < 64 && !raised[dev][inst]) {
      if (const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
          e != hipSuccess)
        return e;
      raised[dev][inst] = true;
    }
  }
  const unsigned wgs = (unsigned)params.total_items;
  const dim3 grid(wgs < (unsigned)kGridX ? wgs : (unsigned)kGridX, (wgs + kGridX - 1) / kGridX);
  hipLaunchKernelGGL(fn, grid, dim3(kThreads), lds, stream, params.records, params.record_stride, params.record_max_seqs, params);
  return hipGetLastError();
}

}  // namespace pat
