// bf16 MFMA blockwise attention for gfx950, head size 128.
//
// Forward (one ring step, carry in / carry out; ringattention_jax.py:130-145):
//   workgroup = 4 wavefronts = 128 query rows of one (batch, head); each wavefront owns 32 rows.
//   K/V tiles of 64 keys are staged global -> registers -> LDS, double buffered.
//   The logits are computed TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16, so that
//   (a) a lane owns one query column: the running max / sum need one cross-lane step, and
//   (b) the fp32 accumulator layout of S^T is, after rounding to bf16, exactly the B-operand
//       layout of the second product O^T = V^T P^T - P never goes through LDS.
//   V^T fragments come from the row-major V tile with ds_read_b64_tr_b16 (LDS transpose read).
//   Softmax runs in the log2 domain: p = exp2(s * log2(e)/sqrt(D) - m2).
#include "common.hpp"

namespace ra {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int HD = 128;          // head size
constexpr int FBM = 128;         // query rows per workgroup
constexpr int FBN = 64;          // keys per tile
constexpr int KSTR = HD + 8;     // LDS row stride of the K tile, elements: conflict-free 16-byte row reads
constexpr int VSTR = HD + 32;    // LDS row stride of the V tile: conflict-free 4-row transpose reads
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct FwdArgs {
  const uint16_t* q; const uint16_t* k; const uint16_t* v;
  int B, Sq, Skv, H;
  int64_t q_sb, q_ss, kv_sb, kv_ss;
  float* num; int64_t num_sb, num_ss;
  float* den; float* mx;
  int64_t st_sb, st_sh;
  MaskView mv;
  const int32_t* cache_idx;
  int carry_is_initial;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32); }

__device__ __forceinline__ s16x4 lds_read_tr(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p));
}

// natural <-> log2-domain running max; the "every key so far was masked" value mask_min is kept as is
__device__ __forceinline__ float max_to_log2(float m, float mask_min) { return m == mask_min ? m : m * kLog2e; }
__device__ __forceinline__ float max_from_log2(float m2, float mask_min) { return m2 == mask_min ? m2 : m2 * kLn2; }

template <bool HAS_SEG, bool HAS_BIAS>
__global__ __launch_bounds__(256, 2) void attn_fwd_mfma_kernel(FwdArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][FBN * KSTR];
  __shared__ __attribute__((aligned(16))) uint16_t Vs[2][FBN * VSTR];
  __shared__ int seg_ks[2][FBN];
  __shared__ float bias_ks[2][FBN];

  MaskView mv = a.mv;
  if (a.cache_idx) mv.q_start = (*a.cache_idx) / mv.qc;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int nqt = a.Sq / FBM;
  int wg = blockIdx.x;
  const int qt = nqt - 1 - (wg % nqt);       // heaviest (latest) query tiles first
  wg /= nqt;
  const int h = wg % a.H, b = wg / a.H;
  const int q0 = qt * FBM;
  const int qrow = q0 + wave * 32 + lo;      // this lane's query row (local)

  // ---- tile range: chunks that run (reference predicate), clipped to tiles with an unmasked pair
  const int qi = q0 / mv.qc;
  int kend = mv.run_prefix_keys(qi, a.Skv);
  // global positions fit 31 bits (checked on the host)
  const int gq0 = (int)mv.global_q(q0);
  const int gk0 = (int)mv.global_k(0);
  if (mv.cbs > 0 && mv.skip_tiles) {
    long long lim = ((long long)(gq0 + FBM - 1) / mv.cbs + 1) * mv.cbs;   // first key position masked for every row
    long long n = lim - gk0;
    if (n < kend) kend = n > 0 ? (int)n : 0;
  }
  const int ntiles = (kend + FBN - 1) / FBN;

  // per-lane mask constants: keys at global position >= klim are masked
  const int gq = gq0 + wave * 32 + lo;
  const int klim = mv.cbs > 0 ? (int)min((long long)(gq / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;
  const int klim_wave = mv.cbs > 0 ? (int)min((long long)((gq0 + wave * 32) / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;
  int seg_q = 0;
  if (HAS_SEG) {
    int idx = clamp_seg_index(((long long)mv.q_start + qi) * mv.qc, mv.qc, mv.seg_len, qrow % mv.qc);
    seg_q = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  const float c = kLog2e / sqrtf((float)HD);
  const float kMask2 = mv.mask_min;

  // ---- Q fragments (B operand of S^T = K Q^T): column = query row, 8 consecutive d per MFMA step
  const uint16_t* qp = a.q + (int64_t)b * a.q_sb + (int64_t)qrow * a.q_ss + (int64_t)h * HD + hi * 8;
  bf16x8 qf[8];
#pragma unroll
  for (int t = 0; t < 8; t++) qf[t] = *(const bf16x8*)(qp + t * 16);

  // ---- carry
  f32x16 acc[4];
  float m2 = RA_NEG_INF, l = 0.f;
  float* nump = a.num + (int64_t)b * a.num_sb + (int64_t)qrow * a.num_ss + (int64_t)h * HD + hi * 4;
  const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + qrow;
  if (a.carry_is_initial) {
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
  } else {
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        f32x4 t = *(const f32x4*)(nump + db * 32 + g * 8);
        acc[db][g * 4 + 0] = t[0]; acc[db][g * 4 + 1] = t[1]; acc[db][g * 4 + 2] = t[2]; acc[db][g * 4 + 3] = t[3];
      }
    m2 = max_to_log2(a.mx[st], kMask2);
    l = hi == 0 ? a.den[st] : 0.f;     // the two half-wave partial sums are added at the end
  }

  // ---- staging: thread -> (row, 16-byte chunk) of the 64 x 128 tile, 4 passes of 16 rows
  const int srow = tid >> 4, schunk = tid & 15;
  const uint16_t* kg = a.k + (int64_t)b * a.kv_sb + (int64_t)h * HD + schunk * 8;
  const uint16_t* vg = a.v + (int64_t)b * a.kv_sb + (int64_t)h * HD + schunk * 8;
  uint4 kr[4], vr[4];
  int seg_r = 0;
  float bias_r = 0.f;
  // Straight-line staging (no lambdas, no conditionals) so the prefetch registers stay registers.
#define RA_LOAD_KV_TILE(J)                                                                              \
  {                                                                                                     \
    const int k0_ = (J) * FBN;                                                                          \
    _Pragma("unroll") for (int p = 0; p < 4; p++) {                                                     \
      const int64_t off_ = (int64_t)(k0_ + p * 16 + srow) * a.kv_ss;                                    \
      kr[p] = *(const uint4*)(kg + off_);                                                               \
      vr[p] = *(const uint4*)(vg + off_);                                                               \
    }                                                                                                   \
    if ((HAS_SEG || HAS_BIAS) && tid < FBN) {                                                           \
      const int kj_ = k0_ + tid;                                                                        \
      if (HAS_SEG) {                                                                                    \
        int idx_ = clamp_seg_index(((long long)mv.k_start + kj_ / mv.kc) * mv.kc, mv.kc, mv.seg_len, kj_ % mv.kc); \
        seg_r = mv.seg[(int64_t)b * mv.seg_sb + idx_];                                                  \
      }                                                                                                 \
      if (HAS_BIAS) {                                                                                   \
        float bv_ = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + (int64_t)(gk0 + kj_) * mv.bias_sk]; \
        if (mv.any_mask) bv_ = fminf(bv_, 0.f);                                                         \
        bias_r = bv_ * kLog2e;                                                                          \
      }                                                                                                 \
    }                                                                                                   \
  }
#define RA_STORE_KV_TILE(BUF, KSTRIDE, VSTRIDE)                                                         \
  {                                                                                                     \
    _Pragma("unroll") for (int p = 0; p < 4; p++) {                                                     \
      *(uint4*)(&Ks[BUF][(p * 16 + srow) * (KSTRIDE) + schunk * 8]) = kr[p];                            \
      *(uint4*)(&Vs[BUF][(p * 16 + srow) * (VSTRIDE) + schunk * 8]) = vr[p];                            \
    }                                                                                                   \
    if ((HAS_SEG || HAS_BIAS) && tid < FBN) {                                                           \
      if (HAS_SEG) seg_ks[BUF][tid] = seg_r;                                                            \
      if (HAS_BIAS) bias_ks[BUF][tid] = bias_r;                                                         \
    }                                                                                                   \
  }

  if (ntiles > 0) {
    RA_LOAD_KV_TILE(0);
    RA_STORE_KV_TILE(0, KSTR, VSTR);
  }
  __syncthreads();

  // V^T fragment addressing for ds_read_b64_tr_b16: within each 16-lane group, lane i supplies the
  // address of 4 consecutive d of key row (i / 4); lane j of the group receives, for d column j,
  // the 4 key rows.  Group g covers d columns 16 * (g & 1) .. +16 and key rows 4 * hi .. +4.
  const int v_lane_off = ((lane & 15) >> 2) * VSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3) + 4 * hi * VSTR;
  const int k_lane_off = lo * KSTR + hi * 8;

  for (int j = 0; j < ntiles; j++) {
    const int cur = j & 1;
    // prefetch the next tile (the last iteration re-reads its own tile into the idle buffer)
    RA_LOAD_KV_TILE(min(j + 1, ntiles - 1));

    // ---- S^T = K Q^T : two 32(key) x 32(query) blocks
    f32x16 s[2];
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
#pragma unroll
      for (int r = 0; r < 16; r++) s[blk][r] = 0.f;
      const uint16_t* kp = &Ks[cur][blk * 32 * KSTR + k_lane_off];
#pragma unroll
      for (int t = 0; t < 8; t++) {
        bf16x8 kf = *(const bf16x8*)(kp + t * 16);
        s[blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[t], s[blk], 0, 0, 0);
      }
    }

    // ---- online softmax in the log2 domain
    const int gk_tile = gk0 + j * FBN;
    bool need_mask = HAS_SEG || HAS_BIAS || (gk_tile + FBN - 1 >= klim_wave);
    float alpha;
    bf16x8 pf[2][2];
    if (!need_mask) {
      float mxv = s[0][0];
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) mxv = fmaxf(mxv, s[blk][r]);
      mxv = fmaxf(mxv, xor32(mxv));
      const float m_new = fmaxf(m2, mxv * c);
      alpha = fast_exp2(m2 - m_new);
      m2 = m_new;
      float ps = 0.f;
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float p = fast_exp2(fmaf(s[blk][r], c, -m_new));
          ps += p;
          pf[blk][r >> 3][r & 7] = (__bf16)p;
        }
      l = l * alpha + ps;
    } else {
      float mxv = RA_NEG_INF;
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int kr_ = blk * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);     // key row inside the tile
          float x = s[blk][r] * c;
          if (HAS_BIAS) x += bias_ks[cur][kr_];
          bool masked = (gk_tile + kr_ >= klim);
          if (HAS_SEG) masked = masked || (seg_ks[cur][kr_] != seg_q);
          x = masked ? kMask2 : x;
          s[blk][r] = x;
          mxv = fmaxf(mxv, x);
        }
      mxv = fmaxf(mxv, xor32(mxv));
      const float m_new = fmaxf(m2, mxv);
      alpha = fast_exp2(m2 - m_new);
      m2 = m_new;
      float ps = 0.f;
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float p = fast_exp2(s[blk][r] - m_new);
          ps += p;
          pf[blk][r >> 3][r & 7] = (__bf16)p;
        }
      l = l * alpha + ps;
    }
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {     // no row of this wavefront raised its max: skip
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[db][r] *= alpha;
    }

    // ---- O^T += V^T P^T : four 32(d) x 32(query) blocks, contraction over the 64 keys
    const uint16_t* vp = &Vs[cur][v_lane_off];
#pragma unroll
    for (int blk = 0; blk < 2; blk++)
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const uint16_t* vrow = vp + (blk * 32 + t * 16) * VSTR;
#pragma unroll
        for (int db = 0; db < 4; db++) {
          s16x4 v0 = lds_read_tr(vrow + db * 32);
          s16x4 v1 = lds_read_tr(vrow + 8 * VSTR + db * 32);
          s16x8 vv = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vv), pf[blk][t], acc[db], 0, 0, 0);
        }
      }

    RA_STORE_KV_TILE(cur ^ 1, KSTR, VSTR);
    __syncthreads();
  }

  // ---- write the carry back: numerator (fp32), denominator, max_score (natural log domain)
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      f32x4 t = {acc[db][g * 4 + 0], acc[db][g * 4 + 1], acc[db][g * 4 + 2], acc[db][g * 4 + 3]};
      *(f32x4*)(nump + db * 32 + g * 8) = t;
    }
  l += xor32(l);
  if (hi == 0) {
    a.den[st] = l;
    a.mx[st] = max_from_log2(m2, kMask2);
  }
}

// ================================================================== backward
// Two deterministic kernels (fp32 atomics reach ~1.3 TB/s at best on this part, far below what a
// fused dQ accumulation would need):
//   dQ   : query-stationary, same shape as the forward.  S^T = K Q^T and dP^T = V dO^T share the
//          lane <-> query-column layout, so max / 1/denominator / delta are per-lane scalars;
//          dQ^T += K^T dS^T takes K^T from the row-major K tile with LDS transpose reads.
//   dK,dV: key-stationary.  S = Q K^T and dP = dO V^T with K / V fragments resident in registers;
//          P and dS (accumulator layout, lane <-> key column) feed dV^T += dO^T P and
//          dK^T += Q^T dS directly as B operands; Q^T / dO^T come from LDS transpose reads.
// Probabilities are recomputed from the saved max_score / denominator (ringattention_jax.py:226).
constexpr int BSTR = HD + 24;    // LDS row stride for tiles read both row-wise and transposed

struct BwdArgs {
  const uint16_t* q; const uint16_t* k; const uint16_t* v; const uint16_t* g;
  int B, Sq, Skv, H;
  int64_t q_sb, q_ss, kv_sb, kv_ss;
  const float* delta; const float* den; const float* mx;
  int64_t st_sb, st_sh;
  float* dq; int64_t dq_sb, dq_ss;
  float* dk; float* dv; int64_t dkv_sb, dkv_ss;
  MaskView mv;
  const int32_t* cache_idx;
};

template <bool HAS_SEG, bool HAS_BIAS>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_mfma_kernel(BwdArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][FBN * BSTR];
  __shared__ __attribute__((aligned(16))) uint16_t Vs[2][FBN * KSTR];
  __shared__ int seg_ks[2][FBN];
  __shared__ float bias_ks[2][FBN];

  MaskView mv = a.mv;
  if (a.cache_idx) mv.q_start = (*a.cache_idx) / mv.qc;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int nqt = a.Sq / FBM;
  int wg = blockIdx.x;
  const int qt = nqt - 1 - (wg % nqt);
  wg /= nqt;
  const int h = wg % a.H, b = wg / a.H;
  const int q0 = qt * FBM;
  const int qrow = q0 + wave * 32 + lo;

  const int qi = q0 / mv.qc;
  int kend = mv.run_prefix_keys(qi, a.Skv);
  const int gq0 = (int)mv.global_q(q0);
  const int gk0 = (int)mv.global_k(0);
  if (mv.cbs > 0 && mv.skip_tiles) {
    long long lim = ((long long)(gq0 + FBM - 1) / mv.cbs + 1) * mv.cbs;
    long long n = lim - gk0;
    if (n < kend) kend = n > 0 ? (int)n : 0;
  }
  const int ntiles = (kend + FBN - 1) / FBN;
  if (ntiles == 0) return;     // nothing to add to dq

  const int gq = gq0 + wave * 32 + lo;
  const int klim = mv.cbs > 0 ? (int)min((long long)(gq / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;
  const int klim_wave = mv.cbs > 0 ? (int)min((long long)((gq0 + wave * 32) / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;
  int seg_q = 0;
  if (HAS_SEG) {
    int idx = clamp_seg_index(((long long)mv.q_start + qi) * mv.qc, mv.qc, mv.seg_len, qrow % mv.qc);
    seg_q = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  const float c = kLog2e / sqrtf((float)HD);
  const float kMask2 = mv.mask_min;

  const int64_t qoff = (int64_t)b * a.q_sb + (int64_t)qrow * a.q_ss + (int64_t)h * HD + hi * 8;
  bf16x8 qf[8], gf[8];
#pragma unroll
  for (int t = 0; t < 8; t++) {
    qf[t] = *(const bf16x8*)(a.q + qoff + t * 16);
    gf[t] = *(const bf16x8*)(a.g + qoff + t * 16);
  }
  const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + qrow;
  const float m2 = max_to_log2(a.mx[st], kMask2);
  const float rden = 1.f / a.den[st];
  const float delta = a.delta[st];

  f32x16 acc[4];
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[db][r] = 0.f;

  const int srow = tid >> 4, schunk = tid & 15;
  const uint16_t* kg = a.k + (int64_t)b * a.kv_sb + (int64_t)h * HD + schunk * 8;
  const uint16_t* vg = a.v + (int64_t)b * a.kv_sb + (int64_t)h * HD + schunk * 8;
  uint4 kr[4], vr[4];
  int seg_r = 0;
  float bias_r = 0.f;
  RA_LOAD_KV_TILE(0);
  RA_STORE_KV_TILE(0, BSTR, KSTR);
  __syncthreads();

  const int ktr_lane_off = ((lane & 15) >> 2) * BSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3) + 4 * hi * BSTR;
  const int k_lane_off = lo * BSTR + hi * 8;
  const int v_lane_off = lo * KSTR + hi * 8;

  for (int j = 0; j < ntiles; j++) {
    const int cur = j & 1;
    RA_LOAD_KV_TILE(min(j + 1, ntiles - 1));
    const int gk_tile = gk0 + j * FBN;
    const bool need_mask = HAS_SEG || HAS_BIAS || (gk_tile + FBN - 1 >= klim_wave);

#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
      const uint16_t* kp = &Ks[cur][blk * 32 * BSTR + k_lane_off];
      const uint16_t* vp = &Vs[cur][blk * 32 * KSTR + v_lane_off];
#pragma unroll
      for (int t = 0; t < 8; t++) {
        bf16x8 kf = *(const bf16x8*)(kp + t * 16);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[t], s, 0, 0, 0);          // S^T = K Q^T
      }
#pragma unroll
      for (int t = 0; t < 8; t++) {
        bf16x8 vf = *(const bf16x8*)(vp + t * 16);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, gf[t], dp, 0, 0, 0);        // dP^T = V dO^T
      }
      bf16x8 dsf[2];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float p;
        if (!need_mask) {
          p = fast_exp2(fmaf(s[r], c, -m2)) * rden;
        } else {
          const int kr_ = blk * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
          float x = s[r] * c;
          if (HAS_BIAS) x += bias_ks[cur][kr_];
          bool masked = (gk_tile + kr_ >= klim);
          if (HAS_SEG) masked = masked || (seg_ks[cur][kr_] != seg_q);
          x = masked ? kMask2 : x;
          p = fast_exp2(x - m2) * rden;                                              // :226
        }
        dsf[r >> 3][r & 7] = (__bf16)(p * (dp[r] - delta));                          // :229
      }
      // dQ^T += K^T dS^T over these 32 keys
      const uint16_t* ktp = &Ks[cur][blk * 32 * BSTR + ktr_lane_off];
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int db = 0; db < 4; db++) {
          s16x4 k0v = lds_read_tr(ktp + t * 16 * BSTR + db * 32);
          s16x4 k1v = lds_read_tr(ktp + (t * 16 + 8) * BSTR + db * 32);
          s16x8 kk = __builtin_shufflevector(k0v, k1v, 0, 1, 2, 3, 4, 5, 6, 7);
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kk), dsf[t], acc[db], 0, 0, 0);
        }
    }
    RA_STORE_KV_TILE(cur ^ 1, BSTR, KSTR);
    __syncthreads();
  }
#undef RA_LOAD_KV_TILE
#undef RA_STORE_KV_TILE

  // dq += acc / sqrt(D)   (:230)
  const float rscale = 1.f / sqrtf((float)HD);
  float* dqp = a.dq + (int64_t)b * a.dq_sb + (int64_t)qrow * a.dq_ss + (int64_t)h * HD + hi * 4;
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      f32x4 t = *(const f32x4*)(dqp + db * 32 + g * 8);
      t[0] += acc[db][g * 4 + 0] * rscale; t[1] += acc[db][g * 4 + 1] * rscale;
      t[2] += acc[db][g * 4 + 2] * rscale; t[3] += acc[db][g * 4 + 3] * rscale;
      *(f32x4*)(dqp + db * 32 + g * 8) = t;
    }
}

constexpr int KBN = 128;   // keys per workgroup in the dK/dV kernel (32 per wavefront)
constexpr int KBM = 64;    // query rows per step

template <bool HAS_SEG, bool HAS_BIAS>
__global__ __launch_bounds__(256) void attn_bwd_dkv_mfma_kernel(BwdArgs a) {
  __shared__ __attribute__((aligned(16))) uint16_t Qs[2][KBM * BSTR];
  __shared__ __attribute__((aligned(16))) uint16_t Gs[2][KBM * BSTR];
  __shared__ __attribute__((aligned(16))) float st_m2[2][KBM];
  __shared__ __attribute__((aligned(16))) float st_rden[2][KBM];
  __shared__ __attribute__((aligned(16))) float st_delta[2][KBM];
  __shared__ __attribute__((aligned(16))) int st_seg[2][KBM];

  MaskView mv = a.mv;
  if (a.cache_idx) mv.q_start = (*a.cache_idx) / mv.qc;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int nkt = a.Skv / KBN;
  int wg = blockIdx.x;
  const int kt = wg % nkt;                 // earliest key blocks (most query tiles under causal) first
  wg /= nkt;
  const int h = wg % a.H, b = wg / a.H;
  const int k0 = kt * KBN;
  const int krow = k0 + wave * 32 + lo;    // this lane's key row (local)

  const int gk0 = (int)mv.global_k(k0);
  const int gk = gk0 + wave * 32 + lo;
  const int gq_base = (int)mv.global_q(0);
  // first query tile that has work for this key block: run prefix (chunk level), then sub-tile clip
  const int nqt = a.Sq / KBM;
  int qt_first = nqt;
  {
    // the run prefix is non-decreasing in the query chunk index: binary search the first chunk that reaches k0
    int nqc = a.Sq / mv.qc, lo_c = 0, hi_c = nqc;
    while (lo_c < hi_c) {
      int mid = (lo_c + hi_c) >> 1;
      if (mv.run_prefix_keys(mid, a.Skv) > k0) hi_c = mid; else lo_c = mid + 1;
    }
    if (lo_c < nqc) qt_first = lo_c * (mv.qc / KBM);
    if (mv.cbs > 0 && mv.skip_tiles && qt_first < nqt) {
      // query tiles whose every row is masked against every key of the block: (gq_max / cbs) < (gk_min / cbs)
      long long need = (long long)(gk0 / mv.cbs) * mv.cbs - gq_base;     // first local query row that can see key gk0
      if (need > 0) {
        int t = (int)(need / KBM);
        if (t > qt_first) qt_first = t < nqt ? t : nqt;
      }
    }
  }
  if (qt_first >= nqt) return;            // no query sees this key block: dk, dv unchanged

  // masked iff gq / cbs < gk / cbs  <=>  gq < qlim
  const int qlim = mv.cbs > 0 ? (gk / mv.cbs) * mv.cbs : -0x7fffffff;
  const int qlim_wave = mv.cbs > 0 ? ((gk0 + wave * 32 + 31) / mv.cbs) * mv.cbs : -0x7fffffff;
  int seg_k = 0;
  float bias2 = 0.f;
  if (HAS_SEG) {
    int idx = clamp_seg_index(((long long)mv.k_start + krow / mv.kc) * mv.kc, mv.kc, mv.seg_len, krow % mv.kc);
    seg_k = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  if (HAS_BIAS) {
    float bv = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + (int64_t)gk * mv.bias_sk];
    if (mv.any_mask) bv = fminf(bv, 0.f);
    bias2 = bv * kLog2e;
  }
  const float c = kLog2e / sqrtf((float)HD);
  const float kMask2 = mv.mask_min;

  // K and V fragments of this lane's key column (B operands), resident for the whole loop
  const int64_t koff = (int64_t)b * a.kv_sb + (int64_t)krow * a.kv_ss + (int64_t)h * HD + hi * 8;
  bf16x8 kf[8], vf[8];
#pragma unroll
  for (int t = 0; t < 8; t++) {
    kf[t] = *(const bf16x8*)(a.k + koff + t * 16);
    vf[t] = *(const bf16x8*)(a.v + koff + t * 16);
  }
  f32x16 dkacc[4], dvacc[4];
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dkacc[db][r] = 0.f; dvacc[db][r] = 0.f; }

  const int srow = tid >> 4, schunk = tid & 15;
  const uint16_t* qg = a.q + (int64_t)b * a.q_sb + (int64_t)h * HD + schunk * 8;
  const uint16_t* gg = a.g + (int64_t)b * a.q_sb + (int64_t)h * HD + schunk * 8;
  uint4 qr[4], gr[4];
  float r_m2 = 0.f, r_rden = 0.f, r_delta = 0.f;
  int r_seg = 0;
#define RA_LOAD_Q_TILE(QT)                                                                              \
  {                                                                                                     \
    const int q0_ = (QT) * KBM;                                                                         \
    _Pragma("unroll") for (int p = 0; p < 4; p++) {                                                     \
      const int64_t off_ = (int64_t)(q0_ + p * 16 + srow) * a.q_ss;                                     \
      qr[p] = *(const uint4*)(qg + off_);                                                               \
      gr[p] = *(const uint4*)(gg + off_);                                                               \
    }                                                                                                   \
    if (tid < KBM) {                                                                                    \
      const int row_ = q0_ + tid;                                                                       \
      const int64_t st_ = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + row_;                           \
      r_m2 = max_to_log2(a.mx[st_], kMask2);                                                            \
      r_rden = 1.f / a.den[st_];                                                                        \
      r_delta = a.delta[st_];                                                                           \
      if (HAS_SEG) {                                                                                    \
        int idx_ = clamp_seg_index(((long long)mv.q_start + row_ / mv.qc) * mv.qc, mv.qc, mv.seg_len, row_ % mv.qc); \
        r_seg = mv.seg[(int64_t)b * mv.seg_sb + idx_];                                                  \
      }                                                                                                 \
    }                                                                                                   \
  }
#define RA_STORE_Q_TILE(BUF)                                                                            \
  {                                                                                                     \
    _Pragma("unroll") for (int p = 0; p < 4; p++) {                                                     \
      *(uint4*)(&Qs[BUF][(p * 16 + srow) * BSTR + schunk * 8]) = qr[p];                                 \
      *(uint4*)(&Gs[BUF][(p * 16 + srow) * BSTR + schunk * 8]) = gr[p];                                 \
    }                                                                                                   \
    if (tid < KBM) {                                                                                    \
      st_m2[BUF][tid] = r_m2; st_rden[BUF][tid] = r_rden; st_delta[BUF][tid] = r_delta;                 \
      if (HAS_SEG) st_seg[BUF][tid] = r_seg;                                                            \
    }                                                                                                   \
  }
  RA_LOAD_Q_TILE(qt_first);
  RA_STORE_Q_TILE(0);
  __syncthreads();

  const int tr_lane_off = ((lane & 15) >> 2) * BSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3) + 4 * hi * BSTR;
  const int nat_lane_off = lo * BSTR + hi * 8;

  for (int qt = qt_first; qt < nqt; qt++) {
    const int cur = (qt - qt_first) & 1;
    RA_LOAD_Q_TILE(min(qt + 1, nqt - 1));
    const int gq_tile = gq_base + qt * KBM;
    const bool need_mask = HAS_SEG || HAS_BIAS || (gq_tile < qlim_wave);

#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
      const uint16_t* qp = &Qs[cur][qb * 32 * BSTR + nat_lane_off];
      const uint16_t* gp = &Gs[cur][qb * 32 * BSTR + nat_lane_off];
#pragma unroll
      for (int t = 0; t < 8; t++) {
        bf16x8 qa = *(const bf16x8*)(qp + t * 16);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[t], s, 0, 0, 0);          // S = Q K^T
      }
#pragma unroll
      for (int t = 0; t < 8; t++) {
        bf16x8 ga = *(const bf16x8*)(gp + t * 16);
        dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ga, vf[t], dp, 0, 0, 0);        // dP = dO V^T
      }
      bf16x8 pf[2], dsf[2];
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int qrow0 = qb * 32 + g * 8 + hi * 4;          // rows qrow0 .. +3 of the tile
        const f32x4 vm2 = *(const f32x4*)&st_m2[cur][qrow0];
        const f32x4 vrd = *(const f32x4*)&st_rden[cur][qrow0];
        const f32x4 vdl = *(const f32x4*)&st_delta[cur][qrow0];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = g * 4 + e;
          float p;
          if (!need_mask) {
            p = fast_exp2(fmaf(s[r], c, -vm2[e])) * vrd[e];
          } else {
            float x = s[r] * c;
            if (HAS_BIAS) x += bias2;
            bool masked = (gq_tile + qrow0 + e < qlim);
            if (HAS_SEG) masked = masked || (st_seg[cur][qrow0 + e] != seg_k);
            x = masked ? kMask2 : x;
            p = fast_exp2(x - vm2[e]) * vrd[e];
          }
          pf[r >> 3][r & 7] = (__bf16)p;
          dsf[r >> 3][r & 7] = (__bf16)(p * (dp[r] - vdl[e]));
        }
      }
      // dV^T += dO^T P ; dK^T += Q^T dS   (contraction over these 32 query rows)
      const uint16_t* gtp = &Gs[cur][qb * 32 * BSTR + tr_lane_off];
      const uint16_t* qtp = &Qs[cur][qb * 32 * BSTR + tr_lane_off];
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int db = 0; db < 4; db++) {
          s16x4 g0 = lds_read_tr(gtp + t * 16 * BSTR + db * 32);
          s16x4 g1 = lds_read_tr(gtp + (t * 16 + 8) * BSTR + db * 32);
          s16x8 gv = __builtin_shufflevector(g0, g1, 0, 1, 2, 3, 4, 5, 6, 7);
          dvacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, gv), pf[t], dvacc[db], 0, 0, 0);
          s16x4 q0v = lds_read_tr(qtp + t * 16 * BSTR + db * 32);
          s16x4 q1v = lds_read_tr(qtp + (t * 16 + 8) * BSTR + db * 32);
          s16x8 qv = __builtin_shufflevector(q0v, q1v, 0, 1, 2, 3, 4, 5, 6, 7);
          dkacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, qv), dsf[t], dkacc[db], 0, 0, 0);
        }
    }
    RA_STORE_Q_TILE(cur ^ 1);
    __syncthreads();
  }
#undef RA_LOAD_Q_TILE
#undef RA_STORE_Q_TILE

  // dk += acc / sqrt(D) (:231), dv += acc (:232); this workgroup owns its key rows
  const float rscale = 1.f / sqrtf((float)HD);
  const int64_t ooff = (int64_t)b * a.dkv_sb + (int64_t)krow * a.dkv_ss + (int64_t)h * HD + hi * 4;
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int g = 0; g < 4; g++) {
      float* pk = a.dk + ooff + db * 32 + g * 8;
      float* pv = a.dv + ooff + db * 32 + g * 8;
      f32x4 tk = *(const f32x4*)pk, tv = *(const f32x4*)pv;
#pragma unroll
      for (int e = 0; e < 4; e++) { tk[e] += dkacc[db][g * 4 + e] * rscale; tv[e] += dvacc[db][g * 4 + e]; }
      *(f32x4*)pk = tk; *(f32x4*)pv = tv;
    }
}

// ------------------------------------------------------------------ host side
static bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

bool attn_fwd_mfma_supported(const ra_attn_fwd_params* p) {
  const ra_mask& m = p->mask;
  return p->dtype == RA_BF16 && p->D == HD && m.query_chunk_size % FBM == 0 && m.key_chunk_size % FBN == 0 &&
         (m.bias == nullptr || m.bias_stride_q == 0) && p->q_stride_s % 8 == 0 && p->kv_stride_s % 8 == 0 &&
         p->q_stride_b % 8 == 0 && p->kv_stride_b % 8 == 0 && p->num_stride_s % 4 == 0 && p->num_stride_b % 4 == 0 &&
         aligned16(p->q) && aligned16(p->k) && aligned16(p->v) && aligned16(p->numerator);
}

int attn_fwd_mfma(const ra_attn_fwd_params* p, hipStream_t s) {
  FwdArgs a{};
  a.q = (const uint16_t*)p->q; a.k = (const uint16_t*)p->k; a.v = (const uint16_t*)p->v;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.num = p->numerator; a.num_sb = p->num_stride_b; a.num_ss = p->num_stride_s;
  a.den = p->denominator; a.mx = p->max_score; a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  a.cache_idx = p->mask.cache_idx;
  a.carry_is_initial = p->carry_is_initial;
  const long long nwg = (long long)(p->Sq / FBM) * p->H * p->B;
  RA_REQUIRE(nwg < (1LL << 31), RA_ERR_UNSUPPORTED, "attn_fwd_mfma: grid too large");
  dim3 grid((unsigned)nwg), block(256);
  const bool seg = p->mask.segment_ids != nullptr, bias = p->mask.bias != nullptr;
  if (seg && bias) attn_fwd_mfma_kernel<true, true><<<grid, block, 0, s>>>(a);
  else if (seg) attn_fwd_mfma_kernel<true, false><<<grid, block, 0, s>>>(a);
  else if (bias) attn_fwd_mfma_kernel<false, true><<<grid, block, 0, s>>>(a);
  else attn_fwd_mfma_kernel<false, false><<<grid, block, 0, s>>>(a);
  RA_CHECK_LAUNCH("attn_fwd_mfma");
  return RA_OK;
}

bool attn_bwd_mfma_supported(const ra_attn_bwd_params* p) {
  const ra_mask& m = p->mask;
  return p->dtype == RA_BF16 && p->D == HD && m.query_chunk_size % FBM == 0 && m.key_chunk_size % KBN == 0 &&
         (m.bias == nullptr || m.bias_stride_q == 0) && p->q_stride_s % 8 == 0 && p->kv_stride_s % 8 == 0 &&
         p->q_stride_b % 8 == 0 && p->kv_stride_b % 8 == 0 && p->dq_stride_s % 4 == 0 && p->dq_stride_b % 4 == 0 &&
         p->dkv_stride_s % 4 == 0 && p->dkv_stride_b % 4 == 0 && aligned16(p->q) && aligned16(p->k) &&
         aligned16(p->v) && aligned16(p->g) && aligned16(p->dq) && aligned16(p->dk) && aligned16(p->dv);
}

int attn_bwd_mfma(const ra_attn_bwd_params* p, hipStream_t s) {
  BwdArgs a{};
  a.q = (const uint16_t*)p->q; a.k = (const uint16_t*)p->k; a.v = (const uint16_t*)p->v; a.g = (const uint16_t*)p->g;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.delta = p->delta; a.den = p->denominator; a.mx = p->max_score;
  a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.dq = p->dq; a.dq_sb = p->dq_stride_b; a.dq_ss = p->dq_stride_s;
  a.dk = p->dk; a.dv = p->dv; a.dkv_sb = p->dkv_stride_b; a.dkv_ss = p->dkv_stride_s;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  a.cache_idx = p->mask.cache_idx;
  const long long nq = (long long)(p->Sq / FBM) * p->H * p->B, nk = (long long)(p->Skv / KBN) * p->H * p->B;
  RA_REQUIRE(nq < (1LL << 31) && nk < (1LL << 31), RA_ERR_UNSUPPORTED, "attn_bwd_mfma: grid too large");
  dim3 gq((unsigned)nq), gk((unsigned)nk), block(256);
  const bool seg = p->mask.segment_ids != nullptr, bias = p->mask.bias != nullptr;
  const bool do_dkv = !(p->impl & RA_BWD_ONLY_DQ), do_dq = !(p->impl & RA_BWD_ONLY_DKV);
#define RA_LAUNCH_BWD(SEG, BIAS)                                                         \
  do {                                                                                   \
    if (do_dkv) attn_bwd_dkv_mfma_kernel<SEG, BIAS><<<gk, block, 0, s>>>(a);             \
    if (do_dq) attn_bwd_dq_mfma_kernel<SEG, BIAS><<<gq, block, 0, s>>>(a);               \
  } while (0)
  if (seg && bias) RA_LAUNCH_BWD(true, true);
  else if (seg) RA_LAUNCH_BWD(true, false);
  else if (bias) RA_LAUNCH_BWD(false, true);
  else RA_LAUNCH_BWD(false, false);
#undef RA_LAUNCH_BWD
  RA_CHECK_LAUNCH("attn_bwd_mfma");
  return RA_OK;
}

}  // namespace ra
