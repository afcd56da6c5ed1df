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
  const long long gq0 = mv.global_q(q0);
  const long long gk0 = mv.global_k(0);
  if (mv.cbs > 0 && mv.skip_tiles) {
    long long lim = ((gq0 + FBM - 1) / mv.cbs + 1) * mv.cbs;   // first key position masked for every row
    long long n = lim - gk0;
    if (n < kend) kend = n > 0 ? (int)n : 0;
  }
  const int ntiles = (kend + FBN - 1) / FBN;

  // per-lane mask constants
  const long long gq = gq0 + wave * 32 + lo;
  const long long klim = mv.cbs > 0 ? (gq / mv.cbs + 1) * mv.cbs : 0x7fffffffffffffffLL;   // keys >= klim are masked
  const long long klim_wave = mv.cbs > 0 ? ((gq0 + wave * 32) / mv.cbs + 1) * mv.cbs : 0x7fffffffffffffffLL;
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
  auto load_tile = [&](int j) {
    const int k0 = j * FBN;
#pragma unroll
    for (int p = 0; p < 4; p++) {
      const int64_t off = (int64_t)(k0 + p * 16 + srow) * a.kv_ss;
      kr[p] = *(const uint4*)(kg + off);
      vr[p] = *(const uint4*)(vg + off);
    }
    if (tid < FBN) {
      const int kj = k0 + tid;
      if (HAS_SEG) {
        int idx = clamp_seg_index(((long long)mv.k_start + kj / mv.kc) * mv.kc, mv.kc, mv.seg_len, kj % mv.kc);
        seg_r = mv.seg[(int64_t)b * mv.seg_sb + idx];
      }
      if (HAS_BIAS) {
        float bv = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + (gk0 + kj) * mv.bias_sk];
        if (mv.any_mask) bv = fminf(bv, 0.f);
        bias_r = bv * kLog2e;
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int p = 0; p < 4; p++) {
      *(uint4*)(&Ks[buf][(p * 16 + srow) * KSTR + schunk * 8]) = kr[p];
      *(uint4*)(&Vs[buf][(p * 16 + srow) * VSTR + schunk * 8]) = vr[p];
    }
    if (tid < FBN) {
      if (HAS_SEG) seg_ks[buf][tid] = seg_r;
      if (HAS_BIAS) bias_ks[buf][tid] = bias_r;
    }
  };

  if (ntiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();

  // V^T fragment addressing for ds_read_b64_tr_b16: within each 16-lane group, lane i supplies the
  // address of 4 consecutive d of key row (i / 4); lane j of the group receives, for d column j,
  // the 4 key rows.  Group g covers d columns 16 * (g & 1) .. +16 and key rows 4 * hi .. +4.
  const int v_lane_off = ((lane & 15) >> 2) * VSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3) + 4 * hi * VSTR;
  const int k_lane_off = lo * KSTR + hi * 8;

  for (int j = 0; j < ntiles; j++) {
    const int cur = j & 1;
    const bool more = j + 1 < ntiles;
    if (more) load_tile(j + 1);

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
    const long long gk_tile = gk0 + (long long)j * FBN;
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
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[db][r] *= alpha;

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

    if (more) store_tile(cur ^ 1);
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

// ------------------------------------------------------------------ host side
bool attn_fwd_mfma_supported(const ra_attn_fwd_params* p) {
  const ra_mask& m = p->mask;
  return p->dtype == RA_BF16 && p->D == HD && m.query_chunk_size % FBM == 0 && m.key_chunk_size % FBN == 0 &&
         (m.bias == nullptr || m.bias_stride_q == 0) && p->q_stride_s % 8 == 0 && p->kv_stride_s % 8 == 0 &&
         p->q_stride_b % 8 == 0 && p->kv_stride_b % 8 == 0 && p->num_stride_s % 4 == 0 && p->num_stride_b % 4 == 0 &&
         ((uintptr_t)p->q % 16 == 0) && ((uintptr_t)p->k % 16 == 0) && ((uintptr_t)p->v % 16 == 0) &&
         ((uintptr_t)p->numerator % 16 == 0);
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

bool attn_bwd_mfma_supported(const ra_attn_bwd_params*) { return false; }
int attn_bwd_mfma(const ra_attn_bwd_params*, hipStream_t) {
  set_error("mfma bwd: not built");
  return RA_ERR_UNSUPPORTED;
}

}  // namespace ra
