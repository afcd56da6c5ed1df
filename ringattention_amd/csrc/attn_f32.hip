// fp32 blockwise attention on the matrix cores of gfx950 (v_mfma_f32_32x32x2_f32): the step of
// _blockwise_attention_fwd / _bwd (ringattention_jax.py:99-179, :181-270) for fp32 q, k, v - the dtype of the
// reference's own CPU-runnable configuration - which otherwise takes the one-row-per-lane vector kernels.
//
// Four wavefronts per workgroup, one per SIMD (the kernels use more than 256 registers a lane), each owning 32 of
// the workgroup's 128 query rows (forward, dQ) or keys (dK/dV) and doing all the work for them: logits, softmax
// and the second product.  Nothing is passed between wavefronts but the K / V (or Q / dO) tiles of 64 rows, which
// sit in LDS as plain rows of HD + 4 floats.
//
// A 32x32x2 product contracts two indices per instruction: lanes 0-31 supply the first, lanes 32-63 the second.
// Which two indices those are is free as long as both operands agree, and that freedom removes every data
// exchange between the two products of a block:
//   * S^T = K Q^T: lane (lo, hi) supplies head dimension hi * HD/2 + s in step s, so a lane keeps half of its
//     query row in registers and reads its half of a key row from LDS sixteen bytes at a time;
//   * the result has lane (lo, hi) holding query column lo and keys 8 (r / 4) + 4 hi + r % 4 in register r;
//     O^T += V^T P^T contracts over keys, and step s pairs exactly the two keys that registers s of lanes lo and
//     lo + 32 hold, so P^T feeds the second product from the registers it was computed in;
//   * output blocks interleave the head dimension (block db, row i is dimension NDB i + db), so the A operands of
//     all blocks of a step are one 16-byte LDS read of a V (or K, Q, dO) row.
#include "common.hpp"

namespace ra {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int XBM = 128;        // rows (forward, dQ) or keys (dK/dV) per workgroup
constexpr int XBN = 64;         // rows of a streamed tile

struct F32Args {
  const float* q; const float* k; const float* v; const float* g;
  int B, Sq, Skv, H;
  int64_t q_sb, q_ss, kv_sb, kv_ss;
  float* num; int64_t num_sb, num_ss;
  float* den; float* mx; const float* delta;
  int64_t st_sb, st_sh;
  float* dq; int64_t dq_sb, dq_ss;
  float* dk; float* dv; int64_t dkv_sb, dkv_ss;
  MaskView mv;
  int carry_is_initial;
  int sdim;                                      // head size that scales the logits (the un-padded one)
  float* out; int64_t out_sb, out_ss;           // forward, nullable: out = num / den instead of the numerator
  float* out32;                                  // forward, nullable: the same once more (strides of out)
  int dq_initial, dkv_initial;
  float* dq_out; int64_t dqo_sb, dqo_ss;         // backward, nullable: the sum goes here instead of the accumulator
  float* dk_out; float* dv_out; int64_t dkvo_sb, dkvo_ss;
};

__device__ __forceinline__ float xor32f(float x) { return __shfl_xor(x, 32); }
__device__ __forceinline__ f32x16 mfma2(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
// row (of 32) that register r of a 32 x 32 result holds in a lane of half hi
__device__ __forceinline__ int crow(int r, int hi) { return 8 * (r >> 2) + 4 * hi + (r & 3); }

// XCD-aware workgroup -> (batch, head, tile): XCD x takes the contiguous range x of the triples, so the workgroups
// resident on one XCD stream the same tiles of one head through that XCD's L2
__device__ __forceinline__ bool f32_tile_of_block(int ntile, int B, int H, int& b, int& h, int& t) {
  const int per_xcd = (B * H * ntile + 7) >> 3;
  int wg = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (wg >= B * H * ntile) return false;
  t = wg % ntile;
  wg /= ntile;
  h = wg % H; b = wg / H;
  return true;
}

// 128 rows of HD floats that the workgroup owns but has nothing to add to: hand the accumulator on (divided by den
// when that is given), or set it to the zeros it holds by definition
template <int HD>
__device__ __forceinline__ void f32_pass_rows(const float* acc, float* acc_w, int64_t acc_ss, float* out, float* out2,
                                              int64_t out_ss, const float* den, int initial, int tid) {
  if (!out && !initial) return;
  for (int i = tid; i < XBM * (HD / 4); i += 256) {
    const int r = i / (HD / 4), c4 = (i % (HD / 4)) * 4;
    f32x4 t = {0.f, 0.f, 0.f, 0.f};
    float d = 0.f;
    if (!initial) {
      t = *(const f32x4*)(acc + (int64_t)r * acc_ss + c4);
      if (den) d = den[r];
    }
    if (den) {
#pragma unroll
      for (int e = 0; e < 4; e++) t[e] /= d;                     // 0 / 0 = NaN when nothing ran at all, as :52
    }
    if (out) {
      *(f32x4*)(out + (int64_t)r * out_ss + c4) = t;
      if (out2) *(f32x4*)(out2 + (int64_t)r * out_ss + c4) = t;
    } else {
      *(f32x4*)(acc_w + (int64_t)r * acc_ss + c4) = t;
    }
  }
}

// ---- staging of a 64-row tile (two arrays, e.g. K and V) through registers: PER 16-byte chunks per thread and array
#define RA_F32_STAGE_DECL                                                                               \
  constexpr int STR = HD + 4, HH = HD / 2, NDB = HD / 32, CPR = HD / 4, PER = XBN * CPR / 256;          \
  f32x4 sa[PER], sb[PER];                                                                               \
  const int s_row = tid / CPR, s_c4 = (tid % CPR) * 4;         /* chunk j of this thread: row s_row + j * (256 / CPR) */
#define RA_F32_LOAD(PA, PB, ROW0, STRIDE)                                                               \
  _Pragma("unroll") for (int j = 0; j < PER; j++) {                                                     \
    const int64_t o_ = (int64_t)((ROW0) + s_row + j * (256 / CPR)) * (STRIDE) + s_c4;                   \
    sa[j] = *(const f32x4*)((PA) + o_);                                                                 \
    sb[j] = *(const f32x4*)((PB) + o_);                                                                 \
  }
#define RA_F32_STORE(LA, LB)                                                                            \
  _Pragma("unroll") for (int j = 0; j < PER; j++) {                                                     \
    const int o_ = (s_row + j * (256 / CPR)) * STR + s_c4;                                              \
    *(f32x4*)((LA) + o_) = sa[j];                                                                       \
    *(f32x4*)((LB) + o_) = sb[j];                                                                       \
  }

// key range [k_base, k_base + 64 ntiles) of the shard that a 128-row query tile has to visit (forward, dQ)
template <bool HAS_SEG, int HAS_KEEP>
__device__ __forceinline__ void f32_key_range(const MaskView& mv, int b, int h, int q0, int Skv, int tid, int* hull2,
                                              int& k_base, int& ntiles) {
  const int qi = q0 / mv.qc;
  int kend = mv.run_prefix_keys(qi, Skv);
  const int gq0 = (int)mv.global_q(q0);
  const int gk0_shard = (int)mv.global_k(0);
  if (mv.cbs > 0 && mv.skip_tiles) {
    long long lim = ((long long)(gq0 + XBM - 1) / mv.cbs + 1) * mv.cbs;
    long long n = lim - gk0_shard;
    if (n < kend) kend = n > 0 ? (int)n : 0;
  }
  ntiles = (kend + XBN - 1) / XBN;
  k_base = 0;
  if (HAS_SEG && mv.seg_mm && mv.skip_tiles && ntiles > 0) {
    int t_first, t_last;
    seg_hull_of_rows(mv, b, gq0, XBM, gk0_shard / RA_SEG_TILE, ntiles, hull2, tid, 256, t_first, t_last);
    k_base = t_first * XBN;
    ntiles = t_last - t_first;
  }
  if (HAS_KEEP && mv.skip_tiles && ntiles > 0) {     // key tiles that hold an attended pair for any of the 128 rows
    int t_first, t_last;
    keep_ktile_hull(mv, b, h, (mv.keep_q0 + q0) / 64, XBM / 64, (gk0_shard + k_base - mv.keep_k0) / 64, ntiles, hull2, tid, 256,
                    t_first, t_last);
    k_base += t_first * XBN;
    ntiles = t_last - t_first;
  }
}

// segment id and (clamped) bias of local key kj, as the reference slices them (:279-295)
template <bool HAS_SEG, bool HAS_BIAS>
__device__ __forceinline__ void f32_key_info(const MaskView& mv, int b, int h, int kj, int& seg, float& bias) {
  if (HAS_SEG) {
    const int ki = kj / mv.kc;
    const int idx = clamp_seg_index(((long long)mv.k_start + ki) * mv.kc, mv.kc, mv.seg_len, kj % mv.kc);
    seg = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  if (HAS_BIAS) {
    float bv = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + mv.global_k(kj) * mv.bias_sk];
    bias = mv.any_mask ? fminf(bv, 0.f) : bv;                    // minimum(), :299, :309
  }
}

// Logit of one pair from its scaled dot product (:134-136, :272-322).  masked: the causal or segment mask hits the
// pair; kept: its bit of the boolean mask (only read when KEEP is set); bias: the key's clamped bias.
template <int KEEP>
__device__ __forceinline__ float f32_logit(float dot_scaled, bool masked, bool kept, float bias, float mask_min) {
  if (KEEP == 2) {
    if (kept) return dot_scaled + (masked ? mask_min : bias);
    // dropped: chunk_bias += mask_min (:321) before the logit is added.  Added to a bias of ordinary size it absorbs
    // it (mask_min), added to mask_min - a masked pair, or a bias at that level: a padding mask - it overflows (-inf)
    return dot_scaled + ((masked ? mask_min : bias) + mask_min);
  }
  if (KEEP == 1) masked = masked || !kept;
  return dot_scaled + (masked ? mask_min : bias);
}

// ------------------------------------------------------------------ forward
// HAS_KEEP (packed boolean mask): 0 none, 1 where(keep, logit, mask_min) (ringattention_inference.py:22), 2 dropout:
// mask_min is ADDED for a dropped pair (ringattention_jax.py:321), so a pair that is masked as well becomes -inf
template <int HD, bool HAS_SEG, bool HAS_BIAS, int HAS_KEEP = 0>
__global__ __launch_bounds__(256) void attn_fwd_f32_kernel(F32Args a) {
  __shared__ __attribute__((aligned(16))) float Ks[XBN * (HD + 4)];
  __shared__ __attribute__((aligned(16))) float Vs[XBN * (HD + 4)];
  __shared__ int seg_ks[XBN];
  __shared__ float bias_ks[XBN];
  __shared__ int hull2[2];
  MaskView mv = a.mv;
  mv.resolve();
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  RA_F32_STAGE_DECL
  const int nqt = a.Sq / XBM;
  int b, h, qt;
  if (!f32_tile_of_block(nqt, a.B, a.H, b, h, qt)) return;
  qt = nqt - 1 - qt;                       // latest query tiles (most keys under a causal mask) first
  const int q0 = qt * XBM, qrow = q0 + wave * 32 + lo;
  int k_base, ntiles;
  f32_key_range<HAS_SEG, HAS_KEEP>(mv, b, h, q0, a.Skv, tid, hull2, k_base, ntiles);
  const int64_t st0 = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + q0;
  if (ntiles == 0) {                       // no key tile runs for these rows: the carry stays as it is
    if (a.carry_is_initial || a.out) {
      float* const np0 = a.num ? a.num + (int64_t)b * a.num_sb + (int64_t)q0 * a.num_ss + (int64_t)h * HD : nullptr;
      const int64_t oo = (int64_t)b * a.out_sb + (int64_t)q0 * a.out_ss + (int64_t)h * HD;
      f32_pass_rows<HD>(np0, np0, a.num_ss, a.out ? a.out + oo : nullptr, (a.out && a.out32) ? a.out32 + oo : nullptr,
                        a.out_ss, a.out ? a.den + st0 : nullptr, a.carry_is_initial, tid);
      if (a.carry_is_initial && tid < XBM) { a.den[st0 + tid] = 0.f; a.mx[st0 + tid] = RA_NEG_INF; }
    }
    return;
  }
  const float rscale = 1.f / sqrtf((float)a.sdim);                   // :118
  const int gk0 = (int)mv.global_k(k_base);
  const float* kg = a.k + (int64_t)b * a.kv_sb + (int64_t)h * HD + (int64_t)k_base * a.kv_ss;
  const float* vg = a.v + (int64_t)b * a.kv_sb + (int64_t)h * HD + (int64_t)k_base * a.kv_ss;
  int s_seg = 0; float s_bias = 0.f;

  // this lane's half of its query row
  float qreg[HH];
  {
    const float* qp = a.q + (int64_t)b * a.q_sb + (int64_t)qrow * a.q_ss + (int64_t)h * HD + hi * HH;
#pragma unroll
    for (int j = 0; j < HH / 4; j++) {
      const f32x4 t = *(const f32x4*)(qp + 4 * j);
#pragma unroll
      for (int e = 0; e < 4; e++) qreg[4 * j + e] = t[e];
    }
  }
  const int gq = (int)mv.global_q(qrow);
  const int klim = mv.cbs > 0 ? (int)min(((long long)gq / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;   // masked iff gk >= klim
  int seg_q = 0;
  if (HAS_SEG) {
    const int idx = clamp_seg_index(((long long)mv.q_start + q0 / mv.qc) * mv.qc, mv.qc, mv.seg_len, qrow % mv.qc);
    seg_q = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  // packed boolean mask: one 64-bit word per query row and key tile (bit i = key i of the tile is attended)
  const uint64_t* kw_ptr = nullptr;
  uint64_t kw = 0, kw_nxt = 0;
  if (HAS_KEEP) {
    kw_ptr = mv.kbits_k + (int64_t)b * mv.kpack_sb + (int64_t)h * mv.kpack_sh +
             (int64_t)((gk0 - mv.keep_k0) / 64) * mv.keep_Q + mv.keep_q0 + qrow;
    kw_nxt = kw_ptr[0];
  }
  (void)kw;
  // O^T accumulators: block db, row i is head dimension NDB i + db; this lane's query is the column
  f32x16 acc[NDB];
  float* nump = a.num ? a.num + (int64_t)b * a.num_sb + (int64_t)qrow * a.num_ss + (int64_t)h * HD : nullptr;
  float m = RA_NEG_INF, l = 0.f;
  if (a.carry_is_initial) {
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float* p_ = nump + NDB * crow(r, hi);
#pragma unroll
      for (int db = 0; db < NDB; db++) acc[db][r] = p_[db];
    }
    m = a.mx[st0 + wave * 32 + lo];
    l = hi == 0 ? a.den[st0 + wave * 32 + lo] : 0.f;
  }

  RA_F32_LOAD(kg, vg, 0, a.kv_ss)
  if (tid < XBN) f32_key_info<HAS_SEG, HAS_BIAS>(mv, b, h, k_base + tid, s_seg, s_bias);
  RA_F32_STORE(Ks, Vs)
  if (tid < XBN) { seg_ks[tid] = s_seg; bias_ks[tid] = s_bias; }
  __syncthreads();
  for (int t = 0; t < ntiles; t++) {
    if (HAS_KEEP) { kw = kw_nxt; kw_nxt = kw_ptr[(int64_t)min(t + 1, ntiles - 1) * mv.keep_Q]; }
    if (t + 1 < ntiles) {                  // the next tile travels while this one is worked on
      RA_F32_LOAD(kg, vg, (t + 1) * XBN, a.kv_ss)
      if (tid < XBN) f32_key_info<HAS_SEG, HAS_BIAS>(mv, b, h, k_base + (t + 1) * XBN + tid, s_seg, s_bias);
    }
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      // S^T = K Q^T (:134), two partial sums so that consecutive products do not wait for each other
      f32x16 s0, s1;
#pragma unroll
      for (int r = 0; r < 16; r++) { s0[r] = 0.f; s1[r] = 0.f; }
      const float* kp = Ks + (blk * 32 + lo) * STR + hi * HH;
#pragma unroll
      for (int j = 0; j < HH / 4; j++) {
        const f32x4 kf = *(const f32x4*)(kp + 4 * j);
        s0 = mfma2(kf[0], qreg[4 * j + 0], s0);
        s1 = mfma2(kf[1], qreg[4 * j + 1], s1);
        s0 = mfma2(kf[2], qreg[4 * j + 2], s0);
        s1 = mfma2(kf[3], qreg[4 * j + 3], s1);
      }
      // logits of this lane's query against its 16 keys of the block (:134-136, :272-322)
      const int gkb = gk0 + t * XBN + blk * 32;
      const uint32_t kwb = HAS_KEEP ? (uint32_t)(kw >> (blk * 32)) >> (4 * hi) : 0u;   // this lane's keys of the block
      (void)kwb;
      float x[16], mloc = RA_NEG_INF;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int kr = blk * 32 + crow(r, hi);
        bool masked = gkb + crow(r, hi) >= klim;
        if (HAS_SEG) masked = masked || seg_ks[kr] != seg_q;
        const bool kept = HAS_KEEP ? ((kwb >> (8 * (r >> 2) + (r & 3))) & 1u) != 0 : true;
        x[r] = f32_logit<HAS_KEEP>((s0[r] + s1[r]) * rscale, masked, kept, HAS_BIAS ? bias_ks[kr] : 0.f, mv.mask_min);
        mloc = fmaxf(mloc, x[r]);
      }
      mloc = fmaxf(mloc, xor32f(mloc));
      const float m_new = fmaxf(m, mloc);                          // :138
      const bool dead = m_new == RA_NEG_INF;                       // nothing finite for this row so far
      const float corr = (dead || m == m_new) ? 1.f : __expf(m - m_new);   // :142
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) { x[r] = dead ? 0.f : __expf(x[r] - m_new); psum += x[r]; }   // :140
      l = l * corr + psum;                                         // :144
      m = m_new;
      if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
        for (int db = 0; db < NDB; db++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[db][r] *= corr;         // :143
      }
      // O^T += V^T P^T (:141): step s contracts the two keys that registers s of lanes lo and lo + 32 hold
#pragma unroll
      for (int s = 0; s < 16; s++) {
        const float* vp = Vs + (blk * 32 + crow(s, hi)) * STR + lo * NDB;
        float vf[NDB];
        if (NDB == 4) { const f32x4 t4 = *(const f32x4*)vp; vf[0] = t4[0]; vf[1] = t4[1]; vf[NDB - 2] = t4[2]; vf[NDB - 1] = t4[3]; }
        else { vf[0] = vp[0]; vf[1] = vp[1]; }
#pragma unroll
        for (int db = 0; db < NDB; db++) acc[db] = mfma2(vf[db], x[s], acc[db]);
      }
    }
    __syncthreads();                       // every wavefront is done with the tile in LDS
    if (t + 1 < ntiles) {
      RA_F32_STORE(Ks, Vs)
      if (tid < XBN) { seg_ks[tid] = s_seg; bias_ks[tid] = s_bias; }
    }
    __syncthreads();
  }
  l += xor32f(l);
  if (hi == 0) { a.den[st0 + wave * 32 + lo] = l; a.mx[st0 + wave * 32 + lo] = m; }
  if (a.out) {                             // last step of the device: out = numerator / denominator (:52)
    const int64_t oo = (int64_t)b * a.out_sb + (int64_t)qrow * a.out_ss + (int64_t)h * HD;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      float t_[NDB];
#pragma unroll
      for (int db = 0; db < NDB; db++) t_[db] = acc[db][r] / l;
#pragma unroll
      for (int db = 0; db < NDB; db++) {
        a.out[oo + NDB * crow(r, hi) + db] = t_[db];
        if (a.out32) a.out32[oo + NDB * crow(r, hi) + db] = t_[db];
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++)
#pragma unroll
      for (int db = 0; db < NDB; db++) nump[NDB * crow(r, hi) + db] = acc[db][r];
  }
}

// ------------------------------------------------------------------ backward, dQ (query-stationary)
template <int HD, bool HAS_SEG, bool HAS_BIAS, int HAS_KEEP = 0>
__global__ __launch_bounds__(256) void attn_bwd_dq_f32_kernel(F32Args a) {
  __shared__ __attribute__((aligned(16))) float Ks[XBN * (HD + 4)];
  __shared__ __attribute__((aligned(16))) float Vs[XBN * (HD + 4)];
  __shared__ int seg_ks[XBN];
  __shared__ float bias_ks[XBN];
  __shared__ int hull2[2];
  MaskView mv = a.mv;
  mv.resolve();
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  RA_F32_STAGE_DECL
  const int nqt = a.Sq / XBM;
  int b, h, qt;
  if (!f32_tile_of_block(nqt, a.B, a.H, b, h, qt)) return;
  qt = nqt - 1 - qt;
  const int q0 = qt * XBM, qrow = q0 + wave * 32 + lo;
  int k_base, ntiles;
  f32_key_range<HAS_SEG, HAS_KEEP>(mv, b, h, q0, a.Skv, tid, hull2, k_base, ntiles);
  if (ntiles == 0) {                       // nothing to add to dq
    float* const dq0 = a.dq ? a.dq + (int64_t)b * a.dq_sb + (int64_t)q0 * a.dq_ss + (int64_t)h * HD : nullptr;
    f32_pass_rows<HD>(dq0, dq0, a.dq_ss,
                      a.dq_out ? a.dq_out + (int64_t)b * a.dqo_sb + (int64_t)q0 * a.dqo_ss + (int64_t)h * HD : nullptr,
                      nullptr, a.dqo_ss, nullptr, a.dq_initial, tid);
    return;
  }
  const float rscale = 1.f / sqrtf((float)a.sdim);
  const int gk0 = (int)mv.global_k(k_base);
  const float* kg = a.k + (int64_t)b * a.kv_sb + (int64_t)h * HD + (int64_t)k_base * a.kv_ss;
  const float* vg = a.v + (int64_t)b * a.kv_sb + (int64_t)h * HD + (int64_t)k_base * a.kv_ss;
  int s_seg = 0; float s_bias = 0.f;

  float qreg[HH], greg[HH];
  {
    const int64_t o = (int64_t)b * a.q_sb + (int64_t)qrow * a.q_ss + (int64_t)h * HD + hi * HH;
#pragma unroll
    for (int j = 0; j < HH / 4; j++) {
      const f32x4 t = *(const f32x4*)(a.q + o + 4 * j), u = *(const f32x4*)(a.g + o + 4 * j);
#pragma unroll
      for (int e = 0; e < 4; e++) { qreg[4 * j + e] = t[e]; greg[4 * j + e] = u[e]; }
    }
  }
  const int gq = (int)mv.global_q(qrow);
  const int klim = mv.cbs > 0 ? (int)min(((long long)gq / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;
  int seg_q = 0;
  if (HAS_SEG) {
    const int idx = clamp_seg_index(((long long)mv.q_start + q0 / mv.qc) * mv.qc, mv.qc, mv.seg_len, qrow % mv.qc);
    seg_q = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  // packed boolean mask: one 64-bit word per query row and key tile (bit i = key i of the tile is attended)
  const uint64_t* kw_ptr = nullptr;
  uint64_t kw = 0, kw_nxt = 0;
  if (HAS_KEEP) {
    kw_ptr = mv.kbits_k + (int64_t)b * mv.kpack_sb + (int64_t)h * mv.kpack_sh +
             (int64_t)((gk0 - mv.keep_k0) / 64) * mv.keep_Q + mv.keep_q0 + qrow;
    kw_nxt = kw_ptr[0];
  }
  (void)kw;
  const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + qrow;
  const float m = a.mx[st], rden = 1.f / a.den[st], delta = a.delta[st];
  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[db][r] = 0.f;

  RA_F32_LOAD(kg, vg, 0, a.kv_ss)
  if (tid < XBN) f32_key_info<HAS_SEG, HAS_BIAS>(mv, b, h, k_base + tid, s_seg, s_bias);
  RA_F32_STORE(Ks, Vs)
  if (tid < XBN) { seg_ks[tid] = s_seg; bias_ks[tid] = s_bias; }
  __syncthreads();
  for (int t = 0; t < ntiles; t++) {
    if (HAS_KEEP) { kw = kw_nxt; kw_nxt = kw_ptr[(int64_t)min(t + 1, ntiles - 1) * mv.keep_Q]; }
    if (t + 1 < ntiles) {
      RA_F32_LOAD(kg, vg, (t + 1) * XBN, a.kv_ss)
      if (tid < XBN) f32_key_info<HAS_SEG, HAS_BIAS>(mv, b, h, k_base + (t + 1) * XBN + tid, s_seg, s_bias);
    }
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      // S^T = K Q^T and dP^T = V dO^T (:225, :228): two independent chains
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
      const float* kp = Ks + (blk * 32 + lo) * STR + hi * HH;
      const float* vp = Vs + (blk * 32 + lo) * STR + hi * HH;
#pragma unroll
      for (int j = 0; j < HH / 4; j++) {
        const f32x4 kf = *(const f32x4*)(kp + 4 * j), vf = *(const f32x4*)(vp + 4 * j);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          s = mfma2(kf[e], qreg[4 * j + e], s);
          dp = mfma2(vf[e], greg[4 * j + e], dp);
        }
      }
      const int gkb = gk0 + t * XBN + blk * 32;
      const uint32_t kwb = HAS_KEEP ? (uint32_t)(kw >> (blk * 32)) >> (4 * hi) : 0u;   // this lane's keys of the block
      (void)kwb;
      float ds[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int kr = blk * 32 + crow(r, hi);
        bool masked = gkb + crow(r, hi) >= klim;
        if (HAS_SEG) masked = masked || seg_ks[kr] != seg_q;
        const bool kept = HAS_KEEP ? ((kwb >> (8 * (r >> 2) + (r & 3))) & 1u) != 0 : true;
        const float x_ = f32_logit<HAS_KEEP>(s[r] * rscale, masked, kept, HAS_BIAS ? bias_ks[kr] : 0.f, mv.mask_min);
        const float p = __expf(x_ - m) * rden;                     // :226
        ds[r] = (dp[r] - delta) * p;                               // :229
      }
      // dQ^T += K^T dS^T (:230)
#pragma unroll
      for (int s_ = 0; s_ < 16; s_++) {
        const float* kq = Ks + (blk * 32 + crow(s_, hi)) * STR + lo * NDB;
        float kf[NDB];
        if (NDB == 4) { const f32x4 t4 = *(const f32x4*)kq; kf[0] = t4[0]; kf[1] = t4[1]; kf[NDB - 2] = t4[2]; kf[NDB - 1] = t4[3]; }
        else { kf[0] = kq[0]; kf[1] = kq[1]; }
#pragma unroll
        for (int db = 0; db < NDB; db++) acc[db] = mfma2(kf[db], ds[s_], acc[db]);
      }
    }
    __syncthreads();
    if (t + 1 < ntiles) {
      RA_F32_STORE(Ks, Vs)
      if (tid < XBN) { seg_ks[tid] = s_seg; bias_ks[tid] = s_bias; }
    }
    __syncthreads();
  }
  // dq += acc / sqrt(D) (:230)
  float* dqp = a.dq ? a.dq + (int64_t)b * a.dq_sb + (int64_t)qrow * a.dq_ss + (int64_t)h * HD : nullptr;
  float* dqo = a.dq_out ? a.dq_out + (int64_t)b * a.dqo_sb + (int64_t)qrow * a.dqo_ss + (int64_t)h * HD : nullptr;
  // all the old values are requested before the first store (a load issued after a store is not waited for until
  // that store has completed too: one in-order counter of outstanding memory operations)
  float old[16][NDB];
#pragma unroll
  for (int r = 0; r < 16; r++)
#pragma unroll
    for (int db = 0; db < NDB; db++) old[r][db] = a.dq_initial ? 0.f : dqp[NDB * crow(r, hi) + db];
#pragma unroll
  for (int r = 0; r < 16; r++)
#pragma unroll
    for (int db = 0; db < NDB; db++) {
      const int d = NDB * crow(r, hi) + db;
      const float t_ = old[r][db] + acc[db][r] * rscale;
      if (dqo) dqo[d] = t_;                // last call for these rows (:89)
      else dqp[d] = t_;
    }
}

// ------------------------------------------------------------------ backward, dK and dV (key-stationary)
template <int HD, bool HAS_SEG, bool HAS_BIAS, int HAS_KEEP = 0>
__global__ __launch_bounds__(256) void attn_bwd_dkv_f32_kernel(F32Args a) {
  __shared__ __attribute__((aligned(16))) float Qs[XBN * (HD + 4)];
  __shared__ __attribute__((aligned(16))) float Gs[XBN * (HD + 4)];
  __shared__ __attribute__((aligned(16))) float st_m[XBN];
  __shared__ __attribute__((aligned(16))) float st_rden[XBN];
  __shared__ __attribute__((aligned(16))) float st_delta[XBN];
  __shared__ __attribute__((aligned(16))) int st_seg[XBN];
  __shared__ int hull2[2];
  MaskView mv = a.mv;
  mv.resolve();
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  RA_F32_STAGE_DECL
  const int nkt = a.Skv / XBM;
  int b, h, kt;
  if (!f32_tile_of_block(nkt, a.B, a.H, b, h, kt)) return;
  const int k0 = kt * XBM, krow = k0 + wave * 32 + lo;
  const int gk0 = (int)mv.global_k(k0), gk = gk0 + wave * 32 + lo;
  const int gq_base = (int)mv.global_q(0);
  // query tiles (64 rows) that meet these keys: chunks whose run prefix covers them, from the first row block that
  // is not wholly before the keys' causal block on
  const int nqt = a.Sq / XBN;
  int qt_first = nqt;
  {
    int nqc = a.Sq / mv.qc, lo_c = 0, hi_c = nqc;
    while (lo_c < hi_c) {
      const int mid = (lo_c + hi_c) >> 1;
      if (mv.run_prefix_keys(mid, a.Skv) > k0) hi_c = mid; else lo_c = mid + 1;
    }
    if (lo_c < nqc) qt_first = lo_c * (mv.qc / XBN);
    if (mv.cbs > 0 && mv.skip_tiles && qt_first < nqt) {
      const long long need = (long long)(gk0 / mv.cbs) * mv.cbs - gq_base;
      if (need > 0) {
        const int t = (int)(need / XBN);
        if (t > qt_first) qt_first = t < nqt ? t : nqt;
      }
    }
  }
  int qt_end = nqt;
  if (HAS_SEG && mv.seg_mm && mv.skip_tiles && qt_first < nqt) {
    int t_first, t_last;
    seg_hull_of_rows(mv, b, gk0, XBM, gq_base / RA_SEG_TILE + qt_first, nqt - qt_first, hull2, tid, 256, t_first, t_last);
    qt_end = qt_first + t_last;
    qt_first += t_first;
  }
  if (HAS_KEEP && mv.skip_tiles && qt_first < qt_end) {
    int t_first, t_last;
    keep_qtile_hull(mv, b, h, (gk0 - mv.keep_k0) / 64, XBM / 64, mv.keep_q0 / 64 + qt_first, qt_end - qt_first, hull2, tid, 256,
                    t_first, t_last);
    qt_end = qt_first + t_last;
    qt_first += t_first;
  }
  if (qt_first >= qt_end) {                // nothing to add for these keys
    const int64_t o = (int64_t)b * a.dkv_sb + (int64_t)k0 * a.dkv_ss + (int64_t)h * HD;
    const int64_t oo = (int64_t)b * a.dkvo_sb + (int64_t)k0 * a.dkvo_ss + (int64_t)h * HD;
    f32_pass_rows<HD>(a.dk ? a.dk + o : nullptr, a.dk ? a.dk + o : nullptr, a.dkv_ss, a.dk_out ? a.dk_out + oo : nullptr,
                      nullptr, a.dkvo_ss, nullptr, a.dkv_initial, tid);
    f32_pass_rows<HD>(a.dv ? a.dv + o : nullptr, a.dv ? a.dv + o : nullptr, a.dkv_ss, a.dv_out ? a.dv_out + oo : nullptr,
                      nullptr, a.dkvo_ss, nullptr, a.dkv_initial, tid);
    return;
  }
  const int ntq = qt_end - qt_first;
  const float rscale = 1.f / sqrtf((float)a.sdim);
  const int qlim = mv.cbs > 0 ? (gk / mv.cbs) * mv.cbs : -0x7fffffff;        // masked iff gq < qlim
  int seg_k = 0; float bias_k = 0.f;
  f32_key_info<HAS_SEG, HAS_BIAS>(mv, b, h, krow, seg_k, bias_k);
  float kreg[HH], vreg[HH];
  {
    const int64_t o = (int64_t)b * a.kv_sb + (int64_t)krow * a.kv_ss + (int64_t)h * HD + hi * HH;
#pragma unroll
    for (int j = 0; j < HH / 4; j++) {
      const f32x4 t = *(const f32x4*)(a.k + o + 4 * j), u = *(const f32x4*)(a.v + o + 4 * j);
#pragma unroll
      for (int e = 0; e < 4; e++) { kreg[4 * j + e] = t[e]; vreg[4 * j + e] = u[e]; }
    }
  }
  f32x16 dkacc[NDB], dvacc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dkacc[db][r] = 0.f; dvacc[db][r] = 0.f; }
  // packed boolean mask: one 64-bit word per key and query tile (bit i = row i of the tile attends to this key)
  const uint64_t* kw_ptr = nullptr;
  uint64_t kw = 0, kw_nxt = 0;
  if (HAS_KEEP) {
    kw_ptr = mv.kbits_q + (int64_t)b * mv.kpack_sb + (int64_t)h * mv.kpack_sh +
             (int64_t)(mv.keep_q0 / 64 + qt_first) * mv.keep_K + gk - mv.keep_k0;
    kw_nxt = kw_ptr[0];
  }
  (void)kw;

  const float* qg = a.q + (int64_t)b * a.q_sb + (int64_t)h * HD + (int64_t)(qt_first * XBN) * a.q_ss;
  const float* gg = a.g + (int64_t)b * a.q_sb + (int64_t)h * HD + (int64_t)(qt_first * XBN) * a.q_ss;
  float r_m = 0.f, r_den = 1.f, r_delta = 0.f;
  int r_seg = 0;
#define RA_F32_ROWSTATS(T)                                                                              \
  if (tid < XBN) {                                                                                      \
    const int row_ = (qt_first + (T)) * XBN + tid;                                                      \
    const int64_t st_ = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + row_;                             \
    r_m = a.mx[st_]; r_den = a.den[st_]; r_delta = a.delta[st_];                                        \
    if (HAS_SEG) {                                                                                      \
      const int idx_ = clamp_seg_index(((long long)mv.q_start + row_ / mv.qc) * mv.qc, mv.qc, mv.seg_len, row_ % mv.qc); \
      r_seg = mv.seg[(int64_t)b * mv.seg_sb + idx_];                                                    \
    }                                                                                                   \
  }
#define RA_F32_ROWSTATS_STORE                                                                           \
  if (tid < XBN) { st_m[tid] = r_m; st_rden[tid] = 1.f / r_den; st_delta[tid] = r_delta; st_seg[tid] = r_seg; }
  RA_F32_LOAD(qg, gg, 0, a.q_ss)
  RA_F32_ROWSTATS(0)
  RA_F32_STORE(Qs, Gs)
  RA_F32_ROWSTATS_STORE
  __syncthreads();
  for (int t = 0; t < ntq; t++) {
    if (HAS_KEEP) { kw = kw_nxt; kw_nxt = kw_ptr[(int64_t)min(t + 1, ntq - 1) * mv.keep_K]; }
    if (t + 1 < ntq) {
      RA_F32_LOAD(qg, gg, (t + 1) * XBN, a.q_ss)
      RA_F32_ROWSTATS(t + 1)
    }
    const int gq_tile = gq_base + (qt_first + t) * XBN;
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      // S = Q K^T and dP = dO V^T (:225, :228): rows are the block's queries, this lane's key is the column
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
      const float* qp = Qs + (blk * 32 + lo) * STR + hi * HH;
      const float* gp = Gs + (blk * 32 + lo) * STR + hi * HH;
#pragma unroll
      for (int j = 0; j < HH / 4; j++) {
        const f32x4 qf = *(const f32x4*)(qp + 4 * j), gf = *(const f32x4*)(gp + 4 * j);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          s = mfma2(qf[e], kreg[4 * j + e], s);
          dp = mfma2(gf[e], vreg[4 * j + e], dp);
        }
      }
      float p[16], ds[16];
      const uint32_t kwb = HAS_KEEP ? (uint32_t)(kw >> (blk * 32)) >> (4 * hi) : 0u;     // this lane's rows of the block
      (void)kwb;
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const int row0 = blk * 32 + 8 * g4 + 4 * hi;               // rows of registers 4 g4 .. 4 g4 + 3
        const f32x4 vm = *(const f32x4*)&st_m[row0], vr = *(const f32x4*)&st_rden[row0], vd = *(const f32x4*)&st_delta[row0];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 4 * g4 + e;
          bool masked = gq_tile + row0 + e < qlim;
          if (HAS_SEG) masked = masked || st_seg[row0 + e] != seg_k;
          const bool kept = HAS_KEEP ? ((kwb >> (8 * g4 + e)) & 1u) != 0 : true;
          const float x_ = f32_logit<HAS_KEEP>(s[r] * rscale, masked, kept, HAS_BIAS ? bias_k : 0.f, mv.mask_min);
          p[r] = __expf(x_ - vm[e]) * vr[e];                       // :226
          ds[r] = (dp[r] - vd[e]) * p[r];                          // :229
        }
      }
      // dV^T += dO^T P (:232) and dK^T += Q^T dS (:231): step s_ contracts the two query rows that registers s_ of
      // lanes lo and lo + 32 hold
#pragma unroll
      for (int s_ = 0; s_ < 16; s_++) {
        const float* gq_ = Gs + (blk * 32 + crow(s_, hi)) * STR + lo * NDB;
        const float* qq_ = Qs + (blk * 32 + crow(s_, hi)) * STR + lo * NDB;
        float gf[NDB], qf[NDB];
        if (NDB == 4) {
          const f32x4 t4 = *(const f32x4*)gq_, u4 = *(const f32x4*)qq_;
          gf[0] = t4[0]; gf[1] = t4[1]; gf[NDB - 2] = t4[2]; gf[NDB - 1] = t4[3];
          qf[0] = u4[0]; qf[1] = u4[1]; qf[NDB - 2] = u4[2]; qf[NDB - 1] = u4[3];
        } else { gf[0] = gq_[0]; gf[1] = gq_[1]; qf[0] = qq_[0]; qf[1] = qq_[1]; }
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          dvacc[db] = mfma2(gf[db], p[s_], dvacc[db]);
          dkacc[db] = mfma2(qf[db], ds[s_], dkacc[db]);
        }
      }
    }
    __syncthreads();
    if (t + 1 < ntq) {
      RA_F32_STORE(Qs, Gs)
      RA_F32_ROWSTATS_STORE
    }
    __syncthreads();
  }
#undef RA_F32_ROWSTATS
#undef RA_F32_ROWSTATS_STORE
  // dk += acc / sqrt(D) (:231), dv += acc (:232)
  const int64_t o = (int64_t)b * a.dkv_sb + (int64_t)krow * a.dkv_ss + (int64_t)h * HD;
  const int64_t oo = (int64_t)b * a.dkvo_sb + (int64_t)krow * a.dkvo_ss + (int64_t)h * HD;
  // all the old values are requested before the first store (see the dQ kernel)
  float oldk[16][NDB], oldv[16][NDB];
#pragma unroll
  for (int r = 0; r < 16; r++)
#pragma unroll
    for (int db = 0; db < NDB; db++) {
      const int d = NDB * crow(r, hi) + db;
      oldk[r][db] = a.dkv_initial ? 0.f : a.dk[o + d];
      oldv[r][db] = a.dkv_initial ? 0.f : a.dv[o + d];
    }
#pragma unroll
  for (int r = 0; r < 16; r++)
#pragma unroll
    for (int db = 0; db < NDB; db++) {
      const int d = NDB * crow(r, hi) + db;
      const float tk = oldk[r][db] + dkacc[db][r] * rscale;
      const float tv = oldv[r][db] + dvacc[db][r];
      if (a.dk_out) { a.dk_out[oo + d] = tk; a.dv_out[oo + d] = tv; }      // last call for these keys (:89)
      else { a.dk[o + d] = tk; a.dv[o + d] = tv; }
    }
}
#undef RA_F32_STAGE_DECL
#undef RA_F32_LOAD
#undef RA_F32_STORE

// ------------------------------------------------------------------ host side
static bool al16(const void* p) { return ((uintptr_t)p % 16) == 0; }

// a boolean mask is taken in packed form only; the attn_mask of ring_attention_inference next to a causal block size
// at most (it has no bias or segment ids there), the dropout mask next to everything
static bool f32_mask_ok(const ra_mask& m) {
  if ((m.keep || m.keep_bits_k) &&
      !(m.keep_bits_k && m.keep_bits_q && m.keep_summary &&
        (m.keep_mode == RA_KEEP_DROPOUT || (!m.bias && !m.segment_ids))))
    return false;
  return m.bias == nullptr || m.bias_stride_q == 0;
}

bool attn_fwd_f32_supported(const ra_attn_fwd_params* p) {
  const ra_mask& m = p->mask;
  return p->dtype == RA_F32 && (p->D == 128 || p->D == 64) && p->Sq % XBM == 0 && p->Skv % XBN == 0 &&
         m.query_chunk_size % XBM == 0 && m.key_chunk_size % XBN == 0 && f32_mask_ok(m) &&
         p->q_stride_s % 4 == 0 && p->kv_stride_s % 4 == 0 && p->q_stride_b % 4 == 0 && p->kv_stride_b % 4 == 0 &&
         p->num_stride_s % 4 == 0 && p->num_stride_b % 4 == 0 && al16(p->q) && al16(p->k) && al16(p->v) &&
         al16(p->numerator) && (!p->out || (al16(p->out) && p->out_stride_s % 4 == 0 && p->out_stride_b % 4 == 0)) &&
         al16(p->out_f32);
}

bool attn_bwd_f32_supported(const ra_attn_bwd_params* p) {
  const ra_mask& m = p->mask;
  return p->dtype == RA_F32 && (p->D == 128 || p->D == 64) && p->Sq % XBM == 0 && p->Skv % XBM == 0 &&
         m.query_chunk_size % XBM == 0 && m.key_chunk_size % XBM == 0 && f32_mask_ok(m) &&
         p->q_stride_s % 4 == 0 && p->kv_stride_s % 4 == 0 && p->q_stride_b % 4 == 0 && p->kv_stride_b % 4 == 0 &&
         p->dq_stride_s % 4 == 0 && p->dq_stride_b % 4 == 0 && p->dkv_stride_s % 4 == 0 && p->dkv_stride_b % 4 == 0 &&
         al16(p->q) && al16(p->k) && al16(p->v) && al16(p->g) && al16(p->dq) && al16(p->dk) && al16(p->dv) &&
         (!p->dq_out || (al16(p->dq_out) && p->dq_out_stride_s % 4 == 0 && p->dq_out_stride_b % 4 == 0)) &&
         (!p->dk_out || (al16(p->dk_out) && al16(p->dv_out) && p->dkv_out_stride_s % 4 == 0 &&
                         p->dkv_out_stride_b % 4 == 0));
}

#define RA_F32_DISPATCH(KERNEL, GRID)                                                    \
  do {                                                                                   \
    if (keep && p->mask.keep_mode == RA_KEEP_DROPOUT) {                                  \
      if (p->D == 128) {                                                                 \
        if (seg && bias) KERNEL<128, true, true, 2><<<GRID, 256, 0, s>>>(a);             \
        else if (seg) KERNEL<128, true, false, 2><<<GRID, 256, 0, s>>>(a);               \
        else if (bias) KERNEL<128, false, true, 2><<<GRID, 256, 0, s>>>(a);              \
        else KERNEL<128, false, false, 2><<<GRID, 256, 0, s>>>(a);                       \
      } else {                                                                           \
        if (seg && bias) KERNEL<64, true, true, 2><<<GRID, 256, 0, s>>>(a);              \
        else if (seg) KERNEL<64, true, false, 2><<<GRID, 256, 0, s>>>(a);                \
        else if (bias) KERNEL<64, false, true, 2><<<GRID, 256, 0, s>>>(a);               \
        else KERNEL<64, false, false, 2><<<GRID, 256, 0, s>>>(a);                        \
      }                                                                                  \
    } else if (keep) {                                                                   \
      if (p->D == 128) KERNEL<128, false, false, 1><<<GRID, 256, 0, s>>>(a);             \
      else KERNEL<64, false, false, 1><<<GRID, 256, 0, s>>>(a);                          \
    } else if (p->D == 128) {                                                            \
      if (seg && bias) KERNEL<128, true, true><<<GRID, 256, 0, s>>>(a);                  \
      else if (seg) KERNEL<128, true, false><<<GRID, 256, 0, s>>>(a);                    \
      else if (bias) KERNEL<128, false, true><<<GRID, 256, 0, s>>>(a);                   \
      else KERNEL<128, false, false><<<GRID, 256, 0, s>>>(a);                            \
    } else {                                                                             \
      if (seg && bias) KERNEL<64, true, true><<<GRID, 256, 0, s>>>(a);                   \
      else if (seg) KERNEL<64, true, false><<<GRID, 256, 0, s>>>(a);                     \
      else if (bias) KERNEL<64, false, true><<<GRID, 256, 0, s>>>(a);                    \
      else KERNEL<64, false, false><<<GRID, 256, 0, s>>>(a);                             \
    }                                                                                    \
  } while (0)

int attn_fwd_f32(const ra_attn_fwd_params* p, hipStream_t s) {
  F32Args a{};
  a.q = (const float*)p->q; a.k = (const float*)p->k; a.v = (const float*)p->v;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.num = p->numerator; a.num_sb = p->num_stride_b; a.num_ss = p->num_stride_s;
  a.den = p->denominator; a.mx = p->max_score; a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  a.carry_is_initial = p->carry_is_initial;
  a.sdim = p->logit_dim > 0 ? p->logit_dim : p->D;
  a.out = (float*)p->out; a.out_sb = p->out_stride_b; a.out_ss = p->out_stride_s; a.out32 = p->out_f32;
  const bool seg = p->mask.segment_ids != nullptr, bias = p->mask.bias != nullptr, keep = p->mask.keep_bits_k != nullptr;
  const long long nwg = (long long)(p->Sq / XBM) * p->H * p->B;
  RA_REQUIRE(nwg < (1LL << 31), RA_ERR_UNSUPPORTED, "attn_fwd_f32: grid too large");
  const dim3 grid((unsigned)((nwg + 7) / 8 * 8));
  RA_F32_DISPATCH(attn_fwd_f32_kernel, grid);
  RA_CHECK_LAUNCH("attn_fwd_f32");
  return RA_OK;
}

int attn_bwd_f32(const ra_attn_bwd_params* p, int parts, hipStream_t s) {   // parts: bit 0 dq, bit 1 dk / dv
  F32Args a{};
  a.q = (const float*)p->q; a.k = (const float*)p->k; a.v = (const float*)p->v; a.g = (const float*)p->g;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.delta = p->delta; a.den = (float*)p->denominator; a.mx = (float*)p->max_score;      // read only here
  a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.dq = p->dq; a.dq_sb = p->dq_stride_b; a.dq_ss = p->dq_stride_s;
  a.dk = p->dk; a.dv = p->dv; a.dkv_sb = p->dkv_stride_b; a.dkv_ss = p->dkv_stride_s;
  a.sdim = p->logit_dim > 0 ? p->logit_dim : p->D;
  a.dq_initial = (p->grads_are_initial & RA_GRAD_INIT_DQ) != 0;
  a.dkv_initial = (p->grads_are_initial & RA_GRAD_INIT_DKV) != 0;
  a.dq_out = (float*)p->dq_out; a.dqo_sb = p->dq_out_stride_b; a.dqo_ss = p->dq_out_stride_s;
  a.dk_out = (float*)p->dk_out; a.dv_out = (float*)p->dv_out;
  a.dkvo_sb = p->dkv_out_stride_b; a.dkvo_ss = p->dkv_out_stride_s;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  const bool seg = p->mask.segment_ids != nullptr, bias = p->mask.bias != nullptr, keep = p->mask.keep_bits_k != nullptr;
  const long long nq = (long long)(p->Sq / XBM) * p->H * p->B, nk = (long long)(p->Skv / XBM) * p->H * p->B;
  RA_REQUIRE(nq < (1LL << 31) && nk < (1LL << 31), RA_ERR_UNSUPPORTED, "attn_bwd_f32: grid too large");
  const dim3 gq((unsigned)((nq + 7) / 8 * 8)), gk((unsigned)((nk + 7) / 8 * 8));
  if (parts & 2) RA_F32_DISPATCH(attn_bwd_dkv_f32_kernel, gk);
  if (parts & 1) RA_F32_DISPATCH(attn_bwd_dq_f32_kernel, gq);
  RA_CHECK_LAUNCH("attn_bwd_f32");
  return RA_OK;
}
#undef RA_F32_DISPATCH

}  // namespace ra
