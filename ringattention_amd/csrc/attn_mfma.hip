// bf16 MFMA blockwise attention for gfx950, head size 128 or 64 (a template parameter): forward, dK/dV and dQ of one ring step
// (carry in / carry out; ringattention_jax.py:130-145 forward, :147-209 backward).
//
// All three kernels share one structure.  A workgroup of 8 wavefronts owns 128 rows of one
// (batch, head) and walks 64-position tiles of the other operand, staged global -> registers -> LDS
// through three tile buffers.  The 8 wavefronts are 4 pairs; wave i and wave i+4 sit on the same SIMD.
// The producer wave of a pair computes the logits product (and dP in the backward) with
// v_mfma_f32_32x32x16_bf16 and does all the vector work (mask, online softmax, dS), then writes the bf16
// P / dS block to LDS; the consumer wave runs one 32-row block behind and does only the accumulation
// products, reading P / dS and the transposed operand with ds_read_b64_tr_b16.
// The logits are computed TRANSPOSED (S^T = K Q^T in the forward) so that a lane owns one query
// column: the running max / sum need one cross-lane step.
// Softmax runs in the log2 domain: p = exp2(s * log2(e)/sqrt(D) - m2).
#include <stdlib.h>
#include "common.hpp"

namespace ra {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int FBM = 128;         // query rows per workgroup
constexpr int FBN = 64;          // keys per tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// One launch for every device of a ring held on this GPU (ra_ring_step): the arrays are then the global ones and
// a workgroup first rebinds its arguments to the device (and K/V shard) its tile belongs to.
struct RingView {
  int n, idx;
  unsigned long long run, first, last, kv_first, kv_last;
};

struct FwdArgs {
  const uint16_t* q; const uint16_t* k; const uint16_t* v;
  int B, Sq, Skv, H;
  int64_t q_sb, q_ss, kv_sb, kv_ss;
  float* num; int64_t num_sb, num_ss;
  float* den; float* mx;
  int64_t st_sb, st_sh;
  MaskView mv;
  int carry_is_initial;
  int sdim;                                   // head size that scales the logits (the un-padded one)
  uint16_t* out; int64_t out_sb, out_ss;      // nullable: last step of the device, out = num / den instead of num
  float* out32;                               // nullable, with out: the quotient before rounding, strides of out
  RingView ring;                              // n == 0: one device per launch
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32); }
// max / sum of a value with its partner lane (lane ^ 32) through v_permlane32_swap: no LDS round trip
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float max_xor32(float x) {
  u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ s16x4 lds_read_tr(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p));
}

// natural <-> log2-domain running max; the "every key so far was masked" value mask_min is kept as is
__device__ __forceinline__ float max_to_log2(float m, float mask_min) { return m == mask_min ? m : m * kLog2e; }
__device__ __forceinline__ float max_from_log2(float m2, float mask_min) { return m2 == mask_min ? m2 : m2 * kLn2; }

// LDS tiles hold rows of 128 bf16 (256 bytes = all 64 banks) with no padding.  The 16-byte slot c
// of row r is stored at slot c ^ swz(r): sixteen consecutive rows then put a given logical slot in
// sixteen different bank groups (conflict-free 16-byte row reads), and four consecutive rows put four
// adjacent slots in sixteen different bank groups (conflict-free 4-row transpose reads).
// With head size 64 a row is 128 bytes (8 slots, two rows per 256 bytes): rows of equal parity two apart swap the
// halves of the slot range and rows four apart shift by one slot, which serves the same two read shapes.
template <int HD> __device__ __forceinline__ int swz(int r) {
  return HD == 128 ? (((r & 3) << 2) | ((r >> 2) & 3)) : ((((r >> 1) & 1) << 2) | ((r >> 2) & 3));
}

// number of leading tiles of a summary row (or column, with the given stride) that are "all kept"
__device__ __forceinline__ int keep_leading_full(const uint8_t* sm, int64_t stride, int n, int lane) {
  for (int base = 0; base < n; base += 64) {
    const int t = base + lane;
    const bool bad = t < n && sm[(int64_t)t * stride] != 2;
    const unsigned long long m = __builtin_amdgcn_ballot_w64(bad);
    if (m) return base + __builtin_ctzll(m);
  }
  return n;
}


// ================================================================== backward
// Two deterministic kernels (fp32 atomics reach ~1.3 TB/s at best on this part, far below what a
// fused dQ accumulation would need), both wave-specialised (see below):
//   dK,dV: key-stationary.  S = Q K^T and dP = dO V^T with K / V fragments resident in registers;
//          P and dS feed dV^T += dO^T P and dK^T += Q^T dS; Q^T / dO^T come from LDS transpose reads.
//   dQ   : query-stationary.  S^T = K Q^T and dP^T = V dO^T share the lane <-> query-column layout, so
//          max / denominator / delta are per-lane scalars; dQ^T += K^T dS^T takes K^T from the row-major
//          K tile with LDS transpose reads.
// Probabilities are recomputed from the saved max_score / denominator (ringattention_jax.py:226).
constexpr int KBN = 128;   // keys per workgroup in the dK/dV kernel (32 per wavefront pair)
constexpr int KBM = 64;    // query rows per tile

struct BwdArgs {
  const uint16_t* q; const uint16_t* k; const uint16_t* v; const uint16_t* g;
  int B, Sq, Skv, H;
  int64_t q_sb, q_ss, kv_sb, kv_ss;
  const float* delta; const float* den; const float* mx;
  int64_t st_sb, st_sh;
  float* dq; int64_t dq_sb, dq_ss;
  float* dk; float* dv; int64_t dkv_sb, dkv_ss;
  MaskView mv;
  int dq_initial, dkv_initial;                 // the fp32 accumulator holds zeros by definition: not read
  int sdim;                                    // head size that scales the logits (the un-padded one)
  uint16_t* dq_out; int64_t dqo_sb, dqo_ss;    // nullable: last call that adds into it, the sum goes here as bf16
  uint16_t* dk_out; uint16_t* dv_out; int64_t dkvo_sb, dkvo_ss;
  RingView ring;                               // n == 0: one device per launch
};

// Rebinds the arguments of a query-stationary workgroup (forward, dQ) to the ring device that owns the global
// 128-row query tile qt; false when that device does not run this ring step.
template <typename Args>
__device__ __forceinline__ bool ring_bind_common(Args& a, MaskView& mv, int dev, int shard) {
  const int n = a.ring.n, q_len = a.Sq / n, kv_len = a.Skv / n;
  a.q += (int64_t)dev * q_len * a.q_ss;
  a.k += (int64_t)shard * kv_len * a.kv_ss;
  a.v += (int64_t)shard * kv_len * a.kv_ss;
  a.den += (int64_t)dev * q_len;
  a.mx += (int64_t)dev * q_len;
  a.Sq = q_len; a.Skv = kv_len;
  mv.q_start = dev * (q_len / mv.qc);        // :32-33
  mv.k_start = shard * (kv_len / mv.kc);     // :37
  return true;
}
__device__ __forceinline__ bool ring_bind(FwdArgs& a, MaskView& mv, int& qt) {
  const int n = a.ring.n, tiles_dev = (a.Sq / n) / FBM;
  const int dev = qt / tiles_dev;
  if (!((a.ring.run >> dev) & 1ULL)) return false;
  const int shard = (dev - a.ring.idx + n) % n;                  // :36
  const int64_t r0 = (int64_t)dev * (a.Sq / n);
  if (a.num) a.num += r0 * a.num_ss;
  a.out = ((a.ring.last >> dev) & 1ULL) ? a.out + r0 * a.out_ss : nullptr;
  if (a.out32) a.out32 += r0 * a.out_ss;
  a.carry_is_initial = (int)((a.ring.first >> dev) & 1ULL);
  ring_bind_common(a, mv, dev, shard);
  qt -= dev * tiles_dev;
  return true;
}
__device__ __forceinline__ void ring_bind_bwd_rows(BwdArgs& a, int dev, int shard) {
  const int n = a.ring.n;
  const int64_t r0 = (int64_t)dev * (a.Sq / n), s0 = (int64_t)shard * (a.Skv / n);
  a.g += r0 * a.q_ss;
  a.delta += r0;
  if (a.dq) a.dq += r0 * a.dq_ss;
  a.dq_out = ((a.ring.last >> dev) & 1ULL) ? a.dq_out + r0 * a.dqo_ss : nullptr;
  a.dq_initial = (int)((a.ring.first >> dev) & 1ULL);
  if (a.dk) { a.dk += s0 * a.dkv_ss; a.dv += s0 * a.dkv_ss; }
  if ((a.ring.kv_last >> shard) & 1ULL) { a.dk_out += s0 * a.dkvo_ss; a.dv_out += s0 * a.dkvo_ss; }
  else { a.dk_out = nullptr; a.dv_out = nullptr; }
  a.dkv_initial = (int)((a.ring.kv_first >> shard) & 1ULL);
}
// dQ kernel: global 128-row query tile qt
__device__ __forceinline__ bool ring_bind_q(BwdArgs& a, MaskView& mv, int& qt) {
  const int n = a.ring.n, tiles_dev = (a.Sq / n) / FBM;
  const int dev = qt / tiles_dev;
  if (!((a.ring.run >> dev) & 1ULL)) return false;
  const int shard = (dev - a.ring.idx + n) % n;
  ring_bind_bwd_rows(a, dev, shard);
  ring_bind_common(a, mv, dev, shard);
  qt -= dev * tiles_dev;
  return true;
}
// dK/dV kernel: global 128-key block kt; its shard is held by device (shard + idx) mod n (:72)
__device__ __forceinline__ bool ring_bind_k(BwdArgs& a, MaskView& mv, int& kt) {
  const int n = a.ring.n, blocks_shard = (a.Skv / n) / 128;
  const int shard = kt / blocks_shard;
  const int dev = (shard + a.ring.idx) % n;
  if (!((a.ring.run >> dev) & 1ULL)) return false;
  ring_bind_bwd_rows(a, dev, shard);
  ring_bind_common(a, mv, dev, shard);
  kt -= shard * blocks_shard;
  return true;
}

typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store_bf16x4(uint16_t* p, const f32x4& t) {
  bf16x4_t o;
#pragma unroll
  for (int e = 0; e < 4; e++) o[e] = (__bf16)t[e];
  *(bf16x4_t*)p = o;
}
// 16-byte loads through a buffer descriptor: scalar base, scalar offset, one 32-bit byte offset per lane
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const uint16_t* p) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ uint4 ld_buf(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0);
  return uint4{v[0], v[1], v[2], v[3]};
}
// The 128 rows of a gradient that a workgroup owns but has nothing to add to (HD floats each, from acc / out, which
// point at row 0, head h): hand the accumulator on as bf16, or set it to the zeros it holds by definition.  In a ring
// step most workgroups may do nothing else (a later shard meets few of a device's documents), so this is written
// as a copy kernel: 16 bytes per lane, a row per 32 lanes, all eight requests of a lane in flight before the first
// store.  den (nullable, one value per row): the forward's out = numerator / denominator, which out32 (nullable, the
// strides of out) takes un-rounded as well.
template <int HD>
__device__ __forceinline__ void pass_rows(const float* acc, float* acc_w, int64_t acc_ss, uint16_t* out, int64_t out_ss,
                                          const float* den, int initial, int tid, float* out32 = nullptr) {
  if (!out && !initial) return;
  constexpr int PER = 128 * (HD / 4) / 512;
  f32x4 t[PER];
  float d[PER];
#pragma unroll
  for (int j = 0; j < PER; j++) {
    const int i = tid + j * 512, r = i / (HD / 4), c4 = (i % (HD / 4)) * 4;
    t[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    d[j] = 0.f;
    if (!initial) {
      t[j] = *(const f32x4*)(acc + (int64_t)r * acc_ss + c4);
      if (den) d[j] = den[r];
    }
  }
#pragma unroll
  for (int j = 0; j < PER; j++) {
    const int i = tid + j * 512, r = i / (HD / 4), c4 = (i % (HD / 4)) * 4;
    if (den) {
#pragma unroll
      for (int e = 0; e < 4; e++) t[j][e] /= d[j];               // 0 / 0 = NaN when nothing ran at all, as :52
    }
    if (out) {
      store_bf16x4(out + (int64_t)r * out_ss + c4, t[j]);
      if (out32) *(f32x4*)(out32 + (int64_t)r * out_ss + c4) = t[j];
    } else {
      *(f32x4*)(acc_w + (int64_t)r * acc_ss + c4) = t[j];
    }
  }
}

// ------------------------------------------------------------------ dK / dV, wave-specialised
// 8 wavefronts per workgroup, 128 keys: pair i = (wave i, wave i + 4) shares a SIMD and owns keys
// 32 i .. 32 i + 31.  The producer (wave i) runs S = Q K^T and dP - delta = dO V^T - delta with its
// K / V fragments in registers, turns them into P and dS (all of the vector work) and leaves both,
// rounded to bf16, in LDS.  The consumer (wave i + 4) reads them back as B operands and runs
// dV^T += dO^T P and dK^T += Q^T dS, with the 128 accumulator registers but no K / V fragments and no
// vector work.  Unlike the separate dK and dV kernels, S, dP and the exponentials are computed once.
//
// Steps are blocks of 32 query rows, one barrier per step.  In step n the producer issues the matrix
// products of block n + 1 between the vector work of block n, and the consumer accumulates block
// n - 1.  Query tiles (64 rows of Q and dO plus row statistics) cycle through three LDS buffers:
// tile t is read by the producer's products in steps 2t-1, 2t, by its vector work in 2t, 2t+1 and by
// the consumer in 2t+1, 2t+2; tile t+2 is stored in step 2t+1 (its buffer held tile t-1) from
// registers loaded two steps earlier.
constexpr int WS_PSTR = 40;                 // P / dS row stride in elements (conflict-free 16-byte reads)
constexpr int WS_PD = 32 * WS_PSTR;         // one 32 x 32 block

template <int HD, bool HAS_SEG, bool HAS_BIAS, int HAS_KEEP = 0>   // HD: head size, 64 or 128; HAS_KEEP: 0 no keep mask, 1 where(keep, w, min), 2 dropout
__global__ __launch_bounds__(512) void attn_bwd_dkv_ws_kernel(BwdArgs a) {
  // head size: elements per LDS tile row, a 64-row tile, contraction steps of 16 (per quarter of a block's products),
  // output blocks of 32, 16-byte chunks per row, rows per staging pass of 256 threads, passes per tile
  constexpr int TROW = HD, WS_TILE = 64 * HD, NK = HD / 16, KPG = HD / 64, NDB = HD / 32, CH = HD / 8;
  constexpr int SRP = 256 / CH, SNP = 64 / SRP;
  // Q tiles then dO tiles in one array: a dO address is the Q address plus a constant (an immediate offset)
  __shared__ __attribute__((aligned(16))) uint16_t QGs[6 * WS_TILE];
  uint16_t* const Qs = QGs;
  uint16_t* const Gs = QGs + 3 * WS_TILE;
  __shared__ __attribute__((aligned(16))) uint16_t Ps[4][2][2][WS_PD];     // [pair][buffer][P | dS]
  __shared__ __attribute__((aligned(16))) float st_m2[3][KBM];
  __shared__ __attribute__((aligned(16))) float st_rden[3][KBM];
  __shared__ __attribute__((aligned(16))) float st_lse2[3][KBM];
  __shared__ __attribute__((aligned(16))) float st_delta[3][KBM];   // holds -delta
  __shared__ __attribute__((aligned(16))) int st_seg[3][KBM];
  __shared__ float st_bias[4][64];           // [pair][lane]: the lane's key's clamped, scaled bias

  MaskView mv = a.mv;
  mv.resolve();
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int role = __builtin_amdgcn_readfirstlane(wave >> 2), pair = wave & 3;
  const int nkt = a.Skv / KBN;
  // Workgroups go to the 8 XCDs round-robin, and each XCD has its own L2.  Give XCD x the contiguous
  // range x of (batch, head, key block) triples: the workgroups resident on one XCD are then
  // neighbouring key blocks of one head, which sweep nearly the same query rows at the same time, so a
  // Q / dO tile is fetched into that L2 once instead of once per workgroup.
  const int per_xcd = (a.B * a.H * nkt + 7) >> 3;
  int wg = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (wg >= a.B * a.H * nkt) return;
  int kt = wg % nkt;
  wg /= nkt;
  const int h = wg % a.H, b = wg / a.H;
  if (a.ring.n && !ring_bind_k(a, mv, kt)) return;
  const int k0 = kt * KBN;
  const int krow = k0 + pair * 32 + lo;    // this lane's key row (local)

  const int gk0 = (int)mv.global_k(k0);
  const int gk = gk0 + pair * 32 + lo;
  const int gq_base = (int)mv.global_q(0);
  const int nqt = a.Sq / KBM;
  int qt_first = nqt;
  {
    int nqc = a.Sq / mv.qc, lo_c = 0, hi_c = nqc;
    while (lo_c < hi_c) {
      int mid = (lo_c + hi_c) >> 1;
      if (mv.run_prefix_keys(mid, a.Skv) > k0) hi_c = mid; else lo_c = mid + 1;
    }
    if (lo_c < nqc) qt_first = lo_c * (mv.qc / KBM);
    if (mv.cbs > 0 && mv.skip_tiles && qt_first < nqt) {
      long long need = (long long)(gk0 / mv.cbs) * mv.cbs - gq_base;
      if (need > 0) {
        int t = (int)(need / KBM);
        if (t > qt_first) qt_first = t < nqt ? t : nqt;
      }
    }
  }
  int qt_end = nqt;
  if (HAS_SEG && mv.seg_mm && mv.skip_tiles && qt_first < nqt) {
    __shared__ int hull2[2];
    int t_first, t_last;
    seg_hull_of_rows(mv, b, gk0, KBN, gq_base / RA_SEG_TILE + qt_first, nqt - qt_first, hull2, tid, 512, t_first, t_last);
    qt_end = qt_first + t_last;
    qt_first += t_first;
  }
  if (HAS_KEEP && mv.skip_tiles && qt_first < qt_end) {
    __shared__ int khull2[2];
    int t_first, t_last;
    keep_qtile_hull(mv, b, h, (gk0 - mv.keep_k0) / 64, KBN / 64, mv.keep_q0 / 64 + qt_first, qt_end - qt_first, khull2, tid, 512,
                    t_first, t_last);
    qt_end = qt_first + t_last;
    qt_first += t_first;
  }
  if (qt_first >= qt_end) {                // nothing to add for these keys
    const int64_t o = (int64_t)b * a.dkv_sb + (int64_t)k0 * a.dkv_ss + (int64_t)h * HD;
    const int64_t oo = (int64_t)b * a.dkvo_sb + (int64_t)k0 * a.dkvo_ss + (int64_t)h * HD;
    pass_rows<HD>(a.dk ? a.dk + o : nullptr, a.dk ? a.dk + o : nullptr, a.dkv_ss, a.dk_out ? a.dk_out + oo : nullptr, a.dkvo_ss,
              nullptr, a.dkv_initial, tid);
    pass_rows<HD>(a.dv ? a.dv + o : nullptr, a.dv ? a.dv + o : nullptr, a.dkv_ss, a.dv_out ? a.dv_out + oo : nullptr, a.dkvo_ss,
              nullptr, a.dkv_initial, tid);
    return;
  }
  const int ntq = qt_end - qt_first;       // query tiles of 64 rows
  const int nblk = 2 * ntq;                // blocks of 32 rows

  const float c = kLog2e / sqrtf((float)a.sdim);
  const float kMask2 = mv.mask_min;

  // ---- staging of the Q / dO tiles through registers: producers bring Q, consumers dO and the statistics
  const int srow = (tid & 255) / CH, schunk = tid & (CH - 1);
  const int s_off = srow * TROW + ((schunk ^ swz<HD>(srow)) << 3);
  // a tile is read through a buffer descriptor at its first row (scalar registers) with one 32-bit byte offset per
  // lane: half the address data of 64-bit pointers per lane, and two registers less
  const uint16_t* sg = (role == 0 ? a.q : a.g) + (int64_t)b * a.q_sb + (int64_t)h * HD + (int64_t)(qt_first * KBM) * a.q_ss;
  const uint32_t sg_lane = 2u * (uint32_t)(schunk * 8 + srow * (int)a.q_ss);
  const uint32_t row16b = 2u * SRP * (uint32_t)a.q_ss;        // one staging pass further
  uint16_t* sl = (role == 0 ? Qs : Gs) + s_off;
  uint4 sr0, sr1, sr2 = {}, sr3 = {};
  float r_m = 0.f, r_den = 1.f, r_delta = 0.f;
  int r_seg = 0;
  // query chunk index and offset inside the chunk of the first row of the next tile to request (tiles are requested
  // in order and never straddle a chunk: query_chunk_size is a multiple of 128): no division per tile
  int ld_c = 0, ld_o = 0;
  if (HAS_SEG) { ld_c = (qt_first * KBM) / mv.qc; ld_o = qt_first * KBM - ld_c * mv.qc; }
#define RA_WS_LOAD(T)                                                                                   \
  {                                                                                                     \
    const int t_ = min((T), ntq - 1);                                                                   \
    const __amdgpu_buffer_rsrc_t rs_ = tile_rsrc(sg + (int64_t)t_ * KBM * a.q_ss);                      \
    sr0 = ld_buf(rs_, sg_lane, 0); sr1 = ld_buf(rs_, sg_lane, row16b);                                  \
    if (SNP == 4) { sr2 = ld_buf(rs_, sg_lane, 2 * row16b); sr3 = ld_buf(rs_, sg_lane, 3 * row16b); }   \
    if (tid >= 256 && tid < 256 + KBM) {                                                                \
      const int row_ = (qt_first + t_) * KBM + tid - 256;                                               \
      const int64_t st_ = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + row_;                           \
      r_m = a.mx[st_]; r_den = a.den[st_]; r_delta = a.delta[st_];                                      \
      if (HAS_SEG) {                                                                                    \
        int idx_ = clamp_seg_index(((long long)mv.q_start + ld_c) * mv.qc, mv.qc, mv.seg_len, ld_o + tid - 256); \
        r_seg = mv.seg[(int64_t)b * mv.seg_sb + idx_];                                                  \
      }                                                                                                 \
    }                                                                                                   \
    if (HAS_SEG && (T) < ntq - 1) { ld_o += KBM; if (ld_o >= mv.qc) { ld_o -= mv.qc; ld_c++; } }         \
  }
#define RA_WS_STORE(BUF)                                                                                \
  {                                                                                                     \
    uint16_t* d_ = sl + (BUF) * WS_TILE;                                                                \
    *(uint4*)(d_) = sr0; *(uint4*)(d_ + SRP * TROW) = sr1;                                              \
    if (SNP == 4) { *(uint4*)(d_ + 2 * SRP * TROW) = sr2; *(uint4*)(d_ + 3 * SRP * TROW) = sr3; }       \
    if (tid >= 256 && tid < 256 + KBM) {                                                                \
      const float m2_ = max_to_log2(r_m, kMask2);                                                       \
      st_m2[BUF][tid - 256] = m2_; st_rden[BUF][tid - 256] = 1.f / r_den;                               \
      st_lse2[BUF][tid - 256] = m2_ + __log2f(r_den); st_delta[BUF][tid - 256] = -r_delta;              \
      if (HAS_SEG) st_seg[BUF][tid - 256] = r_seg;                                                      \
    }                                                                                                   \
  }
  // Both roles stage the first tiles, then meet at the first barrier, each inside its own branch: the producer's K and
  // V fragments are requested before the staging, so that their latency runs next to it instead of after the barrier,
  // and being defined inside the branch they take no register of the consumers
#define RA_WS_PROLOGUE  \
  RA_WS_LOAD(0); RA_WS_STORE(0); RA_WS_LOAD(1); RA_WS_STORE(1); RA_WS_LOAD(2); __syncthreads();

  if (role == 0) {
    // =========================== producer: S, dP -> P, dS
    bf16x8 kf[NK], vf[NK];
    {
      const int64_t koff = (int64_t)b * a.kv_sb + (int64_t)krow * a.kv_ss + (int64_t)h * HD + hi * 8;
#pragma unroll
      for (int t = 0; t < NK; t++) {
        kf[t] = *(const bf16x8*)(a.k + koff + t * 16);
        vf[t] = *(const bf16x8*)(a.v + koff + t * 16);
      }
    }
    RA_WS_PROLOGUE
    const int qlim = mv.cbs > 0 ? (gk / mv.cbs) * mv.cbs : -0x7fffffff;       // masked iff gq < qlim
    const int qlim_wave = __builtin_amdgcn_readfirstlane(mv.cbs > 0 ? ((gk0 + pair * 32 + 31) / mv.cbs) * mv.cbs : -0x7fffffff);
    int seg_k = 0;
    float bias2 = 0.f;
    if (HAS_SEG) {
      int idx = clamp_seg_index(((long long)mv.k_start + krow / mv.kc) * mv.kc, mv.kc, mv.seg_len, krow % mv.kc);
      seg_k = mv.seg[(int64_t)b * mv.seg_sb + idx];
    }
    // a bias at the level of the mask value (a padding mask passed as where(keep, 0, finfo.min)) absorbs the logit in
    // the reference and would overflow here once scaled: the key then counts as masked for every row (its accumulators
    // start at -inf, the masked path puts the mask value itself), and its wavefront takes the masked path throughout
    bool lane_bm = false;
    if (HAS_BIAS) {
      float bv = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + (int64_t)gk * mv.bias_sk];
      if (mv.any_mask) bv = fminf(bv, 0.f);
      lane_bm = bv * kLog2e <= kMask2;
      bias2 = lane_bm ? RA_NEG_INF : bv * kLog2e / c;          // the S accumulators start from it
      st_bias[pair][lane] = bias2;      // kept in LDS, not in a register: every lane reads back its own slot
    }
    const bool wave_bm = HAS_BIAS && __builtin_amdgcn_ballot_w64(lane_bm) != 0ULL;
    int n_off[NK];
#pragma unroll
    for (int t = 0; t < NK; t++) n_off[t] = lo * TROW + (((2 * t + hi) ^ swz<HD>(lo)) << 3);
    uint16_t* const pw = &Ps[pair][0][0][lo * WS_PSTR + hi * 4];
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

    // accumulators start at S = 0 and dP = -delta[row] (rows 8g + 4hi + e of block BLK of buffer BUF)
#define RA_WS_INIT(SN, DPN, BUF, BLK)                                                                   \
  _Pragma("unroll") for (int g = 0; g < 4; g++) {                                                       \
    const f32x4 d_ = *(const f32x4*)&st_delta[BUF][(BLK) * 32 + g * 8 + hi * 4];                        \
    const float b0_ = HAS_BIAS ? st_bias[pair][lane] : 0.f;                                                \
    _Pragma("unroll") for (int e = 0; e < 4; e++) { SN[g * 4 + e] = b0_; DPN[g * 4 + e] = d_[e]; } \
  }
    // A operands of two contraction steps (32 of the 128 head dimensions) of block BLK of buffer BUF
#define RA_WS_AREAD(G, QA, GA, BUF, BLK)                                                                \
  _Pragma("unroll") for (int i = 0; i < KPG; i++) {                                                       \
    const uint16_t* p_ = Qs + (BUF) * WS_TILE + n_off[KPG * (G) + i];                                     \
    QA[i] = *(const bf16x8*)(p_ + (BLK) * 32 * TROW);                                                   \
    GA[i] = *(const bf16x8*)(p_ + (BLK) * 32 * TROW + 3 * WS_TILE);                                     \
  }
#define RA_WS_AMFMA(G, QA, GA, SN, DPN)                                                                 \
  _Pragma("unroll") for (int i = 0; i < KPG; i++) {                                                       \
    SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(QA[i], kf[KPG * (G) + i], SN, 0, 0, 0);                  \
    DPN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(GA[i], vf[KPG * (G) + i], DPN, 0, 0, 0);                \
  }
    // eight rows (registers 4G .. 4G+3 of both halves) of P and dS, no masking: VL = lse2 of the rows
#define RA_WS_VECTOR_PLAIN(G, SC, DPC, VL, PB)                                                          \
  {                                                                                                     \
    bf16x4 p4, d4;                                                                                      \
    _Pragma("unroll") for (int e = 0; e < 4; e++) {                                                     \
      const float p = fast_exp2(fmaf(SC[(G) * 4 + e], c, -VL[e]));                       /* :226 */     \
      p4[e] = (__bf16)p;                                                                                \
      d4[e] = (__bf16)(p * DPC[(G) * 4 + e]);                                            /* :229 */     \
    }                                                                                                   \
    *(bf16x4*)(pw + (PB) * 2 * WS_PD + (G) * 8) = p4;                                                   \
    *(bf16x4*)(pw + (PB) * 2 * WS_PD + WS_PD + (G) * 8) = d4;                                           \
  }
#define RA_WS_VECTOR_MASKED(G, SC, DPC, BUF, BLK, PB)                                                   \
  {                                                                                                     \
    const int qrow0 = (BLK) * 32 + (G) * 8 + hi * 4;                                                    \
    bf16x4 p4, d4;                                                                                      \
    const f32x4 vm2 = *(const f32x4*)&st_m2[BUF][qrow0];                                                \
    const f32x4 vrd = *(const f32x4*)&st_rden[BUF][qrow0];                                              \
    _Pragma("unroll") for (int e = 0; e < 4; e++) {                                                     \
      float x = SC[(G) * 4 + e] * c;                                                                    \
      bool masked = (gq_tile + qrow0 + e < qlim);                                                       \
      /* another document, or this lane's key carries a bias at the level of the mask value */          \
      bool sne_ = HAS_BIAS && lane_bm;                                                                  \
      if (HAS_SEG) sne_ = sne_ || st_seg[BUF][qrow0 + e] != seg_k;                                      \
      masked = masked || sne_;                                                                          \
      if (HAS_KEEP == 2 && (HAS_SEG || HAS_BIAS)) {                                                     \
        /* as below, with such pairs: they count as masked once more */                                 \
        x = (((kw_cur >> ((BLK) * 32 + (G) * 8 + e)) & 1) && !sne_) ? x : kMask2;                       \
        x = (((kw_some >> ((BLK) * 32 + (G) * 8 + e)) & 1) &&                                           \
             (((kw_k >> ((BLK) * 32 + (G) * 8 + e)) & 1) || !sne_)) ? x : RA_NEG_INF;                   \
      } else if (HAS_KEEP == 2) {                                                                       \
        /* dropout adds mask_min (:321).  kw_cur: pairs kept and causally allowed; kw_some: at least    \
           one of the two, so a clear bit there is mask_min added twice = -inf */                       \
        x = ((kw_cur >> ((BLK) * 32 + (G) * 8 + e)) & 1) ? x : kMask2;                                  \
        x = ((kw_some >> ((BLK) * 32 + (G) * 8 + e)) & 1) ? x : RA_NEG_INF;                             \
      } else {                                                                                          \
        if (HAS_KEEP) masked = masked || !((kw_cur >> ((BLK) * 32 + (G) * 8 + e)) & 1);                 \
        x = masked ? kMask2 : x;                                                                        \
      }                                                                                                 \
      const float p = fast_exp2(x - vm2[e]) * vrd[e];                                    /* :226 */     \
      p4[e] = (__bf16)p;                                                                                \
      d4[e] = (__bf16)(p * DPC[(G) * 4 + e]);                                            /* :229 */     \
    }                                                                                                   \
    *(bf16x4*)(pw + (PB) * 2 * WS_PD + (G) * 8) = p4;                                                   \
    *(bf16x4*)(pw + (PB) * 2 * WS_PD + WS_PD + (G) * 8) = d4;                                           \
  }
    // one step: vector work of block BLK of buffer BUF (accumulators SC, DPC) in four groups of eight
    // rows, each preceded by a quarter of the products of block NBLK of buffer NBUF (into SN, DPN);
    // the operands of a group are requested from LDS one group ahead
#define RA_WS_PRODUCE(SC, DPC, SN, DPN, BUF, BLK, NBUF, NBLK, PB, MASKED)                               \
  {                                                                                                     \
    bf16x8 qa_[2][KPG], ga_[2][KPG];                                                                        \
    f32x4 vl_[2];                                                                                       \
    RA_WS_AREAD(0, qa_[0], ga_[0], NBUF, NBLK);                                                         \
    if (!(MASKED)) vl_[0] = *(const f32x4*)&st_lse2[BUF][(BLK) * 32 + hi * 4];                          \
    RA_WS_INIT(SN, DPN, NBUF, NBLK);                                                                    \
    _Pragma("unroll") for (int g = 0; g < 4; g++) {                                                     \
      if (g < 3) {                                                                                      \
        RA_WS_AREAD(g + 1, qa_[(g + 1) & 1], ga_[(g + 1) & 1], NBUF, NBLK);                             \
        if (!(MASKED)) vl_[(g + 1) & 1] = *(const f32x4*)&st_lse2[BUF][(BLK) * 32 + (g + 1) * 8 + hi * 4]; \
      }                                                                                                 \
      __builtin_amdgcn_sched_barrier(0);                                                                \
      RA_WS_AMFMA(g, qa_[g & 1], ga_[g & 1], SN, DPN);                                                  \
      if (MASKED) RA_WS_VECTOR_MASKED(g, SC, DPC, BUF, BLK, PB)                                         \
      else RA_WS_VECTOR_PLAIN(g, SC, DPC, vl_[g & 1], PB)                                               \
      __builtin_amdgcn_sched_barrier(0);                                                                \
    }                                                                                                   \
  }

    f32x16 s_a, dp_a, s_b, dp_b;
    RA_WS_INIT(s_a, dp_a, 0, 0);
#pragma unroll
    for (int g = 0; g < 4; g++) {
      bf16x8 qa_[KPG], ga_[KPG];
      RA_WS_AREAD(g, qa_, ga_, 0, 0);
      RA_WS_AMFMA(g, qa_, ga_, s_a, dp_a);
    }

    // packed keep mask: this lane's word (bits over the 64 rows of a query tile) and this pair's summary byte
    const uint64_t* kw_ptr = nullptr;
    const uint8_t* ks_ptr = nullptr;
    uint64_t kw_cur = 0, kw_nxt = 0, kw_some = 0, kw_k = 0;     // kw_k: the kept bits before the causal limit is folded in
    (void)kw_some; (void)kw_k;
    int ks_cur = 2, ks_nxt = 2;
    if (HAS_KEEP) {
      kw_ptr = mv.kbits_q + (int64_t)b * mv.kpack_sb + (int64_t)h * mv.kpack_sh +
               (int64_t)(mv.keep_q0 / 64 + qt_first) * mv.keep_K + gk - mv.keep_k0;
      ks_ptr = mv.ksum + (int64_t)b * mv.ksum_sb + (int64_t)h * mv.ksum_sh +
               (int64_t)(mv.keep_q0 / 64 + qt_first) * (mv.keep_K / 64) + (gk0 - mv.keep_k0 + pair * 32) / 64;
      kw_nxt = kw_ptr[0]; ks_nxt = ks_ptr[0];
    }
    // segment ids: a query tile whose 64 rows all carry the one id of this pair's keys needs no compare
    const int2* smm_ptr = nullptr;
    bool sk_uniform = false, sp_cur = false, sp_nxt = false;
    int sk_id = 0;
    int2 qmm_nxt = make_int2(0, 0);
    if (HAS_SEG && mv.seg_mm) {
      smm_ptr = (const int2*)(mv.seg_mm + (int64_t)(mv.seg_sb ? b : 0) * mv.seg_tiles * 2);
      const int2 kmm = smm_ptr[min((gk0 + pair * 32) / RA_SEG_TILE, mv.seg_tiles - 1)];
      sk_uniform = kmm.x == kmm.y;
      sk_id = kmm.x;
      if (sk_uniform) {
        const int2 qmm = smm_ptr[min(gq_base / RA_SEG_TILE + qt_first, mv.seg_tiles - 1)];
        sp_nxt = qmm.x == sk_id && qmm.y == sk_id;
        qmm_nxt = smm_ptr[min(gq_base / RA_SEG_TILE + qt_first + min(1, ntq - 1), mv.seg_tiles - 1)];
      }
    }
    int cur = 0;
    for (int t = 0; t < ntq; t++) {
      const int nxt = cur == 2 ? 0 : cur + 1, prv = cur == 0 ? 2 : cur - 1;
      const int gq_tile = gq_base + (qt_first + t) * KBM;
      if (HAS_SEG) {
        sp_cur = sp_nxt;
        if (sk_uniform) {
          // the range of tile t + 1 was requested one tile ago (a use right after the load would stall the
          // producer for a global load's latency in every tile); request that of tile t + 2
          sp_nxt = qmm_nxt.x == sk_id && qmm_nxt.y == sk_id;
          qmm_nxt = smm_ptr[min(gq_base / RA_SEG_TILE + qt_first + min(t + 2, ntq - 1), mv.seg_tiles - 1)];
        }
      }
      if (HAS_KEEP) {                      // this tile's word and summary; request the next tile's
        kw_cur = kw_nxt >> (4 * hi); ks_cur = ks_nxt;
        const int tn = min(t + 1, ntq - 1);
        kw_nxt = kw_ptr[(int64_t)tn * mv.keep_K]; ks_nxt = ks_ptr[(int64_t)tn * (mv.keep_K / 64)];
        if (HAS_KEEP == 2) {               // fold this key's causal limit (rows before qlim are masked) into the words
          const int nmask = (int)max(0LL, min(64LL, (long long)qlim - gq_tile));
          const uint64_t cw = (nmask >= 64 ? 0ULL : (~0ULL << nmask)) >> (4 * hi);
          kw_k = kw_cur;
          kw_some = kw_cur | cw;
          kw_cur &= cw;
        }
      }
      // step 2t: vector work of block 0 of tile t, products of block 1
      if ((HAS_SEG && !sp_cur) || (gq_tile < qlim_wave) || (HAS_KEEP && ks_cur != 2) || wave_bm) {
        RA_WS_PRODUCE(s_a, dp_a, s_b, dp_b, cur, 0, cur, 1, 0, true);
      } else {
        RA_WS_PRODUCE(s_a, dp_a, s_b, dp_b, cur, 0, cur, 1, 0, false);
      }
      __syncthreads();
      // step 2t + 1: tile t + 2 goes to LDS, tile t + 3 is requested; vector work of block 1, products of
      // block 0 of tile t + 1 (the last tile computes a block that is never used)
      RA_WS_STORE(prv);
      RA_WS_LOAD(t + 3);
      if ((HAS_SEG && !sp_cur) || (gq_tile + 32 < qlim_wave) || (HAS_KEEP && ks_cur != 2) || wave_bm) {
        RA_WS_PRODUCE(s_b, dp_b, s_a, dp_a, cur, 1, nxt, 0, 1, true);
      } else {
        RA_WS_PRODUCE(s_b, dp_b, s_a, dp_a, cur, 1, nxt, 0, 1, false);
      }
      __syncthreads();
      cur = nxt;
    }
    __syncthreads();      // step 2 ntq: the consumer's last block
  } else {
    // =========================== consumer: dV^T += dO^T P, dK^T += Q^T dS
    RA_WS_PROLOGUE
    f32x16 dkacc[NDB], dvacc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) { dkacc[db][r] = 0.f; dvacc[db][r] = 0.f; }
    // transpose reads with the natural contraction order: rows 8 hi + (i >> 2) (+4 for the second read)
    int t_off[NDB][2];
    {
      const int i = lane & 15, rr = (i >> 2) + 8 * hi, c0 = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), half = lane & 1;
#pragma unroll
      for (int db = 0; db < NDB; db++) {
        t_off[db][0] = rr * TROW + (((4 * db + c0) ^ swz<HD>(rr)) << 3) + half * 4;
        t_off[db][1] = (rr + 4) * TROW + (((4 * db + c0) ^ swz<HD>(rr + 4)) << 3) + half * 4;
      }
    }
    const uint16_t* const pr = &Ps[pair][0][0][lo * WS_PSTR + hi * 8];   // B operand: key column lo, 8 query rows

    // The 16 products of a block run as four groups of four: dV with query rows 0..15 of the block, dK
    // with the same rows, then both with rows 16..31.  The transposed A operands of a group are read
    // one group ahead, those of the first group before the barrier that publishes the block's P / dS.
#define RA_WS_CREAD(K, F, BUF, BLK)                                                                     \
  {                                                                                                     \
    const uint16_t* tp_ = (((K) & 1) ? Qs : Gs) + (BUF) * WS_TILE + ((BLK) * 32 + ((K) >> 1) * 16) * TROW; \
    _Pragma("unroll") for (int db = 0; db < NDB; db++) {                                                  \
      const s16x4 x0_ = lds_read_tr(tp_ + t_off[db][0]);                                                \
      const s16x4 x1_ = lds_read_tr(tp_ + t_off[db][1]);                                                \
      F[db] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(x0_, x1_, 0, 1, 2, 3, 4, 5, 6, 7));    \
    }                                                                                                   \
  }
#define RA_WS_CMFMA(K, F, BOP)                                                                          \
  _Pragma("unroll") for (int db = 0; db < NDB; db++) {                                                    \
    if ((K) & 1) dkacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[db], BOP, dkacc[db], 0, 0, 0);   \
    else dvacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[db], BOP, dvacc[db], 0, 0, 0);           \
  }
    // block BLK of buffer BUF with the P / dS pair PB; fa holds group 0 on entry and, on exit, group 0
    // of block NBLK of buffer NBUF
#define RA_WS_CONSUME(BUF, BLK, PB, NBUF, NBLK)                                                         \
  {                                                                                                     \
    const bf16x8 p0_ = *(const bf16x8*)(pr + (PB) * 2 * WS_PD);                                         \
    const bf16x8 p1_ = *(const bf16x8*)(pr + (PB) * 2 * WS_PD + 16);                                    \
    const bf16x8 d0_ = *(const bf16x8*)(pr + (PB) * 2 * WS_PD + WS_PD);                                 \
    const bf16x8 d1_ = *(const bf16x8*)(pr + (PB) * 2 * WS_PD + WS_PD + 16);                            \
    RA_WS_CREAD(1, fb, BUF, BLK);                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(0, fa, p0_);                                                                            \
    RA_WS_CREAD(2, fa, BUF, BLK);                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(1, fb, d0_);                                                                            \
    RA_WS_CREAD(3, fb, BUF, BLK);                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(2, fa, p1_);                                                                            \
    RA_WS_CREAD(0, fa, NBUF, NBLK);                                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(3, fb, d1_);                                                                            \
  }
    bf16x8 fa[NDB], fb[NDB];
    int cur = 0;
    RA_WS_CREAD(0, fa, 0, 0);
    __syncthreads();      // step 0
    for (int t = 0; t < ntq; t++) {
      const int prv = cur == 0 ? 2 : cur - 1, nxt = cur == 2 ? 0 : cur + 1;
      // step 2t + 1
      RA_WS_STORE(prv);
      RA_WS_LOAD(t + 3);
      RA_WS_CONSUME(cur, 0, 0, cur, 1);
      __syncthreads();
      // step 2t + 2
      RA_WS_CONSUME(cur, 1, 1, nxt, 0);
      __syncthreads();
      cur = nxt;
    }

    // dk += acc / sqrt(D) (:231), dv += acc (:232); this pair owns its 32 key rows
    const float rscale = 1.f / sqrtf((float)a.sdim);
    const int64_t ooff = (int64_t)b * a.dkv_sb + (int64_t)krow * a.dkv_ss + (int64_t)h * HD + hi * 4;
    const int64_t oout = (int64_t)b * a.dkvo_sb + (int64_t)krow * a.dkvo_ss + (int64_t)h * HD + hi * 4;
    // dk, then dv; all the old values of one are requested before its first store (a load issued after a store is
    // not waited for until that store has completed too: one in-order counter)
#pragma unroll
    for (int which = 0; which < 2; which++) {
      float* const pacc = (which == 0 ? a.dk : a.dv) + ooff;
      uint16_t* const pout = (which == 0 ? a.dk_out : a.dv_out) + oout;
      f32x4 old[NDB][4];
#pragma unroll
      for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          old[db][g] = f32x4{0.f, 0.f, 0.f, 0.f};
          if (!a.dkv_initial) old[db][g] = *(const f32x4*)(pacc + db * 32 + g * 8);
        }
#pragma unroll
      for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          f32x4 t = old[db][g];
#pragma unroll
          for (int e = 0; e < 4; e++) t[e] += which == 0 ? dkacc[db][g * 4 + e] * rscale : dvacc[db][g * 4 + e];
          if (a.dk_out) store_bf16x4(pout + db * 32 + g * 8, t);     // last call for these keys: the sum as bf16 (:89)
          else *(f32x4*)(pacc + db * 32 + g * 8) = t;
        }
    }
  }
#undef RA_WS_PROLOGUE
#undef RA_WS_LOAD
#undef RA_WS_STORE
#undef RA_WS_INIT
#undef RA_WS_AREAD
#undef RA_WS_AMFMA
#undef RA_WS_VECTOR_PLAIN
#undef RA_WS_VECTOR_MASKED
#undef RA_WS_CREAD
#undef RA_WS_CMFMA
#undef RA_WS_PRODUCE
#undef RA_WS_CONSUME
}

// ------------------------------------------------------------------ dQ, wave-specialised
// The mirror image of the dK / dV kernel above: 128 query rows per workgroup, pair i owns rows
// 32 i .. 32 i + 31 and keeps their Q and dO fragments in the producer's registers; K / V tiles of 64
// keys stream through three LDS buffers.  Per block of 32 keys the producer runs S^T = K Q^T and
// dP^T - delta = V dO^T - delta, forms dS^T and leaves it in LDS; the consumer accumulates
// dQ^T += K^T dS^T one block behind.  The row statistics belong to the lane's query column and stay in
// registers.
#ifndef WS_DQ_VALU_PER_MFMA
#define WS_DQ_VALU_PER_MFMA 5
#endif
template <int HD, bool HAS_SEG, bool HAS_BIAS, int HAS_KEEP = 0>   // HD: head size, 64 or 128; HAS_KEEP: 0 no keep mask, 1 where(keep, w, min), 2 dropout
__global__ __launch_bounds__(512) void attn_bwd_dq_ws_kernel(BwdArgs a) {
  // head size: elements per LDS tile row, a 64-row tile, contraction steps of 16 (per quarter of a block's products),
  // output blocks of 32, 16-byte chunks per row, rows per staging pass of 256 threads, passes per tile
  constexpr int TROW = HD, WS_TILE = 64 * HD, NK = HD / 16, KPG = HD / 64, NDB = HD / 32, CH = HD / 8;
  constexpr int SRP = 256 / CH, SNP = 64 / SRP;
  // K tiles then V tiles in one array: a V address is the K address plus a constant (an immediate offset)
  __shared__ __attribute__((aligned(16))) uint16_t KVs[6 * WS_TILE];
  uint16_t* const Ks = KVs;
  uint16_t* const Vs = KVs + 3 * WS_TILE;
  __shared__ __attribute__((aligned(16))) uint16_t Ds[4][2][WS_PD];        // [pair][buffer] dS^T as [q][key]
  __shared__ int seg_ks[3][FBN];
  __shared__ float bias_ks[3][FBN];

  MaskView mv = a.mv;
  mv.resolve();
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int role = __builtin_amdgcn_readfirstlane(wave >> 2), pair = wave & 3;
  const int nqt = a.Sq / FBM;
  // XCD x takes the contiguous range x of (batch, head, query tile) triples: the workgroups resident on
  // one XCD then stream the same K / V tiles of one head through that XCD's L2 at the same time
  const int per_xcd = (a.B * a.H * nqt + 7) >> 3;
  int wg = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (wg >= a.B * a.H * nqt) return;
  int qt = nqt - 1 - (wg % nqt);           // latest query tiles (most keys under causal) first
  wg /= nqt;
  const int h = wg % a.H, b = wg / a.H;
  if (a.ring.n && !ring_bind_q(a, mv, qt)) return;
  const int q0 = qt * FBM;
  const int qrow = q0 + pair * 32 + lo;

  const int qi = q0 / mv.qc;
  int kend = mv.run_prefix_keys(qi, a.Skv);
  const int gq0 = (int)mv.global_q(q0);
  const int gk0_shard = (int)mv.global_k(0);
  if (mv.cbs > 0 && mv.skip_tiles) {
    long long lim = ((long long)(gq0 + FBM - 1) / mv.cbs + 1) * mv.cbs;
    long long n = lim - gk0_shard;
    if (n < kend) kend = n > 0 ? (int)n : 0;
  }
  int ntiles = (kend + FBN - 1) / FBN;
  int k_base = 0;
  if (HAS_SEG && mv.seg_mm && mv.skip_tiles && ntiles > 0) {
    __shared__ int hull2[2];
    int t_first, t_last;
    seg_hull_of_rows(mv, b, gq0, FBM, gk0_shard / RA_SEG_TILE, ntiles, hull2, tid, 512, t_first, t_last);
    k_base = t_first * FBN;
    ntiles = t_last - t_first;
  }
  if (HAS_KEEP && mv.skip_tiles && ntiles > 0) {
    __shared__ int khull2[2];
    int t_first, t_last;
    keep_ktile_hull(mv, b, h, (mv.keep_q0 + q0) / 64, FBM / 64, (gk0_shard + k_base - mv.keep_k0) / 64, ntiles, khull2, tid, 512,
                    t_first, t_last);
    k_base += t_first * FBN;
    ntiles = t_last - t_first;
  }
  if (ntiles == 0) {           // nothing to add to dq
    float* const dq0 = a.dq ? a.dq + (int64_t)b * a.dq_sb + (int64_t)q0 * a.dq_ss + (int64_t)h * HD : nullptr;
    pass_rows<HD>(dq0, dq0, a.dq_ss,
              a.dq_out ? a.dq_out + (int64_t)b * a.dqo_sb + (int64_t)q0 * a.dqo_ss + (int64_t)h * HD : nullptr,
              a.dqo_ss, nullptr, a.dq_initial, tid);
    return;
  }
  const int gk0 = gk0_shard + k_base;
  const float c = kLog2e / sqrtf((float)a.sdim);
  const float bias_scale = kLog2e / c;
  const float kMask2 = mv.mask_min;

  // ---- staging of the K / V tiles through registers, by the consumer waves (which have registers and
  // issue slots to spare), in two register sets A and B: tile T lives in set T & 1 from its request until it is
  // stored to LDS two tiles (four steps) later
  const int srow = (tid & 255) / CH, schunk = tid & (CH - 1), stid = tid & 255;
  const int s_off = srow * TROW + ((schunk ^ swz<HD>(srow)) << 3);
  // a tile is read through a buffer descriptor at its first row (scalar registers) with one 32-bit byte offset per
  // lane: half the address data of 64-bit pointers per lane, and two registers less
  const int64_t sg_base = (int64_t)b * a.kv_sb + (int64_t)h * HD + (int64_t)k_base * a.kv_ss;
  const uint32_t sg_lane = 2u * (uint32_t)(schunk * 8 + srow * (int)a.kv_ss);
  const uint32_t row16b = 2u * SRP * (uint32_t)a.kv_ss;       // one staging pass further
  uint4 Ak0, Ak1, Ak2 = {}, Ak3 = {}, Av0, Av1, Av2 = {}, Av3 = {}, Bk0, Bk1, Bk2 = {}, Bk3 = {}, Bv0, Bv1, Bv2 = {}, Bv3 = {};
  int Aseg = 0, Bseg = 0;
  float Abias = 0.f, Bbias = 0.f;
  // key chunk index and offset inside the chunk of the first key of the next tile to request (tiles are requested
  // in order and never straddle a chunk: key_chunk_size is a multiple of 64): no division per tile
  int ld_c = 0, ld_o = 0;
  if (HAS_SEG) { ld_c = k_base / mv.kc; ld_o = k_base - ld_c * mv.kc; }
  // K half (with the key info) and V half of a tile have their own macros (the forward kernel, which shares this
  // code shape, stores them in different steps); here both are stored in step 2t + 1, see the consumer loop
#define RA_WS_LOAD_K(S, T)                                                                               \
  {                                                                                                     \
    const int t_ = min((T), ntiles - 1);                                                                \
    const __amdgpu_buffer_rsrc_t rk_ = tile_rsrc(a.k + sg_base + (int64_t)t_ * FBN * a.kv_ss);          \
    S##k0 = ld_buf(rk_, sg_lane, 0); S##k1 = ld_buf(rk_, sg_lane, row16b);                              \
    if (SNP == 4) { S##k2 = ld_buf(rk_, sg_lane, 2 * row16b); S##k3 = ld_buf(rk_, sg_lane, 3 * row16b); } \
    if ((HAS_SEG || HAS_BIAS) && stid < FBN) {                                                          \
      const int kj_ = k_base + t_ * FBN + stid;                                                         \
      if (HAS_SEG) {                                                                                    \
        int idx_ = clamp_seg_index(((long long)mv.k_start + ld_c) * mv.kc, mv.kc, mv.seg_len, ld_o + stid); \
        S##seg = mv.seg[(int64_t)b * mv.seg_sb + idx_];                                                 \
      }                                                                                                 \
      /* only the request: using the value here would make this wavefront wait for it right away */     \
      if (HAS_BIAS) S##bias = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + (int64_t)(gk0_shard + kj_) * mv.bias_sk]; \
    }                                                                                                   \
    if (HAS_SEG && (T) < ntiles - 1) { ld_o += FBN; if (ld_o >= mv.kc) { ld_o -= mv.kc; ld_c++; } }      \
  }
#define RA_WS_LOAD_V(S, T)                                                                               \
  {                                                                                                     \
    const int t_ = min((T), ntiles - 1);                                                                \
    const __amdgpu_buffer_rsrc_t rv_ = tile_rsrc(a.v + sg_base + (int64_t)t_ * FBN * a.kv_ss);          \
    S##v0 = ld_buf(rv_, sg_lane, 0); S##v1 = ld_buf(rv_, sg_lane, row16b);                              \
    if (SNP == 4) { S##v2 = ld_buf(rv_, sg_lane, 2 * row16b); S##v3 = ld_buf(rv_, sg_lane, 3 * row16b); } \
  }
#define RA_WS_STORE_K(S, BUF)                                                                            \
  {                                                                                                     \
    uint16_t* dk_ = Ks + (BUF) * WS_TILE + s_off;                                                       \
    *(uint4*)(dk_) = S##k0; *(uint4*)(dk_ + SRP * TROW) = S##k1;                                        \
    if (SNP == 4) { *(uint4*)(dk_ + 2 * SRP * TROW) = S##k2; *(uint4*)(dk_ + 3 * SRP * TROW) = S##k3; } \
    if ((HAS_SEG || HAS_BIAS) && stid < FBN) {                                                          \
      if (HAS_SEG) seg_ks[BUF][stid] = S##seg;                                                          \
      /* clamped when a mask is on (:299,:309) and scaled: the S accumulators start from it.  A bias  \
         at the level of the mask value (a padding mask passed as where(keep, 0, finfo.min)) absorbs    \
         the logit in the reference and would overflow here once scaled: such a key is marked with     \
         -inf; the masked path turns the mark into the mask value itself, the plain path gives the key  \
         the weight exp2(-inf) = 0, which is its weight in every row that sees a real key */           \
      if (HAS_BIAS) {                                                                                   \
        const float bv_ = mv.any_mask ? fminf(S##bias, 0.f) : S##bias;                                  \
        const bool bm_ = bv_ * kLog2e <= kMask2;                                                        \
        bias_ks[BUF][stid] = bm_ ? RA_NEG_INF : bv_ * bias_scale;                                       \
      }                                                                                                 \
    }                                                                                                   \
  }
#define RA_WS_STORE_V(S, BUF)                                                                            \
  {                                                                                                     \
    uint16_t* dv_ = Vs + (BUF) * WS_TILE + s_off;                                                       \
    *(uint4*)(dv_) = S##v0; *(uint4*)(dv_ + SRP * TROW) = S##v1;                                        \
    if (SNP == 4) { *(uint4*)(dv_ + 2 * SRP * TROW) = S##v2; *(uint4*)(dv_ + 3 * SRP * TROW) = S##v3; } \
  }
  // The consumers stage the first tiles; meanwhile the producers request their Q / dO fragments and row statistics.
  // The two roles meet at the first barrier, each inside its own branch.
  if (role == 0) {
    // =========================== producer: S^T, dP^T -> dS^T
    bf16x8 qf[NK], gf[NK];
    float st_den, st_mx, st_delta;
    {
      const int64_t qoff = (int64_t)b * a.q_sb + (int64_t)qrow * a.q_ss + (int64_t)h * HD + hi * 8;
#pragma unroll
      for (int t = 0; t < NK; t++) {
        qf[t] = *(const bf16x8*)(a.q + qoff + t * 16);
        gf[t] = *(const bf16x8*)(a.g + qoff + t * 16);
      }
      const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + qrow;
      st_den = a.den[st]; st_mx = a.mx[st]; st_delta = a.delta[st];
    }
    __syncthreads();
    const int gq = gq0 + pair * 32 + lo;
    const int klim = mv.cbs > 0 ? (int)min((long long)(gq / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;
    const int klim_wave = __builtin_amdgcn_readfirstlane(
        mv.cbs > 0 ? (int)min((long long)((gq0 + pair * 32) / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff);
    int seg_q = 0;
    if (HAS_SEG) {
      int idx = clamp_seg_index(((long long)mv.q_start + qi) * mv.qc, mv.qc, mv.seg_len, qrow % mv.qc);
      seg_q = mv.seg[(int64_t)b * mv.seg_sb + idx];
    }
    const float den = st_den;
    const float m2 = max_to_log2(st_mx, kMask2);
    const float rden = 1.f / den;
    const float lse2 = m2 + __log2f(den);
    const float ndelta = -st_delta;
    int n_off[NK];
#pragma unroll
    for (int t = 0; t < NK; t++) n_off[t] = lo * TROW + (((2 * t + hi) ^ swz<HD>(lo)) << 3);
    uint16_t* const dw = &Ds[pair][0][lo * WS_PSTR + hi * 4];
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

#define RA_WS_INIT(SN, DPN, BUF, BLK)                                                                   \
  _Pragma("unroll") for (int g = 0; g < 4; g++) {                                                       \
    f32x4 b4_ = {0.f, 0.f, 0.f, 0.f};                                                                   \
    if (HAS_BIAS) b4_ = *(const f32x4*)&bias_ks[BUF][(BLK) * 32 + g * 8 + hi * 4];                      \
    _Pragma("unroll") for (int e = 0; e < 4; e++) { SN[g * 4 + e] = b4_[e]; DPN[g * 4 + e] = ndelta; }  \
  }
#define RA_WS_AREAD(G, KA, VA, BUF, BLK)                                                                \
  _Pragma("unroll") for (int i = 0; i < KPG; i++) {                                                       \
    const uint16_t* p_ = Ks + (BUF) * WS_TILE + n_off[KPG * (G) + i];                                     \
    KA[i] = *(const bf16x8*)(p_ + (BLK) * 32 * TROW);                                                   \
    VA[i] = *(const bf16x8*)(p_ + (BLK) * 32 * TROW + 3 * WS_TILE);                                     \
  }
#define RA_WS_AMFMA(G, KA, VA, SN, DPN)                                                                 \
  _Pragma("unroll") for (int i = 0; i < KPG; i++) {                                                       \
    SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(KA[i], qf[KPG * (G) + i], SN, 0, 0, 0);   /* S^T = K Q^T */ \
    DPN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(VA[i], gf[KPG * (G) + i], DPN, 0, 0, 0); /* dP^T = V dO^T */ \
  }
    // eight keys (registers 4G .. 4G+3 of both halves) of dS^T
#define RA_WS_VECTOR(G, SC, DPC, BUF, BLK, PB, MASKED)                                                  \
  {                                                                                                     \
    bf16x4 d4;                                                                                          \
    _Pragma("unroll") for (int e = 0; e < 4; e++) {                                                     \
      float p;                                                                                          \
      if (!(MASKED)) {                                                                                  \
        p = fast_exp2(fmaf(SC[(G) * 4 + e], c, -lse2));                                                 \
      } else {                                                                                          \
        const int kr_ = (BLK) * 32 + (G) * 8 + hi * 4 + e;                                              \
        float x = SC[(G) * 4 + e] * c;                                                                  \
        bool masked = (gk_tile + kr_ >= klim);                                                          \
        /* another document, or a key whose bias is at the level of the mask value (marked -inf) */     \
        bool sne_ = false;                                                                              \
        if (HAS_SEG) sne_ = seg_ks[BUF][kr_] != seg_q;                                                  \
        if (HAS_BIAS) sne_ = sne_ || SC[(G) * 4 + e] == RA_NEG_INF;                                     \
        masked = masked || sne_;                                                                        \
        if (HAS_KEEP == 2 && (HAS_SEG || HAS_BIAS)) {                                                   \
          /* as below, with such pairs: they count as masked once more */                               \
          x = (((kw_cur >> ((BLK) * 32 + (G) * 8 + e)) & 1) && !sne_) ? x : kMask2;                     \
          x = (((kw_some >> ((BLK) * 32 + (G) * 8 + e)) & 1) &&                                         \
               (((kw_k >> ((BLK) * 32 + (G) * 8 + e)) & 1) || !sne_)) ? x : RA_NEG_INF;                 \
        } else if (HAS_KEEP == 2) {                                                                     \
          /* dropout adds mask_min (:321).  kw_cur: pairs kept and causally allowed; kw_some: at least  \
             one of the two, so a clear bit there is mask_min added twice = -inf */                     \
          x = ((kw_cur >> ((BLK) * 32 + (G) * 8 + e)) & 1) ? x : kMask2;                                \
          x = ((kw_some >> ((BLK) * 32 + (G) * 8 + e)) & 1) ? x : RA_NEG_INF;                           \
        } else {                                                                                        \
          if (HAS_KEEP) masked = masked || !((kw_cur >> ((BLK) * 32 + (G) * 8 + e)) & 1);               \
          x = masked ? kMask2 : x;                                                                      \
        }                                                                                               \
        p = fast_exp2(x - m2) * rden;                                                    /* :226 */     \
      }                                                                                                 \
      d4[e] = (__bf16)(p * DPC[(G) * 4 + e]);                                            /* :229 */     \
    }                                                                                                   \
    *(bf16x4*)(dw + (PB) * WS_PD + (G) * 8) = d4;                                                       \
  }
    // one step: vector work of block BLK of buffer BUF (accumulators SC, DPC) in four groups of eight
    // keys, each next to a quarter of the products of block NBLK of buffer NBUF (into SN, DPN).  The
    // K / V operands of a quarter are requested from LDS three quarters ahead - the last three of a step
    // request the first three quarters of the following step's block NNBLK of buffer NNBUF - which
    // covers the LDS latency under load.
#define RA_WS_PRODUCE(SC, DPC, SN, DPN, BUF, BLK, NBUF, NBLK, NNBUF, NNBLK, PB, MASKED)                 \
  {                                                                                                     \
    RA_WS_INIT(SN, DPN, NBUF, NBLK);                                                                    \
    _Pragma("unroll") for (int g = 0; g < 4; g++) {                                                     \
      if (g == 0) { RA_WS_AREAD(3, ka[3], va[3], NBUF, NBLK); }                                         \
      else { RA_WS_AREAD(g - 1, ka[g - 1], va[g - 1], NNBUF, NNBLK); }                                  \
      RA_WS_AMFMA(g, ka[g], va[g], SN, DPN);                                                            \
      RA_WS_VECTOR(g, SC, DPC, BUF, BLK, PB, MASKED);                                                   \
      /* issue order: the LDS reads, then each product followed by a share of the vector work */        \
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * KPG, 0);                                          \
      _Pragma("unroll") for (int i_ = 0; i_ < 2 * KPG; i_++) {                                                \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                              \
        __builtin_amdgcn_sched_group_barrier(0x002, WS_DQ_VALU_PER_MFMA, 0);                            \
      }                                                                                                 \
      __builtin_amdgcn_sched_barrier(0);                                                                \
    }                                                                                                   \
  }

    f32x16 s_a, dp_a, s_b, dp_b;
    bf16x8 ka[4][KPG], va[4][KPG];
    RA_WS_INIT(s_a, dp_a, 0, 0);
#pragma unroll
    for (int g = 0; g < 4; g++) {
      RA_WS_AREAD(g, ka[0], va[0], 0, 0);
      RA_WS_AMFMA(g, ka[0], va[0], s_a, dp_a);
    }
#pragma unroll
    for (int g = 0; g < 3; g++) RA_WS_AREAD(g, ka[g], va[g], 0, 1);

    // Under a causal mask the tiles that need no masking come first: one loop for them, one for the rest
    // (which also takes every tile when segment ids or a bias are present).
    // Which key tiles need no masking at all: below the causal limit of every row, keys all of this wave's
    // single segment id, packed keep summary "all kept".  They form (at most) one run [t_a, t_b) in the
    // cases that matter - document interiors, the part of a causal row left of the diagonal - and get a
    // loop of their own; the tiles before and after take the masked loop.
    const int t_causal = (int)max(0LL, min((long long)ntiles, ((long long)klim_wave - gk0) / FBN));
    const uint64_t* kw_ptr = nullptr;
    const uint8_t* ks_ptr = nullptr;
    uint64_t kw_cur = 0, kw_nxt = 0, kw_some = 0, kw_k = 0;     // kw_k: the kept bits before the causal limit is folded in
    (void)kw_some; (void)kw_k;
    if (HAS_KEEP) {
      ks_ptr = mv.ksum + (int64_t)b * mv.ksum_sb + (int64_t)h * mv.ksum_sh +
               (int64_t)((mv.keep_q0 + q0 + pair * 32) / 64) * (mv.keep_K / 64) + (gk0 - mv.keep_k0) / 64;
      kw_ptr = mv.kbits_k + (int64_t)b * mv.kpack_sb + (int64_t)h * mv.kpack_sh +
               (int64_t)((gk0 - mv.keep_k0) / 64) * mv.keep_Q +
               mv.keep_q0 + qrow;
    }
    const int2* smm_ptr = nullptr;
    bool sq_uniform = false;
    int sq_id = 0;
    if (HAS_SEG && mv.seg_mm) {
      smm_ptr = (const int2*)(mv.seg_mm + (int64_t)(mv.seg_sb ? b : 0) * mv.seg_tiles * 2);
      const int2 qmm = smm_ptr[min((gq0 + pair * 32) / RA_SEG_TILE, mv.seg_tiles - 1)];
      sq_uniform = qmm.x == qmm.y;
      sq_id = qmm.x;
    }
    int t_a = ntiles, t_b = ntiles;
    for (int base = 0; base < ntiles; base += 64) {
      const int tt = base + lane;
      bool ok = tt < t_causal;
      if (HAS_SEG && ok) {
        ok = sq_uniform;
        if (ok) {
          const int2 kmm = smm_ptr[min(gk0 / RA_SEG_TILE + tt, mv.seg_tiles - 1)];
          ok = kmm.x == sq_id && kmm.y == sq_id;
        }
      }
      if (HAS_KEEP && ok) ok = ks_ptr[tt] == 2;
      const unsigned long long m = __builtin_amdgcn_ballot_w64(ok);
      unsigned long long stop;      // tiles of this group of 64 that end the run
      if (t_a == ntiles) {
        if (!m) continue;
        const int f = __builtin_ctzll(m);
        t_a = base + f;
        stop = ~m & (~0ULL << f);
      } else {
        stop = ~m;
      }
      if (stop) { t_b = min(ntiles, base + (int)__builtin_ctzll(stop)); break; }
    }
    t_a = __builtin_amdgcn_readfirstlane(t_a);
    t_b = __builtin_amdgcn_readfirstlane(t_a == ntiles ? ntiles : t_b);
    if (HAS_KEEP) kw_nxt = kw_ptr[(int64_t)min(t_a == 0 ? t_b : 0, ntiles - 1) * mv.keep_Q];
    int cur = 0;
#define RA_WS_TILE(MASKED)                                                                              \
  {                                                                                                     \
    const int nxt = cur == 2 ? 0 : cur + 1;                                                             \
    const int gk_tile = gk0 + t * FBN;                                                                  \
    (void)gk_tile;                                                                                      \
    if (HAS_KEEP && (MASKED)) {        /* this tile's word; request the next tile's */                  \
      kw_cur = kw_nxt >> (4 * hi);                                                                      \
      kw_nxt = kw_ptr[(int64_t)min(t + 1 == t_a ? t_b : t + 1, ntiles - 1) * mv.keep_Q];                \
      if (HAS_KEEP == 2) {             /* fold this row's causal limit into the words */                \
        const int nall_ = max(0, min(64, klim - gk_tile));                                              \
        const uint64_t cw_ = (nall_ >= 64 ? ~0ULL : ((1ULL << nall_) - 1ULL)) >> (4 * hi);              \
        kw_k = kw_cur;                                                                                  \
        kw_some = kw_cur | cw_;                                                                         \
        kw_cur &= cw_;                                                                                  \
      }                                                                                                 \
    }                                                                                                   \
    /* step 2t: vector work of block 0 of tile t, products of block 1 */                                \
    RA_WS_PRODUCE(s_a, dp_a, s_b, dp_b, cur, 0, cur, 1, nxt, 0, 0, MASKED);                             \
    __syncthreads();                                                                                    \
    /* step 2t + 1: vector work of block 1, products of block 0 of tile t + 1 (the last tile computes  \
       a block that is never used) */                                                                   \
    RA_WS_PRODUCE(s_b, dp_b, s_a, dp_a, cur, 1, nxt, 0, nxt, 1, 1, MASKED);                             \
    __syncthreads();                                                                                    \
    cur = nxt;                                                                                          \
  }
    int t = 0;
      for (; t < t_a; t++) RA_WS_TILE(true);
      for (; t < t_b; t++) RA_WS_TILE(false);
      for (; t < ntiles; t++) RA_WS_TILE(true);
#undef RA_WS_TILE
    __syncthreads();      // step 2 ntiles: the consumer's last block
#undef RA_WS_INIT
#undef RA_WS_AREAD
#undef RA_WS_AMFMA
#undef RA_WS_VECTOR
#undef RA_WS_PRODUCE
  } else {
    // =========================== consumer: dQ^T += K^T dS^T
    RA_WS_LOAD_K(A, 0); RA_WS_LOAD_V(A, 0);
    RA_WS_LOAD_K(B, 1); RA_WS_LOAD_V(B, 1);
    RA_WS_STORE_K(A, 0); RA_WS_STORE_V(A, 0);
    RA_WS_LOAD_K(A, 2); RA_WS_LOAD_V(A, 2);
    RA_WS_STORE_K(B, 1); RA_WS_STORE_V(B, 1);
    RA_WS_LOAD_K(B, 3); RA_WS_LOAD_V(B, 3);
    __syncthreads();
    f32x16 acc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
    int t_off[NDB][2];
    {
      const int i = lane & 15, rr = (i >> 2) + 8 * hi, c0 = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), half = lane & 1;
#pragma unroll
      for (int db = 0; db < NDB; db++) {
        t_off[db][0] = rr * TROW + (((4 * db + c0) ^ swz<HD>(rr)) << 3) + half * 4;
        t_off[db][1] = (rr + 4) * TROW + (((4 * db + c0) ^ swz<HD>(rr + 4)) << 3) + half * 4;
      }
    }
    const uint16_t* const dr = &Ds[pair][0][lo * WS_PSTR + hi * 8];   // B operand: query column lo, 8 keys

    // keys 16 K .. 16 K + 15 of block BLK of buffer BUF, transposed
#define RA_WS_CREAD(K, F, BUF, BLK)                                                                     \
  {                                                                                                     \
    const uint16_t* tp_ = Ks + (BUF) * WS_TILE + ((BLK) * 32 + (K) * 16) * TROW;                        \
    _Pragma("unroll") for (int db = 0; db < NDB; db++) {                                                  \
      const s16x4 x0_ = lds_read_tr(tp_ + t_off[db][0]);                                                \
      const s16x4 x1_ = lds_read_tr(tp_ + t_off[db][1]);                                                \
      F[db] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(x0_, x1_, 0, 1, 2, 3, 4, 5, 6, 7));    \
    }                                                                                                   \
  }
#define RA_WS_CMFMA(F, BOP)                                                                             \
  _Pragma("unroll") for (int db = 0; db < NDB; db++)                                                      \
    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[db], BOP, acc[db], 0, 0, 0);
    // fa holds the first 16 keys of the block on entry and, on exit, those of block NBLK of buffer NBUF
#define RA_WS_CONSUME(BUF, BLK, PB, NBUF, NBLK)                                                         \
  {                                                                                                     \
    const bf16x8 d0_ = *(const bf16x8*)(dr + (PB) * WS_PD);                                             \
    const bf16x8 d1_ = *(const bf16x8*)(dr + (PB) * WS_PD + 16);                                        \
    RA_WS_CREAD(1, fb, BUF, BLK);                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(fa, d0_);                                                                               \
    RA_WS_CREAD(0, fa, NBUF, NBLK);                                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(fb, d1_);                                                                               \
  }
    bf16x8 fa[NDB], fb[NDB];
    int cur = 0;
    RA_WS_CREAD(0, fa, 0, 0);
    __syncthreads();      // step 0
    // tile T + 2 (in register set T & 1) goes to the buffer that held tile T - 1, K and V both in step 2T + 1: in
    // step 2T + 2 the producer already requests K and V fragments of block 0 of tile T + 2 from that buffer, so
    // nothing may still be written to it then.  Tile T + 4 is requested into the same set.
#define RA_WS_CTILE(S, T)                                                                               \
  {                                                                                                     \
    const int prv = cur == 0 ? 2 : cur - 1, nxt = cur == 2 ? 0 : cur + 1;                               \
    RA_WS_STORE_K(S, prv);                                                                              \
    RA_WS_STORE_V(S, prv);                                                                              \
    RA_WS_LOAD_K(S, (T) + 4);                                                                           \
    RA_WS_LOAD_V(S, (T) + 4);                                                                           \
    RA_WS_CONSUME(cur, 0, 0, cur, 1);                                                                   \
    __syncthreads();                                                                                    \
    RA_WS_CONSUME(cur, 1, 1, nxt, 0);                                                                   \
    __syncthreads();                                                                                    \
    cur = nxt;                                                                                          \
  }
    int t = 0;
    for (; t + 2 <= ntiles; t += 2) {
      RA_WS_CTILE(A, t);
      RA_WS_CTILE(B, t + 1);
    }
    if (t < ntiles) RA_WS_CTILE(A, t);
#undef RA_WS_CTILE
#undef RA_WS_CREAD
#undef RA_WS_CMFMA
#undef RA_WS_CONSUME

    // dq += acc / sqrt(D)   (:230)
    const float rscale = 1.f / sqrtf((float)a.sdim);
    float* dqp = a.dq + (int64_t)b * a.dq_sb + (int64_t)qrow * a.dq_ss + (int64_t)h * HD + hi * 4;
    uint16_t* dqo = a.dq_out + (int64_t)b * a.dqo_sb + (int64_t)qrow * a.dqo_ss + (int64_t)h * HD + hi * 4;
    // all the old values are requested before the first store: a load issued after a store is not waited for until
    // that store has completed too (one in-order counter), and sixteen such round trips in a row cost tens of us
    f32x4 old[NDB][4];
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        old[db][g] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (!a.dq_initial) old[db][g] = *(const f32x4*)(dqp + db * 32 + g * 8);
      }
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        f32x4 t = old[db][g];
#pragma unroll
        for (int e = 0; e < 4; e++) t[e] += acc[db][g * 4 + e] * rscale;
        if (a.dq_out) store_bf16x4(dqo + db * 32 + g * 8, t);      // last call for these rows: the sum as bf16 (:89)
        else *(f32x4*)(dqp + db * 32 + g * 8) = t;
      }
  }
#undef RA_WS_LOAD_K
#undef RA_WS_LOAD_V
#undef RA_WS_STORE_K
#undef RA_WS_STORE_V
}

// ------------------------------------------------------------------ forward, wave-specialised
// Same structure as the dQ kernel above: 128 query rows per workgroup, pair i = (wave i, wave i + 4) owns
// rows 32 i .. 32 i + 31.  The producer runs S^T = K Q^T and the online softmax (running max and sum are
// per-lane scalars: a lane owns a query column) and leaves P^T, rounded to bf16, in LDS together with the
// factor by which the output accumulator has to shrink when the reference max moved; the consumer runs
// O^T += V^T P^T one block of 32 keys behind.
template <int HD, bool HAS_SEG, bool HAS_BIAS, int HAS_KEEP = 0>   // HD: head size, 64 or 128; HAS_KEEP: 0 no keep mask, 1 where(keep, w, min), 2 dropout
__global__ __launch_bounds__(512) void attn_fwd_ws_kernel(FwdArgs a) {
  // head size: elements per LDS tile row, a 64-row tile, contraction steps of 16 (per quarter of a block's products),
  // output blocks of 32, 16-byte chunks per row, rows per staging pass of 256 threads, passes per tile
  constexpr int TROW = HD, WS_TILE = 64 * HD, NK = HD / 16, KPG = HD / 64, NDB = HD / 32, CH = HD / 8;
  constexpr int SRP = 256 / CH, SNP = 64 / SRP;
  // K tiles then V tiles in one array: a V address is the K address plus a constant (an immediate offset)
  __shared__ __attribute__((aligned(16))) uint16_t KVs[6 * WS_TILE];
  uint16_t* const Ks = KVs;
  uint16_t* const Vs = KVs + 3 * WS_TILE;
  __shared__ __attribute__((aligned(16))) uint16_t Ds[4][2][WS_PD];        // [pair][buffer] P^T as [q][key]
  __shared__ float al[4][2][32];     // [pair][buffer][query]: factor the consumer applies to O before adding the block
  __shared__ float fixs[4][32];      // [pair][query]: final factor (lazy reference max -> exact max)
  __shared__ float dens[4][32];      // [pair][query]: final denominator, for the step that writes out
  __shared__ int seg_ks[3][FBN];
  __shared__ float bias_ks[3][FBN];
  __shared__ int bias_any[3];        // [buffer]: some key of the tile carries a bias at the level of the mask value

  MaskView mv = a.mv;
  mv.resolve();
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int role = __builtin_amdgcn_readfirstlane(wave >> 2), pair = wave & 3;
  const int nqt = a.Sq / FBM;
  // XCD x takes the contiguous range x of (batch, head, query tile) triples: the workgroups resident on
  // one XCD then stream the same K / V tiles of one head through that XCD's L2 at the same time
  const int per_xcd = (a.B * a.H * nqt + 7) >> 3;
  int wg = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (wg >= a.B * a.H * nqt) return;
  int qt = nqt - 1 - (wg % nqt);           // latest query tiles (most keys under causal) first
  wg /= nqt;
  const int h = wg % a.H, b = wg / a.H;
  if (a.ring.n && !ring_bind(a, mv, qt)) return;
  const int q0 = qt * FBM;
  const int qrow = q0 + pair * 32 + lo;

  const int qi = q0 / mv.qc;
  int kend = mv.run_prefix_keys(qi, a.Skv);
  const int gq0 = (int)mv.global_q(q0);
  const int gk0_shard = (int)mv.global_k(0);
  if (mv.cbs > 0 && mv.skip_tiles) {
    long long lim = ((long long)(gq0 + FBM - 1) / mv.cbs + 1) * mv.cbs;
    long long n = lim - gk0_shard;
    if (n < kend) kend = n > 0 ? (int)n : 0;
  }
  int ntiles = (kend + FBN - 1) / FBN;
  int k_base = 0;
  if (HAS_SEG && mv.seg_mm && mv.skip_tiles && ntiles > 0) {
    __shared__ int hull2[2];
    int t_first, t_last;
    seg_hull_of_rows(mv, b, gq0, FBM, gk0_shard / RA_SEG_TILE, ntiles, hull2, tid, 512, t_first, t_last);
    k_base = t_first * FBN;
    ntiles = t_last - t_first;
  }
  if (HAS_KEEP && mv.skip_tiles && ntiles > 0) {
    __shared__ int khull2[2];
    int t_first, t_last;
    keep_ktile_hull(mv, b, h, (mv.keep_q0 + q0) / 64, FBM / 64, (gk0_shard + k_base - mv.keep_k0) / 64, ntiles, khull2, tid, 512,
                    t_first, t_last);
    k_base += t_first * FBN;
    ntiles = t_last - t_first;
  }
  if (ntiles == 0) {           // no key tile runs for these rows: the carry stays as it is
    if (a.carry_is_initial || a.out) {
      const int64_t st0 = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + q0;
      float* const np0 = a.num ? a.num + (int64_t)b * a.num_sb + (int64_t)q0 * a.num_ss + (int64_t)h * HD : nullptr;
      pass_rows<HD>(np0, np0, a.num_ss,
                a.out ? a.out + (int64_t)b * a.out_sb + (int64_t)q0 * a.out_ss + (int64_t)h * HD : nullptr, a.out_ss,
                a.out ? a.den + st0 : nullptr, a.carry_is_initial, tid,
                (a.out && a.out32) ? a.out32 + (int64_t)b * a.out_sb + (int64_t)q0 * a.out_ss + (int64_t)h * HD : nullptr);
      if (a.carry_is_initial && tid < FBM) { a.den[st0 + tid] = 0.f; a.mx[st0 + tid] = RA_NEG_INF; }
    }
    return;
  }
  const int gk0 = gk0_shard + k_base;
  const float c = kLog2e / sqrtf((float)a.sdim);
  const float bias_scale = kLog2e / c;
  const float kMask2 = mv.mask_min;

  // ---- staging of the K / V tiles through registers, by the consumer waves (which have registers and
  // issue slots to spare), in two register sets A and B: tile T lives in set T & 1 from its request until it is
  // stored to LDS two tiles (four steps, about 3.5 us) later.  With one set - a tile in flight for two steps - the
  // LDS stores waited for L2 misses often enough to cost the forward kernel 16 %.
  const int srow = (tid & 255) / CH, schunk = tid & (CH - 1), stid = tid & 255;
  const int s_off = srow * TROW + ((schunk ^ swz<HD>(srow)) << 3);
  // a tile is read through a buffer descriptor at its first row (scalar registers) with one 32-bit byte offset per
  // lane: half the address data of 64-bit pointers per lane, and two registers less
  const int64_t sg_base = (int64_t)b * a.kv_sb + (int64_t)h * HD + (int64_t)k_base * a.kv_ss;
  const uint32_t sg_lane = 2u * (uint32_t)(schunk * 8 + srow * (int)a.kv_ss);
  const uint32_t row16b = 2u * SRP * (uint32_t)a.kv_ss;       // one staging pass further
  uint4 Ak0, Ak1, Ak2 = {}, Ak3 = {}, Av0, Av1, Av2 = {}, Av3 = {}, Bk0, Bk1, Bk2 = {}, Bk3 = {}, Bv0, Bv1, Bv2 = {}, Bv3 = {};
  int Aseg = 0, Bseg = 0;
  float Abias = 0.f, Bbias = 0.f;
  // key chunk index and offset inside the chunk of the first key of the next tile to request (tiles are requested
  // in order and never straddle a chunk: key_chunk_size is a multiple of 64): no division per tile
  int ld_c = 0, ld_o = 0;
  if (HAS_SEG) { ld_c = k_base / mv.kc; ld_o = k_base - ld_c * mv.kc; }
  // K half (with the key info) and V half of a tile are staged separately so that the requests and the
  // LDS writes of a tile spread over two steps
#define RA_WS_LOAD_K(S, T)                                                                               \
  {                                                                                                     \
    const int t_ = min((T), ntiles - 1);                                                                \
    const __amdgpu_buffer_rsrc_t rk_ = tile_rsrc(a.k + sg_base + (int64_t)t_ * FBN * a.kv_ss);          \
    S##k0 = ld_buf(rk_, sg_lane, 0); S##k1 = ld_buf(rk_, sg_lane, row16b);                              \
    if (SNP == 4) { S##k2 = ld_buf(rk_, sg_lane, 2 * row16b); S##k3 = ld_buf(rk_, sg_lane, 3 * row16b); } \
    if ((HAS_SEG || HAS_BIAS) && stid < FBN) {                                                          \
      const int kj_ = k_base + t_ * FBN + stid;                                                         \
      if (HAS_SEG) {                                                                                    \
        int idx_ = clamp_seg_index(((long long)mv.k_start + ld_c) * mv.kc, mv.kc, mv.seg_len, ld_o + stid); \
        S##seg = mv.seg[(int64_t)b * mv.seg_sb + idx_];                                                 \
      }                                                                                                 \
      /* only the request: using the value here would make this wavefront wait for it right away */     \
      if (HAS_BIAS) S##bias = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + (int64_t)(gk0_shard + kj_) * mv.bias_sk]; \
    }                                                                                                   \
    if (HAS_SEG && (T) < ntiles - 1) { ld_o += FBN; if (ld_o >= mv.kc) { ld_o -= mv.kc; ld_c++; } }      \
  }
#define RA_WS_LOAD_V(S, T)                                                                               \
  {                                                                                                     \
    const int t_ = min((T), ntiles - 1);                                                                \
    const __amdgpu_buffer_rsrc_t rv_ = tile_rsrc(a.v + sg_base + (int64_t)t_ * FBN * a.kv_ss);          \
    S##v0 = ld_buf(rv_, sg_lane, 0); S##v1 = ld_buf(rv_, sg_lane, row16b);                              \
    if (SNP == 4) { S##v2 = ld_buf(rv_, sg_lane, 2 * row16b); S##v3 = ld_buf(rv_, sg_lane, 3 * row16b); } \
  }
#define RA_WS_STORE_K(S, BUF)                                                                            \
  {                                                                                                     \
    uint16_t* dk_ = Ks + (BUF) * WS_TILE + s_off;                                                       \
    *(uint4*)(dk_) = S##k0; *(uint4*)(dk_ + SRP * TROW) = S##k1;                                        \
    if (SNP == 4) { *(uint4*)(dk_ + 2 * SRP * TROW) = S##k2; *(uint4*)(dk_ + 3 * SRP * TROW) = S##k3; } \
    if ((HAS_SEG || HAS_BIAS) && stid < FBN) {                                                          \
      if (HAS_SEG) seg_ks[BUF][stid] = S##seg;                                                          \
      /* clamped when a mask is on (:299,:309) and scaled: the S accumulators start from it.  A bias  \
         at the level of the mask value (a padding mask passed as where(keep, 0, finfo.min)) absorbs    \
         the logit in the reference and would overflow here once scaled: such a key is marked with     \
         -inf and its tile takes the masked path, where the mark becomes the mask value itself */      \
      if (HAS_BIAS) {                                                                                   \
        const float bv_ = mv.any_mask ? fminf(S##bias, 0.f) : S##bias;                                  \
        const bool bm_ = bv_ * kLog2e <= kMask2;                                                        \
        bias_ks[BUF][stid] = bm_ ? RA_NEG_INF : bv_ * bias_scale;                                       \
        const unsigned long long any_ = __builtin_amdgcn_ballot_w64(bm_);                               \
        if (stid == 0) bias_any[BUF] = any_ != 0ULL;                                                    \
      }                                                                                                 \
    }                                                                                                   \
  }
#define RA_WS_STORE_V(S, BUF)                                                                            \
  {                                                                                                     \
    uint16_t* dv_ = Vs + (BUF) * WS_TILE + s_off;                                                       \
    *(uint4*)(dv_) = S##v0; *(uint4*)(dv_ + SRP * TROW) = S##v1;                                        \
    if (SNP == 4) { *(uint4*)(dv_ + 2 * SRP * TROW) = S##v2; *(uint4*)(dv_ + 3 * SRP * TROW) = S##v3; } \
  }
  // The consumers stage the first tiles; meanwhile the producers request their Q fragments and the carry's statistics.
  // The two roles meet at the first barrier, each inside its own branch.
  if (role == 0) {
    // =========================== producer: S^T -> online softmax -> P^T
    bf16x8 qf[NK];
    float st_mx = 0.f, st_den = 0.f;
    {
      const int64_t qoff = (int64_t)b * a.q_sb + (int64_t)qrow * a.q_ss + (int64_t)h * HD + hi * 8;
#pragma unroll
      for (int t = 0; t < NK; t++) qf[t] = *(const bf16x8*)(a.q + qoff + t * 16);
      if (!a.carry_is_initial) {
        const int64_t st0 = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + qrow;
        st_mx = a.mx[st0]; st_den = a.den[st0];
      }
    }
    __syncthreads();
    const int gq = gq0 + pair * 32 + lo;
    const int klim = mv.cbs > 0 ? (int)min((long long)(gq / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff;
    const int klim_wave = __builtin_amdgcn_readfirstlane(
        mv.cbs > 0 ? (int)min((long long)((gq0 + pair * 32) / mv.cbs + 1) * mv.cbs, 0x7fffffffLL) : 0x7fffffff);
    int seg_q = 0;
    if (HAS_SEG) {
      int idx = clamp_seg_index(((long long)mv.q_start + qi) * mv.qc, mv.qc, mv.seg_len, qrow % mv.qc);
      seg_q = mv.seg[(int64_t)b * mv.seg_sb + idx];
    }
    const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + qrow;
    // running max (log2 domain; m2 is the lazy reference the probabilities are taken against, m_true the
    // exact one) and this half-row's share of the running sum
    float m2 = RA_NEG_INF, l = 0.f;
    if (!a.carry_is_initial) {
      m2 = max_to_log2(st_mx, kMask2);
      l = hi == 0 ? st_den : 0.f;
    }
    float m_true = m2, ps = 0.f;
    constexpr float kLazy = 16.f;
    int n_off[NK];
#pragma unroll
    for (int t = 0; t < NK; t++) n_off[t] = lo * TROW + (((2 * t + hi) ^ swz<HD>(lo)) << 3);
    uint16_t* const dw = &Ds[pair][0][lo * WS_PSTR + hi * 4];
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

#define RA_WS_INIT(SN, BUF, BLK)                                                                        \
  _Pragma("unroll") for (int g = 0; g < 4; g++) {                                                       \
    f32x4 b4_ = {0.f, 0.f, 0.f, 0.f};                                                                   \
    if (HAS_BIAS) b4_ = *(const f32x4*)&bias_ks[BUF][(BLK) * 32 + g * 8 + hi * 4];                      \
    _Pragma("unroll") for (int e = 0; e < 4; e++) SN[g * 4 + e] = b4_[e];                               \
  }
#define RA_WS_AREAD(G, KA, BUF, BLK)                                                                    \
  _Pragma("unroll") for (int i = 0; i < KPG; i++)                                                         \
    KA[i] = *(const bf16x8*)(Ks + (BUF) * WS_TILE + (BLK) * 32 * TROW + n_off[KPG * (G) + i]);
#define RA_WS_AMFMA(G, KA, SN)                                                                          \
  _Pragma("unroll") for (int i = 0; i < KPG; i++)                                                         \
    SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(KA[i], qf[KPG * (G) + i], SN, 0, 0, 0);   /* S^T = K Q^T (:134) */
    // The block's 32 keys x this lane's query: the running max first (group 0), then eight keys
    // (registers 4G .. 4G+3 of both halves) of P^T per group.  (:138-144)
#define RA_WS_ROWMAX(SC, BUF, BLK, PB, MASKED)                                                          \
  {                                                                                                     \
    float alpha_ = 1.f;                                                                                 \
    if (!(MASKED)) {                                                                                    \
      float mxv_ = SC[0];                                                                               \
      _Pragma("unroll") for (int r = 1; r < 16; r++) mxv_ = fmaxf(mxv_, SC[r]);                         \
      mxv_ = max_xor32(mxv_);                                                                           \
      m_true = fmaxf(m_true, mxv_ * c);                                                                 \
      if (__builtin_amdgcn_ballot_w64(m_true - m2 > kLazy) != 0) {   /* rescale only on a large jump */ \
        alpha_ = fast_exp2(m2 - m_true);                                                                \
        m2 = m_true;                                                                                    \
        l *= alpha_;                                                                                    \
      }                                                                                                 \
    } else {                                                                                            \
      float mxv_ = RA_NEG_INF;                                                                          \
      _Pragma("unroll") for (int r = 0; r < 16; r++) {                                                  \
        const int kr_ = (BLK) * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);                                   \
        float x_ = SC[r] * c;                                                                           \
        bool masked_ = (gk_tile + kr_ >= klim);                                                         \
        /* another document, or a key whose bias is at the level of the mask value (marked -inf) */     \
        bool sne_ = false;                                                                              \
        if (HAS_SEG) sne_ = seg_ks[BUF][kr_] != seg_q;                                                  \
        if (HAS_BIAS) sne_ = sne_ || SC[r] == RA_NEG_INF;                                               \
        masked_ = masked_ || sne_;                                                                      \
        if (HAS_KEEP == 2 && (HAS_SEG || HAS_BIAS)) {                                                   \
          /* as below, with such pairs: they count as masked once more */                               \
          x_ = (((kw_cur >> ((BLK) * 32 + (r >> 2) * 8 + (r & 3))) & 1) && !sne_) ? x_ : kMask2;        \
          x_ = (((kw_some >> ((BLK) * 32 + (r >> 2) * 8 + (r & 3))) & 1) &&                             \
                (((kw_k >> ((BLK) * 32 + (r >> 2) * 8 + (r & 3))) & 1) || !sne_)) ? x_ : RA_NEG_INF;    \
        } else if (HAS_KEEP == 2) {                                                                     \
          /* dropout adds mask_min (:321).  kw_cur: pairs kept and causally allowed; kw_some: at least  \
             one of the two, so a clear bit there is mask_min added twice = -inf */                     \
          x_ = ((kw_cur >> ((BLK) * 32 + (r >> 2) * 8 + (r & 3))) & 1) ? x_ : kMask2;                   \
          x_ = ((kw_some >> ((BLK) * 32 + (r >> 2) * 8 + (r & 3))) & 1) ? x_ : RA_NEG_INF;              \
        } else {                                                                                        \
          if (HAS_KEEP) masked_ = masked_ || !((kw_cur >> ((BLK) * 32 + (r >> 2) * 8 + (r & 3))) & 1);  \
          x_ = masked_ ? kMask2 : x_;                                                                   \
        }                                                                                               \
        SC[r] = x_;                                                                                     \
        mxv_ = fmaxf(mxv_, x_);                                                                         \
      }                                                                                                 \
      mxv_ = max_xor32(mxv_);                                                                           \
      m_true = fmaxf(m_true, mxv_);                                                                     \
      const float m_new_ = fmaxf(m2, mxv_);                                                             \
      /* under dropout every pair so far may be -inf: nothing accumulated yet, nothing to rescale */    \
      alpha_ = (HAS_KEEP == 2 && m_new_ == RA_NEG_INF) ? 1.f : fast_exp2(m2 - m_new_);                       \
      m2 = m_new_;                                                                                      \
      l *= alpha_;                                                                                      \
    }                                                                                                   \
    if (hi == 0) al[pair][PB][lo] = alpha_;                                                             \
  }
#define RA_WS_VECTOR(G, SC, BUF, BLK, PB, MASKED)                                                       \
  {                                                                                                     \
    if ((G) == 0) RA_WS_ROWMAX(SC, BUF, BLK, PB, MASKED);                                               \
    bf16x4 d4;                                                                                          \
    const float mref_ = (HAS_KEEP == 2 && (MASKED) && m2 == RA_NEG_INF) ? 0.f : m2;   /* exp2(-inf - 0) = 0 */ \
    _Pragma("unroll") for (int e = 0; e < 4; e++) {                                                     \
      const float p = (MASKED) ? fast_exp2(SC[(G) * 4 + e] - mref_) : fast_exp2(fmaf(SC[(G) * 4 + e], c, -m2)); \
      ps += p;                                                                                          \
      d4[e] = (__bf16)p;                                                                                \
    }                                                                                                   \
    *(bf16x4*)(dw + (PB) * WS_PD + (G) * 8) = d4;                                                       \
    if ((G) == 3) { l += ps; ps = 0.f; }                                                                \
  }
    // one step: vector work of block BLK of buffer BUF (accumulators SC, DPC) in four groups of eight
    // keys, each next to a quarter of the products of block NBLK of buffer NBUF (into SN, DPN).  The
    // K / V operands of a quarter are requested from LDS three quarters ahead - the last three of a step
    // request the first three quarters of the following step's block NNBLK of buffer NNBUF - which
    // covers the LDS latency under load.
#define RA_WS_PRODUCE(SC, SN, BUF, BLK, NBUF, NBLK, NNBUF, NNBLK, PB, MASKED)                           \
  {                                                                                                     \
    RA_WS_INIT(SN, NBUF, NBLK);                                                                         \
    _Pragma("unroll") for (int g = 0; g < 4; g++) {                                                     \
      if (g == 0) { RA_WS_AREAD(3, ka[3], NBUF, NBLK); }                                                \
      else { RA_WS_AREAD(g - 1, ka[g - 1], NNBUF, NNBLK); }                                             \
      RA_WS_AMFMA(g, ka[g], SN);                                                                        \
      RA_WS_VECTOR(g, SC, BUF, BLK, PB, MASKED);                                                        \
      __builtin_amdgcn_sched_barrier(0);                                                                \
    }                                                                                                   \
  }

    f32x16 s_a, s_b;
    bf16x8 ka[4][KPG];
    RA_WS_INIT(s_a, 0, 0);
#pragma unroll
    for (int g = 0; g < 4; g++) {
      RA_WS_AREAD(g, ka[0], 0, 0);
      RA_WS_AMFMA(g, ka[0], s_a);
    }
#pragma unroll
    for (int g = 0; g < 3; g++) RA_WS_AREAD(g, ka[g], 0, 1);

    // Under a causal mask the tiles that need no masking come first: one loop for them, one for the rest
    // (which also takes every tile when segment ids or a bias are present).
    // Which key tiles need no masking at all: below the causal limit of every row, keys all of this wave's
    // single segment id, packed keep summary "all kept".  They form (at most) one run [t_a, t_b) in the
    // cases that matter - document interiors, the part of a causal row left of the diagonal - and get a
    // loop of their own; the tiles before and after take the masked loop.
    const int t_causal = (int)max(0LL, min((long long)ntiles, ((long long)klim_wave - gk0) / FBN));
    const uint64_t* kw_ptr = nullptr;
    const uint8_t* ks_ptr = nullptr;
    uint64_t kw_cur = 0, kw_nxt = 0, kw_some = 0, kw_k = 0;     // kw_k: the kept bits before the causal limit is folded in
    (void)kw_some; (void)kw_k;
    if (HAS_KEEP) {
      ks_ptr = mv.ksum + (int64_t)b * mv.ksum_sb + (int64_t)h * mv.ksum_sh +
               (int64_t)((mv.keep_q0 + q0 + pair * 32) / 64) * (mv.keep_K / 64) + (gk0 - mv.keep_k0) / 64;
      kw_ptr = mv.kbits_k + (int64_t)b * mv.kpack_sb + (int64_t)h * mv.kpack_sh +
               (int64_t)((gk0 - mv.keep_k0) / 64) * mv.keep_Q +
               mv.keep_q0 + qrow;
    }
    const int2* smm_ptr = nullptr;
    bool sq_uniform = false;
    int sq_id = 0;
    if (HAS_SEG && mv.seg_mm) {
      smm_ptr = (const int2*)(mv.seg_mm + (int64_t)(mv.seg_sb ? b : 0) * mv.seg_tiles * 2);
      const int2 qmm = smm_ptr[min((gq0 + pair * 32) / RA_SEG_TILE, mv.seg_tiles - 1)];
      sq_uniform = qmm.x == qmm.y;
      sq_id = qmm.x;
    }
    int t_a = ntiles, t_b = ntiles;
    for (int base = 0; base < ntiles; base += 64) {
      const int tt = base + lane;
      bool ok = tt < t_causal;
      if (HAS_SEG && ok) {
        ok = sq_uniform;
        if (ok) {
          const int2 kmm = smm_ptr[min(gk0 / RA_SEG_TILE + tt, mv.seg_tiles - 1)];
          ok = kmm.x == sq_id && kmm.y == sq_id;
        }
      }
      if (HAS_KEEP && ok) ok = ks_ptr[tt] == 2;
      const unsigned long long m = __builtin_amdgcn_ballot_w64(ok);
      unsigned long long stop;      // tiles of this group of 64 that end the run
      if (t_a == ntiles) {
        if (!m) continue;
        const int f = __builtin_ctzll(m);
        t_a = base + f;
        stop = ~m & (~0ULL << f);
      } else {
        stop = ~m;
      }
      if (stop) { t_b = min(ntiles, base + (int)__builtin_ctzll(stop)); break; }
    }
    t_a = __builtin_amdgcn_readfirstlane(t_a);
    t_b = __builtin_amdgcn_readfirstlane(t_a == ntiles ? ntiles : t_b);
    if (HAS_KEEP) kw_nxt = kw_ptr[(int64_t)min(t_a == 0 ? t_b : 0, ntiles - 1) * mv.keep_Q];
    int cur = 0;
#define RA_WS_TILE(MASKED)                                                                              \
  {                                                                                                     \
    const int nxt = cur == 2 ? 0 : cur + 1;                                                             \
    const int gk_tile = gk0 + t * FBN;                                                                  \
    (void)gk_tile;                                                                                      \
    if (HAS_KEEP && (MASKED)) {        /* this tile's word; request the next tile's */                  \
      kw_cur = kw_nxt >> (4 * hi);                                                                      \
      kw_nxt = kw_ptr[(int64_t)min(t + 1 == t_a ? t_b : t + 1, ntiles - 1) * mv.keep_Q];                \
      if (HAS_KEEP == 2) {             /* fold this row's causal limit into the words */                \
        const int nall_ = max(0, min(64, klim - gk_tile));                                              \
        const uint64_t cw_ = (nall_ >= 64 ? ~0ULL : ((1ULL << nall_) - 1ULL)) >> (4 * hi);              \
        kw_k = kw_cur;                                                                                  \
        kw_some = kw_cur | cw_;                                                                         \
        kw_cur &= cw_;                                                                                  \
      }                                                                                                 \
    }                                                                                                   \
    /* step 2t: vector work of block 0 of tile t, products of block 1 */                                \
    RA_WS_PRODUCE(s_a, s_b, cur, 0, cur, 1, nxt, 0, 0, MASKED);                                         \
    __syncthreads();                                                                                    \
    /* step 2t + 1: vector work of block 1, products of block 0 of tile t + 1 (the last tile computes  \
       a block that is never used) */                                                                   \
    RA_WS_PRODUCE(s_b, s_a, cur, 1, nxt, 0, nxt, 1, 1, MASKED);                                         \
    __syncthreads();                                                                                    \
    cur = nxt;                                                                                          \
  }
    int t = 0;
    if (HAS_BIAS) {
      // one loop: a tile inside the run still takes the masked path when one of its keys carries a bias at the level
      // of the mask value (the flag its staging left in LDS)
      for (; t < ntiles; t++) {
        if (t < t_a || t >= t_b || __builtin_amdgcn_readfirstlane(bias_any[cur])) RA_WS_TILE(true)
        else RA_WS_TILE(false)
      }
    } else {
      for (; t < t_a; t++) RA_WS_TILE(true);
      for (; t < t_b; t++) RA_WS_TILE(false);
      for (; t < ntiles; t++) RA_WS_TILE(true);
    }
#undef RA_WS_TILE
    __syncthreads();      // step 2 ntiles: the consumer's last block
    // bring the carry to the exact running max (:138) and hand the factor to the consumer
    const float fix = (m_true == m2) ? 1.f : fast_exp2(m2 - m_true);
    m2 = m_true;
    l *= fix;
    l += xor32(l);
    // the last step of the device hands over the denominator too: the consumer then writes numerator / denominator
    if (hi == 0) { fixs[pair][lo] = fix; dens[pair][lo] = l; }
    __syncthreads();
    if (hi == 0) {
      a.den[st] = l;
      a.mx[st] = max_from_log2(m2, kMask2);
    }
#undef RA_WS_ROWMAX
#undef RA_WS_INIT
#undef RA_WS_AREAD
#undef RA_WS_AMFMA
#undef RA_WS_VECTOR
#undef RA_WS_PRODUCE
  } else {
    // =========================== consumer: O^T += V^T P^T   (:141-143)
    RA_WS_LOAD_K(A, 0); RA_WS_LOAD_V(A, 0);
    RA_WS_LOAD_K(B, 1); RA_WS_LOAD_V(B, 1);
    RA_WS_STORE_K(A, 0); RA_WS_STORE_V(A, 0);
    RA_WS_LOAD_K(A, 2); RA_WS_LOAD_V(A, 2);
    RA_WS_STORE_K(B, 1); RA_WS_STORE_V(B, 1);
    RA_WS_LOAD_K(B, 3); RA_WS_LOAD_V(B, 3);
    __syncthreads();
    f32x16 acc[NDB];
    float* nump = a.num + (int64_t)b * a.num_sb + (int64_t)qrow * a.num_ss + (int64_t)h * HD + hi * 4;
    if (a.carry_is_initial) {
#pragma unroll
      for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
    } else {
#pragma unroll
      for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const f32x4 t4 = *(const f32x4*)(nump + db * 32 + g * 8);
#pragma unroll
          for (int e = 0; e < 4; e++) acc[db][g * 4 + e] = t4[e];
        }
    }
    int t_off[NDB][2];
    {
      const int i = lane & 15, rr = (i >> 2) + 8 * hi, c0 = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), half = lane & 1;
#pragma unroll
      for (int db = 0; db < NDB; db++) {
        t_off[db][0] = rr * TROW + (((4 * db + c0) ^ swz<HD>(rr)) << 3) + half * 4;
        t_off[db][1] = (rr + 4) * TROW + (((4 * db + c0) ^ swz<HD>(rr + 4)) << 3) + half * 4;
      }
    }
    const uint16_t* const dr = &Ds[pair][0][lo * WS_PSTR + hi * 8];   // B operand: query column lo, 8 keys

    // keys 16 K .. 16 K + 15 of block BLK of buffer BUF, transposed
#define RA_WS_CREAD(K, F, BUF, BLK)                                                                     \
  {                                                                                                     \
    const uint16_t* tp_ = Vs + (BUF) * WS_TILE + ((BLK) * 32 + (K) * 16) * TROW;                        \
    _Pragma("unroll") for (int db = 0; db < NDB; db++) {                                                  \
      const s16x4 x0_ = lds_read_tr(tp_ + t_off[db][0]);                                                \
      const s16x4 x1_ = lds_read_tr(tp_ + t_off[db][1]);                                                \
      F[db] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(x0_, x1_, 0, 1, 2, 3, 4, 5, 6, 7));    \
    }                                                                                                   \
  }
#define RA_WS_CMFMA(F, BOP)                                                                             \
  _Pragma("unroll") for (int db = 0; db < NDB; db++)                                                      \
    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[db], BOP, acc[db], 0, 0, 0);
    // fa holds the first 16 keys of the block on entry and, on exit, those of block NBLK of buffer NBUF
#define RA_WS_CONSUME(BUF, BLK, PB, NBUF, NBLK)                                                         \
  {                                                                                                     \
    const bf16x8 d0_ = *(const bf16x8*)(dr + (PB) * WS_PD);                                             \
    const bf16x8 d1_ = *(const bf16x8*)(dr + (PB) * WS_PD + 16);                                        \
    const float alpha_ = al[pair][PB][lo];                                                              \
    if (__builtin_amdgcn_ballot_w64(alpha_ != 1.f) != 0) {                                              \
      _Pragma("unroll") for (int db = 0; db < NDB; db++)                                                  \
        _Pragma("unroll") for (int r = 0; r < 16; r++) acc[db][r] *= alpha_;                            \
    }                                                                                                   \
    RA_WS_CREAD(1, fb, BUF, BLK);                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(fa, d0_);                                                                               \
    RA_WS_CREAD(0, fa, NBUF, NBLK);                                                                     \
    __builtin_amdgcn_sched_barrier(0);                                                                  \
    RA_WS_CMFMA(fb, d1_);                                                                               \
  }
    bf16x8 fa[NDB], fb[NDB];
    int cur = 0;
    RA_WS_CREAD(0, fa, 0, 0);
    __syncthreads();      // step 0
    // tile T + 2 (in register set S = (T + 2) & 1 = T & 1) goes to the buffer that held tile T - 1 (K in step
    // 2T + 1, V in step 2T + 2: the producer reads only K here) and tile T + 4 is requested into the same set
#define RA_WS_CTILE(S, T)                                                                               \
  {                                                                                                     \
    const int prv = cur == 0 ? 2 : cur - 1, nxt = cur == 2 ? 0 : cur + 1;                               \
    RA_WS_STORE_K(S, prv);                                                                              \
    RA_WS_LOAD_K(S, (T) + 4);                                                                           \
    RA_WS_CONSUME(cur, 0, 0, cur, 1);                                                                   \
    __syncthreads();                                                                                    \
    RA_WS_STORE_V(S, prv);                                                                              \
    RA_WS_LOAD_V(S, (T) + 4);                                                                           \
    RA_WS_CONSUME(cur, 1, 1, nxt, 0);                                                                   \
    __syncthreads();                                                                                    \
    cur = nxt;                                                                                          \
  }
    int t = 0;
    for (; t + 2 <= ntiles; t += 2) {
      RA_WS_CTILE(A, t);
      RA_WS_CTILE(B, t + 1);
    }
    if (t < ntiles) RA_WS_CTILE(A, t);
#undef RA_WS_CTILE
#undef RA_WS_CREAD
#undef RA_WS_CMFMA
#undef RA_WS_CONSUME

    __syncthreads();      // the producer's final factor
    const float fix = fixs[pair][lo];
    const float den_row = dens[pair][lo];
    const int64_t ooff = (int64_t)b * a.out_sb + (int64_t)qrow * a.out_ss + (int64_t)h * HD + hi * 4;
    uint16_t* outp = a.out + ooff;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        f32x4 t4;
#pragma unroll
        for (int e = 0; e < 4; e++) t4[e] = acc[db][g * 4 + e] * fix;
        if (a.out) {
#pragma unroll
          for (int e = 0; e < 4; e++) t4[e] /= den_row;               // :52
          store_bf16x4(outp + db * 32 + g * 8, t4);
          if (a.out32) *(f32x4*)(a.out32 + ooff + db * 32 + g * 8) = t4;   // the residual of :53
        } else {
          *(f32x4*)(nump + db * 32 + g * 8) = t4;
        }
      }
  }
#undef RA_WS_LOAD_K
#undef RA_WS_LOAD_V
#undef RA_WS_STORE_K
#undef RA_WS_STORE_V
}

// ------------------------------------------------------------------ host side
static bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

// a boolean keep mask is taken in packed form only; the attn_mask of ring_attention_inference next to a causal block
// size at most (it has no bias or segment ids there; the generic kernels serve any combination), the dropout mask
// next to everything
static bool keep_ok(const ra_mask& m) {
  if (!m.keep && !m.keep_bits_k) return true;
  if (!(m.keep_bits_k && m.keep_bits_q && m.keep_summary)) return false;
  return m.keep_mode == RA_KEEP_DROPOUT || (!m.bias && !m.segment_ids);
}

bool attn_fwd_mfma_supported(const ra_attn_fwd_params* p) {
  const ra_mask& m = p->mask;
  return p->dtype == RA_BF16 && (p->D == 128 || p->D == 64) && m.query_chunk_size % FBM == 0 && m.key_chunk_size % FBN == 0 &&
         keep_ok(m) && (m.bias == nullptr || m.bias_stride_q == 0) && p->q_stride_s % 8 == 0 && p->kv_stride_s % 8 == 0 &&
         p->q_stride_b % 8 == 0 && p->kv_stride_b % 8 == 0 && p->num_stride_s % 4 == 0 && p->num_stride_b % 4 == 0 &&
         aligned16(p->q) && aligned16(p->k) && aligned16(p->v) && aligned16(p->numerator) &&
         (!p->out || (aligned16(p->out) && p->out_stride_s % 4 == 0 && p->out_stride_b % 4 == 0)) &&
         aligned16(p->out_f32);
}

static RingView ring_view(const ra_ring_step* r) {
  RingView v{};
  if (r) { v.n = r->n_dev; v.idx = r->idx; v.run = r->run; v.first = r->first; v.last = r->last;
           v.kv_first = r->kv_first; v.kv_last = r->kv_last; }
  return v;
}

// r: nullable; all devices of a ring in one launch (p then describes the global arrays)
int attn_fwd_mfma(const ra_attn_fwd_params* p, const ra_ring_step* r, hipStream_t s) {
  FwdArgs a{};
  a.ring = ring_view(r);
  a.q = (const uint16_t*)p->q; a.k = (const uint16_t*)p->k; a.v = (const uint16_t*)p->v;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.num = p->numerator; a.num_sb = p->num_stride_b; a.num_ss = p->num_stride_s;
  a.den = p->denominator; a.mx = p->max_score; a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  a.carry_is_initial = p->carry_is_initial;
  a.sdim = p->logit_dim > 0 ? p->logit_dim : p->D;
  a.out = (uint16_t*)p->out; a.out_sb = p->out_stride_b; a.out_ss = p->out_stride_s; a.out32 = p->out_f32;
  const bool seg = p->mask.segment_ids != nullptr, bias = p->mask.bias != nullptr;
  const bool keep = p->mask.keep_bits_k != nullptr;      // packed form checked by attn_fwd_mfma_supported
  const long long nwg3 = (long long)(p->Sq / FBM) * p->H * p->B;
  RA_REQUIRE(nwg3 < (1LL << 31), RA_ERR_UNSUPPORTED, "attn_fwd_mfma: grid too large");
  dim3 grid3((unsigned)((nwg3 + 7) / 8 * 8)), block3(512);
#define RA_LAUNCH_FWD(...)                                                               \
  do {                                                                                   \
    if (p->D == 128) attn_fwd_ws_kernel<128, __VA_ARGS__><<<grid3, block3, 0, s>>>(a);   \
    else attn_fwd_ws_kernel<64, __VA_ARGS__><<<grid3, block3, 0, s>>>(a);                \
  } while (0)
  if (keep && p->mask.keep_mode == RA_KEEP_DROPOUT) {
    if (seg && bias) RA_LAUNCH_FWD(true, true, 2);
    else if (seg) RA_LAUNCH_FWD(true, false, 2);
    else if (bias) RA_LAUNCH_FWD(false, true, 2);
    else RA_LAUNCH_FWD(false, false, 2);
  } else if (keep) RA_LAUNCH_FWD(false, false, 1);
  else if (seg && bias) RA_LAUNCH_FWD(true, true);
  else if (seg) RA_LAUNCH_FWD(true, false);
  else if (bias) RA_LAUNCH_FWD(false, true);
  else RA_LAUNCH_FWD(false, false);
#undef RA_LAUNCH_FWD
  RA_CHECK_LAUNCH("attn_fwd_ws");
  return RA_OK;
}

bool attn_bwd_mfma_supported(const ra_attn_bwd_params* p) {
  const ra_mask& m = p->mask;
  return p->dtype == RA_BF16 && (p->D == 128 || p->D == 64) && m.query_chunk_size % FBM == 0 && m.key_chunk_size % KBN == 0 &&
         keep_ok(m) && (m.bias == nullptr || m.bias_stride_q == 0) && p->q_stride_s % 8 == 0 && p->kv_stride_s % 8 == 0 &&
         p->q_stride_b % 8 == 0 && p->kv_stride_b % 8 == 0 && p->dq_stride_s % 4 == 0 && p->dq_stride_b % 4 == 0 &&
         p->dkv_stride_s % 4 == 0 && p->dkv_stride_b % 4 == 0 && aligned16(p->q) && aligned16(p->k) &&
         aligned16(p->v) && aligned16(p->g) && aligned16(p->dq) && aligned16(p->dk) && aligned16(p->dv) &&
         (!p->dq_out || (aligned16(p->dq_out) && p->dq_out_stride_s % 4 == 0 && p->dq_out_stride_b % 4 == 0)) &&
         (!p->dk_out || (aligned16(p->dk_out) && aligned16(p->dv_out) && p->dkv_out_stride_s % 4 == 0 &&
                         p->dkv_out_stride_b % 4 == 0));
}

int attn_bwd_mfma(const ra_attn_bwd_params* p, const ra_ring_step* r, int parts, hipStream_t s) {   // parts: bit 0 dq, bit 1 dk / dv
  BwdArgs a{};
  a.ring = ring_view(r);
  a.q = (const uint16_t*)p->q; a.k = (const uint16_t*)p->k; a.v = (const uint16_t*)p->v; a.g = (const uint16_t*)p->g;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.delta = p->delta; a.den = p->denominator; a.mx = p->max_score;
  a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.dq = p->dq; a.dq_sb = p->dq_stride_b; a.dq_ss = p->dq_stride_s;
  a.dk = p->dk; a.dv = p->dv; a.dkv_sb = p->dkv_stride_b; a.dkv_ss = p->dkv_stride_s;
  a.dq_initial = (p->grads_are_initial & RA_GRAD_INIT_DQ) != 0;
  a.dkv_initial = (p->grads_are_initial & RA_GRAD_INIT_DKV) != 0;
  a.sdim = p->logit_dim > 0 ? p->logit_dim : p->D;
  a.dq_out = (uint16_t*)p->dq_out; a.dqo_sb = p->dq_out_stride_b; a.dqo_ss = p->dq_out_stride_s;
  a.dk_out = (uint16_t*)p->dk_out; a.dv_out = (uint16_t*)p->dv_out;
  a.dkvo_sb = p->dkv_out_stride_b; a.dkvo_ss = p->dkv_out_stride_s;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  const long long nq = (long long)(p->Sq / FBM) * p->H * p->B, nk = (long long)(p->Skv / KBN) * p->H * p->B;
  RA_REQUIRE(nq < (1LL << 31) && nk < (1LL << 31), RA_ERR_UNSUPPORTED, "attn_bwd_mfma: grid too large");
  const dim3 gq((unsigned)((nq + 7) / 8 * 8)), gk((unsigned)((nk + 7) / 8 * 8)), block(512);
  const bool seg = p->mask.segment_ids != nullptr, bias = p->mask.bias != nullptr;
  const bool do_dkv = (parts & 2) != 0, do_dq = (parts & 1) != 0;
#define RA_LAUNCH_BWD(...)                                                               \
  do {                                                                                   \
    if (p->D == 128) {                                                                   \
      if (do_dkv) attn_bwd_dkv_ws_kernel<128, __VA_ARGS__><<<gk, block, 0, s>>>(a);      \
      if (do_dq) attn_bwd_dq_ws_kernel<128, __VA_ARGS__><<<gq, block, 0, s>>>(a);        \
    } else {                                                                             \
      if (do_dkv) attn_bwd_dkv_ws_kernel<64, __VA_ARGS__><<<gk, block, 0, s>>>(a);       \
      if (do_dq) attn_bwd_dq_ws_kernel<64, __VA_ARGS__><<<gq, block, 0, s>>>(a);         \
    }                                                                                    \
  } while (0)
  if (p->mask.keep_bits_k && p->mask.keep_mode == RA_KEEP_DROPOUT) {
    if (seg && bias) RA_LAUNCH_BWD(true, true, 2);
    else if (seg) RA_LAUNCH_BWD(true, false, 2);
    else if (bias) RA_LAUNCH_BWD(false, true, 2);
    else RA_LAUNCH_BWD(false, false, 2);
  } else if (p->mask.keep_bits_k) RA_LAUNCH_BWD(false, false, 1);      // packed boolean mask
  else if (seg && bias) RA_LAUNCH_BWD(true, true);
  else if (seg) RA_LAUNCH_BWD(true, false);
  else if (bias) RA_LAUNCH_BWD(false, true);
  else RA_LAUNCH_BWD(false, false);
#undef RA_LAUNCH_BWD
  RA_CHECK_LAUNCH("attn_bwd_mfma");
  return RA_OK;
}

}  // namespace ra
