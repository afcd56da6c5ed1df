// Matrix-core attention kernels that evaluate the reference's mask element by element: what the generic kernels
// compute (any chunk sizes, any causal block size, a bias per key or per row, segment ids, a boolean mask given as
// bytes, lengths that are no multiple of a tile), with the four matrix products on v_mfma_f32_32x32x16_bf16.  bf16
// inputs, head size 128 or 256 (smaller ones arrive zero-padded).  They serve the calls the wave-specialised kernels
// of attn_mfma.hip do not take; attention dropout stays with the generic kernels.
//
// A workgroup of four wavefronts keeps 128 rows of one operand in registers (32 per wavefront: a lane owns one of
// them, so that row's softmax statistics are lane scalars) and streams 64-row tiles of the others through two LDS
// buffers, loaded straight from global memory a tile ahead (buffer_load ... lds), one barrier per tile.  Products are
// formed transposed, S^T = K Q^T, so the C layout hands every lane its own row's logits; P^T (dS^T) goes back in as a
// B operand from the same registers after one exchange with the partner lane, and the second operand of
// O^T += V^T P^T comes from LDS transpose reads.  At head size 256 the registers leave one wavefront per SIMD and
// nothing hides a wait, so the LDS reads of a group of four products are issued among the MFMAs of the group before;
// at head size 128 the kernels are bounded to 256 registers, so that two workgroups share a CU.  A tile whose pairs all run and are
// not masked skips the element-wise evaluation.
//
// Semantics follow ringattention_jax.py:130-145 (forward tile), :220-233 (backward tile), :272-322 (bias / mask)
// and :324-331 (skip predicate): row_info() of the generic kernels and their logit(), restated over per-tile tables.
#include "generic_args.hpp"
#include "../../include/ringattn_hip_measure.h"

namespace ra {

typedef __bf16 any_bf16x8 __attribute__((ext_vector_type(8)));
typedef float any_f32x16 __attribute__((ext_vector_type(16)));
typedef float any_f32x4 __attribute__((ext_vector_type(4)));
typedef short any_s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned any_u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned any_u32x4 __attribute__((ext_vector_type(4)));

constexpr int ANY_ROWS = 128;      // rows a workgroup keeps: four wavefronts of 32
constexpr int ANY_TILE = 64;       // rows of the streamed operands per step
constexpr int ANY_THREADS = 256;

// LDS tiles hold rows of HD bf16 without padding; the 16-byte slot c of row r sits at slot c ^ any_swz(r), which
// spreads a column of slots over the bank groups for the row reads and the four-row transpose reads below.
__device__ __forceinline__ int any_swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

__device__ __forceinline__ any_s16x4 any_read_tr(const uint16_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((any_s16x4 __attribute__((address_space(3)))*)(p));
}
__device__ __forceinline__ float any_max_xor32(float x) {
  any_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float any_sum_xor32(float x) {
  any_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// One 64-row tile of a (B, S, H, D) operand straight into an LDS buffer: a wavefront's load instruction fills 1024
// consecutive bytes (lane l the 16 bytes at 16 l), that is rows (4 i + wave) * RPL .. + RPL - 1 of the tile; the lane
// fetches the logical slot that belongs at its place (the swizzle is applied on the global side).  `base` is the
// tile's first row; rows past rows_avail repeat the last one (finite data that the mask logic never lets through).
// The loads are asynchronous: any_tile_barrier() before the buffer is read.
typedef __attribute__((address_space(3))) void* any_lds_ptr;
template <int HD>
struct AnyTileLoader {
  static constexpr int SLOTS = HD / 8, RPL = 64 / SLOTS, NL = ANY_TILE / RPL / 4;
  uint32_t voff[NL];                                   // byte offset of this lane's chunk of load i from the tile's first row
  int row0, stride, wave;
  __device__ __forceinline__ void init(int64_t stride_, int wave_, int lane) {
    stride = (int)stride_; wave = wave_; row0 = lane / SLOTS;
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const int r = (4 * i + wave) * RPL + row0, c = (lane % SLOTS) ^ any_swz(r);
      voff[i] = 2u * (uint32_t)(r * stride + c * 8);
    }
  }
  __device__ __forceinline__ void load(uint16_t* lds_tile, const uint16_t* base, int rows_avail) const {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0x7fffffff, 0x00020000);
    if (rows_avail >= ANY_TILE) {
#pragma unroll
      for (int i = 0; i < NL; i++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (any_lds_ptr)(lds_tile + (4 * i + wave) * 512), 16, voff[i], 0, 0, 0);
    } else {                                           // the last tile of a length that is no multiple of 64
#pragma unroll
      for (int i = 0; i < NL; i++) {
        const int r = (4 * i + wave) * RPL + row0;
        const uint32_t v = voff[i] - 2u * (uint32_t)((r - min(r, rows_avail - 1)) * stride);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (any_lds_ptr)(lds_tile + (4 * i + wave) * 512), 16, v, 0, 0, 0);
      }
    }
  }
};
// every load and LDS write of this wavefront has landed, then the workgroup meets: the tile loaded before is complete
// in LDS and nobody reads the buffer the next loads will fill
__device__ __forceinline__ void any_tile_barrier() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// A operand of contraction step ks (16 head dimensions): row `row` of an LDS tile, this lane's eight elements
template <int HD>
__device__ __forceinline__ any_bf16x8 any_row_frag(const uint16_t* tile, int row, int ks, int hi) {
  return *(const any_bf16x8*)(tile + row * HD + (((2 * ks + hi) ^ any_swz(row)) << 3));
}

// Offsets of the two transpose reads that give, for 16 consecutive tile rows starting at a multiple of 16, the A
// operand "32 head dimensions of block db x those 16 rows": lane half hi takes rows 8 hi .. 8 hi + 7.
template <int HD>
struct AnyTr {
  int a0, a1, x;                 // off[db][j] = aj + ((db ^ x) << 5): the swizzle flips the 32-dimension block by the row's low bits
  __device__ __forceinline__ void init(int lane) {
    const int hi = lane >> 5, i = lane & 15, rr = (i >> 2) + 8 * hi;
    const int c0 = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), half = lane & 1;
    x = rr & 3;
    a0 = rr * HD + ((c0 ^ ((rr >> 2) & 3)) << 3) + half * 4;
    a1 = (rr + 4) * HD + ((c0 ^ (((rr + 4) >> 2) & 3)) << 3) + half * 4;
  }
  __device__ __forceinline__ any_bf16x8 frag(const uint16_t* rows16, int db) const {
    const int o = (db ^ x) << 5;
    const any_s16x4 x0 = any_read_tr(rows16 + a0 + o);
    const any_s16x4 x1 = any_read_tr(rows16 + a1 + o);
    return __builtin_bit_cast(any_bf16x8, __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));
  }
};

// A 32 x 32 product block in the C layout: the lane's column is lane % 32, register 4 g + e holds row 8 g + 4 hi + e.
// The B operand of contraction step K over those rows (16 K .. 16 K + 15, lane half hi taking 16 K + 8 hi .. + 7)
// is made of this lane's registers of row group g = 2 K + hi and the partner lane's registers of the same group.
__device__ __forceinline__ any_bf16x8 any_bop(const any_f32x16& c, int K) {
  const uint32_t x0 = f32x2_to_bf16x2(c[8 * K + 0], c[8 * K + 1]), x1 = f32x2_to_bf16x2(c[8 * K + 2], c[8 * K + 3]);
  const uint32_t y0 = f32x2_to_bf16x2(c[8 * K + 4], c[8 * K + 5]), y1 = f32x2_to_bf16x2(c[8 * K + 6], c[8 * K + 7]);
  // lanes 0-31 keep x and receive the partner's x; lanes 32-63 receive the partner's y and keep y
  const any_u32x2 a = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
  const any_u32x2 b = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
  const any_u32x4 v = {a[0], b[0], a[1], b[1]};
  return __builtin_bit_cast(any_bf16x8, v);
}

// C[blk] += (rows 32 blk .. 32 blk + 31 of an LDS tile) x (the lane's resident operand), blk = 0, 1: the LDS reads of
// a group of four contraction steps are issued among the MFMAs of the group before.
template <int HD>
__device__ __forceinline__ void any_products(const uint16_t* tile, const any_bf16x8 (&bq)[HD / 16], any_f32x16 (&C)[2],
                                             int lo, int hi) {
  constexpr int G = 4, GPB = HD / 16 / G, NG = 2 * GPB;                 // groups per 32-row block, groups in all
  any_bf16x8 F[2][G];
#pragma unroll
  for (int i = 0; i < G; i++) F[0][i] = any_row_frag<HD>(tile, lo, i, hi);
  __builtin_amdgcn_sched_barrier(0);                   // all of the first group's reads go out before its first MFMA
#pragma unroll
  for (int g = 0; g < NG; g++) {
    if (g + 1 < NG) {
#pragma unroll
      for (int i = 0; i < G; i++)
        F[(g + 1) & 1][i] = any_row_frag<HD>(tile, ((g + 1) / GPB) * 32 + lo, ((g + 1) % GPB) * G + i, hi);
    }
#pragma unroll
    for (int i = 0; i < G; i++)
      C[g / GPB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[g & 1][i], bq[(g % GPB) * G + i], C[g / GPB], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < G; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (g + 1 < NG) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// One 32-row block of any_products: C += (rows row0 .. row0 + 31 of an LDS tile) x (the lane's resident operand).
template <int HD>
__device__ __forceinline__ void any_products_block(const uint16_t* tile, int row0, const any_bf16x8 (&bq)[HD / 16],
                                                   any_f32x16& C, int lo, int hi) {
  constexpr int G = 4, NG = HD / 16 / G;
  any_bf16x8 F[2][G];
#pragma unroll
  for (int i = 0; i < G; i++) F[0][i] = any_row_frag<HD>(tile, row0 + lo, i, hi);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int g = 0; g < NG; g++) {
    if (g + 1 < NG) {
#pragma unroll
      for (int i = 0; i < G; i++) F[(g + 1) & 1][i] = any_row_frag<HD>(tile, row0 + lo, (g + 1) * G + i, hi);
    }
#pragma unroll
    for (int i = 0; i < G; i++) C = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[g & 1][i], bq[g * G + i], C, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < G; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (g + 1 < NG) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// acc^T (head dimensions x the lanes' rows) += tile^T P^T for the 64 tile rows, P in the C layout of any_products:
// four steps of 16 tile rows, the transpose reads of a step issued among the MFMAs of the step before.
template <int HD>
__device__ __forceinline__ void any_accumulate(const uint16_t* tile, const AnyTr<HD>& tr, const any_f32x16 (&P)[2],
                                               any_f32x16 (&acc)[HD / 32]) {
  constexpr int NDB = HD / 32;
  any_bf16x8 F[2][NDB];
#pragma unroll
  for (int db = 0; db < NDB; db++) F[0][db] = tr.frag(tile, db);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < 4; s++) {
    if (s + 1 < 4) {
#pragma unroll
      for (int db = 0; db < NDB; db++) F[(s + 1) & 1][db] = tr.frag(tile + (s + 1) * 16 * HD, db);
    }
    const any_bf16x8 bop = any_bop(P[s >> 1], s & 1);
#pragma unroll
    for (int db = 0; db < NDB; db++)
      acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[s & 1][db], bop, acc[db], 0, 0, 0);
#pragma unroll
    for (int db = 0; db < NDB; db++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (s + 1 < 4) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// any_accumulate with the four B operands (16 tile rows each) already built
template <int HD>
__device__ __forceinline__ void any_accumulate_bops(const uint16_t* tile, const AnyTr<HD>& tr, const any_bf16x8 (&bops)[4],
                                                    any_f32x16 (&acc)[HD / 32]) {
  constexpr int NDB = HD / 32;
  any_bf16x8 F[2][NDB];
#pragma unroll
  for (int db = 0; db < NDB; db++) F[0][db] = tr.frag(tile, db);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < 4; s++) {
    if (s + 1 < 4) {
#pragma unroll
      for (int db = 0; db < NDB; db++) F[(s + 1) & 1][db] = tr.frag(tile + (s + 1) * 16 * HD, db);
    }
#pragma unroll
    for (int db = 0; db < NDB; db++)
      acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(F[s & 1][db], bops[s], acc[db], 0, 0, 0);
#pragma unroll
    for (int db = 0; db < NDB; db++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (s + 1 < 4) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

__device__ __forceinline__ int any_wave_max(int v) {
  for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off));
  return v;
}
__device__ __forceinline__ int any_wave_min(int v) {
  for (int off = 32; off > 0; off >>= 1) v = min(v, __shfl_xor(v, off));
  return v;
}
__device__ __forceinline__ long long any_wave_min(long long v) {
  for (int off = 32; off > 0; off >>= 1) { const long long o = __shfl_xor(v, off); v = o < v ? o : v; }
  return v;
}

// segment id of key kj (already clamped into the shard)
__device__ __forceinline__ int any_key_seg(const MaskView& mv, int b, int kj) {
  if (!mv.seg) return 0;
  const int ki = kj / mv.kc;
  const int idx = clamp_seg_index(((long long)mv.k_start + ki) * mv.kc, mv.kc, mv.seg_len, kj % mv.kc);
  return mv.seg[(int64_t)b * mv.seg_sb + idx];
}
// causal block (:326-331 compare query and key positions in units of causal_block_size) of local key kj
__device__ __forceinline__ long long any_key_block(const MaskView& mv, int kj) {
  const long long gk = mv.global_k(kj);
  return mv.cbs > 1 ? gk / mv.cbs : gk;
}
// a block index relative to a tile's base, as an int that still orders correctly against offsets 0 .. 64
__device__ __forceinline__ int any_rel(long long x) { return (int)(x < -2 ? -2 : (x > (1 << 20) ? (1 << 20) : x)); }

// What a 64-key tile leaves in LDS for the element-wise evaluation by the lanes that own query rows: per key its
// segment id, its bias (0 without a per-key bias; min(bias, 0) next to a mask, :299,:309) and its causal block
// relative to the block of the tile's first key.
struct AnyKeyTables {
  int seg[ANY_TILE];
  float bias[ANY_TILE];
  int blk[ANY_TILE];
  int segmin, segmax;                                  // range of the tile's segment ids
};
// what the tables hold when no tile writes them (no segment ids, no per-key bias, causal block size 1 or none)
__device__ __forceinline__ void any_init_keys(AnyKeyTables& T, int tid) {
  if (tid < ANY_TILE) { T.seg[tid] = 0; T.bias[tid] = 0.f; T.blk[tid] = tid; }
  if (tid == 0) { T.segmin = 0; T.segmax = 0; }
}
__device__ __forceinline__ void any_stage_keys(AnyKeyTables& T, const MaskView& mv, int b, int h, int k0, int skv,
                                               bool bias_per_key, int tid) {
  if (tid < ANY_TILE) {
    const int kj = min(k0 + tid, skv - 1);
    const int sg = any_key_seg(mv, b, kj);
    T.seg[tid] = sg;
    const int sgmin = any_wave_min(sg), sgmax = any_wave_max(sg);       // the staging threads are one wavefront
    if (tid == 0) { T.segmin = sgmin; T.segmax = sgmax; }
    float add = 0.f;
    if (bias_per_key) {
      add = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + mv.global_k(kj) * mv.bias_sk];
      if (mv.any_mask) add = fminf(add, 0.f);
    }
    T.bias[tid] = add;
    T.blk[tid] = mv.cbs > 1 ? (int)(any_key_block(mv, kj) - any_key_block(mv, min(k0, skv - 1))) : tid;
  }
}

// What a 64-row query tile leaves in LDS for the lanes that own key rows: the softmax statistics of every row and the
// row's part of the mask (run prefix, segment id, causal block relative to the block of the tile's first row).
struct AnyRowTables {
  float m[ANY_TILE], rden[ANY_TILE], delta[ANY_TILE];
  int kend[ANY_TILE], seg[ANY_TILE], blk[ANY_TILE];
  int64_t bias_off[ANY_TILE], keep_off[ANY_TILE];
  long long blk0;
  int kend_min;
  int segmin, segmax;                                  // range of the tile's rows' segment ids
};

__device__ __forceinline__ void any_stage_rows(AnyRowTables& T, const GenericArgs& a, const MaskView& mv, int b, int h,
                                               int q0, int tid) {
  if (tid < ANY_TILE) {
    const int row = q0 + tid;
    const bool rv = row < a.Sq;
    const int rr = rv ? row : a.Sq - 1;
    const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + rr;
    T.m[tid] = a.mx[st]; T.rden[tid] = 1.f / a.den[st]; T.delta[tid] = a.delta[st];
    const RowInfo ri = row_info(mv, b, h, rr, a.Skv);
    const long long g0 = mv.global_q(q0), b0 = mv.cbs > 1 ? g0 / mv.cbs : (mv.cbs == 1 ? g0 : 0);   // the first row's block
    const int kend = rv ? ri.kend : 0;
    T.kend[tid] = kend; T.seg[tid] = ri.seg; T.blk[tid] = mv.cbs > 0 ? (int)(ri.gq_blk - b0) : 0;
    const int sgmin = any_wave_min(ri.seg), sgmax = any_wave_max(ri.seg);       // the staging threads are one wavefront
    if (tid == 0) { T.segmin = sgmin; T.segmax = sgmax; }
    T.bias_off[tid] = ri.bias_off; T.keep_off[tid] = ri.keep_off;
    if (tid == 0) T.blk0 = b0;
    // the smallest run prefix of the tile's rows: rows are in order and the prefix grows with the row's chunk, so it
    // is the first row's, or 0 when a row past the end sits in the tile
    if (tid == 0) T.kend_min = (q0 + ANY_TILE <= a.Sq) ? kend : 0;
  }
}

// logit of (this lane's row, key kk of the tile) from the raw dot product: logit() of the generic kernels with the
// per-key parts read from the tile's tables.  drow: the row's causal block relative to the tile's base.
__device__ __forceinline__ float any_logit_row(const MaskView& mv, const RowInfo& ri, const AnyKeyTables& T, float dot,
                                               float rscale, int k0, int kk, int skv, int drow, bool bias_per_row) {
  const int kj = k0 + kk;
  float add = T.bias[kk];
  bool masked = (mv.cbs > 0 && drow < T.blk[kk]) || (mv.seg && ri.seg != T.seg[kk]);
  if (bias_per_row || mv.keep) {
    const long long gk = mv.global_k(min(kj, skv - 1));
    if (bias_per_row) {
      add = mv.bias[ri.bias_off + gk * mv.bias_sk];
      if (mv.any_mask) add = fminf(add, 0.f);                           // minimum(), :299,:309
    }
    if (mv.keep) masked = masked || !mv.keep[ri.keep_off + (gk - mv.keep_k0) * mv.keep_sk];   // ringattention_inference.py:24
  }
  const float s = masked ? mv.mask_min : fmaf(dot, rscale, add);        // :134-136 (a logit next to finfo.min is absorbed)
  return kj < ri.kend ? s : RA_NEG_INF;                                 // the pair's chunks do not run (:158-164)
}

// ------------------------------------------------------------------ forward
template <int HD>
__global__ __launch_bounds__(ANY_THREADS, HD > 128 ? 1 : 2) void attn_fwd_any_kernel(GenericArgs a) {
  constexpr int NKS = HD / 16, NDB = HD / 32;
  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) uint16_t Vs[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) AnyKeyTables kts[2];
  __shared__ int kend_s[4];
  const MaskView mv = resolve_mask(a);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int b = blockIdx.z, h = blockIdx.y;
  const int qtile = gridDim.x - 1 - blockIdx.x;              // under a causal mask the longest rows start first
  const int row = qtile * ANY_ROWS + wave * 32 + lo;
  const bool valid = row < a.Sq;
  const int rrow = valid ? row : a.Sq - 1;
  const uint16_t* qp = (const uint16_t*)a.q + (int64_t)b * a.q_sb + (int64_t)rrow * a.q_ss + (int64_t)h * HD;
  const uint16_t* kbase = (const uint16_t*)a.k + (int64_t)b * a.kv_sb + (int64_t)h * HD;
  const uint16_t* vbase = (const uint16_t*)a.v + (int64_t)b * a.kv_sb + (int64_t)h * HD;
  const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + rrow;
  const float scale = sqrtf((float)a.sdim);                            // :118

  any_bf16x8 qf[NKS];                                                  // B operands: this lane's query, 8 dims per step
#pragma unroll
  for (int ks = 0; ks < NKS; ks++) qf[ks] = *(const any_bf16x8*)(qp + ks * 16 + hi * 8);

  any_f32x16 acc[NDB];                                                 // O^T: register 4 g + e of block db = dim 32 db + 8 g + 4 hi + e
  float m = RA_NEG_INF, l = 0.f;                                       // l: this lane's share of the denominator
  if (a.carry_is_initial) {
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
  } else {
    const float* nump = a.num + (int64_t)b * a.num_sb + (int64_t)rrow * a.num_ss + (int64_t)h * HD + hi * 4;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const any_f32x4 t4 = *(const any_f32x4*)(nump + db * 32 + g * 8);
#pragma unroll
        for (int e = 0; e < 4; e++) acc[db][g * 4 + e] = t4[e];
      }
    m = a.mx[st];
    l = hi == 0 ? a.den[st] : 0.f;
  }
  RowInfo ri = row_info(mv, b, h, rrow, a.Skv);
  if (!valid) ri.kend = 0;
  const int kend_max_w = any_wave_max(ri.kend), kend_min_w = any_wave_min(ri.kend);
  const long long gqblk_min_w = any_wave_min(ri.gq_blk);
  if (lane == 0) kend_s[wave] = kend_max_w;
  __syncthreads();
  const int kend_wg = max(max(kend_s[0], kend_s[1]), max(kend_s[2], kend_s[3]));
  const int ntile = (kend_wg + ANY_TILE - 1) / ANY_TILE;
  const bool bias_per_key = mv.bias && mv.bias_sq == 0, bias_per_row = mv.bias && mv.bias_sq != 0;
  const bool elementwise_always = mv.keep || bias_per_row;
  const int rseg_min_w = any_wave_min(ri.seg), rseg_max_w = any_wave_max(ri.seg);
  const float rscale = 1.f / scale;

  AnyTr<HD> tr;
  tr.init(lane);
  AnyTileLoader<HD> ld;
  ld.init(a.kv_ss, wave, lane);
  const bool key_tables = mv.seg || bias_per_key || mv.cbs > 1;        // else: no ids, no bias, key i of a tile in block i
  any_init_keys(kts[0], tid);
  any_init_keys(kts[1], tid);
  __syncthreads();
  if (ntile > 0) {
    ld.load(Ks[0], kbase, a.Skv);
    ld.load(Vs[0], vbase, a.Skv);
    if (key_tables) any_stage_keys(kts[0], mv, b, h, 0, a.Skv, bias_per_key, tid);
  }
#pragma unroll 1
  for (int t = 0; t < ntile; t++) {
    const int k0 = t * ANY_TILE;
    any_tile_barrier();                                // tile t is in LDS; the other buffer has been read by everyone
    const uint16_t* Kt = Ks[t & 1];
    const uint16_t* Vt = Vs[t & 1];
    const AnyKeyTables& kt = kts[t & 1];
    // no row of this wavefront runs against these keys; or no key of the tile shares a segment id with a row of the
    // wavefront: every pair is masked, and where the caller vouches that every row has a key of its own
    // (skip_masked_tiles) such a tile weighs exactly nothing
    const bool active = k0 < kend_max_w &&
                        !(mv.seg && mv.skip_tiles && (kt.segmax < rseg_min_w || kt.segmin > rseg_max_w));
    any_f32x16 S[2];                                   // S^T, two blocks of 32 keys: register 4 g + e = key 8 g + 4 hi + e
    if (active) {
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) S[blk][r] = 0.f;
      any_products<HD>(Kt, qf, S, lo, hi);             // :134
    }
    // The next tile travels while this one is worked on.  Here its loads go out behind the first batch of products:
    // they share a counter with every other memory access of the wavefront, and the registers that the compiler keeps
    // in scratch memory at head size 256 are reloaded for those products - behind the loads they would wait for them
    // too (measured: 10-25 % of the forward kernel; the backward kernels measured better with the loads first).
    if (t + 1 < ntile) {
      const int k1 = k0 + ANY_TILE;
      ld.load(Ks[(t + 1) & 1], kbase + (int64_t)k1 * a.kv_ss, a.Skv - k1);
      ld.load(Vs[(t + 1) & 1], vbase + (int64_t)k1 * a.kv_ss, a.Skv - k1);
      if (key_tables) any_stage_keys(kts[(t + 1) & 1], mv, b, h, k1, a.Skv, bias_per_key, tid);
    }
    if (!active) continue;

    // every pair of the tile runs and is unmasked for every row of the wavefront: logit = dot / scale + bias
    const bool plain = !elementwise_always && k0 + ANY_TILE <= kend_min_w &&
                       (mv.cbs <= 0 || gqblk_min_w >= any_key_block(mv, k0 + ANY_TILE - 1)) &&
                       (!mv.seg || (kt.segmin == kt.segmax && rseg_min_w == rseg_max_w && kt.segmin == rseg_min_w));
    float tmax = RA_NEG_INF;
    if (plain) {
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const any_f32x4 b4 = *(const any_f32x4*)&kt.bias[blk * 32 + g * 8 + hi * 4];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float s = fmaf(S[blk][g * 4 + e], rscale, b4[e]);     // :134-136
            S[blk][g * 4 + e] = s;
            tmax = fmaxf(tmax, s);
          }
        }
    } else {
      const int drow = any_rel(ri.gq_blk - any_key_block(mv, min(k0, a.Skv - 1)));
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int kk = blk * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
          const float s = any_logit_row(mv, ri, kt, S[blk][r], rscale, k0, kk, a.Skv, drow, bias_per_row);
          S[blk][r] = s;
          tmax = fmaxf(tmax, s);
        }
    }
    tmax = any_max_xor32(tmax);
    const float m_new = fmaxf(m, tmax);                                 // :138
    const float mm = m_new == RA_NEG_INF ? 0.f : m_new;                 // nothing ran for this row yet: every p is 0
    const float corr = (m == m_new) ? 1.f : __expf(m - mm);             // :142
    float psum = 0.f;
#pragma unroll
    for (int blk = 0; blk < 2; blk++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p = __expf(S[blk][r] - mm);                         // :140
        S[blk][r] = p;
        psum += p;
      }
    l = l * corr + psum;                                                // :144
    m = m_new;
    if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
      for (int db = 0; db < NDB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[db][r] *= corr;                // :143
    }
    any_accumulate<HD>(Vt, tr, S, acc);                // :141
  }
  if (valid) {
    const float den = any_sum_xor32(l);
    const int64_t ooff = (int64_t)b * a.out_sb + (int64_t)rrow * a.out_ss + (int64_t)h * HD + hi * 4;
    float* nump = a.num + (int64_t)b * a.num_sb + (int64_t)rrow * a.num_ss + (int64_t)h * HD + hi * 4;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        any_f32x4 t4;
#pragma unroll
        for (int e = 0; e < 4; e++) t4[e] = acc[db][g * 4 + e];
        if (a.out) {                       // last step of the device: out = numerator / denominator (:52)
#pragma unroll
          for (int e = 0; e < 4; e++) t4[e] /= den;
          uint2 pk = {f32x2_to_bf16x2(t4[0], t4[1]), f32x2_to_bf16x2(t4[2], t4[3])};
          *(uint2*)((uint16_t*)a.out + ooff + db * 32 + g * 8) = pk;
          if (a.out32) *(any_f32x4*)(a.out32 + ooff + db * 32 + g * 8) = t4;      // the residual of :53
        } else {
          *(any_f32x4*)(nump + db * 32 + g * 8) = t4;
        }
      }
    if (hi == 0) { a.mx[st] = m; a.den[st] = den; }
  }
}

// ------------------------------------------------------------------ backward, dq (a lane owns a query row)
template <int HD>
__global__ __launch_bounds__(ANY_THREADS, HD > 128 ? 1 : 2) void attn_bwd_dq_any_kernel(GenericArgs a) {
  constexpr int NKS = HD / 16, NDB = HD / 32;
  __shared__ __attribute__((aligned(16))) uint16_t Ks[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) uint16_t Vs[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) AnyKeyTables kts[2];
  __shared__ int kend_s[4];
  const MaskView mv = resolve_mask(a);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int b = blockIdx.z, h = blockIdx.y;
  const int qtile = gridDim.x - 1 - blockIdx.x;
  const int row = qtile * ANY_ROWS + wave * 32 + lo;
  const bool valid = row < a.Sq;
  const int rrow = valid ? row : a.Sq - 1;
  const int64_t qoff = (int64_t)b * a.q_sb + (int64_t)rrow * a.q_ss + (int64_t)h * HD;
  const uint16_t* qp = (const uint16_t*)a.q + qoff;
  const uint16_t* gp = (const uint16_t*)a.g + qoff;
  const uint16_t* kbase = (const uint16_t*)a.k + (int64_t)b * a.kv_sb + (int64_t)h * HD;
  const uint16_t* vbase = (const uint16_t*)a.v + (int64_t)b * a.kv_sb + (int64_t)h * HD;
  const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + rrow;
  const float scale = sqrtf((float)a.sdim);

  any_bf16x8 qf[NKS], gf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ks++) {
    qf[ks] = *(const any_bf16x8*)(qp + ks * 16 + hi * 8);
    gf[ks] = *(const any_bf16x8*)(gp + ks * 16 + hi * 8);
  }
  any_f32x16 acc[NDB];                                                 // dQ^T
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
  const float m = a.mx[st], rden = 1.f / a.den[st], delta = a.delta[st];
  RowInfo ri = row_info(mv, b, h, rrow, a.Skv);
  if (!valid) ri.kend = 0;
  const int kend_max_w = any_wave_max(ri.kend), kend_min_w = any_wave_min(ri.kend);
  const long long gqblk_min_w = any_wave_min(ri.gq_blk);
  if (lane == 0) kend_s[wave] = kend_max_w;
  __syncthreads();
  const int kend_wg = max(max(kend_s[0], kend_s[1]), max(kend_s[2], kend_s[3]));
  const int ntile = (kend_wg + ANY_TILE - 1) / ANY_TILE;
  const bool bias_per_key = mv.bias && mv.bias_sq == 0, bias_per_row = mv.bias && mv.bias_sq != 0;
  const bool elementwise_always = mv.keep || bias_per_row;
  const int rseg_min_w = any_wave_min(ri.seg), rseg_max_w = any_wave_max(ri.seg);
  const float rscale = 1.f / scale;

  AnyTr<HD> tr;
  tr.init(lane);
  AnyTileLoader<HD> ld;
  ld.init(a.kv_ss, wave, lane);
  const bool key_tables = mv.seg || bias_per_key || mv.cbs > 1;        // else: no ids, no bias, key i of a tile in block i
  any_init_keys(kts[0], tid);
  any_init_keys(kts[1], tid);
  __syncthreads();
  if (ntile > 0) {
    ld.load(Ks[0], kbase, a.Skv);
    ld.load(Vs[0], vbase, a.Skv);
    if (key_tables) any_stage_keys(kts[0], mv, b, h, 0, a.Skv, bias_per_key, tid);
  }
#pragma unroll 1
  for (int t = 0; t < ntile; t++) {
    const int k0 = t * ANY_TILE;
    any_tile_barrier();                                // tile t is in LDS; the other buffer has been read by everyone
    if (t + 1 < ntile) {                               // the next tile travels while this one is worked on
      const int k1 = k0 + ANY_TILE;
      ld.load(Ks[(t + 1) & 1], kbase + (int64_t)k1 * a.kv_ss, a.Skv - k1);
      ld.load(Vs[(t + 1) & 1], vbase + (int64_t)k1 * a.kv_ss, a.Skv - k1);
      if (key_tables) any_stage_keys(kts[(t + 1) & 1], mv, b, h, k1, a.Skv, bias_per_key, tid);
    }
    if (k0 >= kend_max_w) continue;
    const uint16_t* Kt = Ks[t & 1];
    const uint16_t* Vt = Vs[t & 1];
    const AnyKeyTables& kt = kts[t & 1];
    if (mv.seg && mv.skip_tiles && (kt.segmax < rseg_min_w || kt.segmin > rseg_max_w)) continue;   // as in the forward kernel

    const bool plain = !elementwise_always && k0 + ANY_TILE <= kend_min_w &&
                       (mv.cbs <= 0 || gqblk_min_w >= any_key_block(mv, k0 + ANY_TILE - 1)) &&
                       (!mv.seg || (kt.segmin == kt.segmax && rseg_min_w == rseg_max_w && kt.segmin == rseg_min_w));
    const int drow = any_rel(ri.gq_blk - any_key_block(mv, min(k0, a.Skv - 1)));
    // one block of 32 keys at a time: S^T and dP^T of a block are turned into dS^T and packed before the next block's
    // products start, which keeps 32 registers fewer alive than both blocks at once
    any_bf16x8 bops[4];
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      any_f32x16 S, dP;
#pragma unroll
      for (int r = 0; r < 16; r++) { S[r] = 0.f; dP[r] = 0.f; }
      any_products_block<HD>(Kt, blk * 32, qf, S, lo, hi);             // :223-225
      any_products_block<HD>(Vt, blk * 32, gf, dP, lo, hi);            // :228
      if (plain) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const any_f32x4 b4 = *(const any_f32x4*)&kt.bias[blk * 32 + g * 8 + hi * 4];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float p = __expf(fmaf(S[g * 4 + e], rscale, b4[e]) - m) * rden;           // :226
            S[g * 4 + e] = (dP[g * 4 + e] - delta) * p;                                       // dS^T, :229
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int kk = blk * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
          const float s = any_logit_row(mv, ri, kt, S[r], rscale, k0, kk, a.Skv, drow, bias_per_row);
          const float p = __expf(s - m) * rden;                         // :226
          // a pair whose tile does not run contributes nothing (:246-257)
          S[r] = (k0 + kk < ri.kend) ? (dP[r] - delta) * p : 0.f;       // dS^T, :229
          if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);
        }
      }
      bops[2 * blk] = any_bop(S, 0);
      bops[2 * blk + 1] = any_bop(S, 1);
    }
    any_accumulate_bops<HD>(Kt, tr, bops, acc);        // :230
  }
  if (valid) {
    const int64_t off = (int64_t)h * HD + hi * 4;
    float* dqp = a.dq + (int64_t)b * a.dq_sb + (int64_t)rrow * a.dq_ss + off;
    uint16_t* op = (uint16_t*)a.dq_out + (int64_t)b * a.dqo_sb + (int64_t)rrow * a.dqo_ss + off;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        any_f32x4 t4 = {0.f, 0.f, 0.f, 0.f};
        if (!a.dq_initial) t4 = *(const any_f32x4*)(dqp + db * 32 + g * 8);
#pragma unroll
        for (int e = 0; e < 4; e++) t4[e] += acc[db][g * 4 + e] / scale;
        if (a.dq_out) {                                                 // last call for these rows (:89)
          uint2 pk = {f32x2_to_bf16x2(t4[0], t4[1]), f32x2_to_bf16x2(t4[2], t4[3])};
          *(uint2*)(op + db * 32 + g * 8) = pk;
        } else {
          *(any_f32x4*)(dqp + db * 32 + g * 8) = t4;
        }
      }
  }
}

// ------------------------------------------------------------------ backward, dk or dv (a lane owns a key row)
// Head size 128: one launch for each of the two (S is formed twice); head size 256 takes the kernel after this one.
template <int HD, bool WANT_DK>
__global__ __launch_bounds__(ANY_THREADS, HD > 128 ? 1 : 2) void attn_bwd_dkv_any_kernel(GenericArgs a) {
  constexpr int NKS = HD / 16, NDB = HD / 32;
  __shared__ __attribute__((aligned(16))) uint16_t Qs[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) uint16_t Gs[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) AnyRowTables rts[2];
  const MaskView mv = resolve_mask(a);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int b = blockIdx.z, h = blockIdx.y;
  const int first_key = blockIdx.x * ANY_ROWS;
  const int kj = first_key + wave * 32 + lo;
  const bool valid = kj < a.Skv;
  const int rk = valid ? kj : a.Skv - 1;
  const int64_t koff = (int64_t)b * a.kv_sb + (int64_t)rk * a.kv_ss + (int64_t)h * HD;
  const uint16_t* kp = (const uint16_t*)a.k + koff;
  const uint16_t* vp = (const uint16_t*)a.v + koff;
  const uint16_t* qbase = (const uint16_t*)a.q + (int64_t)b * a.q_sb + (int64_t)h * HD;
  const uint16_t* gbase = (const uint16_t*)a.g + (int64_t)b * a.q_sb + (int64_t)h * HD;
  const float scale = sqrtf((float)a.sdim), rscale = 1.f / scale;

  any_bf16x8 kf[NKS], vf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ks++) kf[ks] = *(const any_bf16x8*)(kp + ks * 16 + hi * 8);
  if (WANT_DK) {
#pragma unroll
    for (int ks = 0; ks < NKS; ks++) vf[ks] = *(const any_bf16x8*)(vp + ks * 16 + hi * 8);
  }
  any_f32x16 acc[NDB];                                                 // dK^T or dV^T
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
  const int seg_k = any_key_seg(mv, b, rk);
  const long long gk = mv.global_k(rk);
  const long long kblk = any_key_block(mv, rk);                        // this lane's key
  const int key_hi_w = first_key + wave * 32 + 32;                     // one past the wavefront's last key
  const long long kblk_max_w = any_key_block(mv, min(key_hi_w, a.Skv) - 1);
  const bool bias_per_key = mv.bias && mv.bias_sq == 0, bias_per_row = mv.bias && mv.bias_sq != 0;
  const bool elementwise_always = mv.keep || bias_per_row;
  const int kseg_min_w = any_wave_min(seg_k), kseg_max_w = any_wave_max(seg_k);
  float bias_k = 0.f;                                                  // a bias per key is a lane scalar here
  if (bias_per_key) {
    bias_k = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + gk * mv.bias_sk];
    if (mv.any_mask) bias_k = fminf(bias_k, 0.f);
  }
  const bool wave_valid = first_key + wave * 32 < a.Skv;               // some key of the wavefront exists
  const bool all_valid = key_hi_w <= a.Skv;

  AnyTr<HD> tr;
  tr.init(lane);
  // query tiles whose last row's run prefix ends before this block's first key hold nothing for it; the prefix grows
  // with the query chunk, so the tiles that count are a suffix
  int t_first = 0;
  const int ntile = (a.Sq + ANY_TILE - 1) / ANY_TILE;
  while (t_first < ntile &&
         mv.run_prefix_keys((min((t_first + 1) * ANY_TILE, a.Sq) - 1) / mv.qc, a.Skv) <= first_key) t_first++;
  AnyTileLoader<HD> ld;
  ld.init(a.q_ss, wave, lane);
  if (t_first < ntile) {
    const int q0 = t_first * ANY_TILE;
    ld.load(Qs[t_first & 1], qbase + (int64_t)q0 * a.q_ss, a.Sq - q0);
    ld.load(Gs[t_first & 1], gbase + (int64_t)q0 * a.q_ss, a.Sq - q0);
    any_stage_rows(rts[t_first & 1], a, mv, b, h, q0, tid);
  }
#pragma unroll 1
  for (int t = t_first; t < ntile; t++) {
    const int q0 = t * ANY_TILE;
    any_tile_barrier();                                // tile t is in LDS; the other buffer has been read by everyone
    if (t + 1 < ntile) {
      const int q1 = q0 + ANY_TILE;
      ld.load(Qs[(t + 1) & 1], qbase + (int64_t)q1 * a.q_ss, a.Sq - q1);
      ld.load(Gs[(t + 1) & 1], gbase + (int64_t)q1 * a.q_ss, a.Sq - q1);
      any_stage_rows(rts[(t + 1) & 1], a, mv, b, h, q1, tid);
    }
    if (!wave_valid) continue;
    const uint16_t* Qt = Qs[t & 1];
    const uint16_t* Gt = Gs[t & 1];
    const AnyRowTables& rt = rts[t & 1];
    // no row of the tile shares a segment id with a key of the wavefront (see the forward kernel)
    if (mv.seg && mv.skip_tiles && (rt.segmax < kseg_min_w || rt.segmin > kseg_max_w)) continue;

    // every pair of (tile rows, the wavefront's keys) runs and is unmasked
    const bool plain = !elementwise_always && all_valid && key_hi_w <= rt.kend_min &&
                       (mv.cbs <= 0 || rt.blk0 >= kblk_max_w) &&
                       (!mv.seg || (rt.segmin == rt.segmax && kseg_min_w == kseg_max_w && rt.segmin == kseg_min_w));
    const int dkey = any_rel(kblk - rt.blk0);          // this key's causal block relative to the tile's first row's
    // one block of 32 query rows at a time (S, dP: the lane's key column; register 4 g + e = query 8 g + 4 hi + e), turned
    // into P or dS and packed before the next block's products start
    any_bf16x8 bops[4];
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
      any_f32x16 S, dP;
#pragma unroll
      for (int r = 0; r < 16; r++) { S[r] = 0.f; dP[r] = 0.f; }
      any_products_block<HD>(Qt, blk * 32, kf, S, lo, hi);
      if (WANT_DK) any_products_block<HD>(Gt, blk * 32, vf, dP, lo, hi);
      if (plain) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int q4 = blk * 32 + g * 8 + hi * 4;
          const any_f32x4 m4 = *(const any_f32x4*)&rt.m[q4], d4 = *(const any_f32x4*)&rt.rden[q4];
          const any_f32x4 e4 = *(const any_f32x4*)&rt.delta[q4];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float p = __expf(fmaf(S[g * 4 + e], rscale, bias_k) - m4[e]) * d4[e];               // :226
            S[g * 4 + e] = WANT_DK ? (dP[g * 4 + e] - e4[e]) * p : p;                                   // dS (:229) or P
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qq = blk * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
          float add = bias_k;
          bool masked = (mv.cbs > 0 && rt.blk[qq] < dkey) || (mv.seg && rt.seg[qq] != seg_k);
          if (bias_per_row) {
            add = mv.bias[rt.bias_off[qq] + gk * mv.bias_sk];
            if (mv.any_mask) add = fminf(add, 0.f);                     // minimum(), :299,:309
          }
          if (mv.keep) masked = masked || !mv.keep[rt.keep_off[qq] + (gk - mv.keep_k0) * mv.keep_sk];
          const float s = masked ? mv.mask_min : fmaf(S[r], rscale, add);
          const float p = (valid && kj < rt.kend[qq]) ? __expf(s - rt.m[qq]) * rt.rden[qq] : 0.f;     // :226; (:246-257)
          S[r] = WANT_DK ? (dP[r] - rt.delta[qq]) * p : p;              // dS (:229) or P
          if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);
        }
      }
      bops[2 * blk] = any_bop(S, 0);
      bops[2 * blk + 1] = any_bop(S, 1);
    }
    any_accumulate_bops<HD>(WANT_DK ? Qt : Gt, tr, bops, acc);   // :231 / :232
  }
  if (valid) {
    const int64_t off = (int64_t)h * HD + hi * 4;
    float* outp = (WANT_DK ? a.dk : a.dv) + (int64_t)b * a.dkv_sb + (int64_t)rk * a.dkv_ss + off;
    uint16_t* op = (uint16_t*)(WANT_DK ? a.dk_out : a.dv_out) + (int64_t)b * a.dkvo_sb + (int64_t)rk * a.dkvo_ss + off;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        any_f32x4 t4 = {0.f, 0.f, 0.f, 0.f};
        if (!a.dkv_initial) t4 = *(const any_f32x4*)(outp + db * 32 + g * 8);
#pragma unroll
        for (int e = 0; e < 4; e++) t4[e] += WANT_DK ? acc[db][g * 4 + e] / scale : acc[db][g * 4 + e];
        if (a.dk_out) {                                                 // last call for these keys (:89)
          uint2 pk = {f32x2_to_bf16x2(t4[0], t4[1]), f32x2_to_bf16x2(t4[2], t4[3])};
          *(uint2*)(op + db * 32 + g * 8) = pk;
        } else {
          *(any_f32x4*)(outp + db * 32 + g * 8) = t4;
        }
      }
  }
}

// ------------------------------------------------------------------ backward, dk and dv at head size 256
// Both accumulators of a 256-wide head do not fit one wavefront next to its operands, so two wavefronts share 32 keys:
// each forms S and dP for one half of a query tile's rows (all 256 head dimensions), leaves P and dS, rounded to
// bf16, in LDS as [key][query], and after a barrier accumulates one half of the head dimensions of dK^T and dV^T over
// all 64 rows.  Every product is formed once (8 D per pair).  A workgroup of four wavefronts serves 64 keys.
constexpr int ANY_PSTR = ANY_TILE + 8;                 // row of the P / dS exchange buffers: 64 queries and padding
template <int HD>
__global__ __launch_bounds__(ANY_THREADS) void attn_bwd_dkv_pair_any_kernel(GenericArgs a) {
  constexpr int NKS = HD / 16, NDB = HD / 64;          // head-dimension blocks of 32 per wavefront: half of the head
  __shared__ __attribute__((aligned(16))) uint16_t Qs[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) uint16_t Gs[2][ANY_TILE * HD];
  __shared__ __attribute__((aligned(16))) uint16_t Pt[2][32 * ANY_PSTR];      // [key group][key][query]
  __shared__ __attribute__((aligned(16))) uint16_t Dt[2][32 * ANY_PSTR];
  __shared__ __attribute__((aligned(16))) AnyRowTables rts[2];
  const MaskView mv = resolve_mask(a);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lo = lane & 31, hi = lane >> 5;
  const int kg = wave >> 1, half = wave & 1;           // key group; half of the tile's rows, and of the head dimensions
  const int b = blockIdx.z, h = blockIdx.y;
  const int first_key = blockIdx.x * 64;
  const int kj = first_key + kg * 32 + lo;
  const bool valid = kj < a.Skv;
  const int rk = valid ? kj : a.Skv - 1;
  const int64_t koff = (int64_t)b * a.kv_sb + (int64_t)rk * a.kv_ss + (int64_t)h * HD;
  const uint16_t* kp = (const uint16_t*)a.k + koff;
  const uint16_t* vp = (const uint16_t*)a.v + koff;
  const uint16_t* qbase = (const uint16_t*)a.q + (int64_t)b * a.q_sb + (int64_t)h * HD;
  const uint16_t* gbase = (const uint16_t*)a.g + (int64_t)b * a.q_sb + (int64_t)h * HD;
  const float scale = sqrtf((float)a.sdim), rscale = 1.f / scale;

  any_bf16x8 kf[NKS], vf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ks++) {
    kf[ks] = *(const any_bf16x8*)(kp + ks * 16 + hi * 8);
    vf[ks] = *(const any_bf16x8*)(vp + ks * 16 + hi * 8);
  }
  any_f32x16 acc_k[NDB], acc_v[NDB];                   // dK^T, dV^T: head dimensions 128 half + 32 db + ...
#pragma unroll
  for (int db = 0; db < NDB; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) { acc_k[db][r] = 0.f; acc_v[db][r] = 0.f; }
  const int seg_k = any_key_seg(mv, b, rk);
  const long long gk = mv.global_k(rk);
  const long long kblk = any_key_block(mv, rk);
  const int key_hi_w = first_key + kg * 32 + 32;
  const long long kblk_max_w = any_key_block(mv, min(key_hi_w, a.Skv) - 1);
  const bool bias_per_key = mv.bias && mv.bias_sq == 0, bias_per_row = mv.bias && mv.bias_sq != 0;
  const bool elementwise_always = mv.keep || bias_per_row;
  const int kseg_min_w = any_wave_min(seg_k), kseg_max_w = any_wave_max(seg_k);
  float bias_k = 0.f;
  if (bias_per_key) {
    bias_k = mv.bias[(int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + gk * mv.bias_sk];
    if (mv.any_mask) bias_k = fminf(bias_k, 0.f);
  }
  const bool wave_valid = first_key + kg * 32 < a.Skv;
  const bool all_valid = key_hi_w <= a.Skv;

  AnyTr<HD> tr;
  tr.init(lane);
  int t_first = 0;
  const int ntile = (a.Sq + ANY_TILE - 1) / ANY_TILE;
  while (t_first < ntile &&
         mv.run_prefix_keys((min((t_first + 1) * ANY_TILE, a.Sq) - 1) / mv.qc, a.Skv) <= first_key) t_first++;
  AnyTileLoader<HD> ld;
  ld.init(a.q_ss, wave, lane);
  if (t_first < ntile) {
    const int q0 = t_first * ANY_TILE;
    ld.load(Qs[t_first & 1], qbase + (int64_t)q0 * a.q_ss, a.Sq - q0);
    ld.load(Gs[t_first & 1], gbase + (int64_t)q0 * a.q_ss, a.Sq - q0);
    any_stage_rows(rts[t_first & 1], a, mv, b, h, q0, tid);
  }
  uint16_t* const pw = Pt[kg] + lo * ANY_PSTR + half * 32 + hi * 4;    // this lane's key, its half of the rows
  uint16_t* const dw = Dt[kg] + lo * ANY_PSTR + half * 32 + hi * 4;
  const uint16_t* const pr = Pt[kg] + lo * ANY_PSTR + hi * 8;          // B operands: key lo, eight queries per step
  const uint16_t* const dr = Dt[kg] + lo * ANY_PSTR + hi * 8;
#pragma unroll 1
  for (int t = t_first; t < ntile; t++) {
    const int q0 = t * ANY_TILE;
    any_tile_barrier();                                // tile t is in LDS; the other buffers have been read by everyone
    if (t + 1 < ntile) {
      const int q1 = q0 + ANY_TILE;
      ld.load(Qs[(t + 1) & 1], qbase + (int64_t)q1 * a.q_ss, a.Sq - q1);
      ld.load(Gs[(t + 1) & 1], gbase + (int64_t)q1 * a.q_ss, a.Sq - q1);
      any_stage_rows(rts[(t + 1) & 1], a, mv, b, h, q1, tid);
    }
    const uint16_t* Qt = Qs[t & 1];
    const uint16_t* Gt = Gs[t & 1];
    const AnyRowTables& rt = rts[t & 1];
    // the two wavefronts of a key group decide alike: no key of the group exists, or no row of the tile shares a
    // segment id with one of them (see the forward kernel)
    const bool active = wave_valid && !(mv.seg && mv.skip_tiles && (rt.segmax < kseg_min_w || rt.segmin > kseg_max_w));
    if (active) {
      any_f32x16 S, dP;                                // rows 32 half .. + 31 of the tile x this lane's key
#pragma unroll
      for (int r = 0; r < 16; r++) { S[r] = 0.f; dP[r] = 0.f; }
      any_products_block<HD>(Qt, half * 32, kf, S, lo, hi);
      any_products_block<HD>(Gt, half * 32, vf, dP, lo, hi);
      const bool plain = !elementwise_always && all_valid && key_hi_w <= rt.kend_min &&
                         (mv.cbs <= 0 || rt.blk0 >= kblk_max_w) &&
                         (!mv.seg || (rt.segmin == rt.segmax && kseg_min_w == kseg_max_w && rt.segmin == kseg_min_w));
      if (plain) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int q4 = half * 32 + g * 8 + hi * 4;
          const any_f32x4 m4 = *(const any_f32x4*)&rt.m[q4], d4 = *(const any_f32x4*)&rt.rden[q4];
          const any_f32x4 e4 = *(const any_f32x4*)&rt.delta[q4];
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float p = __expf(fmaf(S[g * 4 + e], rscale, bias_k) - m4[e]) * d4[e];                // :226
            S[g * 4 + e] = p;
            dP[g * 4 + e] = (dP[g * 4 + e] - e4[e]) * p;                                                 // :229
          }
        }
      } else {
        const int dkey = any_rel(kblk - rt.blk0);
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qq = half * 32 + (r >> 2) * 8 + hi * 4 + (r & 3);
          float add = bias_k;
          bool masked = (mv.cbs > 0 && rt.blk[qq] < dkey) || (mv.seg && rt.seg[qq] != seg_k);
          if (bias_per_row) {
            add = mv.bias[rt.bias_off[qq] + gk * mv.bias_sk];
            if (mv.any_mask) add = fminf(add, 0.f);                     // minimum(), :299,:309
          }
          if (mv.keep) masked = masked || !mv.keep[rt.keep_off[qq] + (gk - mv.keep_k0) * mv.keep_sk];
          const float s = masked ? mv.mask_min : fmaf(S[r], rscale, add);
          const float p = (valid && kj < rt.kend[qq]) ? __expf(s - rt.m[qq]) * rt.rden[qq] : 0.f;     // :226; (:246-257)
          S[r] = p;
          dP[r] = (dP[r] - rt.delta[qq]) * p;                           // :229
          if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int g = 0; g < 4; g++) {                    // queries 32 half + 8 g + 4 hi + e of this lane's key
        const uint2 p2 = {f32x2_to_bf16x2(S[g * 4], S[g * 4 + 1]), f32x2_to_bf16x2(S[g * 4 + 2], S[g * 4 + 3])};
        const uint2 d2 = {f32x2_to_bf16x2(dP[g * 4], dP[g * 4 + 1]), f32x2_to_bf16x2(dP[g * 4 + 2], dP[g * 4 + 3])};
        *(uint2*)(pw + g * 8) = p2;
        *(uint2*)(dw + g * 8) = d2;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // P and dS of all 64 rows are in LDS
    if (active) {
      // four steps of 16 rows: dV^T += dO^T P (:232) and dK^T += Q^T dS (:231) over this wavefront's half of the head
      any_bf16x8 FG[2][NDB], FQ[2][NDB];
#pragma unroll
      for (int db = 0; db < NDB; db++) {
        FG[0][db] = tr.frag(Gt, half * NDB + db);
        FQ[0][db] = tr.frag(Qt, half * NDB + db);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int st = 0; st < 4; st++) {
        if (st + 1 < 4) {
#pragma unroll
          for (int db = 0; db < NDB; db++) {
            FG[(st + 1) & 1][db] = tr.frag(Gt + (st + 1) * 16 * HD, half * NDB + db);
            FQ[(st + 1) & 1][db] = tr.frag(Qt + (st + 1) * 16 * HD, half * NDB + db);
          }
        }
        const any_bf16x8 bp = *(const any_bf16x8*)(pr + st * 16);
        const any_bf16x8 bd = *(const any_bf16x8*)(dr + st * 16);
#pragma unroll
        for (int db = 0; db < NDB; db++) {
          acc_v[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FG[st & 1][db], bp, acc_v[db], 0, 0, 0);
          acc_k[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FQ[st & 1][db], bd, acc_k[db], 0, 0, 0);
        }
#pragma unroll
        for (int db = 0; db < 2 * NDB; db++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (st + 1 < 4) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  if (valid) {
    const int64_t off = (int64_t)h * HD + half * (HD / 2) + hi * 4;
    float* dkp = a.dk + (int64_t)b * a.dkv_sb + (int64_t)rk * a.dkv_ss + off;
    float* dvp = a.dv + (int64_t)b * a.dkv_sb + (int64_t)rk * a.dkv_ss + off;
    uint16_t* okp = (uint16_t*)a.dk_out + (int64_t)b * a.dkvo_sb + (int64_t)rk * a.dkvo_ss + off;
    uint16_t* ovp = (uint16_t*)a.dv_out + (int64_t)b * a.dkvo_sb + (int64_t)rk * a.dkvo_ss + off;
#pragma unroll
    for (int db = 0; db < NDB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        any_f32x4 k4 = {0.f, 0.f, 0.f, 0.f}, v4 = {0.f, 0.f, 0.f, 0.f};
        if (!a.dkv_initial) {
          k4 = *(const any_f32x4*)(dkp + db * 32 + g * 8);
          v4 = *(const any_f32x4*)(dvp + db * 32 + g * 8);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) { k4[e] += acc_k[db][g * 4 + e] / scale; v4[e] += acc_v[db][g * 4 + e]; }
        if (a.dk_out) {                                                 // last call for these keys (:89)
          const uint2 pk = {f32x2_to_bf16x2(k4[0], k4[1]), f32x2_to_bf16x2(k4[2], k4[3])};
          const uint2 pv = {f32x2_to_bf16x2(v4[0], v4[1]), f32x2_to_bf16x2(v4[2], v4[3])};
          *(uint2*)(okp + db * 32 + g * 8) = pk;
          *(uint2*)(ovp + db * 32 + g * 8) = pv;
        } else {
          *(any_f32x4*)(dkp + db * 32 + g * 8) = k4;
          *(any_f32x4*)(dvp + db * 32 + g * 8) = v4;
        }
      }
  }
}

// every kernel is instantiated by name: left to the launches below (some of them inside a function template) the host
// pass of the compiler has been seen to reference a kernel's launch stub without emitting it
template __global__ void attn_fwd_any_kernel<128>(GenericArgs);
template __global__ void attn_fwd_any_kernel<256>(GenericArgs);
template __global__ void attn_bwd_dq_any_kernel<128>(GenericArgs);
template __global__ void attn_bwd_dq_any_kernel<256>(GenericArgs);
template __global__ void attn_bwd_dkv_any_kernel<128, true>(GenericArgs);
template __global__ void attn_bwd_dkv_any_kernel<128, false>(GenericArgs);
template __global__ void attn_bwd_dkv_any_kernel<256, true>(GenericArgs);
template __global__ void attn_bwd_dkv_any_kernel<256, false>(GenericArgs);
template __global__ void attn_bwd_dkv_pair_any_kernel<256>(GenericArgs);

// ------------------------------------------------------------------ host side
static bool any_aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

static bool any_mask_ok(const ra_mask& m) {
  // attention dropout (its -inf bookkeeping, :321) and a boolean mask that exists in packed form only stay with the
  // kernels built for them
  return m.keep_mode != RA_KEEP_DROPOUT && !(m.keep_bits_k && !m.keep);
}

// (the tile loader keeps a lane's byte offset within a tile of 64 rows in 32 bits)
static bool any_strides_ok(int64_t q_ss, int64_t kv_ss) { return q_ss > 0 && kv_ss > 0 && q_ss < (1 << 24) && kv_ss < (1 << 24); }

bool attn_fwd_any_supported(const ra_attn_fwd_params* p) {
  return p->dtype == RA_BF16 && (p->D == 128 || p->D == 256) && any_mask_ok(p->mask) &&
         any_strides_ok(p->q_stride_s, p->kv_stride_s) &&
         p->q_stride_s % 8 == 0 && p->kv_stride_s % 8 == 0 && p->q_stride_b % 8 == 0 && p->kv_stride_b % 8 == 0 &&
         any_aligned16(p->q) && any_aligned16(p->k) && any_aligned16(p->v) &&
         (!p->numerator || (any_aligned16(p->numerator) && p->num_stride_s % 4 == 0 && p->num_stride_b % 4 == 0)) &&
         (!p->out || (any_aligned16(p->out) && p->out_stride_s % 4 == 0 && p->out_stride_b % 4 == 0)) &&
         any_aligned16(p->out_f32);
}

bool attn_bwd_any_supported(const ra_attn_bwd_params* p) {
  return p->dtype == RA_BF16 && (p->D == 128 || p->D == 256) && any_mask_ok(p->mask) &&
         any_strides_ok(p->q_stride_s, p->kv_stride_s) &&
         p->q_stride_s % 8 == 0 && p->kv_stride_s % 8 == 0 && p->q_stride_b % 8 == 0 && p->kv_stride_b % 8 == 0 &&
         any_aligned16(p->q) && any_aligned16(p->k) && any_aligned16(p->v) && any_aligned16(p->g) &&
         (!p->dq || (any_aligned16(p->dq) && p->dq_stride_s % 4 == 0 && p->dq_stride_b % 4 == 0)) &&
         (!p->dk || (any_aligned16(p->dk) && any_aligned16(p->dv) && p->dkv_stride_s % 4 == 0 && p->dkv_stride_b % 4 == 0)) &&
         (!p->dq_out || (any_aligned16(p->dq_out) && p->dq_out_stride_s % 4 == 0 && p->dq_out_stride_b % 4 == 0)) &&
         (!p->dk_out || (any_aligned16(p->dk_out) && any_aligned16(p->dv_out) && p->dkv_out_stride_s % 4 == 0 &&
                         p->dkv_out_stride_b % 4 == 0));
}

int attn_fwd_any(const ra_attn_fwd_params* p, hipStream_t s) {
  const GenericArgs a = make_args_fwd(p);
  const dim3 grid((a.Sq + ANY_ROWS - 1) / ANY_ROWS, a.H, a.B), block(ANY_THREADS);
  if (a.D == 128) attn_fwd_any_kernel<128><<<grid, block, 0, s>>>(a);
  else attn_fwd_any_kernel<256><<<grid, block, 0, s>>>(a);
  RA_CHECK_LAUNCH("attn_fwd_any");
  return RA_OK;
}

template <int HD>
static void launch_bwd_any(const GenericArgs& a, int parts, hipStream_t s) {
  const dim3 block(ANY_THREADS);
  const dim3 gq((a.Sq + ANY_ROWS - 1) / ANY_ROWS, a.H, a.B), gk((a.Skv + ANY_ROWS - 1) / ANY_ROWS, a.H, a.B);
  if (parts & RA_BWD_PART_DQ) attn_bwd_dq_any_kernel<HD><<<gq, block, 0, s>>>(a);
  if (parts & RA_BWD_PART_DKV) {
    if (HD == 256) {                                   // both gradients in one pass, a pair of wavefronts per 32 keys
      const dim3 gk2((a.Skv + 63) / 64, a.H, a.B);
      attn_bwd_dkv_pair_any_kernel<256><<<gk2, block, 0, s>>>(a);
    } else {
      attn_bwd_dkv_any_kernel<HD, true><<<gk, block, 0, s>>>(a);
      attn_bwd_dkv_any_kernel<HD, false><<<gk, block, 0, s>>>(a);
    }
  }
}

int attn_bwd_any(const ra_attn_bwd_params* p, int parts, hipStream_t s) {
  const GenericArgs a = make_args_bwd(p);
  if (a.D == 128) launch_bwd_any<128>(a, parts, s);
  else launch_bwd_any<256>(a, parts, s);
  RA_CHECK_LAUNCH("attn_bwd_any");
  return RA_OK;
}

}  // namespace ra
