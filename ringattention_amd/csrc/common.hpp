// Shared host/device helpers for the ring-attention HIP kernels (gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>
#include "../../include/ringattn_hip.h"

#define RA_NEG_INF (-__builtin_inff())

namespace ra {

void set_error(const char* fmt, ...);

#define RA_REQUIRE(cond, code, ...)            \
  do {                                         \
    if (!(cond)) {                             \
      ra::set_error(__VA_ARGS__);              \
      return (code);                           \
    }                                          \
  } while (0)

#define RA_CHECK_LAUNCH(name)                                              \
  do {                                                                     \
    hipError_t e_ = hipGetLastError();                                     \
    if (e_ != hipSuccess) {                                                \
      ra::set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return RA_ERR_LAUNCH;                                                \
    }                                                                      \
  } while (0)

// ---------------------------------------------------------------- bf16 <-> fp32
__device__ __forceinline__ float bf16_to_f32(uint16_t x) { return __uint_as_float(((uint32_t)x) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {  // round to nearest even, NaN kept: v_cvt_pk_bf16_f32
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {  // lo in bits 0..15
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  bf16x2_t v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}
template <typename T> __device__ __forceinline__ float load_f32(const T* p);
template <> __device__ __forceinline__ float load_f32<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_f32<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ __forceinline__ void store_from_f32(T* p, float v);
template <> __device__ __forceinline__ void store_from_f32<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_from_f32<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }

// ---------------------------------------------------------------- mask arithmetic
// Device-side view of ra_mask with the chunk arithmetic of below_or_on_diag
// (ringattention_jax.py:324-331) folded into "how many keys of this shard run
// for a query chunk": the predicate is monotone in the key chunk index, so the
// chunks that run are a prefix.
struct MaskView {
  const float* bias;
  int64_t bias_sb, bias_sh, bias_sq, bias_sk;
  const int32_t* seg;
  int64_t seg_sb;
  int seg_len;
  int cbs, qc, kc;
  int q_start, k_start;   // global chunk indices of local chunk 0
  float mask_min;
  int any_mask;
  int skip_tiles;
  const int32_t* seg_mm;   // per-64-position (min, max) segment ids, or null
  int seg_tiles;
  const int32_t* seg_hull; // per-128-position [first, last) 64-position tile whose id range meets the run's, or null
  int seg_runs;
  const uint8_t* keep;     // boolean mask (local query row, global key - keep_k0), or null
  int64_t keep_sb, keep_sh, keep_sq, keep_sk;
  const uint64_t* kbits_k;   // packed mask, see ra_keep_pack; all null unless the MFMA kernels take the mask
  const uint64_t* kbits_q;
  const uint8_t* ksum;
  int64_t kpack_sb, kpack_sh, ksum_sb, ksum_sh;
  int keep_Q, keep_K, keep_q0, keep_k0;
  int keep_drop;           // 1: dropout semantics (mask_min added: a pair masked twice becomes -inf)
  const int32_t* cache_idx;     // nullable device scalar (ringattention_jax.py:35)
  const int32_t* chunk_starts;  // nullable device pair (q_chunk_idx_start, k_chunk_idx_start) (:31-37, :69-75)

  __host__ __device__ static MaskView make(const ra_mask& m, int q_chunk_idx_start) {
    MaskView v;
    v.bias = m.bias; v.bias_sb = m.bias_stride_b; v.bias_sh = m.bias_stride_h;
    v.bias_sq = m.bias_stride_q; v.bias_sk = m.bias_stride_k;
    v.seg = m.segment_ids; v.seg_sb = m.seg_stride_b; v.seg_len = m.seg_len;
    v.cbs = m.causal_block_size; v.qc = m.query_chunk_size; v.kc = m.key_chunk_size;
    v.q_start = q_chunk_idx_start; v.k_start = m.k_chunk_idx_start;
    v.mask_min = m.mask_min;
    v.any_mask = (m.segment_ids != nullptr) || (m.causal_block_size > 0);
    v.skip_tiles = m.skip_masked_tiles;
    v.seg_mm = m.seg_tile_minmax; v.seg_tiles = m.seg_tiles;
    v.seg_hull = m.seg_run_hulls; v.seg_runs = m.seg_runs;
    v.keep = m.keep; v.keep_sb = m.keep_stride_b; v.keep_sh = m.keep_stride_h;
    v.keep_sq = m.keep_stride_q; v.keep_sk = m.keep_stride_k;
    v.kbits_k = m.keep_bits_k; v.kbits_q = m.keep_bits_q; v.ksum = m.keep_summary;
    v.kpack_sb = m.keep_pack_stride_b; v.kpack_sh = m.keep_pack_stride_h;
    v.ksum_sb = m.keep_sum_stride_b; v.ksum_sh = m.keep_sum_stride_h;
    v.keep_Q = m.keep_q_total; v.keep_K = m.keep_k_total; v.keep_q0 = m.keep_q0;
    v.keep_k0 = m.keep_k0; v.keep_drop = m.keep_mode == RA_KEEP_DROPOUT;
    v.cache_idx = m.cache_idx; v.chunk_starts = m.chunk_starts;
    return v;
  }

  // The chunk starts a kernel works with: the host ints of ra_mask unless the caller left them in device memory -
  // under jit lax.axis_index and cache_idx are traced values (:31-37), which a custom call receives as buffers.
  // Every thread of a kernel calls this first (uniform loads).
  __device__ __forceinline__ void resolve() {
    if (chunk_starts) { q_start = chunk_starts[0]; k_start = chunk_starts[1]; }
    if (cache_idx) q_start = *cache_idx / qc;                        // :35
  }

  // Number of leading local keys (out of skv) whose chunk runs against local query chunk qi.
  __host__ __device__ int run_prefix_keys(int qi, int skv) const {
    if (cbs <= 0) return skv;
    long long cq = cbs > qc ? cbs : qc;
    long long ck = cbs > kc ? cbs : kc;
    long long r = ((long long)q_start + qi) / (cq / qc);
    long long x = (r + 1) * cq - 1;          // run iff x > c' * ck  with c' = c / (ck / kc)
    if (x <= 0) return 0;
    long long cmax = (x - 1) / ck;           // largest c' that runs
    long long climit = (cmax + 1) * (ck / kc);   // global key chunks [0, climit) run
    long long nloc = climit - k_start;
    if (nloc <= 0) return 0;
    long long keys = nloc * kc;
    return keys > skv ? skv : (int)keys;
  }
  __host__ __device__ long long global_q(int local_row) const { return (long long)q_start * qc + local_row; }
  __host__ __device__ long long global_k(int local_col) const { return (long long)k_start * kc + local_col; }
};

__device__ __forceinline__ int clamp_seg_index(long long chunk_offset, int chunk, int seg_len, int within) {
  // lax.dynamic_slice clamps the slice start (ringattention_jax.py:286-295)
  long long s = chunk_offset;
  long long hi = (long long)seg_len - chunk;
  if (s > hi) s = hi;
  if (s < 0) s = 0;
  long long i = s + within;
  if (i >= seg_len) i = seg_len - 1;
  return (int)i;
}

// Hull [first, last+1) of the 64-position tiles, among the n tiles starting at global tile gt0, whose
// segment-id range meets [lo, hi] (ids from ra_segment_tile_ranges).  Conservative: a tile outside the
// hull holds no key (query) of a segment present in the rows at hand; tiles inside may still be fully
// masked.  Every thread of the workgroup must call it; hull2 points at two ints of LDS.
__device__ __forceinline__ void seg_tile_hull(const MaskView& mv, int b, int gt0, int n, int lo, int hi, int* hull2,
                                              int tid, int nthreads, int& first, int& last) {
  if (tid == 0) { hull2[0] = n; hull2[1] = 0; }
  __syncthreads();
  const int32_t* mm = mv.seg_mm + (int64_t)(mv.seg_sb ? b : 0) * mv.seg_tiles * 2;
  for (int t = tid; t < n; t += nthreads) {
    const int g = min(gt0 + t, mv.seg_tiles - 1);
    const int mn = mm[2 * g], mx = mm[2 * g + 1];
    if (mx >= lo && mn <= hi) { atomicMin(&hull2[0], t); atomicMax(&hull2[1], t + 1); }
  }
  __syncthreads();
  first = hull2[0]; last = hull2[1];
  if (last < first) { first = 0; last = 0; }
}
// segment-id range of the rows [g0, g0 + rows) (global positions, multiples of 64)
__device__ __forceinline__ void seg_rows_range(const MaskView& mv, int b, int g0, int rows, int& lo, int& hi) {
  const int32_t* mm = mv.seg_mm + (int64_t)(mv.seg_sb ? b : 0) * mv.seg_tiles * 2;
  lo = 0x7fffffff; hi = -0x7fffffff - 1;
  for (int t = g0 / RA_SEG_TILE; t < (g0 + rows) / RA_SEG_TILE; t++) {
    const int g = min(t, mv.seg_tiles - 1);
    lo = min(lo, mm[2 * g]); hi = max(hi, mm[2 * g + 1]);
  }
}

// The two calls above for the rows [g_rows0, g_rows0 + rows): the hull, among the n tiles starting at global tile gt0,
// of the tiles that can hold a position of one of the rows' segments.  With the table of ra_segment_run_hulls (one
// entry per run of 128 positions, over ALL tiles of the sequence) this is two loads and an intersection instead of a
// scan with two barriers - the table's hull can only be wider than the scan's (tiles between two meeting ones), which
// adds fully masked tiles and changes no result.  Every thread of the workgroup must call it.
__device__ __forceinline__ void seg_hull_of_rows(const MaskView& mv, int b, int g_rows0, int rows, int gt0, int n,
                                                 int* hull2, int tid, int nthreads, int& first, int& last) {
  if (mv.seg_hull && rows == 2 * RA_SEG_TILE && (g_rows0 % (2 * RA_SEG_TILE)) == 0) {
    const int r = min(g_rows0 / (2 * RA_SEG_TILE), mv.seg_runs - 1);
    const int32_t* h = mv.seg_hull + ((int64_t)(mv.seg_sb ? b : 0) * mv.seg_runs + r) * 2;
    first = max(h[0] - gt0, 0);
    last = min(h[1] - gt0, n);
    if (last <= first) { first = 0; last = 0; }
    return;
  }
  int lo, hi;
  seg_rows_range(mv, b, g_rows0, rows, lo, hi);
  seg_tile_hull(mv, b, gt0, n, lo, hi, hull2, tid, nthreads, first, last);
}

// ---- boolean keep mask in packed form (ra_keep_pack): 64-bit words and a per-64x64-tile summary
// (0 none kept, 1 mixed, 2 all kept).  Hull of the key tiles [gkt0, gkt0 + n) that hold a kept pair for
// any of the nrows summary rows starting at qt64 (every thread of the workgroup must call it).
__device__ __forceinline__ void keep_ktile_hull(const MaskView& mv, int b, int h, int qt64, int nrows, int gkt0, int n,
                                                int* hull2, int tid, int nthreads, int& first, int& last) {
  if (tid == 0) { hull2[0] = n; hull2[1] = 0; }
  __syncthreads();
  const int KT = mv.keep_K / 64;
  const uint8_t* sm = mv.ksum + (int64_t)b * mv.ksum_sb + (int64_t)h * mv.ksum_sh + (int64_t)qt64 * KT + gkt0;
  for (int t = tid; t < n; t += nthreads) {
    int any = 0;
    for (int r = 0; r < nrows; r++) any |= sm[(int64_t)r * KT + t];
    if (any) { atomicMin(&hull2[0], t); atomicMax(&hull2[1], t + 1); }
  }
  __syncthreads();
  first = hull2[0]; last = hull2[1];
  if (last < first) { first = 0; last = 0; }
}
// the same over the query tiles [gqt0, gqt0 + n) for the ncols summary columns starting at kt64
__device__ __forceinline__ void keep_qtile_hull(const MaskView& mv, int b, int h, int kt64, int ncols, int gqt0, int n,
                                                int* hull2, int tid, int nthreads, int& first, int& last) {
  if (tid == 0) { hull2[0] = n; hull2[1] = 0; }
  __syncthreads();
  const int KT = mv.keep_K / 64;
  const uint8_t* sm = mv.ksum + (int64_t)b * mv.ksum_sb + (int64_t)h * mv.ksum_sh + (int64_t)gqt0 * KT + kt64;
  for (int t = tid; t < n; t += nthreads) {
    int any = 0;
    for (int cidx = 0; cidx < ncols; cidx++) any |= sm[(int64_t)t * KT + cidx];
    if (any) { atomicMin(&hull2[0], t); atomicMax(&hull2[1], t + 1); }
  }
  __syncthreads();
  first = hull2[0]; last = hull2[1];
  if (last < first) { first = 0; last = 0; }
}

}  // namespace ra
