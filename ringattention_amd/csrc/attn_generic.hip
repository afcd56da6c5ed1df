// Generic blockwise-attention kernels: fp32 arithmetic on the vector ALU, one
// query row (or one key row) per lane, K/V (or Q/dO) tiles broadcast from LDS.
// They accept any chunk sizes, fp32 or bf16 inputs and any supported head size,
// and evaluate the reference's mask element by element; the MFMA kernels are
// checked against them at sizes the CPU oracle cannot reach.
//
// Semantics follow ringattention_jax.py:130-145 (forward tile), :220-233
// (backward tile), :272-322 (bias / mask) and :324-331 (skip predicate).
#include "generic_args.hpp"

namespace ra {

template <typename T, int D>
__device__ __forceinline__ void stage_rows(float* dst, const T* src, int64_t stride_s, int row0, int nrows,
                                           int limit, int tid, int nthreads) {
  // dst[r*D + d] = src[(row0+r)*stride_s + d] for r < nrows, zero past limit
  for (int i = tid; i < nrows * D; i += nthreads) {
    int r = i / D, d = i % D;
    int row = row0 + r;
    dst[i] = row < limit ? load_f32<T>(src + (int64_t)row * stride_s + d) : 0.f;
  }
}

constexpr int GEN_ROWS = 64;   // rows per workgroup = one wavefront
constexpr int GEN_TK = 16;     // keys (or query rows) staged per step

// ------------------------------------------------------------------ forward
template <typename T, int D>
__global__ __launch_bounds__(GEN_ROWS) void attn_fwd_generic_kernel(GenericArgs a) {
  __shared__ float Ks[GEN_TK * D];
  __shared__ float Vs[GEN_TK * D];
  __shared__ int seg_k[GEN_TK];
  const MaskView mv = resolve_mask(a);
  const int tid = threadIdx.x, b = blockIdx.z, h = blockIdx.y;
  const int row = blockIdx.x * GEN_ROWS + tid;
  const bool valid = row < a.Sq;
  const int rrow = valid ? row : a.Sq - 1;
  const T* qp = (const T*)a.q + (int64_t)b * a.q_sb + (int64_t)rrow * a.q_ss + (int64_t)h * D;
  const T* kbase = (const T*)a.k + (int64_t)b * a.kv_sb + (int64_t)h * D;
  const T* vbase = (const T*)a.v + (int64_t)b * a.kv_sb + (int64_t)h * D;
  float* nump = a.num + (int64_t)b * a.num_sb + (int64_t)rrow * a.num_ss + (int64_t)h * D;
  const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + rrow;
  const float scale = sqrtf((float)a.sdim);                            // :118

  float q[D], acc[D];
#pragma unroll
  for (int d = 0; d < D; d++) q[d] = load_f32<T>(qp + d);
  float m = RA_NEG_INF, l = 0.f;
  if (a.carry_is_initial) {
#pragma unroll
    for (int d = 0; d < D; d++) acc[d] = 0.f;
  } else {
#pragma unroll
    for (int d = 0; d < D; d++) acc[d] = nump[d];
    m = a.mx[st]; l = a.den[st];
  }
  RowInfo ri = row_info(mv, b, h, rrow, a.Skv);
  if (!valid) ri.kend = 0;
  int kend_wg = ri.kend;
  for (int off = 32; off > 0; off >>= 1) kend_wg = max(kend_wg, __shfl_xor(kend_wg, off));

  // Under dropout a pair can hold -inf inside a key chunk that runs.  A chunk whose pairs are all -inf while the
  // running max is still -inf makes the reference compute exp(-inf - -inf) = NaN (:138-144) and the row stays NaN
  bool seen_finite = m != RA_NEG_INF, chunk_neg = true, poison = false;
  for (int k0 = 0; k0 < kend_wg; k0 += GEN_TK) {
    __syncthreads();
    stage_rows<T, D>(Ks, kbase, a.kv_ss, k0, GEN_TK, a.Skv, tid, GEN_ROWS);
    stage_rows<T, D>(Vs, vbase, a.kv_ss, k0, GEN_TK, a.Skv, tid, GEN_ROWS);
    if (tid < GEN_TK) {
      int sk = 0;
      if (mv.seg) {
        int kj = min(k0 + tid, a.Skv - 1);
        int ki = kj / mv.kc;
        int idx = clamp_seg_index(((long long)mv.k_start + ki) * mv.kc, mv.kc, mv.seg_len, kj % mv.kc);
        sk = mv.seg[(int64_t)b * mv.seg_sb + idx];
      }
      seg_k[tid] = sk;
    }
    __syncthreads();
    float s[GEN_TK];
    float tile_max = RA_NEG_INF;
#pragma unroll
    for (int j = 0; j < GEN_TK; j++) {
      float dot = 0.f;
#pragma unroll
      for (int d = 0; d < D; d++) dot = fmaf(q[d], Ks[j * D + d], dot);
      s[j] = logit(mv, ri, dot, scale, k0 + j, seg_k[j]);
      tile_max = fmaxf(tile_max, s[j]);
      if (mv.keep_drop && k0 + j < ri.kend) {
        const int in_chunk = (k0 + j) % mv.kc;
        if (in_chunk == 0) chunk_neg = true;
        chunk_neg = chunk_neg && s[j] == RA_NEG_INF;
        if (in_chunk == mv.kc - 1) {
          poison = poison || (chunk_neg && !seen_finite);
          seen_finite = seen_finite || !chunk_neg;
        }
      }
    }
    float m_new = fmaxf(m, tile_max);                             // :138
    if (m_new == RA_NEG_INF) continue;                            // nothing ran for this row yet
    float corr = (m == m_new) ? 1.f : expf(m - m_new);            // :142
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < GEN_TK; j++) { s[j] = expf(s[j] - m_new); psum += s[j]; }   // :140
#pragma unroll
    for (int d = 0; d < D; d++) {
      float t = 0.f;
#pragma unroll
      for (int j = 0; j < GEN_TK; j++) t = fmaf(s[j], Vs[j * D + d], t);           // :141
      acc[d] = acc[d] * corr + t;                                 // :143
    }
    l = l * corr + psum;                                          // :144
    m = m_new;
  }
  if (valid) {
    const float nan = poison ? __builtin_nanf("") : 0.f;
    if (a.out) {                       // last step of the device: out = numerator / denominator (:52)
      const int64_t oo = (int64_t)b * a.out_sb + (int64_t)rrow * a.out_ss + (int64_t)h * D;
      T* op = (T*)a.out + oo;
#pragma unroll
      for (int d = 0; d < D; d++) store_from_f32<T>(op + d, poison ? nan : acc[d] / l);
      if (a.out32) {                   // the residual of :53
#pragma unroll
        for (int d = 0; d < D; d++) a.out32[oo + d] = poison ? nan : acc[d] / l;
      }
    } else {
#pragma unroll
      for (int d = 0; d < D; d++) nump[d] = poison ? nan : acc[d];
    }
    a.mx[st] = m; a.den[st] = poison ? nan : l;
  }
}

// ------------------------------------------------------------------ backward, dq (one query row per lane)
template <typename T, int D>
__global__ __launch_bounds__(GEN_ROWS) void attn_bwd_dq_generic_kernel(GenericArgs a) {
  __shared__ float Ks[GEN_TK * D];
  __shared__ float Vs[GEN_TK * D];
  __shared__ int seg_k[GEN_TK];
  const MaskView mv = resolve_mask(a);
  const int tid = threadIdx.x, b = blockIdx.z, h = blockIdx.y;
  const int row = blockIdx.x * GEN_ROWS + tid;
  const bool valid = row < a.Sq;
  const int rrow = valid ? row : a.Sq - 1;
  const int64_t qoff = (int64_t)b * a.q_sb + (int64_t)rrow * a.q_ss + (int64_t)h * D;
  const T* qp = (const T*)a.q + qoff;
  const T* gp = (const T*)a.g + qoff;
  const T* kbase = (const T*)a.k + (int64_t)b * a.kv_sb + (int64_t)h * D;
  const T* vbase = (const T*)a.v + (int64_t)b * a.kv_sb + (int64_t)h * D;
  float* dqp = a.dq + (int64_t)b * a.dq_sb + (int64_t)rrow * a.dq_ss + (int64_t)h * D;
  const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + rrow;
  const float scale = sqrtf((float)a.sdim);

  float q[D], g[D], dq[D];
#pragma unroll
  for (int d = 0; d < D; d++) { q[d] = load_f32<T>(qp + d); g[d] = load_f32<T>(gp + d); dq[d] = 0.f; }
  const float m = a.mx[st], den = a.den[st], delta = a.delta[st];
  RowInfo ri = row_info(mv, b, h, rrow, a.Skv);
  if (!valid) ri.kend = 0;
  int kend_wg = ri.kend;
  for (int off = 32; off > 0; off >>= 1) kend_wg = max(kend_wg, __shfl_xor(kend_wg, off));

  for (int k0 = 0; k0 < kend_wg; k0 += GEN_TK) {
    __syncthreads();
    stage_rows<T, D>(Ks, kbase, a.kv_ss, k0, GEN_TK, a.Skv, tid, GEN_ROWS);
    stage_rows<T, D>(Vs, vbase, a.kv_ss, k0, GEN_TK, a.Skv, tid, GEN_ROWS);
    if (tid < GEN_TK) {
      int sk = 0;
      if (mv.seg) {
        int kj = min(k0 + tid, a.Skv - 1);
        int ki = kj / mv.kc;
        int idx = clamp_seg_index(((long long)mv.k_start + ki) * mv.kc, mv.kc, mv.seg_len, kj % mv.kc);
        sk = mv.seg[(int64_t)b * mv.seg_sb + idx];
      }
      seg_k[tid] = sk;
    }
    __syncthreads();
#pragma unroll 4
    for (int j = 0; j < GEN_TK; j++) {
      if (k0 + j >= ri.kend) continue;                            // tile does not run: zero contribution (:246-257)
      float dot = 0.f, dp = 0.f;
#pragma unroll
      for (int d = 0; d < D; d++) { dot = fmaf(q[d], Ks[j * D + d], dot); dp = fmaf(g[d], Vs[j * D + d], dp); }
      float s = logit(mv, ri, dot, scale, k0 + j, seg_k[j]);
      float p = expf(s - m) / den;                                // :226
      float ds = (dp - delta) * p;                                // :229
#pragma unroll
      for (int d = 0; d < D; d++) dq[d] = fmaf(ds, Ks[j * D + d], dq[d]);   // :230
    }
  }
  if (valid) {
    T* op = (T*)a.dq_out + (int64_t)b * a.dqo_sb + (int64_t)rrow * a.dqo_ss + (int64_t)h * D;
#pragma unroll
    for (int d = 0; d < D; d++) {
      const float t = (a.dq_initial ? 0.f : dqp[d]) + dq[d] / scale;
      if (a.dq_out) store_from_f32<T>(op + d, t);                  // last call for these rows (:89)
      else dqp[d] = t;
    }
  }
}

// ------------------------------------------------------------------ backward, dk or dv (one key row per lane)
template <typename T, int D, bool WANT_DK>
__global__ __launch_bounds__(GEN_ROWS) void attn_bwd_dkv_generic_kernel(GenericArgs a) {
  __shared__ float Qs[GEN_TK * D];
  __shared__ float Gs[GEN_TK * D];
  __shared__ float r_m[GEN_TK], r_den[GEN_TK], r_delta[GEN_TK];
  __shared__ RowInfo r_info[GEN_TK];
  const MaskView mv = resolve_mask(a);
  const int tid = threadIdx.x, b = blockIdx.z, h = blockIdx.y;
  const int kj = blockIdx.x * GEN_ROWS + tid;
  const bool valid = kj < a.Skv;
  const int rk = valid ? kj : a.Skv - 1;
  const int64_t koff = (int64_t)b * a.kv_sb + (int64_t)rk * a.kv_ss + (int64_t)h * D;
  const T* kp = (const T*)a.k + koff;
  const T* vp = (const T*)a.v + koff;
  const T* qbase = (const T*)a.q + (int64_t)b * a.q_sb + (int64_t)h * D;
  const T* gbase = (const T*)a.g + (int64_t)b * a.q_sb + (int64_t)h * D;
  float* outp = (WANT_DK ? a.dk : a.dv) + (int64_t)b * a.dkv_sb + (int64_t)rk * a.dkv_ss + (int64_t)h * D;
  const float scale = sqrtf((float)a.sdim);

  float k[D], v[WANT_DK ? D : 1], acc[D];
#pragma unroll
  for (int d = 0; d < D; d++) { k[d] = load_f32<T>(kp + d); acc[d] = 0.f; }
  if (WANT_DK) {
#pragma unroll
    for (int d = 0; d < D; d++) v[d] = load_f32<T>(vp + d);
  }
  int seg_k = 0;
  if (mv.seg) {
    int ki = rk / mv.kc;
    int idx = clamp_seg_index(((long long)mv.k_start + ki) * mv.kc, mv.kc, mv.seg_len, rk % mv.kc);
    seg_k = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  const int first_key = blockIdx.x * GEN_ROWS;

  for (int q0 = 0; q0 < a.Sq; q0 += GEN_TK) {
    // the run prefix grows with the query chunk: skip query tiles that end before this block's first key runs
    int last_row = min(q0 + GEN_TK, a.Sq) - 1;
    if (mv.run_prefix_keys(last_row / mv.qc, a.Skv) <= first_key) continue;
    __syncthreads();
    stage_rows<T, D>(Qs, qbase, a.q_ss, q0, GEN_TK, a.Sq, tid, GEN_ROWS);
    stage_rows<T, D>(Gs, gbase, a.q_ss, q0, GEN_TK, a.Sq, tid, GEN_ROWS);
    if (tid < GEN_TK) {
      int row = q0 + tid;
      bool rv = row < a.Sq;
      int rr = rv ? row : a.Sq - 1;
      const int64_t st = (int64_t)b * a.st_sb + (int64_t)h * a.st_sh + rr;
      r_m[tid] = a.mx[st]; r_den[tid] = a.den[st]; r_delta[tid] = a.delta[st];
      RowInfo ri = row_info(mv, b, h, rr, a.Skv);
      if (!rv) ri.kend = 0;
      r_info[tid] = ri;
    }
    __syncthreads();
#pragma unroll 2
    for (int i = 0; i < GEN_TK; i++) {
      const RowInfo ri = r_info[i];
      if (!valid || kj >= ri.kend) continue;
      float dot = 0.f, dp = 0.f;
#pragma unroll
      for (int d = 0; d < D; d++) {
        dot = fmaf(Qs[i * D + d], k[d], dot);
        if (WANT_DK) dp = fmaf(Gs[i * D + d], v[d], dp);
      }
      float s = logit(mv, ri, dot, scale, kj, seg_k);
      float p = expf(s - r_m[i]) / r_den[i];                      // :226
      if (WANT_DK) {
        float ds = (dp - r_delta[i]) * p;                         // :229
#pragma unroll
        for (int d = 0; d < D; d++) acc[d] = fmaf(ds, Qs[i * D + d], acc[d]);   // :231
      } else {
#pragma unroll
        for (int d = 0; d < D; d++) acc[d] = fmaf(p, Gs[i * D + d], acc[d]);    // :232
      }
    }
  }
  if (valid) {
    T* op = (T*)(WANT_DK ? a.dk_out : a.dv_out) + (int64_t)b * a.dkvo_sb + (int64_t)rk * a.dkvo_ss + (int64_t)h * D;
#pragma unroll
    for (int d = 0; d < D; d++) {
      const float t = (a.dkv_initial ? 0.f : outp[d]) + (WANT_DK ? acc[d] / scale : acc[d]);
      if (a.dk_out) store_from_f32<T>(op + d, t);                  // last call for these keys (:89)
      else outp[d] = t;
    }
  }
}

// ------------------------------------------------------------------ small elementwise kernels
__global__ void carry_init_kernel(float* num, int64_t num_sb, int64_t num_ss, float* den, float* mx,
                                  int64_t st_sb, int64_t st_sh, int Sq, int H, int D) {
  const int b = blockIdx.z, row = blockIdx.x;
  const int hd = H * D;
  float* np = num + (int64_t)b * num_sb + (int64_t)row * num_ss;
  for (int i = threadIdx.x; i < hd; i += blockDim.x) np[i] = 0.f;
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    int64_t st = (int64_t)b * st_sb + (int64_t)h * st_sh + row;
    den[st] = 0.f; mx[st] = RA_NEG_INF;
  }
}

template <typename TO>
__global__ void finalize_kernel(const float* num, int64_t num_sb, int64_t num_ss, const float* den,
                                int64_t st_sb, int64_t st_sh, TO* out, int64_t out_sb, int64_t out_ss,
                                int Sq, int H, int D) {
  const int b = blockIdx.z, row = blockIdx.x;
  const int hd = H * D;
  const float* np = num + (int64_t)b * num_sb + (int64_t)row * num_ss;
  TO* op = out + (int64_t)b * out_sb + (int64_t)row * out_ss;
  for (int i = threadIdx.x; i < hd; i += blockDim.x) {
    int h = i / D;
    float dn = den[(int64_t)b * st_sb + (int64_t)h * st_sh + row];
    store_from_f32<TO>(op + i, np[i] / dn);                       // :52
  }
}

template <typename T, typename TO>
__global__ void delta_kernel(const T* g, const TO* o, int64_t sb, int64_t ss, float* delta, int64_t st_sb,
                             int64_t st_sh, int Sq, int H, int D) {
  // one wavefront per (b, row, h)
  const int b = blockIdx.z, row = blockIdx.x;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, nw = blockDim.x / 64;
  for (int h = wave; h < H; h += nw) {
    const int64_t off = (int64_t)b * sb + (int64_t)row * ss + (int64_t)h * D;
    float s = 0.f;
    for (int d = lane; d < D; d += 64) s = fmaf(load_f32<T>(g + off + d), load_f32<TO>(o + off + d), s);
    for (int x = 32; x > 0; x >>= 1) s += __shfl_xor(s, x);
    if (lane == 0) delta[(int64_t)b * st_sb + (int64_t)h * st_sh + row] = s;   // :218
  }
}

// min / max segment id of every run of RA_SEG_TILE positions: one wavefront per run
__global__ void seg_tile_ranges_kernel(const int32_t* seg, int64_t seg_sb, int seg_len, int ntile, int32_t* out) {
  const int b = blockIdx.y;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / 64, lane = threadIdx.x % 64;
  if (wave >= ntile) return;
  const int pos = wave * RA_SEG_TILE + lane;
  const int v = seg[(int64_t)b * seg_sb + min(pos, seg_len - 1)];
  int mn = v, mx = v;
  for (int o = 32; o > 0; o >>= 1) { mn = min(mn, __shfl_xor(mn, o)); mx = max(mx, __shfl_xor(mx, o)); }
  if (lane == 0) { out[((int64_t)b * ntile + wave) * 2] = mn; out[((int64_t)b * ntile + wave) * 2 + 1] = mx; }
}

int seg_tile_ranges(const int32_t* seg, int64_t seg_sb, int Bseg, int seg_len, int32_t* out, hipStream_t s) {
  const int ntile = (seg_len + RA_SEG_TILE - 1) / RA_SEG_TILE;
  dim3 grid((ntile + 3) / 4, Bseg);
  seg_tile_ranges_kernel<<<grid, 256, 0, s>>>(seg, seg_sb, seg_len, ntile, out);
  RA_CHECK_LAUNCH("seg_tile_ranges");
  return RA_OK;
}

// For every run of 2 * RA_SEG_TILE positions: first and one-past-the-last tile (of all ntile) whose id range meets the
// run's.  One workgroup per run; the run's own tiles always meet it, so the hull is never empty.
__global__ __launch_bounds__(256) void seg_run_hulls_kernel(const int32_t* mm, int ntile, int nrun, int32_t* out) {
  __shared__ int hull[2];
  const int r = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int32_t* m = mm + (int64_t)b * ntile * 2;
  const int t0 = 2 * r, t1 = min(2 * r + 1, ntile - 1);
  const int lo = min(m[2 * t0], m[2 * t1]), hi = max(m[2 * t0 + 1], m[2 * t1 + 1]);
  if (tid == 0) { hull[0] = ntile; hull[1] = 0; }
  __syncthreads();
  int first = ntile, last = 0;
  for (int t = tid; t < ntile; t += 256)
    if (m[2 * t + 1] >= lo && m[2 * t] <= hi) { first = min(first, t); last = max(last, t + 1); }
  if (first < ntile) { atomicMin(&hull[0], first); atomicMax(&hull[1], last); }
  __syncthreads();
  if (tid == 0) { out[((int64_t)b * nrun + r) * 2] = hull[0]; out[((int64_t)b * nrun + r) * 2 + 1] = hull[1]; }
}

int seg_run_hulls(const int32_t* mm, int Bseg, int ntile, int32_t* out, hipStream_t s) {
  const int nrun = (ntile + 1) / 2;
  seg_run_hulls_kernel<<<dim3(nrun, Bseg), 256, 0, s>>>(mm, ntile, nrun, out);
  RA_CHECK_LAUNCH("seg_run_hulls");
  return RA_OK;
}

// One 64 x 64 tile of the boolean mask per workgroup of 64 threads: thread i writes the word of query row i
// (bits over the tile's keys) and the word of key column i (bits over the tile's query rows).
__global__ __launch_bounds__(64) void keep_pack_kernel(const uint8_t* keep, int64_t sb, int64_t sh, int64_t sq,
                                                       int64_t sk, int Hm, int Q, int K, uint64_t* bits_k,
                                                       uint64_t* bits_q, uint8_t* summary) {
  __shared__ uint8_t tile[64][65];
  __shared__ int cnt;
  const int kt = blockIdx.x, qt = blockIdx.y, plane = blockIdx.z;
  const int b = plane / Hm, h = plane % Hm;
  const int i = threadIdx.x;
  if (i == 0) cnt = 0;
  const uint8_t* base = keep + sb * b + sh * h;
  for (int r = 0; r < 64; r++) tile[r][i] = base[(int64_t)(qt * 64 + r) * sq + (int64_t)(kt * 64 + i) * sk] != 0;
  __syncthreads();
  uint64_t wrow = 0, wcol = 0;
  for (int j = 0; j < 64; j++) {
    wrow |= (uint64_t)tile[i][j] << j;
    wcol |= (uint64_t)tile[j][i] << j;
  }
  atomicAdd(&cnt, __popcll(wrow));
  __syncthreads();
  const int64_t words = (int64_t)Q * K / 64;
  bits_k[plane * words + (int64_t)kt * Q + qt * 64 + i] = wrow;
  bits_q[plane * words + (int64_t)qt * K + kt * 64 + i] = wcol;
  if (i == 0)
    summary[(int64_t)plane * (Q / 64) * (K / 64) + (int64_t)qt * (K / 64) + kt] = cnt == 0 ? 0 : (cnt == 4096 ? 2 : 1);
}

int keep_pack(const uint8_t* keep, int64_t sb, int64_t sh, int64_t sq, int64_t sk, int Bm, int Hm, int Q, int K,
              uint64_t* bits_k, uint64_t* bits_q, uint8_t* summary, hipStream_t s) {
  dim3 grid(K / 64, Q / 64, Bm * Hm);
  keep_pack_kernel<<<grid, 64, 0, s>>>(keep, sb, sh, sq, sk, Hm, Q, K, bits_k, bits_q, summary);
  RA_CHECK_LAUNCH("keep_pack");
  return RA_OK;
}

// ------------------------------------------------------------------ attention dropout mask
// Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11): ten rounds of
// two 32 x 32 -> 64 bit multiplications, the key bumped by the Weyl constants between rounds.
struct philox4 { uint32_t v[4]; };
__host__ __device__ inline philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                 uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1; c3 = (uint32_t)p0; c0 = n0; c2 = n2;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return philox4{{c0, c1, c2, c3}};
}

// Position e of the dense (B, H, Q, K) mask takes 16 bits: half-word e % 8 of Philox block e / 8 (word (e % 8) / 2, low
// half first); it is dropped iff that half-word is below threshold = floor(attn_pdrop * 2^16).
__device__ __forceinline__ uint32_t philox_keep8(int64_t blk, uint32_t k0, uint32_t k1, uint32_t threshold) {
  const philox4 r = philox4x32_10((uint32_t)blk, (uint32_t)((uint64_t)blk >> 32), 0u, 0u, k0, k1);
  uint32_t bits = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    bits |= ((r.v[j] & 0xFFFFu) >= threshold ? 1u : 0u) << (2 * j);
    bits |= ((r.v[j] >> 16) >= threshold ? 1u : 0u) << (2 * j + 1);
  }
  return bits;      // bit i: position 8 blk + i is kept
}

// byte form: one thread per 16 positions (two blocks)
__global__ __launch_bounds__(256) void dropout_keep_kernel(uint32_t k0, uint32_t k1, uint32_t threshold,
                                                           int64_t nblocks, uint2* keep8) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int64_t blk = 2 * t + j;
    if (blk >= nblocks) return;
    const uint32_t bits = philox_keep8(blk, k0, k1, threshold);
    uint2 w;
    w.x = (bits & 1u) | ((bits >> 1 & 1u) << 8) | ((bits >> 2 & 1u) << 16) | ((bits >> 3 & 1u) << 24);
    w.y = (bits >> 4 & 1u) | ((bits >> 5 & 1u) << 8) | ((bits >> 6 & 1u) << 16) | ((bits >> 7 & 1u) << 24);
    keep8[blk] = w;
  }
}

int dropout_keep(uint64_t seed, uint32_t threshold, int64_t n, uint8_t* keep, hipStream_t s) {
  const int64_t nblocks = n / 8, nthreads = (nblocks + 1) / 2;
  dropout_keep_kernel<<<(unsigned)((nthreads + 255) / 256), 256, 0, s>>>((uint32_t)seed, (uint32_t)(seed >> 32),
                                                                        threshold, nblocks, (uint2*)keep);
  RA_CHECK_LAUNCH("dropout_keep");
  return RA_OK;
}

// packed form, the same bits: one 64 x 64 tile per wavefront, lane i draws the 64 positions of query row i (eight
// blocks) and the columns' words come from 64 ballots.  Writes what keep_pack_kernel would write for the byte form.
__global__ __launch_bounds__(64) void dropout_keep_packed_kernel(uint32_t k0, uint32_t k1, uint32_t threshold, int Q,
                                                                 int K, uint64_t* bits_k, uint64_t* bits_q,
                                                                 uint8_t* summary, MaskView run) {
  const int kt = blockIdx.x, qt = blockIdx.y, plane = blockIdx.z, i = threadIdx.x;
  // under a causal block size only the chunk pairs that run (:324-331) are ever read: leave the other tiles alone.
  // (The chunk of the tile's last row runs the longest key prefix of the tile's rows.)
  if (run.cbs > 0 && kt * 64 >= run.run_prefix_keys((qt * 64 + 63) / run.qc, K)) return;
  const int64_t e0 = ((int64_t)plane * Q + qt * 64 + i) * K + (int64_t)kt * 64;
  uint64_t wrow = 0;
#pragma unroll
  for (int j = 0; j < 8; j++) wrow |= (uint64_t)philox_keep8(e0 / 8 + j, k0, k1, threshold) << (8 * j);
  uint64_t wcol = 0;
  for (int j = 0; j < 64; j++) {
    const unsigned long long m = __builtin_amdgcn_ballot_w64((wrow >> j) & 1);
    if (i == j) wcol = m;
  }
  int cnt = __popcll(wrow);
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off);
  const int64_t words = (int64_t)Q * K / 64;
  bits_k[plane * words + (int64_t)kt * Q + qt * 64 + i] = wrow;
  bits_q[plane * words + (int64_t)qt * K + kt * 64 + i] = wcol;
  if (i == 0)
    summary[(int64_t)plane * (Q / 64) * (K / 64) + (int64_t)qt * (K / 64) + kt] = cnt == 0 ? 0 : (cnt == 4096 ? 2 : 1);
}

int dropout_keep_packed(uint64_t seed, uint32_t threshold, int planes, int Q, int K, uint64_t* bits_k,
                        uint64_t* bits_q, uint8_t* summary, int cbs, int qc, int kc, int q_start, int k_start,
                        hipStream_t s) {
  dim3 grid(K / 64, Q / 64, planes);
  MaskView run{};
  run.cbs = cbs; run.qc = qc; run.kc = kc; run.q_start = q_start; run.k_start = k_start;
  dropout_keep_packed_kernel<<<grid, 64, 0, s>>>((uint32_t)seed, (uint32_t)(seed >> 32), threshold, Q, K, bits_k,
                                                 bits_q, summary, run);
  RA_CHECK_LAUNCH("dropout_keep_packed");
  return RA_OK;
}

// ------------------------------------------------------------------ host-side launchers
template <typename T>
static int launch_fwd_T(const GenericArgs& a, hipStream_t s) {
  dim3 grid((a.Sq + GEN_ROWS - 1) / GEN_ROWS, a.H, a.B), block(GEN_ROWS);
  switch (a.D) {
    case 32: attn_fwd_generic_kernel<T, 32><<<grid, block, 0, s>>>(a); break;
    case 64: attn_fwd_generic_kernel<T, 64><<<grid, block, 0, s>>>(a); break;
    case 128: attn_fwd_generic_kernel<T, 128><<<grid, block, 0, s>>>(a); break;
    case 256: attn_fwd_generic_kernel<T, 256><<<grid, block, 0, s>>>(a); break;      // row vectors partly in scratch memory
    default: set_error("generic attention: head size %d not in {32,64,128,256}", a.D); return RA_ERR_UNSUPPORTED;
  }
  RA_CHECK_LAUNCH("attn_fwd_generic");
  return RA_OK;
}

int attn_fwd_generic(const ra_attn_fwd_params* p, hipStream_t s) {
  GenericArgs a = make_args_fwd(p);
  return p->dtype == RA_F32 ? launch_fwd_T<float>(a, s) : launch_fwd_T<uint16_t>(a, s);
}

template <typename T, int D>
static void launch_bwd_TD(const GenericArgs& a, hipStream_t s) {
  dim3 block(GEN_ROWS);
  dim3 gq((a.Sq + GEN_ROWS - 1) / GEN_ROWS, a.H, a.B), gk((a.Skv + GEN_ROWS - 1) / GEN_ROWS, a.H, a.B);
  attn_bwd_dq_generic_kernel<T, D><<<gq, block, 0, s>>>(a);
  attn_bwd_dkv_generic_kernel<T, D, true><<<gk, block, 0, s>>>(a);
  attn_bwd_dkv_generic_kernel<T, D, false><<<gk, block, 0, s>>>(a);
}

template <typename T>
static int launch_bwd_T(const GenericArgs& a, hipStream_t s) {
  switch (a.D) {
    case 32: launch_bwd_TD<T, 32>(a, s); break;
    case 64: launch_bwd_TD<T, 64>(a, s); break;
    case 128: launch_bwd_TD<T, 128>(a, s); break;
    case 256: launch_bwd_TD<T, 256>(a, s); break;
    default: set_error("generic attention: head size %d not in {32,64,128,256}", a.D); return RA_ERR_UNSUPPORTED;
  }
  RA_CHECK_LAUNCH("attn_bwd_generic");
  return RA_OK;
}

int attn_bwd_generic(const ra_attn_bwd_params* p, hipStream_t s) {
  GenericArgs a = make_args_bwd(p);
  return p->dtype == RA_F32 ? launch_bwd_T<float>(a, s) : launch_bwd_T<uint16_t>(a, s);
}

int carry_init(float* num, int64_t num_sb, int64_t num_ss, float* den, float* mx, int64_t st_sb, int64_t st_sh,
               int B, int Sq, int H, int D, hipStream_t s) {
  dim3 grid(Sq, 1, B);
  carry_init_kernel<<<grid, 256, 0, s>>>(num, num_sb, num_ss, den, mx, st_sb, st_sh, Sq, H, D);
  RA_CHECK_LAUNCH("carry_init");
  return RA_OK;
}

int finalize(const float* num, int64_t num_sb, int64_t num_ss, const float* den, int64_t st_sb, int64_t st_sh,
             void* out, int out_dtype, int64_t out_sb, int64_t out_ss, int B, int Sq, int H, int D,
             hipStream_t s) {
  dim3 grid(Sq, 1, B);
  if (out_dtype == RA_F32)
    finalize_kernel<float><<<grid, 256, 0, s>>>(num, num_sb, num_ss, den, st_sb, st_sh, (float*)out, out_sb,
                                               out_ss, Sq, H, D);
  else
    finalize_kernel<uint16_t><<<grid, 256, 0, s>>>(num, num_sb, num_ss, den, st_sb, st_sh, (uint16_t*)out,
                                                  out_sb, out_ss, Sq, H, D);
  RA_CHECK_LAUNCH("finalize");
  return RA_OK;
}

int bwd_delta(const void* g, const void* o, int dtype, int out_dtype, int64_t sb, int64_t ss, float* delta,
              int64_t st_sb, int64_t st_sh, int B, int Sq, int H, int D, hipStream_t s) {
  dim3 grid(Sq, 1, B);
  if (dtype == RA_F32)
    delta_kernel<float, float><<<grid, 256, 0, s>>>((const float*)g, (const float*)o, sb, ss, delta, st_sb, st_sh,
                                                   Sq, H, D);
  else if (out_dtype == RA_F32)
    delta_kernel<uint16_t, float><<<grid, 256, 0, s>>>((const uint16_t*)g, (const float*)o, sb, ss, delta, st_sb,
                                                      st_sh, Sq, H, D);
  else
    delta_kernel<uint16_t, uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)g, (const uint16_t*)o, sb, ss, delta,
                                                         st_sb, st_sh, Sq, H, D);
  RA_CHECK_LAUNCH("bwd_delta");
  return RA_OK;
}

}  // namespace ra
