// The steps a model runs either side of the hot path, as bandwidth-bound kernels:
//   rope_kv_append   before a decode step: rotary position embedding of the new token's query and key at
//                    position cache_idx, and the write of the new key / value into the cache buffers that
//                    ringattention(..., cache_idx) then streams (ringattention_jax.py:31-35 reads them whole);
//   rmsnorm_residual around blockwise_feedforward (ringattention_jax.py:333-352): y = x + r, n = y * rstd * w,
//                    forward and backward.
// The reference repository holds neither (its README points at the LWM model code for them); the formulas are the
// LLaMA ones and are restated by the CPU oracle.
#include "common.hpp"

namespace ra {

// ------------------------------------------------------------------ rotary embedding + cache append
struct RopeArgs {
  const void* q; void* q_out; const void* k_new; const void* v_new; void* k_cache; void* v_cache;
  const int32_t* cache_idx; int cache_idx_host;
  int B, L, H, D;
  int64_t q_sb, qo_sb, new_sb, c_sb, c_ss;
  double log2_theta;      // <= 0: no rotation
  int style;              // 0: pairs (2j, 2j+1); 1: pairs (j, j + D/2)
};

// one thread per (batch row, head, pair of rotated elements).  The angle pos * theta^(-2j/D) grows to 1e5 rad and
// more at long contexts: it and its sine / cosine are taken in double, the rotation itself in fp32.
template <typename T>
__global__ void rope_kv_append_kernel(RopeArgs a) {
  const int half = a.D / 2;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)a.B * a.H * half) return;
  const int j = (int)(idx % half);
  const int h = (int)((idx / half) % a.H);
  const int b = (int)(idx / ((int64_t)half * a.H));
  const int pos = a.cache_idx ? *a.cache_idx : a.cache_idx_host;
  if (pos < 0 || pos >= a.L) return;              // a position outside the buffer is not written
  const int e0 = a.style == 0 ? 2 * j : j, e1 = a.style == 0 ? 2 * j + 1 : j + half;
  float cs = 1.f, sn = 0.f;
  if (a.log2_theta > 0.0) {
    const double ang = (double)pos * exp2(-(2.0 * j / a.D) * a.log2_theta);
    double sd, cd;
    sincos(ang, &sd, &cd);
    cs = (float)cd; sn = (float)sd;
  }
  const int64_t hd = (int64_t)h * a.D;
  const T* qp = (const T*)a.q + b * a.q_sb + hd;
  const T* kp = (const T*)a.k_new + b * a.new_sb + hd;
  const T* vp = (const T*)a.v_new + b * a.new_sb + hd;
  T* qo = (T*)a.q_out + b * a.qo_sb + hd;
  T* kc = (T*)a.k_cache + b * a.c_sb + (int64_t)pos * a.c_ss + hd;
  T* vc = (T*)a.v_cache + b * a.c_sb + (int64_t)pos * a.c_ss + hd;
  const float q0 = load_f32(qp + e0), q1 = load_f32(qp + e1);
  const float k0 = load_f32(kp + e0), k1 = load_f32(kp + e1);
  store_from_f32(qo + e0, q0 * cs - q1 * sn);
  store_from_f32(qo + e1, q0 * sn + q1 * cs);
  store_from_f32(kc + e0, k0 * cs - k1 * sn);
  store_from_f32(kc + e1, k0 * sn + k1 * cs);
  vc[e0] = vp[e0];
  vc[e1] = vp[e1];
}

int rope_kv_append(const ra_rope_append_params* p, hipStream_t s) {
  RopeArgs a{};
  a.q = p->q; a.q_out = p->q_out; a.k_new = p->k_new; a.v_new = p->v_new; a.k_cache = p->k_cache; a.v_cache = p->v_cache;
  a.cache_idx = p->cache_idx; a.cache_idx_host = p->cache_idx_host;
  a.B = p->B; a.L = p->L; a.H = p->H; a.D = p->D;
  a.q_sb = p->q_stride_b; a.qo_sb = p->q_out_stride_b; a.new_sb = p->new_stride_b;
  a.c_sb = p->cache_stride_b; a.c_ss = p->cache_stride_s;
  a.log2_theta = p->rope_theta > 0.f ? log2((double)p->rope_theta) : 0.0;
  a.style = p->rope_style;
  const int64_t n = (int64_t)p->B * p->H * (p->D / 2);
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (p->dtype == RA_BF16) rope_kv_append_kernel<uint16_t><<<blocks, 256, 0, s>>>(a);
  else rope_kv_append_kernel<float><<<blocks, 256, 0, s>>>(a);
  RA_CHECK_LAUNCH("rope_kv_append");
  return RA_OK;
}

// ------------------------------------------------------------------ residual add + RMSNorm
// One workgroup of 256 threads per row; a thread owns 16-byte slices (8 bf16) of the row at stride 256 * 8.
constexpr int RMS_THREADS = 256;
constexpr int RMS_MAX_D = RMS_THREADS * 8 * 4;     // up to four slices per thread: rows of up to 8192 elements

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  v = red[0] + red[1] + red[2] + red[3];
  __syncthreads();
  return v;
}

__device__ __forceinline__ void unpack8(const uint4& u, float* o) {
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int i = 0; i < 4; i++) { o[2 * i] = __uint_as_float(w[i] << 16); o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
}
__device__ __forceinline__ uint4 pack8(const float* v) {
  uint4 u;
  u.x = f32x2_to_bf16x2(v[0], v[1]); u.y = f32x2_to_bf16x2(v[2], v[3]);
  u.z = f32x2_to_bf16x2(v[4], v[5]); u.w = f32x2_to_bf16x2(v[6], v[7]);
  return u;
}

// y = x (+ r), rstd = rsqrt(mean(y^2) + eps), n = y * rstd * w.  y is written only when r is given.
template <int NS>
__global__ __launch_bounds__(RMS_THREADS) void rmsnorm_fwd_kernel(const uint16_t* x, const uint16_t* r, const uint16_t* w,
                                                                  uint16_t* y, uint16_t* n, float* rstd, int d, float eps) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  // d is a multiple of 8 and at most NS * 2048; the last slice may be partial
  float v[NS][8];
  float ss = 0.f;
#pragma unroll
  for (int s = 0; s < NS; s++) {
    if ((s * RMS_THREADS + (int)threadIdx.x) * 8 < d) {
      const int64_t o = row * d + (int64_t)(s * RMS_THREADS + threadIdx.x) * 8;
      unpack8(*(const uint4*)(x + o), v[s]);
      if (r) {
        float rv[8];
        unpack8(*(const uint4*)(r + o), rv);
#pragma unroll
        for (int e = 0; e < 8; e++) v[s][e] += rv[e];
        const uint4 yy = pack8(v[s]);
        *(uint4*)(y + o) = yy;
        unpack8(yy, v[s]);                    // the norm is taken of the residual stream as it is stored (bf16)
      }
#pragma unroll
      for (int e = 0; e < 8; e++) ss += v[s][e] * v[s][e];
    }
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / d + eps);
  if (threadIdx.x == 0) rstd[row] = inv;
#pragma unroll
  for (int s = 0; s < NS; s++) {
    if ((s * RMS_THREADS + (int)threadIdx.x) * 8 < d) {
      const int c = (s * RMS_THREADS + threadIdx.x) * 8;
      float wv[8], o8[8];
      unpack8(*(const uint4*)(w + c), wv);
#pragma unroll
      for (int e = 0; e < 8; e++) o8[e] = v[s][e] * inv * wv[e];
      *(uint4*)(n + row * d + c) = pack8(o8);
    }
  }
}

// dy = rstd * (dn * w) - y * rstd^3 / d * sum(dn * w * y) (+ dres);  dw partial of this workgroup's rows into
// dw_part[workgroup][d] (summed by rmsnorm_dw_reduce_kernel: deterministic, no atomics).
template <int NS>
__global__ __launch_bounds__(RMS_THREADS) void rmsnorm_bwd_kernel(const uint16_t* dn, const uint16_t* y, const uint16_t* w,
                                                                  const float* rstd, const uint16_t* dres, uint16_t* dy,
                                                                  float* dw_part, int64_t T, int d, int rows_per_wg) {
  __shared__ float red[4];
  float wv[NS][8], dwv[NS][8];
#pragma unroll
  for (int s = 0; s < NS; s++) {
    if ((s * RMS_THREADS + (int)threadIdx.x) * 8 < d) {
      unpack8(*(const uint4*)(w + (s * RMS_THREADS + threadIdx.x) * 8), wv[s]);
#pragma unroll
      for (int e = 0; e < 8; e++) dwv[s][e] = 0.f;
    }
  }
  const int64_t row0 = (int64_t)blockIdx.x * rows_per_wg;
  for (int64_t row = row0; row < min(T, row0 + rows_per_wg); row++) {
    const float inv = rstd[row];
    float g[NS][8], yv[NS][8];
    float dot = 0.f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
      if ((s * RMS_THREADS + (int)threadIdx.x) * 8 < d) {
        const int64_t o = row * d + (int64_t)(s * RMS_THREADS + threadIdx.x) * 8;
        unpack8(*(const uint4*)(dn + o), g[s]);
        unpack8(*(const uint4*)(y + o), yv[s]);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          dwv[s][e] += g[s][e] * yv[s][e] * inv;
          g[s][e] *= wv[s][e];
          dot += g[s][e] * yv[s][e];
        }
      }
    }
    dot = block_sum(dot, red);
    const float k3 = inv * inv * inv * dot / d;
#pragma unroll
    for (int s = 0; s < NS; s++) {
      if ((s * RMS_THREADS + (int)threadIdx.x) * 8 < d) {
        const int64_t o = row * d + (int64_t)(s * RMS_THREADS + threadIdx.x) * 8;
        float o8[8];
#pragma unroll
        for (int e = 0; e < 8; e++) o8[e] = g[s][e] * inv - yv[s][e] * k3;
        if (dres) {
          float rv[8];
          unpack8(*(const uint4*)(dres + o), rv);
#pragma unroll
          for (int e = 0; e < 8; e++) o8[e] += rv[e];
        }
        *(uint4*)(dy + o) = pack8(o8);
      }
    }
  }
#pragma unroll
  for (int s = 0; s < NS; s++) {
    if ((s * RMS_THREADS + (int)threadIdx.x) * 8 < d) {
      float* p = dw_part + (int64_t)blockIdx.x * d + (s * RMS_THREADS + threadIdx.x) * 8;
      *(float4*)p = make_float4(dwv[s][0], dwv[s][1], dwv[s][2], dwv[s][3]);
      *(float4*)(p + 4) = make_float4(dwv[s][4], dwv[s][5], dwv[s][6], dwv[s][7]);
    }
  }
}

// dw[c] += sum over parts of dw_part[part][c]: a workgroup owns 32 columns, eight threads per column take every
// eighth part (independent loads, 128-byte rows), LDS adds the eight partial sums in a fixed order.
__global__ __launch_bounds__(256) void rmsnorm_dw_reduce_kernel(const float* dw_part, float* dw, int nparts, int d) {
  __shared__ float part[8][32];
  const int cl = threadIdx.x & 31, pl = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + cl;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (c < d) {
    int p = pl;
    for (; p + 24 < nparts; p += 32) {
      s0 += dw_part[(int64_t)p * d + c];
      s1 += dw_part[(int64_t)(p + 8) * d + c];
      s2 += dw_part[(int64_t)(p + 16) * d + c];
      s3 += dw_part[(int64_t)(p + 24) * d + c];
    }
    for (; p < nparts; p += 8) s0 += dw_part[(int64_t)p * d + c];
  }
  part[pl][cl] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (pl == 0 && c < d) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) s += part[i][cl];
    dw[c] += s;
  }
}

int rmsnorm_bwd_parts(int64_t T) {
  // enough workgroups to fill the GPU several times over, few enough for a short reduction
  const int64_t parts = (T + 15) / 16;
  return (int)(parts < 1 ? 1 : parts > 4096 ? 4096 : parts);
}

#define RA_RMS_DISPATCH(KERNEL, GRID, ...)                                                               \
  {                                                                                                     \
    const int ns_ = (p->d + RMS_THREADS * 8 - 1) / (RMS_THREADS * 8);                                    \
    if (ns_ <= 1) KERNEL<1><<<GRID, RMS_THREADS, 0, s>>>(__VA_ARGS__);                                   \
    else if (ns_ <= 2) KERNEL<2><<<GRID, RMS_THREADS, 0, s>>>(__VA_ARGS__);                              \
    else KERNEL<4><<<GRID, RMS_THREADS, 0, s>>>(__VA_ARGS__);                                            \
  }

int rmsnorm_max_d() { return RMS_MAX_D; }

int rmsnorm_fwd(const ra_rmsnorm_params* p, hipStream_t s) {
  RA_RMS_DISPATCH(rmsnorm_fwd_kernel, (unsigned)p->T, (const uint16_t*)p->x, (const uint16_t*)p->residual,
                  (const uint16_t*)p->weight, (uint16_t*)p->y, (uint16_t*)p->normed, p->rstd, p->d, p->eps);
  RA_CHECK_LAUNCH("rmsnorm_fwd");
  return RA_OK;
}

int rmsnorm_bwd(const ra_rmsnorm_params* p, hipStream_t s) {
  const int parts = rmsnorm_bwd_parts(p->T);
  const int rows = (int)((p->T + parts - 1) / parts);
  RA_RMS_DISPATCH(rmsnorm_bwd_kernel, parts, (const uint16_t*)p->d_normed, (const uint16_t*)p->y, (const uint16_t*)p->weight,
                  p->rstd, (const uint16_t*)p->d_residual, (uint16_t*)p->d_y, p->dw_workspace, p->T, p->d, rows);
  RA_CHECK_LAUNCH("rmsnorm_bwd");
  rmsnorm_dw_reduce_kernel<<<(p->d + 31) / 32, 256, 0, s>>>(p->dw_workspace, p->d_weight, (int)((p->T + rows - 1) / rows), p->d);
  RA_CHECK_LAUNCH("rmsnorm_dw_reduce");
  return RA_OK;
}

}  // namespace ra
