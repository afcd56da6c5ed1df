// Decode (cache_idx path, one query token per batch row): a bandwidth-bound
// streaming kernel.  The cache layout (B, L, H, D) makes one key position a
// contiguous H*D slab, so a workgroup owns (batch row, key range, a group of
// heads) and every wavefront load instruction covers 1 KiB of consecutive
// bytes.  A head is spread over LPH = D / (16 B / elem) lanes; the q.k dot
// product is reduced across those lanes, the running max / sum are replicated
// in them, and each lane keeps its 16-byte slice of the output accumulator.
// The key range is split over workgroups; partials are merged by a second pass.
//
// Mask semantics are those of ringattention_jax.py with query_chunk_size == 1:
// key chunks run iff below_or_on_diag (:324-331) says so, keys inside a chunk
// that runs are masked with finfo.min (:301-309), bias is added after the
// 1/sqrt(D) scaling and clamped to <= 0 when a mask is on (:134-136,:299,:309).
#include <mutex>
#include "common.hpp"

namespace ra {

struct DecodeArgs {
  const void* q; const void* k; const void* v; void* out;
  int B, L, H, D;
  int64_t q_sb, kv_sb, kv_ss, out_sb;
  MaskView mv;
  float* ws;          // [B][H][nsplit][D + 2]
  int nsplit;
  // ring step: the carry of ringattention_jax.py:22-23,:49 for the one query row, merged in place (nullable)
  float* c_num; float* c_den; float* c_max;
  int64_t c_num_sb, c_stat_sb;
  int carry_is_initial;
};

constexpr int DEC_THREADS = 512;
constexpr int DEC_UNROLL = 8;

template <typename T> struct Vec16;
template <> struct Vec16<uint16_t> {
  static constexpr int N = 8;
  __device__ static void load(const uint16_t* p, float* o) {
    uint4 u = *(const uint4*)p;
    uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; i++) { o[2 * i] = __uint_as_float(w[i] << 16); o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
  }
};
template <> struct Vec16<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float* o) {
    float4 u = *(const float4*)p;
    o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
  }
};

constexpr int dec_pow2_ge(int x) { int p = 1; while (p < x) p <<= 1; return p; }

// D: any multiple of the 16 bytes a lane loads (8 bf16 / 4 fp32 elements).  A head's elements take D / EPL lanes; the
// group of lanes that reduces a logit is the next power of two, and the lanes beyond the head's (head size 96: 12 of
// 16) go along with a zero query - they load what lane 0 loads and write nothing.
template <typename T, int D>
__global__ __launch_bounds__(DEC_THREADS) void decode_split_kernel(DecodeArgs a) {
  constexpr int EPL = Vec16<T>::N;        // elements per lane
  constexpr int LPA = D / EPL;            // lanes that hold a head's elements
  constexpr int LPH = dec_pow2_ge(LPA);   // lanes per head
  constexpr int HP = DEC_THREADS / LPH;   // heads per workgroup
  MaskView mv = a.mv;
  mv.resolve();                      // query_chunk_size == 1: q_start = cache_idx (:35)
  const int tid = threadIdx.x, b = blockIdx.z, split = blockIdx.x;
  const int h = blockIdx.y * HP + tid / LPH;
  const bool lane_on = tid % LPH < LPA;
  const int dl = lane_on ? tid % LPH : 0;
  const bool hvalid = h < a.H;
  const int hh = hvalid ? h : a.H - 1;

  // the single query row: local row 0 of query chunk 0
  const int kend = mv.run_prefix_keys(0, a.L);
  const long long gq = mv.global_q(0);
  const long long gq_blk = mv.cbs > 0 ? gq / mv.cbs : 0;
  int seg_q = 0;
  if (mv.seg) seg_q = mv.seg[(int64_t)b * mv.seg_sb + clamp_seg_index(gq, 1, mv.seg_len, 0)];
  const int64_t bias_off = (int64_t)b * mv.bias_sb + (int64_t)hh * mv.bias_sh;

  // key range of this split, in units of DEC_UNROLL keys
  int per = (kend + a.nsplit - 1) / a.nsplit;
  per = (per + DEC_UNROLL - 1) / DEC_UNROLL * DEC_UNROLL;
  const int ks = min(split * per, kend);
  const int ke = min(ks + per, kend);

  float qf[EPL], acc[EPL];
  Vec16<T>::load((const T*)a.q + (int64_t)b * a.q_sb + (int64_t)hh * D + dl * EPL, qf);
#pragma unroll
  for (int e = 0; e < EPL; e++) { acc[e] = 0.f; if (LPA != LPH && !lane_on) qf[e] = 0.f; }
  float m = RA_NEG_INF, l = 0.f;
  const float scale = sqrtf((float)D);
  const T* kb = (const T*)a.k + (int64_t)b * a.kv_sb + (int64_t)hh * D + dl * EPL;
  const T* vb = (const T*)a.v + (int64_t)b * a.kv_sb + (int64_t)hh * D + dl * EPL;
  // First local key behind the query's causal block (none when there is no causal mask).  From there on the cache may
  // never have been written: such a key is masked - finfo.min absorbs its logit, so the logit is not looked at - and
  // where its weight exp(finfo.min - max) is 0 its value is not multiplied (0 times an uninitialised slot's NaN or inf
  // is not 0).  With finite data in those slots nothing changes, bit for bit.
  const long long jd = mv.cbs > 0 ? (gq_blk + 1) * (long long)mv.cbs - mv.global_k(0) : (long long)a.L;
  const int jdead = (int)max(0LL, min(jd, (long long)a.L));

  for (int j0 = ks; j0 < ke; j0 += DEC_UNROLL) {
    float kf[DEC_UNROLL][EPL], vf[DEC_UNROLL][EPL], s[DEC_UNROLL];
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      int j = min(j0 + u, ke - 1);
      Vec16<T>::load(kb + (int64_t)j * a.kv_ss, kf[u]);
    }
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      int j = min(j0 + u, ke - 1);
      Vec16<T>::load(vb + (int64_t)j * a.kv_ss, vf[u]);
    }
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < EPL; e++) dot = fmaf(qf[e], kf[u][e], dot);
      s[u] = dot;
    }
#pragma unroll
    for (int off = 1; off < LPH; off <<= 1) {
#pragma unroll
      for (int u = 0; u < DEC_UNROLL; u++) s[u] += __shfl_xor(s[u], off);
    }
    float tile_max = RA_NEG_INF;
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) {
      const int j = j0 + u;
      const long long gk = mv.global_k(min(j, ke - 1));
      float add = 0.f;
      if (mv.bias) {
        add = mv.bias[bias_off + gk * mv.bias_sk];
        if (mv.any_mask) add = fminf(add, 0.f);
      }
      bool masked = (mv.cbs > 0 && gq_blk < gk / mv.cbs);
      if (mv.seg) {
        int jj = min(j, ke - 1);
        int idx = clamp_seg_index((mv.k_start + (long long)(jj / mv.kc)) * mv.kc, mv.kc, mv.seg_len, jj % mv.kc);
        masked = masked || (mv.seg[(int64_t)b * mv.seg_sb + idx] != seg_q);
      }
      s[u] = (j < ke) ? (masked ? mv.mask_min : s[u] / scale + add) : RA_NEG_INF;
      tile_max = fmaxf(tile_max, s[u]);
    }
    const float m_new = fmaxf(m, tile_max);
    const float corr = (m == m_new) ? 1.f : expf(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int u = 0; u < DEC_UNROLL; u++) { s[u] = expf(s[u] - m_new); psum += s[u]; }
    if (j0 + DEC_UNROLL > jdead) {           // the few steps that reach behind the query
#pragma unroll
      for (int e = 0; e < EPL; e++) {
        float t = 0.f;
#pragma unroll
        for (int u = 0; u < DEC_UNROLL; u++) t = s[u] != 0.f ? fmaf(s[u], vf[u][e], t) : t;
        acc[e] = acc[e] * corr + t;
      }
    } else {
#pragma unroll
      for (int e = 0; e < EPL; e++) {
        float t = 0.f;
#pragma unroll
        for (int u = 0; u < DEC_UNROLL; u++) t = fmaf(s[u], vf[u][e], t);
        acc[e] = acc[e] * corr + t;
      }
    }
    l = l * corr + psum;
    m = m_new;
  }
  if (hvalid && lane_on) {
    float* w = a.ws + (((int64_t)b * a.H + h) * a.nsplit + split) * (D + 2);
#pragma unroll
    for (int e = 0; e < EPL; e++) w[dl * EPL + e] = acc[e];
    if (dl == 0) { w[D] = m; w[D + 1] = l; }
  }
}

// Merges the split partials - and, in a ring step, the incoming carry - in a fixed order.  Without a carry the
// result is the normalised output; with one, (numerator, denominator, max_score) are updated in place as
// _blockwise_attention_fwd does per key chunk (:138-144), and out (nullable then) is written when the step is the
// last one of its device (:52).
template <typename T, int D>
__global__ void decode_combine_kernel(DecodeArgs a) {
  const int b = blockIdx.y, h = blockIdx.x, d = threadIdx.x;
  const float* w = a.ws + ((int64_t)b * a.H + h) * a.nsplit * (D + 2);
  float M = RA_NEG_INF;
  for (int s = 0; s < a.nsplit; s++) M = fmaxf(M, w[s * (D + 2) + D]);
  const bool merge = a.c_num && !a.carry_is_initial;
  float m_in = RA_NEG_INF, num_in = 0.f, den_in = 0.f;
  if (merge) {
    m_in = a.c_max[(int64_t)b * a.c_stat_sb + h];
    den_in = a.c_den[(int64_t)b * a.c_stat_sb + h];
    num_in = a.c_num[(int64_t)b * a.c_num_sb + (int64_t)h * D + d];
    M = fmaxf(M, m_in);
  }
  float num = 0.f, den = 0.f;
  // a part whose factor is 0 is left out rather than multiplied: a split that saw masked keys only (its own weights
  // are 1 then) may have summed what uninitialised cache slots hold, and 0 times inf is not 0
  if (merge && m_in != RA_NEG_INF) {
    const float c = expf(m_in - M);
    if (c != 0.f) {
      num = c * num_in;
      den = c * den_in;
    }
  }
  for (int s = 0; s < a.nsplit; s++) {
    const float ms = w[s * (D + 2) + D];
    if (ms == RA_NEG_INF) continue;
    const float c = expf(ms - M);
    if (c == 0.f) continue;
    num = fmaf(c, w[s * (D + 2) + d], num);
    den = fmaf(c, w[s * (D + 2) + D + 1], den);
  }
  if (a.c_num) {
    a.c_num[(int64_t)b * a.c_num_sb + (int64_t)h * D + d] = num;
    if (d == 0) {
      a.c_den[(int64_t)b * a.c_stat_sb + h] = den;
      a.c_max[(int64_t)b * a.c_stat_sb + h] = M;
    }
  }
  // no key ran at all: 0/0 = NaN, as numerator/denominator in ringattention_jax.py:52
  if (a.out) store_from_f32<T>((T*)a.out + (int64_t)b * a.out_sb + (int64_t)h * D + d, num / den);
}

int decode_pick_splits(int B, int L, int H, int D, int dtype) {
  const int epl = dtype == RA_F32 ? 4 : 8;
  const int hp = DEC_THREADS / dec_pow2_ge(D / epl);
  const int hg = (H + hp - 1) / hp;
  int want = (2048 + B * hg - 1) / (B * hg);
  int maxs = (L + 255) / 256;
  if (want > maxs) want = maxs;
  if (want < 1) want = 1;
  if (want > 256) want = 256;
  return want;
}

template <typename T, int D>
static int launch_decode(const DecodeArgs& a, hipStream_t s) {
  constexpr int LPH = dec_pow2_ge(D / Vec16<T>::N);
  constexpr int HP = DEC_THREADS / LPH;
  dim3 grid(a.nsplit, (a.H + HP - 1) / HP, a.B);
  decode_split_kernel<T, D><<<grid, DEC_THREADS, 0, s>>>(a);
  RA_CHECK_LAUNCH("decode_split");
  decode_combine_kernel<T, D><<<dim3(a.H, a.B), D, 0, s>>>(a);
  RA_CHECK_LAUNCH("decode_combine");
  return RA_OK;
}

// ---- the buffer of ra_decode_fwd_static: split-KV partials for callers that cannot allocate.  Each GPU holds its
// own copy of the array at its own address; in host code the array's name is only a handle for
// hipGetSymbolAddress, never a device address, so every launch takes the pointer looked up here.
static __device__ __align__(256) unsigned char decode_scratch[RA_DECODE_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[kMaxDevices];     // per device, filled on the first call with that device current

int decode_static_scratch(float** ptr, hipStream_t stream) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess && stream) {          // each GPU has its own copy of the array: the stream's GPU must be current
    hipDevice_t sdev = -1;
    if (hipStreamGetDevice(stream, &sdev) == hipSuccess && (int)sdev != dev) {
      set_error("decode_fwd_static: the stream belongs to device %d but device %d is current", (int)sdev, dev);
      return RA_ERR_INVALID;
    }
  }
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("decode_fwd_static: no usable current device (%s, device %d)", hipGetErrorString(e), dev);
    return RA_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(decode_scratch));
    if (e != hipSuccess || !sym) {
      set_error("decode_fwd_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return RA_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = (float*)sym;
  }
  *ptr = g_scratch_ptr[dev];
  return RA_OK;
}

int decode_fwd(const ra_decode_params* p, float* partials, int nsplit, hipStream_t s) {
  DecodeArgs a{};
  a.q = p->q; a.k = p->k; a.v = p->v; a.out = p->out;
  a.B = p->B; a.L = p->L; a.H = p->H; a.D = p->D;
  a.q_sb = p->q_stride_b; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s; a.out_sb = p->out_stride_b;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  a.ws = partials; a.nsplit = nsplit;
  a.c_num = p->carry_numerator; a.c_den = p->carry_denominator; a.c_max = p->carry_max_score;
  a.c_num_sb = p->carry_num_stride_b; a.c_stat_sb = p->carry_stat_stride_b;
  a.carry_is_initial = p->carry_is_initial;
#define RA_DECODE_D(DD)                                                              \
  if (p->D == DD) return p->dtype == RA_BF16 ? launch_decode<uint16_t, DD>(a, s) : launch_decode<float, DD>(a, s);
  RA_DECODE_D(128) RA_DECODE_D(64) RA_DECODE_D(256) RA_DECODE_D(32) RA_DECODE_D(40) RA_DECODE_D(80) RA_DECODE_D(96)
  RA_DECODE_D(112) RA_DECODE_D(160) RA_DECODE_D(192)
#undef RA_DECODE_D
  set_error("decode: head size %d not in {32,40,64,80,96,112,128,160,192,256}", p->D);
  return RA_ERR_UNSUPPORTED;
}

}  // namespace ra
