// extern "C" surface of libringattn_hip.so: argument validation, kernel-family
// dispatch and per-thread error text.  Declarations: include/ringattn_hip.h.
#include <stdarg.h>
#include <stdio.h>
#include "common.hpp"
#include "../../include/ringattn_hip_measure.h"

namespace ra {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int attn_fwd_generic(const ra_attn_fwd_params* p, hipStream_t s);
int attn_bwd_generic(const ra_attn_bwd_params* p, hipStream_t s);
int attn_fwd_mfma(const ra_attn_fwd_params* p, const ra_ring_step* ring, hipStream_t s);   // ring: nullable
int attn_bwd_mfma(const ra_attn_bwd_params* p, const ra_ring_step* ring, int parts, hipStream_t s);   // parts: RA_BWD_PART_* bits
bool attn_fwd_mfma_supported(const ra_attn_fwd_params* p);
bool attn_bwd_mfma_supported(const ra_attn_bwd_params* p);
int attn_fwd_f32(const ra_attn_fwd_params* p, hipStream_t s);                  // fp32 inputs on the matrix cores
int attn_bwd_f32(const ra_attn_bwd_params* p, int parts, hipStream_t s);
bool attn_fwd_f32_supported(const ra_attn_fwd_params* p);
bool attn_bwd_f32_supported(const ra_attn_bwd_params* p);
int attn_fwd_any(const ra_attn_fwd_params* p, hipStream_t s);                  // bf16, the mask element by element
int attn_bwd_any(const ra_attn_bwd_params* p, int parts, hipStream_t s);
bool attn_fwd_any_supported(const ra_attn_fwd_params* p);
bool attn_bwd_any_supported(const ra_attn_bwd_params* p);
int carry_init(float*, int64_t, int64_t, float*, float*, int64_t, int64_t, int, int, int, int, hipStream_t);
int finalize(const float*, int64_t, int64_t, const float*, int64_t, int64_t, void*, int, int64_t, int64_t, int,
             int, int, int, hipStream_t);
int bwd_delta(const void*, const void*, int, int, int64_t, int64_t, float*, int64_t, int64_t, int, int, int, int,
              hipStream_t);
int seg_tile_ranges(const int32_t*, int64_t, int, int, int32_t*, hipStream_t);
int seg_run_hulls(const int32_t*, int, int, int32_t*, hipStream_t);
int keep_pack(const uint8_t*, int64_t, int64_t, int64_t, int64_t, int, int, int, int, uint64_t*, uint64_t*, uint8_t*, hipStream_t);
int dropout_keep(uint64_t seed, uint32_t threshold, int64_t n, uint8_t* keep, hipStream_t s);
int dropout_keep_packed(uint64_t seed, uint32_t threshold, int planes, int Q, int K, uint64_t* bits_k,
                        uint64_t* bits_q, uint8_t* summary, int cbs, int qc, int kc, int q_start, int k_start,
                        hipStream_t s);
int decode_pick_splits(int B, int L, int H, int D, int dtype);
int decode_fwd(const ra_decode_params* p, float* partials, int nsplit, hipStream_t s);
int decode_static_scratch(float** ptr, hipStream_t stream);
int swiglu_fwd(const ra_swiglu_params* p, hipStream_t s);
int swiglu_bwd(const ra_swiglu_params* p, hipStream_t s);
int swiglu_weight_grads(const ra_swiglu_params* p, hipStream_t s);
int gemm_bf16(const void* A, const void* B, void* C, int M, int N, int K, int ta, int tb, int c_dtype,
              int beta_one, int tile, hipStream_t s);

int gemm_bf16_pair(const void* A, const void* B1, const void* B2, void* C1, void* C2, int M, int N, int K, int tile,
                   hipStream_t s);
int rope_kv_append(const ra_rope_append_params* p, hipStream_t s);
int rmsnorm_fwd(const ra_rmsnorm_params* p, hipStream_t s);
int rmsnorm_bwd(const ra_rmsnorm_params* p, hipStream_t s);
int rmsnorm_bwd_parts(int64_t T);
int rmsnorm_max_d();

static int check_mask(const ra_mask& m, int Sq, int Skv, const char* who) {
  RA_REQUIRE(m.query_chunk_size > 0 && m.key_chunk_size > 0, RA_ERR_INVALID, "%s: chunk sizes must be positive", who);
  RA_REQUIRE(Sq % m.query_chunk_size == 0, RA_ERR_INVALID, "%s: q_len %d is not a multiple of query_chunk_size %d",
             who, Sq, m.query_chunk_size);
  RA_REQUIRE(Skv % m.key_chunk_size == 0, RA_ERR_INVALID, "%s: kv_len %d is not a multiple of key_chunk_size %d",
             who, Skv, m.key_chunk_size);
  RA_REQUIRE(m.causal_block_size >= 0, RA_ERR_INVALID, "%s: causal_block_size must be >= 0 (0 = None)", who);
  if (m.causal_block_size > 0) {
    const int cbs = m.causal_block_size;
    RA_REQUIRE((cbs <= m.query_chunk_size || cbs % m.query_chunk_size == 0) &&
                   (cbs <= m.key_chunk_size || cbs % m.key_chunk_size == 0),
               RA_ERR_INVALID, "%s: causal_block_size %d larger than a chunk must be a multiple of it", who, cbs);
  }
  RA_REQUIRE(m.q_chunk_idx_start >= 0 && m.k_chunk_idx_start >= 0, RA_ERR_INVALID, "%s: negative chunk start", who);
  RA_REQUIRE(!m.chunk_starts || (!m.keep && !m.keep_bits_k && !m.keep_bits_q && !m.keep_summary), RA_ERR_UNSUPPORTED,
             "%s: chunk starts in device memory do not go with a keep mask (the host lays out its slices)", who);
  if (m.segment_ids) RA_REQUIRE(m.seg_len > 0, RA_ERR_INVALID, "%s: segment_ids given with seg_len 0", who);
  if (m.seg_tile_minmax)
    RA_REQUIRE(m.segment_ids && m.seg_tiles == (m.seg_len + RA_SEG_TILE - 1) / RA_SEG_TILE, RA_ERR_INVALID,
               "%s: seg_tile_minmax needs segment_ids and seg_tiles == ceil(seg_len / %d)", who, (int)RA_SEG_TILE);
  if (m.seg_run_hulls)
    RA_REQUIRE(m.seg_tile_minmax && m.seg_runs == (m.seg_tiles + 1) / 2, RA_ERR_INVALID,
               "%s: seg_run_hulls needs seg_tile_minmax and seg_runs == ceil(seg_tiles / 2)", who);
  if (m.keep_bits_k || m.keep_bits_q || m.keep_summary) {
    RA_REQUIRE(m.keep_bits_k && m.keep_bits_q && m.keep_summary, RA_ERR_INVALID,
               "%s: the packed keep mask needs keep_bits_k, keep_bits_q and keep_summary together", who);
    RA_REQUIRE(m.keep_q_total > 0 && m.keep_k_total > 0 && m.keep_q_total % 64 == 0 && m.keep_k_total % 64 == 0 &&
                   m.keep_q0 >= 0 && m.keep_q0 % 64 == 0 && m.keep_q0 + Sq <= m.keep_q_total &&
                   m.keep_k0 >= 0 && m.keep_k0 % 64 == 0 &&
                   (long long)m.k_chunk_idx_start * m.key_chunk_size >= m.keep_k0 &&
                   (long long)m.k_chunk_idx_start * m.key_chunk_size - m.keep_k0 + Skv <= m.keep_k_total,
               RA_ERR_INVALID, "%s: packed keep mask does not cover the rows / keys of the call", who);
  }
  if (m.keep || m.keep_bits_k) {
    RA_REQUIRE(m.keep_mode == RA_KEEP_WHERE || m.keep_mode == RA_KEEP_DROPOUT, RA_ERR_INVALID,
               "%s: keep_mode must be RA_KEEP_WHERE or RA_KEEP_DROPOUT", who);
    RA_REQUIRE(m.keep_k0 >= 0 && (long long)m.k_chunk_idx_start * m.key_chunk_size >= m.keep_k0, RA_ERR_INVALID,
               "%s: keep_k0 lies after the first key of the call", who);
  }
  RA_REQUIRE((long long)m.q_chunk_idx_start * m.query_chunk_size + Sq < (1LL << 31) - 4096 &&
                 (long long)m.k_chunk_idx_start * m.key_chunk_size + Skv < (1LL << 31) - 4096,
             RA_ERR_UNSUPPORTED, "%s: global positions must stay below 2^31", who);
  return RA_OK;
}

}  // namespace ra

using namespace ra;

extern "C" {

int ra_rope_kv_append(const ra_rope_append_params* p, ra_stream_t stream) {
  RA_REQUIRE(p, RA_ERR_INVALID, "rope_kv_append: null params");
  RA_REQUIRE(p->q && p->q_out && p->k_new && p->v_new && p->k_cache && p->v_cache, RA_ERR_INVALID,
             "rope_kv_append: null tensor");
  RA_REQUIRE(p->dtype == RA_F32 || p->dtype == RA_BF16, RA_ERR_UNSUPPORTED, "rope_kv_append: dtype %d", p->dtype);
  RA_REQUIRE(p->B > 0 && p->L > 0 && p->H > 0 && p->D > 0 && p->D % 2 == 0, RA_ERR_INVALID,
             "rope_kv_append: bad shape (B %d, L %d, H %d, D %d; D must be even)", p->B, p->L, p->H, p->D);
  RA_REQUIRE(p->rope_style == RA_ROPE_ADJACENT || p->rope_style == RA_ROPE_HALF, RA_ERR_INVALID,
             "rope_kv_append: rope_style %d", p->rope_style);
  if (!p->cache_idx)
    RA_REQUIRE(p->cache_idx_host >= 0 && p->cache_idx_host < p->L, RA_ERR_INVALID,
               "rope_kv_append: position %d outside the cache buffer of %d positions", p->cache_idx_host, p->L);
  return rope_kv_append(p, (hipStream_t)stream);
}

size_t ra_rmsnorm_workspace_bytes(int64_t T, int32_t d) {
  if (T <= 0 || d <= 0) return 0;
  return (size_t)rmsnorm_bwd_parts(T) * (size_t)d * sizeof(float);
}

static int check_rmsnorm(const ra_rmsnorm_params* p, const char* who) {
  RA_REQUIRE(p, RA_ERR_INVALID, "%s: null params", who);
  RA_REQUIRE(p->T > 0 && p->T <= 0x7fffffff && p->d > 0, RA_ERR_INVALID, "%s: empty or oversized shape", who);
  RA_REQUIRE(p->d % 8 == 0 && p->d <= rmsnorm_max_d(), RA_ERR_UNSUPPORTED,
             "%s: row length %d must be a multiple of 8 and at most %d", who, p->d, rmsnorm_max_d());
  return RA_OK;
}

int ra_rmsnorm_fwd(const ra_rmsnorm_params* p, ra_stream_t stream) {
  if (int rc = check_rmsnorm(p, "rmsnorm_fwd")) return rc;
  RA_REQUIRE(p->x && p->weight && p->normed && p->rstd && (p->residual == nullptr || p->y), RA_ERR_INVALID,
             "rmsnorm_fwd: null tensor (y is needed when a residual is given)");
  return rmsnorm_fwd(p, (hipStream_t)stream);
}

int ra_rmsnorm_bwd(const ra_rmsnorm_params* p, ra_stream_t stream) {
  if (int rc = check_rmsnorm(p, "rmsnorm_bwd")) return rc;
  RA_REQUIRE(p->d_normed && p->y && p->weight && p->rstd && p->d_y && p->d_weight && p->dw_workspace, RA_ERR_INVALID,
             "rmsnorm_bwd: null tensor");
  RA_REQUIRE(p->dw_workspace_bytes >= ra_rmsnorm_workspace_bytes(p->T, p->d), RA_ERR_INVALID,
             "rmsnorm_bwd: workspace %zu bytes < %zu needed", p->dw_workspace_bytes,
             ra_rmsnorm_workspace_bytes(p->T, p->d));
  return rmsnorm_bwd(p, (hipStream_t)stream);
}

const char* ra_last_error(void) { return g_err; }
int ra_version(void) { return RA_ABI_VERSION; }

int ra_attn_carry_init(float* numerator, int64_t num_stride_b, int64_t num_stride_s, float* denominator,
                       float* max_score, int64_t stat_stride_b, int64_t stat_stride_h, int32_t B, int32_t Sq,
                       int32_t H, int32_t D, ra_stream_t stream) {
  RA_REQUIRE(numerator && denominator && max_score, RA_ERR_INVALID, "carry_init: null pointer");
  RA_REQUIRE(B > 0 && Sq > 0 && H > 0 && D > 0, RA_ERR_INVALID, "carry_init: empty shape");
  return carry_init(numerator, num_stride_b, num_stride_s, denominator, max_score, stat_stride_b, stat_stride_h, B,
                    Sq, H, D, (hipStream_t)stream);
}

int ra_segment_tile_ranges(const int32_t* segment_ids, int64_t seg_stride_b, int32_t Bseg, int32_t seg_len,
                           int32_t* out, ra_stream_t stream) {
  RA_REQUIRE(segment_ids && out, RA_ERR_INVALID, "segment_tile_ranges: null pointer");
  RA_REQUIRE(Bseg > 0 && Bseg <= 65535 && seg_len > 0, RA_ERR_INVALID, "segment_tile_ranges: bad shape");
  return seg_tile_ranges(segment_ids, seg_stride_b, Bseg, seg_len, out, (hipStream_t)stream);
}

int ra_segment_run_hulls(const int32_t* seg_tile_minmax, int32_t Bseg, int32_t seg_tiles, int32_t* out,
                         ra_stream_t stream) {
  RA_REQUIRE(seg_tile_minmax && out, RA_ERR_INVALID, "segment_run_hulls: null pointer");
  RA_REQUIRE(Bseg > 0 && Bseg <= 65535 && seg_tiles > 0, RA_ERR_INVALID, "segment_run_hulls: bad shape");
  return seg_run_hulls(seg_tile_minmax, Bseg, seg_tiles, out, (hipStream_t)stream);
}

int ra_keep_pack(const uint8_t* keep, int64_t stride_b, int64_t stride_h, int64_t stride_q, int64_t stride_k,
                 int32_t Bm, int32_t Hm, int32_t Q, int32_t K, uint64_t* bits_k, uint64_t* bits_q,
                 uint8_t* summary, ra_stream_t stream) {
  RA_REQUIRE(keep && bits_k && bits_q && summary, RA_ERR_INVALID, "keep_pack: null pointer");
  RA_REQUIRE(Bm > 0 && Hm > 0 && (long long)Bm * Hm <= 65535, RA_ERR_INVALID, "keep_pack: bad plane count");
  RA_REQUIRE(Q > 0 && K > 0 && Q % 64 == 0 && K % 64 == 0 && Q / 64 <= 65535, RA_ERR_UNSUPPORTED,
             "keep_pack: Q and K must be positive multiples of 64 (got %d, %d)", Q, K);
  return keep_pack(keep, stride_b, stride_h, stride_q, stride_k, Bm, Hm, Q, K, bits_k, bits_q, summary,
                   (hipStream_t)stream);
}

static uint32_t dropout_threshold(float attn_pdrop) { return (uint32_t)((double)attn_pdrop * 65536.0); }   // floor

int ra_dropout_keep(uint64_t seed, float attn_pdrop, int32_t B, int32_t H, int32_t Q, int32_t K, uint8_t* keep,
                    ra_stream_t stream) {
  RA_REQUIRE(keep, RA_ERR_INVALID, "dropout_keep: null pointer");
  RA_REQUIRE(((uintptr_t)keep % 8) == 0, RA_ERR_UNSUPPORTED, "dropout_keep: keep must be 8-byte aligned");
  RA_REQUIRE(B > 0 && H > 0 && Q > 0 && K > 0, RA_ERR_INVALID, "dropout_keep: empty shape");
  RA_REQUIRE(K % 8 == 0, RA_ERR_UNSUPPORTED, "dropout_keep: K must be a multiple of 8 (got %d)", K);
  RA_REQUIRE(attn_pdrop > 0.f && attn_pdrop < 1.f, RA_ERR_INVALID, "dropout_keep: attn_pdrop must lie in (0, 1)");
  const int64_t n = (int64_t)B * H * Q * K;
  RA_REQUIRE(n / 16 / 256 < (1LL << 31), RA_ERR_UNSUPPORTED, "dropout_keep: mask too large");
  return dropout_keep(seed, dropout_threshold(attn_pdrop), n, keep, (hipStream_t)stream);
}

int ra_dropout_keep_packed(uint64_t seed, float attn_pdrop, int32_t B, int32_t H, int32_t Q, int32_t K,
                           uint64_t* bits_k, uint64_t* bits_q, uint8_t* summary, int32_t causal_block_size,
                           int32_t query_chunk_size, int32_t key_chunk_size, int32_t q_chunk_idx_start,
                           int32_t k_chunk_idx_start, ra_stream_t stream) {
  RA_REQUIRE(bits_k && bits_q && summary, RA_ERR_INVALID, "dropout_keep_packed: null pointer");
  RA_REQUIRE(B > 0 && H > 0 && (long long)B * H <= 65535, RA_ERR_INVALID, "dropout_keep_packed: bad plane count");
  RA_REQUIRE(Q > 0 && K > 0 && Q % 64 == 0 && K % 64 == 0 && Q / 64 <= 65535, RA_ERR_UNSUPPORTED,
             "dropout_keep_packed: Q and K must be positive multiples of 64 (got %d, %d)", Q, K);
  RA_REQUIRE(attn_pdrop > 0.f && attn_pdrop < 1.f, RA_ERR_INVALID,
             "dropout_keep_packed: attn_pdrop must lie in (0, 1)");
  if (causal_block_size > 0) {
    const int cbs = causal_block_size, qc = query_chunk_size, kc = key_chunk_size;
    RA_REQUIRE(qc > 0 && kc > 0 && Q % qc == 0 && K % kc == 0 && q_chunk_idx_start >= 0 && k_chunk_idx_start >= 0 &&
                   (cbs <= qc || cbs % qc == 0) && (cbs <= kc || cbs % kc == 0),
               RA_ERR_INVALID, "dropout_keep_packed: chunk sizes must divide Q and K, and a causal_block_size larger "
                               "than a chunk must be a multiple of it");
  }
  return dropout_keep_packed(seed, dropout_threshold(attn_pdrop), B * H, Q, K, bits_k, bits_q, summary,
                             causal_block_size, query_chunk_size, key_chunk_size, q_chunk_idx_start,
                             k_chunk_idx_start, (hipStream_t)stream);
}

int ra_attn_fwd_block(const ra_attn_fwd_params* p, ra_stream_t stream) {
  RA_REQUIRE(p, RA_ERR_INVALID, "attn_fwd_block: null params");
  RA_REQUIRE(p->q && p->k && p->v && p->denominator && p->max_score, RA_ERR_INVALID, "attn_fwd_block: null tensor");
  RA_REQUIRE(p->numerator || (p->carry_is_initial && p->out), RA_ERR_INVALID,
             "attn_fwd_block: the numerator may be null only when carry_is_initial is set and out is given");
  RA_REQUIRE(!p->out_f32 || p->out, RA_ERR_INVALID, "attn_fwd_block: out_f32 goes with out");
  RA_REQUIRE(p->logit_dim >= 0, RA_ERR_INVALID, "attn_fwd_block: negative logit_dim");
  RA_REQUIRE(p->dtype == RA_F32 || p->dtype == RA_BF16, RA_ERR_UNSUPPORTED, "attn_fwd_block: dtype %d", p->dtype);
  RA_REQUIRE(p->B > 0 && p->Sq > 0 && p->Skv > 0 && p->H > 0 && p->D > 0, RA_ERR_INVALID, "attn_fwd_block: empty shape");
  RA_REQUIRE(p->B <= 65535 && p->H <= 65535, RA_ERR_UNSUPPORTED, "attn_fwd_block: B and H must be <= 65535");
  if (int rc = check_mask(p->mask, p->Sq, p->Skv, "attn_fwd_block")) return rc;
  hipStream_t s = (hipStream_t)stream;
  RA_REQUIRE(p->impl == RA_IMPL_AUTO || p->impl == RA_IMPL_GENERIC || p->impl == RA_IMPL_MFMA ||
             p->impl == RA_IMPL_MFMA_ANY, RA_ERR_INVALID, "attn_fwd_block: impl %d", p->impl);
  if (p->impl == RA_IMPL_GENERIC) return attn_fwd_generic(p, s);
  if (p->impl != RA_IMPL_MFMA_ANY) {
    if (attn_fwd_mfma_supported(p)) return attn_fwd_mfma(p, nullptr, s);
    if (attn_fwd_f32_supported(p)) return attn_fwd_f32(p, s);
    RA_REQUIRE(p->impl != RA_IMPL_MFMA, RA_ERR_UNSUPPORTED,
               "attn_fwd_block: MFMA kernels need bf16 or fp32, head size 64 or 128, chunk sizes that are multiples of 128");
  }
  if (attn_fwd_any_supported(p)) return attn_fwd_any(p, s);
  RA_REQUIRE(p->impl != RA_IMPL_MFMA_ANY, RA_ERR_UNSUPPORTED,
             "attn_fwd_block: the element-wise-mask MFMA kernels need bf16, head size 128 or 256, no attention dropout");
  return attn_fwd_generic(p, s);
}

int ra_attn_fwd_family(const ra_attn_fwd_params* p) {
  if (!p || (p->dtype != RA_F32 && p->dtype != RA_BF16)) return 0;
  if (p->impl == RA_IMPL_GENERIC) return RA_FAMILY_GENERIC;
  if (p->impl != RA_IMPL_MFMA_ANY) {
    if (attn_fwd_mfma_supported(p)) return RA_FAMILY_MFMA_BF16;
    if (attn_fwd_f32_supported(p)) return RA_FAMILY_MFMA_F32;
    if (p->impl == RA_IMPL_MFMA) return 0;
  }
  if (attn_fwd_any_supported(p)) return RA_FAMILY_MFMA_BF16_ANY;
  return p->impl == RA_IMPL_MFMA_ANY ? 0 : RA_FAMILY_GENERIC;
}

int ra_attn_bwd_family(const ra_attn_bwd_params* p) {
  if (!p || (p->dtype != RA_F32 && p->dtype != RA_BF16)) return 0;
  if (p->impl == RA_IMPL_GENERIC) return RA_FAMILY_GENERIC;
  if (p->impl != RA_IMPL_MFMA_ANY) {
    if (attn_bwd_mfma_supported(p)) return RA_FAMILY_MFMA_BF16;
    if (attn_bwd_f32_supported(p)) return RA_FAMILY_MFMA_F32;
    if (p->impl == RA_IMPL_MFMA) return 0;
  }
  if (attn_bwd_any_supported(p)) return RA_FAMILY_MFMA_BF16_ANY;
  return p->impl == RA_IMPL_MFMA_ANY ? 0 : RA_FAMILY_GENERIC;
}

int ra_attn_finalize(const float* numerator, int64_t num_stride_b, int64_t num_stride_s, const float* denominator,
                     int64_t stat_stride_b, int64_t stat_stride_h, void* out, int32_t out_dtype,
                     int64_t out_stride_b, int64_t out_stride_s, int32_t B, int32_t Sq, int32_t H, int32_t D,
                     ra_stream_t stream) {
  RA_REQUIRE(numerator && denominator && out, RA_ERR_INVALID, "finalize: null pointer");
  RA_REQUIRE(out_dtype == RA_F32 || out_dtype == RA_BF16, RA_ERR_UNSUPPORTED, "finalize: dtype %d", out_dtype);
  RA_REQUIRE(B > 0 && Sq > 0 && H > 0 && D > 0 && B <= 65535, RA_ERR_INVALID, "finalize: bad shape");
  return finalize(numerator, num_stride_b, num_stride_s, denominator, stat_stride_b, stat_stride_h, out, out_dtype,
                  out_stride_b, out_stride_s, B, Sq, H, D, (hipStream_t)stream);
}

int ra_attn_bwd_delta(const void* g, const void* out, int32_t dtype, int32_t out_dtype, int64_t stride_b,
                      int64_t stride_s, float* delta, int64_t stat_stride_b, int64_t stat_stride_h, int32_t B,
                      int32_t Sq, int32_t H, int32_t D, ra_stream_t stream) {
  RA_REQUIRE(g && out && delta, RA_ERR_INVALID, "bwd_delta: null pointer");
  RA_REQUIRE(dtype == RA_F32 || dtype == RA_BF16, RA_ERR_UNSUPPORTED, "bwd_delta: dtype %d", dtype);
  RA_REQUIRE(out_dtype == dtype || out_dtype == RA_F32, RA_ERR_UNSUPPORTED,
             "bwd_delta: out is either in the cotangent's dtype or fp32 (got %d)", out_dtype);
  RA_REQUIRE(B > 0 && Sq > 0 && H > 0 && D > 0 && B <= 65535, RA_ERR_INVALID, "bwd_delta: bad shape");
  return bwd_delta(g, out, dtype, out_dtype, stride_b, stride_s, delta, stat_stride_b, stat_stride_h, B, Sq, H, D,
                   (hipStream_t)stream);
}

static int attn_bwd_block(const ra_attn_bwd_params* p, int parts, const char* who, hipStream_t s) {
  const bool dq_part = parts & RA_BWD_PART_DQ, dkv_part = parts & RA_BWD_PART_DKV;
  RA_REQUIRE(p, RA_ERR_INVALID, "%s: null params", who);
  RA_REQUIRE(p->q && p->k && p->v && p->g && p->delta && p->denominator && p->max_score, RA_ERR_INVALID,
             "%s: null tensor", who);
  RA_REQUIRE((p->dk_out == nullptr) == (p->dv_out == nullptr), RA_ERR_INVALID, "%s: dk_out and dv_out go together", who);
  RA_REQUIRE((p->grads_are_initial & ~(RA_GRAD_INIT_DQ | RA_GRAD_INIT_DKV)) == 0, RA_ERR_INVALID,
             "%s: unknown bits in grads_are_initial", who);
  RA_REQUIRE(!dq_part || p->dq || ((p->grads_are_initial & RA_GRAD_INIT_DQ) && p->dq_out), RA_ERR_INVALID,
             "%s: dq may be null only when it is initial and dq_out is given", who);
  RA_REQUIRE(!dkv_part || (p->dk && p->dv) || ((p->grads_are_initial & RA_GRAD_INIT_DKV) && p->dk_out), RA_ERR_INVALID,
             "%s: dk / dv may be null only when they are initial and dk_out / dv_out are given", who);
  RA_REQUIRE(p->dtype == RA_F32 || p->dtype == RA_BF16, RA_ERR_UNSUPPORTED, "%s: dtype %d", who, p->dtype);
  RA_REQUIRE(p->B > 0 && p->Sq > 0 && p->Skv > 0 && p->H > 0 && p->D > 0, RA_ERR_INVALID, "%s: empty shape", who);
  RA_REQUIRE(p->B <= 65535 && p->H <= 65535, RA_ERR_UNSUPPORTED, "%s: B and H must be <= 65535", who);
  RA_REQUIRE(p->logit_dim >= 0, RA_ERR_INVALID, "%s: negative logit_dim", who);
  RA_REQUIRE(p->impl == RA_IMPL_AUTO || p->impl == RA_IMPL_GENERIC || p->impl == RA_IMPL_MFMA ||
             p->impl == RA_IMPL_MFMA_ANY, RA_ERR_INVALID, "%s: impl %d", who, p->impl);
  if (int rc = check_mask(p->mask, p->Sq, p->Skv, who)) return rc;
  const bool whole = dq_part && dkv_part;
  if (p->impl == RA_IMPL_GENERIC && whole) return attn_bwd_generic(p, s);
  const bool tiled = p->impl == RA_IMPL_AUTO || p->impl == RA_IMPL_MFMA;
  if (tiled && attn_bwd_mfma_supported(p)) return attn_bwd_mfma(p, nullptr, parts, s);
  if (tiled && attn_bwd_f32_supported(p)) return attn_bwd_f32(p, parts, s);
  RA_REQUIRE(p->impl != RA_IMPL_MFMA, RA_ERR_UNSUPPORTED,
             "%s: MFMA kernels need bf16 or fp32, head size 64 or 128, chunk sizes that are multiples of 128", who);
  if (p->impl != RA_IMPL_GENERIC && attn_bwd_any_supported(p)) return attn_bwd_any(p, parts, s);
  RA_REQUIRE(p->impl != RA_IMPL_MFMA_ANY, RA_ERR_UNSUPPORTED,
             "%s: the element-wise-mask MFMA kernels need bf16, head size 128 or 256, no attention dropout", who);
  RA_REQUIRE(whole, RA_ERR_UNSUPPORTED, "%s: one part alone is launched by the MFMA kernels only, which do not take "
             "this call (impl, dtype, head size or chunk sizes)", who);
  return attn_bwd_generic(p, s);
}

int ra_attn_bwd_block(const ra_attn_bwd_params* p, ra_stream_t stream) {
  return attn_bwd_block(p, RA_BWD_PART_DQ | RA_BWD_PART_DKV, "attn_bwd_block", (hipStream_t)stream);
}

int ra_attn_bwd_block_part(const ra_attn_bwd_params* p, int32_t part, ra_stream_t stream) {
  RA_REQUIRE(part == RA_BWD_PART_DQ || part == RA_BWD_PART_DKV, RA_ERR_INVALID,
             "attn_bwd_block_part: part must be RA_BWD_PART_DQ or RA_BWD_PART_DKV");
  return attn_bwd_block(p, part, "attn_bwd_block_part", (hipStream_t)stream);
}

// The checks the two ring-step entry points share; q_len / kv_len: one device's shard lengths
static int check_ring(const ra_ring_step* r, const ra_mask& m, int Sq, int Skv, int impl, const char* who) {
  RA_REQUIRE(r, RA_ERR_INVALID, "%s: null ring step", who);
  RA_REQUIRE(r->n_dev >= 1 && r->n_dev <= 64 && r->idx >= 0 && r->idx < r->n_dev, RA_ERR_INVALID,
             "%s: ring of %d devices, step %d", who, r->n_dev, r->idx);
  RA_REQUIRE(Sq % r->n_dev == 0 && Skv % r->n_dev == 0, RA_ERR_INVALID,
             "%s: sequence lengths (%d, %d) must divide by the ring size %d", who, Sq, Skv, r->n_dev);
  const uint64_t all = r->n_dev == 64 ? ~0ULL : ((1ULL << r->n_dev) - 1ULL);
  RA_REQUIRE(((r->run | r->first | r->last | r->kv_first | r->kv_last) & ~all) == 0, RA_ERR_INVALID,
             "%s: bits set beyond device %d", who, r->n_dev - 1);
  RA_REQUIRE(impl != RA_IMPL_GENERIC, RA_ERR_UNSUPPORTED, "%s: the MFMA kernels only", who);
  RA_REQUIRE(!m.keep && !m.keep_bits_k && !m.cache_idx && !m.chunk_starts, RA_ERR_UNSUPPORTED,
             "%s: no keep mask, no cache_idx and no device-side chunk starts in a ring-step launch", who);
  return check_mask(m, Sq / r->n_dev, Skv / r->n_dev, who);
}

int ra_attn_fwd_ring_step(const ra_attn_fwd_params* p, const ra_ring_step* ring, ra_stream_t stream) {
  const char* who = "attn_fwd_ring_step";
  RA_REQUIRE(p, RA_ERR_INVALID, "%s: null params", who);
  RA_REQUIRE(p->q && p->k && p->v && p->denominator && p->max_score, RA_ERR_INVALID, "%s: null tensor", who);
  RA_REQUIRE(p->B > 0 && p->Sq > 0 && p->Skv > 0 && p->H > 0 && p->D > 0, RA_ERR_INVALID, "%s: empty shape", who);
  RA_REQUIRE(p->B <= 65535 && p->H <= 65535, RA_ERR_UNSUPPORTED, "%s: B and H must be <= 65535", who);
  if (int rc = check_ring(ring, p->mask, p->Sq, p->Skv, p->impl, who)) return rc;
  // a device that neither starts its carry here nor writes out needs the numerator in both directions
  RA_REQUIRE(p->numerator || (ring->run & ~(ring->first & ring->last)) == 0, RA_ERR_INVALID,
             "%s: the numerator may be null only when every running device both starts and ends here", who);
  RA_REQUIRE(p->out || (ring->run & ring->last) == 0, RA_ERR_INVALID, "%s: a device writes out but out is null", who);
  RA_REQUIRE(!p->out_f32 || p->out, RA_ERR_INVALID, "%s: out_f32 goes with out", who);
  ra_attn_fwd_params dev = *p;        // the shape one device sees: what the kernels' chunk grid has to fit
  dev.Sq = p->Sq / ring->n_dev; dev.Skv = p->Skv / ring->n_dev;
  RA_REQUIRE(attn_fwd_mfma_supported(&dev), RA_ERR_UNSUPPORTED,
             "%s: MFMA kernels need bf16, head size 64 or 128, chunk sizes that are multiples of 128", who);
  return attn_fwd_mfma(p, ring, (hipStream_t)stream);
}

static int attn_bwd_ring_step(const ra_attn_bwd_params* p, const ra_ring_step* ring, int parts, const char* who,
                              hipStream_t stream) {
  const bool dq_part = parts & RA_BWD_PART_DQ, dkv_part = parts & RA_BWD_PART_DKV;
  RA_REQUIRE(p, RA_ERR_INVALID, "%s: null params", who);
  RA_REQUIRE(p->q && p->k && p->v && p->g && p->delta && p->denominator && p->max_score, RA_ERR_INVALID,
             "%s: null tensor", who);
  RA_REQUIRE((p->dk_out == nullptr) == (p->dv_out == nullptr), RA_ERR_INVALID, "%s: dk_out and dv_out go together", who);
  RA_REQUIRE((p->dk == nullptr) == (p->dv == nullptr), RA_ERR_INVALID, "%s: dk and dv go together", who);
  RA_REQUIRE(p->B > 0 && p->Sq > 0 && p->Skv > 0 && p->H > 0 && p->D > 0, RA_ERR_INVALID, "%s: empty shape", who);
  RA_REQUIRE(p->B <= 65535 && p->H <= 65535, RA_ERR_UNSUPPORTED, "%s: B and H must be <= 65535", who);
  if (int rc = check_ring(ring, p->mask, p->Sq, p->Skv, p->impl, who)) return rc;
  uint64_t shards = 0;                // the K/V shards that the running devices hold in this step
  for (int d = 0; d < ring->n_dev; d++)
    if ((ring->run >> d) & 1ULL) shards |= 1ULL << ((d - ring->idx + ring->n_dev) % ring->n_dev);
  RA_REQUIRE(!dq_part || p->dq || (ring->run & ~(ring->first & ring->last)) == 0, RA_ERR_INVALID,
             "%s: dq may be null only when every running device both starts and ends its dq here", who);
  RA_REQUIRE(!dkv_part || p->dk || (shards & ~(ring->kv_first & ring->kv_last)) == 0, RA_ERR_INVALID,
             "%s: dk / dv may be null only when every shard in use both starts and ends here", who);
  RA_REQUIRE(!dq_part || p->dq_out || (ring->run & ring->last) == 0, RA_ERR_INVALID, "%s: dq_out is null but a device writes it", who);
  RA_REQUIRE(!dkv_part || p->dk_out || (shards & ring->kv_last) == 0, RA_ERR_INVALID, "%s: dk_out is null but a shard writes it", who);
  ra_attn_bwd_params dev = *p;
  dev.Sq = p->Sq / ring->n_dev; dev.Skv = p->Skv / ring->n_dev;
  RA_REQUIRE(attn_bwd_mfma_supported(&dev), RA_ERR_UNSUPPORTED,
             "%s: MFMA kernels need bf16, head size 64 or 128, chunk sizes that are multiples of 128", who);
  return attn_bwd_mfma(p, ring, parts, stream);
}

int ra_attn_bwd_ring_step(const ra_attn_bwd_params* p, const ra_ring_step* ring, ra_stream_t stream) {
  return attn_bwd_ring_step(p, ring, RA_BWD_PART_DQ | RA_BWD_PART_DKV, "attn_bwd_ring_step", (hipStream_t)stream);
}

int ra_attn_bwd_ring_step_part(const ra_attn_bwd_params* p, const ra_ring_step* ring, int32_t part, ra_stream_t stream) {
  RA_REQUIRE(part == RA_BWD_PART_DQ || part == RA_BWD_PART_DKV, RA_ERR_INVALID,
             "attn_bwd_ring_step_part: part must be RA_BWD_PART_DQ or RA_BWD_PART_DKV");
  return attn_bwd_ring_step(p, ring, part, "attn_bwd_ring_step_part", (hipStream_t)stream);
}

int ra_decode_auto_splits(int32_t B, int32_t L, int32_t H, int32_t D, int32_t dtype) {
  if (B <= 0 || L <= 0 || H <= 0 || (D != 64 && D != 128) || (dtype != RA_F32 && dtype != RA_BF16)) return 0;
  return decode_pick_splits(B, L, H, D, dtype);
}

size_t ra_decode_workspace_bytes(int32_t B, int32_t L, int32_t H, int32_t D, int32_t num_splits) {
  if (B <= 0 || L <= 0 || H <= 0 || D <= 0) return 0;
  int ns = num_splits > 0 ? num_splits : 256;   // upper bound of the automatic choice
  return (size_t)B * H * ns * (D + 2) * sizeof(float);
}

static int check_decode(const ra_decode_params* p, const char* who) {
  RA_REQUIRE(p, RA_ERR_INVALID, "%s: null params", who);
  RA_REQUIRE(p->q && p->k && p->v, RA_ERR_INVALID, "%s: null tensor", who);
  const bool carry = p->carry_numerator || p->carry_denominator || p->carry_max_score;
  RA_REQUIRE(!carry || (p->carry_numerator && p->carry_denominator && p->carry_max_score), RA_ERR_INVALID,
             "%s: the carry is numerator, denominator and max_score together", who);
  RA_REQUIRE(p->out || carry, RA_ERR_INVALID, "%s: out may be null only in a ring step that hands on a carry", who);
  RA_REQUIRE(p->dtype == RA_F32 || p->dtype == RA_BF16, RA_ERR_UNSUPPORTED, "%s: dtype %d", who, p->dtype);
  RA_REQUIRE(p->B > 0 && p->L > 0 && p->H > 0 && p->D > 0 && p->B <= 65535, RA_ERR_INVALID, "%s: bad shape", who);
  RA_REQUIRE(p->D == 32 || p->D == 40 || p->D == 64 || p->D == 80 || p->D == 96 || p->D == 112 || p->D == 128 ||
                 p->D == 160 || p->D == 192 || p->D == 256,
             RA_ERR_UNSUPPORTED, "%s: head size %d not in {32, 40, 64, 80, 96, 112, 128, 160, 192, 256}", who, p->D);
  RA_REQUIRE(p->mask.query_chunk_size == 1, RA_ERR_INVALID,
             "%s: one query token needs query_chunk_size == 1 (q_len // query_chunk_size chunks)", who);
  if (int rc = check_mask(p->mask, 1, p->L, who)) return rc;
  RA_REQUIRE(p->mask.keep == nullptr && p->mask.keep_bits_k == nullptr, RA_ERR_UNSUPPORTED,
             "%s: the boolean keep mask is taken by the generic attention kernels only", who);
  RA_REQUIRE(p->num_splits >= 0 && p->num_splits <= 256, RA_ERR_INVALID, "%s: num_splits %d outside [0, 256]", who,
             p->num_splits);
  return RA_OK;
}

int ra_decode_fwd(const ra_decode_params* p, ra_stream_t stream) {
  if (int rc = check_decode(p, "decode_fwd")) return rc;
  RA_REQUIRE(p->workspace, RA_ERR_INVALID, "decode_fwd: null workspace");
  int ns = p->num_splits > 0 ? p->num_splits : decode_pick_splits(p->B, p->L, p->H, p->D, p->dtype);
  size_t need = (size_t)p->B * p->H * ns * (p->D + 2) * sizeof(float);
  RA_REQUIRE(p->workspace_bytes >= need, RA_ERR_INVALID, "decode_fwd: workspace %zu bytes < %zu needed",
             p->workspace_bytes, need);
  return decode_fwd(p, (float*)p->workspace, ns, (hipStream_t)stream);
}

int ra_decode_fwd_static(const ra_decode_params* p, ra_stream_t stream) {
  if (int rc = check_decode(p, "decode_fwd_static")) return rc;
  const size_t per_split = (size_t)p->B * p->H * (p->D + 2) * sizeof(float);
  RA_REQUIRE(per_split <= (size_t)RA_DECODE_STATIC_SCRATCH_BYTES, RA_ERR_UNSUPPORTED,
             "decode_fwd_static: B * H * (D + 2) * 4 = %zu bytes exceed the built-in scratch buffer of %d bytes; "
             "use ra_decode_fwd with a workspace", per_split, (int)RA_DECODE_STATIC_SCRATCH_BYTES);
  int ns = p->num_splits > 0 ? p->num_splits : decode_pick_splits(p->B, p->L, p->H, p->D, p->dtype);
  const int fit = (int)((size_t)RA_DECODE_STATIC_SCRATCH_BYTES / per_split);
  if (ns > fit) ns = fit;
  float* scratch = nullptr;
  if (int rc = decode_static_scratch(&scratch, (hipStream_t)stream)) return rc;
  return decode_fwd(p, scratch, ns, (hipStream_t)stream);
}

int ra_swiglu_fwd(const ra_swiglu_params* p, ra_stream_t stream) {
  RA_REQUIRE(p, RA_ERR_INVALID, "swiglu_fwd: null params");
  RA_REQUIRE(p->x && p->w1 && p->w2 && p->w3 && p->a && p->b && p->h && p->y, RA_ERR_INVALID, "swiglu_fwd: null tensor");
  RA_REQUIRE(p->T > 0 && p->d > 0 && p->f > 0, RA_ERR_INVALID, "swiglu_fwd: empty shape");
  RA_REQUIRE(p->gemm_tile >= 0 && p->gemm_tile <= 4, RA_ERR_INVALID, "swiglu_fwd: gemm_tile %d outside [0, 4]", p->gemm_tile);
  return swiglu_fwd(p, (hipStream_t)stream);
}

int ra_swiglu_bwd(const ra_swiglu_params* p, ra_stream_t stream) {
  RA_REQUIRE(p, RA_ERR_INVALID, "swiglu_bwd: null params");
  RA_REQUIRE(p->x && p->w1 && p->w2 && p->w3 && p->a && p->b && p->h && p->dy && p->dx && p->da && p->db &&
                 (p->defer_weight_grads || (p->dw1 && p->dw2 && p->dw3)),
             RA_ERR_INVALID, "swiglu_bwd: null tensor");
  RA_REQUIRE(p->T > 0 && p->d > 0 && p->f > 0, RA_ERR_INVALID, "swiglu_bwd: empty shape");
  RA_REQUIRE(p->gemm_tile >= 0 && p->gemm_tile <= 4, RA_ERR_INVALID, "swiglu_bwd: gemm_tile %d outside [0, 4]", p->gemm_tile);
  return swiglu_bwd(p, (hipStream_t)stream);
}

int ra_swiglu_weight_grads(const ra_swiglu_params* p, ra_stream_t stream) {
  RA_REQUIRE(p, RA_ERR_INVALID, "swiglu_weight_grads: null params");
  RA_REQUIRE(p->x && p->dy && p->h && p->da && p->db && p->dw1 && p->dw2 && p->dw3, RA_ERR_INVALID,
             "swiglu_weight_grads: null tensor");
  RA_REQUIRE(p->T > 0 && p->d > 0 && p->f > 0, RA_ERR_INVALID, "swiglu_weight_grads: empty shape");
  RA_REQUIRE(p->gemm_tile >= 0 && p->gemm_tile <= 4, RA_ERR_INVALID, "swiglu_weight_grads: gemm_tile %d outside [0, 4]", p->gemm_tile);
  return swiglu_weight_grads(p, (hipStream_t)stream);
}

int ra_gemm_bf16(const void* A, const void* Bm, void* C, int32_t M, int32_t N, int32_t K, int32_t trans_a,
                 int32_t trans_b, int32_t c_dtype, int32_t beta_one, ra_stream_t stream) {
  RA_REQUIRE(A && Bm && C, RA_ERR_INVALID, "gemm_bf16: null pointer");
  RA_REQUIRE(M > 0 && N > 0 && K > 0, RA_ERR_INVALID, "gemm_bf16: empty shape");
  RA_REQUIRE(c_dtype == RA_F32 || c_dtype == RA_BF16, RA_ERR_UNSUPPORTED, "gemm_bf16: c_dtype %d", c_dtype);
  return gemm_bf16(A, Bm, C, M, N, K, trans_a, trans_b, c_dtype, beta_one, -1, (hipStream_t)stream);
}

int ra_gemm_bf16_tile(const void* A, const void* Bm, void* C, int32_t M, int32_t N, int32_t K, int32_t trans_a,
                      int32_t trans_b, int32_t c_dtype, int32_t beta_one, int32_t tile, ra_stream_t stream) {
  RA_REQUIRE(A && Bm && C, RA_ERR_INVALID, "gemm_bf16_tile: null pointer");
  RA_REQUIRE(M > 0 && N > 0 && K > 0, RA_ERR_INVALID, "gemm_bf16_tile: empty shape");
  RA_REQUIRE(c_dtype == RA_F32 || c_dtype == RA_BF16, RA_ERR_UNSUPPORTED, "gemm_bf16_tile: c_dtype %d", c_dtype);
  RA_REQUIRE(tile >= -1 && tile <= 3, RA_ERR_INVALID, "gemm_bf16_tile: tile %d outside [-1, 3]", tile);
  return gemm_bf16(A, Bm, C, M, N, K, trans_a, trans_b, c_dtype, beta_one, tile, (hipStream_t)stream);
}

int ra_gemm_bf16_pair(const void* A, const void* B1, const void* B2, void* C1, void* C2, int32_t M, int32_t N,
                      int32_t K, int32_t tile, ra_stream_t stream) {
  RA_REQUIRE(A && B1 && B2 && C1 && C2, RA_ERR_INVALID, "gemm_bf16_pair: null pointer");
  RA_REQUIRE(M > 0 && N > 0 && K > 0, RA_ERR_INVALID, "gemm_bf16_pair: empty shape");
  RA_REQUIRE(tile >= -1 && tile <= 3, RA_ERR_INVALID, "gemm_bf16_pair: tile %d outside [-1, 3]", tile);
  return gemm_bf16_pair(A, B1, B2, C1, C2, M, N, K, tile, (hipStream_t)stream);
}

}  // extern "C"
