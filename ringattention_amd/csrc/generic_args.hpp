// What the generic (vector-ALU) kernels and the element-wise-mask matrix-core kernels share: the argument block and
// the reference's mask evaluated element by element (ringattention_jax.py:272-322, :324-331).
#pragma once
#include "common.hpp"

namespace ra {

struct GenericArgs {
  const void* q; const void* k; const void* v; const void* g;
  int B, Sq, Skv, H, D;
  int64_t q_sb, q_ss, kv_sb, kv_ss;
  float* num; int64_t num_sb, num_ss;
  float* den; float* mx; const float* delta;
  int64_t st_sb, st_sh;
  float* dq; int64_t dq_sb, dq_ss;
  float* dk; float* dv; int64_t dkv_sb, dkv_ss;
  MaskView mv;
  int carry_is_initial;
  int sdim;                                      // head size that scales the logits (the un-padded one)
  void* out; int64_t out_sb, out_ss;             // forward, nullable: out = num / den instead of the numerator
  float* out32;                                  // forward, nullable: the same quotient un-rounded, strides of out
  int dq_initial, dkv_initial;                   // backward: that accumulator holds zeros by definition
  void* dq_out; int64_t dqo_sb, dqo_ss;          // backward, nullable: the sum goes here in the primal dtype
  void* dk_out; void* dv_out; int64_t dkvo_sb, dkvo_ss;
};

__device__ __forceinline__ MaskView resolve_mask(const GenericArgs& a) {
  MaskView mv = a.mv;
  mv.resolve();
  return mv;
}

// per-row constants of the mask
struct RowInfo {
  int kend;        // keys [0,kend) of this shard are in chunks that run for this row
  long long gq_blk;
  int seg;
  int64_t bias_off;
  int64_t keep_off;
  int64_t kbit_off;
};

__device__ __forceinline__ RowInfo row_info(const MaskView& mv, int b, int h, int row, int skv) {
  RowInfo r;
  int qi = row / mv.qc;
  r.kend = mv.run_prefix_keys(qi, skv);
  long long gq = mv.global_q(row);
  r.gq_blk = mv.cbs > 1 ? gq / mv.cbs : (mv.cbs == 1 ? gq : 0);     // block size 1, the usual one: no 64-bit division
  r.seg = 0;
  if (mv.seg) {
    int idx = clamp_seg_index(((long long)mv.q_start + qi) * mv.qc, mv.qc, mv.seg_len, row % mv.qc);
    r.seg = mv.seg[(int64_t)b * mv.seg_sb + idx];
  }
  r.bias_off = (int64_t)b * mv.bias_sb + (int64_t)h * mv.bias_sh + (int64_t)(row % mv.qc) * mv.bias_sq;
  r.keep_off = (int64_t)b * mv.keep_sb + (int64_t)h * mv.keep_sh + (int64_t)row * mv.keep_sq;
  r.kbit_off = (int64_t)b * mv.kpack_sb + (int64_t)h * mv.kpack_sh + mv.keep_q0 + row;
  return r;
}

// logit of (row, local key kj) given the raw dot product; -inf when the pair's tile does not run
__device__ __forceinline__ float logit(const MaskView& mv, const RowInfo& r, float dot, float scale, int kj,
                                       int seg_k) {
  if (kj >= r.kend) return RA_NEG_INF;
  long long gk = mv.global_k(kj);
  float add = 0.f;
  if (mv.bias) {
    add = mv.bias[r.bias_off + gk * mv.bias_sk];
    if (mv.any_mask) add = fminf(add, 0.f);                       // minimum(), :299,:309
  }
  bool masked = (mv.cbs > 0 && r.gq_blk < (mv.cbs == 1 ? gk : gk / mv.cbs)) || (mv.seg && r.seg != seg_k);
  bool off = false;
  if (mv.keep) {
    off = !mv.keep[r.keep_off + (gk - mv.keep_k0) * mv.keep_sk];
  } else if (mv.kbits_k) {            // packed form only: bit (gk - keep_k0) % 64 of the row's word of that key tile
    const long long kk = gk - mv.keep_k0;
    off = !((mv.kbits_k[r.kbit_off + (kk >> 6) * mv.keep_Q] >> (kk & 63)) & 1);
  }
  if (off && mv.keep_drop) {
    // chunk_bias += dropped * finfo.min (:321), before the logit is added: on top of a bias of ordinary size it
    // absorbs bias and logit (finfo.min), on top of finfo.min - a masked pair, or a bias at that level (a padding
    // mask) - it overflows to -inf
    return dot / scale + ((masked ? mv.mask_min : add) + mv.mask_min);
  }
  if (off) masked = true;                  // where(mask, w, finfo.min), ringattention_inference.py:24
  if (masked) add = mv.mask_min;
  return dot / scale + add;                                       // :134-136
}

inline GenericArgs make_args_fwd(const ra_attn_fwd_params* p) {
  GenericArgs a{};
  a.q = p->q; a.k = p->k; a.v = p->v; a.g = nullptr;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H; a.D = p->D;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.num = p->numerator; a.num_sb = p->num_stride_b; a.num_ss = p->num_stride_s;
  a.den = p->denominator; a.mx = p->max_score; a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  a.carry_is_initial = p->carry_is_initial;
  a.sdim = p->logit_dim > 0 ? p->logit_dim : p->D;
  a.out = p->out; a.out_sb = p->out_stride_b; a.out_ss = p->out_stride_s; a.out32 = p->out_f32;
  return a;
}


inline GenericArgs make_args_bwd(const ra_attn_bwd_params* p) {
  GenericArgs a{};
  a.q = p->q; a.k = p->k; a.v = p->v; a.g = p->g;
  a.B = p->B; a.Sq = p->Sq; a.Skv = p->Skv; a.H = p->H; a.D = p->D;
  a.q_sb = p->q_stride_b; a.q_ss = p->q_stride_s; a.kv_sb = p->kv_stride_b; a.kv_ss = p->kv_stride_s;
  a.den = const_cast<float*>(p->denominator); a.mx = const_cast<float*>(p->max_score); a.delta = p->delta;
  a.st_sb = p->stat_stride_b; a.st_sh = p->stat_stride_h;
  a.dq = p->dq; a.dq_sb = p->dq_stride_b; a.dq_ss = p->dq_stride_s;
  a.dk = p->dk; a.dv = p->dv; a.dkv_sb = p->dkv_stride_b; a.dkv_ss = p->dkv_stride_s;
  a.sdim = p->logit_dim > 0 ? p->logit_dim : p->D;
  a.dq_initial = (p->grads_are_initial & RA_GRAD_INIT_DQ) != 0;
  a.dkv_initial = (p->grads_are_initial & RA_GRAD_INIT_DKV) != 0;
  a.dq_out = p->dq_out; a.dqo_sb = p->dq_out_stride_b; a.dqo_ss = p->dq_out_stride_s;
  a.dk_out = p->dk_out; a.dv_out = p->dv_out; a.dkvo_sb = p->dkv_out_stride_b; a.dkvo_ss = p->dkv_out_stride_s;
  a.mv = MaskView::make(p->mask, p->mask.q_chunk_idx_start);
  return a;
}

}  // namespace ra
