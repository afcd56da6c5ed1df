/*
 * C-ABI of libringattn_hip.so: the per-device hot path of ring attention with
 * blockwise transformers, written for MI355X (gfx950).
 *
 * Every entry point enqueues work on the caller's HIP stream and returns; none
 * allocates, frees, retains a pointer or synchronises the device.  All pointers
 * are device pointers owned by the caller.  Return value: RA_OK or an RA_ERR_*
 * code; ra_last_error() gives the text of the calling thread's last failure.
 *
 * Tensor layout (the reference's, ringattention/ringattention_jax.py:20-23):
 *   q, k, v, out, gradients, numerator      (B, S, H, D), D contiguous, head stride D
 *   denominator, max_score, delta           (B, H, S),    S contiguous
 * Sequence and batch strides are explicit (in elements) so that a ring shard can
 * be a slice of the caller's global array.
 */
#ifndef RINGATTN_HIP_H_
#define RINGATTN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* ra_stream_t; /* == hipStream_t */

/* Version of this interface: bumped whenever a struct below grows or a signature changes.  ra_version() returns the
 * value the library was built with; a binding compares the two before its first call (the ctypes binding does). */
#define RA_ABI_VERSION 2

enum { RA_OK = 0, RA_ERR_INVALID = 1, RA_ERR_UNSUPPORTED = 2, RA_ERR_LAUNCH = 3 };
enum { RA_F32 = 0, RA_BF16 = 1 };

/* kernel family selector (ra_attn_*_params.impl) */
enum {
  RA_IMPL_AUTO = 0,    /* MFMA kernels when the shape allows, else the generic ones */
  RA_IMPL_GENERIC = 1, /* fp32 vector-ALU kernels: any chunk sizes, fp32 or bf16 inputs */
  RA_IMPL_MFMA = 2,    /* the tiled matrix-core kernels only (bf16 inputs: v_mfma_f32_32x32x16_bf16, fp32 inputs:
                          v_mfma_f32_32x32x2_f32; head size 64 or 128, chunk sizes multiples of 128);
                          RA_ERR_UNSUPPORTED if the shape does not fit */
  RA_IMPL_MFMA_ANY = 3 /* the matrix-core kernels that evaluate the mask element by element only (bf16 inputs, head
                          size 128 or 256; any chunk sizes and lengths, a bias per row, a boolean mask in bytes; no
                          attention dropout): what RA_IMPL_AUTO falls back to before the generic kernels;
                          RA_ERR_UNSUPPORTED if the call does not fit */
};

/*
 * The additive-bias / mask description of one (ring step, device):
 * what _chunk_attention_bias (ringattention_jax.py:272-322) and below_or_on_diag
 * (:324-331) take, in global chunk coordinates.
 */
typedef struct ra_mask {
  const float* bias;          /* nullable; values already rounded to blockwise_kwargs["dtype"] */
  int64_t bias_stride_b;      /* element strides; 0 broadcasts that axis */
  int64_t bias_stride_h;
  int64_t bias_stride_q;      /* indexed by the row INSIDE the query chunk (:281 slices rows 0:qc) */
  int64_t bias_stride_k;      /* indexed by the GLOBAL key position (:281) */
  const int32_t* segment_ids; /* nullable; (B or 1, seg_len), indexed by GLOBAL positions (:286-295) */
  int64_t seg_stride_b;
  int32_t seg_len;
  int32_t causal_block_size;  /* 0 = None */
  int32_t query_chunk_size;
  int32_t key_chunk_size;
  int32_t q_chunk_idx_start;  /* :33 ; ignored when cache_idx is given */
  int32_t k_chunk_idx_start;  /* :37 */
  const int32_t* cache_idx;   /* nullable device scalar: q_chunk_idx_start = *cache_idx / query_chunk_size (:35) */
  const int32_t* chunk_starts; /* nullable device pair {q_chunk_idx_start, k_chunk_idx_start}: read by the kernels in
                                 place of the two host ints above.  Under jit both come from lax.axis_index
                                 (:31-37, :69-75), a traced value that a custom call receives as a buffer and cannot
                                 read without a sync; the kernels derive which tiles run from it themselves, so a
                                 call whose every tile is skipped still launches (and passes its rows on).  cache_idx,
                                 when given too, still decides the query start.  Not together with a keep mask (its
                                 slices are laid out by the host) and not in a ring-step launch. */
  float mask_min;             /* finfo(blockwise_kwargs["dtype"]).min (:298,:308) */
  int32_t skip_masked_tiles;  /* 1: kernels may also skip sub-tiles whose every pair is masked; exact
                                 unless a query row has no unmasked key at all in the whole ring */
  const int32_t* seg_tile_minmax; /* nullable; from ra_segment_tile_ranges: (B or 1, seg_tiles, 2) = min and max
                                     segment id of every run of RA_SEG_TILE global positions.  With
                                     skip_masked_tiles it lets kernels skip key (query) tiles whose id range
                                     cannot meet the ids of the query (key) rows at hand */
  int32_t seg_tiles;
  const int32_t* seg_run_hulls;   /* nullable; from ra_segment_run_hulls: (B or 1, seg_runs, 2) = for every run of
                                     2 * RA_SEG_TILE global positions the first and one-past-the-last tile (of
                                     RA_SEG_TILE positions, over the whole sequence) whose id range meets the run's.
                                     Lets a workgroup find its key (query) tiles with two loads instead of a scan.
                                     Only when segment_ids covers every position the call touches */
  int32_t seg_runs;               /* ceil(seg_tiles / 2) */
  const uint8_t* keep;        /* nullable; a boolean mask, nonzero = attend.  keep_mode says what a zero does:
                                 RA_KEEP_WHERE, the attn_mask of ring_attention_inference
                                 (ringattention_inference.py:19-22): the logit becomes mask_min;
                                 RA_KEEP_DROPOUT, the attention dropout mask (ringattention_jax.py:311-321, zero =
                                 dropped): mask_min is ADDED to the logit and its bias, so the logit becomes mask_min,
                                 or -inf where segment ids or the causal mask had already set it to mask_min.
                                 Indexed by the LOCAL query row of the call and by the GLOBAL key position minus
                                 keep_k0; only the generic kernels take this byte form (they read the packed
                                 form below when keep is null) */
  int64_t keep_stride_b;      /* element (byte) strides; 0 broadcasts that axis */
  int64_t keep_stride_h;
  int64_t keep_stride_q;
  int64_t keep_stride_k;
  /* Packed forms of the same mask from ra_keep_pack, which let the MFMA kernels take it (all three null:
     generic kernels only).  They cover the GLOBAL mask (keep_q_total x keep_k_total, both multiples of 64);
     keep_q0 is the global row of the call's local query row 0 (a multiple of 64), keep_k0 the global key position
     of the mask's column 0 (a multiple of 64; 0 when the mask spans the global key axis). */
  const uint64_t* keep_bits_k;   /* [b][h][k_total/64][q_total]: bit i = keep[q][64 kt + i] */
  const uint64_t* keep_bits_q;   /* [b][h][q_total/64][k_total]: bit i = keep[64 qt + i][k] */
  const uint8_t* keep_summary;   /* [b][h][q_total/64][k_total/64]: 0 none kept, 1 mixed, 2 all kept */
  int64_t keep_pack_stride_b;    /* of both bit arrays, in 64-bit words; 0 broadcasts */
  int64_t keep_pack_stride_h;
  int64_t keep_sum_stride_b;     /* of keep_summary, in bytes; 0 broadcasts */
  int64_t keep_sum_stride_h;
  int32_t keep_q_total, keep_k_total, keep_q0;
  int32_t keep_k0;
  int32_t keep_mode;             /* RA_KEEP_WHERE | RA_KEEP_DROPOUT */
} ra_mask;

enum { RA_KEEP_WHERE = 0, RA_KEEP_DROPOUT = 1 };

/* _blockwise_attention_fwd (ringattention_jax.py:99-179): one ring step on one device.
 * Updates the carry (numerator, denominator, max_score) in place. */
typedef struct ra_attn_fwd_params {
  const void* q; const void* k; const void* v;
  int32_t dtype;              /* RA_F32 | RA_BF16, of q, k and v */
  int32_t B, Sq, Skv, H, D;
  int64_t q_stride_b, q_stride_s;     /* elements */
  int64_t kv_stride_b, kv_stride_s;
  float* numerator;  int64_t num_stride_b, num_stride_s;   /* (B,Sq,H,D) fp32 */
  float* denominator; float* max_score;                    /* (B,H,Sq) fp32 */
  int64_t stat_stride_b, stat_stride_h;
  ra_mask mask;
  int32_t impl;
  int32_t carry_is_initial;   /* 1: the carry holds (0, 0, -inf) by definition; kernels need not read it */
  void* out;                  /* nullable.  When given, this call is the LAST ring step of its device: out =
                                 numerator / denominator (:52) is written here in `dtype`, (B,Sq,H,D) with the strides
                                 below, and the numerator is not written back (it may then be null when
                                 carry_is_initial); denominator and max_score are updated as always (they are
                                 residuals, :53).  Saves the numerator's round trip through memory and
                                 ra_attn_finalize */
  int64_t out_stride_b, out_stride_s;
  int32_t logit_dim;          /* the head size whose square root divides the logits (:118, :134); 0 = D.  For callers
                                 that hand over q, k, v zero-padded along D to a head size the matrix-core kernels
                                 take (the products are those of the un-padded rows, the scale must stay the
                                 original's) */
  float* out_f32;             /* nullable, only together with `out`: the same quotient BEFORE it is rounded to `dtype`,
                                 (B,Sq,H,D) fp32 with the element strides of `out`.  It is the `output` the reference
                                 keeps as a residual (:53) and multiplies with the cotangent in its backward pass
                                 (:218); ra_attn_bwd_delta takes it in place of the rounded `out` */
} ra_attn_fwd_params;

/* _blockwise_attention_bwd (ringattention_jax.py:181-270): adds this step's gradients into the
 * fp32 accumulators dq (Sq side) and dk, dv (Skv side). */
typedef struct ra_attn_bwd_params {
  const void* q; const void* k; const void* v; const void* g;   /* g: cotangent of out, same dtype */
  int32_t dtype;
  int32_t B, Sq, Skv, H, D;
  int64_t q_stride_b, q_stride_s;     /* q and g */
  int64_t kv_stride_b, kv_stride_s;
  const float* delta;                 /* (B,H,Sq): sum_d g*out (:218), from ra_attn_bwd_delta */
  const float* denominator; const float* max_score;
  int64_t stat_stride_b, stat_stride_h;
  float* dq; int64_t dq_stride_b, dq_stride_s;
  float* dk; float* dv; int64_t dkv_stride_b, dkv_stride_s;
  ra_mask mask;
  int32_t impl;
  int32_t grads_are_initial;  /* RA_GRAD_INIT_DQ | RA_GRAD_INIT_DKV: that accumulator holds zeros by definition
                                 (:61-63): it is not read, and may be null when the matching *_out is given */
  void* dq_out;               /* nullable.  When given, this call is the LAST one that adds into this dq: the sum is
                                 written here in `dtype` (the cast of :89), (B,Sq,H,D), and the fp32 dq is left as it
                                 was */
  int64_t dq_out_stride_b, dq_out_stride_s;
  void* dk_out; void* dv_out; /* the same for dk and dv (both or neither), (B,Skv,H,D) */
  int64_t dkv_out_stride_b, dkv_out_stride_s;
  int32_t logit_dim;          /* as in ra_attn_fwd_params; 0 = D */
} ra_attn_bwd_params;

enum { RA_GRAD_INIT_DQ = 1, RA_GRAD_INIT_DKV = 2 };

enum { RA_SEG_TILE = 64 };
/* min / max segment id per run of RA_SEG_TILE positions: out (Bseg, ceil(seg_len / RA_SEG_TILE), 2).
 * No counterpart in the reference (it evaluates the segment mask element by element, :285-299); this
 * only feeds the tile-skipping of the kernels. */
int ra_segment_tile_ranges(const int32_t* segment_ids, int64_t seg_stride_b, int32_t Bseg, int32_t seg_len,
                           int32_t* out, ra_stream_t stream);

/* From the ranges of ra_segment_tile_ranges (minmax: (Bseg, seg_tiles, 2)) to ra_mask.seg_run_hulls:
 * out (Bseg, ceil(seg_tiles / 2), 2).  No counterpart in the reference; only feeds the tile skipping. */
int ra_segment_run_hulls(const int32_t* seg_tile_minmax, int32_t Bseg, int32_t seg_tiles, int32_t* out,
                         ra_stream_t stream);

/* Packs a boolean mask (nonzero = attend; byte strides, 0 broadcasts an axis) of Q x K positions, both
 * multiples of 64, into the three arrays ra_mask.keep_bits_k / keep_bits_q / keep_summary describe, for Bm x Hm
 * (batch, head) planes.  No counterpart in the reference (ringattention_inference.py:22 applies the mask
 * element by element); this only lets the MFMA kernels read 64 mask bits per load and skip uniform tiles. */
int ra_keep_pack(const uint8_t* keep, int64_t stride_b, int64_t stride_h, int64_t stride_q, int64_t stride_k,
                 int32_t Bm, int32_t Hm, int32_t Q, int32_t K, uint64_t* bits_k, uint64_t* bits_q,
                 uint8_t* summary, ra_stream_t stream);

/* The attention dropout mask of ringattention_jax.py:119-121 / :206-208 (jax.random.bernoulli(rng, attn_pdrop,
 * (batch, heads, q_len, kv_len)), true = dropped), written as the boolean KEEP mask ra_mask.keep takes with
 * RA_KEEP_DROPOUT: keep (B, H, Q, K) dense bytes, 1 = attend, 0 = dropped.  The bits do not come from the
 * jax.random stream (threefry, not restated) but from Philox4x32-10 (Salmon et al., SC'11), 16 bits a position,
 * one block per eight consecutive key positions:
 *   e = ((b * H + h) * Q + q) * K + k          (position in the dense mask; K is a multiple of 8)
 *   block = philox4x32_10(counter = (lo32(e / 8), hi32(e / 8), 0, 0), key = (lo32(seed), hi32(seed)))
 *   half  = e % 8;  r = 16 bits of block[half / 2]: the low half for even half, the high half for odd
 *   dropped(e) = r < floor(attn_pdrop * 2^16)
 * so the mask is a pure function of (seed, attn_pdrop, shape); forward and backward pass take the same array. */
int ra_dropout_keep(uint64_t seed, float attn_pdrop, int32_t B, int32_t H, int32_t Q, int32_t K, uint8_t* keep,
                    ra_stream_t stream);
/* The same mask written directly in the packed form of ra_keep_pack (Q and K multiples of 64), without the byte
 * array: what ra_keep_pack would make of ra_dropout_keep's output.  The attention entry points take the packed
 * form alone (ra_mask.keep null).  With causal_block_size > 0 (and the chunk sizes and chunk starts of the ring step
 * the mask is for, as in ra_mask) only the 64 x 64 tiles of chunk pairs that below_or_on_diag lets run
 * (ringattention_jax.py:324-331) are written - about half of them in causal self-attention - and the others are left
 * as they are: no kernel reads them.  The bits of a position do not depend on which tiles are written. */
int ra_dropout_keep_packed(uint64_t seed, float attn_pdrop, int32_t B, int32_t H, int32_t Q, int32_t K,
                           uint64_t* bits_k, uint64_t* bits_q, uint8_t* summary, int32_t causal_block_size,
                           int32_t query_chunk_size, int32_t key_chunk_size, int32_t q_chunk_idx_start,
                           int32_t k_chunk_idx_start, ra_stream_t stream);

/* Carry initialisation (ringattention_jax.py:22-23,:49): numerator = 0, denominator = 0, max = -inf. */
int ra_attn_carry_init(float* numerator, int64_t num_stride_b, int64_t num_stride_s,
                       float* denominator, float* max_score, int64_t stat_stride_b, int64_t stat_stride_h,
                       int32_t B, int32_t Sq, int32_t H, int32_t D, ra_stream_t stream);

/* _blockwise_attention_fwd, ringattention_jax.py:99-179 (called at :38-46). */
int ra_attn_fwd_block(const ra_attn_fwd_params* p, ra_stream_t stream);

/* Which kernel family ra_attn_fwd_block / ra_attn_bwd_block would run for these params (nothing is launched), or 0
 * when the call would be refused.  The generic kernels serve every shape but run on the vector ALU, two orders of
 * magnitude below the matrix-core kernels on long sequences: a caller that lets RA_IMPL_AUTO choose can ask here
 * what it got (the Python layer warns once when a large problem lands on them). */
enum { RA_FAMILY_GENERIC = 1, RA_FAMILY_MFMA_BF16 = 2, RA_FAMILY_MFMA_F32 = 3, RA_FAMILY_MFMA_BF16_ANY = 4 };
int ra_attn_fwd_family(const ra_attn_fwd_params* p);
int ra_attn_bwd_family(const ra_attn_bwd_params* p);

/* output = numerator / denominator, cast (ringattention_jax.py:52-53).  out_dtype RA_F32|RA_BF16. */
int ra_attn_finalize(const float* numerator, int64_t num_stride_b, int64_t num_stride_s,
                     const float* denominator, int64_t stat_stride_b, int64_t stat_stride_h,
                     void* out, int32_t out_dtype, int64_t out_stride_b, int64_t out_stride_s,
                     int32_t B, int32_t Sq, int32_t H, int32_t D, ra_stream_t stream);

/* delta[b,h,s] = sum_d g*out (ringattention_jax.py:218).  g: the cotangent in `dtype`; out: the forward output,
 * either rounded (out_dtype == dtype) or the un-rounded fp32 quotient (out_dtype RA_F32, from out_f32 of the last
 * forward step: what the reference multiplies, :53).  Same element strides for both. */
int ra_attn_bwd_delta(const void* g, const void* out, int32_t dtype, int32_t out_dtype, int64_t stride_b,
                      int64_t stride_s, float* delta, int64_t stat_stride_b, int64_t stat_stride_h,
                      int32_t B, int32_t Sq, int32_t H, int32_t D, ra_stream_t stream);

/* _blockwise_attention_bwd, ringattention_jax.py:181-270 (called at :76-84). */
int ra_attn_bwd_block(const ra_attn_bwd_params* p, ra_stream_t stream);

/*
 * One step of the ring loop for EVERY device of a ring whose devices all live on this GPU: the body of the
 * lax.scan at ringattention_jax.py:29-51 (forward) / :65-88 (backward) as the devices of a mesh run it side by side,
 * in one launch per kernel instead of one per device.  In step idx device d holds the K/V shard
 * (d - idx) mod n_dev (:36, :72).  The params describe the GLOBAL arrays: Sq and Skv are the whole sequence lengths
 * (n_dev shards of Sq / n_dev and Skv / n_dev positions, device d owning query shard d), mask.q_chunk_idx_start /
 * k_chunk_idx_start are ignored (each device gets d * q_len / query_chunk_size and shard * kv_len / key_chunk_size,
 * :32-33, :37), and carry_is_initial / grads_are_initial / the nullness of out, dq_out, dk_out, dv_out as "last step"
 * markers are replaced by the per-device bits below (the output pointers must be non-null when any bit asks for
 * them).  Results are bit-identical to the n_dev separate ra_attn_fwd_block / ra_attn_bwd_block calls.
 * MFMA kernels only (RA_ERR_UNSUPPORTED otherwise: fall back to the per-device calls); no keep mask, no cache_idx.
 */
typedef struct ra_ring_step {
  int32_t n_dev;      /* ring size, 1 .. 64 */
  int32_t idx;        /* scan index, 0 .. n_dev - 1 */
  uint64_t run;       /* bit d: device d runs this step; the rows of the others are left untouched */
  uint64_t first;     /* bit d: forward, the carry of device d is initial; backward, its dq is initial */
  uint64_t last;      /* bit d: forward, device d writes out; backward, it writes dq_out */
  uint64_t kv_first;  /* backward, bit s: dk / dv of K/V SHARD s (held by device (s + idx) mod n_dev) are initial */
  uint64_t kv_last;   /* backward, bit s: dk_out / dv_out of shard s are written */
} ra_ring_step;
int ra_attn_fwd_ring_step(const ra_attn_fwd_params* p, const ra_ring_step* ring, ra_stream_t stream);
int ra_attn_bwd_ring_step(const ra_attn_bwd_params* p, const ra_ring_step* ring, ra_stream_t stream);

/*
 * Decode: the cache_idx path (ringattention_jax.py:31-35 with q_len == 1): one query token per
 * batch row against the whole KV cache buffer, streamed once.  Same mask semantics as above with
 * query_chunk_size == 1.  workspace: ra_decode_workspace_bytes() bytes of device memory.
 */
typedef struct ra_decode_params {
  const void* q;              /* (B,1,H,D) */
  const void* k; const void* v;   /* (B,L,H,D) cache buffers */
  void* out;                  /* (B,1,H,D), same dtype */
  int32_t dtype;
  int32_t B, L, H, D;
  int64_t q_stride_b, kv_stride_b, kv_stride_s, out_stride_b;
  ra_mask mask;               /* query_chunk_size must be 1; cache_idx pointer or q_chunk_idx_start */
  void* workspace; size_t workspace_bytes;
  int32_t num_splits;         /* 0 = choose */
  /* One step of a ring whose K/V cache is sharded over the sequence axis (ringattention_jax.py:31-37 with cache_idx
     and an axis size above one): k, v are then the shard that has arrived, mask.k_chunk_idx_start its first chunk
     (:37), and the step's result is merged into the carry of the device's one query row instead of being
     normalised - numerator (B,1,H,D) fp32, denominator and max_score (B,H,1) fp32, updated in place as
     _blockwise_attention_fwd does (:138-144); the max is the natural-domain one, as in ra_attn_fwd_params.  All three
     null: no carry, out = the normalised result (a ring of one).  With a carry, out may be null (the step hands the
     carry on); when given, the step is the last one of its device and out = numerator / denominator (:52). */
  float* carry_numerator; float* carry_denominator; float* carry_max_score;
  int64_t carry_num_stride_b;   /* elements; head stride D */
  int64_t carry_stat_stride_b;  /* elements; head stride 1 */
  int32_t carry_is_initial;     /* 1: the carry holds (0, 0, -inf) by definition and is not read */
} ra_decode_params;

/* num_splits == 0: the size for the largest split count the library may choose (256); a caller that wants no more
 * than the automatic choice needs asks ra_decode_auto_splits first and passes that count here and in the params. */
size_t ra_decode_workspace_bytes(int32_t B, int32_t L, int32_t H, int32_t D, int32_t num_splits);
/* The split count ra_decode_fwd picks for num_splits == 0 (0 for a shape it does not take). */
int ra_decode_auto_splits(int32_t B, int32_t L, int32_t H, int32_t D, int32_t dtype);
int ra_decode_fwd(const ra_decode_params* p, ra_stream_t stream);

/*
 * ra_decode_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same computation and same kernels as
 * ra_decode_fwd, but the split-KV partials go to a buffer that lives inside the library (a file-scope device array
 * of RA_DECODE_STATIC_SCRATCH_BYTES per GPU, held until the process ends) instead of p->workspace, which is ignored
 * together with p->workspace_bytes.  The call allocates and frees nothing.  The number of key splits is
 * p->num_splits, or the automatic choice, lowered to what fits the buffer:
 *   B * H * splits * (D + 2) * sizeof(float) <= RA_DECODE_STATIC_SCRATCH_BYTES;
 * a shape whose single split does not fit (B * H * (D + 2) * 4 bytes above the limit) is refused with
 * RA_ERR_UNSUPPORTED.  Every call on a GPU shares that GPU's buffer: two calls that overlap in time on one GPU (two
 * streams, two threads) race; calls on one stream are ordered.  Nothing in the buffer has to start at zero: every
 * partial a call reads was written by that call.
 * The first call on a GPU looks the array's address up (hipGetSymbolAddress, which may load the code object, under a
 * mutex): make one eager call per GPU before capturing this entry point into a HIP graph; later calls only launch.
 * The GPU that owns `stream` must be the current device (refused otherwise): each GPU has its own copy of the array.
 */
enum { RA_DECODE_STATIC_SCRATCH_BYTES = 16 * 1024 * 1024 };
int ra_decode_fwd_static(const ra_decode_params* p, ra_stream_t stream);

/*
 * SwiGLU feed-forward on one chunk of tokens, the body that blockwise_feedforward
 * (ringattention_jax.py:333-352) scans: y = (silu(x w1) * (x w3)) w2, bf16, fp32 accumulation.
 * x (T,d) ; w1,w3 (d,f) ; w2 (f,d) ; row-major.  a,b (T,f) bf16 are written by the forward
 * (pre-activations) and read by the backward, which recomputes them first unless preact_saved is set.
 */
typedef struct ra_swiglu_params {
  int32_t T, d, f;
  const void* x; const void* w1; const void* w2; const void* w3;
  void* a; void* b; void* h;      /* (T,f) bf16 scratch: x w1, x w3, silu(a)*b */
  void* y;                        /* (T,d) bf16 */
  /* backward only */
  const void* dy;                 /* (T,d) */
  void* dx;                       /* (T,d) */
  float* dw1; float* dw2; float* dw3;   /* fp32 accumulators, added into (weights are broadcast
                                           over the scan, so their gradients sum over chunks) */
  void* da; void* db;             /* (T,f) bf16 scratch */
  int32_t preact_saved;           /* backward: 1 = a and b still hold what the forward wrote for these tokens (the
                                     caller kept them: `policy` other than nothing_saveable, ringattention_jax.py:334);
                                     0 = recompute them from x (the reference's default policy) */
  int32_t defer_weight_grads;     /* backward: 1 = leave dw1, dw2, dw3 alone (they may be null); the caller adds them
                                     later with ra_swiglu_weight_grads, over the tokens of several consecutive calls
                                     at once - their h, da, db kept side by side - so that the fp32 accumulators are
                                     read and written once per group instead of once per call */
  int32_t gemm_tile;              /* 0: the library picks the tile kernel of each product (the default).  1 + t forces
                                     tile kernel t wherever the shape divides (0: 256 x 256 over four wavefronts,
                                     1: 256 x 128 over eight, 2: 128 x 128, 3: 256 x 128 over four), so that tests reach every
                                     kernel */
} ra_swiglu_params;

int ra_swiglu_fwd(const ra_swiglu_params* p, ra_stream_t stream);
int ra_swiglu_bwd(const ra_swiglu_params* p, ra_stream_t stream);
/* The weight gradients alone, for T tokens whose h, da, db an earlier ra_swiglu_bwd (with defer_weight_grads) left
 * in the buffers of p: dw1 += x^T da, dw3 += x^T db, dw2 += h^T dy (the sums over chunks of ringattention_jax.py:344-350,
 * whose weights are broadcast over the scan).  Reads x, dy, h, da, db, T, d, f, gemm_tile. */
int ra_swiglu_weight_grads(const ra_swiglu_params* p, ra_stream_t stream);

/* C (M,N) = op(A) op(B), bf16 inputs, fp32 accumulation.  trans_a: A is stored (K,M); trans_b: B is
 * stored (N,K).  c_dtype RA_BF16 (overwrite) or RA_F32 (accumulate when beta_one != 0). */
int ra_gemm_bf16(const void* A, const void* Bm, void* C, int32_t M, int32_t N, int32_t K,
                 int32_t trans_a, int32_t trans_b, int32_t c_dtype, int32_t beta_one, ra_stream_t stream);

/*
 * Steps either side of the hot path (the reference repository has no counterpart: its README points at the LWM
 * model code for them; the formulas are the LLaMA ones).
 *
 * ra_rope_kv_append: before a decode step.  Rotates the new token's query and key by position pos = *cache_idx
 * (or cache_idx_host when cache_idx is null): pair (x0, x1) -> (x0 cos a - x1 sin a, x0 sin a + x1 cos a),
 * a = pos * rope_theta^(-2j/D), j = 0 .. D/2-1, pairs (2j, 2j+1) [RA_ROPE_ADJACENT] or (j, j+D/2) [RA_ROPE_HALF];
 * writes the rotated key and the value into the cache buffers at position pos of every batch row - the buffers
 * that ra_decode_fwd / ringattention(..., cache_idx) then read whole (ringattention_jax.py:31-35).  rope_theta <= 0
 * appends without rotating.  A position outside [0, L) writes nothing.
 */
enum { RA_ROPE_ADJACENT = 0, RA_ROPE_HALF = 1 };
typedef struct ra_rope_append_params {
  const void* q; void* q_out;             /* (B,1,H,D); q_out may alias q */
  const void* k_new; const void* v_new;   /* (B,1,H,D) */
  void* k_cache; void* v_cache;           /* (B,L,H,D) */
  const int32_t* cache_idx;               /* device int32 scalar, nullable */
  int32_t cache_idx_host;
  int32_t dtype;
  int32_t B, L, H, D;
  int64_t q_stride_b, q_out_stride_b, new_stride_b, cache_stride_b, cache_stride_s;   /* elements; head stride D */
  float rope_theta;
  int32_t rope_style;
} ra_rope_append_params;
int ra_rope_kv_append(const ra_rope_append_params* p, ra_stream_t stream);

/*
 * ra_rmsnorm_fwd / _bwd: around blockwise_feedforward (ringattention_jax.py:333-352).  bf16 rows of d elements
 * (d a multiple of 8, at most 8192), fp32 arithmetic:
 *   forward   y = x + residual (residual nullable: then y is not written and y = x), rstd = rsqrt(mean(y^2) + eps),
 *             normed = y * rstd * weight
 *   backward  d_y = rstd * (d_normed * weight) - y * rstd^3 / d * sum(d_normed * weight * y) (+ d_residual, nullable),
 *             d_weight += sum over rows of d_normed * y * rstd      (fp32, added into)
 * dw_workspace: ra_rmsnorm_workspace_bytes(T, d) bytes, backward only.
 */
typedef struct ra_rmsnorm_params {
  int64_t T; int32_t d; float eps;
  const void* x; const void* residual; const void* weight;
  void* y; void* normed; float* rstd;                 /* rstd (T) fp32: written by the forward, read by the backward */
  const void* d_normed; const void* d_residual;       /* backward */
  void* d_y; float* d_weight; float* dw_workspace; size_t dw_workspace_bytes;
} ra_rmsnorm_params;
size_t ra_rmsnorm_workspace_bytes(int64_t T, int32_t d);
int ra_rmsnorm_fwd(const ra_rmsnorm_params* p, ra_stream_t stream);
int ra_rmsnorm_bwd(const ra_rmsnorm_params* p, ra_stream_t stream);

const char* ra_last_error(void);
int ra_version(void);

#ifdef __cplusplus
}
#endif
#endif /* RINGATTN_HIP_H_ */
