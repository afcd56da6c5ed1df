#include "common.hpp"
namespace ra {
bool attn_fwd_mfma_supported(const ra_attn_fwd_params*) { return false; }
bool attn_bwd_mfma_supported(const ra_attn_bwd_params*) { return false; }
int attn_fwd_mfma(const ra_attn_fwd_params*, hipStream_t) { set_error("mfma fwd: not built"); return RA_ERR_UNSUPPORTED; }
int attn_bwd_mfma(const ra_attn_bwd_params*, hipStream_t) { set_error("mfma bwd: not built"); return RA_ERR_UNSUPPORTED; }
}
