#include "common.hpp"
namespace ra {
int swiglu_fwd(const ra_swiglu_params*, hipStream_t) { set_error("swiglu: not built"); return RA_ERR_UNSUPPORTED; }
int swiglu_bwd(const ra_swiglu_params*, hipStream_t) { set_error("swiglu: not built"); return RA_ERR_UNSUPPORTED; }
int gemm_bf16(const void*, const void*, void*, int, int, int, int, int, int, int, hipStream_t) { set_error("gemm: not built"); return RA_ERR_UNSUPPORTED; }
}
