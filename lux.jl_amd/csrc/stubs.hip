// Entry points that are declared in the header but whose kernels are not written yet.
#include "common.h"
using namespace luxhip;
extern "C" {
#define NOT_YET(name) return set_error(LUXHIP_UNSUPPORTED, name ": not implemented yet")
int luxhip_matmul(luxhip_stream_t, int, int, int, int64_t, int64_t, int64_t, const void*, int64_t, const void*, int64_t, const void*, void*, int64_t) { NOT_YET("matmul"); }
int luxhip_fused_dense_fwd(luxhip_stream_t, int, int, int64_t, int64_t, int64_t, const void*, int64_t, const void*, int64_t, const void*, void*, int64_t, void*) { NOT_YET("fused_dense_fwd"); }
int luxhip_fused_dense_bwd(luxhip_stream_t, int, int, int64_t, int64_t, int64_t, const void*, const void*, const void*, const void*, int64_t, const void*, int64_t, void*, void*, void*, void*) { NOT_YET("fused_dense_bwd"); }
int luxhip_conv_fwd(luxhip_stream_t, int, int, const luxhip_conv_dims_t*, const void*, const void*, const void*, void*, void*) { NOT_YET("conv_fwd"); }
int luxhip_conv_bwd_data(luxhip_stream_t, int, const luxhip_conv_dims_t*, const void*, const void*, void*) { NOT_YET("conv_bwd_data"); }
int luxhip_conv_bwd_filter(luxhip_stream_t, int, const luxhip_conv_dims_t*, const void*, const void*, void*) { NOT_YET("conv_bwd_filter"); }
int luxhip_fused_conv_bwd(luxhip_stream_t, int, int, const luxhip_conv_dims_t*, const void*, const void*, const void*, const void*, const void*, void*, void*, void*, void*) { NOT_YET("fused_conv_bwd"); }
}
