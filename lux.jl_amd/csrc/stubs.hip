// Entry points that are declared in the header but whose kernels are not written yet.
#include "common.h"
using namespace luxhip;
extern "C" {
#define NOT_YET(name) return set_error(LUXHIP_UNSUPPORTED, name ": not implemented yet")
int luxhip_conv_fwd(luxhip_stream_t, int, int, const luxhip_conv_dims_t*, const void*, const void*, const void*, void*, void*) { NOT_YET("conv_fwd"); }
int luxhip_conv_bwd_data(luxhip_stream_t, int, const luxhip_conv_dims_t*, const void*, const void*, void*) { NOT_YET("conv_bwd_data"); }
int luxhip_conv_bwd_filter(luxhip_stream_t, int, const luxhip_conv_dims_t*, const void*, const void*, void*) { NOT_YET("conv_bwd_filter"); }
int luxhip_fused_conv_bwd(luxhip_stream_t, int, int, const luxhip_conv_dims_t*, const void*, const void*, const void*, const void*, const void*, void*, void*, void*, void*) { NOT_YET("fused_conv_bwd"); }
}
