// Host-side helpers shared by the C-ABI entry points: error reporting and launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hgq_hip.h"

namespace hgq {

int fail(int code, const char *fmt, ...);  // records a thread-local message, returns `code`

inline int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HGQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return HGQ_OK;
}

// Number of workgroups for a persistent (grid-stride) launch: enough to fill all 256 CUs of
// an MI355X several times over without exceeding the work available.
inline int persistent_grid(int64_t work_items, int per_cu = 4) {
    static int n_cu = 0;
    if (n_cu == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            n_cu = prop.multiProcessorCount;
        if (n_cu <= 0) n_cu = 256;
    }
    int64_t g = (int64_t)n_cu * per_cu;
    if (g > work_items) g = work_items;
    if (g < 1) g = 1;
    return (int)g;
}

__global__ void fill_u32_kernel(uint32_t *p, uint32_t v, int64_t n);
int fill_u32(uint32_t *p, uint32_t v, int64_t n, hipStream_t s);
inline int fill_f32(float *p, float v, int64_t n, hipStream_t s) {
    union {
        float f;
        uint32_t u;
    } c;
    c.f = v;
    return fill_u32((uint32_t *)p, c.u, n, s);
}

// out[e] = sum over the n_parts slices of part[slice][e] (slice length M), in a fixed order; the
// first n_dqw entries go to dqw, the next n_dqb to dqb, the remaining n_df to df (null = skip).
// Every sum is multiplied by `scale` as it is stored (1: stored as it is).
int reduce_parts(const float *part, int n_parts, int64_t M, float *dqw, int64_t n_dqw, float *dqb, int64_t n_dqb, float *df,
                 int64_t n_df, hipStream_t s, float scale = 1.0f);

// Convolution through LDS-resident operands (hgq_conv_patch.hip): mode 0 forward, 1 data gradient.
bool conv_patch_ok(int mode, const hgq_conv_geom &g, int F);
int conv_patch_launch(int mode, const float *src, const float *mask, const float *w, const float *bias, float *out,
                      const hgq_conv_geom &g, int F, int act, hipStream_t s);
// Weight / bias gradient through LDS-resident operands (3 x 3 and 5 x 5 kernels, unit stride and dilation, channel and
// filter counts multiples of 4 up to 32, 16-byte aligned operands, bf16-part matrix instruction selected): slices
// [conv_patch_wgrad_slices][kh kw C F + F] into `part`.
bool conv_patch_wgrad_ok(const hgq_conv_geom &g, int F);
int conv_patch_wgrad_slices(const hgq_conv_geom &g, int F);
int conv_patch_wgrad_launch(const float *x, const float *dy, const float *mask, float *part, const hgq_conv_geom &g, int F, int act,
                            hipStream_t s);

}  // namespace hgq
