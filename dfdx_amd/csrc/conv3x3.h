// 3 x 3, unit-stride, padding-1 convolution forward for the 16-bit types without a patch matrix (conv3x3.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace dfdx_rocm {

struct Conv3x3Problem {
    int dtype;                 // DT_F16 / DT_BF16
    int batch, chan_in, chan_out, h, w;
    const void *img;           // [batch][chan_in][h][w]
    const void *filters;       // [chan_out][chan_in][3][3]; `transposed_filters`: [chan_in][chan_out][3][3], applied turned
                               // by 180 degrees (the image gradient of a convolution with these filters: img = its grad_out)
    void *out;                 // [batch][chan_out][h][w]
    int accumulate = 0;        // out += ... instead of out = ...
    int transposed_filters = 0;
    void *wt;                  // scratch for the filters as [chan_out][9][chan_in]: conv3x3_filter_bytes(), 16-byte aligned
};

bool conv3x3_supported(const Conv3x3Problem &c);
size_t conv3x3_filter_bytes(const Conv3x3Problem &c);
// hipErrorNotSupported when the shape does not fit (the caller then takes another path)
hipError_t launch_conv3x3(const Conv3x3Problem &c, hipStream_t stream);

// The filter gradient of the same convolution without a patch matrix (conv3x3_wgrad.hip).  `c` as above with `out` =
// grad_out [batch][chan_out][h][w] and `filters` = grad_filters, which is accumulated into; `workspace`: f32 shares of the
// sums, conv3x3_wgrad_workspace_bytes(), 16-byte aligned.
bool conv3x3_wgrad_supported(const Conv3x3Problem &c, int compute_units);
size_t conv3x3_wgrad_workspace_bytes(const Conv3x3Problem &c, int compute_units);
hipError_t launch_conv3x3_wgrad(const Conv3x3Problem &c, int compute_units, void *workspace, hipStream_t stream);

}  // namespace dfdx_rocm
