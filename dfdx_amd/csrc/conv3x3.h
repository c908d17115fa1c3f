// 3 x 3, unit-stride, padding-1 convolution forward for the 16-bit types without a patch matrix (conv3x3.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace dfdx_rocm {

struct Conv3x3Problem {
    int dtype;                 // DT_F16 / DT_BF16
    int batch, chan_in, chan_out, h, w;
    const void *img;           // [batch][chan_in][h][w]
    const void *filters;       // [chan_out][chan_in][3][3]
    void *out;                 // [batch][chan_out][h][w]
    void *wt;                  // scratch for the filters as [chan_out][9][chan_in]: conv3x3_filter_bytes(), 16-byte aligned
};

bool conv3x3_supported(const Conv3x3Problem &c);
size_t conv3x3_filter_bytes(const Conv3x3Problem &c);
// hipErrorNotSupported when the shape does not fit (the caller then takes another path)
hipError_t launch_conv3x3(const Conv3x3Problem &c, hipStream_t stream);

}  // namespace dfdx_rocm
