// Tiled kernel families: dispatch.  (Kernels are added family by family.)
#include "d2c_tiled.hpp"

bool d2c_tiled_supported(const d2c_conv3d_desc &) { return false; }
int d2c_tiled_algo(const d2c_conv3d_desc &) { return D2C_ALGO_GENERIC; }
size_t d2c_tiled_forward_ws(const d2c_conv3d_desc &) { return 0; }
size_t d2c_tiled_backward_ws(const d2c_conv3d_desc &) { return 0; }
int d2c_tiled_forward(const d2c_conv3d_desc &, const void *, const void *, const void *, const void *,
                      const void *, void *, void *, hipStream_t)
{
    d2c_set_error("tiled kernels not available");
    return D2C_ERR_UNSUPPORTED;
}
int d2c_tiled_backward(const d2c_conv3d_desc &, const void *, const void *, const void *, const void *,
                       const void *, void *, void *, void *, void *, void *, void *, hipStream_t)
{
    d2c_set_error("tiled kernels not available");
    return D2C_ERR_UNSUPPORTED;
}
