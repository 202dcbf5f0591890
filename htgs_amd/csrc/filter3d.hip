// Mip-Splatting style 3-D filter size per point: over the views in which a point lies inside the (dilated)
// frustum, the minimum of distance2filter * depth.  Restates update_3d_filter_cu
// (HTGSCudaBackend/HTGSCudaBackend/filter3d/src/filter3d_kernels.cu:6-35) and the frustum bounds of
// update_3d_filter_wrapper (filter3d/src/filter3d_api.cu:6-47).  No fused operations: operand order of the source.
#include "common.h"

namespace htgs {

__global__ void __launch_bounds__(256) update_3d_filter_kernel(
    const float *__restrict__ positions, const float *__restrict__ w2c, float *__restrict__ filter_3d, uint8_t *__restrict__ visibility_mask,
    int n, float left, float right, float top, float bottom, float near_plane, float distance2filter)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float px = positions[3 * (size_t)i], py = positions[3 * (size_t)i + 1], pz = positions[3 * (size_t)i + 2];
    const float z = (w2c[8] * px + w2c[9] * py + w2c[10] * pz) + w2c[11];
    if (z < near_plane) return;
    const float x_clip = (w2c[0] * px + w2c[1] * py + w2c[2] * pz) + w2c[3];
    if (x_clip < left * z || x_clip > right * z) return;
    const float y_clip = (w2c[4] * px + w2c[5] * py + w2c[6] * pz) + w2c[7];
    if (y_clip < top * z || y_clip > bottom * z) return;
    const float candidate = distance2filter * z;
    if (filter_3d[i] < candidate) return;
    filter_3d[i] = candidate;
    visibility_mask[i] = 1;
}

}  // namespace htgs

using namespace htgs;

extern "C" int htgs_update_3d_filter(const float *positions, const float *w2c, float *filter_3d, uint8_t *visibility_mask, int n_points,
                                     int width, int height, float focal_x, float focal_y, float center_x, float center_y,
                                     float near_plane, float clipping_tolerance, float distance2filter, void *stream)
{
    if (n_points < 0) return fail(HTGS_ERR_ARGUMENT, "htgs_update_3d_filter: negative size");
    if (n_points == 0) return HTGS_OK;
    if (!positions || !w2c || !filter_3d || !visibility_mask) return fail(HTGS_ERR_ARGUMENT, "htgs_update_3d_filter: null pointer");
    const float bounds_factor = clipping_tolerance + 0.5f;                      // filter3d_api.cu:22-33
    const float width_f = (float)width, height_f = (float)height;
    const float max_x = bounds_factor * width_f, max_y = bounds_factor * height_f;
    const float off_x = center_x - 0.5f * width_f, off_y = center_y - 0.5f * height_f;
    const float left = (-max_x - off_x) / focal_x, right = (max_x - off_x) / focal_x;
    const float top = (-max_y - off_y) / focal_y, bottom = (max_y - off_y) / focal_y;
    hipLaunchKernelGGL(update_3d_filter_kernel, dim3(div_up(n_points, 256)), dim3(256), 0, (hipStream_t)stream, positions, w2c, filter_3d,
                       visibility_mask, n_points, left, right, top, bottom, near_plane, distance2filter);
    return check_launch("update_3d_filter");
}
