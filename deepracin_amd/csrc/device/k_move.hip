// Box copy between [C][H][W] tensors and element-wise scalar ops (bandwidth-bound helpers).
//
// copy3d serves the Concat node when its producers could not be planned straight into the concat
// buffer (the reference always launches a generated copy kernel, src/dR_nodes_transform.c:468-553)
// and the Slice node (`extractSlice`, Kernels/dR_transform.cl:5-24).
#include "drhip_common.hpp"

namespace drhip {

__global__ void __launch_bounds__(256)
copy3d_kernel(const float* __restrict__ src, int sW, int sH, int sx0, int sy0, int sz0,
              float* __restrict__ dst, int dW, int dH, int dx0, int dy0, int dz0, int w, int h, int c) {
    const int total = w * h * c;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        const int x = i % w, y = (i / w) % h, z = i / (w * h);
        dst[((size_t)(z + dz0) * dH + (y + dy0)) * dW + (x + dx0)] =
            src[((size_t)(z + sz0) * sH + (y + sy0)) * sW + (x + sx0)];
    }
}

__global__ void __launch_bounds__(256)
scalar_op_kernel(const float* __restrict__ x, float* __restrict__ y, size_t n, int op, float s) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        const float v = x[i];
        float r;
        switch (op) {
            case 0: r = v + s; break;
            case 1: r = v - s; break;
            case 2: r = v * s; break;
            case 3: r = v / s; break;
            case 4: r = logf(v); break;
            case 5: r = expf(v); break;
            case 6: r = sqrtf(v); break;
            case 7: r = s; break;
            default: r = powf(v, s); break;
        }
        y[i] = r;
    }
}

}  // namespace drhip

using namespace drhip;

extern "C" int drhip_copy3d_f32(const float* src, int sW, int sH, int sx0, int sy0, int sz0,
                                float* dst, int dW, int dH, int dx0, int dy0, int dz0,
                                int w, int h, int c, void* stream) {
    DRHIP_REQUIRE(src && dst, "drhip_copy3d_f32: NULL tensor");
    DRHIP_REQUIRE(w > 0 && h > 0 && c > 0, "drhip_copy3d_f32: empty box %dx%dx%d", w, h, c);
    DRHIP_REQUIRE(sx0 >= 0 && sy0 >= 0 && sz0 >= 0 && dx0 >= 0 && dy0 >= 0 && dz0 >= 0, "drhip_copy3d_f32: negative origin");
    DRHIP_REQUIRE(sx0 + w <= sW && sy0 + h <= sH, "drhip_copy3d_f32: box leaves the source plane (%d+%d>%d or %d+%d>%d)", sx0, w, sW, sy0, h, sH);
    DRHIP_REQUIRE(dx0 + w <= dW && dy0 + h <= dH, "drhip_copy3d_f32: box leaves the destination plane");
    DRHIP_REQUIRE((long long)w * h * c < (1ll << 31), "drhip_copy3d_f32: box too large");
    const int total = w * h * c, block = 256;
    int blocks = ceil_div(total, block);
    if (blocks > 16 * num_cu()) blocks = 16 * num_cu();
    launch(copy3d_kernel, dim3(blocks), dim3(block), 0, as_stream(stream),
                       src, sW, sH, sx0, sy0, sz0, dst, dW, dH, dx0, dy0, dz0, w, h, c);
    return launched("copy3d_kernel");
}

extern "C" int drhip_scalar_op_f32(const float* x, float* y, size_t n, int op, float s, void* stream) {
    DRHIP_REQUIRE(x && y, "drhip_scalar_op_f32: NULL tensor");
    DRHIP_REQUIRE(op >= 0 && op <= 8, "drhip_scalar_op_f32: unknown op %d", op);
    if (n == 0) return DRHIP_OK;
    const int block = 256;
    size_t blocks = (n + block - 1) / block;
    if (blocks > (size_t)16 * num_cu()) blocks = (size_t)16 * num_cu();
    launch(scalar_op_kernel, dim3((unsigned)blocks), dim3(block), 0, as_stream(stream), x, y, n, op, s);
    return launched("scalar_op_kernel");
}
