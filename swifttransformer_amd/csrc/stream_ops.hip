// Small float operations on the residual stream that are no product's epilogue:
//
//   dynamic tanh   y = tanh(alpha x) * w + b   per element (no mean, no variance), alpha one number on
//                  the device; optionally of picked rows, optionally added to a second stream
//                  (out32 = base + y: a branch's result normalised on its way into the stream), and
//                  optionally followed by a second dynamic tanh of that sum in the storage type (what
//                  the next sublayer reads), so that norm-after, residual sum and norm-before are one pass;
//   unit add       x += y / sqrt(mean(y^2) + eps) * w   per row (a branch that enters the stream at
//                  unit root mean square);
//   row add        out = x (+ first) + vec   (a pass over a group of layers that starts from the stream
//                  plus the step's embedding plus that pass's vector).
//
// Everything is float except the optional copy of the dynamic tanh in the storage type.
#include "api.h"
#include "common.h"

namespace st {

template <typename T>
__global__ __launch_bounds__(256) void dynamic_tanh_kernel(
    T* __restrict__ out_t, float* __restrict__ out32, const float* __restrict__ x, const int* __restrict__ rows,
    const float* __restrict__ w, const float* __restrict__ b, const float* __restrict__ alpha,
    const float* __restrict__ base, const float* __restrict__ w2, const float* __restrict__ b2,
    const float* __restrict__ alpha2, int width, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t r = idx / width;
    const int c = (int)(idx - r * width);
    int64_t src = r;
    if (rows) {
        src = rows[r];
        if (src < 0) return;                              // a padding entry
    }
    float y = tanhf(alpha[0] * x[src * width + c]) * w[c] + (b ? b[c] : 0.f);
    if (base) y += base[idx];
    if (out32) out32[idx] = y;
    if (w2) y = tanhf(alpha2[0] * y) * w2[c] + (b2 ? b2[c] : 0.f);     // the next norm, of the sum just made
    if (out_t) Elem<T>::store(out_t + idx, y);
}

// a workgroup a row
__global__ __launch_bounds__(256) void unit_add_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                       const float* __restrict__ w, int width, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    const float* yr = y + row * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += 256) ss = fmaf(yr[c], yr[c], ss);
    ss = block_sum(ss, red);
    const float r = 1.f / sqrtf(ss / (float)width + eps);
    float* xr = x + row * width;
    for (int c = threadIdx.x; c < width; c += 256) xr[c] += yr[c] * r * w[c];
}

__global__ __launch_bounds__(256) void row_add_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                      const float* __restrict__ first, const float* __restrict__ vec,
                                                      int width, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    float v = x[idx];
    if (first) v += first[idx];
    out[idx] = v + vec[idx % width];
}

}  // namespace st

using namespace st;

extern "C" int st_dynamic_tanh(void* out_t, float* out32, const float* x, const int* rows, const float* w,
                               const float* b, const float* alpha, const float* base, const float* w2,
                               const float* b2, const float* alpha2, int num_rows, int width, int dtype,
                               hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && width > 0, "dynamic_tanh: bad sizes");
    if (num_rows == 0) return 0;
    ST_CHECK(x && w && alpha && (out_t || out32), "dynamic_tanh: null operand");
    ST_CHECK(!w2 || (alpha2 && out_t), "dynamic_tanh: a second norm needs its alpha and the storage-type output");
    const int64_t total = (int64_t)num_rows * width;
    const unsigned grid = (unsigned)((total + 255) / 256);
    if (dtype == kF32)
        dynamic_tanh_kernel<float><<<grid, 256, 0, stream>>>((float*)out_t, out32, x, rows, w, b, alpha, base, w2, b2, alpha2, width, total);
    else if (dtype == kBF16)
        dynamic_tanh_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out_t, out32, x, rows, w, b, alpha, base, w2, b2, alpha2, width, total);
    else ST_CHECK(false, "dynamic_tanh: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("dynamic_tanh");
    return 0;
}

extern "C" int st_unit_add(float* x, const float* y, const float* w, int num_rows, int width, float eps,
                           hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && width > 0 && eps > 0.f, "unit_add: bad sizes");
    if (num_rows == 0) return 0;
    ST_CHECK(x && y && w, "unit_add: null operand");
    unit_add_kernel<<<(unsigned)num_rows, 256, 0, stream>>>(x, y, w, width, eps);
    ST_LAUNCH_CHECK("unit_add");
    return 0;
}

extern "C" int st_row_add(float* out, const float* x, const float* first, const float* vec, int num_rows, int width,
                          hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && width > 0, "row_add: bad sizes");
    if (num_rows == 0) return 0;
    ST_CHECK(out && x && vec, "row_add: null operand");
    const int64_t total = (int64_t)num_rows * width;
    row_add_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(out, x, first, vec, width, total);
    ST_LAUNCH_CHECK("row_add");
    return 0;
}
