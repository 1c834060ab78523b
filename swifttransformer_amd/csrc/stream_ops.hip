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
//   token side     x += unit(P (gelu_tanh(G x) * e[token])) * w   per row: a narrow embedding row gates a
//                  projection of the stream, which re-enters it at unit root mean square; lookup, the two
//                  small products, the activation, the norm and the sum in one kernel.
//
// Everything is float except the optional copy of the dynamic tanh in the storage type and the token side
// input's matrices and table, which are of the storage type.
#include "activation.h"
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

// logits through a factor and a smooth limit: cap * tanh(x * scale / cap)
__global__ __launch_bounds__(256) void scale_softcap_kernel(float* __restrict__ x, int64_t n, float scale, float cap) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = x[i] * scale;
    x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
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

// A workgroup a row: 16 waves where rows are few (a decode step: every gate feature's row of G in flight
// at once, the kernel's time a handful of dependent trips to memory), 4 otherwise.  LDS: the float row,
// later the projection's result; the gated vector.  Only the matrices and the table are of the storage
// type: the row, the gate's sums and the gated vector stay float (a unit norm follows, and a gated vector
// of a few entries near zero would turn a rounding into a direction).
// g_j = gelu(G_j . x) * e_j, y = P g, x += y / sqrt(mean(y^2) + eps) * w.
// VEC: rows of G and P allow 16-byte loads.
template <typename T, bool VEC>
__global__ __launch_bounds__(1024) void token_side_kernel(
    float* __restrict__ x, const int* __restrict__ token_ids, const int* __restrict__ token_item,
    const T* __restrict__ table, int64_t table_stride, int vocab, const T* __restrict__ w_gate,
    const T* __restrict__ w_proj, const float* __restrict__ gain, int dim, int width, float eps) {
    extern __shared__ __attribute__((aligned(16))) float side_lds[];
    __shared__ float red[16];
    float* xs = side_lds;                 // [width]
    float* gs = side_lds + width;         // [dim]
    const int64_t row = blockIdx.x;
    if (token_item && token_item[row] < 0) return;        // a padding row (uniform over the workgroup)
    constexpr int V = Elem<T>::kVec;
    const int threads = blockDim.x, waves = threads >> 6;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float* xr = x + row * width;
    const int tok = token_ids[row];
    const bool known = tok >= 0 && tok < vocab;
    const T* er = table + (int64_t)(known ? tok : 0) * table_stride;
    // the first feature's table entry is asked for before the row arrives
    float e = (known && wave < dim) ? Elem<T>::load(er + wave) : 0.f;
    for (int c = threadIdx.x; c < width; c += threads) xs[c] = xr[c];
    __syncthreads();
    for (int j = wave; j < dim; j += waves) {
        const T* gr = w_gate + (int64_t)j * width;
        float acc = 0.f;
        if (VEC) {
            for (int c = lane * V; c < width; c += 64 * V) {
                float w[V];
                Elem<T>::load_vec(gr + c, w);
#pragma unroll
                for (int u = 0; u < V; ++u) acc = fmaf(w[u], xs[c + u], acc);
            }
        } else {
            for (int c = lane; c < width; c += 64) acc = fmaf(Elem<T>::load(gr + c), xs[c], acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) gs[j] = apply_activation(kActGeluTanh, acc) * e;
        if (j + waves < dim) e = known ? Elem<T>::load(er + j + waves) : 0.f;
    }
    __syncthreads();                      // every wave has read xs; gs is complete
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += threads) {
        const T* pr = w_proj + (int64_t)c * dim;
        float y = 0.f;
        if (VEC) {
            for (int j = 0; j < dim; j += V) {
                float w[V];
                Elem<T>::load_vec(pr + j, w);
#pragma unroll
                for (int u = 0; u < V; ++u) y = fmaf(w[u], gs[j + u], y);
            }
        } else {
            for (int j = 0; j < dim; ++j) y = fmaf(Elem<T>::load(pr + j), gs[j], y);
        }
        xs[c] = y;                        // this thread's own entries from here on
        ss = fmaf(y, y, ss);
    }
    ss = block_sum(ss, red);
    const float r = 1.f / sqrtf(ss / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += threads) xr[c] += xs[c] * r * gain[c];
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

extern "C" int st_scale_softcap(float* x, int64_t n, float scale, float cap, hipStream_t stream) {
    ST_CHECK(n >= 0 && scale == scale && cap == cap, "scale_softcap: bad operands");
    if (n == 0) return 0;
    ST_CHECK(x, "scale_softcap: null operand");
    scale_softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, n, scale, cap);
    ST_LAUNCH_CHECK("scale_softcap");
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

extern "C" int st_token_side(float* x, const int* token_ids, const int* token_item, const void* table,
                             int64_t table_stride, int vocab, const void* w_gate, const void* w_proj,
                             const float* gain, int num_rows, int dim, int width, float eps, int dtype,
                             hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && width > 0 && dim > 0 && vocab > 0 && eps > 0.f && table_stride >= dim,
             "token_side: bad sizes");
    ST_CHECK(dtype == kF32 || dtype == kBF16, "token_side: unknown dtype %d", dtype);
    const size_t lds = sizeof(float) * ((size_t)width + dim);
    ST_CHECK(lds <= 60 * 1024, "token_side: a row of %d and a gated vector of %d do not fit the LDS", width, dim);
    if (num_rows == 0) return 0;
    ST_CHECK(x && token_ids && table && w_gate && w_proj && gain, "token_side: null operand");
    const int threads = num_rows <= 256 ? 1024 : 256;
    const int vec = dtype == kF32 ? 4 : 8;
    const bool aligned = width % vec == 0 && dim % vec == 0 && (uintptr_t)w_gate % 16 == 0 && (uintptr_t)w_proj % 16 == 0;
#define ST_SIDE(T, VEC)                                                                                          \
    token_side_kernel<T, VEC><<<(unsigned)num_rows, threads, lds, stream>>>(                                         \
        x, token_ids, token_item, (const T*)table, table_stride, vocab, (const T*)w_gate, (const T*)w_proj, gain, dim, \
        width, eps)
    if (dtype == kF32) {
        if (aligned) ST_SIDE(float, true); else ST_SIDE(float, false);
    } else {
        if (aligned) ST_SIDE(bf16_t, true); else ST_SIDE(bf16_t, false);
    }
#undef ST_SIDE
    ST_LAUNCH_CHECK("token_side");
    return 0;
}
