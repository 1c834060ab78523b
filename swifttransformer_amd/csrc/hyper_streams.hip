// A residual stream kept as several copies ("streams") that every sublayer reads as one weighted sum
// and writes back through a small mixing matrix:
//
//   read    u = sum_s a[s] x_s;  out = u * rsqrt(mean(u^2) + eps) * gain   (the sublayer's input, storage type)
//   write   x_t <- sum_s M[s, t] x_s + b[t] * y   for all t at once (in place: an element of the new streams
//           depends on the same element of the old ones only), optionally followed in the same pass by the
//           next sublayer's read of the streams just written;
//   expand  x_s = x for every s (the streams start as copies of the embedding's output);
//   sum     out = sum_s x_s of picked rows (what the final norm reads).
//
// x is float [rows, streams, width]; every sum is float.  A workgroup a row; the row's weighted sum waits
// in LDS between the pass that squares it and the pass that scales it.
#include "api.h"
#include "common.h"

namespace st {

constexpr int kMaxStreams = 16;

__global__ __launch_bounds__(256) void streams_expand_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                             int streams, int width, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;      // over rows * width
    if (idx >= total) return;
    const int64_t r = idx / width;
    const int c = (int)(idx - r * width);
    const float v = x[idx];
    for (int s = 0; s < streams; ++s) out[(r * streams + s) * width + c] = v;
}

__global__ __launch_bounds__(256) void streams_sum_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                          const int* __restrict__ rows, int streams, int width,
                                                          int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t r = idx / width;
    const int c = (int)(idx - r * width);
    int64_t src = r;
    if (rows) src = rows[r];
    float v = 0.f;
    if (src >= 0)
        for (int s = 0; s < streams; ++s) v += x[(src * streams + s) * width + c];
    out[idx] = v;                                     // a padding entry of the row list reads as zeros
}

// The norm of the row's sum u (in LDS) into out_t / out32.  VEC: four columns a thread and pass (the width a
// multiple of 4, every pointer 16-byte aligned).
template <typename T, bool VEC>
__device__ inline void finish_read(T* __restrict__ out_t, float* __restrict__ out32, const float* u,
                                   const float* __restrict__ gain, float ss, int width, float eps, float* red) {
    ss = block_sum(ss, red);
    const float r = eps > 0.f ? 1.f / sqrtf(ss / (float)width + eps) : 1.f;
    if (VEC) {
        for (int c = threadIdx.x * 4; c < width; c += 1024) {
            const float4 uv = *reinterpret_cast<const float4*>(u + c);
            const float4 g = gain ? *reinterpret_cast<const float4*>(gain + c) : make_float4(1.f, 1.f, 1.f, 1.f);
            const float v[4] = {uv.x * r * g.x, uv.y * r * g.y, uv.z * r * g.z, uv.w * r * g.w};
            if (out_t) Elem<T>::store4(out_t + c, v);
            if (out32) *reinterpret_cast<float4*>(out32 + c) = make_float4(v[0], v[1], v[2], v[3]);
        }
        return;
    }
    for (int c = threadIdx.x; c < width; c += 256) {
        const float v = u[c] * r * (gain ? gain[c] : 1.f);
        if (out_t) Elem<T>::store(out_t + c, v);
        if (out32) out32[c] = v;
    }
}

// eps <= 0: no norm, the sum itself.
// S: the number of streams where it is one the launcher has an instance for (the loops over the streams then
// unroll and a column's values stay in registers), 0: taken from `streams_rt`.
template <typename T, int S, bool VEC>
__global__ __launch_bounds__(256) void streams_read_kernel(
    T* __restrict__ out_t, float* __restrict__ out32, const float* __restrict__ x, const float* __restrict__ a,
    const float* __restrict__ gain, int streams_rt, int width, float eps) {
    const int streams = S ? S : streams_rt;
    extern __shared__ float4 u4[];
    float* u = reinterpret_cast<float*>(u4);
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    const float* xr = x + row * streams * width;
    float w[S ? S : kMaxStreams];
#pragma unroll
    for (int s = 0; s < streams; ++s) w[s] = a[s];
    float ss = 0.f;
    if (VEC) {
        for (int c = threadIdx.x * 4; c < width; c += 1024) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int s = 0; s < streams; ++s) {
                const float4 xv = *reinterpret_cast<const float4*>(xr + (int64_t)s * width + c);
                v.x = fmaf(w[s], xv.x, v.x); v.y = fmaf(w[s], xv.y, v.y);
                v.z = fmaf(w[s], xv.z, v.z); v.w = fmaf(w[s], xv.w, v.w);
            }
            *reinterpret_cast<float4*>(u + c) = v;
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
        }
    } else {
        for (int c = threadIdx.x; c < width; c += 256) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < streams; ++s) v = fmaf(w[s], xr[(int64_t)s * width + c], v);
            u[c] = v;
            ss = fmaf(v, v, ss);
        }
    }
    finish_read<T, VEC>(out_t ? out_t + row * width : nullptr, out32 ? out32 + row * width : nullptr, u, gain, ss, width,
                        eps, red);
}

template <typename T, int S, bool VEC>
__global__ __launch_bounds__(256) void streams_write_kernel(
    float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ mix, const float* __restrict__ b,
    T* __restrict__ out_t, const float* __restrict__ a2, const float* __restrict__ gain2, int streams_rt, int width,
    float eps2) {
    const int streams = S ? S : streams_rt;
    extern __shared__ float4 u4[];
    float* u = reinterpret_cast<float*>(u4);
    __shared__ float red[16];
    __shared__ float s_mix[kMaxStreams * kMaxStreams], s_b[kMaxStreams], s_a2[kMaxStreams];
    const int64_t row = blockIdx.x;
    for (int i = threadIdx.x; i < streams * streams; i += 256) s_mix[i] = mix[i];
    if ((int)threadIdx.x < streams) {
        s_b[threadIdx.x] = b[threadIdx.x];
        s_a2[threadIdx.x] = a2 ? a2[threadIdx.x] : 0.f;
    }
    __syncthreads();
    float* xr = x + row * streams * width;
    const float* yr = y + row * width;
    float ss = 0.f;
    if (VEC) {
        for (int c = threadIdx.x * 4; c < width; c += 1024) {
            float4 old[S ? S : kMaxStreams];
#pragma unroll
            for (int s = 0; s < streams; ++s) old[s] = *reinterpret_cast<const float4*>(xr + (int64_t)s * width + c);
            const float4 yv = *reinterpret_cast<const float4*>(yr + c);
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int t = 0; t < streams; ++t) {
                const float bt = s_b[t];
                float4 nv = make_float4(bt * yv.x, bt * yv.y, bt * yv.z, bt * yv.w);
#pragma unroll
                for (int s = 0; s < streams; ++s) {
                    const float m = s_mix[s * streams + t];
                    nv.x = fmaf(m, old[s].x, nv.x); nv.y = fmaf(m, old[s].y, nv.y);
                    nv.z = fmaf(m, old[s].z, nv.z); nv.w = fmaf(m, old[s].w, nv.w);
                }
                *reinterpret_cast<float4*>(xr + (int64_t)t * width + c) = nv;
                const float at = s_a2[t];
                v.x = fmaf(at, nv.x, v.x); v.y = fmaf(at, nv.y, v.y); v.z = fmaf(at, nv.z, v.z); v.w = fmaf(at, nv.w, v.w);
            }
            if (out_t) {
                *reinterpret_cast<float4*>(u + c) = v;
                ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
            }
        }
    } else {
        for (int c = threadIdx.x; c < width; c += 256) {
            float old[S ? S : kMaxStreams];
#pragma unroll
            for (int s = 0; s < streams; ++s) old[s] = xr[(int64_t)s * width + c];
            const float yv = yr[c];
            float v = 0.f;
#pragma unroll
            for (int t = 0; t < streams; ++t) {
                float nv = s_b[t] * yv;
#pragma unroll
                for (int s = 0; s < streams; ++s) nv = fmaf(s_mix[s * streams + t], old[s], nv);
                xr[(int64_t)t * width + c] = nv;
                v = fmaf(s_a2[t], nv, v);
            }
            if (out_t) {
                u[c] = v;
                ss = fmaf(v, v, ss);
            }
        }
    }
    if (out_t) finish_read<T, VEC>(out_t + row * width, nullptr, u, gain2, ss, width, eps2, red);
}

}  // namespace st

using namespace st;

extern "C" int st_streams_expand(float* out, const float* x, int num_rows, int streams, int width,
                                 hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && streams >= 1 && width > 0, "streams_expand: bad sizes");
    if (num_rows == 0) return 0;
    ST_CHECK(out && x, "streams_expand: null operand");
    const int64_t total = (int64_t)num_rows * width;
    streams_expand_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(out, x, streams, width, total);
    ST_LAUNCH_CHECK("streams_expand");
    return 0;
}

// out[r] = sum_s x[rows ? rows[r] : r, s]; a negative row gives zeros.
extern "C" int st_streams_sum(float* out, const float* x, const int* rows, int num_rows, int streams, int width,
                              hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && streams >= 1 && width > 0, "streams_sum: bad sizes");
    if (num_rows == 0) return 0;
    ST_CHECK(out && x, "streams_sum: null operand");
    const int64_t total = (int64_t)num_rows * width;
    streams_sum_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(out, x, rows, streams, width, total);
    ST_LAUNCH_CHECK("streams_sum");
    return 0;
}

// u = sum_s a[s] x[row, s]; out = u * rsqrt(mean(u^2) + eps) * gain (gain null: ones; eps <= 0: u itself);
// out_t (`dtype`) and / or out32.
extern "C" int st_streams_read(void* out_t, float* out32, const float* x, const float* a, const float* gain,
                               int num_rows, int streams, int width, float eps, int dtype, hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && streams >= 1 && streams <= kMaxStreams && width > 0 && width <= 16384,
             "streams_read: bad sizes (up to %d streams of up to 16384)", kMaxStreams);
    if (num_rows == 0) return 0;
    ST_CHECK(x && a && (out_t || out32), "streams_read: null operand");
    const size_t lds = (size_t)width * 4;
    ST_CHECK(dtype == kF32 || dtype == kBF16, "streams_read: unknown dtype %d", dtype);
#define ST_READ_V(S, V)                                                                                                 \
    do {                                                                                                            \
        if (dtype == kF32)                                                                                          \
            streams_read_kernel<float, S, V><<<num_rows, 256, lds, stream>>>((float*)out_t, out32, x, a, gain,      \
                                                                             streams, width, eps);                  \
        else                                                                                                        \
            streams_read_kernel<bf16_t, S, V><<<num_rows, 256, lds, stream>>>((bf16_t*)out_t, out32, x, a, gain,    \
                                                                              streams, width, eps);                 \
    } while (0)
    // four columns a thread where the rows allow 16-byte accesses
    const bool vec = width % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out_t) |
                                         reinterpret_cast<uintptr_t>(out32) | reinterpret_cast<uintptr_t>(gain)) & 15) == 0;
#define ST_READ(S) do { if (vec) ST_READ_V(S, true); else ST_READ_V(S, false); } while (0)
    switch (streams) {
        case 1: ST_READ(1); break;
        case 2: ST_READ(2); break;
        case 3: ST_READ(3); break;
        case 4: ST_READ(4); break;
        case 6: ST_READ(6); break;
        case 8: ST_READ(8); break;
        default: ST_READ(0); break;
    }
#undef ST_READ
#undef ST_READ_V
    ST_LAUNCH_CHECK("streams_read");
    return 0;
}

// In place: x[row, t] <- sum_s mix[s, t] x[row, s] + b[t] * y[row].  With out_t: also the next read of the
// new streams, out_t = norm(sum_t a2[t] x[row, t]) with gain2 and eps2 as st_streams_read.
extern "C" int st_streams_write(float* x, const float* y, const float* mix, const float* b, void* out_t,
                                const float* a2, const float* gain2, int num_rows, int streams, int width,
                                float eps2, int dtype, hipStream_t stream) {
    ST_CHECK(num_rows >= 0 && streams >= 1 && streams <= kMaxStreams && width > 0 && width <= 16384,
             "streams_write: bad sizes (up to %d streams of up to 16384)", kMaxStreams);
    if (num_rows == 0) return 0;
    ST_CHECK(x && y && mix && b, "streams_write: null operand");
    ST_CHECK(!out_t || a2, "streams_write: a following read needs its weights");
    const size_t lds = out_t ? (size_t)width * 4 : 0;
    ST_CHECK(dtype == kF32 || dtype == kBF16, "streams_write: unknown dtype %d", dtype);
#define ST_WRITE_V(S, V)                                                                                                 \
    do {                                                                                                             \
        if (dtype == kF32)                                                                                           \
            streams_write_kernel<float, S, V><<<num_rows, 256, lds, stream>>>(x, y, mix, b, (float*)out_t, a2, gain2, \
                                                                              streams, width, eps2);                 \
        else                                                                                                         \
            streams_write_kernel<bf16_t, S, V><<<num_rows, 256, lds, stream>>>(x, y, mix, b, (bf16_t*)out_t, a2,      \
                                                                               gain2, streams, width, eps2);         \
    } while (0)
    const bool vec = width % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) |
                                         reinterpret_cast<uintptr_t>(out_t) | reinterpret_cast<uintptr_t>(gain2)) & 15) == 0;
#define ST_WRITE(S) do { if (vec) ST_WRITE_V(S, true); else ST_WRITE_V(S, false); } while (0)
    switch (streams) {
        case 1: ST_WRITE(1); break;
        case 2: ST_WRITE(2); break;
        case 3: ST_WRITE(3); break;
        case 4: ST_WRITE(4); break;
        case 6: ST_WRITE(6); break;
        case 8: ST_WRITE(8); break;
        default: ST_WRITE(0); break;
    }
#undef ST_WRITE
#undef ST_WRITE_V
    ST_LAUNCH_CHECK("streams_write");
    return 0;
}
