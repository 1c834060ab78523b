// Recurrent mixers with a matrix state S [key channels x value channels] a head and one scalar
// decay a head and token, for batches of portions of sequences.  Two recurrences share one kernel:
//
//   additive (state-space duality):  S <- a_t S + (b_t k_t) v_t^T;          o_t = S^T q_t + D v_t
//   delta rule:                      S <- a_t S;  u = b_t (v_t - S^T k_t);
//                                    S <- S + k_t u^T;                      o_t = S^T q_t
//
// a_t (the decay) and b_t (the step size, or the write strength) are float [T, heads] made by
// `recurrence_gates` (or one row of constants for every token: a fixed decay a head); q, k, v are float rows; the state is float, lives in the request's slot and is
// loaded before and stored after the item's rows, so prompts, portions and single tokens take the
// same route and a position's sums are formed in the same order however the tokens were cut.
//
// Launch: a two-wave workgroup a (head, block of 16 value channels, item), see the kernel.
#include "api.h"
#include "common.h"

namespace st {

constexpr int kScanMaxKeys = 256;     // key channels a head: four lanes of up to 64

__device__ inline float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// mode 0: raw [T, heads]: a = softplus(raw + bias) (step size), b = exp(-exp(a_log) * a) (decay)
// mode 1: raw [T, 2 * heads] = write logits | decay logits:
//         a = sigmoid(raw[:, :heads]), b = exp(-exp(a_log) * softplus(raw[:, heads:] + bias))
__global__ __launch_bounds__(256) void recurrence_gates_kernel(
    float* __restrict__ out_a, float* __restrict__ out_b, const float* __restrict__ raw, int64_t raw_stride,
    const float* __restrict__ a_log, const float* __restrict__ bias, int64_t n, int heads, int mode) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / heads;
    const int h = (int)(i - t * heads);
    const float* r = raw + t * raw_stride;
    if (mode == 0) {
        const float dt = softplus_f(r[h] + bias[h]);
        out_a[i] = dt;
        out_b[i] = expf(-expf(a_log[h]) * dt);
    } else {
        out_a[i] = 1.f / (1.f + expf(-r[h]));
        out_b[i] = expf(-expf(a_log[h]) * softplus_f(r[heads + h] + bias[h]));
    }
}

// x[t, h, :] <- x[t, h, :] / sqrt(sum x^2 + eps) * scale, float rows, a wave a (row, head)
__global__ __launch_bounds__(256) void unit_norm_kernel(float* __restrict__ x, int64_t stride, int64_t units,
                                                        int heads, int dim, float eps, float scale) {
    const int64_t u = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= units) return;
    const int lane = threadIdx.x & 63;
    const int64_t t = u / heads;
    const int h = (int)(u - t * heads);
    float* p = x + t * stride + (int64_t)h * dim;
    float ss = 0.f;
    for (int j = lane; j < dim; j += 64) ss = fmaf(p[j], p[j], ss);
    ss = wave_sum(ss);
    const float r = scale / sqrtf(ss + eps);
    for (int j = lane; j < dim; j += 64) p[j] *= r;
}

// Two waves a workgroup.  The walker: lane = (quarter of the key channels, one of 16 value channels); a
// lane keeps its KQ key channels of its value channel's column of the state in registers; sums over the
// key channels are sums over a lane's registers and then over the four lanes that share a value channel
// (row swaps, no LDS traffic between lanes).  The loader stages the operands of the next `chunk` tokens
// in LDS while the walker walks the current chunk, and stores the results of the chunk before: a trip to
// memory costs as much as the walk over a dozen tokens, and this way the walker waits for none.  The two
// meet at one barrier a chunk.  A staging buffer: q [chunk, 4 KQ] | k [chunk, 4 KQ] (rows padded with
// zeros) | v [chunk, 16] | a [chunk] | b [chunk]; two of them, then two result buffers [chunk, 16].
// VEC: rows and sizes allow 16-byte loads (the host checks alignment).
template <int MODE, int KQ, bool VEC>
__global__ __launch_bounds__(128) void state_scan_kernel(
    float* __restrict__ out, const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k,
    int64_t k_stride, const float* __restrict__ v, int64_t v_stride, const float* __restrict__ ga,
    const float* __restrict__ gb, int64_t gate_stride, const float* __restrict__ skip, float* __restrict__ state, int64_t slot_stride,
    const int* __restrict__ item_len, const int* __restrict__ item_tok_off, const int* __restrict__ item_slot,
    int heads, int qk_heads, int key_dim, int value_dim, int chunk) {
    extern __shared__ __attribute__((aligned(16))) float staged[];
    constexpr int KW = 4 * KQ;                          // a staged row of q or k
    const int head = blockIdx.x, item = blockIdx.z;
    const int lane = threadIdx.x & 63;
    const bool loader = threadIdx.x >= 64;
    const int quarter = lane >> 4, vc = lane & 15;
    const int col0 = blockIdx.y * 16, col = col0 + vc;
    const bool live = col < value_dim;
    const int slot = item_slot[item], n = item_len[item];
    if (slot < 0 || n <= 0) return;                     // uniform over the workgroup
    const int64_t row0 = item_tok_off[item];
    const int qk_head = head / (heads / qk_heads);
    const int k0 = quarter * KQ;
    const float* qp = q + row0 * q_stride + (int64_t)qk_head * key_dim;
    const float* kp = k + row0 * k_stride + (int64_t)qk_head * key_dim;
    const float* vp = v + row0 * v_stride + (int64_t)head * value_dim + col0;
    const float* ap = ga + row0 * gate_stride + head;
    const float* bp = gb + row0 * gate_stride + head;
    float* op = out + row0 * ((int64_t)heads * value_dim) + (int64_t)head * value_dim + col0;
    const int nq = chunk * KW, nv = chunk * 16;
    const int total = 2 * nq + nv + 2 * chunk;          // floats of a staging buffer
    float* res_base = staged + 2 * total;
    const int chunks = (n + chunk - 1) / chunk;

    // the loader's two jobs (its 64 lanes)
    auto stage = [&](int c) {
        float* buf = staged + (c & 1) * total;
        const int t0 = c * chunk, rows = min(chunk, n - t0);
        if (VEC) {
            constexpr int NB = KQ <= 16 ? 16 : 8;       // 16-byte loads a lane in flight
            const int kv4 = key_dim >> 2;
            const int nqv = chunk * kv4, totalv = 2 * nqv + chunk * 4;
            float gate = 0.f;
            if (lane < 2 * chunk) {
                const int r = lane < chunk ? lane : lane - chunk;
                if (r < rows) gate = (lane < chunk ? ap : bp)[(int64_t)(t0 + r) * gate_stride];
            }
            for (int base = 0; base < totalv; base += 64 * NB) {
                float4 x[NB];
#pragma unroll
                for (int u = 0; u < NB; ++u) {
                    const int idx = base + u * 64 + lane;
                    const float* src = nullptr;
                    if (idx < 2 * nqv) {
                        const int j = idx < nqv ? idx : idx - nqv;
                        const int r = j / kv4, cc = (j - r * kv4) * 4;
                        if (r < rows)
                            src = idx < nqv ? qp + (int64_t)(t0 + r) * q_stride + cc : kp + (int64_t)(t0 + r) * k_stride + cc;
                    } else if (idx < totalv) {
                        const int j = idx - 2 * nqv, r = j >> 2, cc = (j & 3) * 4;
                        if (r < rows && col0 + cc < value_dim) src = vp + (int64_t)(t0 + r) * v_stride + cc;
                    }
                    x[u] = src ? *reinterpret_cast<const float4*>(src) : make_float4(0.f, 0.f, 0.f, 0.f);
                }
#pragma unroll
                for (int u = 0; u < NB; ++u) {
                    const int idx = base + u * 64 + lane;
                    if (idx < 2 * nqv) {
                        const int j = idx < nqv ? idx : idx - nqv;
                        const int r = j / kv4, cc = (j - r * kv4) * 4;
                        *reinterpret_cast<float4*>(buf + (idx < nqv ? 0 : nq) + r * KW + cc) = x[u];
                    } else if (idx < totalv) {
                        *reinterpret_cast<float4*>(buf + 2 * nq + (idx - 2 * nqv) * 4) = x[u];
                    }
                }
            }
            if (lane < 2 * chunk) buf[2 * nq + nv + lane] = gate;
        } else {
            for (int base = 0; base < total; base += 64 * 8) {
                float x[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int idx = base + u * 64 + lane;
                    const float* src = nullptr;
                    if (idx < 2 * nq) {
                        const int j = idx < nq ? idx : idx - nq;
                        const int r = j / KW, cc = j % KW;
                        if (r < rows && cc < key_dim)
                            src = idx < nq ? qp + (int64_t)(t0 + r) * q_stride + cc : kp + (int64_t)(t0 + r) * k_stride + cc;
                    } else if (idx < 2 * nq + nv) {
                        const int j = idx - 2 * nq, r = j >> 4, cc = j & 15;
                        if (r < rows && col0 + cc < value_dim) src = vp + (int64_t)(t0 + r) * v_stride + cc;
                    } else if (idx < total) {
                        const int j = idx - 2 * nq - nv;
                        const int r = j < chunk ? j : j - chunk;
                        if (r < rows) src = (j < chunk ? ap : bp) + (int64_t)(t0 + r) * gate_stride;
                    }
                    x[u] = src ? *src : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int idx = base + u * 64 + lane;
                    if (idx < total) buf[idx] = x[u];
                }
            }
        }
    };
    auto store_results = [&](int c) {
        const float* res = res_base + (c & 1) * nv;
        const int t0 = c * chunk, rows = min(chunk, n - t0);
        for (int j = lane; j < rows * 16; j += 64) {
            const int r = j >> 4, cc = j & 15;
            if (col0 + cc < value_dim) op[(int64_t)(t0 + r) * heads * value_dim + cc] = res[j];
        }
    };

    // the walker's state
    float S[KQ];
    float* sp = state + (int64_t)slot * slot_stride + ((int64_t)head * key_dim + k0) * value_dim + col;
    float d_skip = 0.f;
    if (!loader) {
#pragma unroll
        for (int i = 0; i < KQ; ++i) S[i] = (live && k0 + i < key_dim) ? sp[(int64_t)i * value_dim] : 0.f;
        d_skip = skip ? skip[head] : 0.f;
    } else {
        if (VEC && key_dim < KW)                         // the rows' padding beyond key_dim stays zero in both buffers
            for (int idx = lane; idx < 2 * total; idx += 64) staged[idx] = 0.f;
        stage(0);
    }
    __syncthreads();
    for (int c = 0; c < chunks; ++c) {
        if (loader) {
            if (c + 1 < chunks) stage(c + 1);           // the buffer the walker left a chunk ago
            if (c > 0) store_results(c - 1);
        } else {
            const float* buf = staged + (c & 1) * total;
            float* res = res_base + (c & 1) * nv;
            const int rows = min(chunk, n - c * chunk);
            for (int r = 0; r < rows; ++r) {
                float cq[KQ], ck[KQ];
                const float4* q4 = reinterpret_cast<const float4*>(buf + r * KW + k0);
                const float4* k4 = reinterpret_cast<const float4*>(buf + nq + r * KW + k0);
#pragma unroll
                for (int i = 0; i < KQ / 4; ++i) {
                    const float4 a4 = q4[i], b4 = k4[i];
                    cq[4 * i] = a4.x; cq[4 * i + 1] = a4.y; cq[4 * i + 2] = a4.z; cq[4 * i + 3] = a4.w;
                    ck[4 * i] = b4.x; ck[4 * i + 1] = b4.y; ck[4 * i + 2] = b4.z; ck[4 * i + 3] = b4.w;
                }
                const float cv = buf[2 * nq + r * 16 + vc];
                const float ca = buf[2 * nq + nv + r], cb = buf[2 * nq + nv + chunk + r];
                float o;
                if (MODE == 0) {
                    // ca: the step size, cb: the decay
                    const float w = ca * cv;
                    float acc = 0.f;
#pragma unroll
                    for (int i = 0; i < KQ; ++i) {
                        S[i] = fmaf(cb, S[i], ck[i] * w);
                        acc = fmaf(S[i], cq[i], acc);
                    }
                    o = fmaf(d_skip, cv, rows4_sum(acc));
                } else {
                    // ca: the write strength, cb: the decay.  With the state before this token, S:
                    //   u = ca (v - cb S^T k),  o = (cb S + k u^T)^T q = cb S^T q + (k . q) u:
                    // the two sums over the old state and k . q are formed in one pass
                    float rk = 0.f, rq = 0.f, kq = 0.f;
#pragma unroll
                    for (int i = 0; i < KQ; ++i) {
                        rk = fmaf(S[i], ck[i], rk);
                        rq = fmaf(S[i], cq[i], rq);
                        kq = fmaf(ck[i], cq[i], kq);
                    }
                    rk = rows4_sum(rk);
                    rq = rows4_sum(rq);
                    kq = rows4_sum(kq);
                    const float u = ca * (cv - cb * rk);
#pragma unroll
                    for (int i = 0; i < KQ; ++i) S[i] = fmaf(cb, S[i], ck[i] * u);
                    o = fmaf(cb, rq, kq * u);
                }
                if (quarter == 0) res[r * 16 + vc] = o;
            }
        }
        __syncthreads();
    }
    if (loader) {
        store_results(chunks - 1);
    } else if (live) {
#pragma unroll
        for (int i = 0; i < KQ; ++i)
            if (k0 + i < key_dim) sp[(int64_t)i * value_dim] = S[i];
    }
}

// out[t, g, j] = val * rsqrt(mean_j(val^2) + eps) * gain * (gate_first ? 1 : silu(gate)),
// val = o[t, g, j] * (gate_first ? silu(gate[t, g, j]) : 1); a workgroup a (row, group)
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ gate, int64_t gate_stride,
    const float* __restrict__ gain, int groups, int width, int gain_per_group, int gate_first, int gate_kind,
    float eps) {
    __shared__ float red[16];
    const int64_t t = blockIdx.x / groups;
    const int g = blockIdx.x - (int)t * groups;
    const float* op = o + (t * groups + g) * width;
    const T* gp = gate + t * gate_stride + (int64_t)g * width;
    const float* wp = gain + (gain_per_group ? (int64_t)g * width : 0);
    T* dst = out + (t * groups + g) * width;
    float ss = 0.f;
    for (int j = threadIdx.x; j < width; j += 256) {
        float val = op[j];
        if (gate_first) {
            const float z = Elem<T>::load(gp + j);
            val *= (gate_kind ? 1.f : z) / (1.f + expf(-z));
        }
        ss = fmaf(val, val, ss);
    }
    ss = block_sum(ss, red);
    const float r = 1.f / sqrtf(ss / (float)width + eps);
    for (int j = threadIdx.x; j < width; j += 256) {
        const float z = Elem<T>::load(gp + j);
        const float s = (gate_kind ? 1.f : z) / (1.f + expf(-z));
        const float val = op[j] * r * wp[j] * s;
        Elem<T>::store(dst + j, val);
    }
}

}  // namespace st

using namespace st;

extern "C" int st_recurrence_gates(float* out_a, float* out_b, const float* raw, int64_t raw_stride,
                                   const float* a_log, const float* bias, int num_tokens, int heads, int mode,
                                   hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && (mode == 0 || mode == 1), "recurrence_gates: bad sizes or mode");
    if (num_tokens == 0) return 0;
    ST_CHECK(out_a && out_b && raw && a_log && bias, "recurrence_gates: null operand");
    const int64_t n = (int64_t)num_tokens * heads;
    recurrence_gates_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(out_a, out_b, raw, raw_stride, a_log,
                                                                           bias, n, heads, mode);
    ST_LAUNCH_CHECK("recurrence_gates");
    return 0;
}

extern "C" int st_unit_norm(float* x, int64_t stride, int num_tokens, int heads, int dim, float eps, float scale,
                            hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && dim > 0, "unit_norm: bad sizes");
    if (num_tokens == 0) return 0;
    ST_CHECK(x, "unit_norm: null operand");
    const int64_t units = (int64_t)num_tokens * heads;
    unit_norm_kernel<<<(unsigned)((units + 3) / 4), 256, 0, stream>>>(x, stride, units, heads, dim, eps, scale);
    ST_LAUNCH_CHECK("unit_norm");
    return 0;
}

extern "C" int st_state_scan(float* out, const float* q, int64_t q_stride, const float* k, int64_t k_stride,
                             const float* v, int64_t v_stride, const float* gate_a, const float* gate_b,
                             int64_t gate_stride, const float* skip, float* state, int64_t slot_stride, const int* item_len,
                             const int* item_tok_off, const int* item_slot, int num_items, int max_item_rows, int heads,
                             int qk_heads, int key_dim, int value_dim, int mode, hipStream_t stream) {
    ST_CHECK(num_items >= 0 && heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && key_dim > 0 && value_dim > 0,
             "state_scan: bad sizes");
    ST_CHECK(key_dim <= kScanMaxKeys, "state_scan: up to %d key channels a head, not %d", kScanMaxKeys, key_dim);
    ST_CHECK(mode == 0 || mode == 1, "state_scan: mode 0 (additive) or 1 (delta rule)");
    ST_CHECK(gate_stride == 0 || gate_stride >= heads, "state_scan: gate rows overlap");
    ST_CHECK(num_items <= 65535 && (value_dim + 15) / 16 <= 65535, "state_scan: too many items or value channels");
    if (num_items == 0) return 0;
    ST_CHECK(out && q && k && v && gate_a && gate_b && state && item_len && item_tok_off && item_slot,
             "state_scan: null operand");
    // key channels a lane: a quarter of the head's, rounded up to a power of two from 4 on
    int kq = 4;
    while (4 * kq < key_dim) kq <<= 1;
    const dim3 grid(heads, (value_dim + 15) / 16, num_items);
    // tokens a chunk (at most 32: a lane a gate value): two staging buffers and two result buffers in 48 KB of LDS
    // and no more than an item's rows can be (the caller's bound): steps of single tokens stage little
    int chunk = 32;
    while (chunk > 2 && (2 * 4 * chunk * (8 * kq + 18 + 16) > 48 * 1024 || chunk >= 2 * max_item_rows)) chunk >>= 1;
    const size_t lds = (size_t)2 * 4 * chunk * (8 * kq + 18 + 16);
    // 16-byte loads where every row of q, k and v starts on a 16-byte border and the sizes are whole fours
    const bool vec = key_dim % 4 == 0 && value_dim % 4 == 0 && q_stride % 4 == 0 && k_stride % 4 == 0 &&
                     v_stride % 4 == 0 && (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) == 0;
#define ST_SCAN(MODE, KQ, VEC)                                                                                      \
    state_scan_kernel<MODE, KQ, VEC><<<grid, 128, lds, stream>>>(out, q, q_stride, k, k_stride, v, v_stride, gate_a, \
        gate_b, gate_stride, skip, state, slot_stride, item_len, item_tok_off, item_slot, heads, qk_heads, key_dim,              \
        value_dim, chunk)
#define ST_SCAN_MODE(KQ) do { if (mode == 0) { if (vec) ST_SCAN(0, KQ, true); else ST_SCAN(0, KQ, false); }        \
                              else { if (vec) ST_SCAN(1, KQ, true); else ST_SCAN(1, KQ, false); } } while (0)
    switch (kq) {
        case 4: ST_SCAN_MODE(4); break;
        case 8: ST_SCAN_MODE(8); break;
        case 16: ST_SCAN_MODE(16); break;
        case 32: ST_SCAN_MODE(32); break;
        default: ST_SCAN_MODE(64); break;
    }
#undef ST_SCAN_MODE
#undef ST_SCAN
    ST_LAUNCH_CHECK("state_scan");
    return 0;
}

extern "C" int st_gated_group_norm(void* out, const float* o, const void* gate, int64_t gate_stride,
                                   const float* gain, int num_tokens, int groups, int width, int gain_per_group,
                                   int gate_first, int gate_kind, float eps, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && groups > 0 && width > 0, "gated_group_norm: bad sizes");
    ST_CHECK(eps > 0.f, "gated_group_norm: eps must be positive");
    if (num_tokens == 0) return 0;
    ST_CHECK(out && o && gate && gain, "gated_group_norm: null operand");
    ST_CHECK((int64_t)num_tokens * groups <= 0x7fffffff, "gated_group_norm: too many rows");
    const unsigned grid = (unsigned)(num_tokens * groups);
    if (dtype == kF32)
        gated_group_norm_kernel<float><<<grid, 256, 0, stream>>>((float*)out, o, (const float*)gate, gate_stride,
                                                                 gain, groups, width, gain_per_group, gate_first, gate_kind, eps);
    else if (dtype == kBF16)
        gated_group_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, o, (const bf16_t*)gate, gate_stride,
                                                                  gain, groups, width, gain_per_group, gate_first, gate_kind, eps);
    else ST_CHECK(false, "gated_group_norm: unknown dtype %d", dtype);
    ST_LAUNCH_CHECK("gated_group_norm");
    return 0;
}
