// Routed experts: every token sends its vector, scaled by a routing weight, through `top` of
// `experts` small gated feed-forward layers.
//
// Everything stays on the device and has a fixed launch shape, so a step can be recorded:
//   route    per token the `top` largest router logits and the sigmoid of each;
//   align    the (token, choice) pairs sorted by expert into tiles of 16, 64 or 128 places, a tile
//            holding pairs of one expert only (places left over are marked -1);
//   up       per tile and 64 inner features: both input products on the matrix cores, rows
//            gathered through the sorted list, then clamp, gate and product of the two halves;
//   down     per tile and 64 output features: the output product; with one expert a token the
//            result goes straight into the residual stream, otherwise to a row per pair that
//   combine  sums in the order of the token's choices.
// A wave computes a 16 x 16 block of results with operands read straight from memory in the
// matrix instruction's own layout (16 bytes a lane and step): with 16 rows a tile the products
// are bound by the stream of expert weights, which every tile reads once.
#include "api.h"
#include "common.h"

namespace st {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kRows = 16;            // rows of one matrix-instruction block
constexpr int kMaxTop = 16;

__global__ __launch_bounds__(256) void moe_route_kernel(
    int* __restrict__ ids, float* __restrict__ weights, const float* __restrict__ logits,
    const int* __restrict__ token_item, int num_tokens, int experts, int top, int mode, int groups, int keep,
    int stage) {
    // The rows of the workgroup's tokens go to LDS first, read side by side (a thread that walked its own row in
    // memory would wait for every logit by itself, several times over); rows are experts + 1 floats apart.
    extern __shared__ float s_z[];
    const int t0 = blockIdx.x * blockDim.x, t = t0 + threadIdx.x;
    if (stage) {
        const int n = min((int)blockDim.x, num_tokens - t0);
        const float* src = logits + (int64_t)t0 * experts;
        for (int i = threadIdx.x; i < n * experts; i += blockDim.x) {
            const int r = i / experts;
            s_z[r * (experts + 1) + (i - r * experts)] = src[i];
        }
        __syncthreads();
    }
    if (t >= num_tokens) return;
    if (token_item && token_item[t] < 0) {
        for (int j = 0; j < top; ++j) { ids[(int64_t)t * top + j] = -1; weights[(int64_t)t * top + j] = 0.f; }
        return;
    }
    const float* z = stage ? s_z + threadIdx.x * (experts + 1) : logits + (int64_t)t * experts;
    // mode 2: only the experts of the `keep` groups (of `groups` equal groups of neighbours) whose largest
    // logit is largest can be chosen; bit g of `open` says that group g is one of them
    uint64_t open = ~0ull;
    const int per = experts / groups;
    if (mode == 2 && keep < groups) {
        open = 0;
        for (int j = 0; j < keep; ++j) {
            int best = -1;
            float bv = 0.f;
            for (int g = 0; g < groups; ++g) {
                if ((open >> g) & 1) continue;
                float gv = z[g * per];
                for (int e = 1; e < per; ++e) gv = fmaxf(gv, z[g * per + e]);
                if (best < 0 || gv > bv) { best = g; bv = gv; }
            }
            open |= 1ull << best;
        }
    }
    // mode 2: the weights are the chosen experts' shares of the softmax over all experts, as they are
    float m_all = 0.f, inv_sum = 1.f;
    if (mode == 2) {
        m_all = z[0];
        for (int e = 1; e < experts; ++e) m_all = fmaxf(m_all, z[e]);
        float sum = 0.f;
        for (int e = 0; e < experts; ++e) sum += expf(z[e] - m_all);
        inv_sum = 1.f / sum;
    }
    auto weight_of = [&](float v) { return mode == 0 ? 1.f / (1.f + expf(-v)) : mode == 2 ? expf(v - m_all) * inv_sum : v; };
    if (experts <= 64) {
        // which experts can still be chosen, a bit each: no list of the chosen ones to walk
        uint64_t free_ = experts == 64 ? ~0ull : (1ull << experts) - 1;
        if (mode == 2 && keep < groups) {
            const uint64_t one_group = per == 64 ? ~0ull : (1ull << per) - 1;
            free_ = 0;
            for (int g = 0; g < groups; ++g)
                if ((open >> g) & 1) free_ |= one_group << (g * per);
        }
        for (int j = 0; j < top; ++j) {
            int best = -1;
            float bv = 0.f;
            for (int e = 0; e < experts; ++e) {
                const float v = z[e];
                if (((free_ >> e) & 1) && (best < 0 || v > bv)) { best = e; bv = v; }
            }
            free_ &= ~(1ull << best);
            ids[(int64_t)t * top + j] = best;
            weights[(int64_t)t * top + j] = weight_of(bv);
        }
    } else {
        int chosen[kMaxTop];
        for (int j = 0; j < top; ++j) {
            int best = -1;
            float bv = 0.f;
            for (int e = 0; e < experts; ++e) {
                bool taken = mode == 2 && !((open >> (e / per)) & 1);
                for (int u = 0; u < j; ++u) taken |= chosen[u] == e;
                const float v = z[e];
                if (!taken && (best < 0 || v > bv)) { best = e; bv = v; }
            }
            chosen[j] = best;
            ids[(int64_t)t * top + j] = best;
            weights[(int64_t)t * top + j] = weight_of(bv);
        }
    }
    if (mode == 1) {
        // softmax over the chosen logits alone; the first chosen is the largest
        float* w = weights + (int64_t)t * top;
        const float m = w[0];
        float sum = 0.f;
        for (int j = 0; j < top; ++j) { w[j] = expf(w[j] - m); sum += w[j]; }
        for (int j = 0; j < top; ++j) w[j] /= sum;
    }
}

// One workgroup: counts, padded offsets, then places.  Which place of its expert's tiles a pair
// gets depends on the order of the atomics; a pair's result does not depend on its place.
__global__ __launch_bounds__(1024) void moe_align_kernel(
    int* __restrict__ sorted, int* __restrict__ place_of_pair, int* __restrict__ tile_expert,
    const int* __restrict__ ids, int num_pairs, int experts, int capacity, int kTile) {
    extern __shared__ int lds[];
    int* count = lds;                  // [experts]
    int* offset = lds + experts;       // [experts + 1]
    const int tid = threadIdx.x;
    for (int e = tid; e < experts; e += 1024) count[e] = 0;
    for (int i = tid; i < capacity; i += 1024) sorted[i] = -1;
    for (int i = tid; i < capacity / kTile; i += 1024) tile_expert[i] = -1;
    __syncthreads();
    for (int p = tid; p < num_pairs; p += 1024) {
        const int e = ids[p];
        if (e >= 0) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < experts; ++e) {
            offset[e] = run;
            run += (count[e] + kTile - 1) / kTile * kTile;
        }
        offset[experts] = run;
    }
    __syncthreads();
    for (int e = tid; e < experts; e += 1024) {
        for (int i = offset[e] / kTile; i < offset[e + 1] / kTile; ++i) tile_expert[i] = e;
        count[e] = offset[e];          // from here on: the next free place of the expert
    }
    __syncthreads();
    for (int p = tid; p < num_pairs; p += 1024) {
        const int e = ids[p];
        int place = -1;
        if (e >= 0) {
            place = atomicAdd(&count[e], 1);
            sorted[place] = p;
        }
        place_of_pair[p] = place;
    }
}

// ---- operands in the matrix instructions' layout: lane (r16, g) holds, of row r16, the elements
// k0 + 8g .. 8g+7 (bfloat16, one product of depth 32) or k0 + 4g .. 4g+3 (float, four products
// of depth 4, the u-th taking element u of every lane).
template <typename T> struct Frag;
template <> struct Frag<bf16_t> {
    static constexpr int kDepth = 32, kLane = 8;
    bf16x8 v;
    __device__ inline void load(const bf16_t* row, int k, int K, bool ok, bool vec) {
        if (ok && vec && k + 8 <= K) {
            v = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(row + k));
        } else {
            uint16_t e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = (ok && k + i < K) ? row[k + i].bits : (uint16_t)0;
            v = __builtin_bit_cast(bf16x8, make_uint4(e[0] | ((uint32_t)e[1] << 16), e[2] | ((uint32_t)e[3] << 16),
                                                      e[4] | ((uint32_t)e[5] << 16), e[6] | ((uint32_t)e[7] << 16)));
        }
    }
    __device__ static inline floatx4 mma(const Frag& a, const Frag& b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
    }
};
template <> struct Frag<float> {
    static constexpr int kDepth = 16, kLane = 4;
    float v[4];
    __device__ inline void load(const float* row, int k, int K, bool ok, bool vec) {
        if (ok && vec && k + 4 <= K) {
            const float4 x = *reinterpret_cast<const float4*>(row + k);
            v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = (ok && k + i < K) ? row[k + i] : 0.f;
        }
    }
    __device__ static inline floatx4 mma(const Frag& a, const Frag& b, floatx4 c) {
#pragma unroll
        for (int u = 0; u < 4; ++u) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[u], b.v[u], c, 0, 0, 0);
        return c;
    }
};

// grid (tiles, ceil(inner / 64)); wave w of the workgroup takes inner features f0 + 16 w .. +15 of
// the tile's RT blocks of 16 rows: a step's weight operands are loaded once and meet RT blocks of
// rows (RT = 1 for few rows an expert, where only the weights' stream counts; RT = 4 or 8 for
// prompts, where every tile reads its expert's weights again from the L2).
// Result layout of a block: lane (r16, g) holds rows 4g .. 4g+3 of feature r16.
template <typename T, int RT>
__global__ __launch_bounds__(256) void moe_up_kernel(
    T* __restrict__ y, const T* __restrict__ x, const T* __restrict__ w_gate, const T* __restrict__ w_up,
    const int* __restrict__ sorted, const int* __restrict__ tile_expert, const float* __restrict__ weights,
    int top, int width, int inner, float limit, int style, int vec) {
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    const int f = blockIdx.y * 64 + wave * 16 + r16;           // this lane's feature as an operand row
    const bool f_ok = f < inner;
    const int base = tile * (kRows * RT);
    const T* xr[RT];
    bool p_ok[RT];
#pragma unroll
    for (int b = 0; b < RT; ++b) {
        const int pair = sorted[base + b * kRows + r16];       // this lane's token row as an operand row
        p_ok[b] = pair >= 0;
        xr[b] = x + (int64_t)(p_ok[b] ? pair / top : 0) * width;
    }
    const T* gr = w_gate + ((int64_t)e * inner + (f_ok ? f : 0)) * width;
    const T* ur = w_up + ((int64_t)e * inner + (f_ok ? f : 0)) * width;
    floatx4 cg[RT], cu[RT];
#pragma unroll
    for (int b = 0; b < RT; ++b) { cg[b] = floatx4{0.f, 0.f, 0.f, 0.f}; cu[b] = floatx4{0.f, 0.f, 0.f, 0.f}; }
    constexpr int D = Frag<T>::kDepth, L = Frag<T>::kLane;

    for (int k0 = 0; k0 < width; k0 += D) {
        Frag<T> a[RT], bg, bu;
        const int k = k0 + L * g;
        bg.load(gr, k, width, f_ok, vec);
        bu.load(ur, k, width, f_ok, vec);
#pragma unroll
        for (int b = 0; b < RT; ++b) a[b].load(xr[b], k, width, p_ok[b], vec);
#pragma unroll
        for (int b = 0; b < RT; ++b) {
            cg[b] = Frag<T>::mma(a[b], bg, cg[b]);
            cu[b] = Frag<T>::mma(a[b], bu, cu[b]);
        }
    }
    if (!f_ok) return;
#pragma unroll
    for (int b = 0; b < RT; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int place = base + b * kRows + 4 * g + r;
            const int p = sorted[place];
            float out = 0.f;
            if (p >= 0 && style == 1) {
                const float gv = cg[b][r];
                out = gv / (1.f + expf(-gv)) * cu[b][r];
            } else if (p >= 0) {
                const float s = weights[p];
                const float gv = fminf(s * cg[b][r], limit);
                const float uv = fminf(fmaxf(s * cu[b][r], -limit), limit);
                out = gv / (1.f + expf(-1.702f * gv)) * (uv + 1.f);
            }
            Elem<T>::store(y + (int64_t)place * inner + f, out);
        }
}

// grid (tiles, ceil(width / 64)).
template <typename T, int RT>
__global__ __launch_bounds__(256) void moe_down_kernel(
    float* __restrict__ out, const float* __restrict__ residual, float* __restrict__ pair_out,
    const T* __restrict__ y, const T* __restrict__ w_down, const int* __restrict__ sorted,
    const int* __restrict__ tile_expert, int top, int width, int inner, float out_scale, int vec) {
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    const int n = blockIdx.y * 64 + wave * 16 + r16;
    const bool n_ok = n < width;
    const int base = tile * (kRows * RT);
    const T* yr = y + (int64_t)(base + r16) * inner;
    const T* wr = w_down + ((int64_t)e * width + (n_ok ? n : 0)) * inner;
    floatx4 c[RT];
#pragma unroll
    for (int b = 0; b < RT; ++b) c[b] = floatx4{0.f, 0.f, 0.f, 0.f};
    constexpr int D = Frag<T>::kDepth, L = Frag<T>::kLane;

    for (int k0 = 0; k0 < inner; k0 += D) {
        Frag<T> a[RT], bw;
        const int k = k0 + L * g;
        bw.load(wr, k, inner, n_ok, vec);
#pragma unroll
        for (int b = 0; b < RT; ++b) a[b].load(yr + (int64_t)b * kRows * inner, k, inner, true, vec);
#pragma unroll
        for (int b = 0; b < RT; ++b) c[b] = Frag<T>::mma(a[b], bw, c[b]);
    }
    if (!n_ok) return;
#pragma unroll
    for (int b = 0; b < RT; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int place = base + b * kRows + 4 * g + r;
            const int p = sorted[place];
            if (p < 0) continue;
            if (pair_out) {
                pair_out[(int64_t)place * width + n] = c[b][r];
            } else {                                           // one expert a token: p is the token
                const int64_t at = (int64_t)p * width + n;
                out[at] = fmaf(out_scale, c[b][r], residual[at]);
            }
        }
}

// ---- prompts in bfloat16: tiles of 128 places, operands staged through LDS ----------------------
// With a hundred rows and more an expert the products are bound by arithmetic, not by the weights'
// stream, and operands read straight from memory leave the matrix cores waiting.  Here a workgroup
// computes 128 places x 128 weight rows in steps of 64 in depth: all threads bring the two operand
// tiles into registers with 16-byte loads (the next step's while this one is multiplied), store
// them into LDS with the rows' chunks rotated so that the matrix instruction's reads spread over
// the banks, and every wave multiplies a 64 x 64 part (v_mfma_f32_32x32x16_bf16).
// UP: the 128 weight rows are 64 inner features of the gate matrix and the same 64 of the other
// one, dealt so that a lane holds both halves of a result; rows of x are gathered through the
// sorted list.  Otherwise: 128 output features of the expert's output matrix over the rows of y.
typedef float floatx16 __attribute__((ext_vector_type(16)));
__device__ inline int rot(int row, int chunk) { return row * 8 + (chunk ^ ((row >> 1) & 7)); }

template <bool UP>
__global__ __launch_bounds__(256) void moe_tiled_kernel(
    bf16_t* __restrict__ y_out, float* __restrict__ out, const float* __restrict__ residual,
    float* __restrict__ pair_out, const bf16_t* __restrict__ a_rows, const bf16_t* __restrict__ w0,
    const bf16_t* __restrict__ w1, const int* __restrict__ sorted, const int* __restrict__ tile_expert,
    const float* __restrict__ weights, int top, int N, int K, float limit, float out_scale, int style) {
    __shared__ uint4 sw[128 * 8];      // weight rows: [row][chunk of 8 in depth]
    __shared__ uint4 sx[128 * 8];      // places
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave & 1, wm = wave >> 1, l32 = lane & 31, lh = lane >> 5;
    const int base = tile * 128;
    const int n0 = blockIdx.y * (UP ? 64 : 128);
    // the four rows of each tile that this thread brings in, fixed over the steps
    const bf16_t* wrow[4];
    const bf16_t* xrow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (tid + i * 256) >> 3;
        int n;
        const bf16_t* m;
        if (UP) { n = n0 + (row >> 6) * 32 + (row & 31); m = ((row >> 5) & 1) ? w1 : w0; }
        else { n = n0 + row; m = w0; }
        wrow[i] = n < N ? m + ((int64_t)e * N + n) * K : nullptr;
        const int p = sorted[base + row];
        xrow[i] = UP ? (p >= 0 ? a_rows + (int64_t)(p / top) * K : nullptr) : a_rows + (int64_t)(base + row) * K;
    }
    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
    uint4 rw[4], rx[4];
    auto load_global = [&](int k0) {
        const int k = k0 + (tid & 7) * 8;
        const bool in = k < K;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // (addresses clamped and values cleared rather than loads behind a branch)
            const bf16_t* pw = wrow[i] ? wrow[i] : w0;
            const bf16_t* px = xrow[i] ? xrow[i] : a_rows;
            const uint4 vw = *reinterpret_cast<const uint4*>(pw + (in ? k : 0));
            const uint4 vx = *reinterpret_cast<const uint4*>(px + (in ? k : 0));
            rw[i] = (in && wrow[i]) ? vw : make_uint4(0, 0, 0, 0);
            rx[i] = (in && xrow[i]) ? vx : make_uint4(0, 0, 0, 0);
        }
    };
    load_global(0);
    for (int k0 = 0; k0 < K; k0 += 64) {
        __syncthreads();               // the step before has been read
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256;
            sw[rot(c >> 3, c & 7)] = rw[i];
            sx[rot(c >> 3, c & 7)] = rx[i];
        }
        __syncthreads();
        if (k0 + 64 < K) load_global(k0 + 64);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const int chunk = kk * 2 + lh;
            bf16x8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = __builtin_bit_cast(bf16x8, sw[rot(wn * 64 + i * 32 + l32, chunk)]);
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = __builtin_bit_cast(bf16x8, sx[rot(wm * 64 + j * 32 + l32, chunk)]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }
    // acc[i][j][q]: weight row wn*64 + i*32 + 8*(q/4) + 4*lh + q%4, place base + wm*64 + j*32 + l32
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int place = base + wm * 64 + j * 32 + l32;
        const int p = sorted[place];
        if (UP) {
            const float s = p >= 0 && style == 0 ? weights[p] : 0.f;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int f = n0 + wn * 32 + 8 * q4 + 4 * lh;
                if (f >= N) continue;
                float r[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (style == 1) {
                        const float gv = acc[0][j][4 * q4 + u];
                        r[u] = p >= 0 ? gv / (1.f + expf(-gv)) * acc[1][j][4 * q4 + u] : 0.f;
                        continue;
                    }
                    const float gv = fminf(s * acc[0][j][4 * q4 + u], limit);
                    const float uv = fminf(fmaxf(s * acc[1][j][4 * q4 + u], -limit), limit);
                    r[u] = p >= 0 ? gv / (1.f + expf(-1.702f * gv)) * (uv + 1.f) : 0.f;
                }
                bf16_t* dst = y_out + (int64_t)place * N + f;
                if (f + 3 < N && (N & 3) == 0) Elem<bf16_t>::store4(dst, r);
                else
                    for (int u = 0; u < 4 && f + u < N; ++u) Elem<bf16_t>::store(dst + u, r[u]);
            }
        } else {
            if (p < 0) continue;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const int n = n0 + wn * 64 + i * 32 + 8 * q4 + 4 * lh;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (n + u >= N) continue;
                        const float v = acc[i][j][4 * q4 + u];
                        if (pair_out) pair_out[(int64_t)place * N + n + u] = v;
                        else {
                            const int64_t at = (int64_t)p * N + n + u;       // one expert a token: p is the token
                            out[at] = fmaf(out_scale, v, residual[at]);
                        }
                    }
                }
        }
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(
    float* __restrict__ out, const float* __restrict__ residual, const float* __restrict__ pair_out,
    const int* __restrict__ place_of_pair, const float* __restrict__ weights, int top, int width, float out_scale) {
    const int t = blockIdx.x;
    for (int n = threadIdx.x; n < width; n += 256) {
        float sum = 0.f;
        bool any = false;
        for (int j = 0; j < top; ++j) {
            const int place = place_of_pair[(int64_t)t * top + j];
            if (place >= 0) {
                const float v = pair_out[(int64_t)place * width + n];
                sum = weights ? fmaf(weights[(int64_t)t * top + j], v, sum) : sum + v;
                any = true;
            }
        }
        const int64_t at = (int64_t)t * width + n;
        if (!residual) out[at] = any ? out_scale * sum : 0.f;
        else if (any) out[at] = fmaf(out_scale, sum, residual[at]);
        else if (out != residual) out[at] = residual[at];
    }
}

}  // namespace st

using namespace st;

extern "C" int st_moe_route(int* ids, float* weights, const float* logits, const int* token_item, int num_tokens,
                            int experts, int top, int mode, int groups, int keep, hipStream_t stream) {
    ST_CHECK(mode >= 0 && mode <= 2, "moe_route: mode 0 (sigmoid of each), 1 (softmax over the chosen) or 2 (softmax "
             "over all, the choice within the best groups)");
    if (mode != 2) groups = keep = 1;
    ST_CHECK(groups >= 1 && groups <= 64 && experts % groups == 0 && keep >= 1 && keep <= groups,
             "moe_route: %d experts in %d groups of which %d are kept (up to 64 equal groups)", experts, groups, keep);
    ST_CHECK(top <= keep * (experts / groups), "moe_route: %d experts a token do not fit %d groups of %d", top, keep,
             experts / groups);
    ST_CHECK(num_tokens >= 0 && experts > 0, "moe_route: bad sizes");
    ST_CHECK(top >= 1 && top <= kMaxTop && top <= experts, "moe_route: 1 to %d experts a token (of %d), not %d",
             kMaxTop, experts, top);
    ST_CHECK(ids && weights && logits, "moe_route: null operand");
    if (num_tokens == 0) return 0;
    // workgroups of as many tokens as have their rows side by side in 48 KB of LDS (256, 64, or none staged)
    const size_t row = (size_t)(experts + 1) * sizeof(float);
    const int threads = 256 * row <= 48 * 1024 ? 256 : 64;
    const int stage = threads * row <= 48 * 1024;
    moe_route_kernel<<<(num_tokens + threads - 1) / threads, threads, stage ? threads * row : 0, stream>>>(
        ids, weights, logits, token_item, num_tokens, experts, top, mode, groups, keep, stage);
    ST_LAUNCH_CHECK("moe_route");
    return 0;
}

extern "C" int st_moe_align(int* sorted, int* place_of_pair, int* tile_expert, const int* ids, int num_pairs,
                            int experts, int capacity, int tile, hipStream_t stream) {
    const int kTile = tile;
    ST_CHECK(num_pairs >= 0 && experts > 0 && experts <= 4096, "moe_align: bad sizes (up to 4096 experts)");
    ST_CHECK(tile == 16 || tile == 64 || tile == 128, "moe_align: tiles of 16, 64 or 128 places, not %d", tile);
    ST_CHECK(capacity % kTile == 0 && capacity >= (num_pairs + kTile - 1) / kTile * kTile + kTile * experts,
             "moe_align: %d places do not hold %d pairs of %d experts in tiles of %d", capacity, num_pairs, experts, kTile);
    ST_CHECK(sorted && place_of_pair && tile_expert && ids, "moe_align: null operand");
    moe_align_kernel<<<1, 1024, (2 * experts + 1) * sizeof(int), stream>>>(sorted, place_of_pair, tile_expert, ids,
                                                                          num_pairs, experts, capacity, tile);
    ST_LAUNCH_CHECK("moe_align");
    return 0;
}

static bool rows_vectorised(const void* a, const void* b, const void* c, int depth, int dtype) {
    const int per = dtype == kF32 ? 4 : 8;
    return depth % per == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                                 reinterpret_cast<uintptr_t>(c)) & 15) == 0;
}

extern "C" int st_moe_up(void* y, const void* x, const void* w_gate, const void* w_up, const int* sorted,
                         const int* tile_expert, const float* weights, int capacity, int tile, int top, int width,
                         int inner, float limit, int style, int dtype, hipStream_t stream) {
    const int kTile = tile;
    ST_CHECK(style == 0 || style == 1, "moe_up: style 0 (weighted, clamped inputs) or 1 (plain gated unit)");
    ST_CHECK(tile == 16 || tile == 64 || tile == 128, "moe_up: tiles of 16, 64 or 128 places, not %d", tile);
    ST_CHECK(capacity > 0 && capacity % kTile == 0 && top >= 1 && width > 0 && inner > 0, "moe_up: bad sizes");
    ST_CHECK(y && x && w_gate && w_up && sorted && tile_expert && weights, "moe_up: null operand");
    const dim3 grid(capacity / kTile, (inner + 63) / 64);
    ST_CHECK(grid.y <= 65535, "moe_up: too many inner features");
    const int vec = rows_vectorised(x, w_gate, w_up, width, dtype);
    if (dtype == kBF16 && tile == 128 && vec) {
        const dim3 g2(capacity / 128, (inner + 63) / 64);
        moe_tiled_kernel<true><<<g2, 256, 0, stream>>>((bf16_t*)y, nullptr, nullptr, nullptr, (const bf16_t*)x,
            (const bf16_t*)w_gate, (const bf16_t*)w_up, sorted, tile_expert, weights, top, inner, width, limit, 1.f, style);
        ST_LAUNCH_CHECK("moe_up (tiled)");
        return 0;
    }
#define ST_UP(T, RT)                                                                                         \
    moe_up_kernel<T, RT><<<grid, 256, 0, stream>>>((T*)y, (const T*)x, (const T*)w_gate, (const T*)w_up, sorted, \
                                                   tile_expert, weights, top, width, inner, limit, style, vec)
    if (dtype == kF32) { if (tile == 16) ST_UP(float, 1); else if (tile == 64) ST_UP(float, 4); else ST_UP(float, 8); }
    else if (dtype == kBF16) { if (tile == 16) ST_UP(bf16_t, 1); else if (tile == 64) ST_UP(bf16_t, 4); else ST_UP(bf16_t, 8); }
    else ST_CHECK(false, "moe_up: unknown dtype %d", dtype);
#undef ST_UP
    ST_LAUNCH_CHECK("moe_up");
    return 0;
}

extern "C" int st_moe_down(float* out, const float* residual, float* pair_out, const void* y, const void* w_down,
                           const int* sorted, const int* tile_expert, int capacity, int tile, int top, int width,
                           int inner, float out_scale, int dtype, hipStream_t stream) {
    const int kTile = tile;
    ST_CHECK(tile == 16 || tile == 64 || tile == 128, "moe_down: tiles of 16, 64 or 128 places, not %d", tile);
    ST_CHECK(capacity > 0 && capacity % kTile == 0 && top >= 1 && width > 0 && inner > 0, "moe_down: bad sizes");
    ST_CHECK(y && w_down && sorted && tile_expert, "moe_down: null operand");
    ST_CHECK(pair_out ? true : (top == 1 && out && residual),
             "moe_down: without a row per pair the result goes to the stream, for one expert a token only");
    const dim3 grid(capacity / kTile, (width + 63) / 64);
    ST_CHECK(grid.y <= 65535, "moe_down: too wide");
    const int vec = rows_vectorised(y, w_down, w_down, inner, dtype);
    if (dtype == kBF16 && tile == 128 && vec) {
        const dim3 g2(capacity / 128, (width + 127) / 128);
        moe_tiled_kernel<false><<<g2, 256, 0, stream>>>(nullptr, out, residual, pair_out, (const bf16_t*)y,
            (const bf16_t*)w_down, nullptr, sorted, tile_expert, nullptr, top, width, inner, 0.f, out_scale, 0);
        ST_LAUNCH_CHECK("moe_down (tiled)");
        return 0;
    }
#define ST_DOWN(T, RT)                                                                                        \
    moe_down_kernel<T, RT><<<grid, 256, 0, stream>>>(out, residual, pair_out, (const T*)y, (const T*)w_down,      \
                                                     sorted, tile_expert, top, width, inner, out_scale, vec)
    if (dtype == kF32) { if (tile == 16) ST_DOWN(float, 1); else if (tile == 64) ST_DOWN(float, 4); else ST_DOWN(float, 8); }
    else if (dtype == kBF16) { if (tile == 16) ST_DOWN(bf16_t, 1); else if (tile == 64) ST_DOWN(bf16_t, 4); else ST_DOWN(bf16_t, 8); }
    else ST_CHECK(false, "moe_down: unknown dtype %d", dtype);
#undef ST_DOWN
    ST_LAUNCH_CHECK("moe_down");
    return 0;
}

extern "C" int st_moe_combine(float* out, const float* residual, const float* pair_out, const int* place_of_pair,
                              const float* weights, int num_tokens, int top, int width, float out_scale,
                              hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && top >= 1 && width > 0, "moe_combine: bad sizes");
    ST_CHECK(out && pair_out && place_of_pair, "moe_combine: null operand");
    if (num_tokens == 0) return 0;
    moe_combine_kernel<<<num_tokens, 256, 0, stream>>>(out, residual, pair_out, place_of_pair, weights, top, width, out_scale);
    ST_LAUNCH_CHECK("moe_combine");
    return 0;
}
