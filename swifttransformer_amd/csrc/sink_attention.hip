// Attention over a paged cache whose heads are coupled before the softmax, with a sink and a
// sliding window, and keys and values of different sizes:
//
//   r_g(i, j)  = scale * q_g(i) . k_c(g)(j)                  c(g) = g / (heads / kv_heads)
//   s_h(i, j)  = sum_g M[h, g] r_g(i, j)                     (M null: s = r)
//   p_h(i, j)  = exp(s_h(i, j)) / (sink + sum_j' exp(s_h(i, j')))      over max(0, i - window + 1) <= j' <= i
//                and, with keep_first > 0, over j' < keep_first as well (the first tokens stay visible)
//   o_h(i)     = sum_j p_h(i, j) v_c(h)(j)
//
// sink = 1 puts a key of score 0 and no value into every row's sum (its softmax starts from the
// maximum 0 and the sum 1); sink = 0 is the ordinary softmax.  Scores, the mix, maxima, sums and
// the weighted values are float.
//
// Because every head's score of a key needs all heads' products with that key, a workgroup owns
// a query row with all its heads and walks the row's keys in blocks of 64: products of all heads
// with the block (a lane a key), the mix, one softmax update a head (a wave a head, a lane a key),
// then the weighted sum of the block's values (a thread a group of output coordinates).  Keys may
// be split over several workgroups a row (`splits`); their partial results are merged by a second
// kernel.
#include "api.h"
#include "common.h"

namespace st {

constexpr int kKeyBlock = 64;

struct SinkAttnArgs {
    void* out;                 // [T, heads * value_dim] storage type
    float* part_o;             // [T, splits, heads * value_dim] and
    float* part_ml;            // [T, splits, heads, 2] (maximum, sum) when splits > 1
    const void* q; int64_t q_stride;
    const void* k_cache; int64_t k_page_stride;
    const void* v_cache; int64_t v_page_stride;
    const float* mix;          // [heads, heads] or null
    const int* token_item; const int* positions; const int* block_table;
    int max_pages, page_size, heads, kv_heads, key_dim, value_dim, window, keep_first, sink, splits;
    float scale;
};

// Products of up to four heads' queries (LDS, floats) with one key row: the row is loaded once, in
// batches of four 16-byte pieces so that the loads are in flight together.
template <typename T, int NQ>
__device__ inline void dot_rows(const float* __restrict__ qs, int q_stride, const T* __restrict__ kp, int dim,
                                float* acc) {
    constexpr int V = Elem<T>::kVec;
#pragma unroll
    for (int n = 0; n < NQ; ++n) acc[n] = 0.f;
    int d = 0;
    if (dim % V == 0) {
        for (; d + 4 * V <= dim; d += 4 * V) {
            uint4 raw[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) raw[u] = *reinterpret_cast<const uint4*>(kp + d + u * V);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                float kv[V];
                Elem<T>::unpack(raw[u], kv);
#pragma unroll
                for (int n = 0; n < NQ; ++n) {
                    // (the queries lie on 16-byte borders in LDS: dim is a multiple of four here)
                    const float4* q4 = reinterpret_cast<const float4*>(qs + n * q_stride + d + u * V);
#pragma unroll
                    for (int i = 0; i < V / 4; ++i) {
                        const float4 qv = q4[i];
                        acc[n] = fmaf(qv.x, kv[4 * i], acc[n]);
                        acc[n] = fmaf(qv.y, kv[4 * i + 1], acc[n]);
                        acc[n] = fmaf(qv.z, kv[4 * i + 2], acc[n]);
                        acc[n] = fmaf(qv.w, kv[4 * i + 3], acc[n]);
                    }
                }
            }
        }
        for (; d < dim; d += V) {
            float kv[V];
            Elem<T>::load_vec(kp + d, kv);
#pragma unroll
            for (int n = 0; n < NQ; ++n)
#pragma unroll
                for (int i = 0; i < V; ++i) acc[n] = fmaf(qs[n * q_stride + d + i], kv[i], acc[n]);
        }
    } else {
        for (; d < dim; ++d) {
            const float kv = Elem<T>::load(kp + d);
#pragma unroll
            for (int n = 0; n < NQ; ++n) acc[n] = fmaf(qs[n * q_stride + d], kv, acc[n]);
        }
    }
}

// NG groups of W neighbouring output coordinates a thread (W = 1, or the elements of a 16-byte load
// where the value size is a multiple of that)
template <typename T, int NG, int W>
__global__ __launch_bounds__(256) void sink_attention_kernel(SinkAttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int H = a.heads, G = a.kv_heads, dk = a.key_dim, dv = a.value_dim, per = a.heads / a.kv_heads;
    float* qs = lds;                               // [H * dk]
    float* sraw = qs + H * dk;                     // [H * 64]
    float* smix = sraw + H * kKeyBlock;            // [H * 64]
    float* mix_s = smix + H * kKeyBlock;           // [H * H] (if mix)
    float* m_s = mix_s + (a.mix ? H * H : 0);      // [H]
    float* l_s = m_s + H;
    float* al_s = l_s + H;
    // where each key of the block lies in the two pools (elements from the pool's start, before the
    // head's share of the page); keys beyond the block's last repeat its first and weigh nothing
    int64_t* koff = (int64_t*)(al_s + H + (((al_s + H) - lds) & 1));     // [64], 8-byte aligned
    int64_t* voff = koff + kKeyBlock;                             // [64]
    const int t = blockIdx.x, split = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int item = a.token_item[t], pos = a.positions[t];
    const int width = H * dv;
    T* out = (T*)a.out + (int64_t)t * width;
    if (item < 0 || pos < 0) {                     // a padding row
        if (a.splits == 1)
            for (int e = tid; e < width; e += 256) Elem<T>::store(out + e, 0.f);
        else if (tid < H) {
            float* ml = a.part_ml + (((int64_t)t * a.splits + split) * H + tid) * 2;
            ml[0] = -INFINITY; ml[1] = 0.f;
        }
        return;
    }
    const T* q = (const T*)a.q + (int64_t)t * a.q_stride;
    for (int e = tid; e < H * dk; e += 256) qs[e] = Elem<T>::load(q + e) * a.scale;
    if (a.mix) for (int e = tid; e < H * H; e += 256) mix_s[e] = a.mix[e];
    const bool with_sink = a.sink && split == 0;   // the sink belongs to one split only
    if (tid < H) { m_s[tid] = with_sink ? 0.f : -INFINITY; l_s[tid] = with_sink ? 1.f : 0.f; }
    // the output coordinates of this thread: head, and where its value channel lies within a key's values
    // (a thread beyond the row's width repeats coordinate 0 and stores nothing)
    float o[NG][W];
    int oh[NG], ov[NG];
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int e = (tid + 256 * i) * W < width ? (tid + 256 * i) * W : 0;
#pragma unroll
        for (int w = 0; w < W; ++w) o[i][w] = 0.f;
        oh[i] = e / dv;
        ov[i] = (oh[i] / per) * a.page_size * dv + (e - oh[i] * dv);
    }
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    // the row's key blocks: those of the first tokens that stay visible behind the window (positions
    // below both keep_first and lo), then those of the window; this split's share of them
    const int kept = min(a.keep_first, lo);
    const int kept_blocks = (kept + kKeyBlock - 1) / kKeyBlock;
    const int blocks = kept_blocks + (pos - lo) / kKeyBlock + 1;
    const int share = (blocks + a.splits - 1) / a.splits;
    const int b0 = split * share, b1 = min(blocks, b0 + share);
    const int* bt = a.block_table + (int64_t)item * a.max_pages;
    const T* kc = (const T*)a.k_cache;
    const T* vc = (const T*)a.v_cache;
    for (int b = b0; b < b1; ++b) {
        const int j0 = b < kept_blocks ? b * kKeyBlock : lo + (b - kept_blocks) * kKeyBlock;
        const int nk = min(kKeyBlock, (b < kept_blocks ? kept : pos + 1) - j0);
        __syncthreads();                           // the block before is done with the shared lists
        if (tid < kKeyBlock) {
            const int j = j0 + (tid < nk ? tid : 0), pi = j / a.page_size;
            const int page = max(bt[pi], 0);
            const int place = j - pi * a.page_size;
            koff[tid] = (int64_t)page * a.k_page_stride + (int64_t)place * dk;
            voff[tid] = (int64_t)page * a.v_page_stride + (int64_t)place * dv;
        }
        __syncthreads();
        // a thread a (key head, key): the key row is loaded once for the heads that share it
        for (int p = tid; p < G * kKeyBlock; p += 256) {
            const int c = p >> 6, jj = p & 63;
            const T* kp = kc + koff[jj] + (int64_t)c * a.page_size * dk;
            for (int g0 = c * per; g0 < (c + 1) * per; g0 += 4) {
                const int n = min(4, (c + 1) * per - g0);
                float acc[4] = {0.f, 0.f, 0.f, 0.f};
                if (n == 4) dot_rows<T, 4>(qs + g0 * dk, dk, kp, dk, acc);
                else if (n == 3) dot_rows<T, 3>(qs + g0 * dk, dk, kp, dk, acc);
                else if (n == 2) dot_rows<T, 2>(qs + g0 * dk, dk, kp, dk, acc);
                else dot_rows<T, 1>(qs + g0 * dk, dk, kp, dk, acc);
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (u < n) sraw[(g0 + u) * kKeyBlock + jj] = acc[u];
            }
        }
        __syncthreads();
        if (a.mix && H % 4 == 0) {
            // a thread's outputs share its key (the lane) and differ in the head (wave + 4 i): the key's
            // products are read once four heads at a time, the mix's rows in 16-byte pieces
            const int jj = lane, nout = H >> 2;
            for (int i0 = 0; i0 < nout; i0 += 8) {
                float acc[8];
#pragma unroll
                for (int ii = 0; ii < 8; ++ii) acc[ii] = 0.f;
                for (int g0 = 0; g0 < H; g0 += 4) {
                    const float s0 = sraw[g0 * kKeyBlock + jj], s1 = sraw[(g0 + 1) * kKeyBlock + jj];
                    const float s2 = sraw[(g0 + 2) * kKeyBlock + jj], s3 = sraw[(g0 + 3) * kKeyBlock + jj];
#pragma unroll
                    for (int ii = 0; ii < 8; ++ii) {
                        if (i0 + ii < nout) {
                            const int h = wave + 4 * (i0 + ii);
                            const float4 m = *reinterpret_cast<const float4*>(mix_s + h * H + g0);
                            acc[ii] = fmaf(m.w, s3, fmaf(m.z, s2, fmaf(m.y, s1, fmaf(m.x, s0, acc[ii]))));
                        }
                    }
                }
#pragma unroll
                for (int ii = 0; ii < 8; ++ii)
                    if (i0 + ii < nout) smix[(wave + 4 * (i0 + ii)) * kKeyBlock + jj] = jj < nk ? acc[ii] : -INFINITY;
            }
        } else
        for (int p = tid; p < H * kKeyBlock; p += 256) {
            const int h = p >> 6, jj = p & 63;
            float s = -INFINITY;
            if (jj < nk) {
                if (a.mix) {
                    s = 0.f;
                    for (int g = 0; g < H; ++g) s = fmaf(mix_s[h * H + g], sraw[g * kKeyBlock + jj], s);
                } else {
                    s = sraw[p];
                }
            }
            smix[p] = s;
        }
        __syncthreads();
        for (int h = wave; h < H; h += 4) {
            const float s = smix[h * kKeyBlock + lane];
            const float m_old = m_s[h];
            const float m_new = fmaxf(m_old, wave_max(s));
            const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
            smix[h * kKeyBlock + lane] = p;
            const float sum = wave_sum(p);
            if (lane == 0) {
                const float alpha = (m_old == -INFINITY) ? 0.f : expf(m_old - m_new);
                al_s[h] = alpha;
                l_s[h] = l_s[h] * alpha + sum;
                m_s[h] = m_new;
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            const float al = al_s[oh[i]];
#pragma unroll
            for (int w = 0; w < W; ++w) o[i][w] *= al;
        }
#pragma unroll 1
        for (int jj = 0; jj < kKeyBlock; jj += 4) {              // loads of four keys in flight, then their sums
            const int64_t v0 = voff[jj], v1 = voff[jj + 1], v2 = voff[jj + 2], v3 = voff[jj + 3];
#pragma unroll
            for (int i = 0; i < NG; ++i) {
                const T* vh = vc + ov[i];
                float x0[W], x1[W], x2[W], x3[W];
                if (W == 1) {
                    x0[0] = Elem<T>::load(vh + v0); x1[0] = Elem<T>::load(vh + v1);
                    x2[0] = Elem<T>::load(vh + v2); x3[0] = Elem<T>::load(vh + v3);
                } else {
                    Elem<T>::load_vec(vh + v0, x0); Elem<T>::load_vec(vh + v1, x1);
                    Elem<T>::load_vec(vh + v2, x2); Elem<T>::load_vec(vh + v3, x3);
                }
                const float* pw = smix + oh[i] * kKeyBlock + jj;
                const float p0 = pw[0], p1 = pw[1], p2 = pw[2], p3 = pw[3];
#pragma unroll
                for (int w = 0; w < W; ++w)
                    o[i][w] = fmaf(p3, x3[w], fmaf(p2, x2[w], fmaf(p1, x1[w], fmaf(p0, x0[w], o[i][w]))));
            }
        }
    }
    __syncthreads();
    float* po = a.splits == 1 ? nullptr : a.part_o + ((int64_t)t * a.splits + split) * width;
#pragma unroll
    for (int i = 0; i < NG; ++i) {
        const int e = (tid + 256 * i) * W;
        if (e >= width) break;
        if (po) {
#pragma unroll
            for (int w = 0; w < W; ++w) po[e + w] = o[i][w];
        } else {
            const float l = l_s[oh[i]];
            const float r = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
            for (int w = 0; w < W; ++w) Elem<T>::store(out + e + w, o[i][w] * r);
        }
    }
    if (po && tid < H) {
        float* ml = a.part_ml + (((int64_t)t * a.splits + split) * H + tid) * 2;
        ml[0] = m_s[tid]; ml[1] = l_s[tid];
    }
}

// out[t, h, :] = sum_s e^(m_s - m) o_s / sum_s e^(m_s - m) l_s over the splits of a row
template <typename T>
__global__ __launch_bounds__(256) void sink_attention_merge_kernel(
    T* __restrict__ out, const float* __restrict__ part_o, const float* __restrict__ part_ml, int splits, int heads,
    int value_dim) {
    __shared__ float wgt[256 * 16];                // [heads, splits]: a split's weight in its head's sum
    const int t = blockIdx.x;
    const int width = heads * value_dim;
    const float* ml = part_ml + (int64_t)t * splits * heads * 2;
    const float* po = part_o + (int64_t)t * splits * width;
    for (int h = threadIdx.x; h < heads; h += 256) {
        float m = -INFINITY;
        for (int s = 0; s < splits; ++s) m = fmaxf(m, ml[(s * heads + h) * 2]);
        float den = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float ms = ml[(s * heads + h) * 2];
            const float w = ms == -INFINITY ? 0.f : expf(ms - m);
            wgt[h * splits + s] = w;
            den = fmaf(w, ml[(s * heads + h) * 2 + 1], den);
        }
        const float r = den > 0.f ? 1.f / den : 0.f;
        for (int s = 0; s < splits; ++s) wgt[h * splits + s] *= r;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < width; e += 256) {
        const float* w = wgt + (e / value_dim) * splits;
        float num = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float x = po[(int64_t)s * width + e];      // (a split without keys may hold anything)
            num = fmaf(w[s], w[s] > 0.f ? x : 0.f, num);
        }
        Elem<T>::store(out + (int64_t)t * width + e, num);
    }
}

template <typename T>
static int launch_sink_attention(const SinkAttnArgs& a, int num_tokens, size_t lds_bytes, hipStream_t stream) {
    constexpr int V = Elem<T>::kVec;
    const int width = a.heads * a.value_dim;
    const dim3 grid(num_tokens, a.splits);
    if (a.value_dim % V == 0) {
        const int per_thread = (width / V + 255) / 256;
        if (per_thread <= 1) sink_attention_kernel<T, 1, V><<<grid, 256, lds_bytes, stream>>>(a);
        else if (per_thread <= 2) sink_attention_kernel<T, 2, V><<<grid, 256, lds_bytes, stream>>>(a);
        else if (per_thread <= 4) sink_attention_kernel<T, 4, V><<<grid, 256, lds_bytes, stream>>>(a);
        else sink_attention_kernel<T, 32 / V, V><<<grid, 256, lds_bytes, stream>>>(a);
    } else {
        const int per_thread = (width + 255) / 256;
        if (per_thread <= 2) sink_attention_kernel<T, 2, 1><<<grid, 256, lds_bytes, stream>>>(a);
        else if (per_thread <= 8) sink_attention_kernel<T, 8, 1><<<grid, 256, lds_bytes, stream>>>(a);
        else sink_attention_kernel<T, 32, 1><<<grid, 256, lds_bytes, stream>>>(a);
    }
    ST_LAUNCH_CHECK("sink_attention");
    if (a.splits > 1) {
        sink_attention_merge_kernel<T><<<num_tokens, 256, 0, stream>>>((T*)a.out, a.part_o, a.part_ml, a.splits,
                                                                      a.heads, a.value_dim);
        ST_LAUNCH_CHECK("sink_attention_merge");
    }
    return 0;
}

}  // namespace st

using namespace st;

// LDS bytes a workgroup of st_sink_attention needs (the host checks it against the device's limit)
extern "C" int64_t st_sink_attention_lds(int heads, int key_dim, int mixed) {
    return 4 * ((int64_t)heads * key_dim + 2 * (int64_t)heads * kKeyBlock + (mixed ? (int64_t)heads * heads : 0) +
                3 * (int64_t)heads + 1 + 4 * kKeyBlock);
}

extern "C" int st_sink_attention(void* out, float* part_o, float* part_ml, const void* q, int64_t q_stride,
                                 const void* k_cache, int64_t k_page_stride, const void* v_cache,
                                 int64_t v_page_stride, const float* mix, const int* token_item, const int* positions,
                                 const int* block_table, int max_pages, int page_size, int num_tokens, int heads,
                                 int kv_heads, int key_dim, int value_dim, float scale, int window, int keep_first,
                                 int sink, int splits, int dtype, hipStream_t stream) {
    ST_CHECK(num_tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && key_dim > 0 && value_dim > 0,
             "sink_attention: bad sizes");
    ST_CHECK(page_size > 0 && max_pages > 0 && window >= 0 && keep_first >= 0 && splits >= 1 && splits <= 16, "sink_attention: 1 to 16 splits");
    ST_CHECK(heads <= 256, "sink_attention: up to 256 heads, not %d", heads);
    ST_CHECK(heads * value_dim <= 32 * 256, "sink_attention: heads x value size up to 8192, not %d", heads * value_dim);
    const int64_t lds_bytes = st_sink_attention_lds(heads, key_dim, mix != nullptr);
    ST_CHECK(lds_bytes <= 64 * 1024, "sink_attention: %lld bytes of LDS a row (heads x key size too large)",
             (long long)lds_bytes);
    if (num_tokens == 0) return 0;
    ST_CHECK(out && q && k_cache && v_cache && token_item && positions && block_table, "sink_attention: null operand");
    ST_CHECK(splits == 1 || (part_o && part_ml), "sink_attention: split keys need room for the partial results");
    SinkAttnArgs a;
    a.out = out; a.part_o = part_o; a.part_ml = part_ml; a.q = q; a.q_stride = q_stride;
    a.k_cache = k_cache; a.k_page_stride = k_page_stride; a.v_cache = v_cache; a.v_page_stride = v_page_stride;
    a.mix = mix; a.token_item = token_item; a.positions = positions; a.block_table = block_table;
    a.max_pages = max_pages; a.page_size = page_size; a.heads = heads; a.kv_heads = kv_heads;
    a.key_dim = key_dim; a.value_dim = value_dim; a.window = window; a.keep_first = keep_first; a.sink = sink; a.splits = splits;
    a.scale = scale;
    if (dtype == kF32) return launch_sink_attention<float>(a, num_tokens, (size_t)lds_bytes, stream);
    if (dtype == kBF16) return launch_sink_attention<bf16_t>(a, num_tokens, (size_t)lds_bytes, stream);
    ST_CHECK(false, "sink_attention: unknown dtype %d", dtype);
    return 0;
}
