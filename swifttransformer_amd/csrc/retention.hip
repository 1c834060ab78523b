// Retention over prompts and portions in chunks: linear attention with one decay a head that does not
// change over time,
//
//   S_t = g S_(t-1) + (f k_t) v_t^T,   o_t = S_t^T q_t          (S [key channels x value channels] a head)
//
// Because g is constant, a chunk of n tokens that starts from the state S is
//
//   o_i = g^(i+1) S^T q_i + sum_(j<=i) g^(i-j) (q_i . f k_j) v_j,     S' = g^n S + sum_j g^(n-1-j) (f k_j) v_j^T
//
// so the chunks' own sums need no state and run side by side, and only the carry S -> S' walks a request's
// chunks in order.  Three kernels: the chunks' sums U (a workgroup a head, chunk and block of 32 value
// channels), the carry (a thread an element of the state; U's place then holds the chunk's start state),
// the outputs (a workgroup a head, chunk and value block).  Chunks are counted from an item's first row of
// the step, so a portion may start anywhere; the state comes from and goes back to the request's slot.
// Everything is float: the scan's recurrence in another order of sums.  Steps of single tokens keep the
// scan (csrc/state_scan.hip), whose walk is then one token long.
#include "api.h"
#include "common.h"

namespace st {

constexpr int kRetVB = 32;            // value channels a workgroup

// the chunk of an item that a global chunk index means; false past the last one
__device__ inline bool retention_find_chunk(int idx, const int* __restrict__ item_len,
                                            const int* __restrict__ item_slot, int num_items, int C, int& item,
                                            int& chunk) {
    int base = 0;
    for (int b = 0; b < num_items; ++b) {
        const int len = item_len[b];
        const int n = (item_slot[b] >= 0 && len > 0) ? (len + C - 1) / C : 0;
        if (idx < base + n) {
            item = b;
            chunk = idx - base;
            return true;
        }
        base += n;
    }
    return false;
}

// g^n with g^0 = 1 also for g = 0
__device__ inline float decay_pow(float g, int n) { return n == 0 ? 1.f : powf(g, (float)n); }

// U[idx, head, kk, col] = sum_j g^(n-1-j) f k_j[kk] v_j[col].  LDS: k [C, dk] | v [C, 32] | weights [C].
// Thread (group of 8, value channel): key channels group + 8 i.
template <int KQ>
__global__ __launch_bounds__(256) void retention_chunk_state_kernel(
    float* __restrict__ U, const float* __restrict__ k, int64_t k_stride, const float* __restrict__ v,
    int64_t v_stride, const float* __restrict__ decay, float key_factor, const int* __restrict__ item_len,
    const int* __restrict__ item_tok_off, const int* __restrict__ item_slot, int num_items, int heads, int dk,
    int dv, int C) {
    extern __shared__ __attribute__((aligned(16))) float ret_lds[];
    const int head = blockIdx.x, idx = blockIdx.y, vb = blockIdx.z * kRetVB;
    int item, c;
    if (!retention_find_chunk(idx, item_len, item_slot, num_items, C, item, c)) return;
    const int n = min(C, item_len[item] - c * C);
    const int64_t row0 = (int64_t)item_tok_off[item] + (int64_t)c * C;
    float* ks = ret_lds;
    float* vs = ks + C * dk;
    float* pw = vs + C * kRetVB;
    const float g = decay[head];
    for (int e = threadIdx.x; e < n * dk; e += 256) {
        const int j = e / dk, kk = e - j * dk;
        ks[e] = k[(row0 + j) * k_stride + (int64_t)head * dk + kk] * key_factor;
    }
    for (int e = threadIdx.x; e < n * kRetVB; e += 256) {
        const int j = e / kRetVB, col = vb + (e - j * kRetVB);
        vs[e] = col < dv ? v[(row0 + j) * v_stride + (int64_t)head * dv + col] : 0.f;
    }
    if (threadIdx.x < n) pw[threadIdx.x] = decay_pow(g, n - 1 - threadIdx.x);
    __syncthreads();
    const int vv = threadIdx.x & (kRetVB - 1), g8 = threadIdx.x >> 5;
    float acc[KQ];
#pragma unroll
    for (int i = 0; i < KQ; ++i) acc[i] = 0.f;
    for (int j = 0; j < n; ++j) {
        const float vw = vs[j * kRetVB + vv] * pw[j];
        const float* kr = ks + j * dk;
#pragma unroll
        for (int i = 0; i < KQ; ++i) {
            const int kk = g8 + 8 * i;
            acc[i] = fmaf(kk < dk ? kr[kk] : 0.f, vw, acc[i]);
        }
    }
    const int col = vb + vv;
    if (col >= dv) return;
    float* u = U + ((int64_t)idx * heads + head) * dk * dv + col;
#pragma unroll
    for (int i = 0; i < KQ; ++i) {
        const int kk = g8 + 8 * i;
        if (kk < dk) u[(int64_t)kk * dv] = acc[i];
    }
}

// A thread an element of a request's state: S walks the item's chunks, leaving at U's place the state each
// chunk starts from; the last S goes back to the slot.
__global__ __launch_bounds__(256) void retention_carry_kernel(
    float* __restrict__ U, float* __restrict__ state, int64_t slot_stride, const float* __restrict__ decay,
    const int* __restrict__ item_len, const int* __restrict__ item_slot, int heads, int dk, int dv, int C) {
    const int head = blockIdx.x, item = blockIdx.y;
    const int e = blockIdx.z * 256 + threadIdx.x;
    const int slot = item_slot[item], len = item_len[item];
    if (slot < 0 || len <= 0 || e >= dk * dv) return;
    int base = 0;
    for (int b = 0; b < item; ++b) {
        const int l = item_len[b];
        base += (item_slot[b] >= 0 && l > 0) ? (l + C - 1) / C : 0;
    }
    const int chunks = (len + C - 1) / C;
    const float g = decay[head];
    const float gC = decay_pow(g, C), gLast = decay_pow(g, len - (chunks - 1) * C);
    const int64_t plane = (int64_t)dk * dv;
    float* sp = state + (int64_t)slot * slot_stride + (int64_t)head * plane + e;
    float* u = U + ((int64_t)base * heads + head) * plane + e;
    float S = *sp;
    for (int c = 0; c < chunks; ++c) {
        const float add = *u;
        *u = S;
        S = fmaf(c == chunks - 1 ? gLast : gC, S, add);
        u += (int64_t)heads * plane;
    }
    *sp = S;
}

// o_i = g^(i+1) S^T q_i + sum_(j<=i) P[i, j] v_j, P[i, j] = g^(i-j) (q_i . f k_j).
// LDS: q [C, dk + 1] | k [C, dk + 1] | v [C, 32] | P [C, C] | powers [C + 1].  Rows of q and k are one float
// longer than they need be, so that lanes that read different rows at one channel hit different banks.
// Thread (group of 8, value channel): rows group + 8 r.
template <int C>
__global__ __launch_bounds__(256) void retention_chunk_out_kernel(
    float* __restrict__ out, const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k,
    int64_t k_stride, const float* __restrict__ v, int64_t v_stride, const float* __restrict__ S0,
    const float* __restrict__ decay, float key_factor, const int* __restrict__ item_len,
    const int* __restrict__ item_tok_off, const int* __restrict__ item_slot, int num_items, int heads, int dk,
    int dv) {
    extern __shared__ __attribute__((aligned(16))) float ret_lds[];
    constexpr int R = C / 8;
    const int head = blockIdx.x, idx = blockIdx.y, vb = blockIdx.z * kRetVB;
    int item, c;
    if (!retention_find_chunk(idx, item_len, item_slot, num_items, C, item, c)) return;
    const int n = min(C, item_len[item] - c * C);
    const int64_t row0 = (int64_t)item_tok_off[item] + (int64_t)c * C;
    const int dkp = dk + 1;
    float* qs = ret_lds;
    float* ks = qs + C * dkp;
    float* vs = ks + C * dkp;
    float* P = vs + C * kRetVB;
    float* pw = P + C * C;
    const float g = decay[head];
    for (int e = threadIdx.x; e < C * dk; e += 256) {
        const int j = e / dk, kk = e - j * dk;
        const bool in = j < n;
        qs[j * dkp + kk] = in ? q[(row0 + j) * q_stride + (int64_t)head * dk + kk] : 0.f;
        ks[j * dkp + kk] = in ? k[(row0 + j) * k_stride + (int64_t)head * dk + kk] * key_factor : 0.f;
    }
    for (int e = threadIdx.x; e < C * kRetVB; e += 256) {
        const int j = e / kRetVB, col = vb + (e - j * kRetVB);
        vs[e] = (j < n && col < dv) ? v[(row0 + j) * v_stride + (int64_t)head * dv + col] : 0.f;
    }
    if (threadIdx.x <= C) pw[threadIdx.x] = decay_pow(g, threadIdx.x);
    __syncthreads();
    for (int e = threadIdx.x; e < C * C; e += 256) {
        const int i = e / C, j = e - i * C;
        float val = 0.f;
        if (j <= i && i < n) {
            const float* qi = qs + i * dkp;
            const float* kj = ks + j * dkp;
            float dot = 0.f;
            for (int kk = 0; kk < dk; ++kk) dot = fmaf(qi[kk], kj[kk], dot);
            val = dot * pw[i - j];
        }
        P[e] = val;
    }
    __syncthreads();
    const int vv = threadIdx.x & (kRetVB - 1), g8 = threadIdx.x >> 5;
    const int col = vb + vv;
    float within[R], carried[R];
#pragma unroll
    for (int r = 0; r < R; ++r) within[r] = carried[r] = 0.f;
    for (int j = 0; j < n; ++j) {
        const float vj = vs[j * kRetVB + vv];
#pragma unroll
        for (int r = 0; r < R; ++r) within[r] = fmaf(P[(g8 + 8 * r) * C + j], vj, within[r]);
    }
    if (col < dv) {
        const float* s = S0 + ((int64_t)idx * heads + head) * dk * dv + col;
        for (int kk = 0; kk < dk; ++kk) {
            const float sv = s[(int64_t)kk * dv];
#pragma unroll
            for (int r = 0; r < R; ++r) carried[r] = fmaf(qs[(g8 + 8 * r) * dkp + kk], sv, carried[r]);
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int i = g8 + 8 * r;
            if (i < n) out[(row0 + i) * ((int64_t)heads * dv) + (int64_t)head * dv + col] = fmaf(pw[i + 1], carried[r], within[r]);
        }
    }
}

}  // namespace st

using namespace st;

extern "C" int st_retention_chunk_rows(int key_dim) { return key_dim <= 64 ? 64 : key_dim <= 128 ? 32 : 16; }

extern "C" int st_retention_chunks(float* out, const float* q, int64_t q_stride, const float* k, int64_t k_stride,
                                   const float* v, int64_t v_stride, const float* decay, float key_factor,
                                   float* state, int64_t slot_stride, const int* item_len, const int* item_tok_off,
                                   const int* item_slot, int num_items, int num_rows, int heads, int key_dim,
                                   int value_dim, float* scratch, int64_t scratch_chunks, hipStream_t stream) {
    ST_CHECK(num_items >= 0 && num_rows >= 0 && heads > 0 && key_dim > 0 && value_dim > 0, "retention_chunks: bad sizes");
    ST_CHECK(key_dim <= 256, "retention_chunks: up to 256 key channels a head, not %d", key_dim);
    if (num_items == 0 || num_rows == 0) return 0;
    ST_CHECK(out && q && k && v && decay && state && item_len && item_tok_off && item_slot && scratch,
             "retention_chunks: null operand");
    const int C = st_retention_chunk_rows(key_dim);
    // every item's last chunk may be a short one
    const int64_t chunks = num_rows / C + num_items;
    ST_CHECK(scratch_chunks >= chunks, "retention_chunks: scratch for %lld chunks, %lld needed", (long long)scratch_chunks,
             (long long)chunks);
    const int vblocks = (value_dim + kRetVB - 1) / kRetVB;
    ST_CHECK(chunks <= 65535 && vblocks <= 65535 && num_items <= 65535, "retention_chunks: too many chunks, items or value channels");
    const dim3 grid(heads, (unsigned)chunks, vblocks);
    const size_t lds1 = sizeof(float) * ((size_t)C * key_dim + C * kRetVB + C);
#define ST_RET_STATE(KQ)                                                                                              \
    retention_chunk_state_kernel<KQ><<<grid, 256, lds1, stream>>>(scratch, k, k_stride, v, v_stride, decay, key_factor, \
        item_len, item_tok_off, item_slot, num_items, heads, key_dim, value_dim, C)
    if (key_dim <= 64) ST_RET_STATE(8);
    else if (key_dim <= 128) ST_RET_STATE(16);
    else ST_RET_STATE(32);
#undef ST_RET_STATE
    ST_LAUNCH_CHECK("retention_chunks (sums)");
    const dim3 carry(heads, num_items, (unsigned)((key_dim * value_dim + 255) / 256));
    retention_carry_kernel<<<carry, 256, 0, stream>>>(scratch, state, slot_stride, decay, item_len, item_slot, heads,
                                                      key_dim, value_dim, C);
    ST_LAUNCH_CHECK("retention_chunks (carry)");
    const size_t lds3 = sizeof(float) * ((size_t)2 * C * (key_dim + 1) + C * kRetVB + C * C + C + 1);
    ST_CHECK(lds3 <= 64 * 1024, "retention_chunks: %zu bytes of LDS", lds3);
#define ST_RET_OUT(CC)                                                                                               \
    retention_chunk_out_kernel<CC><<<grid, 256, lds3, stream>>>(out, q, q_stride, k, k_stride, v, v_stride, scratch,  \
        decay, key_factor, item_len, item_tok_off, item_slot, num_items, heads, key_dim, value_dim)
    if (C == 64) ST_RET_OUT(64);
    else if (C == 32) ST_RET_OUT(32);
    else ST_RET_OUT(16);
#undef ST_RET_OUT
    ST_LAUNCH_CHECK("retention_chunks (outputs)");
    return 0;
}
