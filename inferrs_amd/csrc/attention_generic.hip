// Paged grouped-query attention, plain variant: one wave per (token, query head), any head
// size up to 512, any page size, optional window; 32-bit or bfloat16 storage, all arithmetic
// in 32-bit.  It is the 32-bit path of the engine and the fallback for head sizes that the
// matrix-core kernels do not take.
//
// Formula as in the reference: S = (q . k) * scale after the dot product, keys j <= position
// (inferrs-models/src/models/attention_utils.rs:61-85), softmax over keys, O = P v
// (inferrs-models/src/models/qwen3.rs:166-192); query head h reads key/value head
// h / (nq / nkv) (attention_utils.rs:38-49).
//
// A (token, head) pair walks its keys in ascending order in tiles of 64 that are aligned to
// absolute position, with a running maximum and sum.  Nothing in that order depends on how
// the tokens were cut into steps, on the other rows of the batch or on which pages hold the
// keys, so the result for a position is the same bit pattern under every cutting.
#include "common.h"
#include "api.h"

#define AG_MAX_HEAD_DIM 512
#define AG_DIMS_PER_LANE (AG_MAX_HEAD_DIM / IA_WAVE)

template <typename T>
__global__ __launch_bounds__(IA_WAVE) void attn_generic_kernel(
    T* __restrict__ out,                 // [n, nq, d]
    const T* __restrict__ q,             // [n, nq, d]
    const T* __restrict__ k_cache,       // [pages, nkv, page_size, d]
    const T* __restrict__ v_cache,       // [pages, nkv, d, page_size]  (transposed inside a page)
    const int* __restrict__ positions,   // [n]
    const int* __restrict__ token_seq,   // [n] row of block_table
    const int* __restrict__ block_table, // [seqs, max_pages]
    int max_pages, int nq, int nkv, int d, int page_size, int window, float scale) {
    __shared__ float sq[AG_MAX_HEAD_DIM];
    __shared__ float sp[IA_WAVE];
    const int lane = threadIdx.x;
    const int tok = blockIdx.x / nq;
    const int h = blockIdx.x - tok * nq;
    const int kvh = h / (nq / nkv);
    const int pos = positions[tok];
    const int* bt = block_table + (size_t)token_seq[tok] * max_pages;
    const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;

    const T* qrow = q + ((size_t)tok * nq + h) * d;
    for (int e = lane; e < d; e += IA_WAVE) sq[e] = ld(qrow + e);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float o[AG_DIMS_PER_LANE];
#pragma unroll
    for (int t = 0; t < AG_DIMS_PER_LANE; ++t) o[t] = 0.f;

    for (int tile = lo / IA_WAVE; tile <= pos / IA_WAVE; ++tile) {
        const int j = tile * IA_WAVE + lane;
        const bool valid = j >= lo && j <= pos;
        float s = -INFINITY;
        if (valid) {
            const int page = bt[j / page_size], off = j % page_size;
            const T* kp = k_cache + (((size_t)page * nkv + kvh) * page_size + off) * d;
            float acc = 0.f;
            for (int e = 0; e < d; ++e) acc = fmaf(sq[e], ld(kp + e), acc);
            s = acc * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float alpha = expf(m - m_new);
        l = l * alpha + wave_sum(p);
        sp[lane] = p;
        __syncthreads();
#pragma unroll
        for (int t = 0; t < AG_DIMS_PER_LANE; ++t) o[t] *= alpha;
        const int j0 = tile * IA_WAVE;
        const int first = lo > j0 ? lo - j0 : 0;
        const int last = pos - j0 < IA_WAVE - 1 ? pos - j0 : IA_WAVE - 1;
        for (int jj = first; jj <= last; ++jj) {
            const int key = j0 + jj;
            const int page = bt[key / page_size], off = key % page_size;
            const T* vp = v_cache + ((size_t)page * nkv + kvh) * d * page_size + off;
            const float pv = sp[jj];
#pragma unroll
            for (int t = 0; t < AG_DIMS_PER_LANE; ++t) {
                const int e = lane + t * IA_WAVE;
                if (e < d) o[t] = fmaf(pv, ld(vp + (size_t)e * page_size), o[t]);
            }
        }
        __syncthreads();
        m = m_new;
    }
    T* orow = out + ((size_t)tok * nq + h) * d;
    const float inv = 1.0f / l;
#pragma unroll
    for (int t = 0; t < AG_DIMS_PER_LANE; ++t) {
        const int e = lane + t * IA_WAVE;
        if (e < d) st(orow + e, o[t] * inv);
    }
}

extern "C" int ia_attention_generic(void* out, const void* q, const void* k_cache, const void* v_cache,
                                    const int* positions, const int* token_seq, const int* block_table,
                                    int n, int max_pages, int nq, int nkv, int d, int page_size,
                                    int window, float scale, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention: bad head counts nq=%d nkv=%d (n=%d)", nq, nkv, n);
    IA_CHECK(d > 0 && d <= AG_MAX_HEAD_DIM, "attention: head_dim %d is outside 1..%d", d, AG_MAX_HEAD_DIM);
    IA_CHECK(page_size > 0 && max_pages > 0, "attention: bad page geometry page_size=%d max_pages=%d", page_size, max_pages);
    IA_CHECK(window >= 0, "attention: window %d must be >= 0 (0 = all keys)", window);
    if (n == 0) return 0;
    IA_CHECK((long long)n * nq < 2147483647LL, "attention: %d tokens x %d heads exceed the grid", n, nq);
    const unsigned grid = (unsigned)n * (unsigned)nq;
    if (dtype == IA_F32)
        attn_generic_kernel<float><<<grid, IA_WAVE, 0, stream>>>(
            (float*)out, (const float*)q, (const float*)k_cache, (const float*)v_cache, positions,
            token_seq, block_table, max_pages, nq, nkv, d, page_size, window, scale);
    else if (dtype == IA_BF16)
        attn_generic_kernel<bf16_t><<<grid, IA_WAVE, 0, stream>>>(
            (bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, positions,
            token_seq, block_table, max_pages, nq, nkv, d, page_size, window, scale);
    else
        IA_CHECK(false, "attention: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("attention_generic");
    return 0;
}
