// Paged grouped-query attention, plain variant: any head size up to 512, any page size, optional
// window; 32-bit or bfloat16 storage, all arithmetic in 32-bit on the vector units.  It is the
// 32-bit path of the engine and the fallback for head sizes that the matrix-core kernels do not take.
//
// Formula as in the reference: S = (q . k) * scale after the dot product, keys j <= position
// (inferrs-models/src/models/attention_utils.rs:61-85), softmax over keys, O = P v
// (inferrs-models/src/models/qwen3.rs:166-192); query head h reads key/value head
// h / (nq / nkv) (attention_utils.rs:38-49).
//
// A (token, query head) pair walks its keys in ascending order in tiles of 64 that are aligned to
// absolute position, with a running maximum and sum; a score is one chain of fused multiply-adds
// over the head's dimensions in ascending order, an output one chain over the tile's keys in
// ascending order.  Nothing in that order depends on how the tokens were cut into steps, on the other
// rows of the batch or on which pages hold the keys, so the result for a position is the same bit
// pattern under every cutting.  The keys are walked in segments of 512 (aligned to absolute position as well):
// a segment's maximum, sum and outputs are formed from nothing and then merged into the totals in ascending order.
// That merge is the same arithmetic whether one wave walks all segments of a token (steps of many tokens) or one
// wave a segment leaves them in memory for a merge kernel (steps of few tokens, which would otherwise keep a few
// waves busy for a long walk): both forms give the same bits.
//
// One wave a (token, key/value head, group of up to four of its query heads): the heads of a group share
// every key and value that is read.  A tile's keys come into shared memory 64 dimensions at a time in whole
// rows (a lane fetching a key's row for itself asks for 64 cache lines with every load), then lane j forms
// key j's scores with the queries broadcast from shared memory; the values come the same way, 64 dimensions
// x 64 keys as they lie in a page (dimension-major), and lane e adds up dimension e.  Keys outside the range
// of a token are staged as zeros and take the probability 0, so that what a page holds beyond a request's
// range never meets arithmetic.
#include "common.h"
#include "api.h"

#define AG_MAX_HEAD_DIM 512
#define AG_TILE 64                      // keys of a tile = lanes of a wave
#define AG_CHUNK 64                     // dimensions staged at a time
#define AG_PITCH 68                     // floats between staged rows: 16-byte aligned, no two of 16 lanes on a bank
#define AG_HEADS 4                      // query heads a wave takes together
#define AG_SEGMENT 512                  // keys of a segment
#define AG_SEG_TILES (AG_SEGMENT / AG_TILE)

__device__ __forceinline__ float4 ag_load4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 ag_load4(const bf16_t* p) {
    const uint2 v = *(const uint2*)p;
    return make_float4(bf16_bits_to_f32((uint16_t)v.x), bf16_bits_to_f32((uint16_t)(v.x >> 16)),
                       bf16_bits_to_f32((uint16_t)v.y), bf16_bits_to_f32((uint16_t)(v.y >> 16)));
}

// Totals (big_m, big_l, big_o) take in a segment (m, l, o): the one place where this is written down.
__device__ __forceinline__ void ag_merge_scales(float big_m, float m, float& m_out, float& a, float& b) {
    m_out = fmaxf(big_m, m);
    a = expf(big_m - m_out);
    b = expf(m - m_out);
}
// (written so that the compiler has no choice of which product to fuse: both forms must round alike)
__device__ __forceinline__ float ag_merge_value(float big, float a, float part, float b) { return fmaf(part, b, big * a); }

// VEC: the head size and the page size are multiples of four, so that four neighbouring dimensions of a key and
// four neighbouring keys of a value's dimension are fetched with one load.  HEADS: query heads of a group (1 to 4).
template <typename T, bool VEC, int HEADS, bool AHEAD>
__global__ __launch_bounds__(IA_WAVE) void attn_generic_kernel(
    T* __restrict__ out,                 // [n, nq, d]
    const T* __restrict__ q,             // [n, nq, d]
    const T* __restrict__ k_cache,       // [pages, nkv, page_size, d]
    const T* __restrict__ v_cache,       // [pages, nkv, d, page_size]  (transposed inside a page)
    const int* __restrict__ positions,   // [n]
    const int* __restrict__ token_seq,   // [n] row of block_table
    const int* __restrict__ block_table, // [seqs, max_pages]
    int max_pages, int nq, int nkv, int d, int page_size, int window, float scale,
    float* __restrict__ partial,         // null: a wave walks all segments; else [n, nq, segs, dpad + 2], a wave a segment
    int segs) {
    __shared__ __attribute__((aligned(16))) float stage[AG_TILE * AG_PITCH];     // keys: [key][dim]; values: [dim][key]
    __shared__ __attribute__((aligned(16))) float sp[HEADS][AG_TILE];
    extern __shared__ __attribute__((aligned(16))) float ag_rows[];       // queries, a segment's outputs, the totals: [HEADS][dpad] each
    const int lane = threadIdx.x;
    const int g = nq / nkv;
    const int groups = (g + HEADS - 1) / HEADS;
    const int unit = partial != nullptr ? blockIdx.x / segs : blockIdx.x;
    const int only_seg = partial != nullptr ? blockIdx.x - unit * segs : -1;
    const int tok = unit / (nkv * groups);
    const int rest = unit - tok * (nkv * groups);
    const int kvh = rest / groups;
    const int h0 = kvh * g + (rest - kvh * groups) * HEADS;            // first query head of the group
    const int heads = kvh * g + g - h0 < HEADS ? kvh * g + g - h0 : HEADS;
    const int pos = positions[tok];
    const int* bt = block_table + (size_t)token_seq[tok] * max_pages;
    const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
    const int chunks = (d + AG_CHUNK - 1) / AG_CHUNK;
    const int dpad = chunks * AG_CHUNK;
    float* const sq = ag_rows;
    float* const so = ag_rows + HEADS * dpad;
    float* const st_ = ag_rows + 2 * HEADS * dpad;

    // the queries, zeros beyond the head size and for heads the group does not have
    for (int h = 0; h < HEADS; ++h)
        for (int e = lane; e < dpad; e += IA_WAVE)
            sq[h * dpad + e] = (h < heads && e < d) ? ld(q + ((size_t)tok * nq + h0 + h) * d + e) : 0.f;

    const int seg_first = lo / AG_SEGMENT, seg_last = pos / AG_SEGMENT;
    if (only_seg >= 0 && (only_seg < seg_first || only_seg > seg_last)) return;       // (the whole wave)
    float big_m[HEADS], big_l[HEADS];
#pragma unroll
    for (int h = 0; h < HEADS; ++h) { big_m[h] = -INFINITY; big_l[h] = 0.f; }
    if (only_seg < 0)
        for (int h = 0; h < HEADS; ++h)
            for (int e = lane; e < dpad; e += IA_WAVE) st_[h * dpad + e] = 0.f;
    for (int seg = only_seg >= 0 ? only_seg : seg_first; seg <= (only_seg >= 0 ? only_seg : seg_last); ++seg) {
    // the segment's outputs so far: lane e owns dimensions e, e + 64, ... of every head (nobody else touches them)
    for (int h = 0; h < HEADS; ++h)
        for (int e = lane; e < dpad; e += IA_WAVE) so[h * dpad + e] = 0.f;
    float m[HEADS], l[HEADS];
#pragma unroll
    for (int h = 0; h < HEADS; ++h) { m[h] = -INFINITY; l[h] = 0.f; }
    const int tile_first = seg * AG_SEG_TILES > lo / AG_TILE ? seg * AG_SEG_TILES : lo / AG_TILE;
    const int tile_last = seg * AG_SEG_TILES + AG_SEG_TILES - 1 < pos / AG_TILE ? seg * AG_SEG_TILES + AG_SEG_TILES - 1 : pos / AG_TILE;

    // ---- the pieces of a tile's work (the same arithmetic in the same order whoever stages the operands) -----------
    float s[HEADS], alpha[HEADS];
    // scores: lane j against key j, chunk c of the dimensions from the stage
    auto scores = [&](int c) {
        const float* mine = stage + lane * AG_PITCH;
#pragma unroll 4
        for (int e4 = 0; e4 < AG_CHUNK / 4; ++e4) {
            const float4 kv = *(const float4*)(mine + e4 * 4);
#pragma unroll
            for (int h = 0; h < HEADS; ++h) {
                const float4 qv = *(const float4*)(sq + h * dpad + c * AG_CHUNK + e4 * 4);
                s[h] = fmaf(qv.x, kv.x, s[h]);
                s[h] = fmaf(qv.y, kv.y, s[h]);
                s[h] = fmaf(qv.z, kv.z, s[h]);
                s[h] = fmaf(qv.w, kv.w, s[h]);
            }
        }
    };
    // running maximum and sum; the tile's probabilities go to shared memory
    auto softmax = [&](bool valid) {
#pragma unroll
        for (int h = 0; h < HEADS; ++h) {
            const float sc = valid ? s[h] * scale : -INFINITY;
            const float m_new = fmaxf(m[h], wave_max(sc));
            const float p = valid ? expf(sc - m_new) : 0.f;
            alpha[h] = expf(m[h] - m_new);
            l[h] = l[h] * alpha[h] + wave_sum(p);
            sp[h][lane] = p;
            m[h] = m_new;
        }
    };
    // values: lane e adds up dimension c * 64 + e over the tile's keys from the stage
    auto values = [&](int c) {
        const float* mine = stage + lane * AG_PITCH;
        float o[HEADS];
#pragma unroll
        for (int h = 0; h < HEADS; ++h) o[h] = so[h * dpad + c * AG_CHUNK + lane] * alpha[h];
#pragma unroll 4
        for (int k4 = 0; k4 < AG_TILE / 4; ++k4) {
            const float4 vv = *(const float4*)(mine + k4 * 4);
#pragma unroll
            for (int h = 0; h < HEADS; ++h) {
                const float4 pv = *(const float4*)(&sp[h][k4 * 4]);
                o[h] = fmaf(pv.x, vv.x, o[h]);
                o[h] = fmaf(pv.y, vv.y, o[h]);
                o[h] = fmaf(pv.z, vv.z, o[h]);
                o[h] = fmaf(pv.w, vv.w, o[h]);
            }
        }
#pragma unroll
        for (int h = 0; h < HEADS; ++h) so[h * dpad + c * AG_CHUNK + lane] = o[h];
    };
    // key j's page of a tile, in lane j - j0: asked for once a tile, handed round
    auto tile_pages = [&](int tile) {
        const int j = tile * AG_TILE + lane;
        return (j >= lo && j <= pos) ? bt[j / page_size] : 0;
    };

    if constexpr (VEC && AHEAD) {
        // Steps of few tokens, a wave a segment.  A tile is 2 * chunks steps: the chunks of its keys, then the chunks of
        // its values.  A step's operands are asked for while the step before it is multiplied (a wave is alone in its
        // block and mostly alone on its SIMD: nobody else would hide the memory's latency), held in registers meanwhile
        // and put on the stage when it is free: a decode step of 8 requests at a context of 8,192 in 32-bit 220 -> 150 us
        // a layer.  (Steps of many tokens have waves enough on every SIMD, and the registers that hold a step's operands
        // would cost them a tenth of their speed.)
        constexpr int LOADS = AG_TILE / 4;
        static_assert(AG_TILE == AG_CHUNK, "a step of either kind is as many loads");
        const int steps = 2 * chunks;
        float4 held[LOADS];
        // keys: a load instruction takes four keys' rows of the chunk, 16 lanes a row, four dimensions a lane;
        // values: four dimensions, 16 lanes a dimension, four neighbouring keys a lane (four keys never straddle a page)
        auto ask = [&](int tile, int step, int pages) {
            const int j0 = tile * AG_TILE;
            if (step < chunks) {
                const int e = step * AG_CHUNK + (lane & 15) * 4;
#pragma unroll
                for (int i = 0; i < LOADS; ++i) {
                    const int r = 4 * i + (lane >> 4);
                    const int key = j0 + r;
                    const int page = __shfl(pages, r);
                    held[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (key >= lo && key <= pos && e < d)
                        held[i] = ag_load4(k_cache + (((size_t)page * nkv + kvh) * page_size + key % page_size) * d + e);
                }
            } else {
                const int c = step - chunks;
                const int k4 = (lane & 15) * 4;
                const int key = j0 + k4;
                const int off = key % page_size;
                const bool any = key + 3 >= lo && key <= pos;
                // the page of the four keys, from a lane whose key is in the range (a page that a window has passed is
                // not in the table any more; the keys of these four that are in the range share their page)
                const int first_in = key >= lo ? k4 : (lo - j0 < AG_TILE ? lo - j0 : k4);
                const int page = __shfl(pages, first_in);
#pragma unroll
                for (int i = 0; i < LOADS; ++i) {
                    const int e = c * AG_CHUNK + 4 * i + (lane >> 4);
                    held[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (any && e < d) held[i] = ag_load4(v_cache + (((size_t)page * nkv + kvh) * d + e) * page_size + off);
                }
            }
        };
        // what was asked for goes on the stage; values of keys outside the token's range as zeros
        auto put = [&](int tile, int step) {
            if (step < chunks) {
#pragma unroll
                for (int i = 0; i < LOADS; ++i)
                    *(float4*)(stage + (4 * i + (lane >> 4)) * AG_PITCH + (lane & 15) * 4) = held[i];
            } else {
                const int k4 = (lane & 15) * 4;
                const int key = tile * AG_TILE + k4;
                const bool in0 = key >= lo && key <= pos, in1 = key + 1 >= lo && key + 1 <= pos;
                const bool in2 = key + 2 >= lo && key + 2 <= pos, in3 = key + 3 >= lo && key + 3 <= pos;
#pragma unroll
                for (int i = 0; i < LOADS; ++i) {
                    float4 v = held[i];
                    v.x = in0 ? v.x : 0.f;
                    v.y = in1 ? v.y : 0.f;
                    v.z = in2 ? v.z : 0.f;
                    v.w = in3 ? v.w : 0.f;
                    *(float4*)(stage + (4 * i + (lane >> 4)) * AG_PITCH + k4) = v;
                }
            }
        };
        int pages = tile_pages(tile_first);
        if (tile_first <= tile_last) ask(tile_first, 0, pages);
        for (int tile = tile_first; tile <= tile_last; ++tile) {
            const int j = tile * AG_TILE + lane;
            const bool valid = j >= lo && j <= pos;
            const int pages_next = tile < tile_last ? tile_pages(tile + 1) : 0;
#pragma unroll
            for (int h = 0; h < HEADS; ++h) s[h] = 0.f;
            for (int step = 0; step < steps; ++step) {
                if (step == chunks) softmax(valid);
                __syncthreads();                                      // the stage is free (and the probabilities are there)
                put(tile, step);
                if (step + 1 < steps) ask(tile, step + 1, pages);
                else if (tile < tile_last) ask(tile + 1, 0, pages_next);
                __syncthreads();
                if (step < chunks) scores(step);
                else values(step - chunks);
            }
            pages = pages_next;
        }
    } else {
    for (int tile = tile_first; tile <= tile_last; ++tile) {
        const int j0 = tile * AG_TILE;
        const int j = j0 + lane;
        const bool valid = j >= lo && j <= pos;
        const int my_page = tile_pages(tile);
#pragma unroll
        for (int h = 0; h < HEADS; ++h) s[h] = 0.f;
        for (int c = 0; c < chunks; ++c) {
            __syncthreads();                                          // the stage is free
            if constexpr (VEC) {
                // a load instruction takes four keys' rows of this chunk: 16 lanes a row, four dimensions a lane
                const int e = c * AG_CHUNK + (lane & 15) * 4;
                float4 v[AG_TILE / 4];
#pragma unroll
                for (int i = 0; i < AG_TILE / 4; ++i) {
                    const int r = 4 * i + (lane >> 4);
                    const int key = j0 + r;
                    const int page = __shfl(my_page, r);
                    v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (key >= lo && key <= pos && e < d)
                        v[i] = ag_load4(k_cache + (((size_t)page * nkv + kvh) * page_size + key % page_size) * d + e);
                }
#pragma unroll
                for (int i = 0; i < AG_TILE / 4; ++i)
                    *(float4*)(stage + (4 * i + (lane >> 4)) * AG_PITCH + (lane & 15) * 4) = v[i];
            } else {
                for (int r = 0; r < AG_TILE; ++r) {
                    const int key = j0 + r, e = c * AG_CHUNK + lane;
                    float v = 0.f;
                    const int page = __shfl(my_page, r);
                    if (key >= lo && key <= pos && e < d)
                        v = ld(k_cache + (((size_t)page * nkv + kvh) * page_size + key % page_size) * d + e);
                    stage[r * AG_PITCH + lane] = v;
                }
            }
            __syncthreads();
            scores(c);
        }
        softmax(valid);
        for (int c = 0; c < chunks; ++c) {
            __syncthreads();                                          // the stage is free, the probabilities are there
            if constexpr (VEC) {
                // a load instruction takes four dimensions: 16 lanes a dimension, four neighbouring keys a lane
                const int k4 = (lane & 15) * 4;
                const int key = j0 + k4;
                const int off = key % page_size;                      // (four keys never straddle a page)
                const bool any = key + 3 >= lo && key <= pos;
                // the page of the four keys, from a lane whose key is in the range (a page that a window has passed is
                // not in the table any more; the keys of these four that are in the range share their page)
                const int first_in = key >= lo ? k4 : (lo - j0 < AG_TILE ? lo - j0 : k4);
                const int page = __shfl(my_page, first_in);
                float4 v[AG_CHUNK / 4];
#pragma unroll
                for (int i = 0; i < AG_CHUNK / 4; ++i) {
                    const int e = c * AG_CHUNK + 4 * i + (lane >> 4);
                    v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (any && e < d) {
                        v[i] = ag_load4(v_cache + (((size_t)page * nkv + kvh) * d + e) * page_size + off);
                        v[i].x = (key >= lo && key <= pos) ? v[i].x : 0.f;
                        v[i].y = (key + 1 >= lo && key + 1 <= pos) ? v[i].y : 0.f;
                        v[i].z = (key + 2 >= lo && key + 2 <= pos) ? v[i].z : 0.f;
                        v[i].w = (key + 3 >= lo && key + 3 <= pos) ? v[i].w : 0.f;
                    }
                }
#pragma unroll
                for (int i = 0; i < AG_CHUNK / 4; ++i)
                    *(float4*)(stage + (4 * i + (lane >> 4)) * AG_PITCH + k4) = v[i];
            } else {
                const int off = j % page_size;
                for (int r = 0; r < AG_CHUNK; ++r) {
                    const int e = c * AG_CHUNK + r;
                    stage[r * AG_PITCH + lane] =
                        (valid && e < d) ? ld(v_cache + (((size_t)my_page * nkv + kvh) * d + e) * page_size + off) : 0.f;
                }
            }
            __syncthreads();
            values(c);
        }
    }
    }
    // ---- the segment is done ---------------------------------------------------------------------------------------
    if (only_seg >= 0) {
#pragma unroll
        for (int h = 0; h < HEADS; ++h) {
            if (h >= heads) break;
            float* row = partial + (((size_t)tok * nq + h0 + h) * segs + seg) * (dpad + 2);
            for (int e = lane; e < dpad; e += IA_WAVE) row[e] = so[h * dpad + e];
            if (lane == 0) { row[dpad] = m[h]; row[dpad + 1] = l[h]; }
        }
        return;
    }
#pragma unroll
    for (int h = 0; h < HEADS; ++h) {
        float m_out, a, b;
        ag_merge_scales(big_m[h], m[h], m_out, a, b);
        big_l[h] = ag_merge_value(big_l[h], a, l[h], b);
        big_m[h] = m_out;
        for (int e = lane; e < dpad; e += IA_WAVE)
            st_[h * dpad + e] = ag_merge_value(st_[h * dpad + e], a, so[h * dpad + e], b);
    }
    }
#pragma unroll
    for (int h = 0; h < HEADS; ++h) {
        if (h >= heads) break;
        T* orow = out + ((size_t)tok * nq + h0 + h) * d;
        const float inv = 1.0f / big_l[h];
        for (int e = lane; e < d; e += IA_WAVE) st(orow + e, st_[h * dpad + e] * inv);
    }
}

// The segments of a (token, query head) that waves of their own have left in `partial`, merged in ascending order.
template <typename T>
__global__ __launch_bounds__(IA_WAVE) void attn_generic_merge_kernel(
    T* __restrict__ out, const float* __restrict__ partial, const int* __restrict__ positions, int nq, int d, int dpad,
    int window, int segs) {
    const int lane = threadIdx.x;
    const int tok = blockIdx.x / nq, h = blockIdx.x - tok * nq;
    const int pos = positions[tok];
    const int lo = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
    float big_m = -INFINITY, big_l = 0.f;
    float big_o[AG_MAX_HEAD_DIM / IA_WAVE];
#pragma unroll
    for (int t = 0; t < AG_MAX_HEAD_DIM / IA_WAVE; ++t) big_o[t] = 0.f;
    // (a position beyond the caller's bound has segments that nobody wrote: they are left out rather than read)
    const int seg_last = pos / AG_SEGMENT < segs - 1 ? pos / AG_SEGMENT : segs - 1;
    for (int seg = lo / AG_SEGMENT; seg <= seg_last; ++seg) {
        const float* row = partial + (((size_t)tok * nq + h) * segs + seg) * (dpad + 2);
        float m_out, a, b;
        ag_merge_scales(big_m, row[dpad], m_out, a, b);
        big_l = ag_merge_value(big_l, a, row[dpad + 1], b);
        big_m = m_out;
#pragma unroll
        for (int t = 0; t < AG_MAX_HEAD_DIM / IA_WAVE; ++t) {
            const int e = lane + t * IA_WAVE;
            if (e < dpad) big_o[t] = ag_merge_value(big_o[t], a, row[e], b);
        }
    }
    const float inv = 1.0f / big_l;
    T* orow = out + ((size_t)tok * nq + h) * d;
#pragma unroll
    for (int t = 0; t < AG_MAX_HEAD_DIM / IA_WAVE; ++t) {
        const int e = lane + t * IA_WAVE;
        if (e < d) st(orow + e, big_o[t] * inv);
    }
}

// Floats of the workspace that steps of few tokens need (0: the step has tokens enough for a wave each to walk
// all its segments).  `max_kv_len`: an upper bound of the positions + 1.
extern "C" long long ia_attention_generic_workspace(int n, int nq, int nkv, int d, int max_kv_len) {
    if (n <= 0 || nq <= 0 || nkv <= 0 || d <= 0 || max_kv_len <= AG_SEGMENT) return 0;
    const int g = nq / nkv;
    const int per_group = g < AG_HEADS ? g : AG_HEADS;
    const long long units = (long long)n * nkv * ((g + per_group - 1) / per_group);
    if (units >= 2048) return 0;
    const int segs = (max_kv_len + AG_SEGMENT - 1) / AG_SEGMENT;
    const int dpad = (d + AG_CHUNK - 1) / AG_CHUNK * AG_CHUNK;
    return (long long)n * nq * segs * (dpad + 2);
}

extern "C" int ia_attention_generic(void* out, const void* q, const void* k_cache, const void* v_cache,
                                    const int* positions, const int* token_seq, const int* block_table,
                                    int n, int max_pages, int nq, int nkv, int d, int page_size,
                                    int window, float scale, int dtype, float* workspace, int max_kv_len,
                                    hipStream_t stream) {
    IA_CHECK(n >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention: bad head counts nq=%d nkv=%d (n=%d)", nq, nkv, n);
    IA_CHECK(d > 0 && d <= AG_MAX_HEAD_DIM, "attention: head_dim %d is outside 1..%d", d, AG_MAX_HEAD_DIM);
    IA_CHECK(page_size > 0 && max_pages > 0, "attention: bad page geometry page_size=%d max_pages=%d", page_size, max_pages);
    IA_CHECK(window >= 0, "attention: window %d must be >= 0 (0 = all keys)", window);
    if (n == 0) return 0;
    const int g = nq / nkv;
    const int per_group = g < AG_HEADS ? g : AG_HEADS;                 // query heads a wave takes together
    const int groups = (g + per_group - 1) / per_group;
    IA_CHECK((long long)n * nkv * groups < 2147483647LL, "attention: %d tokens x %d heads exceed the grid", n, nq);
    // a wave a segment when the workspace is given (ia_attention_generic_workspace says when it is needed)
    const int segs = workspace != nullptr ? (max_kv_len + AG_SEGMENT - 1) / AG_SEGMENT : 1;
    IA_CHECK(workspace == nullptr || (max_kv_len > 0 && ia_attention_generic_workspace(n, nq, nkv, d, max_kv_len) > 0),
             "attention: a workspace goes with max_kv_len and a step of few tokens");
    IA_CHECK((long long)n * nkv * groups * segs < 2147483647LL, "attention: %d tokens x %d heads exceed the grid", n, nq);
    const unsigned grid = (unsigned)n * (unsigned)nkv * (unsigned)groups * (unsigned)segs;
    const int dpad = (d + AG_CHUNK - 1) / AG_CHUNK * AG_CHUNK;
    const size_t rows_bytes = (size_t)3 * per_group * ((d + AG_CHUNK - 1) / AG_CHUNK * AG_CHUNK) * sizeof(float);
    const size_t elem = dtype == IA_F32 ? 4 : 2;
    // loads of four elements: rows of the caches start at multiples of four elements, on aligned arrays
    const bool vec = d % 4 == 0 && page_size % 4 == 0 &&
                     (((uintptr_t)k_cache | (uintptr_t)v_cache) % (4 * elem)) == 0;
#define AG_ARGS(T) (T*)out, (const T*)q, (const T*)k_cache, (const T*)v_cache, positions, token_seq, block_table, max_pages, nq, nkv, \
        d, page_size, window, scale, workspace, segs
    // (a wave a segment, steps of few tokens: the operands are asked for a step ahead)
#define AG_LAUNCH(T, V, H) do { \
        if (V && workspace != nullptr) attn_generic_kernel<T, V, H, true><<<grid, IA_WAVE, rows_bytes, stream>>>(AG_ARGS(T)); \
        else attn_generic_kernel<T, V, H, false><<<grid, IA_WAVE, rows_bytes, stream>>>(AG_ARGS(T)); } while (0)
#define AG_HEADS_OF(T, V) do { \
        if (per_group == 1) AG_LAUNCH(T, V, 1); else if (per_group == 2) AG_LAUNCH(T, V, 2); \
        else if (per_group == 3) AG_LAUNCH(T, V, 3); else AG_LAUNCH(T, V, 4); } while (0)
    if (dtype == IA_F32) { if (vec) AG_HEADS_OF(float, true); else AG_HEADS_OF(float, false); }
    else if (dtype == IA_BF16) { if (vec) AG_HEADS_OF(bf16_t, true); else AG_HEADS_OF(bf16_t, false); }
    else IA_CHECK(false, "attention: unknown dtype %d", dtype);
#undef AG_HEADS_OF
#undef AG_LAUNCH
#undef AG_ARGS
    IA_LAUNCH_CHECK("attention_generic");
    if (workspace != nullptr) {
        if (dtype == IA_F32)
            attn_generic_merge_kernel<float><<<(unsigned)n * nq, IA_WAVE, 0, stream>>>((float*)out, workspace, positions, nq, d, dpad, window, segs);
        else
            attn_generic_merge_kernel<bf16_t><<<(unsigned)n * nq, IA_WAVE, 0, stream>>>((bf16_t*)out, workspace, positions, nq, d, dpad, window, segs);
        IA_LAUNCH_CHECK("attention_generic_merge");
    }
    return 0;
}
