// Paged grouped-query attention on the matrix cores, bfloat16, for one head size per build
// (IA_HEAD_DIM, a multiple of 16 up to 256).  One kernel serves prefill and decode: a wave
// owns up to 16 * NB columns, a column being one (query token, query head) pair of one
// request and one key/value head, and walks that request's keys 32 at a time straight from
// the cache pages into MFMA operands.  Where a step has few columns and long key ranges, the
// keys are split between waves and the partial results are merged by a second kernel.  Decode
// steps (one token a request) at head sizes in steps of 64 have a kernel of their own with the
// per-head norm, the rotation, the cache write and that merge inside (attn_decode_kernel).  At
// head size 128, steps with 128 columns or more of a request (portions of prompts) go to blocks
// of four waves that share keys and values through shared memory (attn_tile_kernel).
//
// Formula as in the reference: S = (q . k) * scale after the product, keys j <= position
// (inferrs-models/src/models/attention_utils.rs:61-85), softmax over keys, O = P v
// (inferrs-models/src/models/qwen3.rs:166-192); query head h reads key/value head
// h / (nq / nkv) (attention_utils.rs:38-49).  Scores, the running maximum and sum, and the
// output accumulators are 32-bit; probabilities are rounded to bfloat16 for the second product.
//
// Everything is computed transposed so that no operand needs a transpose in flight:
//   S^T[key][col] = K[key][:] . Q[col][:]      A = 16 keys x 32 dims (rows of the K page),
//                                              B = 32 dims x 16 columns (rows of Q)
//   O^T[dim][col] = V^T[dim][:] . P^T[:][col]  A = 16 dims x 32 keys (rows of the V^T page),
//                                              B = 32 keys x 16 columns (the S^T accumulators)
// The cache keeps keys as [page][kv head][slot][dim] and values transposed, as
// [page][kv head][dim][slot], so both A operands are 16-byte pieces of contiguous rows.
// v_mfma_f32_16x16x32_bf16: lane l supplies row l%16 of A and column l%16 of B with the eight
// k values 8*(l/16)..+8, and receives D[4*(l/16)+i][l%16], i = 0..3.  The two S^T tiles of a
// 32-key step assign key k0 + 8G + 4t + i to row 4G+i of tile t, so that lane (col, G) ends
// up holding the probabilities of keys k0+8G .. k0+8G+7 in order: exactly the B operand of the
// second product.
#include <type_traits>

#include "common.h"
#include "api.h"

#ifndef IA_HEAD_DIM
#error "compile with -DIA_HEAD_DIM=<multiple of 16 up to 256>"
#endif
static_assert(IA_HEAD_DIM % 16 == 0 && IA_HEAD_DIM >= 16 && IA_HEAD_DIM <= 256, "head size");

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define HD IA_HEAD_DIM
#define DB (HD / 16)            // 16-dim blocks of the output
#define KS ((HD + 31) / 32)     // 32-dim steps of the first product

struct AttnParams {
    bf16_t* out;                // [n, nq, d]
    float* part_o;              // [n, nq, splits, d]   when splits > 1
    float* part_ml;             // [n, nq, splits, 2]   running maximum (log2 domain) and sum
    const bf16_t* q;            // [n, nq, d]
    const bf16_t* k_cache;      // [pages, nkv, page, d]
    const bf16_t* v_cache;      // [pages, nkv, d, page]
    bf16_t* k_cache_w;          // the same arrays for the fused form's writes
    bf16_t* v_cache_w;
    const int* block_table;     // [seqs, max_pages]
    const int* cu_tokens;       // [seqs + 1]  request s owns tokens cu[s]..cu[s+1]
    const int* positions;       // [n]         absolute position of each token
    int max_pages, nq, nkv, page, window, splits, chunk, pair, seq_begin;   // pair: see the kernels
    int token_begin;            // decode kernel: request seq_begin + i owns token token_begin + i
    float scale_log2;           // scale * log2(e)
    // The decode kernel, with the per-head norm, the rotation and the cache write inside: q is not
    // read from `q` but formed from the projections' output, and the wave that walks a request's
    // newest key forms that key and value, uses them and writes them to the cache.
    const bf16_t* qkv;          // [n, (nq + 2 nkv) * d]: q heads, then k heads, then v heads
    const float* q_norm_w;      // [d], or null: no norm
    const float* k_norm_w;
    const float* cos_t;         // [n, d / 2], or null: no rotation
    const float* sin_t;
    const int* slots;           // [n] cache slot of each token, or null: this layer writes no cache
    float norm_eps;
    int norm_add_one;
};

__device__ __forceinline__ uint4 zero4() { return make_uint4(0, 0, 0, 0); }

// One column block (16 * NB columns) of one request and key/value head, over one split of the keys.
template <int NB>
__device__ __forceinline__ void attn_column_block(const AttnParams& p, int cb, int kvh, int split, int seq) {
    const int lane = threadIdx.x;
    const int r = lane & 15, G = lane >> 4;
    const int g = p.nq / p.nkv;
    const int t0 = p.cu_tokens[seq], q_len = p.cu_tokens[seq + 1] - t0;
    const int n_cols = q_len * g;
    const int col0 = cb * 16 * NB;
    if (col0 >= n_cols) return;
    const int kv_start = p.positions[t0];
    const int kv_total = kv_start + q_len;
    const int* bt = p.block_table + (size_t)seq * p.max_pages;

    // this lane's columns
    int tq[NB], head[NB], pos[NB];
    bool cvalid[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int c = col0 + nb * 16 + r;
        cvalid[nb] = c < n_cols;
        const int cc = cvalid[nb] ? c : n_cols - 1;
        tq[nb] = cc / g;
        head[nb] = kvh * g + (cc - tq[nb] * g);
        pos[nb] = kv_start + tq[nb];
    }
    const int last_col = (col0 + 16 * NB <= n_cols ? col0 + 16 * NB : n_cols) - 1;
    const int pmin = kv_start + col0 / g, pmax = kv_start + last_col / g;

    // Q^T operands stay in registers for the whole walk.
    uint4 qreg[NB][KS];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const bf16_t* qrow = p.q + ((size_t)(t0 + tq[nb]) * p.nq + head[nb]) * HD;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int dim = ks * 32 + G * 8;
            qreg[nb][ks] = (cvalid[nb] && dim < HD) ? *(const uint4*)(qrow + dim) : zero4();
        }
    }

    f32x4 acc[NB][DB];
    float m[NB], l[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        m[nb] = -INFINITY;
        l[nb] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[nb][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }

    const int window_floor = p.window > 0 ? (pmin - p.window + 1 > 0 ? pmin - p.window + 1 : 0) : 0;   // first key any column sees
    int lo = window_floor;
    int hi = pmax + 1;
    if (p.splits > 1) {
        const int c_lo = split * p.chunk, c_hi = c_lo + p.chunk;
        lo = lo > c_lo ? lo : c_lo;
        hi = hi < c_hi ? hi : c_hi;
    }
    lo &= ~31;

    // ---- operands of a step: 32 keys = two 16-slot halves, each inside one page --------------
    struct Operands {
        uint4 k[2][KS];         // tile t, dim step ks: row r <-> key k0 + 8*(r/4) + 4t + r%4
        uint4 v[DB];            // dim block db: row r <-> dim 16 db + r, keys k0 + 8G .. +7
    };
    // A step's 32 keys are two groups of 16 slots, each inside one page (page sizes are multiples of
    // 16): a Place says where a group lies, and moves on without a division.
    struct Place { int idx, off; };                  // page index in the block table, slot in that page
    auto advance = [&](Place& at, int slots) {
        at.off += slots;
        while (at.off >= p.page) { at.off -= p.page; ++at.idx; }
    };
    // This lane's part of the addresses does not change from step to step: its key rows' slots inside
    // their group, its piece of a row, and which of the two groups they belong to.
    const bool k_second = r >= 8, v_second = G >= 2;
    const uint32_t k_lane[2] = {(uint32_t)((((8 * (r >> 2) + (r & 3)) & 15) * HD + G * 8) * 2),
                                (uint32_t)((((8 * (r >> 2) + 4 + (r & 3)) & 15) * HD + G * 8) * 2)};
    const uint32_t v_lane = (uint32_t)((r * p.page + 8 * (G & 1)) * 2);
    const size_t v_stride = (size_t)16 * p.page * 2;
    auto load_step = [&](Operands& op, int k0, const Place& at) {
        if (k0 + 32 <= kv_total) {
            // every slot of the step is written: the pages' numbers and the groups' places are the same
            // for all lanes (they come through the scalar cache), a lane adds its constant part
            Place next = at;
            advance(next, 16);
            const int page_a = bt[at.idx], page_b = bt[next.idx];
            const char* ka = (const char*)(p.k_cache + (((size_t)page_a * p.nkv + kvh) * p.page + at.off) * HD);
            const char* kb = (const char*)(p.k_cache + (((size_t)page_b * p.nkv + kvh) * p.page + next.off) * HD);
            const char* va = (const char*)(p.v_cache + ((size_t)page_a * p.nkv + kvh) * HD * p.page + at.off);
            const char* vb = (const char*)(p.v_cache + ((size_t)page_b * p.nkv + kvh) * HD * p.page + next.off);
            const char* kbase = k_second ? kb : ka;
            const char* vbase = (v_second ? vb : va) + v_lane;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    op.k[t][ks] = (ks * 32 + G * 8 < HD) ? *(const uint4*)(kbase + k_lane[t] + ks * 64) : zero4();
#pragma unroll
            for (int db = 0; db < DB; ++db) op.v[db] = *(const uint4*)(vbase + db * v_stride);
            return;
        }
        // The request's last step.  Rows past its length are read from its last written slot instead
        // (their scores are masked in the step): the pages behind them may not exist.
        const int last_idx = (kv_total - 1) / p.page;
        const int idx_a = k0 / p.page;
        const int idx_b = (k0 + 16) / p.page < last_idx ? (k0 + 16) / p.page : last_idx;
        const int page_a = bt[idx_a], page_b = bt[idx_b];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            int key = k0 + 8 * (r >> 2) + 4 * t + (r & 3);
            key = key < kv_total ? key : kv_total - 1;
            const int kpage = key / p.page == idx_a ? page_a : page_b;
            const bf16_t* krow = p.k_cache + (((size_t)kpage * p.nkv + kvh) * p.page + key % p.page) * HD + G * 8;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                op.k[t][ks] = (ks * 32 + G * 8 < HD) ? *(const uint4*)(krow + ks * 32) : zero4();
        }
        int vkey = k0 + 8 * G;
        vkey = vkey < kv_total ? vkey : (kv_total - 1) & ~7;
        const int vpage = vkey / p.page == idx_a ? page_a : page_b;
        const bf16_t* vbase = p.v_cache + (((size_t)vpage * p.nkv + kvh) * HD + r) * p.page + vkey % p.page;
#pragma unroll
        for (int db = 0; db < DB; ++db) op.v[db] = *(const uint4*)(vbase + (size_t)db * 16 * p.page);
    };
    auto compute_step = [&](Operands& op, int k0) {
        const bool edge = k0 + 31 > pmin || (p.window > 0 && k0 < pmax - p.window + 1);
        if (k0 + 32 > kv_total) {
            // slots beyond the request's length hold anything at all: zero those values so that
            // a probability of zero times their content stays zero
            const int first_bad = kv_total - (k0 + 8 * G);          // keys >= this index are unwritten
            if (first_bad < 8) {
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    uint32_t w[4] = {op.v[db].x, op.v[db].y, op.v[db].z, op.v[db].w};
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (j >= first_bad) w[j >> 1] &= (j & 1) ? 0x0000ffffu : 0xffff0000u;
                    op.v[db] = make_uint4(w[0], w[1], w[2], w[3]);
                }
            }
        }
        if (p.window > 0 && k0 < window_floor) {
            // The walk starts at a multiple of 32 below the first key that any column sees: the keys in between
            // may lie in pages that the window has passed and the request has given back (the block table then
            // names some other page, which holds anything at all).  Their scores are masked below; their values
            // are zeroed here, for the same reason as the slots beyond the length.
            const int first_good = window_floor - (k0 + 8 * G);     // keys below this index are outside every window
            if (first_good > 0) {
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    uint32_t w[4] = {op.v[db].x, op.v[db].y, op.v[db].z, op.v[db].w};
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (j < first_good) w[j >> 1] &= (j & 1) ? 0x0000ffffu : 0xffff0000u;
                    op.v[db] = make_uint4(w[0], w[1], w[2], w[3]);
                }
            }
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            // ---- S^T for 32 keys x 16 columns ----------------------------------------------
            f32x4 s[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                s[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, op.k[t][ks]), __builtin_bit_cast(bf16x8, qreg[nb][ks]), s[t], 0, 0, 0);
            }
            // raw scores; the scale (> 0) and the change to base 2 are folded into the exponent below
            float sc[8];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) sc[4 * t + i] = s[t][i];
            if (edge) {
                const int kbase_idx = k0 + 8 * G;
                const int floor_key = p.window > 0 ? pos[nb] - p.window + 1 : 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int key = kbase_idx + j;
                    if (key > pos[nb] || key < floor_key) sc[j] = -INFINITY;
                }
            }
            float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mx = fmaxf(mx, __shfl_xor(mx, 16, IA_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, IA_WAVE));
            const float m_new = fmaxf(m[nb], mx * p.scale_log2);        // running maximum of scale * log2(e) * score
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m[nb] - m_use);  // m = -inf gives 0
            float pr[8], psum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[j], p.scale_log2, -m_use));
                psum += pr[j];
            }
            l[nb] = l[nb] * alpha + psum;
            m[nb] = m_new;
            uint4 pb;
            pb.x = pack_bf16x2(pr[0], pr[1]);
            pb.y = pack_bf16x2(pr[2], pr[3]);
            pb.z = pack_bf16x2(pr[4], pr[5]);
            pb.w = pack_bf16x2(pr[6], pr[7]);
            // ---- O^T += V^T . P^T ----------------------------------------------------------
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    acc[nb][db][0] *= alpha; acc[nb][db][1] *= alpha;
                    acc[nb][db][2] *= alpha; acc[nb][db][3] *= alpha;
                }
            }
#pragma unroll
            for (int db = 0; db < DB; ++db)
                acc[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8, op.v[db]), __builtin_bit_cast(bf16x8, pb), acc[nb][db], 0, 0, 0);
        }
    };

    // What bounds the walk of a long prompt, and what was tried (each variant measured against this
    // one in the same run; prompts of 2,048 and 8,192 tokens, head size 128).  At 8,192 tokens a layer's
    // waves ask the L2 for 121 M lines (15 GB, 12 TB/s) and the matrix pipes are busy 18 % of the time;
    // with 16 columns a wave instead of 32 (twice the reads, the same arithmetic) the walk takes 1.9
    // times as long: it is the L2's bandwidth.
    // - Blocks of four waves that bring keys and values into shared memory once, through registers and
    //   in the cache's own layout (stages of 64 keys, the next stage on its way in registers, one barrier
    //   a stage), halved the L2's requests and were still 3 % slower: a third of the shared memory's busy
    //   cycles were bank conflicts, and the registers of the stage on its way cost occupancy.  With loads
    //   straight into shared memory and a swizzled layout it pays: attn_tile_kernel below, which takes the
    //   prompt portions of head size 128 from this kernel.
    // - Loading the next step's operands ahead of this step's products doubles the operand registers,
    //   which costs a wave per SIMD, and that wave hid more latency.  Asking for the next keys right
    //   after the scores and for the next values right after the second product (no register held
    //   twice): prompts 5 % slower.
    // - Moving the exponents' reference point only when the running maximum has risen by 2^8 (the
    //   accumulators are then rescaled a few times a walk, not at most steps), row maxima through
    //   v_permlane swaps instead of shared memory, late and early column blocks as separate waves
    //   instead of one after the other in a wave: within 1 % each.
    // - Addresses without a division in the step (above): 1 % at 2,048 tokens.
    Place at = {lo / p.page, lo % p.page};
    for (int k0 = lo; k0 < hi; k0 += 32) {
        Operands op;
        load_step(op, k0, at);
        compute_step(op, k0);
        advance(at, 32);
    }

    // ---- results: lane (col, G) holds dims 16 db + 4 G + i of its column ---------------------
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        float lt = l[nb];
        lt += __shfl_xor(lt, 16, IA_WAVE);
        lt += __shfl_xor(lt, 32, IA_WAVE);
        if (!cvalid[nb]) continue;
        const size_t row = (size_t)(t0 + tq[nb]) * p.nq + head[nb];
        if (p.splits == 1) {
            const float inv = 1.0f / lt;
            bf16_t* o = p.out + row * HD + 4 * G;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                uint2 w;
                w.x = pack_bf16x2(acc[nb][db][0] * inv, acc[nb][db][1] * inv);
                w.y = pack_bf16x2(acc[nb][db][2] * inv, acc[nb][db][3] * inv);
                *(uint2*)(o + 16 * db) = w;
            }
        } else {
            float* o = p.part_o + (row * p.splits + split) * HD + 4 * G;
#pragma unroll
            for (int db = 0; db < DB; ++db) *(f32x4*)(o + 16 * db) = acc[nb][db];
            if (G == 0) {
                float* ml = p.part_ml + (row * p.splits + split) * 2;
                ml[0] = m[nb];
                ml[1] = lt;
            }
        }
    }
}

// With `pair` a wave takes column block i from the end of its request and then block i from the
// start: under a causal mask the late blocks walk many keys and the early ones few, and every
// pair walks about the same number, so all waves end together.  It pays when the step's queries
// span most of the context; a short portion late in a long context has equal blocks already.
template <int NB>
__global__ __launch_bounds__(IA_WAVE) __attribute__((amdgpu_waves_per_eu(HD <= 128 ? 2 : 1, HD > 64 ? 2 : 8)))
void attn_mfma_kernel(const AttnParams p) {
    const int kvh = blockIdx.y / p.splits, split = blockIdx.y - kvh * p.splits;
    const int seq = p.seq_begin + blockIdx.z;
    const int n_cols = (p.cu_tokens[seq + 1] - p.cu_tokens[seq]) * (p.nq / p.nkv);
    const int n_blocks = (n_cols + 16 * NB - 1) / (16 * NB);
    if (!p.pair) {
        // heavy column blocks first
        if ((int)blockIdx.x < n_blocks) attn_column_block<NB>(p, n_blocks - 1 - (int)blockIdx.x, kvh, split, seq);
        return;
    }
    const int late = n_blocks - 1 - (int)blockIdx.x, early = (int)blockIdx.x;
    if (late < early) return;
    attn_column_block<NB>(p, late, kvh, split, seq);
    if (early != late) attn_column_block<NB>(p, early, kvh, split, seq);
}

// The maximum / the sum over the four lanes that hold a column's values (lanes l, l ^ 16, l ^ 32, l ^ 48), in all
// of them, by swaps between rows of 16 lanes and between the halves of the wave: no trip through shared memory.
__device__ __forceinline__ float column_max(float x) {
    const uint32_t u = __float_as_uint(x);
    auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const uint32_t w = __float_as_uint(x);
    auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float column_sum(float x) {
    const uint32_t u = __float_as_uint(x);
    auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const uint32_t w = __float_as_uint(x);
    auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// ---- decode steps: one token a request, with the norm, the rotation, the cache write and the merge inside ------
// A wave owns up to 16 query heads of one request and key/value head and one split of that request's keys, as
// in the kernel above, but a decode step is short and every microsecond of it is latency, so the walk is laid
// out for that:
//  * the first step's keys and values are asked for before anything else: the query row is normed and rotated,
//    and the request's new key and value are formed and written to the cache, while they are on their way;
//  * a step's operands are asked for one step ahead (two sets of registers: a decode wave holds 16 columns and
//    has the room), so a wave waits for the memory once, not once a step;
//  * the waves of a block (`team`: 1, 2 or 4 neighbouring splits) add their results up in shared memory and
//    leave one partial result a block; the block that finishes last for its (request, key/value head), known by
//    a counter in memory, merges the blocks' partial results and writes the output.  No second kernel, and no
//    wave reads another compute unit's results before they are there: every wave waits until the memory has taken
//    its stores (`s_waitcnt vmcnt(0)`) before the barrier that precedes the block's one atomic increment, and the
//    last block reads past the caches after it has seen the full count.  The counters are zero
//    between calls (the last block puts its counter back), so calls that share them must not overlap.
// The sum over the splits runs in the order of the splits whoever comes last: the result is the same every time.
// Measured (head size 128, 32 query and 8 key/value heads, context 8,192, time stamps inside the kernel): a wave
// knows its token's position 0.8 us after it starts, has asked for the rows and the first keys at 2.5, has its rows
// formed at 4.6 and its two steps done at 6.6 (batch 1, 64 keys a wave); the block's waves have met at 7.0, the
// partial result is out at 7.5, the count back at 9.3 and the last block has merged at 13 to 16 us.  A fence of
// device scope in place of the write-through stores cost 100 us a layer at batch 8 (it writes back and empties
// the whole L2 of the die, once a block).  The kernel needs a SIMD's whole register file for a wave (two sets of
// operands, and more in the rows' forming), so a compute unit holds one block: the step's split keeps its waves
// within one round of the chip.  Against the kernel above with a merge kernel behind it, a layer, each at its
// best split: batch 8 52.4 against 56.5 us, batch 3 26.0 against 29.0, batch 16 98.8 against 103, batch 32 189
// against 195, batch 64 358 against 366; batch 8 at a context of 2,048 20.9 against 24.4, batch 64 at 1,024 49.0
// against 56.7; batch 1 17 to 18 us both ways.
// Partial results that blocks on other compute units read within the same kernel: written through to memory and
// read past the caches that are not coherent between the chip's dies (32-bit accesses of device scope, no order
// of their own), so that no cache has to be written back or emptied as a whole.
__device__ __forceinline__ void put_across(float* at, float v) {
    __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float get_across(const float* at) {
    return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct DecodeOperands {
    uint4 k[2][KS];             // as Operands above
    uint4 v[DB];
};

template <bool ENABLED = (HD % 64 == 0)>
__global__ __launch_bounds__(4 * IA_WAVE) void attn_decode_kernel(const AttnParams p, int* counters, int team) {
    if constexpr (ENABLED) {
        extern __shared__ __align__(16) float team_mem[];       // [team][columns][HD] partial outputs, then [team][columns][2]
        __shared__ int s_last;
        // (the wave's number through a scalar register: what follows from it, the split's range and the pages' numbers,
        // is then the same for all lanes by construction, and the block table is read through the scalar cache)
        const int lane = threadIdx.x & (IA_WAVE - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / IA_WAVE);
        const int r = lane & 15, G = lane >> 4;
        const int g = p.nq / p.nkv;
        const int teams = p.splits / team;
        const int kvh = blockIdx.y / teams, tm = blockIdx.y - kvh * teams;
        const int split = tm * team + wave;
        const int seq = p.seq_begin + blockIdx.z;
        const int col0 = blockIdx.x * 16;
        const int n_cols = g - col0 < 16 ? g - col0 : 16;       // this block's columns (the grid has no empty block)
        // What a wave needs before it can ask for its first keys is a chain of small reads, each a trip to the
        // memory: the token's position, then the pages' numbers.  A decode step's token is known without a read
        // (request seq_begin + i owns token token_begin + i), and where no window moves the walk's start the first
        // two steps' pages are read from the block table at the same time as the position (entries past the
        // request's last page are read but not used).
        const int t0 = p.token_begin + (int)blockIdx.z;
        const int* bt = p.block_table + (size_t)seq * p.max_pages;
        const int c_lo = p.splits > 1 ? split * p.chunk : 0;
        int early[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = (c_lo + 16 * i) / p.page;
            early[i] = bt[idx < p.max_pages ? idx : p.max_pages - 1];
        }
        const int kv_start = p.positions[t0];
        const int kv_total = kv_start + 1;
        const bool cvalid = r < n_cols;
        const int head = kvh * g + col0 + (cvalid ? r : n_cols - 1);

        const int window_floor = p.window > 0 ? (kv_start - p.window + 1 > 0 ? kv_start - p.window + 1 : 0) : 0;
        int lo = window_floor > c_lo ? window_floor : c_lo, hi = kv_total;
        if (p.splits > 1 && hi > c_lo + p.chunk) hi = c_lo + p.chunk;
        lo &= ~31;

        // ---- loads, in the order in which their results are needed ------------------------------------
        // The rows of the projections' output that this wave norms and rotates (its query heads' rows and the new
        // key's: every wave asks for it, one wave uses it), the norms' weights and the angles, then the first
        // step's keys and values: the rows are formed while those are on their way, and the second step's are asked
        // for after that (a wave can have 63 loads outstanding: all at once would stall the issue of the last ones
        // until the first come back).
        const int qkv_row = (p.nq + 2 * p.nkv) * HD;
        const bf16_t* token_row = p.qkv + (size_t)t0 * qkv_row;
        uint4 qraw[KS], kraw[KS];
        uint32_t vnew[DB];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qraw[ks] = *(const uint4*)(token_row + (size_t)head * HD + ks * 32 + G * 8);
            kraw[ks] = *(const uint4*)(token_row + (size_t)(p.nq + kvh) * HD + ks * 32 + G * 8);
        }
        // the norms' weights and the token's angles for this lane's features (a feature's rotation partner, HD / 2
        // further on, lies in the same lane)
        constexpr int HK = KS / 2 > 0 ? KS / 2 : 1;      // (head sizes without this kernel still parse it)
        float4 qw[KS][2], kw[KS][2], cs[HK][2], sn[HK][2];
        if (p.q_norm_w != nullptr) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    qw[ks][h] = *(const float4*)(p.q_norm_w + ks * 32 + G * 8 + 4 * h);
                    kw[ks][h] = *(const float4*)(p.k_norm_w + ks * 32 + G * 8 + 4 * h);
                }
        }
        if (p.cos_t != nullptr) {
#pragma unroll
            for (int ks = 0; ks < KS / 2; ++ks)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const size_t a0 = (size_t)t0 * (HD / 2) + ks * 32 + G * 8 + 4 * h;
                    cs[ks][h] = *(const float4*)(p.cos_t + a0);
                    sn[ks][h] = *(const float4*)(p.sin_t + a0);
                }
        }


        // A step's 32 keys are two groups of 16 slots, each inside one page (page sizes are multiples of 16).
        // Slots past the request's length are read like any others as long as their page is the request's (their
        // scores are masked and their values zeroed in the step); pages past its last are not asked for.
        const int last_idx = (kv_total - 1) / p.page;
        const bool k_second = r >= 8, v_second = G >= 2;
        const uint32_t k_lane[2] = {(uint32_t)((((8 * (r >> 2) + (r & 3)) & 15) * HD + G * 8) * 2),
                                    (uint32_t)((((8 * (r >> 2) + 4 + (r & 3)) & 15) * HD + G * 8) * 2)};
        const uint32_t v_lane = (uint32_t)((r * p.page + 8 * (G & 1)) * 2);
        const size_t v_stride = (size_t)16 * p.page * 2;
        auto load_pages = [&](DecodeOperands& op, int k0, int page_a, int page_b) __attribute__((always_inline)) {
            const int off_a = k0 % p.page, off_b = (k0 + 16) % p.page;
            const char* ka = (const char*)(p.k_cache + (((size_t)page_a * p.nkv + kvh) * p.page + off_a) * HD);
            const char* kb = (const char*)(p.k_cache + (((size_t)page_b * p.nkv + kvh) * p.page + off_b) * HD);
            const char* va = (const char*)(p.v_cache + ((size_t)page_a * p.nkv + kvh) * HD * p.page + off_a);
            const char* vb = (const char*)(p.v_cache + ((size_t)page_b * p.nkv + kvh) * HD * p.page + off_b);
            const char* kbase = k_second ? kb : ka;
            const char* vbase = (v_second ? vb : va) + v_lane;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) op.k[t][ks] = *(const uint4*)(kbase + k_lane[t] + ks * 64);
#pragma unroll
            for (int db = 0; db < DB; ++db) op.v[db] = *(const uint4*)(vbase + db * v_stride);
        };
        auto load_step = [&](DecodeOperands& op, int k0) __attribute__((always_inline)) {
            int idx_a = k0 / p.page, idx_b = (k0 + 16) / p.page;
            idx_a = idx_a < last_idx ? idx_a : last_idx;
            idx_b = idx_b < last_idx ? idx_b : last_idx;
            load_pages(op, k0, bt[idx_a], bt[idx_b]);
        };
        // the first two steps, with the pages read ahead where the walk starts at the split's own start
        auto load_early = [&](DecodeOperands& op, int k0, int i) __attribute__((always_inline)) {
            if (lo == c_lo && (k0 + 16) / p.page <= last_idx) load_pages(op, k0, early[2 * i], early[2 * i + 1]);
            else load_step(op, k0);
        };
        const int n_steps = lo < hi ? (hi - lo + 31) / 32 : 0;
        DecodeOperands opa, opb;
        load_early(opa, lo, 0);

        // One head's row, normed and rotated as the separate kernel does it (32-bit throughout, one rounding at
        // the end): lane (., G) holds the features ks * 32 + G * 8 .. + 8 of the row, and a feature's rotation
        // partner, HD / 2 further on, lies in the same lane.
        auto normed_rotated = [&](const uint4 (&raw)[KS], const float4 (&nw)[KS][2], uint4 (&packed)[KS]) __attribute__((always_inline)) {
            float f[KS][8];
            float ss = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint32_t w[4] = {raw[ks].x, raw[ks].y, raw[ks].z, raw[ks].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    f[ks][2 * j] = __uint_as_float(w[j] << 16);
                    f[ks][2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) ss += f[ks][j] * f[ks][j];
            }
            if (p.q_norm_w != nullptr) {
                ss += __shfl_xor(ss, 16, IA_WAVE);
                ss += __shfl_xor(ss, 32, IA_WAVE);
                const float scale = 1.0f / sqrtf(ss / (float)HD + p.norm_eps);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const float gw[8] = {nw[ks][0].x, nw[ks][0].y, nw[ks][0].z, nw[ks][0].w,
                                         nw[ks][1].x, nw[ks][1].y, nw[ks][1].z, nw[ks][1].w};
#pragma unroll
                    for (int j = 0; j < 8; ++j) f[ks][j] = scale * f[ks][j] * (p.norm_add_one ? 1.0f + gw[j] : gw[j]);
                }
            }
            if (p.cos_t != nullptr) {
#pragma unroll
                for (int ks = 0; ks < KS / 2; ++ks) {
                    const float c[8] = {cs[ks][0].x, cs[ks][0].y, cs[ks][0].z, cs[ks][0].w,
                                        cs[ks][1].x, cs[ks][1].y, cs[ks][1].z, cs[ks][1].w};
                    const float sv[8] = {sn[ks][0].x, sn[ks][0].y, sn[ks][0].z, sn[ks][0].w,
                                         sn[ks][1].x, sn[ks][1].y, sn[ks][1].z, sn[ks][1].w};
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float a = f[ks][j], b = f[ks + KS / 2][j];
                        f[ks][j] = a * c[j] - b * sv[j];
                        f[ks + KS / 2][j] = a * sv[j] + b * c[j];
                    }
                }
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                packed[ks] = make_uint4(pack_bf16x2(f[ks][0], f[ks][1]), pack_bf16x2(f[ks][2], f[ks][3]),
                                        pack_bf16x2(f[ks][4], f[ks][5]), pack_bf16x2(f[ks][6], f[ks][7]));
        };
        uint4 qreg[KS], knew[KS];
        normed_rotated(qraw, qw, qreg);
        normed_rotated(kraw, kw, knew);
        if (n_steps >= 2) load_early(opb, lo + 32, 1);

        const bool has_new = p.slots != nullptr && hi == kv_total && lo < hi;

        f32x4 acc[DB];
        float m = -INFINITY, l = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};

        auto compute_step = [&](DecodeOperands& op, int k0) __attribute__((always_inline)) {
            if (k0 + 32 > kv_total) {
                // slots beyond the request's length hold anything at all: zero those values so that a probability
                // of zero times their content stays zero
                const int first_bad = kv_total - (k0 + 8 * G);
                if (first_bad < 8) {
#pragma unroll
                    for (int db = 0; db < DB; ++db) {
                        uint32_t w[4] = {op.v[db].x, op.v[db].y, op.v[db].z, op.v[db].w};
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            if (j >= first_bad) w[j >> 1] &= (j & 1) ? 0x0000ffffu : 0xffff0000u;
                        op.v[db] = make_uint4(w[0], w[1], w[2], w[3]);
                    }
                }
            }
            if (p.window > 0 && k0 < window_floor) {
                // keys below the window may lie in pages that the request has given back: as above
                const int first_good = window_floor - (k0 + 8 * G);
                if (first_good > 0) {
#pragma unroll
                    for (int db = 0; db < DB; ++db) {
                        uint32_t w[4] = {op.v[db].x, op.v[db].y, op.v[db].z, op.v[db].w};
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            if (j < first_good) w[j >> 1] &= (j & 1) ? 0x0000ffffu : 0xffff0000u;
                        op.v[db] = make_uint4(w[0], w[1], w[2], w[3]);
                    }
                }
            }
            if (has_new && k0 + 32 >= kv_total) {
                // (values chosen, never addresses: the operands stay in registers)
                const int kk = kv_total - 1 - k0;
                const bool mine = r == (((kk >> 3) << 2) | (kk & 3));
                const bool first = mine && ((kk >> 2) & 1) == 0, second = mine && ((kk >> 2) & 1) == 1;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    op.k[0][ks].x = first ? knew[ks].x : op.k[0][ks].x; op.k[0][ks].y = first ? knew[ks].y : op.k[0][ks].y;
                    op.k[0][ks].z = first ? knew[ks].z : op.k[0][ks].z; op.k[0][ks].w = first ? knew[ks].w : op.k[0][ks].w;
                    op.k[1][ks].x = second ? knew[ks].x : op.k[1][ks].x; op.k[1][ks].y = second ? knew[ks].y : op.k[1][ks].y;
                    op.k[1][ks].z = second ? knew[ks].z : op.k[1][ks].z; op.k[1][ks].w = second ? knew[ks].w : op.k[1][ks].w;
                }
                const int j = kk & 7;
                const bool vmine = G == (kk >> 3);
                const uint32_t keep = (j & 1) ? 0x0000ffffu : 0xffff0000u;
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const uint32_t put = (j & 1) ? vnew[db] << 16 : vnew[db];
                    op.v[db].x = vmine && (j >> 1) == 0 ? (op.v[db].x & keep) | put : op.v[db].x;
                    op.v[db].y = vmine && (j >> 1) == 1 ? (op.v[db].y & keep) | put : op.v[db].y;
                    op.v[db].z = vmine && (j >> 1) == 2 ? (op.v[db].z & keep) | put : op.v[db].z;
                    op.v[db].w = vmine && (j >> 1) == 3 ? (op.v[db].w & keep) | put : op.v[db].w;
                }
            }
            f32x4 s[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                s[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, op.k[t][ks]), __builtin_bit_cast(bf16x8, qreg[ks]), s[t], 0, 0, 0);
            }
            float sc[8];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) sc[4 * t + i] = s[t][i];
            if (k0 + 31 > kv_start || (p.window > 0 && k0 < window_floor)) {
                const int kbase_idx = k0 + 8 * G;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int key = kbase_idx + j;
                    if (key > kv_start || key < window_floor) sc[j] = -INFINITY;
                }
            }
            float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mx = fmaxf(mx, __shfl_xor(mx, 16, IA_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, IA_WAVE));
            const float m_new = fmaxf(m, mx * p.scale_log2);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m - m_use);
            float pr[8], psum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[j], p.scale_log2, -m_use));
                psum += pr[j];
            }
            l = l * alpha + psum;
            m = m_new;
            uint4 pb;
            pb.x = pack_bf16x2(pr[0], pr[1]);
            pb.y = pack_bf16x2(pr[2], pr[3]);
            pb.z = pack_bf16x2(pr[4], pr[5]);
            pb.w = pack_bf16x2(pr[6], pr[7]);
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    acc[db][0] *= alpha; acc[db][1] *= alpha;
                    acc[db][2] *= alpha; acc[db][3] *= alpha;
                }
            }
#pragma unroll
            for (int db = 0; db < DB; ++db)
                acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8, op.v[db]), __builtin_bit_cast(bf16x8, pb), acc[db], 0, 0, 0);
        };

        // The walk: two steps' operands are under way at any time.  Inside the loop every step has a step two
        // further on, so its loads are unconditional (the compiler counts what is outstanding and waits for the
        // older set only); the last one to three steps follow it.  opa holds step k0, opb step k0 + 32.
        int k0 = lo, left = n_steps;
        while (left > 3) {
            compute_step(opa, k0);
            load_step(opa, k0 + 64);
            compute_step(opb, k0 + 32);
            load_step(opb, k0 + 96);
            k0 += 64;
            left -= 2;
        }
        if (left == 3) {
            compute_step(opa, k0);
            load_step(opa, k0 + 64);
            compute_step(opb, k0 + 32);
            k0 += 64;
            left = 1;
        }
        // (the new value's features, for the wave that ends with the new key: asked for here, where they are needed)
        if (has_new) {
#pragma unroll
            for (int db = 0; db < DB; ++db) vnew[db] = token_row[(size_t)(p.nq + p.nkv + kvh) * HD + db * 16 + r].bits;
        }
        if (left == 2) {
            compute_step(opa, k0);
            compute_step(opb, k0 + 32);
        } else if (left == 1) {
            compute_step(opa, k0);
        }

        // The request's newest key (position kv_total - 1, this step's token) is in no page yet: the wave whose
        // keys end with it has put it and its value into its last step's operands in place of what the loads
        // brought, and now writes them to the cache for the steps to come.  (After the walk: with no store before
        // them, the block table's reads go through the scalar cache.)
        if (has_new) {
            const int slot = p.slots[t0];
            const int page = slot / p.page, off = slot - page * p.page;
            const int kk = (kv_total - 1) & 31;
            if (r == (((kk >> 3) << 2) | (kk & 3))) {
                bf16_t* krow = p.k_cache_w + (((size_t)page * p.nkv + kvh) * p.page + off) * HD + G * 8;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) *(uint4*)(krow + ks * 32) = knew[ks];
            }
            if (G == (kk >> 3)) {
                bf16_t* vdst = p.v_cache_w + (((size_t)page * p.nkv + kvh) * HD + r) * p.page + off;
#pragma unroll
                for (int db = 0; db < DB; ++db) vdst[(size_t)db * 16 * p.page].bits = (uint16_t)vnew[db];
            }
        }

        float lt = l;
        lt += __shfl_xor(lt, 16, IA_WAVE);
        lt += __shfl_xor(lt, 32, IA_WAVE);
        const size_t row0 = (size_t)t0 * p.nq + kvh * g + col0;        // the block's first (token, head) row
        if (p.splits == 1) {
            if (!cvalid) return;
            const float inv = 1.0f / lt;
            bf16_t* o = p.out + (row0 + r) * HD + 4 * G;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                uint2 w;
                w.x = pack_bf16x2(acc[db][0] * inv, acc[db][1] * inv);
                w.y = pack_bf16x2(acc[db][2] * inv, acc[db][3] * inv);
                *(uint2*)(o + 16 * db) = w;
            }
            return;
        }

        // ---- the block's waves add up: lane (col, G) holds dims 16 db + 4 G + i of its column --------
        float* team_o = team_mem;                                       // [team][n_cols][HD]
        float* team_ml = team_mem + (size_t)team * n_cols * HD;         // [team][n_cols][2]
        if (cvalid) {
            float* o = team_o + ((size_t)wave * n_cols + r) * HD + 4 * G;
#pragma unroll
            for (int db = 0; db < DB; ++db) *(f32x4*)(o + 16 * db) = acc[db];
            if (G == 0) {
                team_ml[(wave * n_cols + r) * 2] = m;
                team_ml[(wave * n_cols + r) * 2 + 1] = lt;
            }
        }
        __syncthreads();
        const int pieces = n_cols * (HD / 4);                           // 16-byte pieces of the block's result
        for (int e = threadIdx.x; e < pieces; e += blockDim.x) {
            const int col = e / (HD / 4), piece = e - col * (HD / 4);
            float mx = -INFINITY;
            for (int w = 0; w < team; ++w) mx = fmaxf(mx, team_ml[(w * n_cols + col) * 2]);
            f32x4 o = (f32x4){0.f, 0.f, 0.f, 0.f};
            float total = 0.f;
            for (int w = 0; w < team; ++w) {
                const float mw = team_ml[(w * n_cols + col) * 2];
                const float wt = mw == -INFINITY ? 0.f : exp2f(mw - mx);      // a split that held no key of this row
                const f32x4 v = *(const f32x4*)(team_o + ((size_t)w * n_cols + col) * HD + piece * 4);
                o[0] = fmaf(v[0], wt, o[0]); o[1] = fmaf(v[1], wt, o[1]);
                o[2] = fmaf(v[2], wt, o[2]); o[3] = fmaf(v[3], wt, o[3]);
                total = fmaf(team_ml[(w * n_cols + col) * 2 + 1], wt, total);
            }
            if (teams == 1) {
                const float inv = 1.0f / total;
                uint2 w;
                w.x = pack_bf16x2(o[0] * inv, o[1] * inv);
                w.y = pack_bf16x2(o[2] * inv, o[3] * inv);
                *(uint2*)(p.out + (row0 + col) * HD + piece * 4) = w;
            } else {
                float* po = p.part_o + ((row0 + col) * teams + tm) * HD + piece * 4;
                put_across(po, o[0]); put_across(po + 1, o[1]); put_across(po + 2, o[2]); put_across(po + 3, o[3]);
                if (piece == 0) {
                    float* ml = p.part_ml + ((row0 + col) * teams + tm) * 2;
                    put_across(ml, mx);
                    put_across(ml + 1, total);
                }
            }
        }
        if (teams == 1) return;

        // ---- the last block of this (request, key/value head, column block) merges the blocks' results --------
        int* counter = counters + ((size_t)blockIdx.z * p.nkv + kvh) * gridDim.x + blockIdx.x;
        // The hand-over.  Writer: a wave's vector-memory counter counts a store down when the memory has taken it
        // (the stores above are written through, so that is the point where every die reads it), and
        // `s_waitcnt vmcnt(0)` holds the wave until all of its stores are there; then the barrier, so that this
        // holds for every wave of the block; only then the count.  (A release fence of workgroup scope does not wait
        // for stores that leave the compute unit, and one of device scope writes the die's L2 back.)  The compiler
        // moves no store across the wait (the asm names memory).
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0)
            s_last = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == teams - 1 ? 1 : 0;
        __syncthreads();
        if (!s_last) return;
        // Reader: thread 0 has the counter's old value in a register before it can write s_last, so the increment
        // that made it teams - 1, and with it every other block's stores, is in memory before any thread passes the
        // barrier above; the loads below are issued after it, and they read past the caches (device scope), so they
        // cannot meet a line that was fetched before the stores arrived.
        // Every thread takes part: the block's threads form as many groups as there are 16-byte pieces of the result
        // in them, group i sums the blocks i, i + groups, ... in that order, and the groups' sums meet in shared
        // memory and are added in the groups' order.
        const int groups = pieces <= (int)blockDim.x ? (int)blockDim.x / pieces : 1;
        float* red = team_mem;                                          // [groups][pieces][6]: maximum, sum, four outputs
        for (int e0 = 0; e0 < pieces; e0 += blockDim.x) {
            const int grp = groups > 1 ? (int)threadIdx.x / pieces : 0;
            const int e = groups > 1 ? (int)threadIdx.x - grp * pieces : e0 + (int)threadIdx.x;
            const bool active = grp < groups && e < pieces;
            float mx = -INFINITY, total = 0.f;
            f32x4 o = (f32x4){0.f, 0.f, 0.f, 0.f};
            const int col = active ? e / (HD / 4) : 0, piece = active ? e - col * (HD / 4) : 0;
            if (active) {
                const float* ml = p.part_ml + (row0 + col) * teams * 2;
                const float* po = p.part_o + (row0 + col) * teams * HD + piece * 4;
#pragma unroll 8
                for (int t = grp; t < teams; t += groups) {
                    const float2 mt = make_float2(get_across(ml + 2 * t), get_across(ml + 2 * t + 1));
                    const float* pv = po + (size_t)t * HD;
                    const f32x4 v = (f32x4){get_across(pv), get_across(pv + 1), get_across(pv + 2), get_across(pv + 3)};
                    const float m_new = fmaxf(mx, mt.x);
                    const float back = m_new == -INFINITY ? 0.f : exp2f(mx - m_new);        // rescales what is summed so far
                    const float wt = mt.x == -INFINITY ? 0.f : exp2f(mt.x - m_new);
                    o[0] = fmaf(v[0], wt, o[0] * back); o[1] = fmaf(v[1], wt, o[1] * back);
                    o[2] = fmaf(v[2], wt, o[2] * back); o[3] = fmaf(v[3], wt, o[3] * back);
                    total = fmaf(mt.y, wt, total * back);
                    mx = m_new;
                }
            }
            if (groups > 1) {
                if (active) {                                           // (the waves' results in this memory were read before the count)
                    float* mine = red + ((size_t)grp * pieces + e) * 6;
                    mine[0] = mx; mine[1] = total; mine[2] = o[0]; mine[3] = o[1]; mine[4] = o[2]; mine[5] = o[3];
                }
                __syncthreads();
                if (!active || grp != 0) continue;
                for (int gi = 1; gi < groups; ++gi) {
                    const float* other = red + ((size_t)gi * pieces + e) * 6;
                    const float m_new = fmaxf(mx, other[0]);
                    const float back = m_new == -INFINITY ? 0.f : exp2f(mx - m_new);
                    const float wt = other[0] == -INFINITY ? 0.f : exp2f(other[0] - m_new);
                    o[0] = fmaf(other[2], wt, o[0] * back); o[1] = fmaf(other[3], wt, o[1] * back);
                    o[2] = fmaf(other[4], wt, o[2] * back); o[3] = fmaf(other[5], wt, o[3] * back);
                    total = fmaf(other[1], wt, total * back);
                    mx = m_new;
                }
            } else if (!active) {
                continue;
            }
            const float inv = 1.0f / total;
            uint2 w;
            w.x = pack_bf16x2(o[0] * inv, o[1] * inv);
            w.y = pack_bf16x2(o[2] * inv, o[3] * inv);
            *(uint2*)(p.out + (row0 + col) * HD + piece * 4) = w;
        }
        if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);     // zero again for the next call
    }
}

// ---- prompt portions, head size 128: blocks of eight waves that share keys and values ----------
// A block owns 128 columns of one request and key/value head and walks the keys in stages of 64: four waves
// (32 columns each) share a stage, and the block has two such groups, one on the even stages and one on the odd
// ones, that add up at the end.  A stage's keys and values come from the cache pages straight into shared memory
// (global_load_lds, 16 bytes a lane: no register holds them on the way), a group's next stage while this
// one is multiplied, and every wave reads its MFMA operands from there: the L2 is asked for a key once
// a block instead of once a wave.  A load instruction fills 1 KiB of shared memory in lane order, so
// the lane picks the piece it fetches such that the layout comes out swizzled:
//   keys    row of 256 bytes a key, the 16-byte piece c of key k at place c ^ ((k & 3) | ((k >> 3) & 3) << 2)
//   values  by groups of 16 keys: row of 32 bytes a feature, as the cache page holds it
// The swizzle of the keys spreads the 16 rows that a read takes at the same place over the banks (rows of 256
// bytes would all begin in the same one).  The counters show no bank conflict for either array
// (SQ_LDS_BANK_CONFLICT = 0); values with their halves swapped in every other block of eight features, which
// looked as good on paper, cost two extra cycles a read.
// Measured (one request, 32 query and 8 key/value heads; the kernel of single waves, then blocks of four waves, two
// a compute unit, then these): a prompt of 2,048 tokens 118 -> 77 -> 68 us, of 4,096 tokens 257 -> 201 us, of 8,192
// tokens 1.20 -> 0.75 -> 0.77 ms; a portion of 512 tokens at 7,680 181 -> 99 -> 116 us (keys split between two
// blocks).  Time stamps inside the kernel, 2,048 tokens: with blocks of four waves a compute unit held a long walk
// and a short one, the short one was done at once and the long one ran alone, a wave a SIMD, so the prompt took as
// long as its longest walk alone; and the blocks were handed out head by head (x was the tile), the longest walks of
// the last heads starting when the first heads' were done: compute units were busy between 15 and 102 us.  With the
// order of the kernel's comment and these blocks every unit runs two blocks and is busy 57 to 63 us; a block's
// pass over two stages takes 2.9 us (29 % of the matrix pipes' time), its start 1.2 us, the groups' sum 0.6, its
// end 2.4.  Timing-only variants of the blocks of four waves showed no single bound: without the exponentials 6 %
// faster, without the barrier 7 %, without the column maxima 8 %, without the second product 11 %, without the loads
// into shared memory 16 %.  Measured on a SIMD by itself: a matrix product takes 16 cycles and holds the issue for
// about 8 of them, an exponential 8 to 10, a 16-byte read of shared memory 32 when all four SIMDs read (128 bytes a
// cycle a compute unit: at 32 columns a wave the reads take as long as the products).
// 16 bytes a lane from memory straight into shared memory, 1 KiB a wave in lane order from `lds_at` on (the same for
// all lanes).  Written out so that the compiler does not count it among the loads it waits for: whoever reads the
// shared memory it fills waits for it by hand (s_waitcnt vmcnt) and passes a barrier.
__device__ __forceinline__ void lds_load16(const char* from, uint32_t lds_at) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(lds_at) : "memory");     // (m0 holds nothing of the compiler's across statements)
}

#define TILE_WAVES 4              // waves that share a stage: each with its own columns
#define TILE_GROUPS 2             // groups of such waves in a block: each with its own stages (see the kernel)
#define TILE_STAGE 64
#define TILE_K_BYTES (TILE_STAGE * HD * 2)
#define TILE_BUF_BYTES (2 * TILE_K_BYTES)

// Two column tiles of 16 a wave, two blocks a compute unit, two waves a SIMD.  (Four tiles a wave, so that every key and
// value read out of shared memory serves twice as many products, take the registers of a whole SIMD; with the softmax of
// one tile laid beside the products of the others in the instruction stream that ran at 530 TFLOP/s on a prompt of
// 8,192 tokens where two waves a SIMD run at 730, and the rescaling of accumulators that live in the matrix cores' own
// registers cost as much again.)
#define TILE_NBW 2
// NBW_: column tiles of 16 a wave.  One instead of two halves a block's columns (64) and doubles the blocks: for steps
// whose blocks of 128 columns would leave compute units without one (short prompts, few heads).
template <bool ENABLED = (HD == 128), int NBW_ = TILE_NBW>
__global__ __launch_bounds__(TILE_GROUPS * TILE_WAVES * IA_WAVE) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attn_tile_kernel(const AttnParams p) {
    if constexpr (ENABLED) {
        constexpr int NBW = NBW_;
        constexpr int WAVE_COLS = 16 * NBW;
        constexpr int TILE_COLS = TILE_WAVES * WAVE_COLS;
        // Two stages for each group.  The loads that fill them are written as instructions of their own below
        // (lds_load16): the compiler then neither knows of them nor waits for them before it reads an operand of
        // the other stage (it would, not knowing which stage a pointer chosen at run time names); the waits that
        // are needed stand in the code, one at the start of a stage.
        __shared__ __align__(16) char stage_mem[TILE_GROUPS * 2 * TILE_BUF_BYTES];
        // Two groups of four waves walk the same 128 columns: group 0 takes the even stages of the keys, group 1
        // the odd ones, each through its own two stages of shared memory, and at the end group 1 hands its sums
        // to group 0 through that memory.  A compute unit holds one block, two waves a SIMD that walk equally
        // far, and takes the next block when it is done.  (Two blocks of four waves, a long walk and a short
        // one so that a unit's work came out even, left the long walk alone on its unit for most of its time, a
        // wave a SIMD: a prompt of 2,048 tokens took as long as its longest walk took alone.)
        const int lane = threadIdx.x & (IA_WAVE - 1), wave = (threadIdx.x / IA_WAVE) & (TILE_WAVES - 1);
        const int kg = __builtin_amdgcn_readfirstlane(threadIdx.x / (IA_WAVE * TILE_WAVES));
        const int r = lane & 15, G = lane >> 4;
        // The blocks of a launch are handed out in the order of their numbers, x fastest, to the chip's eight dies in
        // turn: x holds the key/value head, the split and the request, y the tile, longest walk first.  So the
        // longest walks of all heads and requests start first and a compute unit that is done takes the longest
        // that is left, and a head's tiles, which read the same keys, meet on one die and its L2 (eight heads).
        const int heads_splits = p.nkv * p.splits;
        const int seq_local = blockIdx.x / heads_splits, head_split = blockIdx.x - seq_local * heads_splits;
        const int kvh = head_split / p.splits, split = head_split - kvh * p.splits;
        const int seq = p.seq_begin + seq_local;
        const int g = p.nq / p.nkv;
        const int t0 = p.cu_tokens[seq], q_len = p.cu_tokens[seq + 1] - t0;
        const int n_cols = q_len * g;
        const int n_tiles = (n_cols + TILE_COLS - 1) / TILE_COLS;
        if ((int)blockIdx.y >= n_tiles) return;
        const int bcol0 = (n_tiles - 1 - (int)blockIdx.y) * TILE_COLS;
        const int kv_start = p.positions[t0];
        const int kv_total = kv_start + q_len;
        const int* bt = p.block_table + (size_t)seq * p.max_pages;
        const int blast = (bcol0 + TILE_COLS <= n_cols ? bcol0 + TILE_COLS : n_cols) - 1;
        const int bpmin = kv_start + bcol0 / g, bpmax = kv_start + blast / g;
        const int bfloor = p.window > 0 ? (bpmin - p.window + 1 > 0 ? bpmin - p.window + 1 : 0) : 0;   // first key the block sees
        int lo = bfloor;
        lo &= ~(TILE_STAGE - 1);
        int hi = bpmax + 1;
        if (p.splits > 1) {             // this block's share of the keys (`chunk` is a multiple of a stage)
            const int c_lo = split * p.chunk, c_hi = c_lo + p.chunk;
            lo = lo > c_lo ? lo : c_lo;
            hi = hi < c_hi ? hi : c_hi;
        }
        const int stages = hi > lo ? (hi - lo + TILE_STAGE - 1) / TILE_STAGE : 0;

        // this wave's columns (a wave without any still brings its share of the stages)
        const int col0 = bcol0 + wave * WAVE_COLS;
        const bool has_cols = col0 < n_cols;
        int tq[NBW], head[NBW], pos[NBW];
        bool cvalid[NBW];
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const int c = col0 + nb * 16 + r;
            cvalid[nb] = c < n_cols;
            const int cc = cvalid[nb] ? c : n_cols - 1;
            tq[nb] = cc / g;
            head[nb] = kvh * g + (cc - tq[nb] * g);
            pos[nb] = kv_start + tq[nb];
        }
        const int wlast = (col0 + WAVE_COLS <= n_cols ? col0 + WAVE_COLS : n_cols) - 1;
        const int pmin = kv_start + (has_cols ? col0 : 0) / g, pmax = has_cols ? kv_start + wlast / g : -1;
        const int wlo = p.window > 0 ? (pmin - p.window + 1 > 0 ? pmin - p.window + 1 : 0) : 0;

        uint4 qreg[NBW][KS];
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const bf16_t* qrow = p.q + ((size_t)(t0 + tq[nb]) * p.nq + head[nb]) * HD;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) qreg[nb][ks] = cvalid[nb] ? *(const uint4*)(qrow + ks * 32 + G * 8) : zero4();
        }
        f32x4 acc[NBW][DB];
        float m[NBW], l[NBW];
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            m[nb] = -INFINITY;
            l[nb] = 0.f;
#pragma unroll
            for (int db = 0; db < DB; ++db) acc[nb][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }

        // ---- a stage on its way: wave w brings keys 16 w .. + 16 and features 32 w .. + 32 ----------
        // Groups of 16 keys past the request's length are read from the group of its last key instead
        // (their scores are masked and their values zeroed below): the pages behind may not exist.
        // Wave w brings the stage's w-th group of 16 keys and their values: one place in one page, the same
        // for all its lanes.  The pages' numbers come 64 at a time into a register, lane i with the entry
        // pages_base + i of the block table, and a stage takes its number from there with a lane read: a read
        // of the block table in every stage, through the scalar cache, kept each wave waiting for a trip to the
        // memory before its first operand of the stage (the counter of those reads is the shared memory's too).
        // What a lane adds to that place does not change from stage to stage.
        const int wave_s = __builtin_amdgcn_readfirstlane(wave);
        const int last_idx = (kv_total - 1) / p.page;
        int pages_base = 0, pages_reg = 0;
        auto pages_load = [&](int base) {
            pages_base = base;
            const int idx = base + lane;
            pages_reg = bt[idx < last_idx ? idx : last_idx];
        };
        auto pages_for = [&](int s, int& page, int& off) {
            const int key0 = lo + s * TILE_STAGE + 16 * wave_s;
            const int k = key0 < kv_total ? key0 : (kv_total - 1) & ~15;
            const int idx = k / p.page;
            if (idx >= pages_base + IA_WAVE) pages_load(idx);
            page = __builtin_amdgcn_readlane(pages_reg, idx - pages_base);
            off = k - idx * p.page;
        };
        uint32_t k_from[4];             // keys: chunk c is rows 4 c .. + 4 of the group, a lane's piece swizzled
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int row = 4 * c + (lane >> 4), key = 16 * wave + row;
            const int piece = (lane & 15) ^ ((key & 3) | (((key >> 3) & 3) << 2));
            k_from[c] = (uint32_t)(row * (HD * 2) + piece * 16);
        }
        // values: chunk c is features 32 c .. + 32, two lanes a feature (its 16 keys)
        const int v_half = lane & 1;                                            // which eight keys the lane's piece holds
        const uint32_t v_from = (uint32_t)(((lane >> 1) * p.page + v_half * 8) * 2);
        auto issue = [&](char* buf, int page, int off) {
            const char* krows = (const char*)(p.k_cache + (((size_t)page * p.nkv + kvh) * p.page + off) * HD);
            const char* vrows = (const char*)(p.v_cache + ((size_t)page * p.nkv + kvh) * HD * p.page + off);
            const uint32_t at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)buf;
#pragma unroll
            for (int c = 0; c < 4; ++c) lds_load16(krows + k_from[c], at + (16 * wave_s + 4 * c) * (HD * 2));
#pragma unroll
            for (int c = 0; c < 4; ++c)
                lds_load16(vrows + (size_t)c * 32 * p.page * 2 + v_from, at + TILE_K_BYTES + wave_s * (16 * HD * 2) + c * 1024);
        };
        // values of keys past the request's length may hold anything at all: a lane zeroes them in the
        // pieces that it brought itself, once they have arrived
        // So may the values of keys below the block's window, between the stage's start and the first key that any
        // of its columns sees: the window has passed them, and their pages may have been given back.
        auto zero_tail = [&](int s, char* buf) {
            const int kb = lo + s * TILE_STAGE;
            const int mine = kb + 16 * wave_s + 8 * v_half;          // the first of this lane's eight keys
            const int first_bad = kb + TILE_STAGE <= kv_total ? 8 : kv_total - mine;
            const int first_good = kb < bfloor ? bfloor - mine : 0;
            if (first_bad >= 8 && first_good <= 0) return;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                uint4* at = (uint4*)(buf + TILE_K_BYTES + wave_s * (16 * HD * 2) + c * 1024 + lane * 16);
                const uint4 v = *at;
                uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (j >= first_bad || j < first_good) w[j >> 1] &= (j & 1) ? 0x0000ffffu : 0xffff0000u;
                *at = make_uint4(w[0], w[1], w[2], w[3]);
            }
        };

        // this lane's places in a stage: they do not change from stage to stage
        uint32_t k_at[KS];              // keys: the lane's row of tile 0 of step 0 and its swizzled piece of dim step ks
        {
            const int kl = 8 * (r >> 2) + (r & 3);
            const uint32_t k_xor = (uint32_t)((kl & 3) | (((kl >> 3) & 3) << 2));
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) k_at[ks] = (uint32_t)(kl * (HD * 2)) + (((uint32_t)(ks * 4 + G) ^ k_xor) * 16);
        }
        // values: group of 16 keys (G >> 1 of the step's two), feature row of 32 bytes, half G & 1
        const uint32_t v_at = (uint32_t)((G >> 1) * (16 * HD * 2) + r * 32 + (G & 1) * 16);
        int page_l, off_l;
        auto stage = [&](int s, char* buf, char* other) __attribute__((always_inline)) {
            if (s >= stages) {                             // the other group has a stage more: its barrier is kept
                __syncthreads();
                return;
            }
            __builtin_amdgcn_s_waitcnt(0);                 // this wave's part of stage s has arrived
            zero_tail(s, buf);
            __syncthreads();                               // everybody's has, and everybody is done with the stage before
            // The loads of the group's next stage: group 0 asks for them here, group 1 between its two steps.  A load
            // instruction holds its wave until the compute unit's one address unit takes it, 1 KiB in 16 cycles: with
            // all eight waves asking at once after the barrier (64 KiB a pass) each waited some 1,100 to 1,700 cycles
            // of a pass's 6,500, all at the same time (8,192 tokens 736 -> 655 us).
            const bool more = s + TILE_GROUPS < stages;
            if (more && kg == 0) issue(other, page_l, off_l);
            const int kb = lo + s * TILE_STAGE;
            // Steps of 32 keys.  A wave's operands are asked for a phase ahead of their use: the values of a
            // step before its softmax is worked out, the keys of the next step before this step's second
            // product, so that the shared memory's latency passes behind arithmetic.
            bool live[2];
#pragma unroll
            for (int u = 0; u < 2; ++u)        // something of the step is visible to this wave's columns
                live[u] = !(kb + 32 * u > pmax || kb + 32 * u + 31 < wlo);
            uint4 kop[2][KS];
            auto read_keys = [&](int u) {
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        kop[t][ks] = *(const uint4*)(buf + (32 * u + 4 * t) * (HD * 2) + k_at[ks]);
            };
            if (live[0]) read_keys(0);
            else if (live[1]) read_keys(1);
            // A step of 32 keys.  The wave's two column tiles take turns so that the softmax of one (vector
            // arithmetic) has matrix products of the other beside it in the same stretch of code: the scores of
            // tile 1 beside the softmax of tile 0, the second product of tile 0 beside the softmax of tile 1.  The
            // order of every sum is as before.  EDGE: some key of the step is masked for some column.
            auto scores = [&](int nb, f32x4 (&sacc)[2]) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    sacc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8, kop[t][ks]), __builtin_bit_cast(bf16x8, qreg[nb][ks]), sacc[t], 0, 0, 0);
                }
            };
            auto softmax = [&](auto edge_c, int nb, int k0, const f32x4 (&sacc)[2], uint4& pb, float& alpha) {
                constexpr bool EDGE = decltype(edge_c)::value;
                float sc[8];
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) sc[4 * t + i] = sacc[t][i];
                if constexpr (EDGE) {
                    const int kbase_idx = k0 + 8 * G;
                    const int floor_key = p.window > 0 ? pos[nb] - p.window + 1 : 0;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int key = kbase_idx + j;
                        if (key > pos[nb] || key < floor_key) sc[j] = -INFINITY;
                    }
                }
                // (the compiler's own maximum: written out as v_max3 instructions, which the compiler does not check
                // against the matrix products that wrote the scores, the maxima could read a score's register before
                // its product had written it, and took a probability of the step before for a score; with the wait
                // that forbids that tied to the scores a prompt of 8,192 tokens took 823 us, so 728)
                float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
                mx = column_max(mx);
                // The exponents' reference point moves only when the step's maximum has passed it by 2^8
                // (probabilities then reach 2^8 at most, which 32-bit sums and bfloat16 operands hold as
                // well as 1): the accumulators are rescaled a few times a walk instead of at most steps.
                const float cand = mx * p.scale_log2;
                const bool rise = cand > m[nb] + 8.0f;              // also the first finite maximum after -inf
                const float m_new = rise ? cand : m[nb];
                const float m_use = m_new == -INFINITY ? 0.f : m_new;
                alpha = rise ? __builtin_amdgcn_exp2f(m[nb] - m_use) : 1.0f;
                float pr[8], psum = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[j], p.scale_log2, -m_use));
                    psum += pr[j];
                }
                l[nb] = l[nb] * alpha + psum;
                m[nb] = m_new;
                pb.x = pack_bf16x2(pr[0], pr[1]);
                pb.y = pack_bf16x2(pr[2], pr[3]);
                pb.z = pack_bf16x2(pr[4], pr[5]);
                pb.w = pack_bf16x2(pr[6], pr[7]);
            };
            auto rescale = [&](int nb, float alpha) {
                if (__any(alpha != 1.0f)) {
#pragma unroll
                    for (int db = 0; db < DB; ++db) {
                        acc[nb][db][0] *= alpha; acc[nb][db][1] *= alpha;
                        acc[nb][db][2] *= alpha; acc[nb][db][3] *= alpha;
                    }
                }
            };
            auto weighted = [&](int nb, const uint4 (&vop)[DB], const uint4& pb) {
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    acc[nb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, vop[db]), __builtin_bit_cast(bf16x8, pb), acc[nb][db], 0, 0, 0);
            };
            // eight matrix products with a share of the vector instructions after each
            auto beside = [&]() {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one matrix product
                    __builtin_amdgcn_sched_group_barrier(0x002, 9, 0);      // nine vector instructions
                }
            };
            auto pin = [&](uint4& pb, float& alpha) {
                // (pins the probabilities to the stretch of code they are formed in: left alone, the compiler moves
                // their arithmetic behind the branch of the rescaling, next to the product that uses them)
                asm volatile("" : "+v"(pb.x), "+v"(pb.y), "+v"(pb.z), "+v"(pb.w), "+v"(alpha));
            };
            auto step = [&](auto edge_c, int u) {
                const int k0 = kb + 32 * u;
                uint4 vop[DB];
                if constexpr (NBW == 1) {
                    // one column tile: nothing of its own to lay beside the softmax (the SIMD's other wave is)
                    f32x4 s0[2];
                    uint4 pb0;
                    float alpha0;
                    scores(0, s0);
#pragma unroll
                    for (int db = 0; db < DB; ++db)
                        vop[db] = *(const uint4*)(buf + TILE_K_BYTES + u * (32 * HD * 2) + db * 512 + v_at);
                    softmax(edge_c, 0, k0, s0, pb0, alpha0);
                    if (u == 0) read_keys(1);
                    rescale(0, alpha0);
                    weighted(0, vop, pb0);
                } else {
                f32x4 s0[2], s1[2];
                uint4 pb0, pb1;
                float alpha0, alpha1;
                scores(0, s0);
#pragma unroll
                for (int db = 0; db < DB; ++db)
                    vop[db] = *(const uint4*)(buf + TILE_K_BYTES + u * (32 * HD * 2) + db * 512 + v_at);
                __builtin_amdgcn_sched_barrier(0);
                scores(1, s1);
                softmax(edge_c, 0, k0, s0, pb0, alpha0);
                pin(pb0, alpha0);
                beside();
                __builtin_amdgcn_sched_barrier(0);
                if (u == 0) read_keys(1);               // (a step that this wave skips: read all the same, used by nobody)
                rescale(0, alpha0);
                __builtin_amdgcn_sched_barrier(0);
                weighted(0, vop, pb0);
                softmax(edge_c, 1, k0, s1, pb1, alpha1);
                pin(pb1, alpha1);
                beside();
                __builtin_amdgcn_sched_barrier(0);
                rescale(1, alpha1);
                weighted(1, vop, pb1);
                }
            };
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                if (u == 1 && more && kg != 0) issue(other, page_l, off_l);
                if (!live[u]) continue;
                const int k0 = kb + 32 * u;
                const bool edge = k0 + 31 > pmin || (p.window > 0 && k0 < pmax - p.window + 1);
                if (edge) step(std::true_type(), u);
                else step(std::false_type(), u);
            }
            if (s + 2 * TILE_GROUPS < stages) pages_for(s + 2 * TILE_GROUPS, page_l, off_l);
        };
        // A group's walk: its stages are kg, kg + 2, ...; both groups pass the same number of barriers.
        auto walk = [&](char* first, char* second) __attribute__((always_inline)) {
            if (kg < stages) {
                const int key0 = lo + kg * TILE_STAGE + 16 * wave_s;
                pages_load((key0 < kv_total ? key0 : (kv_total - 1) & ~15) / p.page);
                pages_for(kg, page_l, off_l);
                issue(first, page_l, off_l);
                if (kg + TILE_GROUPS < stages) pages_for(kg + TILE_GROUPS, page_l, off_l);
            }
            for (int s = kg; s - kg < stages; s += 2 * TILE_GROUPS) {
                stage(s, first, second);
                if (s - kg + TILE_GROUPS < stages) stage(s + TILE_GROUPS, second, first);
            }
        };
        walk(stage_mem + (2 * kg) * TILE_BUF_BYTES, stage_mem + (2 * kg + 1) * TILE_BUF_BYTES);

        // ---- group 1 hands its sums to group 0: accumulators through its own two stages, maxima and sums through
        // group 0's first ------------------------------------------------------------------------------------------
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        {
            f32x4* xacc = (f32x4*)(stage_mem + 2 * TILE_BUF_BYTES + wave_s * (TILE_BUF_BYTES / 2));      // [nb][db][lane]
            __shared__ float2 xml_mem[TILE_WAVES * NBW * IA_WAVE];
            float2* xml = xml_mem + wave_s * NBW * IA_WAVE;                                             // [nb][lane]
            if (kg == 1) {
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) {
#pragma unroll
                    for (int db = 0; db < DB; ++db) xacc[(nb * DB + db) * IA_WAVE + lane] = acc[nb][db];
                    xml[nb * IA_WAVE + lane] = make_float2(m[nb], l[nb]);
                }
            }
            __syncthreads();
            if (kg == 1) return;
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) {
                const float2 other = xml[nb * IA_WAVE + lane];
                const float top = fmaxf(m[nb], other.x);
                const float mine_w = m[nb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[nb] - top);
                const float other_w = other.x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(other.x - top);
                l[nb] = l[nb] * mine_w + other.y * other_w;
                m[nb] = top;
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const f32x4 o = xacc[(nb * DB + db) * IA_WAVE + lane];
                    acc[nb][db][0] = acc[nb][db][0] * mine_w + o[0] * other_w;
                    acc[nb][db][1] = acc[nb][db][1] * mine_w + o[1] * other_w;
                    acc[nb][db][2] = acc[nb][db][2] * mine_w + o[2] * other_w;
                    acc[nb][db][3] = acc[nb][db][3] * mine_w + o[3] * other_w;
                }
            }
        }
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const float lt = column_sum(l[nb]);
            if (!cvalid[nb]) continue;
            const size_t row = (size_t)(t0 + tq[nb]) * p.nq + head[nb];
            if (p.splits == 1) {
                const float inv = 1.0f / lt;
                bf16_t* o = p.out + row * HD + 4 * G;
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    uint2 w;
                    w.x = pack_bf16x2(acc[nb][db][0] * inv, acc[nb][db][1] * inv);
                    w.y = pack_bf16x2(acc[nb][db][2] * inv, acc[nb][db][3] * inv);
                    *(uint2*)(o + 16 * db) = w;
                }
            } else {
                // for the merge: sums and accumulators relative to the exponents' reference point m
                float* o = p.part_o + (row * p.splits + split) * HD + 4 * G;
#pragma unroll
                for (int db = 0; db < DB; ++db) *(f32x4*)(o + 16 * db) = acc[nb][db];
                if (G == 0) {
                    float* ml = p.part_ml + (row * p.splits + split) * 2;
                    ml[0] = m[nb];
                    ml[1] = lt;
                }
            }
        }
    }
}

static int g_tiles = 1;
// Measurement switch: 0 keeps prompt portions on the kernel of single waves; 2: blocks of 64 columns whatever the
// step's size; 3: of 128.
extern "C" void ia_attention_mfma_tiles(int on) { g_tiles = on; }

// Compute units of the current device (asked for once a device).
static int attn_cus() {
    static int cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cus[dev] == 0) {
        int n = 0;
        cus[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
    }
    return cus[dev];
}

// Merges the partial results of the key splits of one (token, head): one block a row.  The
// partial results were written by other compute units, so every read is a long way off: the
// block's waves share the splits between them (wave w takes splits w, w + waves, ...) and
// every lane has all its loads in flight at once; the waves' sums meet in shared memory and
// are added in wave order.
#define MERGE_WAVES 16
__global__ __launch_bounds__(MERGE_WAVES * IA_WAVE) void attn_merge_kernel(
    bf16_t* __restrict__ out, const float* __restrict__ part_o, const float* __restrict__ part_ml, int splits,
    size_t first_row) {
    constexpr int PER = (HD + IA_WAVE - 1) / IA_WAVE;
    __shared__ float weight[256];
    __shared__ float red[MERGE_WAVES][PER * IA_WAVE];
    __shared__ float s_total;
    const size_t row = first_row + blockIdx.x;
    const int lane = threadIdx.x & (IA_WAVE - 1), wave = threadIdx.x / IA_WAVE;
    const float* ml = part_ml + row * splits * 2;
    const float* po = part_o + row * splits * HD;
    // this wave's partial outputs, asked for before anything is waited for
    float v[256 / MERGE_WAVES][PER];
#pragma unroll
    for (int i = 0; i < 256 / MERGE_WAVES; ++i) {
        const int s = wave + i * MERGE_WAVES;
#pragma unroll
        for (int t = 0; t < PER; ++t) {
            const int e = lane + t * IA_WAVE;
            v[i][t] = (s < splits && e < HD) ? po[(size_t)s * HD + e] : 0.f;
        }
    }
    if (wave == 0) {
        float mx = -INFINITY;
        for (int s = lane; s < splits; s += IA_WAVE) mx = fmaxf(mx, ml[2 * s]);
        mx = wave_max(mx);
        float total = 0.f;
        for (int s = lane; s < splits; s += IA_WAVE) {
            const float ms = ml[2 * s];
            const float w = ms == -INFINITY ? 0.f : exp2f(ms - mx);      // a split that held no key of this row
            weight[s] = w;
            total += ml[2 * s + 1] * w;
        }
        total = wave_sum(total);
        if (lane == 0) s_total = total;
    }
    __syncthreads();
    float o[PER];
#pragma unroll
    for (int t = 0; t < PER; ++t) o[t] = 0.f;
#pragma unroll
    for (int i = 0; i < 256 / MERGE_WAVES; ++i) {
        const int s = wave + i * MERGE_WAVES;
        if (s < splits) {
            const float w = weight[s];
#pragma unroll
            for (int t = 0; t < PER; ++t) o[t] = fmaf(v[i][t], w, o[t]);
        }
    }
#pragma unroll
    for (int t = 0; t < PER; ++t) red[wave][lane + t * IA_WAVE] = o[t];
    __syncthreads();
    if (wave != 0) return;
    const float inv = 1.0f / s_total;
#pragma unroll
    for (int t = 0; t < PER; ++t) {
        const int e = lane + t * IA_WAVE;
        float sum = red[0][e];
        for (int w = 1; w < MERGE_WAVES; ++w) sum += red[w][e];
        if (e < HD) out[row * HD + e].bits = f32_to_bf16_bits(sum * inv);
    }
}

// The same merge for steps with many rows and few splits (portions of prompts, decode steps of many
// requests): a wave a row, every lane with the splits' maxima and sums of its row and HD / 64 features.
// Kernel times at head size 128, context 8,192, 32 heads (the block-a-row kernel against this one):
// 512 rows of 8 splits 4.9 against 7.6 us, 1,024 rows of 4 splits 7.0 against 5.1, 2,048 rows of 4 splits
// 12.2 against 5.0.
#define MERGE_ROWS_WAVES 4
#define MERGE_ROWS_FROM 1024
__global__ __launch_bounds__(MERGE_ROWS_WAVES * IA_WAVE) void attn_merge_rows_kernel(
    bf16_t* __restrict__ out, const float* __restrict__ part_o, const float* __restrict__ part_ml, int splits,
    size_t first_row, size_t n_rows) {
    constexpr int PER = (HD + IA_WAVE - 1) / IA_WAVE;
    const int lane = threadIdx.x & (IA_WAVE - 1), wave = threadIdx.x / IA_WAVE;
    const size_t local = (size_t)blockIdx.x * MERGE_ROWS_WAVES + wave;
    if (local >= n_rows) return;
    const size_t row = first_row + local;
    const float* ml = part_ml + row * splits * 2;
    const float* po = part_o + row * splits * HD;
    float mx = -INFINITY;
    for (int s = 0; s < splits; ++s) mx = fmaxf(mx, ml[2 * s]);
    float total = 0.f, o[PER];
#pragma unroll
    for (int t = 0; t < PER; ++t) o[t] = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float ms = ml[2 * s];
        const float w = ms == -INFINITY ? 0.f : exp2f(ms - mx);          // a split that held no key of this row
        total += ml[2 * s + 1] * w;
#pragma unroll
        for (int t = 0; t < PER; ++t) {
            const int e = lane + t * IA_WAVE;
            if (e < HD) o[t] = fmaf(po[(size_t)s * HD + e], w, o[t]);
        }
    }
    const float inv = 1.0f / total;
#pragma unroll
    for (int t = 0; t < PER; ++t) {
        const int e = lane + t * IA_WAVE;
        if (e < HD) out[row * HD + e].bits = f32_to_bf16_bits(o[t] * inv);
    }
}

extern "C" int ia_attention_mfma_head_dim(void) { return HD; }

// Floats of workspace that `splits` > 1 needs: partial outputs, then maxima and sums.
extern "C" long long ia_attention_mfma_workspace(int n, int nq, int splits) {
    return splits > 1 ? (long long)n * nq * splits * (HD + 2) : 0;
}

// The requests seq_begin .. seq_begin + n_seqs of the step, whose tokens are token_begin ..
// token_begin + n_tokens of its n.  max_q_len: the most tokens any of them has in this step;
// max_kv_len: their greatest length after it; `chunk`: keys per split (a multiple of 32,
// splits * chunk >= max_kv_len).  The workspace is sized for all n tokens.
struct FusedArgs {
    const void* qkv; const float* q_norm_w; const float* k_norm_w; const float* cos_t; const float* sin_t;
    const int* slots; float eps; int add_one;
    int* counters; int n_counters;
};

// Neighbouring splits that one block of the decode kernel takes (a wave each): four, or two where the waves'
// results for g query heads of a key/value head would not fit 64 KiB of shared memory.
static size_t decode_team_bytes(int team, int g) {
    const size_t waves = (size_t)team * (g < 16 ? g : 16) * (HD + 2), groups = (size_t)team * IA_WAVE * 6;   // (see the kernel's end)
    return (waves > groups ? waves : groups) * sizeof(float);
}
static int decode_team(int splits, int g) {
    const int team = decode_team_bytes(4, g) <= 65536 ? 4 : 2;
    return splits >= team ? team : splits;
}

// Floats of workspace that a decode step of `splits` key splits needs (one partial result a block), and the
// zeroed 32-bit counters (one for each request, key/value head and block of 16 query heads).
extern "C" long long ia_attention_decode_workspace(int n, int nq, int nkv, int splits) {
    if (n <= 0 || nq <= 0 || nkv <= 0 || splits <= 0) return 0;
    const int teams = splits / decode_team(splits, nq / nkv);
    return teams > 1 ? (long long)n * nq * teams * (HD + 2) : 0;
}
extern "C" long long ia_attention_decode_counters(int n, int nq, int nkv, int splits) {
    if (n <= 0 || nq <= 0 || nkv <= 0 || splits <= 0) return 0;
    const int teams = splits / decode_team(splits, nq / nkv);
    return teams > 1 ? (long long)n * nkv * ((nq / nkv + 15) / 16) : 0;
}

static int attention_launch(void* out, float* workspace, const void* q, const void* k_cache,
                            const void* v_cache, const int* block_table, const int* cu_tokens,
                            const int* positions, int n, int seq_begin, int n_seqs, int token_begin,
                            int n_tokens, int max_q_len, int max_kv_len, int max_pages,
                            int nq, int nkv, int d, int page_size, int window, float scale,
                            int splits, int chunk, const FusedArgs* fused, hipStream_t stream) {
    IA_CHECK(d == HD, "attention_mfma: built for head_dim %d, called with %d", HD, d);
    IA_CHECK(n >= 0 && n_seqs >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0,
             "attention_mfma: bad sizes n=%d seqs=%d nq=%d nkv=%d", n, n_seqs, nq, nkv);
    IA_CHECK(seq_begin >= 0 && token_begin >= 0 && n_tokens >= 0 && token_begin + n_tokens <= n,
             "attention_mfma: bad ranges seq_begin=%d tokens %d..+%d of %d", seq_begin, token_begin, n_tokens, n);
    IA_CHECK(page_size > 0 && page_size % 16 == 0, "attention_mfma: page size %d must be a multiple of 16", page_size);
    IA_CHECK(max_pages > 0 && window >= 0 && max_q_len >= 1, "attention_mfma: bad geometry max_pages=%d window=%d max_q_len=%d",
             max_pages, window, max_q_len);
    IA_CHECK(splits >= 1 && splits <= 256 &&
             (splits == 1 || ((workspace != nullptr || fused != nullptr) && chunk >= 32 && chunk % 32 == 0)),
             "attention_mfma: bad split of the keys (splits=%d chunk=%d)", splits, chunk);
    IA_CHECK((long long)nkv * splits <= 65535 && n_seqs <= 65535, "attention_mfma: grid too large (nkv*splits=%d seqs=%d)",
             nkv * splits, n_seqs);
    if (n_tokens == 0 || n_seqs == 0) return 0;
    const int g = nq / nkv;
    AttnParams p;
    p.out = (bf16_t*)out;
    p.part_o = workspace;
    p.part_ml = workspace ? workspace + (size_t)n * nq * splits * HD : nullptr;
    p.q = (const bf16_t*)q;
    p.k_cache = (const bf16_t*)k_cache;
    p.v_cache = (const bf16_t*)v_cache;
    p.k_cache_w = (bf16_t*)k_cache;
    p.v_cache_w = (bf16_t*)v_cache;
    p.qkv = nullptr; p.q_norm_w = p.k_norm_w = p.cos_t = p.sin_t = nullptr; p.slots = nullptr;
    p.norm_eps = 0.f; p.norm_add_one = 0;
    p.block_table = block_table;
    p.cu_tokens = cu_tokens;
    p.positions = positions;
    p.max_pages = max_pages; p.nq = nq; p.nkv = nkv; p.page = page_size; p.window = window;
    p.splits = splits; p.chunk = chunk; p.seq_begin = seq_begin; p.token_begin = token_begin;
    p.scale_log2 = scale * 1.4426950408889634f;
    const long long cols = (long long)max_q_len * g;
    // Columns a wave: 16 for decode, 32 for portions of prompts.  (64 keep every loaded key and
    // value in use for twice as many products but need the registers of a whole SIMD; with 32
    // two waves share a SIMD and one's matrix work overlaps the other's softmax, which is faster.)
    p.pair = (splits == 1 && cols > 16 && 2LL * max_q_len > max_kv_len) ? 1 : 0;
    const int nb = cols > 16 ? 2 : 1;
    const long long col_blocks = (cols + 16 * nb - 1) / (16 * nb);
    const dim3 grid((unsigned)(p.pair ? (col_blocks + 1) / 2 : col_blocks), nkv * splits, n_seqs);
    if (fused != nullptr) {
        IA_CHECK(HD % 64 == 0 && max_q_len == 1, "attention_mfma: the fused form takes single tokens and head sizes in "
                 "steps of 64 (head size %d, %d tokens a request)", HD, max_q_len);
        p.qkv = (const bf16_t*)fused->qkv;
        p.q_norm_w = fused->q_norm_w; p.k_norm_w = fused->k_norm_w;
        p.cos_t = fused->cos_t; p.sin_t = fused->sin_t; p.slots = fused->slots;
        p.norm_eps = fused->eps; p.norm_add_one = fused->add_one;
        // 16 columns a wave, whatever the number of query heads of a key/value head
        IA_CHECK(splits == 1 || (splits & (splits - 1)) == 0, "attention_mfma: the decode kernel splits the keys 2^k ways, not %d", splits);
        const int team = decode_team(splits, g), teams = splits / team;
        const int col_blocks = (g + 15) / 16;
        IA_CHECK(teams == 1 || workspace != nullptr, "attention_mfma: the decode kernel needs a workspace for %d blocks a request "
                 "and key/value head", teams);
        IA_CHECK(teams == 1 || (fused->counters != nullptr && (long long)n_seqs * nkv * col_blocks <= fused->n_counters),
                 "attention_mfma: the decode kernel needs %lld zeroed counters, got %d", (long long)n_seqs * nkv * col_blocks,
                 fused->counters ? fused->n_counters : 0);
        IA_CHECK((long long)nkv * teams <= 65535, "attention_mfma: grid too large (nkv*blocks=%d)", nkv * teams);
        p.part_ml = workspace ? workspace + (size_t)n * nq * teams * HD : nullptr;
        const dim3 fgrid((unsigned)col_blocks, nkv * teams, n_seqs);
        const size_t shared = team > 1 ? decode_team_bytes(team, g) : 0;
        attn_decode_kernel<><<<fgrid, team * IA_WAVE, shared, stream>>>(p, fused->counters, team);
        IA_LAUNCH_CHECK("attention_decode");
        return 0;
    } else if (HD == 128 && g_tiles && cols >= 16 * TILE_NBW * TILE_WAVES && (splits == 1 || chunk % TILE_STAGE == 0)) {
        // portions of prompts: blocks of four waves that share the keys through shared memory
        // Blocks of 128 columns; of 64 (twice as many, the same bits) where the keys are not split and the blocks of 128
        // would be half a compute unit's worth or less, or, under a causal mask over most of the context, where the
        // blocks' walks differ in length, one a compute unit or less.  Measured, 32 query and 8 key/value heads, whole
        // prompts: 512 tokens 17.8 -> 15.1 us, 1,024 tokens (256 blocks) 28.2 -> 24.5, 2,048 tokens (512 blocks) 55.8 -> 69.7
        // (not taken); 16 query heads: 1,024 tokens 25.8 -> 18.2, 2,048 tokens 44.4 -> 36.3; a portion of 512 tokens at a
        // context of 2,048: 42.3 -> 29.7 (36.8 with the keys split in two), with 40 query heads (160 blocks) 43.0 -> 47.9 (not taken).
        const long long tiles128 = (cols + 16 * TILE_NBW * TILE_WAVES - 1) / (16 * TILE_NBW * TILE_WAVES);
        const long long blocks128 = tiles128 * nkv * n_seqs;
        const bool causal_most = 2LL * max_q_len > max_kv_len;
        const bool narrow = g_tiles == 2 || (g_tiles == 1 && splits == 1 &&
                                             blocks128 <= (causal_most ? attn_cus() : attn_cus() / 2));
        const int tile_cols = 16 * (narrow ? 1 : TILE_NBW) * TILE_WAVES;
        const long long tiles = (cols + tile_cols - 1) / tile_cols;
        IA_CHECK(tiles <= 65535, "attention_mfma: %lld tiles of columns in a request (at most 65535)", tiles);
        const dim3 tgrid((unsigned)(nkv * splits * n_seqs), (unsigned)tiles, 1);
        p.pair = 0;
        if (narrow) attn_tile_kernel<(HD == 128), 1><<<tgrid, TILE_GROUPS * TILE_WAVES * IA_WAVE, 0, stream>>>(p);
        else attn_tile_kernel<><<<tgrid, TILE_GROUPS * TILE_WAVES * IA_WAVE, 0, stream>>>(p);
    } else if (nb == 1) {
        attn_mfma_kernel<1><<<grid, IA_WAVE, 0, stream>>>(p);
    } else {
        attn_mfma_kernel<2><<<grid, IA_WAVE, 0, stream>>>(p);
    }
    IA_LAUNCH_CHECK("attention_mfma");
    if (splits > 1) {
        const long long rows = (long long)n_tokens * nq;
        if (rows >= MERGE_ROWS_FROM && splits <= 16)
            attn_merge_rows_kernel<<<(unsigned)((rows + MERGE_ROWS_WAVES - 1) / MERGE_ROWS_WAVES), MERGE_ROWS_WAVES * IA_WAVE,
                                     0, stream>>>((bf16_t*)out, p.part_o, p.part_ml, splits, (size_t)token_begin * nq,
                                                  (size_t)rows);
        else
            attn_merge_kernel<<<(unsigned)rows, MERGE_WAVES * IA_WAVE, 0, stream>>>(
                (bf16_t*)out, p.part_o, p.part_ml, splits, (size_t)token_begin * nq);
        IA_LAUNCH_CHECK("attention_merge");
    }
    return 0;
}

extern "C" int ia_attention_mfma(void* out, float* workspace, const void* q, const void* k_cache,
                                 const void* v_cache, const int* block_table, const int* cu_tokens,
                                 const int* positions, int n, int seq_begin, int n_seqs, int token_begin,
                                 int n_tokens, int max_q_len, int max_kv_len, int max_pages,
                                 int nq, int nkv, int d, int page_size, int window, float scale,
                                 int splits, int chunk, hipStream_t stream) {
    return attention_launch(out, workspace, q, k_cache, v_cache, block_table, cu_tokens, positions, n, seq_begin,
                            n_seqs, token_begin, n_tokens, max_q_len, max_kv_len, max_pages, nq, nkv, d, page_size,
                            window, scale, splits, chunk, nullptr, stream);
}

// Whether this head size has the fused decode form.
extern "C" int ia_attention_mfma_has_fused(void) { return HD % 64 == 0 ? 1 : 0; }

// Decode steps, one token a request: the per-head norm of q and k (weights may be null: none), the rotation
// by each token's angles (cos, sin [n, d / 2], whole heads, halves paired; may be null: none) and the write
// of the new key and value at `slots` (may be null: nothing is written and the cache is only read) happen
// inside the attention kernel.  `qkv` [n, (nq + 2 nkv) * d] is the projections' output.
extern "C" int ia_attention_mfma_decode_fused(void* out, float* workspace, const void* qkv, void* k_cache,
                                              void* v_cache, const int* block_table, const int* cu_tokens,
                                              const int* positions, const int* slots, const float* q_norm_w,
                                              const float* k_norm_w, const float* cos_t, const float* sin_t,
                                              float eps, int add_one, int n, int seq_begin, int n_seqs,
                                              int token_begin, int n_tokens, int max_kv_len, int max_pages,
                                              int nq, int nkv, int d, int page_size, int window, float scale,
                                              int splits, int chunk, int* counters, int n_counters,
                                              hipStream_t stream) {
    IA_CHECK(qkv != nullptr && (q_norm_w == nullptr) == (k_norm_w == nullptr) && (cos_t == nullptr) == (sin_t == nullptr),
             "attention_mfma_decode_fused: qkv is needed; norm weights and angle tables come in pairs");
    IA_CHECK((((uintptr_t)qkv | (uintptr_t)q_norm_w | (uintptr_t)k_norm_w | (uintptr_t)cos_t | (uintptr_t)sin_t) & 15) == 0,
             "attention_mfma_decode_fused: arrays must be 16-byte aligned");
    IA_CHECK(n_seqs == n_tokens, "attention_mfma_decode_fused: one token a request (%d requests, %d tokens)", n_seqs, n_tokens);
    const FusedArgs fused = {qkv, q_norm_w, k_norm_w, cos_t, sin_t, slots, eps, add_one, counters, n_counters};
    return attention_launch(out, workspace, nullptr, k_cache, v_cache, block_table, cu_tokens, positions, n, seq_begin,
                            n_seqs, token_begin, n_tokens, 1, max_kv_len, max_pages, nq, nkv, d, page_size,
                            window, scale, splits, chunk, &fused, stream);
}
