// bfloat16 products for steps of 17 to 128 rows (decode steps of many requests, short prompt portions):
// out[M, N] = x[M, K] . w[N, K]^T, bound by reading the weights once, like the skinny product, but with so
// many rows that the activations can no longer be fetched by every wave for itself (at 64 rows they are as
// large as a block's share of the weights).  65 to 128 rows (six or eight tiles of rows) walk k in chunks of 64, four
// stages deep, so that the stages still fit a compute unit's shared memory.  From 49 rows on a wave takes two tiles of
// weight rows over half of the step's rows where a block has an even number of waves (PAIRED below): at 128 rows six
// operand reads from shared memory for eight matrix products instead of nine, in the same time that the memory takes to
// deliver the weights.  A [gate; up] whose blocks fill the chip evenly comes here with fewer rows
// too (ia_gemm_mid_bf16_scaled: rows of a residual stream whose norm the product finishes).
//
// The reference hands these products to cuBLAS like all others (`candle-core/src/cuda_backend/mod.rs:2260-2305`).
//
// A block of W waves (2 to 8) owns 16 W rows of w and a range of k, and walks it in chunks of 128, each block from another
// place of its range (blocks that are started together and walk in step ask the same few memory channels at any moment).
// A stage of shared memory holds a chunk's rows of x (up to 64) and the block's rows of w alike, 256 bytes a row, brought by
// all waves together straight from memory (global_load_lds: 16 bytes a lane, four whole rows an instruction, no register on
// the way), one or two stages ahead of their use.  A wave multiplies its tile of 16 weight rows (the MFMA A-operand:
// v_mfma_f32_16x16x32_bf16, lane l supplies row l % 16 with the eight k values 8 * (l / 16) .. + 8) with every row tile of
// x, both read from the stage.  Piece c (16 bytes) of row r lies at place c ^ (r % 16) of the row's 256 bytes, so that the
// 16 rows which one operand read takes at the same k fall on 16 different places; a load instruction fills 1 KiB (four
// rows) in lane order, and the lane picks the piece it fetches accordingly.
//
// How many waves a block has and how k is split follow from the weight's shape (mid_plan below): the chip should get a block
// for every compute unit and no more, three stages deep; a weight that no such shape fits takes four waves a block, two
// stages and several blocks a unit.
//
// The weights went straight from memory into the A-operands before (a load of 16 rows x 64 bytes a lane group): such a
// load holds the compute unit's address unit for about 86 cycles, a load of 1 KiB in whole rows for about 32, and by its
// own clocks that kernel spent 40 % of a step issuing its loads at 64 rows.  Through shared memory: q|k|v of 6,144 x
// 4,096 at 64 rows 17.1 -> 14.5 us, [gate; up] with the activation 56 -> 50, the 32B shape's 5,120 x 25,600 82 -> 69.
//
// With few rows of w (the output projection, the feed-forward's second product) whole columns of k leave too few
// blocks to fill the chip, so k is split between blocks (gridDim.y) and every split leaves its sums in 32-bit:
// [splits][M][N].  They are added up, in the order of the splits, by whoever reads them: the kernel that adds a
// product to the residual stream and norms it (ia_add_rmsnorm_partials), or ia_sum_partials.  The split depends
// on the weight's shape alone, never on the rows of the step.
//
// DUAL: w = [gate; up] (N rows each); a block owns 8 W output features, the first half of its waves their gate rows, the
// second half their up rows, and the result is silu(gate . x) * (up . x), the first product rounded to bfloat16 before the
// activation as the two-kernel path rounds it.  No split of k (the activation needs whole sums).
#include <type_traits>

#include "common.h"
#include "api.h"

typedef __bf16 gmid_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gmid_f32x4 __attribute__((ext_vector_type(4)));

#define MID_CHUNK_MIN_K 128               // k is shared out in multiples of this

// s_waitcnt that waits until at most n vector-memory operations of this wave are under way (gfx9 encoding:
// vmcnt in bits 3:0 and 15:14; the other counters left alone).
#define MID_VMCNT(n) (((n) & 15) | ((((n) >> 4) & 3) << 14) | (7 << 4) | (15 << 8))

enum { MID_OUT_BF16 = 0, MID_OUT_F32 = 1, MID_OUT_PARTIAL = 2 };

// The end of the kernel.  Lane (r, g) holds features n_first + 4 g + i of row 16 mt + r.  DUAL: the up rows' sums go through
// shared memory (swap_up, in a stage's place) to the waves that hold the gate rows' sums of the same features.
template <int MT, bool DUAL, int TILES>
__device__ __forceinline__ void mid_finish(gmid_f32x4 (&acc)[MT], gmid_f32x4* swap_up, void* out, int out_mode,
                                           int M, int N, int lane, int r, int g, int tile, int part, int n_first, int split,
                                           int act) {
    constexpr int FEATURE_TILES = DUAL ? TILES / 2 : TILES;
    if (DUAL) __syncthreads();                                            // everybody is done with the stages
    if (DUAL) {
        if (part == 1) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) swap_up[((tile % FEATURE_TILES) * MT + mt) * IA_WAVE + lane] = acc[mt];
        }
        __syncthreads();
        if (part != 0) return;
        const int nb = n_first + 4 * g;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            if (m >= M) continue;
            const gmid_f32x4 up = swap_up[(tile * MT + mt) * IA_WAVE + lane];
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float gate = bf16_bits_to_f32(f32_to_bf16_bits(acc[mt][i]));
                const float u = bf16_bits_to_f32(f32_to_bf16_bits(up[i]));
                v[i] = gate_act(gate, act) * u;
            }
            bf16_t* o = (bf16_t*)out + (size_t)m * N + nb;
            if (nb + 3 < N && (N & 3) == 0) {
                *(uint2*)o = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (nb + i < N) o[i].bits = f32_to_bf16_bits(v[i]);
            }
        }
        return;
    }
    const int nb = n_first + 4 * g;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        if (m >= M) continue;
        if (out_mode == MID_OUT_BF16) {
            bf16_t* o = (bf16_t*)out + (size_t)m * N + nb;
            if (nb + 3 < N && (N & 3) == 0) {
                *(uint2*)o = make_uint2(pack_bf16x2(acc[mt][0], acc[mt][1]), pack_bf16x2(acc[mt][2], acc[mt][3]));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (nb + i < N) o[i].bits = f32_to_bf16_bits(acc[mt][i]);
            }
        } else {
            float* o = (float*)out + ((size_t)(out_mode == MID_OUT_PARTIAL ? split : 0) * M + m) * N + nb;
            if (nb + 3 < N && (N & 3) == 0) {
                *(gmid_f32x4*)o = acc[mt];
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (nb + i < N) o[i] = acc[mt][i];
            }
        }
    }
}

// The end of the kernel for waves that hold two tiles of weight rows over MH tiles of rows from tile mt_first on
// (PAIRED below).  DUAL: the two are the gate rows and the up rows of the same 16 features from n_first on, so nothing is
// exchanged; otherwise the features n_first .. + 32.  The arithmetic is mid_finish's.
template <int MH, bool DUAL>
__device__ __forceinline__ void mid_finish_paired(gmid_f32x4 (&acc0)[MH], gmid_f32x4 (&acc1)[MH], void* out, int out_mode,
                                                  int M, int N, int r, int g, int mt_first, int n_first, int split, int act) {
#pragma unroll
    for (int mt = 0; mt < MH; ++mt) {
        const int m = (mt_first + mt) * 16 + r;
        if (m >= M) continue;
        if (DUAL) {
            const int nb = n_first + 4 * g;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float gate = bf16_bits_to_f32(f32_to_bf16_bits(acc0[mt][i]));
                const float u = bf16_bits_to_f32(f32_to_bf16_bits(acc1[mt][i]));
                v[i] = gate_act(gate, act) * u;
            }
            bf16_t* o = (bf16_t*)out + (size_t)m * N + nb;
            if (nb + 3 < N && (N & 3) == 0) {
                *(uint2*)o = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (nb + i < N) o[i].bits = f32_to_bf16_bits(v[i]);
            }
            continue;
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const gmid_f32x4 a = t == 0 ? acc0[mt] : acc1[mt];
            const int nb = n_first + 16 * t + 4 * g;
            if (out_mode == MID_OUT_BF16) {
                bf16_t* o = (bf16_t*)out + (size_t)m * N + nb;
                if (nb + 3 < N && (N & 3) == 0) {
                    *(uint2*)o = make_uint2(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]));
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (nb + i < N) o[i].bits = f32_to_bf16_bits(a[i]);
                }
            } else {
                float* o = (float*)out + ((size_t)(out_mode == MID_OUT_PARTIAL ? split : 0) * M + m) * N + nb;
                if (nb + 3 < N && (N & 3) == 0) {
                    *(gmid_f32x4*)o = a;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (nb + i < N) o[i] = a[i];
                }
            }
        }
    }
}

// KC: k steps of 32 in a chunk (a staged row is KC * 64 bytes); NS: stages, this chunk's and NS - 1 on their way; W: waves of
// a block, a tile of 16 weight rows each (DUAL: W / 2 of gate rows, then W / 2 of up rows).
// PAIRED: a wave multiplies two tiles of weight rows (DUAL: the gate rows and the up rows of the same features) with half of
// the tiles of x, the block's first W / 2 waves with the first half and the others with the second: 2 + MT / 2 operand reads
// from shared memory for MT matrix products instead of 1 + MT, and every sum in the same order.
template <int MT, bool DUAL, int KC, int NS, int W, bool PAIRED = false>
__global__ __launch_bounds__(W * IA_WAVE) void gemm_mid_kernel(
    void* __restrict__ out, int out_mode, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
    int M, int N, int K, int k_per_block, const float* __restrict__ sums_in, int n_sums, float eps, int act) {
    constexpr int CHUNK_K = KC * 32;
    constexpr int ROW_BYTES = KC * 64;
    constexpr int ROWS_PER_LOAD = 1024 / ROW_BYTES;
    constexpr int PIECES = KC * 4;
    constexpr int TILES = W;
    constexpr int X_ROWS = MT * 16;
    constexpr int W_ROWS = TILES * 16;
    constexpr int ROWS = X_ROWS + W_ROWS;
    constexpr int ROW_LOADS = ROWS / ROWS_PER_LOAD;         // load instructions (1 KiB each) that a stage's rows take
    constexpr int LOADS = (ROW_LOADS + W - 1) / W;          // load instructions a wave issues for a stage; where they do not
    constexpr int STAGE_BYTES = LOADS * W * 1024;           // divide, the last ones fetch a row of x again into a place nobody reads
    static_assert(!DUAL || W % 2 == 0, "gate and up rows: an even number of waves");
    static_assert(!PAIRED || (W % 2 == 0 && MT % 2 == 0), "pairs of tiles over halves of the rows: even numbers of both");
    static_assert(NS >= 2 && NS <= 4 && (KC == 2 || KC == 4), "pipeline shape");
    constexpr int MH = PAIRED ? MT / 2 : MT;                // tiles of rows a wave multiplies
    constexpr int PAIRS = W / 2;
    __shared__ __attribute__((aligned(1024))) char mid_s0[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char mid_s1[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char mid_s2[NS > 2 ? STAGE_BYTES : 16];
    __shared__ __attribute__((aligned(1024))) char mid_s3[NS > 3 ? STAGE_BYTES : 16];
    auto stage_of = [&](auto stage_c) -> char* {
        constexpr int S = decltype(stage_c)::value;
        if constexpr (S == 0) return mid_s0;
        else if constexpr (S == 1) return mid_s1;
        else if constexpr (S == 2) return mid_s2;
        else return mid_s3;
    };
    const int lane = threadIdx.x & (IA_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / IA_WAVE);
    const int r = lane & 15, g = lane >> 4;
    const int tile = wave;
    const int split = blockIdx.y;
    const int k_begin = split * k_per_block;
    const int k_len = K - k_begin < k_per_block ? K - k_begin : k_per_block;
    const int nchunks = k_len / CHUNK_K;
    constexpr int FEATURE_TILES = DUAL ? TILES / 2 : TILES;
    const int part = DUAL ? tile / FEATURE_TILES : 0;
    const int n_first = blockIdx.x * (16 * FEATURE_TILES) + 16 * (tile % FEATURE_TILES);
    // PAIRED: the wave's two tiles of weight rows and the first of its tiles of x
    const int pair = PAIRED ? wave % PAIRS : 0;
    const int mt_first = PAIRED ? (wave / PAIRS) * MH : 0;
    const int tile0 = PAIRED ? (DUAL ? pair : 2 * pair) : tile;
    const int tile1 = PAIRED ? (DUAL ? FEATURE_TILES + pair : 2 * pair + 1) : tile;
    // rows 16 t + i of a stage's 256-byte (or 128-byte) rows collide on the same banks for every i: a row's pieces are
    // exchanged so that 16 rows at the same k fall on different places
    auto swizzle = [](int row) { return KC == 4 ? (row & 15) : ((row >> 1) & 7); };

    // ---- rows that come scaled by a norm's weight, with their sums of squares block by block (sums_in [M][n_sums]; one tile
    // of rows): every sum of the product is multiplied by the row's rsqrt(mean of squares + eps) before it is rounded.  The
    // sums of squares are asked for now, before any stage (loads return in order: they are there when the stages are),
    // a row a wave, and added up at the end in the order of the skinny product (a lane's four neighbours, its second four,
    // then across the lanes), so that a row gets the same scale from both kernels.
    constexpr int SS_ROWS = (16 + W - 1) / W;
    float4 ss_mine[MT == 1 ? SS_ROWS : 1][2];
    const bool ss_wide = MT == 1 && sums_in != nullptr && (n_sums & 3) == 0 && n_sums <= 8 * IA_WAVE;
    if constexpr (MT == 1) {
        if (ss_wide) {
#pragma unroll
            for (int j = 0; j < SS_ROWS; ++j) {
                const int m = wave + j * W;
#pragma unroll
                for (int v = 0; v < 2; ++v) {
                    const int at = 4 * (lane + v * IA_WAVE);
                    ss_mine[j][v] = (m < M && at < n_sums) ? *(const float4*)(sums_in + (size_t)m * n_sums + at)
                                                           : make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        }
    }
    __shared__ float mid_ss[16];

    // ---- what this lane fetches of a stage: load i covers rows ROWS_PER_LOAD * (W i + wave) .. of the stage ----
    const char* src[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int row = ROWS_PER_LOAD * (W * i + wave) + lane / PIECES;              // row of the stage
        const int piece = (lane % PIECES) ^ swizzle(row);
        const bf16_t* base;
        if (row < X_ROWS || row >= ROWS) {
            base = x + (size_t)(row < M ? row : 0) * K;                   // (rows beyond the step read row 0: never stored)
        } else {
            const int wr = row - X_ROWS, t = wr / 16;                          // weight row of the block: tile t, row wr % 16
            const int pt = DUAL ? t / FEATURE_TILES : 0;
            const int n = blockIdx.x * (16 * FEATURE_TILES) + 16 * (t % FEATURE_TILES) + (wr & 15);
            base = w + ((size_t)pt * N + (n < N ? n : N - 1)) * K;        // (rows beyond the matrix: never stored)
        }
        src[i] = (const char*)(base + k_begin) + piece * 16;
    }
    uint32_t a_at[KC], a1_at[KC], b_at[KC];
#pragma unroll
    for (int ks = 0; ks < KC; ++ks) {
        const uint32_t in_tile = (uint32_t)(r * ROW_BYTES + (((4 * ks + g) ^ swizzle(r)) * 16));
        b_at[ks] = (uint32_t)(mt_first * 16 * ROW_BYTES) + in_tile;
        a_at[ks] = (uint32_t)((X_ROWS + 16 * tile0) * ROW_BYTES) + in_tile;
        a1_at[ks] = (uint32_t)((X_ROWS + 16 * tile1) * ROW_BYTES) + in_tile;
    }
    gmid_f32x4 acc[MH], acc1[PAIRED ? MH : 1];
#pragma unroll
    for (int mt = 0; mt < MH; ++mt) acc[mt] = (gmid_f32x4){0.f, 0.f, 0.f, 0.f};
    if constexpr (PAIRED) {
#pragma unroll
        for (int mt = 0; mt < MH; ++mt) acc1[mt] = (gmid_f32x4){0.f, 0.f, 0.f, 0.f};
    }
    // Blocks start at different places of their range of k and wrap around: blocks that are started together and walk k in
    // step ask the same few memory channels at any moment (rows are a power of two apart).  The order of a sum depends
    // on the block, that is on the output feature, never on the step's rows.
    // (in steps of 128 k whatever the chunk, so that every pipeline shape adds up in the same order)
    const int rot = k_len >= MID_CHUNK_MIN_K
        ? (int)((blockIdx.x * 5u + blockIdx.y * 3u) % (unsigned)(k_len / MID_CHUNK_MIN_K)) * (MID_CHUNK_MIN_K / CHUNK_K) : 0;

    auto issue = [&](auto stage_c, int c) {
        char* stage = stage_of(stage_c);
        const int cc = c + rot < nchunks ? c + rot : c + rot - nchunks;
#pragma unroll
        for (int i = 0; i < LOADS; ++i)
            __builtin_amdgcn_global_load_lds(
                (const void __attribute__((address_space(1)))*)(src[i] + (size_t)cc * ROW_BYTES),
                (void __attribute__((address_space(3)))*)(stage + (W * i + wave) * 1024), 16, 0, 0);
    };
    auto multiply = [&](auto stage_c) {
        const char* stage = stage_of(stage_c);
#pragma unroll
        for (int ks = 0; ks < KC; ++ks) {
            const uint4 a = *(const uint4*)(stage + a_at[ks]);
            uint4 a1 = a;
            if constexpr (PAIRED) a1 = *(const uint4*)(stage + a1_at[ks]);
#pragma unroll
            for (int mt = 0; mt < MH; ++mt) {
                const uint4 b = *(const uint4*)(stage + mt * (16 * ROW_BYTES) + b_at[ks]);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(gmid_bf16x8, a), __builtin_bit_cast(gmid_bf16x8, b), acc[mt], 0, 0, 0);
                if constexpr (PAIRED)
                    acc1[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(gmid_bf16x8, a1), __builtin_bit_cast(gmid_bf16x8, b), acc1[mt], 0, 0, 0);
            }
        }
    };
    auto full_step = [&](auto stage_c, int c) {              // chunks c + 1 .. c + NS - 1 exist
        constexpr int S = decltype(stage_c)::value;
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(MID_VMCNT((NS - 2) * LOADS));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        issue(std::integral_constant<int, (S + NS - 1) % NS>(), c + NS - 1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(stage_c);
    };
    auto last_step = [&](auto stage_c, int c) {              // the last NS - 1 chunks: nothing left to ask for
        __builtin_amdgcn_sched_barrier(0);
        if (NS > 3 && c + 2 < nchunks) __builtin_amdgcn_s_waitcnt(MID_VMCNT(2 * LOADS));
        else if (NS > 2 && c + 1 < nchunks) __builtin_amdgcn_s_waitcnt(MID_VMCNT(LOADS));
        else __builtin_amdgcn_s_waitcnt(MID_VMCNT(0));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        multiply(stage_c);
    };
    auto ring = [&](auto fn, int c) {
        fn(std::integral_constant<int, 0>(), c);
        fn(std::integral_constant<int, 1>(), c + 1);
        if constexpr (NS > 2) fn(std::integral_constant<int, 2>(), c + 2);
        if constexpr (NS > 3) fn(std::integral_constant<int, 3>(), c + 3);
    };
    int c = 0;
    if (nchunks >= 2 * NS - 1) {
        issue(std::integral_constant<int, 0>(), 0);
        if constexpr (NS > 2) issue(std::integral_constant<int, 1>(), 1);
        if constexpr (NS > 3) issue(std::integral_constant<int, 2>(), 2);
        for (; c + 2 * NS - 1 <= nchunks; c += NS) ring(full_step, c);
    } else {
        if (nchunks > 0) issue(std::integral_constant<int, 0>(), 0);
        if constexpr (NS > 2) { if (nchunks > 1) issue(std::integral_constant<int, 1>(), 1); }
        if constexpr (NS > 3) { if (nchunks > 2) issue(std::integral_constant<int, 2>(), 2); }
    }
    auto tail_step = [&](auto stage_c, int cc) {
        if (cc >= nchunks) return;
        if (cc + NS - 1 < nchunks) full_step(stage_c, cc);
        else last_step(stage_c, cc);
    };
    ring(tail_step, c);
    ring(tail_step, c + NS);
    static_assert(!DUAL || FEATURE_TILES * MT * IA_WAVE * sizeof(gmid_f32x4) <= STAGE_BYTES, "the up rows' sums fit a stage");
    static_assert(NS * STAGE_BYTES <= 160 * 1024, "the stages fit a compute unit's shared memory");
    if constexpr (MT == 1) {
        if (sums_in != nullptr) {
#pragma unroll
            for (int j = 0; j < SS_ROWS; ++j) {
                const int m = wave + j * W;
                if (m >= M) continue;
                float ss = 0.f;
                if (ss_wide) {
                    ss = ((ss_mine[j][0].x + ss_mine[j][0].y) + ss_mine[j][0].z) + ss_mine[j][0].w;
                    ss += ((ss_mine[j][1].x + ss_mine[j][1].y) + ss_mine[j][1].z) + ss_mine[j][1].w;
                } else {
                    for (int b = lane; b < n_sums; b += IA_WAVE) ss += sums_in[(size_t)m * n_sums + b];
                }
                ss = wave_sum(ss);
                if (lane == 0) mid_ss[m] = ss;
            }
            __syncthreads();
            const float scale = 1.0f / sqrtf(mid_ss[r < M ? r : 0] / (float)K + eps);
            acc[0][0] *= scale; acc[0][1] *= scale; acc[0][2] *= scale; acc[0][3] *= scale;
        }
    }
    if constexpr (PAIRED) {
        const int n_pair = blockIdx.x * (16 * FEATURE_TILES) + (DUAL ? 16 : 32) * pair;
        mid_finish_paired<MH, DUAL>(acc, acc1, out, out_mode, M, N, r, g, mt_first, n_pair, split, act);
    } else {
        mid_finish<MT, DUAL, TILES>(acc, (gmid_f32x4*)mid_s1, out, out_mode, M, N, lane, r, g, tile, part, n_first, split, act);
    }
}

// How a weight is shared out: a function of its shape and the chip alone, never of the rows of the step.
//   waves  tiles of 16 weight rows a block (DUAL: half of them gate rows, half the up rows of the same features)
//   splits ways k is split between blocks (gridDim.y); the splits' sums are added up by the reader
//   stages of the pipeline
// Wanted: a block for every compute unit and no more, three stages deep (a block a unit: what it has under way is all that
// hides the memory's latency; two rounds of blocks would leave the second half empty).  Among the ways that fill nine
// tenths of the chip, the one with the most waves a block wins (the rows of x are fetched once a block) as long as a block
// keeps eight chunks of k.  A weight that no way fits (a logits head: thousands of blocks) takes four waves a block two stages
// deep, several blocks a unit, k split until there is a block for every unit.
static int mid_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    return cus;
}

struct MidPlan { int waves, splits, stages; };
// a plan for measurements and tests: waves (0: the rule), splits, stages
static MidPlan g_mid_forced = {0, 0, 0};
#define MID_MAX_WAVES 8
extern "C" int ia_gemm_mid_plan(int waves, int splits, int stages) {
    IA_CHECK(waves == 0 || (waves >= 2 && waves <= MID_MAX_WAVES && splits >= 1 && splits <= 16 && (splits & (splits - 1)) == 0
                            && (stages == 3 || (waves == 4 && stages == 2))),
             "gemm_mid_plan: no block of %d waves with %d splits of k, %d stages deep (2 to 8 waves, 2^k splits up to 16, "
             "3 stages, or 4 waves with 2; 0 waves: the plan's own)", waves, splits, stages);
    g_mid_forced = {waves, splits, stages};
    return 0;
}

static MidPlan mid_plan(int N, int K, bool dual) {
    const int cus = mid_cus();
    const int tiles = (N + 15) / 16;                       // of a part
    const int chunks = K / MID_CHUNK_MIN_K;
    if (g_mid_forced.waves > 0) return g_mid_forced;
    MidPlan best = {0, 0, 0};
    double best_fill = 0.0;
    bool best_long = false;
    for (int t = 1; t <= (dual ? MID_MAX_WAVES / 2 : MID_MAX_WAVES); ++t) {
        if (!dual && t < 2) continue;
        const int blocks = (tiles + t - 1) / t;
        for (int splits = 1; splits <= (dual ? 1 : 16); splits *= 2) {
            if (chunks % splits || chunks / splits < 4) break;
            if ((long long)blocks * splits > cus) break;
            // the share of the chip's compute units that get a block, times the share of a block's tiles that are real
            const double fill = (double)blocks * splits / cus * ((double)tiles / ((double)blocks * t));
            const bool is_long = chunks / splits >= 8;
            const bool better = fill > best_fill + 0.02 || (fill > best_fill - 0.02 && (is_long || !best_long));
            if (best.waves == 0 || better) {
                best = {dual ? 2 * t : t, splits, 3};
                best_fill = fill > best_fill ? fill : best_fill;
                best_long = is_long;
            }
        }
    }
    if (best.waves != 0 && best_fill >= 0.9) return best;
    MidPlan wide = {4, 1, 2};
    if (!dual) {
        const int blocks = (N + 63) / 64;
        while (blocks * wide.splits < cus && wide.splits < 16 && chunks % (2 * wide.splits) == 0 && chunks / (2 * wide.splits) >= 4)
            wide.splits *= 2;
    }
    return wide;
}

// Whether the weight's blocks fill the chip evenly, one a compute unit, three stages deep (dual: [gate; up] of N features).
extern "C" int ia_gemm_mid_fills(int N, int K, int dual) {
    if (N <= 0 || K <= 0 || K % MID_CHUNK_MIN_K) return 0;
    return mid_plan(N, K, dual != 0).stages == 3;
}

extern "C" int ia_gemm_mid_splits(int N, int K) {
    if (N <= 0 || K <= 0 || K % MID_CHUNK_MIN_K) return 0;
    return mid_plan(N, K, false).splits;
}

// ia_gemm_mid_tune(kc, ns): a fixed pipeline of four waves a block for tests (chunks of kc k steps, 2 or 4, ns deep;
// 0, 0: the plan's own).  Every pipeline adds an output's products up in the same order; plans differ in where a block
// starts its walk of k.
static int g_mid_kc = 0, g_mid_ns = 0;
extern "C" int ia_gemm_mid_tune(int kc, int ns) {
    IA_CHECK((kc == 0 && ns == 0) || (kc == 4 && ns == 2) || (kc == 2 && (ns == 3 || ns == 4)),
             "gemm_mid_tune: no pipeline of chunks of %d k steps, %d deep (4 x 2, 2 x 3, 2 x 4, or 0, 0 for the plan's own)", kc, ns);
    g_mid_kc = kc;
    g_mid_ns = ns;
    return 0;
}

// ia_gemm_mid_blocking(how): 0 the rule (two tiles of weight rows a wave over half of the rows where a step has more than
// 48 rows and the block an even number of waves), 1 a tile a wave over all rows, always, 2 pairs wherever they can be.
// For measurements and tests: both give the same bits.
static int g_mid_blocking = 0;
extern "C" int ia_gemm_mid_blocking(int how) {
    IA_CHECK(how >= 0 && how <= 2, "gemm_mid_blocking: 0 (the rule), 1 (a tile a wave) or 2 (pairs), got %d", how);
    g_mid_blocking = how;
    return 0;
}

template <int MT, bool DUAL>
static int launch_mid(void* out, int out_mode, const bf16_t* x, const bf16_t* w, int M, int N, int K, int splits,
                      const float* sums_in, int n_sums, float eps, int act, hipStream_t stream) {
    MidPlan plan = mid_plan(N, K, DUAL);
    if (out_mode != MID_OUT_PARTIAL && !DUAL && plan.splits != 1) {
        // a stored product cannot be split: four waves a block over all of k
        plan = {4, 1, 2};
    }
    if (g_mid_kc != 0 && MT <= 4) plan = {4, DUAL || out_mode != MID_OUT_PARTIAL ? 1 : plan.splits, g_mid_ns};
    const int kc = g_mid_kc != 0 ? g_mid_kc : 4;
    IA_CHECK(plan.splits == splits, "gemm_mid: the plan's %d splits against the caller's %d", plan.splits, splits);
    const int features = 16 * plan.waves / (DUAL ? 2 : 1);            // output features of a block
    const dim3 grid((N + features - 1) / features, splits);
    // every block's share of k is whole chunks (a share that is not would lose its tail and start off the loads' alignment)
    IA_CHECK(splits >= 1 && K % (splits * MID_CHUNK_MIN_K) == 0, "gemm_mid: K=%d does not split %d ways in multiples of %d",
             K, splits, MID_CHUNK_MIN_K);
    IA_CHECK(plan.waves >= 2 && plan.waves <= MID_MAX_WAVES, "gemm_mid: a block of %d waves", plan.waves);
    const int k_block = K / splits;
#define MID_SHAPE(KC, NS, W) gemm_mid_kernel<MT, DUAL, KC, NS, W><<<grid, W * IA_WAVE, 0, stream>>>(out, out_mode, x, w, M, N, K, k_block, sums_in, n_sums, eps, act)
#define MID_PAIRED(KC, NS, W) gemm_mid_kernel<MT, DUAL, KC, NS, W, true><<<grid, W * IA_WAVE, 0, stream>>>(out, out_mode, x, w, M, N, K, k_block, sums_in, n_sums, eps, act)
    if constexpr (MT > 4) {
        // more than 64 rows: chunks of 64 k, four stages deep, whatever the plan's depth
        if (g_mid_blocking != 1) {
            switch (plan.waves) {
                case 2: MID_PAIRED(2, 4, 2); return 0;
                case 4: MID_PAIRED(2, 4, 4); return 0;
                case 6: MID_PAIRED(2, 4, 6); return 0;
                case 8: MID_PAIRED(2, 4, 8); return 0;
            }
        }
        switch (plan.waves) {
            case 2: MID_SHAPE(2, 4, 2); return 0;
            case 4: MID_SHAPE(2, 4, 4); return 0;
            case 6: MID_SHAPE(2, 4, 6); return 0;
            case 8: MID_SHAPE(2, 4, 8); return 0;
        }
        if constexpr (!DUAL) {
            switch (plan.waves) {
                case 3: MID_SHAPE(2, 4, 3); return 0;
                case 5: MID_SHAPE(2, 4, 5); return 0;
                case 7: MID_SHAPE(2, 4, 7); return 0;
            }
        }
    } else if (kc == 4 && plan.stages == 3) {
        if constexpr (MT == 4 || MT == 2) {
            if (MT == 4 ? g_mid_blocking != 1 : g_mid_blocking == 2) {
                switch (plan.waves) {
                    case 2: MID_PAIRED(4, 3, 2); return 0;
                    case 4: MID_PAIRED(4, 3, 4); return 0;
                    case 6: MID_PAIRED(4, 3, 6); return 0;
                    case 8: MID_PAIRED(4, 3, 8); return 0;
                }
            }
        }
        switch (plan.waves) {
            case 2: MID_SHAPE(4, 3, 2); return 0;
            case 4: MID_SHAPE(4, 3, 4); return 0;
            case 6: MID_SHAPE(4, 3, 6); return 0;
            case 8: MID_SHAPE(4, 3, 8); return 0;
        }
        if constexpr (!DUAL) {
            switch (plan.waves) {
                case 3: MID_SHAPE(4, 3, 3); return 0;
                case 5: MID_SHAPE(4, 3, 5); return 0;
                case 7: MID_SHAPE(4, 3, 7); return 0;
            }
        }
    } else if (plan.waves == 4) {
        if (kc == 4 && plan.stages == 2) { MID_SHAPE(4, 2, 4); return 0; }
        if (kc == 2 && plan.stages == 3) { MID_SHAPE(2, 3, 4); return 0; }
        if (kc == 2 && plan.stages == 4) { MID_SHAPE(2, 4, 4); return 0; }
    }
#undef MID_SHAPE
#undef MID_PAIRED
    IA_CHECK(false, "gemm_mid: no pipeline of %d waves, chunks of %d k steps, %d deep", plan.waves, kc, plan.stages);
    return 0;
}

// out_mode 0: out [M, N] bfloat16; 1: out [M, N] float; 2: out [splits][M][N] float with splits =
// ia_gemm_mid_splits(N, K), to be added up by the reader.  dual (an activation, IA_ACT_*): w = [gate; up] of N rows each, out = act(x . gate^T)
// * (x . up^T) in bfloat16 (mode 0 only).  M in 1..128, K a multiple of 128.
// sums_in [M][n_sums] (or null): the rows of x are a norm's input times its weight, and every sum of the product is multiplied by
// the row's rsqrt(sum of its sums_in / K + eps); up to 16 rows, whole sums only (no split of k).
extern "C" int ia_gemm_mid_bf16_scaled(void* out, const void* x, const void* w, int M, int N, int K, int out_mode, int dual,
                                       const float* sums_in, int n_sums, float eps, hipStream_t stream) {
    IA_CHECK(sums_in == nullptr || (M <= 16 && n_sums > 0 && out_mode != MID_OUT_PARTIAL && (((uintptr_t)sums_in) & 15) == 0),
             "gemm_mid: rows with their sums of squares: up to 16 rows, whole sums (M=%d, n_sums=%d, mode %d)", M, n_sums, out_mode);
    IA_CHECK(M >= 1 && M <= 128 && N > 0 && K > 0, "gemm_mid: takes 1 to 128 rows, got M=%d N=%d K=%d", M, N, K);
    IA_CHECK(K % MID_CHUNK_MIN_K == 0, "gemm_mid: K=%d must be a multiple of %d (use another product)", K, MID_CHUNK_MIN_K);
    IA_CHECK(out_mode >= 0 && out_mode <= 2 && (!dual || out_mode == MID_OUT_BF16), "gemm_mid: output mode %d%s", out_mode,
             dual ? " does not go with the activation inside" : " is unknown");
    IA_CHECK(dual >= 0 && dual <= IA_ACT_LAST, "gemm_mid: unknown activation %d", dual);
    IA_CHECK((((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15) == 0, "gemm_mid: operands must be 16-byte aligned");
    const int splits = out_mode == MID_OUT_PARTIAL && !dual ? mid_plan(N, K, false).splits : 1;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    const int mt = (M + 15) / 16;
    int rc = 0;
    if (dual) {
        if (mt == 1) rc = launch_mid<1, true>(out, out_mode, xb, wb, M, N, K, 1, sums_in, n_sums, eps, dual, stream);
        else if (mt == 2) rc = launch_mid<2, true>(out, out_mode, xb, wb, M, N, K, 1, sums_in, n_sums, eps, dual, stream);
        else if (mt == 3) rc = launch_mid<3, true>(out, out_mode, xb, wb, M, N, K, 1, sums_in, n_sums, eps, dual, stream);
        else if (mt == 4) rc = launch_mid<4, true>(out, out_mode, xb, wb, M, N, K, 1, sums_in, n_sums, eps, dual, stream);
        else if (mt <= 6) rc = launch_mid<6, true>(out, out_mode, xb, wb, M, N, K, 1, sums_in, n_sums, eps, dual, stream);
        else rc = launch_mid<8, true>(out, out_mode, xb, wb, M, N, K, 1, sums_in, n_sums, eps, dual, stream);
    } else {
        if (mt == 1) rc = launch_mid<1, false>(out, out_mode, xb, wb, M, N, K, splits, sums_in, n_sums, eps, dual, stream);
        else if (mt == 2) rc = launch_mid<2, false>(out, out_mode, xb, wb, M, N, K, splits, sums_in, n_sums, eps, dual, stream);
        else if (mt == 3) rc = launch_mid<3, false>(out, out_mode, xb, wb, M, N, K, splits, sums_in, n_sums, eps, dual, stream);
        else if (mt == 4) rc = launch_mid<4, false>(out, out_mode, xb, wb, M, N, K, splits, sums_in, n_sums, eps, dual, stream);
        else if (mt <= 6) rc = launch_mid<6, false>(out, out_mode, xb, wb, M, N, K, splits, sums_in, n_sums, eps, dual, stream);
        else rc = launch_mid<8, false>(out, out_mode, xb, wb, M, N, K, splits, sums_in, n_sums, eps, dual, stream);
    }
    if (rc != 0) return rc;
    IA_LAUNCH_CHECK("gemm_mid");
    return 0;
}

extern "C" int ia_gemm_mid_bf16(void* out, const void* x, const void* w, int M, int N, int K, int out_mode, int dual,
                                hipStream_t stream) {
    return ia_gemm_mid_bf16_scaled(out, x, w, M, N, K, out_mode, dual, nullptr, 0, 0.f, stream);
}

// ---- readers of the splits' sums ------------------------------------------------------------------------------
// out[m][n] = sum over the splits, in their order, rounded once.
__global__ __launch_bounds__(256) void sum_partials_kernel(bf16_t* __restrict__ out, const float* __restrict__ part,
                                                           int splits, size_t mn) {
    const size_t i4 = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i4 >= mn) return;
    if (i4 + 3 < mn) {
        float4 s = *(const float4*)(part + i4);
        for (int k = 1; k < splits; ++k) {
            const float4 o = *(const float4*)(part + (size_t)k * mn + i4);
            s.x += o.x; s.y += o.y; s.z += o.z; s.w += o.w;
        }
        *(uint2*)(out + i4) = make_uint2(pack_bf16x2(s.x, s.y), pack_bf16x2(s.z, s.w));
    } else {
        for (size_t i = i4; i < mn; ++i) {
            float s = part[i];
            for (int k = 1; k < splits; ++k) s += part[(size_t)k * mn + i];
            out[i].bits = f32_to_bf16_bits(s);
        }
    }
}

extern "C" int ia_sum_partials(void* out, const float* part, int splits, int M, int N, hipStream_t stream) {
    IA_CHECK(splits >= 1 && M >= 0 && N > 0, "sum_partials: bad sizes splits=%d M=%d N=%d", splits, M, N);
    IA_CHECK(((size_t)M * N) % 4 == 0 || splits >= 1, "sum_partials: bad sizes");
    if (M == 0) return 0;
    const size_t mn = (size_t)M * N;
    IA_CHECK((mn & 3) == 0 && (((uintptr_t)out | (uintptr_t)part) & 15) == 0, "sum_partials: M * N must be a multiple of 4 "
             "and the arrays 16-byte aligned");
    sum_partials_kernel<<<(unsigned)((mn / 4 + 255) / 256), 256, 0, stream>>>((bf16_t*)out, part, splits, mn);
    IA_LAUNCH_CHECK("sum_partials");
    return 0;
}

// x[row] += the product (the splits' sums added up in their order and rounded to bfloat16, as a product that is stored
// would be), the sum formed in 32-bit and rounded; out[row] = rmsnorm(x[row]) * w.  One block a row, a thread four
// neighbouring features at a time, all its splits' loads under way together; the row stays in registers between the
// two passes.  The same arithmetic as the add-and-norm kernel of elementwise.hip on a stored product.
#define APN_MAX_THREADS 1024
#define APN_MAX_PER_THREAD 2             // rows of up to 1024 * 4 * 2 = 8192 features
template <int SPLITS>                    // 0: any number, walked one by one
__global__ __launch_bounds__(APN_MAX_THREADS) void add_rmsnorm_partials_kernel(
    bf16_t* __restrict__ out, bf16_t* __restrict__ x, const float* __restrict__ part, int splits, size_t mn,
    const float* __restrict__ w, float eps, int cols, int add_one) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    float h[APN_MAX_PER_THREAD][4];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < APN_MAX_PER_THREAD; ++j) {
        const int c = (j * (int)blockDim.x + (int)threadIdx.x) * 4;
        if (c >= cols) break;
        const size_t at = row * cols + c;
        float4 s;
        if constexpr (SPLITS > 0) {
            float4 p[SPLITS];
#pragma unroll
            for (int k = 0; k < SPLITS; ++k) p[k] = *(const float4*)(part + (size_t)k * mn + at);
            s = p[0];
#pragma unroll
            for (int k = 1; k < SPLITS; ++k) { s.x += p[k].x; s.y += p[k].y; s.z += p[k].z; s.w += p[k].w; }
        } else {
            s = *(const float4*)(part + at);
            for (int k = 1; k < splits; ++k) {
                const float4 o = *(const float4*)(part + (size_t)k * mn + at);
                s.x += o.x; s.y += o.y; s.z += o.z; s.w += o.w;
            }
        }
        const uint2 old = *(const uint2*)(x + at);
        const float sv[4] = {s.x, s.y, s.z, s.w};
        const uint16_t ob[4] = {(uint16_t)old.x, (uint16_t)(old.x >> 16), (uint16_t)old.y, (uint16_t)(old.y >> 16)};
        uint16_t nb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float product = bf16_bits_to_f32(f32_to_bf16_bits(sv[i]));
            nb[i] = f32_to_bf16_bits(product + bf16_bits_to_f32(ob[i]));
            h[j][i] = bf16_bits_to_f32(nb[i]);
            ss += h[j][i] * h[j][i];
        }
        *(uint2*)(x + at) = make_uint2((uint32_t)nb[0] | ((uint32_t)nb[1] << 16), (uint32_t)nb[2] | ((uint32_t)nb[3] << 16));
    }
    const float total = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(total / (float)cols + eps);
#pragma unroll
    for (int j = 0; j < APN_MAX_PER_THREAD; ++j) {
        const int c = (j * (int)blockDim.x + (int)threadIdx.x) * 4;
        if (c >= cols) break;
        const float4 g4 = *(const float4*)(w + c);
        const float gw[4] = {g4.x, g4.y, g4.z, g4.w};
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = h[j][i] * scale * (add_one ? 1.0f + gw[i] : gw[i]);
        *(uint2*)(out + row * cols + c) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
    }
}

extern "C" int ia_add_rmsnorm_partials(void* out, void* x, const float* part, int splits, const float* w, float eps,
                                       int rows, int cols, int add_one, hipStream_t stream) {
    IA_CHECK(rows >= 0 && cols > 0 && splits >= 1, "add_rmsnorm_partials: bad sizes rows=%d cols=%d splits=%d", rows, cols, splits);
    IA_CHECK(cols % 4 == 0 && cols <= APN_MAX_THREADS * 4 * APN_MAX_PER_THREAD,
             "add_rmsnorm_partials: rows of %d features: takes multiples of 4 up to %d", cols, APN_MAX_THREADS * 4 * APN_MAX_PER_THREAD);
    IA_CHECK((((uintptr_t)out | (uintptr_t)x | (uintptr_t)part | (uintptr_t)w) & 15) == 0,
             "add_rmsnorm_partials: arrays must be 16-byte aligned");
    if (rows == 0) return 0;
    // as many threads as the row has groups of four features, in whole waves, up to 1,024
    int threads = ((cols / 4 + IA_WAVE - 1) / IA_WAVE) * IA_WAVE;
    threads = threads > APN_MAX_THREADS ? APN_MAX_THREADS : threads;
    bf16_t* o = (bf16_t*)out;
    bf16_t* xs = (bf16_t*)x;
    const size_t mn = (size_t)rows * cols;
#define APN_LAUNCH(S) add_rmsnorm_partials_kernel<S><<<rows, threads, 0, stream>>>(o, xs, part, splits, mn, w, eps, cols, add_one)
    if (splits == 2) APN_LAUNCH(2);
    else if (splits == 4) APN_LAUNCH(4);
    else if (splits == 8) APN_LAUNCH(8);
    else APN_LAUNCH(0);
#undef APN_LAUNCH
    IA_LAUNCH_CHECK("add_rmsnorm_partials");
    return 0;
}
