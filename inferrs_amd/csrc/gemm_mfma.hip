// Large bfloat16 products on the matrix cores: out[M, N] = x[M, K] . w[N, K]^T for steps with many rows
// (prompt portions), optionally with the feed-forward's activation inside: w = [gate; up] and
// out = silu(x . gate^T) * (x . up^T).
//
// The reference hands all its products to cuBLAS (`candle-core/src/cuda_backend/mod.rs:2260-2305`) and runs
// SiLU and the product of the halves as kernels of their own (`inferrs-models/src/models/attention_utils.rs:94-118`).
//
// A block of four waves owns a tile of 256 rows of x by 256 rows of w and walks k in stages of 32 (one step of the
// matrix instruction), four of them in shared memory.  A stage's two operand tiles (256 rows of 64 bytes each) go
// from memory straight into shared memory (global_load_lds, 16 bytes a lane, no register on the way), three stages
// ahead of their use.  A wave owns 128 by 128 of the tile: 8 x 8 tiles of v_mfma_f32_16x16x32_bf16, whose A operand
// is a tile of w (16 output features) and whose B operand a tile of x (16 rows), so that a lane ends up with four
// neighbouring features of one row of the result: an 8-byte store.  Blocks stay on their compute units and take
// tile after tile.
//
// Shared memory: a row of 64 bytes holds four 16-byte pieces; piece c of row r lies at place c ^ ((r >> 1) & 3),
// so that the eight rows that a read takes in one cycle (eight lanes, 128 bytes: the banks cover 128 bytes) fall on
// eight different places of them (with (r >> 2) & 3 rows r and r + 2 met on the same banks: twice the cycles).  A load instruction fills 1 KiB (16 rows) in lane order: the lane picks the piece it fetches accordingly.
//
// Measured at 2,048 rows and the sizes of an 8 B model (TFLOP/s; the vendor's GEMM in brackets, for gate|up with its
// SiLU kernel): gate|up 1,081 (1,240; with the SiLU kernel 382 against 332 + 30 us), qkv 1,041 (1,265: 192 tiles on
// 256 compute units), o 760 (1,170: 128 tiles), down 893 (1,280: 128 tiles).  The vendor's kernels are the default
// for these products; this one runs when the package is told to do without the library.
// What bounds it (time stamps inside the kernel).  With stages of 64 k, two in shared memory, and a stage's sixteen
// loads a wave in a row after the barrier (947 TFLOP/s on gate|up): a load holds its wave until the compute unit's
// address unit takes it (1 KiB in 16 cycles), and a wave has its SIMD to itself, so the matrix pipe stood idle a
// third of a stage.  With a load beside every group of eight products, and the products written out with their
// accumulators tied to the matrix cores' registers (left the choice, the compiler renames accumulators from stage
// to stage and copies them back: 350 moves for every 128 products): a stage of 64 products took 1,455 cycles with a
// group's reads and load in a row at its start, 1,300 with one behind a product each (the waits for loads and the
// barrier are 90 of them).  And the clock: 2.1 to 2.2 GHz while half the compute units multiply (o, down), 1.8 to
// 2.0 with three quarters (qkv), 1.46 to 1.67 GHz with all of them (gate|up), lower the fewer cycles the matrix
// pipes stand idle (1.67 GHz at 1,455 cycles a stage, 1.56 at 1,300, 1.46 with no gap between a unit's tiles):
// the chip holds its power, not its clock, and 2.5 PFLOP/s are the matrix pipes' rate at 2.4 GHz.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "common.h"
#include "api.h"

typedef __bf16 gm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gm_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t gm_u32x4 __attribute__((ext_vector_type(4)));

#define GM_BM 256
#define GM_BN 256
#define GM_BK 32                            // k of a stage: one step of the matrix instruction
#define GM_ROW 64                           // bytes of a tile row in shared memory (GM_BK bfloat16)
#define GM_TILE (256 * GM_ROW)              // bytes of one operand tile
#define GM_STAGE (2 * GM_TILE)              // x tile, then w tile
#define GM_RING 4                           // stages in shared memory
#define GM_LDS (GM_RING * GM_STAGE)

struct GemmMfmaParams {
    bf16_t* out;
    const bf16_t* x;
    const bf16_t* w;
    int M, N, K;            // N: output features (with the activation inside, w has 2 N rows)
    int act;                // DUAL: the gate's activation (IA_ACT_*)
    int tiles_m, tiles_n;
};

// 16 bytes a lane from memory straight into shared memory, 1 KiB a wave in lane order from `lds_at` on (the same for
// all lanes).  Written out so that the compiler neither counts it among the loads it waits for nor moves registers
// about for it: the waits stand in the code (s_waitcnt vmcnt: loads come back in the order they were asked for).
__device__ __forceinline__ void gm_load16(const char* from, uint32_t lds_at) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(lds_at) : "memory");
}

// DUAL: the block's 256 rows of w are 128 output features: for each wave 64 rows of gate, then the 64 rows
// of up of the same features.
template <bool DUAL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_mfma_kernel(const GemmMfmaParams p) {
    __shared__ __attribute__((aligned(1024))) char gm_lds[GM_LDS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    constexpr int FEATS = DUAL ? GM_BN / 2 : GM_BN;        // output features of a block

    // Blocks go round the eight dies in turn, and each die has an L2 of its own: a die takes a contiguous
    // range of tiles, walked with the rows of x fastest, so that the blocks that run together on a die share
    // tiles of w.
    // A block stays on its compute unit and takes the tiles vb = blockIdx.x, + gridDim.x, ...: a new block of this
    // size (128 KiB of shared memory, a SIMD's registers a wave) started some 25 us after the one before it had
    // ended, so that 768 tiles took three and a half times a tile's 107 us instead of three times.
    const int n_tiles = p.tiles_m * p.tiles_n;
    for (int vb = blockIdx.x; vb < n_tiles; vb += gridDim.x) {
    if (vb != (int)blockIdx.x) __syncthreads();         // everybody is done with the shared memory of the tile before
    int tile = vb;
    if ((n_tiles & 7) == 0 && (gridDim.x & 7) == 0) tile = (vb & 7) * (n_tiles >> 3) + (vb >> 3);
    const int tm_blk = tile % p.tiles_m, tn_blk = tile / p.tiles_m;
    const int m0 = tm_blk * GM_BM, n0 = tn_blk * FEATS;

    // ---- what this lane fetches: a stage is 32 loads of 16 rows (1 KiB), the first 16 of x, the others of w; wave v
    // issues the loads 4 i + v, i = 0..7.  A load fills shared memory in lane order: lane l brings, for row l / 4 of
    // its 16, the piece that belongs at place l % 4 of the row (see the layout below).
    const char* gsrc[8];
    const size_t pitch = (size_t)p.K * 2;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = ((i & 3) * 4 + wave) * 16 + (lane >> 2);       // row of the operand's tile
        const int piece = (lane & 3) ^ ((row >> 1) & 3);
        if (i < 4) {
            int m = m0 + row;
            m = m < p.M ? m : p.M - 1;
            gsrc[i] = (const char*)p.x + (size_t)m * pitch + piece * 16;
        } else {
            int n;
            if (DUAL) {
                const int wn = row >> 7, q = row & 127;
                const int f = n0 + wn * 64 + (q & 63);
                n = (f < p.N ? f : p.N - 1) + (q >= 64 ? p.N : 0);
            } else {
                n = n0 + row;
                n = n < p.N ? n : p.N - 1;
            }
            gsrc[i] = (const char*)p.w + (size_t)n * pitch + piece * 16;
        }
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)gm_lds;
    const int stages = p.K / GM_BK;
    // load i (of the wave's own eight) of stage `kt` into the place of stage `slot` (the two differ past the walk's
    // end only: a load is issued there all the same, of the last stage again into a place that nobody reads, so that
    // the walk has no branch and the count of loads under way is the same at every stage)
    auto fetch = [&](int kt, int slot, int i) __attribute__((always_inline)) {
        gm_load16(gsrc[i] + (size_t)kt * (GM_BK * 2),
                  lds0 + (uint32_t)(slot & (GM_RING - 1)) * GM_STAGE + (i < 4 ? 0 : GM_TILE) + (uint32_t)((i & 3) * 4 + wave) * 1024);
    };
    // ---- the wave's share: rows wm * 128 .. of x, rows wn * 128 .. of w -------------------------------------
    // Shared memory: a row of 64 bytes holds four 16-byte pieces; piece c of row r lies at place c ^ ((r >> 1) & 3), so
    // that the eight rows which a read takes in one cycle fall on eight different places of the 128 bytes the banks cover.
    const int wm = wave & 1, wn = wave >> 1;
    const uint32_t at = (uint32_t)(r * GM_ROW + ((g ^ ((r >> 1) & 3)) * 16));      // the lane's place in a 16-row tile
    const uint32_t x_at = (uint32_t)(wm * 128 * GM_ROW) + at, w_at = (uint32_t)(GM_TILE + wn * 128 * GM_ROW) + at;

    gm_f32x4 acc[8][8];                 // [tile of w rows][tile of x rows]
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[a][b] = (gm_f32x4){0.f, 0.f, 0.f, 0.f};

    // The operand reads are written out as instructions, with their waits: a wait names how many reads may still be
    // under way (they come back in order) and passes the registers it vouches for through, so that no product moves
    // ahead of it.
    auto read16 = [&](gm_u32x4& dst, uint32_t addr, auto off) __attribute__((always_inline)) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(decltype(off)::value));
    };

    // ---- the walk.  Stage s is multiplied while the x operands of stage s + 1 are read from shared memory and stage
    // s + 3 is asked for from memory, a load beside every group of eight products: a load holds its wave until the
    // compute unit's address unit takes it, and a wave has its SIMD to itself, so the sixteen loads of a stage in a
    // row (as this kernel had them) stood between the products for a third of a stage's time.
    // At the top of stage s the wave waits for its own loads of stage s + 1 (those of stage s + 2 may be under way)
    // and passes the barrier: everybody's part of stage s + 1 is there, and everybody is done with stage s - 1,
    // into whose place stage s + 3 goes.
#pragma unroll
    for (int pre = 0; pre < GM_RING - 1; ++pre) {
#pragma unroll
        for (int i = 0; i < 8; ++i) fetch(pre < stages ? pre : stages - 1, pre, i);
    }
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    __syncthreads();
    gm_u32x4 fx[2][8], fw[2];
    {
        const uint32_t xa = lds0 + x_at, wa = lds0 + w_at;
        read16(fx[0][0], xa, std::integral_constant<int, 0 * 1024>());
        read16(fx[0][1], xa, std::integral_constant<int, 1 * 1024>());
        read16(fx[0][2], xa, std::integral_constant<int, 2 * 1024>());
        read16(fx[0][3], xa, std::integral_constant<int, 3 * 1024>());
        read16(fx[0][4], xa, std::integral_constant<int, 4 * 1024>());
        read16(fx[0][5], xa, std::integral_constant<int, 5 * 1024>());
        read16(fx[0][6], xa, std::integral_constant<int, 6 * 1024>());
        read16(fx[0][7], xa, std::integral_constant<int, 7 * 1024>());
        read16(fw[0], wa, std::integral_constant<int, 0>());
    }
    // One stage: CUR names the half of fx that holds its x operands (the other half takes the next stage's).
#define GM_MFMA(CUR, A, B)                                                                                              \
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[A][B]) : "v"(fw[(A) & 1]), "v"(fx[CUR][B]));
    // A group: a tile of w against the stage's eight tiles of x.  A product holds the issue for half of its 16 cycles:
    // the group's other instructions (the read of the next group's tile of w, of one tile of x of the next stage, a
    // load from memory and its address) stand one behind a product each, not in a row at the group's start, where
    // the matrix pipe stood idle meanwhile (a stage of 64 products took 1,455 cycles).
#define GM_GROUP(CUR, A, LAST)                                                                                          \
        {                                                                                                               \
            if ((A) == 0)                                                                                               \
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fw[0]), "+v"(fx[CUR][0]), "+v"(fx[CUR][1]), "+v"(fx[CUR][2]), \
                             "+v"(fx[CUR][3]), "+v"(fx[CUR][4]), "+v"(fx[CUR][5]), "+v"(fx[CUR][6]), "+v"(fx[CUR][7])); \
            else asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(fw[(A) & 1]));                                             \
            GM_MFMA(CUR, A, 0)                                                                                          \
            if ((A) < 7) read16(fw[((A) + 1) & 1], wa, std::integral_constant<int, (((A) + 1) & 7) * 1024>());          \
            else read16(fw[0], wa_next, std::integral_constant<int, 0>());                                             \
            GM_MFMA(CUR, A, 1)                                                                                          \
            read16(fx[1 - (CUR)][A], xa_next, std::integral_constant<int, (A) * 1024>());                              \
            GM_MFMA(CUR, A, 2)                                                                                          \
            GM_MFMA(CUR, A, 3)                                                                                          \
            fetch(kt3, s + 3, A);                                                                                       \
            GM_MFMA(CUR, A, 4)                                                                                          \
            GM_MFMA(CUR, A, 5)                                                                                          \
            GM_MFMA(CUR, A, 6)                                                                                          \
            if (LAST && (A) == 7)       /* (nothing may read a product's result for 7 wait states after it) */          \
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\ts_nop 15" : "+a"(acc[A][7]) : "v"(fw[(A) & 1]), "v"(fx[CUR][7])); \
            else GM_MFMA(CUR, A, 7)                                                                                     \
            __builtin_amdgcn_sched_barrier(0);                                                                          \
        }
#define GM_STAGE_BODY(CUR, LAST)                                                                                            \
        {                                                                                                               \
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory");                                                           \
            __syncthreads();                                                                                            \
            const int kt3 = s + 3 < stages ? s + 3 : stages - 1;                                                        \
            const int sn = s + 1 < stages ? s + 1 : s;          /* (past the end: read again what is there) */          \
            const uint32_t wa = lds0 + (uint32_t)(s & (GM_RING - 1)) * GM_STAGE + w_at;                                 \
            const uint32_t xa_next = lds0 + (uint32_t)(sn & (GM_RING - 1)) * GM_STAGE + x_at;                           \
            const uint32_t wa_next = lds0 + (uint32_t)(sn & (GM_RING - 1)) * GM_STAGE + w_at;                           \
            GM_GROUP(CUR, 0, LAST) GM_GROUP(CUR, 1, LAST) GM_GROUP(CUR, 2, LAST) GM_GROUP(CUR, 3, LAST)                 \
            GM_GROUP(CUR, 4, LAST) GM_GROUP(CUR, 5, LAST) GM_GROUP(CUR, 6, LAST) GM_GROUP(CUR, 7, LAST)                 \
        }
    int s2 = 0;
    for (; s2 + 2 < stages; s2 += 2) {                  // (K is a multiple of 64: an even number of stages)
        {
            const int s = s2;
            GM_STAGE_BODY(0, false)
        }
        {
            const int s = s2 + 1;
            GM_STAGE_BODY(1, false)
        }
    }
    {
        const int s = s2;
        GM_STAGE_BODY(0, false)
    }
    {
        const int s = s2 + 1;
        GM_STAGE_BODY(1, true)
    }
#undef GM_STAGE_BODY
#undef GM_GROUP
#undef GM_MFMA
    // (the products are written out as instructions with their accumulators tied to the matrix cores' own registers:
    // the compiler, given the choice, renames accumulators from stage to stage and copies them back, 350 moves for
    // every 128 products; what it then does not know: a product's result may be read 7 wait states after it at the
    // earliest)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

    // ---- results: the lane holds features 4 g .. + 4 of w tile a for row r of x tile b ----------------------
    const bool vec = (p.N & 3) == 0;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const int m = m0 + wm * 128 + b * 16 + r;
        if (m >= p.M) continue;
        bf16_t* orow = p.out + (size_t)m * p.N;
        constexpr int TA = DUAL ? 4 : 8;
#pragma unroll
        for (int a = 0; a < TA; ++a) {
            float v[4];
            int n;
            if (DUAL) {
                n = n0 + wn * 64 + a * 16 + 4 * g;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // the products are rounded to the storage precision before the activation, as the
                    // two-kernel way rounds them
                    const float gate = bf16_bits_to_f32(f32_to_bf16_bits(acc[a][b][i]));
                    const float up = bf16_bits_to_f32(f32_to_bf16_bits(acc[a + 4][b][i]));
                    v[i] = gate_act(gate, p.act) * up;
                }
            } else {
                n = n0 + wn * 128 + a * 16 + 4 * g;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = acc[a][b][i];
            }
            if (vec && n + 3 < p.N) {
                uint2 pk;
                pk.x = pack_bf16x2(v[0], v[1]);
                pk.y = pack_bf16x2(v[2], v[3]);
                *(uint2*)(orow + n) = pk;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < p.N) orow[n + i].bits = f32_to_bf16_bits(v[i]);
            }
        }
    }
    }
}

template <bool DUAL>
static int gemm_mfma_launch(const GemmMfmaParams& p, hipStream_t stream) {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            cus <= 0)
            cus = 256;
    }
    const long long tiles = (long long)p.tiles_m * p.tiles_n;
    gemm_mfma_kernel<DUAL><<<(unsigned)(tiles < cus ? tiles : cus), 256, 0, stream>>>(p);
    return 0;
}

// out[M, N] = x[M, K] . w[N, K]^T, or with `dual` (an activation, IA_ACT_*) out[M, N] = act(x . w[0:N]^T) * (x . w[N:2N]^T); bfloat16,
// K a multiple of 64.
extern "C" int ia_gemm_mfma_bf16(void* out, const void* x, const void* w, int M, int N, int K, int dual,
                                 hipStream_t stream) {
    IA_CHECK(M > 0 && N > 0 && K > 0, "gemm_mfma: bad sizes M=%d N=%d K=%d", M, N, K);
    IA_CHECK(dual >= 0 && dual <= IA_ACT_LAST, "gemm_mfma: unknown activation %d", dual);
    IA_CHECK(K % (2 * GM_BK) == 0, "gemm_mfma: K=%d must be a multiple of %d", K, 2 * GM_BK);
    IA_CHECK((((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15) == 0, "gemm_mfma: operands must be 16-byte aligned");
    GemmMfmaParams p;
    p.out = (bf16_t*)out; p.x = (const bf16_t*)x; p.w = (const bf16_t*)w;
    p.M = M; p.N = N; p.K = K;
    p.act = dual;
    p.tiles_m = (M + GM_BM - 1) / GM_BM;
    p.tiles_n = dual ? (N + GM_BN / 2 - 1) / (GM_BN / 2) : (N + GM_BN - 1) / GM_BN;
    IA_CHECK((long long)p.tiles_m * p.tiles_n < (1LL << 31), "gemm_mfma: too many tiles");
    const int rc = dual ? gemm_mfma_launch<true>(p, stream) : gemm_mfma_launch<false>(p, stream);
    if (rc) return rc;
    IA_LAUNCH_CHECK("gemm_mfma");
    return 0;
}
