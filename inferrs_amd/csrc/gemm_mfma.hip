// Large bfloat16 products on the matrix cores: out[M, N] = x[M, K] . w[N, K]^T for steps with many rows
// (prompt portions), optionally with the feed-forward's activation inside: w = [gate; up] and
// out = silu(x . gate^T) * (x . up^T).
//
// The reference hands all its products to cuBLAS (`candle-core/src/cuda_backend/mod.rs:2260-2305`) and runs
// SiLU and the product of the halves as kernels of their own (`inferrs-models/src/models/attention_utils.rs:94-118`).
//
// A block of four waves owns a tile of 256 rows of x by 256 rows of w and walks k in stages of 64.  A stage's
// two operand tiles (256 rows of 128 bytes each) go from memory straight into shared memory (global_load_lds,
// 16 bytes a lane, no register on the way), the next stage while this one is multiplied.  A wave owns 128 by 128
// of the tile: 8 x 8 tiles of v_mfma_f32_16x16x32_bf16, whose A operand is a tile of w (16 output features) and
// whose B operand a tile of x (16 rows), so that a lane ends up with four neighbouring features of one row of
// the result: an 8-byte store.
//
// Shared memory: a row of 128 bytes holds eight 16-byte pieces; piece c of row r lies at place c ^ ((r >> 1) & 7),
// so that the 16 rows that one operand read takes at the same k fall into 16 different places of the 256 bytes
// that the banks cover.  A load instruction fills 1 KiB (eight rows) in lane order: the lane picks the piece it
// fetches accordingly.  The counters show no bank conflict (SQ_LDS_BANK_CONFLICT = 0).
//
// Measured at 2,048 rows and the sizes of an 8 B model (TFLOP/s; the vendor's GEMM in brackets, for gate|up with its
// SiLU kernel): gate|up 947 (1,230), qkv 824 (1,231: 192 tiles on 256 compute units), o 579 (1,140: 128 tiles),
// down 638 (1,229: 128 tiles).  The vendor's kernels are the default for these products; this one runs when
// the package is told to do without the library.  What bounds it, from timing-only variants of gate|up (435 us):
// without the loads of the next stage 317 us, with those loads always from the same, cached place 390 us: a third
// of the loads' cost is the memory's latency (a stage is asked for one stage ahead, about 1 us), two thirds the
// loads' own way into shared memory beside the operand reads.  Tried: the two stages as two arrays with the loop
// unrolled twice (the compiler then moves accumulators between register files inside the loop: 757), the reads
// left to the compiler (it waits for the other stage's loads before every read and puts each read next to its
// first use: 808), one load a group instead of sixteen at the stage's start (accumulator moves again: 713).
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
#define GM_BK 64
#define GM_ROW 128                          // bytes of a tile row in shared memory (GM_BK bfloat16)
#define GM_TILE (256 * GM_ROW)              // bytes of one operand tile
#define GM_STAGE (2 * GM_TILE)              // x tile, then w tile
#define GM_LDS (2 * GM_STAGE)

struct GemmMfmaParams {
    bf16_t* out;
    const bf16_t* x;
    const bf16_t* w;
    int M, N, K;            // N: output features (with the activation inside, w has 2 N rows)
    int tiles_m, tiles_n;
};

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
    const int n_tiles = p.tiles_m * p.tiles_n;
    int tile = blockIdx.x;
    if ((n_tiles & 7) == 0) tile = (blockIdx.x & 7) * (n_tiles >> 3) + (blockIdx.x >> 3);
    const int tm_blk = tile % p.tiles_m, tn_blk = tile / p.tiles_m;
    const int m0 = tm_blk * GM_BM, n0 = tn_blk * FEATS;

    // ---- what this lane fetches: eight instructions an operand, each eight rows of a tile ----------------
    const char* gx[8];
    const char* gw[8];
    const size_t pitch = (size_t)p.K * 2;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int row = (j * 4 + wave) * 8 + (lane >> 3);              // row of the tile
        const int piece = (lane & 7) ^ ((row >> 1) & 7);
        int m = m0 + row;
        m = m < p.M ? m : p.M - 1;
        gx[j] = (const char*)p.x + (size_t)m * pitch + piece * 16;
        int n;
        if (DUAL) {
            const int wn = row >> 7, q = row & 127;
            const int f = n0 + wn * 64 + (q & 63);
            n = (f < p.N ? f : p.N - 1) + (q >= 64 ? p.N : 0);
        } else {
            n = n0 + row;
            n = n < p.N ? n : p.N - 1;
        }
        gw[j] = (const char*)p.w + (size_t)n * pitch + piece * 16;
    }
    auto issue = [&](int kt, char* buf) {
        const size_t koff = (size_t)kt * (GM_BK * 2);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(gx[j] + koff),
                                             (void __attribute__((address_space(3)))*)(buf + (j * 4 + wave) * 1024), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(gw[j] + koff),
                                             (void __attribute__((address_space(3)))*)(buf + GM_TILE + (j * 4 + wave) * 1024), 16, 0, 0);
    };

    // ---- the wave's share: rows wm * 128 .. of x, rows wn * 128 .. of w -------------------------------------
    const int wm = wave & 1, wn = wave >> 1;
    uint32_t at[2];                     // the lane's place in a 16-row tile at k step 0 and 1
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) at[ks] = (uint32_t)(r * GM_ROW + (((ks * 4 + g) ^ ((r >> 1) & 7)) * 16));
    const uint32_t x_at = (uint32_t)(wm * 128 * GM_ROW), w_at = (uint32_t)(GM_TILE + wn * 128 * GM_ROW);

    gm_f32x4 acc[8][8];                 // [tile of w rows][tile of x rows]
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[a][b] = (gm_f32x4){0.f, 0.f, 0.f, 0.f};

    // The operand reads are written out as instructions, with their waits: the compiler would wait for the loads
    // that are on their way into the other stage before any read of shared memory (it cannot tell the stages
    // apart), and it would put every read next to its first use.  A wait names how many reads may still be under
    // way (they come back in order) and passes the registers it vouches for through, so that no product moves
    // ahead of it.
    auto read16 = [&](gm_u32x4& dst, uint32_t addr, auto off) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(decltype(off)::value));
    };
    const uint32_t lds0 = (uint32_t)(uintptr_t)gm_lds;
    const int stages = p.K / GM_BK;
    issue(0, gm_lds);
    for (int kt = 0; kt < stages; ++kt) {
        const uint32_t base = lds0 + (uint32_t)(kt & 1) * GM_STAGE;
        __builtin_amdgcn_s_waitcnt(0);          // this wave's part of the stage has arrived
        __syncthreads();                        // everybody's has, and everybody is done with the stage before
        if (kt + 1 < stages) issue(kt + 1, gm_lds + ((kt + 1) & 1) * GM_STAGE);
        // Sixteen groups of eight products: a group's tile of w against the k step's eight tiles of x.  A group's
        // tile of w is asked for a group ahead, the tiles of x of the second k step one a group during the first.
        const uint32_t xa0 = base + x_at + at[0], xa1 = base + x_at + at[1];
        const uint32_t wa0 = base + w_at + at[0], wa1 = base + w_at + at[1];
        gm_u32x4 fx[2][8], fw[2];
        read16(fx[0][0], xa0, std::integral_constant<int, 0 * 2048>());
        read16(fx[0][1], xa0, std::integral_constant<int, 1 * 2048>());
        read16(fx[0][2], xa0, std::integral_constant<int, 2 * 2048>());
        read16(fx[0][3], xa0, std::integral_constant<int, 3 * 2048>());
        read16(fx[0][4], xa0, std::integral_constant<int, 4 * 2048>());
        read16(fx[0][5], xa0, std::integral_constant<int, 5 * 2048>());
        read16(fx[0][6], xa0, std::integral_constant<int, 6 * 2048>());
        read16(fx[0][7], xa0, std::integral_constant<int, 7 * 2048>());
        read16(fw[0], wa0, std::integral_constant<int, 0>());
#define GM_GROUP(IDX)                                                                                                   \
        {                                                                                                               \
            constexpr int ks = (IDX) >> 3, a = (IDX) & 7, nx = ((IDX) + 1) & 7;                                       \
            if ((IDX) + 1 < 16) read16(fw[((IDX) + 1) & 1], (IDX) + 1 < 8 ? wa0 : wa1, std::integral_constant<int, nx * 2048>()); \
            if (ks == 0) read16(fx[1][a], xa1, std::integral_constant<int, a * 2048>());                              \
            if ((IDX) == 0)                                                                                             \
                asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(fw[0]), "+v"(fx[0][0]), "+v"(fx[0][1]), "+v"(fx[0][2]), "+v"(fx[0][3]), \
                             "+v"(fx[0][4]), "+v"(fx[0][5]), "+v"(fx[0][6]), "+v"(fx[0][7]));                        \
            else if ((IDX) < 8) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(fw[(IDX) & 1]));                            \
            else if ((IDX) == 8)                                                                                        \
                asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(fw[0]), "+v"(fx[1][0]), "+v"(fx[1][1]), "+v"(fx[1][2]), "+v"(fx[1][3]), \
                             "+v"(fx[1][4]), "+v"(fx[1][5]), "+v"(fx[1][6]), "+v"(fx[1][7]));                        \
            else if ((IDX) < 15) asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(fw[(IDX) & 1]));                           \
            else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fw[(IDX) & 1]));                                           \
            _Pragma("unroll") for (int b = 0; b < 8; ++b)                                                              \
                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gm_bf16x8, fw[(IDX) & 1]),      \
                                                                    __builtin_bit_cast(gm_bf16x8, fx[ks][b]), acc[a][b], 0, 0, 0); \
        }
        GM_GROUP(0) GM_GROUP(1) GM_GROUP(2) GM_GROUP(3) GM_GROUP(4) GM_GROUP(5) GM_GROUP(6) GM_GROUP(7)
        GM_GROUP(8) GM_GROUP(9) GM_GROUP(10) GM_GROUP(11) GM_GROUP(12) GM_GROUP(13) GM_GROUP(14) GM_GROUP(15)
#undef GM_GROUP
    }

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
                    v[i] = gate / (1.0f + expf(-gate)) * up;
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

template <bool DUAL>
static int gemm_mfma_launch(const GemmMfmaParams& p, hipStream_t stream) {
    gemm_mfma_kernel<DUAL><<<(unsigned)(p.tiles_m * p.tiles_n), 256, 0, stream>>>(p);
    return 0;
}

// out[M, N] = x[M, K] . w[N, K]^T, or with `dual` out[M, N] = silu(x . w[0:N]^T) * (x . w[N:2N]^T); bfloat16,
// K a multiple of 64.
extern "C" int ia_gemm_mfma_bf16(void* out, const void* x, const void* w, int M, int N, int K, int dual,
                                 hipStream_t stream) {
    IA_CHECK(M > 0 && N > 0 && K > 0, "gemm_mfma: bad sizes M=%d N=%d K=%d", M, N, K);
    IA_CHECK(K % GM_BK == 0, "gemm_mfma: K=%d must be a multiple of %d", K, GM_BK);
    IA_CHECK((((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15) == 0, "gemm_mfma: operands must be 16-byte aligned");
    GemmMfmaParams p;
    p.out = (bf16_t*)out; p.x = (const bf16_t*)x; p.w = (const bf16_t*)w;
    p.M = M; p.N = N; p.K = K;
    p.tiles_m = (M + GM_BM - 1) / GM_BM;
    p.tiles_n = dual ? (N + GM_BN / 2 - 1) / (GM_BN / 2) : (N + GM_BN - 1) / GM_BN;
    IA_CHECK((long long)p.tiles_m * p.tiles_n < (1LL << 31), "gemm_mfma: too many tiles");
    const int rc = dual ? gemm_mfma_launch<true>(p, stream) : gemm_mfma_launch<false>(p, stream);
    if (rc) return rc;
    IA_LAUNCH_CHECK("gemm_mfma");
    return 0;
}
