// Matrix products y[m, n] = sum_k x[m, k] * w[n, k] for weights stored [out, in] as the
// checkpoints hold them (the reference's Linear is x . W^T, candle-nn/src/linear.rs:64-72).
//
//   * ia_gemm_tiled: plain 64x64 tiles through shared memory, fused multiply-adds in 32-bit
//     with k ascending for every output, whatever the number of rows: a row's result does
//     not depend on what else is in the batch.  It is the matrix product of the true 32-bit
//     path and takes bfloat16 inputs of any size as the fallback of the kernel below.
//   * ia_gemm_skinny_bf16: few rows (decode batches, logits of a few positions) against a
//     large weight matrix.  The product is bound by reading the weights once, so each wave
//     streams 16 weight rows in 16-byte pieces straight into MFMA 16x16x32 operands and
//     the waves of a block split k between them; partial tiles are summed in a fixed order.
//     A variant takes [gate; up] and writes silu(gate) * up.
#include <type_traits>

#include "common.h"
#include "api.h"

// ---- tiled product ----------------------------------------------------------------------------
#define GT 64
#define GK 16

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(TO* __restrict__ out, const TI* __restrict__ x,
                                                         const TI* __restrict__ w, int M, int N, int K) {
    __shared__ float xs[GK][GT + 1];
    __shared__ float ws[GK][GT + 1];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    const int lr = tid >> 2;          // row of the tile this thread loads
    const int lk = (tid & 3) * 4;     // first of its four k
    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int m = m0 + lr, n = n0 + lr;
            xs[lk + i][lr] = (m < M && k < K) ? ld(x + (size_t)m * K + k) : 0.f;
            ws[lk + i][lr] = (n < N && k < K) ? ld(w + (size_t)n * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty + 16 * i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n < N) st(out + (size_t)m * N + n, acc[i][j]);
        }
    }
}

__device__ __forceinline__ float4 gr_load4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 gr_load4(const bf16_t* p) {
    const uint2 v = *(const uint2*)p;
    return make_float4(bf16_bits_to_f32((uint16_t)v.x), bf16_bits_to_f32((uint16_t)(v.x >> 16)),
                       bf16_bits_to_f32((uint16_t)v.y), bf16_bits_to_f32((uint16_t)(v.y >> 16)));
}

// The same sums in tiles of 128 x 128 for many rows (prompts of the 32-bit path): a thread owns 8 x 8 outputs (rows
// 4 ty .. + 4 and 64 + 4 ty .. + 4, features likewise with tx), so that every value read from shared memory meets eight
// fused multiply-adds instead of four; k ascending for every output as above, hence the same bits.  K a multiple of 4.
#define GB 128
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled128_kernel(TO* __restrict__ out, const TI* __restrict__ x,
                                                            const TI* __restrict__ w, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) float xs[GK][GB + 4];
    __shared__ __attribute__((aligned(16))) float ws[GK][GB + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * GB, n0 = blockIdx.x * GB;
    float acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
    // a tile is 128 rows x 16 k = 512 pieces of four k: two a thread, of rows lr and lr + 64
    const int lr = tid >> 2, lk = (tid & 3) * 4;
    const TI* xp[2];
    const TI* wp[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int m = m0 + lr + 64 * h, n = n0 + lr + 64 * h;
        xp[h] = x + (size_t)(m < M ? m : M - 1) * K + lk;       // (rows beyond the matrices: never stored)
        wp[h] = w + (size_t)(n < N ? n : N - 1) * K + lk;
    }
    float4 xr[2], wr[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const bool in = k0 + lk < K;
            xr[h] = in ? gr_load4(xp[h] + k0) : make_float4(0.f, 0.f, 0.f, 0.f);
            wr[h] = in ? gr_load4(wp[h] + k0) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += GK) {
        __syncthreads();
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int r = lr + 64 * h;
            xs[lk][r] = xr[h].x; xs[lk + 1][r] = xr[h].y; xs[lk + 2][r] = xr[h].z; xs[lk + 3][r] = xr[h].w;
            ws[lk][r] = wr[h].x; ws[lk + 1][r] = wr[h].y; ws[lk + 2][r] = wr[h].z; ws[lk + 3][r] = wr[h].w;
        }
        if (k0 + GK < K) fetch(k0 + GK);
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            const float4 a0 = *(const float4*)(&xs[kk][4 * ty]), a1 = *(const float4*)(&xs[kk][64 + 4 * ty]);
            const float4 b0 = *(const float4*)(&ws[kk][4 * tx]), b1 = *(const float4*)(&ws[kk][64 + 4 * tx]);
            const float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int m = m0 + (i < 4 ? 4 * ty + i : 64 + 4 * ty + i - 4);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int n = n0 + (j < 4 ? 4 * tx + j : 64 + 4 * tx + j - 4);
            if (n < N) st(out + (size_t)m * N + n, acc[i][j]);
        }
    }
}

// The same product for up to 16 rows (decode steps of the 32-bit path), bound by reading the weights.  A wave owns GN
// output features and stages ROWS rows; lane (feature, group of ROWS * GN / 64 rows) adds up its rows' sums with k
// ascending, one chain of fused multiply-adds each, which gives the bits of the tiled kernel whatever GN and ROWS are.
// Chunks of 256 k come into shared memory in whole rows, the next chunk on its way from memory while this one is
// multiplied.  A wave's time for a chunk is what its lanes multiply and what it stages of the rows, so fewer rows
// and fewer features a wave (more waves) read the weights faster; the shapes that exist and the rule that picks one are
// at the launch below.  K a multiple of 4.
#define GR_K 256
#define GR_PITCH (GR_K + 4)             // floats between staged rows: 16-byte aligned, no two of 16 lanes on a bank
#define GR_ROWS 16                      // the most rows of one launch

template <typename TI, typename TO, int GN, int ROWS>
__global__ __launch_bounds__(IA_WAVE) void gemm_rows_kernel(TO* __restrict__ out, const TI* __restrict__ x,
                                                            const TI* __restrict__ w, int M, int N, int K) {
    constexpr int GROUPS = IA_WAVE / GN;                    // groups of rows
    constexpr int RPL = ROWS / GROUPS;                      // rows a lane adds up
    static_assert(GN * GROUPS == IA_WAVE && RPL * GROUPS == ROWS && RPL >= 1, "lane = (feature, group of rows)");
    static_assert(GR_K / 4 == IA_WAVE, "a lane brings one piece of every staged row");
    __shared__ __attribute__((aligned(16))) float ws[GN * GR_PITCH];
    __shared__ __attribute__((aligned(16))) float xs[ROWS * GR_PITCH];
    const int lane = threadIdx.x;
    const int nn = lane % GN, mg = lane / GN;
    const int n0 = blockIdx.x * GN;
    // what this lane fetches: load i takes piece (lane % 64) of row i (a row of a chunk is 64 pieces of four)
    const int piece = lane * 4;
    float4 wr[GN], xr[ROWS];
    auto fetch = [&](int k0, float4* wq, float4* xq) {
        const int k = k0 + piece;
#pragma unroll
        for (int i = 0; i < GN; ++i) {
            const int n = n0 + i < N ? n0 + i : N - 1;         // (features beyond the matrix: never stored)
            wq[i] = k < K ? gr_load4(w + (size_t)n * K + k) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < ROWS; ++i)
            xq[i] = (k < K && i < M) ? gr_load4(x + (size_t)i * K + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    };
    float acc[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) acc[i] = 0.f;
    // chunk k0 goes from its registers into shared memory, the next chunk takes the registers, and the sums go on
    auto chunk = [&](int k0, float4* wq, float4* xq) {
        __syncthreads();                                        // everybody is done with the chunk before
#pragma unroll
        for (int i = 0; i < GN; ++i) *(float4*)(ws + i * GR_PITCH + piece) = wq[i];
#pragma unroll
        for (int i = 0; i < ROWS; ++i) *(float4*)(xs + i * GR_PITCH + piece) = xq[i];
        if (k0 + GR_K < K) fetch(k0 + GR_K, wq, xq);
        __syncthreads();
        const float* wmine = ws + nn * GR_PITCH;
        const float* xmine = xs + mg * RPL * GR_PITCH;
#pragma unroll 4
        for (int k4 = 0; k4 < GR_K / 4; ++k4) {
            const float4 wv = *(const float4*)(wmine + k4 * 4);
#pragma unroll
            for (int i = 0; i < RPL; ++i) {
                const float4 xv = *(const float4*)(xmine + i * GR_PITCH + k4 * 4);
                acc[i] = fmaf(xv.x, wv.x, acc[i]);
                acc[i] = fmaf(xv.y, wv.y, acc[i]);
                acc[i] = fmaf(xv.z, wv.z, acc[i]);
                acc[i] = fmaf(xv.w, wv.w, acc[i]);
            }
        }
    };
    fetch(0, wr, xr);
    for (int k0 = 0; k0 < K; k0 += GR_K) chunk(k0, wr, xr);
    const int n = n0 + nn;
    if (n < N)
#pragma unroll
        for (int i = 0; i < RPL; ++i)
            if (mg * RPL + i < M) st(out + (size_t)(mg * RPL + i) * N + n, acc[i]);
}

static int skinny_cus();
static int g_rows_shape = 0;         // 0: by the rule below; else 100 * features + rows, forced (measurements and tests)
extern "C" int ia_gemm_rows_tune(int shape) {
    IA_CHECK(shape == 0 || shape == 816 || shape == 808 || shape == 416 || shape == 1608,
             "gemm_rows_tune: no kernel of %d features and %d rows a wave", shape / 100, shape % 100);
    g_rows_shape = shape;
    return 0;
}

template <typename TI, typename TO, int GN, int ROWS>
static void launch_rows_shape(void* o, const void* xi, const void* w, int rows, int N, int K, hipStream_t stream) {
    gemm_rows_kernel<TI, TO, GN, ROWS><<<(unsigned)((N + GN - 1) / GN), IA_WAVE, 0, stream>>>((TO*)o, (const TI*)xi, (const TI*)w, rows, N, K);
}

// Up to 8 rows: 8 features a wave, 16 where that still makes eight waves for every compute unit's four schedulers;
// 9 to 16 rows: 8 features, 4 while 8 would leave a scheduler without a wave.  (Measured at 8 rows and 4,096 k, this
// rule against 16 features and 16 rows for every size: 6,144 features 77 -> 41 us, 4,096 72 -> 36, 24,576 162 -> 88,
// 151,936 790 -> 483; at 16 rows 75 -> 50, 72 -> 44, 165 -> 144, 803 -> 796.)
template <typename TI, typename TO>
static void launch_rows(void* o, const void* xi, const void* w, int rows, int N, int K, hipStream_t stream) {
    const int cus = skinny_cus();
    int shape = g_rows_shape;
    if (shape != 0 && shape % 100 < rows) shape = 816;            // a forced shape that does not hold the rows
    if (shape == 0) shape = rows <= 8 ? (N >= 64 * cus ? 1608 : 808) : (N <= 32 * cus ? 416 : 816);
    switch (shape) {
    case 1608: launch_rows_shape<TI, TO, 16, 8>(o, xi, w, rows, N, K, stream); break;
    case 808: launch_rows_shape<TI, TO, 8, 8>(o, xi, w, rows, N, K, stream); break;
    case 416: launch_rows_shape<TI, TO, 4, 16>(o, xi, w, rows, N, K, stream); break;
    default: launch_rows_shape<TI, TO, 8, 16>(o, xi, w, rows, N, K, stream); break;
    }
}

// in_dtype: storage of x and w; out_dtype: storage of the result.
extern "C" int ia_gemm_tiled(void* out, const void* x, const void* w, int M, int N, int K,
                             int in_dtype, int out_dtype, hipStream_t stream) {
    IA_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    const size_t elem = in_dtype == IA_F32 ? 4 : 2;
    // up to 64 rows, 16 at a time, where the tiles of 64 x 64 would be few (the weights are read once for every 16 rows:
    // at 32 rows of the 32-bit path a decode step of four layers at the sizes of an 8B model still takes a third of the time)
    if (M <= 4 * GR_ROWS && (M <= GR_ROWS || N <= 4096 * 4) && K % 4 == 0 && (((uintptr_t)x | (uintptr_t)w) % (4 * elem)) == 0) {
        const size_t out_elem = out_dtype == IA_F32 ? 4 : 2;
        for (int m0 = 0; m0 < M; m0 += GR_ROWS) {
            const int rows = M - m0 < GR_ROWS ? M - m0 : GR_ROWS;
            void* o = (char*)out + (size_t)m0 * N * out_elem;
            const void* xi = (const char*)x + (size_t)m0 * K * elem;
            if (in_dtype == IA_F32 && out_dtype == IA_F32) launch_rows<float, float>(o, xi, w, rows, N, K, stream);
            else if (in_dtype == IA_BF16 && out_dtype == IA_BF16) launch_rows<bf16_t, bf16_t>(o, xi, w, rows, N, K, stream);
            else if (in_dtype == IA_BF16 && out_dtype == IA_F32) launch_rows<bf16_t, float>(o, xi, w, rows, N, K, stream);
            else IA_CHECK(false, "gemm_tiled: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
        }
        IA_LAUNCH_CHECK("gemm_rows");
        return 0;
    }
    if (M > 2 * GT && N >= GB && K % 4 == 0 && (((uintptr_t)x | (uintptr_t)w) % (4 * elem)) == 0) {
        const dim3 grid((N + GB - 1) / GB, (M + GB - 1) / GB);
        IA_CHECK(grid.y <= 65535, "gemm_tiled: %d rows exceed the grid", M);
        if (in_dtype == IA_F32 && out_dtype == IA_F32)
            gemm_tiled128_kernel<float, float><<<grid, 256, 0, stream>>>((float*)out, (const float*)x, (const float*)w, M, N, K);
        else if (in_dtype == IA_BF16 && out_dtype == IA_BF16)
            gemm_tiled128_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        else if (in_dtype == IA_BF16 && out_dtype == IA_F32)
            gemm_tiled128_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((float*)out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
        else
            IA_CHECK(false, "gemm_tiled: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
        IA_LAUNCH_CHECK("gemm_tiled128");
        return 0;
    }
    const dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
    IA_CHECK(grid.y <= 65535, "gemm_tiled: %d rows exceed the grid", M);
    if (in_dtype == IA_F32 && out_dtype == IA_F32)
        gemm_tiled_kernel<float, float><<<grid, 256, 0, stream>>>((float*)out, (const float*)x, (const float*)w, M, N, K);
    else if (in_dtype == IA_BF16 && out_dtype == IA_BF16)
        gemm_tiled_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    else if (in_dtype == IA_BF16 && out_dtype == IA_F32)
        gemm_tiled_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((float*)out, (const bf16_t*)x, (const bf16_t*)w, M, N, K);
    else
        IA_CHECK(false, "gemm_tiled: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
    IA_LAUNCH_CHECK("gemm_tiled");
    return 0;
}

// ---- skinny bfloat16 product on the matrix cores ----------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define SK_KSTEP 32     // k per MFMA
#define SK_MAX_WAVES 16

// Operand layout of v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16) of A and column
// (l % 16) of B, each with the eight k values (l / 16) * 8 .. + 8; lane l receives
// D[4 * (l / 16) + i][l % 16], i = 0..3.  A is a tile of 16 weight rows (output features),
// B the activations (columns = batch rows).
//
// A block owns 16 * RT output features; its waves split k between them in contiguous ranges
// (a wave streams RT * 16 rows of `kper` * 64 bytes each) and add their tiles up through
// shared memory in wave order.  How k is split depends on the weight's shape alone, so a
// row's rounding does not depend on the batch it is in.  MT tiles of 16 batch rows share
// every weight load.  DUAL: the weight holds two matrices stacked along the output ([gate;
// up], N features each) and the result is silu(gate . x) * (up . x).
//
// STAGE (one tile of batch rows only): the activations do not come to the MFMA operand straight
// from memory (a load of 16 rows x 64 bytes asks for 16 half cache lines, and with every block
// asking for the same few lines of x the caches' request rate, not the memory, sets the pace), but
// a wave brings its piece of x for a chunk of k steps in whole rows (512 contiguous bytes a row,
// two rows a load), puts it into its own corner of shared memory and reads the operand layout from
// there.  Measured on the logits head at 8 rows: 4.8 -> 5.9 TB/s.
#define SK_STAGE_PAD 16     // bytes between staged rows, against bank conflicts

// A residual stream around the product, so that no kernel of its own adds and norms between two
// products (decode steps: such a kernel is all launch and latency).  The norm of a row,
// x * rsqrt(mean(x^2) + eps) * g, is split in two: the product before the norm forms x * g while it
// has the row's new values at hand, and the product after it applies the row's scale to its sums.
//   resid / sums_out / scaled_out / next_w: the product is not stored but added to `resid` [M, N] in place, as
//     the add kernel would (the product rounded to the storage precision, the sum formed in 32-bit and
//     rounded); the block writes the sum of squares of its 16 features of every new row to
//     sums_out[row][block] and the new values times next_w (or 1 + next_w) to scaled_out [M, N].
//   sums_in: x holds such scaled rows, and sums_in[row][0 .. n_sums) their sums of squares: every sum of
//     the product is multiplied by rsqrt(sum of the row's sums_in / K + eps) before it is rounded.
//   bias: a vector that is added to every row of the product (after the scale, before the activation, the
//     rounding and the sum into the stream).
// One rounding of the normed value, as in the norm kernel, at another place (before the scale instead of
// after it); the sum of squares is added up in another order than there.
struct SkinnyStream {
    bf16_t* resid;
    float* sums_out;
    bf16_t* scaled_out;
    const float* next_w;
    const float* sums_in;
    int n_sums;
    float eps;
    int add_one;
    int act;                    // DUAL: the gate's activation (IA_ACT_*)
    const bf16_t* bias;         // [N] ([2 N] with DUAL), added to every row's sums before anything is rounded; or null
};

// STAGE: 0, or the k steps of a staged chunk (8 or 16).
template <int MT, int RT, bool DUAL, int STAGE>
__global__ __launch_bounds__(SK_MAX_WAVES * IA_WAVE) void gemm_skinny_kernel(
    void* __restrict__ out, int out_f32, const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
    int M, int N, int K, int kper, int rpb, int m_base, int rot_mul, const SkinnyStream st) {
    constexpr int NA = DUAL ? 2 : 1;
    static_assert(!STAGE || MT == 1, "staging holds one tile of batch rows");
    extern __shared__ f32x4 red[];      // [waves][NA][RT][MT][64], then with STAGE [waves][rows][chunk of x]
    const int lane = threadIdx.x & (IA_WAVE - 1);
    const int wave = threadIdx.x / IA_WAVE;
    const int waves = blockDim.x / IA_WAVE;
    const int n0 = blockIdx.x * rpb;
    const int r = lane & 15, g = lane >> 4;
    const int ksteps = (K + SK_KSTEP - 1) / SK_KSTEP;
    const int ks0 = wave * kper, ks1 = ks0 + kper < ksteps ? ks0 + kper : ksteps;

    const bf16_t* wrow[NA][RT];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            // (rows beyond the block's share or beyond N read the last row inside both: their sums are never stored)
            const int j = t * 16 + r < rpb ? t * 16 + r : rpb - 1;
            const int n = n0 + j;
            wrow[a][t] = w + ((size_t)a * N + (n < N ? n : N - 1)) * K + g * 8;
        }
    // Batch rows beyond M are read from row 0: their columns of the result are never stored.
    const bf16_t* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = m_base + t * 16 + r;
        xrow[t] = x + (size_t)(m < M ? m : 0) * K + g * 8;
    }
    f32x4 acc[NA][RT][MT];
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int u = 0; u < MT; ++u) acc[a][t][u] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // Blocks start at different places of their k range and wrap around: rows are a power of
    // two apart in memory, and blocks that walk them in step would all ask the same few memory
    // channels at any moment.  The order of the sum depends on the block (the output feature)
    // only, never on the batch.  Whole steps run without a condition; a last step that K does
    // not fill is done apart, with zeros beyond K.
    // A chunk of k steps has all its loads under way before its first product: a wave is one of
    // few on its SIMD when the weight is small, and what it has in flight is what hides the memory's
    // latency.
    constexpr int UNROLL = STAGE ? STAGE : (NA * RT * MT >= 8) ? 2 : (NA * RT * MT >= 4 ? 4 : (NA * RT * MT == 2 ? 8 : 16));
    constexpr int STAGE_PITCH = UNROLL * 2 * SK_KSTEP + SK_STAGE_PAD;      // bytes of a staged row
    constexpr int STAGE_LANES = UNROLL * 4;                               // lanes that bring one row
    const int stage_rows = M - m_base < 16 ? M - m_base : 16;
    char* const stage = (char*)(red + (size_t)waves * NA * RT * MT * IA_WAVE) + (size_t)wave * stage_rows * STAGE_PITCH;
    // What the end of the kernel needs of a stream is asked for now, so that its way from memory lies behind the
    // product: the rows' sums of squares (a row a wave, 16 bytes a lane), and for the wave that stores, the
    // stream's old values and the next norm's weights.
    __shared__ float ss_row[16];
    constexpr int SS_ROWS = (16 + 7) / 8;                   // rows a wave when eight waves share out sixteen
    constexpr int SS_VEC = 2;                               // 16-byte pieces a lane: rows of up to 512 sums
    float4 ss_mine[SS_ROWS][SS_VEC];
    const bool ss_wide = st.sums_in != nullptr && (st.n_sums & 3) == 0 && st.n_sums <= 4 * IA_WAVE * SS_VEC;
    if (ss_wide) {                                          // (a stream has one tile of batch rows)
#pragma unroll
        for (int j = 0; j < SS_ROWS; ++j) {
            const int m = wave + j * waves;
#pragma unroll
            for (int v = 0; v < SS_VEC; ++v) {
                const int at = 4 * (lane + v * IA_WAVE);
                ss_mine[j][v] = (m < stage_rows && at < st.n_sums)
                                    ? *(const float4*)(st.sums_in + (size_t)(m_base + m) * st.n_sums + at)
                                    : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    }
    uint2 resid_old = make_uint2(0u, 0u);
    float4 next_w4 = make_float4(0.f, 0.f, 0.f, 0.f);
    const bool resid_ahead = st.resid != nullptr && wave == 0 && ((N | n0) & 3) == 0 && n0 + 4 * g + 3 < N &&
                             4 * g + 3 < rpb && m_base + r < M;
    if (resid_ahead) {
        resid_old = *(const uint2*)(st.resid + (size_t)(m_base + r) * N + n0 + 4 * g);
        if (st.scaled_out != nullptr) next_w4 = *(const float4*)(st.next_w + n0 + 4 * g);
    }
    const int whole = K / SK_KSTEP;                         // steps that lie inside K entirely
    const int ke = ks1 < whole ? ks1 : whole;
    const int len = ke - ks0;
    // (in steps of 16 whatever the chunk: the order of a row's sum must not depend on the variant
    // of the kernel that the batch size picks)
    const int rot = len > 0 ? (int)((blockIdx.x * (unsigned)rot_mul) % (unsigned)len) / 16 * 16 : 0;
    for (int part = 0; part < 2; ++part) {
        const int pa = part == 0 ? ks0 + rot : ks0, pb = part == 0 ? ke : ks0 + rot;
        int ks = pa;
        for (; ks + UNROLL <= pb; ks += UNROLL) {
            uint4 a[UNROLL][NA][RT], b[UNROLL][MT];
            if (STAGE) {
                // the loads of x go first: loads come back in the order they were asked for
                const int sub = lane / STAGE_LANES, piece = lane % STAGE_LANES;
                for (int m = 0; m < stage_rows; m += IA_WAVE / STAGE_LANES) {
                    const int row = m + sub;
                    if (row < stage_rows)
                        *(uint4*)(stage + row * STAGE_PITCH + piece * 16) =
                            *(const uint4*)(x + (size_t)(m_base + row) * K + (size_t)ks * SK_KSTEP + piece * 8);
                }
            }
#pragma unroll
            for (int i = 0; i < UNROLL; ++i)
#pragma unroll
                for (int q = 0; q < NA; ++q)
#pragma unroll
                    for (int t = 0; t < RT; ++t) a[i][q][t] = *(const uint4*)(wrow[q][t] + (ks + i) * SK_KSTEP);
            if (STAGE) {
                // one wave's own corner: its shared-memory operations run in program order
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const char* mine = stage + (r < stage_rows ? r : 0) * STAGE_PITCH + g * 16;
#pragma unroll
                for (int i = 0; i < UNROLL; ++i) b[i][0] = *(const uint4*)(mine + i * 2 * SK_KSTEP);
            } else {
#pragma unroll
                for (int i = 0; i < UNROLL; ++i)
#pragma unroll
                    for (int u = 0; u < MT; ++u) b[i][u] = *(const uint4*)(xrow[u] + (ks + i) * SK_KSTEP);
            }
#pragma unroll
            for (int i = 0; i < UNROLL; ++i)
#pragma unroll
                for (int u = 0; u < MT; ++u)
#pragma unroll
                    for (int q = 0; q < NA; ++q)
#pragma unroll
                        for (int t = 0; t < RT; ++t)
                            acc[q][t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                __builtin_bit_cast(bf16x8, a[i][q][t]), __builtin_bit_cast(bf16x8, b[i][u]), acc[q][t][u], 0, 0, 0);
        }
        if constexpr (!STAGE) {
            // what the chunks leave: a chunk of 8 and one of 4 steps before single steps, each with its
            // loads under way together (a wave's k range need not be a multiple of the chunk)
            auto short_chunk = [&](auto steps) {
                constexpr int C = decltype(steps)::value;
                if (ks + C > pb) return;
                uint4 a[C][NA][RT], b[C][MT];
#pragma unroll
                for (int i = 0; i < C; ++i) {
#pragma unroll
                    for (int q = 0; q < NA; ++q)
#pragma unroll
                        for (int t = 0; t < RT; ++t) a[i][q][t] = *(const uint4*)(wrow[q][t] + (ks + i) * SK_KSTEP);
#pragma unroll
                    for (int u = 0; u < MT; ++u) b[i][u] = *(const uint4*)(xrow[u] + (ks + i) * SK_KSTEP);
                }
#pragma unroll
                for (int i = 0; i < C; ++i)
#pragma unroll
                    for (int u = 0; u < MT; ++u)
#pragma unroll
                        for (int q = 0; q < NA; ++q)
#pragma unroll
                            for (int t = 0; t < RT; ++t)
                                acc[q][t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                    __builtin_bit_cast(bf16x8, a[i][q][t]), __builtin_bit_cast(bf16x8, b[i][u]), acc[q][t][u], 0, 0, 0);
                ks += C;
            };
            if constexpr (UNROLL > 8) short_chunk(std::integral_constant<int, 8>());
            if constexpr (UNROLL > 4) short_chunk(std::integral_constant<int, 4>());
        }
        for (; ks < pb; ++ks) {
            const int k0 = ks * SK_KSTEP;
#pragma unroll
            for (int u = 0; u < MT; ++u) {
                const uint4 b = *(const uint4*)(xrow[u] + k0);
#pragma unroll
                for (int q = 0; q < NA; ++q)
#pragma unroll
                    for (int t = 0; t < RT; ++t) {
                        const uint4 a = *(const uint4*)(wrow[q][t] + k0);
                        acc[q][t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc[q][t][u], 0, 0, 0);
                    }
            }
        }
    }
    if (ks1 > whole && ks0 <= whole) {                      // the step that K leaves unfilled
        const int k0 = whole * SK_KSTEP;
        const bool kin = k0 + g * 8 < K;                    // K is a multiple of 8: a piece is in or out
        const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int u = 0; u < MT; ++u) {
            const uint4 b = kin ? *(const uint4*)(xrow[u] + k0) : zero;
#pragma unroll
            for (int q = 0; q < NA; ++q)
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    const uint4 a = kin ? *(const uint4*)(wrow[q][t] + k0) : zero;
                    acc[q][t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc[q][t][u], 0, 0, 0);
                }
        }
    }
    if (st.sums_in != nullptr) {
        // every row's sum of squares, a row a wave: a lane's four neighbours first, then across the lanes
        auto one_by_one = [&](int m) {
            float ss = 0.f;
            for (int b = lane; b < st.n_sums; b += IA_WAVE) ss += st.sums_in[(size_t)(m_base + m) * st.n_sums + b];
            return ss;
        };
#pragma unroll
        for (int j = 0; j < SS_ROWS; ++j) {
            const int m = wave + j * waves;
            if (m >= stage_rows) continue;
            float ss;
            if (ss_wide) {
                ss = ((ss_mine[j][0].x + ss_mine[j][0].y) + ss_mine[j][0].z) + ss_mine[j][0].w;
#pragma unroll
                for (int v = 1; v < SS_VEC; ++v)
                    ss += ((ss_mine[j][v].x + ss_mine[j][v].y) + ss_mine[j][v].z) + ss_mine[j][v].w;
            } else {
                ss = one_by_one(m);
            }
            ss = wave_sum(ss);
            if (lane == 0) ss_row[m] = ss;
        }
        for (int m = wave + SS_ROWS * waves; m < stage_rows; m += waves) {
            const float ss = wave_sum(one_by_one(m));
            if (lane == 0) ss_row[m] = ss;
        }
    }
    if (waves > 1) {
#pragma unroll
        for (int q = 0; q < NA; ++q)
#pragma unroll
            for (int t = 0; t < RT; ++t)
#pragma unroll
                for (int u = 0; u < MT; ++u)
                    red[(((wave * NA + q) * RT + t) * MT + u) * IA_WAVE + lane] = acc[q][t][u];
        __syncthreads();
    } else if (st.sums_in != nullptr) {
        __syncthreads();
    }
    // the tiles are shared out between the waves for the sum and the store
    int tile = 0;
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int u = 0; u < MT; ++u, ++tile) {
            if (tile % waves != wave) continue;
            f32x4 s[NA];
#pragma unroll
            for (int q = 0; q < NA; ++q) {
                if (waves > 1) {
                    s[q] = red[((q * RT + t) * MT + u) * IA_WAVE + lane];
                    for (int wv = 1; wv < waves; ++wv) {
                        const f32x4 o = red[(((wv * NA + q) * RT + t) * MT + u) * IA_WAVE + lane];
                        s[q][0] += o[0]; s[q][1] += o[1]; s[q][2] += o[2]; s[q][3] += o[3];
                    }
                } else {
                    s[q] = acc[q][t][u];
                }
            }
            const int m = m_base + u * 16 + r;
            if constexpr (MT == 1) {
                if (st.sums_in != nullptr) {
                    const float scale = 1.0f / sqrtf(ss_row[r < stage_rows ? r : 0] / (float)K + st.eps);
#pragma unroll
                    for (int q = 0; q < NA; ++q) { s[q][0] *= scale; s[q][1] *= scale; s[q][2] *= scale; s[q][3] *= scale; }
                }
            }
            if (st.bias != nullptr) {
                const int fb = n0 + t * 16 + 4 * g;
#pragma unroll
                for (int q = 0; q < NA; ++q)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (fb + i < N) s[q][i] += bf16_bits_to_f32(st.bias[(size_t)q * N + fb + i].bits);
            }
            if constexpr (!DUAL && RT == 1 && MT == 1) {
                if (st.resid != nullptr) {
                    // (all lanes of the wave stay for the sums; rows and features outside add nothing)
                    const int nb = n0 + 4 * g;
                    float sq = 0.f;
                    if (resid_ahead) {
                        const uint16_t old[4] = {(uint16_t)resid_old.x, (uint16_t)(resid_old.x >> 16),
                                                 (uint16_t)resid_old.y, (uint16_t)(resid_old.y >> 16)};
                        const float gw[4] = {next_w4.x, next_w4.y, next_w4.z, next_w4.w};
                        uint16_t h[4], hw[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float product = bf16_bits_to_f32(f32_to_bf16_bits(s[0][i]));
                            h[i] = f32_to_bf16_bits(product + bf16_bits_to_f32(old[i]));
                            const float hf = bf16_bits_to_f32(h[i]);
                            sq += hf * hf;
                            hw[i] = f32_to_bf16_bits(hf * (st.add_one ? 1.0f + gw[i] : gw[i]));
                        }
                        *(uint2*)(st.resid + (size_t)m * N + nb) =
                            make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
                        if (st.scaled_out != nullptr)
                            *(uint2*)(st.scaled_out + (size_t)m * N + nb) =
                                make_uint2((uint32_t)hw[0] | ((uint32_t)hw[1] << 16), (uint32_t)hw[2] | ((uint32_t)hw[3] << 16));
                    } else if (m < M) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            if (nb + i >= N || 4 * g + i >= rpb) continue;
                            bf16_t* at = st.resid + (size_t)m * N + nb + i;
                            const float product = bf16_bits_to_f32(f32_to_bf16_bits(s[0][i]));
                            const uint16_t h = f32_to_bf16_bits(product + bf16_bits_to_f32(at->bits));
                            at->bits = h;
                            const float hf = bf16_bits_to_f32(h);
                            sq += hf * hf;
                            if (st.scaled_out != nullptr) {
                                const float gw = st.next_w[nb + i];
                                st.scaled_out[(size_t)m * N + nb + i].bits = f32_to_bf16_bits(hf * (st.add_one ? 1.0f + gw : gw));
                            }
                        }
                    }
                    sq += __shfl_xor(sq, 16, IA_WAVE);
                    sq += __shfl_xor(sq, 32, IA_WAVE);
                    if (g == 0 && m < M) st.sums_out[(size_t)m * gridDim.x + blockIdx.x] = sq;
                    continue;
                }
            }
            if (m >= M) continue;
            const int nb = n0 + t * 16 + 4 * g;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (DUAL) {
                    // the first product is rounded to the storage precision before the
                    // activation, as the two-kernel path rounds it
                    const float gate = bf16_bits_to_f32(f32_to_bf16_bits(s[0][i]));
                    const float up = bf16_bits_to_f32(f32_to_bf16_bits(s[NA - 1][i]));
                    v[i] = gate_act(gate, st.act) * up;
                } else {
                    v[i] = s[0][i];
                }
            }
            if (nb + 3 < N && ((N | n0) & 3) == 0 && t * 16 + 4 * g + 3 < rpb) {
                if (out_f32) {
                    *(f32x4*)((float*)out + (size_t)m * N + nb) = (f32x4){v[0], v[1], v[2], v[3]};
                } else {
                    uint2 pk;
                    pk.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
                    pk.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
                    *(uint2*)((bf16_t*)out + (size_t)m * N + nb) = pk;
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (nb + i >= N || t * 16 + 4 * g + i >= rpb) continue;
                    if (out_f32) ((float*)out)[(size_t)m * N + nb + i] = v[i];
                    else ((bf16_t*)out)[(size_t)m * N + nb + i].bits = f32_to_bf16_bits(v[i]);
                }
            }
        }
}

// Tuning knobs (ia_gemm_skinny_tune): waves wanted on the chip before k stops being split,
// fewest k steps worth a wave, and the stagger of the blocks' starting points.
static int g_target_waves = 2048, g_min_ksteps = 8, g_rot_mul = 5, g_min_waves = 8, g_stage = 1;

extern "C" void ia_gemm_skinny_tune(int target_waves, int min_ksteps, int rot_mul, int min_waves, int stage) {
    g_target_waves = target_waves; g_min_ksteps = min_ksteps; g_rot_mul = rot_mul; g_min_waves = min_waves;
    g_stage = stage;
}

static int skinny_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    return cus;
}

// Output features a block owns (one tile of rows a wave: 8 to 16 of the tile's 16).  A weight whose blocks of 16
// go round the compute units once or twice and leave a round partly filled (5,120 features: 320 blocks on 256
// units) is read at the pace of the units that got two; smaller blocks fill the rounds (10 features: 512 blocks).
// Depends on the number of features and the chip alone.
static int skinny_rows_per_block(int N, int rt) {
    if (rt != 1) return 16 * rt;
    const int cus = skinny_cus();
    if ((N + 15) / 16 >= 8 * cus) return 16;
    // rows of the fullest compute unit; the largest block within a sixteenth of the best (smaller blocks spend
    // more of their time starting and adding up)
    auto fullest = [&](int rows) { return ((N + rows - 1) / rows + cus - 1) / cus * rows; };
    int least = fullest(16);
    for (int rows = 15; rows >= 8; --rows) least = fullest(rows) < least ? fullest(rows) : least;
    int best = 16;
    while (fullest(best) * 16 > least * 17) --best;
    return best;
}

// How many waves share k, and how many k steps each takes: a function of the weight's shape, of the row
// tiling and of the chip only.
#define SK_CHUNK 16     // k steps of the longest chunk a wave has in flight
// Weights whose blocks go round the compute units three times or more stream for long (gate|up, a logits head);
// the others are read in one burst.
static bool skinny_tall(int blocks) { return blocks >= 3 * skinny_cus(); }

static void skinny_split(int N, int K, int rt, int tiles_per_wave, int* waves_out, int* kper_out) {
    const int rpb = skinny_rows_per_block(N, rt);
    const int groups = (N + rpb - 1) / rpb;
    const int ksteps = (K + SK_KSTEP - 1) / SK_KSTEP;
    // the waves' tiles meet in shared memory: at most 64 KiB of it
    const int most = 65536 / (tiles_per_wave * IA_WAVE * (int)sizeof(f32x4));
    // (a logits head, two row tiles a wave, has blocks to spare: half as many waves with ranges twice as long read it
    // faster, 151,936 x 4,096 at 8 rows 228 -> 215 us, and leave room for the staging area of 16 rows, 296 -> 240 us)
    // So does a tall weight whose halved number of waves still takes whole chunks of 16 steps: gate|up of
    // 2 x 12,288 x 4,096 at 8 rows 40.1 -> 38.8 us, at 16 rows 49.4 -> 42.8 (5,120 wide it does not: 72.4 -> 74.4 us).
    const int half = (g_min_waves + 1) / 2;
    const int min_waves = (rt == 2 || (skinny_tall(groups) && ksteps % (SK_CHUNK * half) == 0)) ? half : g_min_waves;
    int waves = 1;
    while (waves * 2 <= SK_MAX_WAVES && waves * 2 <= most && ksteps / (waves * 2) >= g_min_ksteps &&
           (groups * waves < g_target_waves || waves < min_waves))
        waves *= 2;
    int kper = (ksteps + waves - 1) / waves;
    // A range that is no multiple of the chunk ends in short chunks and single steps, each of which waits
    // for the memory on its own, and keeps the staged variants out (a width of 5,120 leaves 20 steps to each of
    // eight waves).  Long rows are shared out in whole chunks instead, of 8 steps for tall weights (what their
    // staged variant takes) and of 16 for the others, between no more waves than by the rule above: blocks of more
    // than eight waves streamed slower (24,576 x 5,120 at 8 rows: 7 waves of 24 steps 55.7 us, 10 of 16 62.5;
    // 5,120 x 17,408 at one row: 7 waves of 80 steps 35.0 us, 12 of 48 38.6; 5,120 x 5,120 at 8 rows: 5 waves of
    // 32 steps 14.4 us, 10 of 16 16.0), and their staging areas leave room for one block a compute unit only.  The
    // last wave takes what is left.
    if (ksteps >= 8 * SK_CHUNK && kper % SK_CHUNK != 0) {
        const int unit = skinny_tall(groups) ? 8 : SK_CHUNK;
        const int chunks = (ksteps + unit - 1) / unit;
        kper = (chunks + waves - 1) / waves * unit;
        waves = (ksteps + kper - 1) / kper;
    }
    *waves_out = waves;
    *kper_out = kper;
}

#define SK_STAGE_LDS_MOST (80 * 1024)         // two blocks a compute unit
#define SK_STAGE16_LDS_MOST (160 * 1024)     // one block a compute unit: all of its shared memory
#define SK_SCALES_RESERVE 256                // the rows' sums of squares: static shared memory beside the launch's own area

// Shared memory beyond 64 KiB has to be asked for, once per instantiation.
template <int MT, int RT, bool DUAL, int STAGE>
static int skinny_ask_shared(int bytes) {
    static bool asked = false;
    if (!asked) {
        const hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_kernel<MT, RT, DUAL, STAGE>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        IA_CHECK(e == hipSuccess, "gemm_skinny: cannot ask for %d bytes of shared memory: %s", bytes, hipGetErrorString(e));
        asked = true;
    }
    return 0;
}

template <int MT, int RT, bool DUAL>
static int launch_skinny(void* out, int out_f32, const bf16_t* x, const bf16_t* w, int M, int N, int K,
                         int m_base, const SkinnyStream& st, hipStream_t stream) {
    int waves, kper;
    skinny_split(N, K, RT, (DUAL ? 2 : 1) * RT * MT, &waves, &kper);
    // the kernel places the staging area behind the tiles of all waves, also when there is one wave
    const size_t tiles = (size_t)waves * (DUAL ? 2 : 1) * RT * MT * IA_WAVE * sizeof(f32x4);
    const int rpb = skinny_rows_per_block(N, RT);
    const unsigned grid = (unsigned)((N + rpb - 1) / rpb);
    if constexpr (MT == 1) {
        const int rows = M - m_base < 16 ? M - m_base : 16;
        const size_t staged8 = tiles + (size_t)waves * rows * (8 * 2 * SK_KSTEP + SK_STAGE_PAD);
        const size_t staged16 = tiles + (size_t)waves * rows * (16 * 2 * SK_KSTEP + SK_STAGE_PAD);
        int stage = 0;
        if (g_stage && rows >= 1 && skinny_tall((int)grid)) {
            // Staging pays where blocks stream for long: with at least three blocks for every compute unit (also with
            // one batch row: gate|up 39.2 -> 37.0 us, a decode step of one request 3.97 -> 3.84 ms), with whole chunks of 8 k steps in a wave's
            // range, and while the staging area leaves room for two blocks on a compute unit (eight waves: up to 15
            // rows; at 16 rows, one block a unit, a decode step at the sizes of an 8 B model took 5.73 ms against
            // 5.44 without staging; seven waves, a width of 5,120: all 16).  Measured at 8 rows: gate|up 46 -> 40 us,
            // logits head 261 -> 224 us; at 14 rows a decode step of the 14B shape 10.9 -> 9.7 ms.
            if (kper >= 8 && staged8 <= SK_STAGE_LDS_MOST - SK_SCALES_RESERVE) stage = 8;
        } else if (g_stage && rows >= 1 && !DUAL && RT == 1) {
            // A weight that one or two rounds of blocks cover (o, down, qkv) is read in one burst, and what counts
            // is how much a wave has in flight: chunks of 16 steps, as much as without staging, and up to
            // all of a compute unit's shared memory for its block.  Measured at 8 rows: down 25.6 -> 22.3 us,
            // o 11.5 -> 9.9, qkv 16.8 -> 14.2; at 16 rows 30.4 -> 24.5, 12.9 -> 10.6, 19.1 -> 16.8.  (From 9 rows on
            // the area leaves room for one block of qkv's 384 on a compute unit, and they go in two rounds;
            // chunks of 8, which keep it one round, were no faster: 15.8 against 16.4 us at 10 rows, 17.4
            // against 16.7 at 16.)
            if (kper % 16 == 0 && staged16 <= SK_STAGE16_LDS_MOST - SK_SCALES_RESERVE) stage = 16;
        }
        if (stage == 8) {
            if (skinny_ask_shared<MT, RT, DUAL, 8>(SK_STAGE_LDS_MOST - SK_SCALES_RESERVE)) return 1;
            gemm_skinny_kernel<MT, RT, DUAL, 8><<<grid, waves * IA_WAVE, staged8, stream>>>(
                out, out_f32, x, w, M, N, K, kper, rpb, m_base, g_rot_mul, st);
            return 0;
        }
        if constexpr (!DUAL && RT == 1) {
            if (stage == 16) {
                if (skinny_ask_shared<MT, RT, DUAL, 16>(SK_STAGE16_LDS_MOST - SK_SCALES_RESERVE)) return 1;
                gemm_skinny_kernel<MT, RT, DUAL, 16><<<grid, waves * IA_WAVE, staged16, stream>>>(
                    out, out_f32, x, w, M, N, K, kper, rpb, m_base, g_rot_mul, st);
                return 0;
            }
        }
    }
    gemm_skinny_kernel<MT, RT, DUAL, 0><<<grid, waves * IA_WAVE, waves > 1 ? tiles : 0, stream>>>(
        out, out_f32, x, w, M, N, K, kper, rpb, m_base, g_rot_mul, st);
    return 0;
}

static int skinny_product(void* out, const void* x, const void* w, int M, int N, int K, int out_dtype, int dual,
                          SkinnyStream st, hipStream_t stream) {
    IA_CHECK(M >= 0 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    IA_CHECK(dual >= 0 && dual <= IA_ACT_LAST, "gemm_skinny: unknown activation %d", dual);
    st.act = dual;
    IA_CHECK(K % 8 == 0, "gemm_skinny: K=%d must be a multiple of 8 (use the tiled product)", K);
    IA_CHECK(out_dtype == IA_F32 || out_dtype == IA_BF16, "gemm_skinny: unknown output dtype %d", out_dtype);
    IA_CHECK((((uintptr_t)x | (uintptr_t)w) & 15) == 0, "gemm_skinny: x and w must be 16-byte aligned");
    IA_CHECK((((uintptr_t)out) & 15) == 0, "gemm_skinny: out must be 16-byte aligned");
    const bool streams = st.resid != nullptr || st.sums_in != nullptr;
    IA_CHECK(!streams || (M <= 16 && N < 65536), "gemm_skinny: a residual stream around the product takes up to 16 rows "
             "and fewer than 65536 features, got M=%d N=%d", M, N);
    IA_CHECK(st.resid == nullptr || (!dual && st.sums_out != nullptr && (st.scaled_out == nullptr) == (st.next_w == nullptr)),
             "gemm_skinny: the sum into a residual stream is for plain products, needs a place for the sums of squares, "
             "and the next norm's weight together with a place for the scaled rows");
    IA_CHECK(st.sums_in == nullptr || st.n_sums > 0, "gemm_skinny: scaled rows come with their sums of squares");
    IA_CHECK((((uintptr_t)st.resid | (uintptr_t)st.scaled_out | (uintptr_t)st.next_w) & 15) == 0,
             "gemm_skinny: the stream's arrays must be 16-byte aligned");
    IA_CHECK((((uintptr_t)st.bias) & 1) == 0, "gemm_skinny: the bias must be 2-byte aligned");
    if (M == 0) return 0;
    const int out_f32 = out_dtype == IA_F32;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    for (int m_base = 0; m_base < M; m_base += 64) {
        const int rows = M - m_base;
        int rc = 0;
        if (dual) {
            if (rows <= 16) rc = launch_skinny<1, 1, true>(out, out_f32, xb, wb, M, N, K, m_base, st, stream);
            else if (rows <= 32) rc = launch_skinny<2, 1, true>(out, out_f32, xb, wb, M, N, K, m_base, st, stream);
            else rc = launch_skinny<4, 1, true>(out, out_f32, xb, wb, M, N, K, m_base, st, stream);
        } else {
            // very tall weights (a logits head) have blocks to spare: two row tiles a wave halve the
            // loads of the activations
            if (rows <= 16 && N >= 65536) rc = launch_skinny<1, 2, false>(out, out_f32, xb, wb, M, N, K, m_base, st, stream);
            else if (rows <= 16) rc = launch_skinny<1, 1, false>(out, out_f32, xb, wb, M, N, K, m_base, st, stream);
            else if (rows <= 32) rc = launch_skinny<2, 1, false>(out, out_f32, xb, wb, M, N, K, m_base, st, stream);
            else rc = launch_skinny<4, 1, false>(out, out_f32, xb, wb, M, N, K, m_base, st, stream);
        }
        if (rc) return rc;
        IA_LAUNCH_CHECK("gemm_skinny");
    }
    return 0;
}

// out[M, N] = x[M, K] . w[N, K]^T, or with `dual` (an activation, IA_ACT_*) out[M, N] = act(x . w[0:N]^T) * (x . w[N:2N]^T);
// bias [N] ([2 N] with dual) in bfloat16, or null: added to every row of the product(s).
extern "C" int ia_gemm_skinny_bf16(void* out, const void* x, const void* w, const void* bias, int M, int N, int K,
                                   int out_dtype, int dual, hipStream_t stream) {
    const SkinnyStream none = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0.f, 0, 0, (const bf16_t*)bias};
    return skinny_product(out, x, w, M, N, K, out_dtype, dual, none, stream);
}

// Blocks of the plain product with N output features: the columns of its sums of squares.
// Features of a block of the plain product.
extern "C" int ia_gemm_skinny_block_rows(int N) { return skinny_rows_per_block(N, 1); }

extern "C" int ia_gemm_skinny_blocks(int N) {
    const int rpb = skinny_rows_per_block(N, 1);
    return (N + rpb - 1) / rpb;
}

// The product with a residual stream around it (up to 16 rows; see SkinnyStream).
//   resid != null (plain products): resid[M, N] += product in place, nothing goes to `out` (may be null);
//     sums_out[M][ia_gemm_skinny_blocks(N)] receives the sums of squares of the new rows, block by block, and
//     scaled_out[M, N] (may be null, with next_w) the new rows times next_w [N] (1 + next_w with add_one).
//   sums_in != null: x [M, K] holds such scaled rows and sums_in[M][n_sums] their sums of squares; the
//     product's sums are multiplied by rsqrt(sum / K + eps) before anything else happens to them.
extern "C" int ia_gemm_skinny_stream(void* out, const void* x, const void* w, const void* bias, int M, int N, int K, int out_dtype,
                                     int dual, void* resid, float* sums_out, void* scaled_out, const float* next_w,
                                     int add_one, const float* sums_in, int n_sums, float eps, hipStream_t stream) {
    const SkinnyStream st = {(bf16_t*)resid, sums_out, (bf16_t*)scaled_out, next_w, sums_in, n_sums, eps, add_one, 0,
                             (const bf16_t*)bias};
    IA_CHECK(out != nullptr || resid != nullptr, "gemm_skinny: no place for the result");
    return skinny_product(out, x, w, M, N, K, out_dtype, dual, st, stream);
}
