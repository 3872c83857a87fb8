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
//     the waves of a block (and, for short outputs, several blocks) split k between them;
//     partial tiles are summed in a fixed order.
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

// in_dtype: storage of x and w; out_dtype: storage of the result.
extern "C" int ia_gemm_tiled(void* out, const void* x, const void* w, int M, int N, int K,
                             int in_dtype, int out_dtype, hipStream_t stream) {
    IA_CHECK(M >= 0 && N > 0 && K > 0, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
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

#define SK_WAVES 4
#define SK_ROWS 16      // weight rows (output features) per block
#define SK_KSTEP 32     // k per MFMA

// Operand layout of v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16) of A and column
// (l % 16) of B, each with the eight k values (l / 16) * 8 .. + 8; lane l receives
// D[4 * (l / 16) + i][l % 16], i = 0..3.  A is the weight tile (rows = output features),
// B the activations (columns = batch rows).
template <int MT>
__global__ __launch_bounds__(SK_WAVES * IA_WAVE) void gemm_skinny_kernel(
    float* __restrict__ partial,        // [splits, M, N] when gridDim.y > 1, else unused
    void* __restrict__ out, int out_f32,
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, int M, int N, int K, int m_base) {
    __shared__ f32x4 red[SK_WAVES][MT][IA_WAVE];
    const int lane = threadIdx.x & (IA_WAVE - 1);
    const int wave = threadIdx.x / IA_WAVE;
    const int n0 = blockIdx.x * SK_ROWS;
    const int r = lane & 15, g = lane >> 4;
    const int n_read = n0 + r < N ? n0 + r : N - 1;
    const bf16_t* wrow = w + (size_t)n_read * K + g * 8;
    const int ksteps = (K + SK_KSTEP - 1) / SK_KSTEP;
    const int stride = SK_WAVES * gridDim.y;

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = m_base + t * 16 + r;
        xok[t] = m < M;
        xrow[t] = x + (size_t)(xok[t] ? m : 0) * K + g * 8;
    }
    const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll 4
    for (int ks = blockIdx.y * SK_WAVES + wave; ks < ksteps; ks += stride) {
        const int k0 = ks * SK_KSTEP;
        const bool kin = k0 + g * 8 < K;          // K is a multiple of 8: a piece is in or out
        const uint4 a = kin ? *(const uint4*)(wrow + k0) : zero;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const uint4 b = (kin && xok[t]) ? *(const uint4*)(xrow[t] + k0) : zero;
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                             __builtin_bit_cast(bf16x8, b), acc[t], 0, 0, 0);
        }
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) red[wave][t][lane] = acc[t];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        f32x4 s = red[0][t][lane];
#pragma unroll
        for (int wv = 1; wv < SK_WAVES; ++wv) {
            const f32x4 o = red[wv][t][lane];
            s[0] += o[0]; s[1] += o[1]; s[2] += o[2]; s[3] += o[3];
        }
        const int m = m_base + t * 16 + r;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + 4 * g + i;
            if (n >= N) continue;
            if (gridDim.y > 1)
                partial[((size_t)blockIdx.y * M + m) * N + n] = s[i];
            else if (out_f32)
                ((float*)out)[(size_t)m * N + n] = s[i];
            else
                ((bf16_t*)out)[(size_t)m * N + n].bits = f32_to_bf16_bits(s[i]);
        }
    }
}

__global__ void gemm_split_reduce_kernel(void* __restrict__ out, int out_f32, const float* __restrict__ partial,
                                         int splits, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        float s = partial[i];
        for (int p = 1; p < splits; ++p) s += partial[(size_t)p * total + i];
        if (out_f32) ((float*)out)[i] = s;
        else ((bf16_t*)out)[i].bits = f32_to_bf16_bits(s);
    }
}

// `splits` > 1 needs `partial` with room for splits * M * N floats.
extern "C" int ia_gemm_skinny_bf16(void* out, const void* x, const void* w, float* partial,
                                   int M, int N, int K, int splits, int out_dtype, hipStream_t stream) {
    IA_CHECK(M >= 0 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    IA_CHECK(K % 8 == 0, "gemm_skinny: K=%d must be a multiple of 8 (use the tiled product)", K);
    IA_CHECK(out_dtype == IA_F32 || out_dtype == IA_BF16, "gemm_skinny: unknown output dtype %d", out_dtype);
    IA_CHECK(splits >= 1 && splits <= 64, "gemm_skinny: splits=%d is outside 1..64", splits);
    IA_CHECK(splits == 1 || partial != nullptr, "gemm_skinny: splits=%d without a partial buffer", splits);
    IA_CHECK((((uintptr_t)x | (uintptr_t)w) & 15) == 0, "gemm_skinny: x and w must be 16-byte aligned");
    if (M == 0) return 0;
    const int out_f32 = out_dtype == IA_F32;
    const dim3 grid((N + SK_ROWS - 1) / SK_ROWS, splits);
    for (int m_base = 0; m_base < M; m_base += 64) {
        const int rows = M - m_base;
        // Rows beyond the first 64 are written by later launches: offset by m_base inside.
        if (rows <= 16)
            gemm_skinny_kernel<1><<<grid, SK_WAVES * IA_WAVE, 0, stream>>>(partial, out, out_f32, (const bf16_t*)x, (const bf16_t*)w, M, N, K, m_base);
        else if (rows <= 32)
            gemm_skinny_kernel<2><<<grid, SK_WAVES * IA_WAVE, 0, stream>>>(partial, out, out_f32, (const bf16_t*)x, (const bf16_t*)w, M, N, K, m_base);
        else
            gemm_skinny_kernel<4><<<grid, SK_WAVES * IA_WAVE, 0, stream>>>(partial, out, out_f32, (const bf16_t*)x, (const bf16_t*)w, M, N, K, m_base);
        IA_LAUNCH_CHECK("gemm_skinny");
    }
    if (splits > 1) {
        const size_t total = (size_t)M * N;
        const size_t want = (total + 255) / 256;
        gemm_split_reduce_kernel<<<(unsigned)(want < 65535 ? want : 65535), 256, 0, stream>>>(out, out_f32, partial, splits, total);
        IA_LAUNCH_CHECK("gemm_split_reduce");
    }
    return 0;
}
