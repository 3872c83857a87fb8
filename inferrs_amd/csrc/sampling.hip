// Token selection on the device.
//
// ia_argmax: greedy choice, the lowest index among equal maxima (the reference's CPU argmax
// keeps the first maximum, candle-core/src/cpu_backend/mod.rs:150-157; its CUDA reduction
// leaves ties unspecified, inferrs-kernels/candle-kernels/src/reduce.cu:500-520).
#include "common.h"
#include "api.h"

__global__ __launch_bounds__(1024) void argmax_kernel(int* __restrict__ out, const float* __restrict__ logits, int vocab) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (size_t)blockIdx.x * vocab;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int c = threadIdx.x; c < vocab; c += blockDim.x) {
        const float v = row[c];
        if (v > best || (v == best && c < idx)) { best = v; idx = c; }
    }
    if (idx == 0x7fffffff && threadIdx.x < vocab) idx = threadIdx.x;   // row of NaN or -inf
#pragma unroll
    for (int o = IA_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, IA_WAVE);
        const int oi = __shfl_xor(idx, o, IA_WAVE);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    const int lane = threadIdx.x & (IA_WAVE - 1), wave = threadIdx.x / IA_WAVE;
    if (lane == 0) { sv[wave] = best; si[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nw = (blockDim.x + IA_WAVE - 1) / IA_WAVE;
        for (int w = 1; w < nw; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < idx)) { best = sv[w]; idx = si[w]; }
        out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
    }
}

extern "C" int ia_argmax(int* out, const float* logits, int rows, int vocab, hipStream_t stream) {
    IA_CHECK(rows >= 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    argmax_kernel<<<rows, 1024, 0, stream>>>(out, logits, vocab);
    IA_LAUNCH_CHECK("argmax");
    return 0;
}
