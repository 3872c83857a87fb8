// Row-wise and element-wise kernels: embedding gather, RMS norm (plain and fused with the
// residual add), SiLU-gate product, rotary angle tables, row gather, residual add.
//
// Formulas follow the reference's CUDA kernels: rmsnorm keeps the sum of squares and the
// scale in 32-bit and rounds once (inferrs-kernels/candle-kernels/src/reduce.cu:189-228);
// silu(z) = z / (1 + exp(-z)) (unary.cu:59-61); rotary angles are position * inv_freq in
// 32-bit (inferrs-models/src/models/attention_utils.rs:186-216).
#include "common.h"
#include "api.h"

// A row copied by a block: 16 bytes a thread at a time where the row's size and both addresses allow it.
template <typename T>
__device__ __forceinline__ void copy_row(T* __restrict__ dst, const T* __restrict__ src, int n) {
    const size_t bytes = (size_t)n * sizeof(T);
    if ((bytes & 15) == 0 && (((uintptr_t)dst | (uintptr_t)src) & 15) == 0) {
        const int pieces = (int)(bytes / 16);
        for (int c = threadIdx.x; c < pieces; c += blockDim.x) ((uint4*)dst)[c] = ((const uint4*)src)[c];
    } else {
        for (int c = threadIdx.x; c < n; c += blockDim.x) dst[c] = src[c];
    }
}

// ---- embedding ------------------------------------------------------------------------------
template <typename T>
__global__ void embed_gather_kernel(T* __restrict__ out, const T* __restrict__ table,
                                    const int* __restrict__ ids, int hidden, int vocab) {
    const int row = blockIdx.x;
    const int id = ids[row];
    const bool ok = id >= 0 && id < vocab;
    const T* src = table + (size_t)(ok ? id : 0) * hidden;
    T* dst = out + (size_t)row * hidden;
    if (ok) { copy_row(dst, src, hidden); return; }
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) st(dst + c, 0.f);
}

extern "C" int ia_embed_gather(void* out, const void* table, const int* ids, int n, int hidden,
                               int vocab, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && hidden > 0 && vocab > 0, "embed_gather: bad sizes n=%d hidden=%d vocab=%d", n, hidden, vocab);
    if (n == 0) return 0;
    const int block = hidden >= 1024 ? 256 : 64;
    if (dtype == IA_F32)
        embed_gather_kernel<float><<<n, block, 0, stream>>>((float*)out, (const float*)table, ids, hidden, vocab);
    else if (dtype == IA_BF16)
        embed_gather_kernel<bf16_t><<<n, block, 0, stream>>>((bf16_t*)out, (const bf16_t*)table, ids, hidden, vocab);
    else
        IA_CHECK(false, "embed_gather: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("embed_gather");
    return 0;
}

// ---- row gather -----------------------------------------------------------------------------
template <typename T>
__global__ void gather_rows_kernel(T* __restrict__ out, const T* __restrict__ x,
                                   const int* __restrict__ rows, int cols) {
    copy_row(out + (size_t)blockIdx.x * cols, x + (size_t)rows[blockIdx.x] * cols, cols);
}

extern "C" int ia_gather_rows(void* out, const void* x, const int* rows, int n, int cols,
                              int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && cols > 0, "gather_rows: bad sizes n=%d cols=%d", n, cols);
    if (n == 0) return 0;
    const int block = cols >= 1024 ? 256 : 64;
    if (dtype == IA_F32)
        gather_rows_kernel<float><<<n, block, 0, stream>>>((float*)out, (const float*)x, rows, cols);
    else if (dtype == IA_BF16)
        gather_rows_kernel<bf16_t><<<n, block, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, rows, cols);
    else
        IA_CHECK(false, "gather_rows: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("gather_rows");
    return 0;
}

// ---- RMS norm -------------------------------------------------------------------------------
// One block per row.  The block size depends on the row length only, so a row's result does
// not depend on how many rows are normalised together.
template <typename T, bool ADD>
__global__ void rmsnorm_kernel(T* __restrict__ out, T* __restrict__ x, const T* __restrict__ delta,
                               const float* __restrict__ w, float eps, int cols, int add_one) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * cols;
    float ss = 0.f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        float v = ld(x + base + c);
        if (ADD) {
            v = round_to(x, v + ld(delta + base + c));
            st(x + base + c, v);
        }
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)cols + eps);
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const float v = ld(x + base + c);
        const float g = add_one ? 1.0f + w[c] : w[c];
        st(out + base + c, scale * v * g);
    }
}

// bfloat16 rows whose length is a multiple of 8 and at most 8 * 1024 * NORM_VECS: every thread
// keeps its pieces of the row in registers, so the row is read once.  The block size depends
// on the row length only.
#define NORM_VECS 2
template <bool ADD>
__global__ __launch_bounds__(1024) void rmsnorm_bf16_vec_kernel(bf16_t* __restrict__ out, bf16_t* __restrict__ x,
                                                                const bf16_t* __restrict__ delta,
                                                                const float* __restrict__ w, float eps, int cols,
                                                                int add_one) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * cols;
    const int nvec = cols / 8;
    float v[NORM_VECS][8];
    float4 w0[NORM_VECS], w1[NORM_VECS];        // asked for now, used after the sum: one wait instead of two
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NORM_VECS; ++i) {
        const int vi = threadIdx.x + i * blockDim.x;
        if (vi < nvec) {
            w0[i] = *(const float4*)(w + (size_t)vi * 8);
            w1[i] = *(const float4*)(w + (size_t)vi * 8 + 4);
        }
    }
#pragma unroll
    for (int i = 0; i < NORM_VECS; ++i) {
        const int vi = threadIdx.x + i * blockDim.x;
        if (vi < nvec) {
            const uint4 raw = *(const uint4*)(x + base + (size_t)vi * 8);
            const uint32_t wd[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[i][2 * j] = __uint_as_float(wd[j] << 16);
                v[i][2 * j + 1] = __uint_as_float(wd[j] & 0xffff0000u);
            }
            if (ADD) {
                const uint4 rd = *(const uint4*)(delta + base + (size_t)vi * 8);
                const uint32_t dd[4] = {rd.x, rd.y, rd.z, rd.w};
                uint32_t packed[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint16_t lo = f32_to_bf16_bits(v[i][2 * j] + __uint_as_float(dd[j] << 16));
                    const uint16_t hi = f32_to_bf16_bits(v[i][2 * j + 1] + __uint_as_float(dd[j] & 0xffff0000u));
                    v[i][2 * j] = bf16_bits_to_f32(lo);
                    v[i][2 * j + 1] = bf16_bits_to_f32(hi);
                    packed[j] = (uint32_t)lo | ((uint32_t)hi << 16);
                }
                *(uint4*)(x + base + (size_t)vi * 8) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += v[i][j] * v[i][j];
        }
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)cols + eps);
#pragma unroll
    for (int i = 0; i < NORM_VECS; ++i) {
        const int vi = threadIdx.x + i * blockDim.x;
        if (vi < nvec) {
            const float g[8] = {w0[i].x, w0[i].y, w0[i].z, w0[i].w, w1[i].x, w1[i].y, w1[i].z, w1[i].w};
            uint32_t packed[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float a = scale * v[i][2 * j] * (add_one ? 1.0f + g[2 * j] : g[2 * j]);
                const float b = scale * v[i][2 * j + 1] * (add_one ? 1.0f + g[2 * j + 1] : g[2 * j + 1]);
                packed[j] = (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
            }
            *(uint4*)(out + base + (size_t)vi * 8) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        }
    }
}

static int norm_block(int cols) { return cols >= 2048 ? 512 : (cols >= 512 ? 256 : 64); }

// Threads for the register-resident kernel, or 0 when the row does not fit it.
static int norm_vec_block(int cols, const void* a, const void* b, const void* c, const void* w) {
    if (cols % 8 || cols > 8 * 1024 * NORM_VECS) return 0;
    if ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)w) & 15) != 0) return 0;
    const int nvec = cols / 8;
    int block = 64;
    while (block * NORM_VECS < nvec) block *= 2;       // 64 .. 1024
    return block;
}

extern "C" int ia_rmsnorm(void* out, const void* x, const float* w, float eps, int rows, int cols,
                          int add_one, int dtype, hipStream_t stream) {
    IA_CHECK(rows >= 0 && cols > 0, "rmsnorm: bad sizes rows=%d cols=%d", rows, cols);
    if (rows == 0) return 0;
    const int block = norm_block(cols);
    const int vblock = dtype == IA_BF16 ? norm_vec_block(cols, out, x, nullptr, w) : 0;
    if (dtype == IA_F32)
        rmsnorm_kernel<float, false><<<rows, block, 0, stream>>>((float*)out, (float*)x, nullptr, w, eps, cols, add_one);
    else if (dtype == IA_BF16 && vblock)
        rmsnorm_bf16_vec_kernel<false><<<rows, vblock, 0, stream>>>((bf16_t*)out, (bf16_t*)x, nullptr, w, eps, cols, add_one);
    else if (dtype == IA_BF16)
        rmsnorm_kernel<bf16_t, false><<<rows, block, 0, stream>>>((bf16_t*)out, (bf16_t*)x, nullptr, w, eps, cols, add_one);
    else
        IA_CHECK(false, "rmsnorm: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("rmsnorm");
    return 0;
}

// x += delta (sum in 32-bit, stored in the model's precision); out = rmsnorm(x).
extern "C" int ia_add_rmsnorm(void* out, void* x, const void* delta, const float* w, float eps,
                              int rows, int cols, int add_one, int dtype, hipStream_t stream) {
    IA_CHECK(rows >= 0 && cols > 0, "add_rmsnorm: bad sizes rows=%d cols=%d", rows, cols);
    if (rows == 0) return 0;
    const int block = norm_block(cols);
    const int vblock = dtype == IA_BF16 ? norm_vec_block(cols, out, x, delta, w) : 0;
    if (dtype == IA_F32)
        rmsnorm_kernel<float, true><<<rows, block, 0, stream>>>((float*)out, (float*)x, (const float*)delta, w, eps, cols, add_one);
    else if (dtype == IA_BF16 && vblock)
        rmsnorm_bf16_vec_kernel<true><<<rows, vblock, 0, stream>>>((bf16_t*)out, (bf16_t*)x, (const bf16_t*)delta, w, eps, cols, add_one);
    else if (dtype == IA_BF16)
        rmsnorm_kernel<bf16_t, true><<<rows, block, 0, stream>>>((bf16_t*)out, (bf16_t*)x, (const bf16_t*)delta, w, eps, cols, add_one);
    else
        IA_CHECK(false, "add_rmsnorm: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("add_rmsnorm");
    return 0;
}

// ---- residual add ---------------------------------------------------------------------------
template <typename T>
__global__ void add_kernel(T* __restrict__ x, const T* __restrict__ delta, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        st(x + i, ld(x + i) + ld(delta + i));
}

extern "C" int ia_add_inplace(void* x, const void* delta, long long n, int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0, "add_inplace: bad size %lld", n);
    if (n == 0) return 0;
    const int block = 256;
    const int grid = (int)((n + block - 1) / block < 65535 ? (n + block - 1) / block : 65535);
    if (dtype == IA_F32)
        add_kernel<float><<<grid, block, 0, stream>>>((float*)x, (const float*)delta, (size_t)n);
    else if (dtype == IA_BF16)
        add_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)x, (const bf16_t*)delta, (size_t)n);
    else
        IA_CHECK(false, "add_inplace: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("add_inplace");
    return 0;
}

// ---- x[row][c] += bias[c] -------------------------------------------------------------------
// For products whose kernel has no place for a bias; the sum is formed in 32-bit and rounded once.
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const T* __restrict__ bias, int cols, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        st(x + i, ld(x + i) + ld(bias + (i % cols)));
}

extern "C" int ia_add_bias(void* x, const void* bias, int rows, int cols, int dtype, hipStream_t stream) {
    IA_CHECK(rows >= 0 && cols > 0, "add_bias: bad sizes rows=%d cols=%d", rows, cols);
    if (rows == 0) return 0;
    const size_t total = (size_t)rows * cols;
    const size_t want = (total + 255) / 256;
    const int grid = (int)(want < 65535 ? want : 65535);
    if (dtype == IA_F32)
        add_bias_kernel<float><<<grid, 256, 0, stream>>>((float*)x, (const float*)bias, cols, total);
    else if (dtype == IA_BF16)
        add_bias_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)x, (const bf16_t*)bias, cols, total);
    else
        IA_CHECK(false, "add_bias: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("add_bias");
    return 0;
}

// ---- act(gate) * up -------------------------------------------------------------------------
// `gu` holds rows of [gate(0..inter) | up(0..inter)]; the product is formed in 32-bit.
template <typename T>
__global__ void gate_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter, size_t total, int act) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / inter;
        const int c = (int)(i - row * inter);
        const float g = ld(gu + row * 2 * inter + c);
        const float u = ld(gu + row * 2 * inter + inter + c);
        st(out + i, gate_act(g, act) * u);
    }
}

// bfloat16 rows whose half length is a multiple of 8: eight products a thread, 16-byte accesses.
__global__ void gate_mul_bf16_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ gu, int inter, size_t total_vecs,
                                         int act) {
    const int vecs_per_row = inter / 8;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_vecs; i += (size_t)gridDim.x * blockDim.x) {
        const size_t row = i / vecs_per_row;
        const int c = (int)(i - row * vecs_per_row) * 8;
        const uint4 gr = *(const uint4*)(gu + row * 2 * inter + c);
        const uint4 ur = *(const uint4*)(gu + row * 2 * inter + inter + c);
        const uint32_t gw[4] = {gr.x, gr.y, gr.z, gr.w}, uw[4] = {ur.x, ur.y, ur.z, ur.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
            const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
            o[j] = pack_bf16x2(gate_act(g0, act) * u0, gate_act(g1, act) * u1);
        }
        *(uint4*)(out + row * inter + c) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

extern "C" int ia_gate_mul(void* out, const void* gu, int rows, int inter, int act, int dtype, hipStream_t stream) {
    IA_CHECK(rows >= 0 && inter > 0, "gate_mul: bad sizes rows=%d inter=%d", rows, inter);
    IA_CHECK(act >= IA_ACT_SILU && act <= IA_ACT_LAST, "gate_mul: unknown activation %d", act);
    if (rows == 0) return 0;
    const size_t total = (size_t)rows * inter;
    const int block = 256;
    if (dtype == IA_BF16 && inter % 8 == 0 && ((((uintptr_t)out) | ((uintptr_t)gu)) & 15) == 0) {
        const size_t vecs = total / 8;
        const size_t want = (vecs + block - 1) / block;
        gate_mul_bf16_vec_kernel<<<(unsigned)(want < 65535 * 8 ? want : 65535 * 8), block, 0, stream>>>(
            (bf16_t*)out, (const bf16_t*)gu, inter, vecs, act);
        IA_LAUNCH_CHECK("gate_mul");
        return 0;
    }
    const size_t want = (total + block - 1) / block;
    const int grid = (int)(want < 65535 ? want : 65535);
    if (dtype == IA_F32)
        gate_mul_kernel<float><<<grid, block, 0, stream>>>((float*)out, (const float*)gu, inter, total, act);
    else if (dtype == IA_BF16)
        gate_mul_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, inter, total, act);
    else
        IA_CHECK(false, "gate_mul: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("gate_mul");
    return 0;
}

// ---- random fill ---------------------------------------------------------------------------------
// Element i of a tensor is a function of (seed, i) alone: two outputs of the splitmix64 sequence
// started at seed + 2 i steps give two uniforms, Box and Muller turn them into a standard normal
// value in 64-bit arithmetic, and mean + std * z is rounded to 32-bit and then to the storage
// type.  The host fill (inferrs_amd/weights/random_init.py) is the same formula in NumPy.
__device__ __forceinline__ uint64_t splitmix_out(uint64_t state) {
    uint64_t z = state;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

template <typename T>
__global__ void fill_normal_kernel(T* __restrict__ out, size_t n, uint64_t seed, double mean, double std) {
    const uint64_t golden = 0x9e3779b97f4a7c15ull;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const uint64_t h1 = splitmix_out(seed + (2 * (uint64_t)i + 1) * golden);
        const uint64_t h2 = splitmix_out(seed + (2 * (uint64_t)i + 2) * golden);
        const double u1 = (double)((h1 >> 11) + 1) * (1.0 / 9007199254740992.0);      // (0, 1]
        const double u2 = (double)(h2 >> 11) * (1.0 / 9007199254740992.0);            // [0, 1)
        const double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2);
        st(out + i, (float)(mean + std * z));
    }
}

extern "C" int ia_fill_normal(void* out, long long n, unsigned long long seed, double mean, double std,
                              int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0, "fill_normal: bad size %lld", n);
    if (n == 0) return 0;
    const size_t want = ((size_t)n + 255) / 256;
    const unsigned grid = (unsigned)(want < 65535 * 16 ? want : 65535 * 16);
    if (dtype == IA_F32)
        fill_normal_kernel<float><<<grid, 256, 0, stream>>>((float*)out, (size_t)n, seed, mean, std);
    else if (dtype == IA_BF16)
        fill_normal_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (size_t)n, seed, mean, std);
    else
        IA_CHECK(false, "fill_normal: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("fill_normal");
    return 0;
}

// ---- widening copy ---------------------------------------------------------------------------
__global__ void widen_kernel(float* __restrict__ out, const bf16_t* __restrict__ x, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        out[i] = bf16_bits_to_f32(x[i].bits);
}

extern "C" int ia_widen_bf16(float* out, const void* x, long long n, hipStream_t stream) {
    IA_CHECK(n >= 0, "widen: bad size %lld", n);
    if (n == 0) return 0;
    const size_t want = ((size_t)n + 255) / 256;
    widen_kernel<<<(unsigned)(want < 65535 * 4 ? want : 65535 * 4), 256, 0, stream>>>(out, (const bf16_t*)x, (size_t)n);
    IA_LAUNCH_CHECK("widen");
    return 0;
}

// ---- rotary angle table for the tokens of one step ----------------------------------------------
__global__ void rope_table_kernel(float* __restrict__ cos_out, float* __restrict__ sin_out,
                                  const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  int half, int total) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = i / half, f = i - t * half;
    const float ang = (float)positions[t] * inv_freq[f];
    cos_out[i] = cosf(ang);
    sin_out[i] = sinf(ang);
}

extern "C" int ia_rope_table(float* cos_out, float* sin_out, const int* positions,
                             const float* inv_freq, int n, int half, hipStream_t stream) {
    IA_CHECK(n >= 0 && half > 0, "rope_table: bad sizes n=%d half=%d", n, half);
    if (n == 0) return 0;
    const int total = n * half;
    rope_table_kernel<<<(total + 255) / 256, 256, 0, stream>>>(cos_out, sin_out, positions, inv_freq, half, total);
    IA_LAUNCH_CHECK("rope_table");
    return 0;
}

// ---- a pure streaming read: the measured roof of this GPU's memory for the measurement script ----------------
// A block owns a contiguous range; its threads read 16-byte pieces a block's width apart, four under way at a time, and
// fold them into one word (kept by a condition that the data never meets, so that nothing of the read can be dropped).
// Nothing of the engine calls it.  (Measured over 8 GB: 6.3 to 6.5 TB/s with 16 k to 64 k blocks; pieces a whole grid
// apart: 5.5 to 6.3.)
__global__ __launch_bounds__(512) void stream_read_kernel(unsigned* __restrict__ out, const uint4* __restrict__ x, size_t n16) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t begin = per * blockIdx.x;
    const size_t end = begin + per < n16 ? begin + per : n16;
    unsigned acc = 0;
    size_t i = begin + threadIdx.x;
    for (; i + 3 * (size_t)blockDim.x < end; i += 4 * (size_t)blockDim.x) {
        const uint4 a = x[i], b = x[i + blockDim.x], c = x[i + 2 * (size_t)blockDim.x], d = x[i + 3 * (size_t)blockDim.x];
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < end; i += blockDim.x) {
        const uint4 a = x[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u) out[blockIdx.x] = acc;
}

// out: `blocks` words (written only where a block's fold happens to equal a constant); x: `bytes` bytes, 16-byte aligned,
// a multiple of 16.
extern "C" int ia_stream_read(unsigned* out, const void* x, long long bytes, int blocks, hipStream_t stream) {
    IA_CHECK(bytes >= 0 && bytes % 16 == 0 && blocks > 0 && blocks <= 1048576, "stream_read: bad sizes bytes=%lld blocks=%d", bytes, blocks);
    IA_CHECK((((uintptr_t)x) & 15) == 0, "stream_read: x must be 16-byte aligned");
    stream_read_kernel<<<blocks, 512, 0, stream>>>(out, (const uint4*)x, (size_t)bytes / 16);
    IA_LAUNCH_CHECK("stream_read");
    return 0;
}
