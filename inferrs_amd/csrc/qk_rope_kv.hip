// Per-head RMS norm of queries and keys, rotary position encoding, and the write of the new
// keys and values into their cache pages, in one pass over the projection output.
//
// Order as in the reference: norm per head over head_dim with one shared weight vector
// (inferrs-models/src/models/qwen3.rs:128-129, attention_utils.rs:52-58), then rotation
// (qwen3.rs:132-135) with out[i] = x[i]c - x[j]s, out[j] = x[i]s + x[j]c
// (inferrs-kernels/candle-kernels/src/reduce.cu:292-312 for j = i + rot/2, :275-289 for the
// interleaved pairing), then the cache append (qwen3.rs:145-161).  Values are copied as they are.
// Norm, angles and rotation stay in 32-bit registers; one rounding happens at the store.
#include "common.h"
#include "api.h"

#define QK_MAX_HEAD_DIM 512
#define QK_WAVES 4

// One wave per (token, head).  Heads 0..nq are queries, nq..nq+nkv keys, the rest values.
template <typename T>
__global__ __launch_bounds__(QK_WAVES * IA_WAVE) void qk_rope_kv_kernel(
    T* __restrict__ q_out,              // [n, nq, d]
    T* __restrict__ k_cache,            // [pages, nkv, page_size, d] or null
    T* __restrict__ v_cache,            // [pages, nkv, d, page_size] or null
    const T* __restrict__ qkv,          // [n, (nq + 2 nkv) d]
    const float* __restrict__ q_norm_w, // [d] or null
    const float* __restrict__ k_norm_w, // [d] or null
    const float* __restrict__ cos_t,    // [n, rot/2] or null
    const float* __restrict__ sin_t,
    const int* __restrict__ slots,      // [n] page * page_size + offset, or null (no write)
    int n, int nq, int nkv, int d, int rot, int interleaved, int page_size, float eps, int add_one) {
    __shared__ float buf[QK_WAVES][QK_MAX_HEAD_DIM];
    const int lane = threadIdx.x & (IA_WAVE - 1);
    const int wave = threadIdx.x / IA_WAVE;
    const int heads = slots ? nq + 2 * nkv : nq;
    const long long unit = (long long)blockIdx.x * QK_WAVES + wave;
    const bool active = unit < (long long)n * heads;
    const int tok = active ? (int)(unit / heads) : 0;
    const int hh = active ? (int)(unit % heads) : 0;
    const int kind = hh < nq ? 0 : (hh < nq + nkv ? 1 : 2);
    const T* src = qkv + ((size_t)tok * (nq + 2 * nkv) + hh) * d;
    float* row = buf[wave];

    float ss = 0.f;
    if (active) {
        for (int j = lane; j < d; j += IA_WAVE) {
            const float v = ld(src + j);
            row[j] = v;
            ss += v * v;
        }
    }
    const float* nw = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
    if (nw != nullptr) {
        ss = wave_sum(ss);
        const float scale = 1.0f / sqrtf(ss / (float)d + eps);
        if (active)
            for (int j = lane; j < d; j += IA_WAVE) row[j] = scale * row[j] * (add_one ? 1.0f + nw[j] : nw[j]);
    }
    __syncthreads();
    if (!active) return;

    T* dst;
    if (kind == 0) {
        dst = q_out + ((size_t)tok * nq + hh) * d;
    } else {
        const int slot = slots[tok];
        const int page = slot / page_size, off = slot - page * page_size;
        if (kind == 2) {
            // values are kept transposed inside a page: [dim][slot]
            T* vt = v_cache + ((size_t)page * nkv + (hh - nq - nkv)) * d * page_size + off;
            for (int j = lane; j < d; j += IA_WAVE) st(vt + (size_t)j * page_size, row[j]);
            return;
        }
        dst = k_cache + (((size_t)page * nkv + (hh - nq)) * page_size + off) * d;
    }
    if (cos_t == nullptr) {
        for (int j = lane; j < d; j += IA_WAVE) st(dst + j, row[j]);
        return;
    }
    const int half = rot / 2;
    for (int i = lane; i < half; i += IA_WAVE) {
        const float c = cos_t[(size_t)tok * half + i], s = sin_t[(size_t)tok * half + i];
        const int ia = interleaved ? 2 * i : i;
        const int ib = interleaved ? 2 * i + 1 : i + half;
        const float a = row[ia], b = row[ib];
        st(dst + ia, a * c - b * s);
        st(dst + ib, a * s + b * c);
    }
    for (int j = rot + lane; j < d; j += IA_WAVE) st(dst + j, row[j]);
}

#define QKV_THREADS 256
#define QKV_GROUP 8

// The values of eight neighbouring tokens, for as many heads as the block's threads cover (see below).
__device__ __forceinline__ void values_in_groups(uint16_t* tile /* [head of the block][token of the group][d] */,
                                                 bf16_t* __restrict__ v_cache, const bf16_t* __restrict__ qkv,
                                                 const int* __restrict__ slots, int vb, int n, int nq, int nkv,
                                                 int d, int page_size) {
    const int tpu = d / 8;
    const int units_per_block = QKV_THREADS / tpu;
    const int u = threadIdx.x / tpu, t = threadIdx.x - u * tpu;
    const int hpb = units_per_block / QKV_GROUP;      // heads a block
    const int head_groups = (nkv + hpb - 1) / hpb;
    const int tok0 = vb / head_groups * QKV_GROUP, head0 = vb % head_groups * hpb;
    if (u < hpb * QKV_GROUP) {
        const int hl = u / QKV_GROUP, ti = u - hl * QKV_GROUP;
        if (tok0 + ti < n && head0 + hl < nkv)
            *(uint4*)(tile + (size_t)u * d + t * 8) =
                *(const uint4*)(qkv + ((size_t)(tok0 + ti) * (nq + 2 * nkv) + nq + nkv + head0 + hl) * d + t * 8);
    }
    int slot[QKV_GROUP];
    bool together = tok0 + QKV_GROUP <= n;
#pragma unroll
    for (int i = 0; i < QKV_GROUP; ++i) {
        slot[i] = tok0 + i < n ? slots[tok0 + i] : -1;
        together = together && slot[i] == slot[0] + i;
    }
    together = together && slot[0] % QKV_GROUP == 0 && page_size % QKV_GROUP == 0;
    __syncthreads();
    for (int p = threadIdx.x; p < hpb * d; p += QKV_THREADS) {
        const int hl = p / d, j = p - hl * d;
        if (head0 + hl >= nkv) continue;
        const uint16_t* col = tile + (size_t)hl * QKV_GROUP * d + j;
        bf16_t* feature = v_cache + ((size_t)(head0 + hl) * d + j) * page_size;   // + page * nkv * d * page_size
        if (together) {
            const int page = slot[0] / page_size, off = slot[0] - page * page_size;
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = (uint32_t)col[(2 * i) * d] | ((uint32_t)col[(2 * i + 1) * d] << 16);
            *(uint4*)(feature + (size_t)page * nkv * d * page_size + off) = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
#pragma unroll
            for (int i = 0; i < QKV_GROUP; ++i) {
                if (slot[i] < 0) continue;
                const int page = slot[i] / page_size, off = slot[i] - page * page_size;
                feature[(size_t)page * nkv * d * page_size + off].bits = col[i * d];
            }
        }
    }
}

// The same work with 16-byte accesses, for bfloat16 and head sizes that are a multiple of 8:
// a thread owns eight neighbouring features of one (token, head); the threads of a head meet in
// shared memory for the sum of squares and for their rotation partners.
//
// Values lie transposed inside a page ([dim][slot]): written token by token, every feature is a
// store of two bytes of its own.  With `v_from` >= 0 the blocks from that index on write the values
// instead, eight tokens at a time: a block turns the rows of eight neighbouring tokens (of as many
// heads as its threads cover) round in shared memory, and where the eight tokens' slots are
// neighbours in one page, starting at a multiple of eight, a thread stores a feature's eight
// slots as 16 bytes.  Other groups (a page's edge inside, a sequence's end, the last tokens of the
// batch) are stored slot by slot.  The other blocks then leave the values alone.
__global__ __launch_bounds__(QKV_THREADS) void qk_rope_kv_bf16_vec_kernel(
    bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    const bf16_t* __restrict__ qkv, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ slots,
    int n, int nq, int nkv, int d, int rot, int interleaved, int page_size, float eps, int add_one, int v_from) {
    __shared__ float rows[QKV_THREADS * 8];          // normalised features, unit after unit
    __shared__ float partial[QKV_THREADS];
    const int tpu = d / 8;                            // threads a (token, head) unit
    const int units_per_block = QKV_THREADS / tpu;
    const int u = threadIdx.x / tpu, t = threadIdx.x - u * tpu;
    if (v_from >= 0 && (int)blockIdx.x >= v_from) {
        values_in_groups((uint16_t*)rows, v_cache, qkv, slots, (int)blockIdx.x - v_from, n, nq, nkv, d, page_size);
        return;
    }
    const int heads = slots ? (v_from >= 0 ? nq + nkv : nq + 2 * nkv) : nq;
    const long long unit = (long long)blockIdx.x * units_per_block + u;
    const bool active = u < units_per_block && unit < (long long)n * heads;
    const int tok = active ? (int)(unit / heads) : 0;
    const int hh = active ? (int)(unit % heads) : 0;
    const int kind = hh < nq ? 0 : (hh < nq + nkv ? 1 : 2);
    // Everything that does not depend on the features is asked for before the first barrier, in
    // 16-byte pieces: norm weights, and the angles when a thread's eight features lie on one
    // side of the rotation's halves (else they are read one by one further down).
    const float* nw = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
    const int half = rot / 2;
    const bool vec_angles = interleaved ? rot % 8 == 0 : half % 8 == 0;
    const bool rotates = active && cos_t != nullptr && kind != 2 && t * 8 < rot;
    float gw[8], cs[8], sn[8];
    if (active && nw != nullptr) {
        const float4 g0 = *(const float4*)(nw + t * 8), g1 = *(const float4*)(nw + t * 8 + 4);
        gw[0] = g0.x; gw[1] = g0.y; gw[2] = g0.z; gw[3] = g0.w; gw[4] = g1.x; gw[5] = g1.y; gw[6] = g1.z; gw[7] = g1.w;
    }
    if (rotates && vec_angles) {
        if (interleaved) {
            const size_t at = (size_t)tok * half + t * 4;
            const float4 c0 = *(const float4*)(cos_t + at), s0 = *(const float4*)(sin_t + at);
            cs[0] = cs[1] = c0.x; cs[2] = cs[3] = c0.y; cs[4] = cs[5] = c0.z; cs[6] = cs[7] = c0.w;
            sn[0] = sn[1] = s0.x; sn[2] = sn[3] = s0.y; sn[4] = sn[5] = s0.z; sn[6] = sn[7] = s0.w;
        } else {
            const int e0 = t * 8;
            const size_t at = (size_t)tok * half + (e0 < half ? e0 : e0 - half);
            const float4 c0 = *(const float4*)(cos_t + at), c1 = *(const float4*)(cos_t + at + 4);
            const float4 s0 = *(const float4*)(sin_t + at), s1 = *(const float4*)(sin_t + at + 4);
            cs[0] = c0.x; cs[1] = c0.y; cs[2] = c0.z; cs[3] = c0.w; cs[4] = c1.x; cs[5] = c1.y; cs[6] = c1.z; cs[7] = c1.w;
            sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
        }
    }
    float v[8];
    float ss = 0.f;
    if (active) {
        const uint4 raw = *(const uint4*)(qkv + ((size_t)tok * (nq + 2 * nkv) + hh) * d + t * 8);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = __uint_as_float(w[j] << 16);
            v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
    }
    partial[threadIdx.x] = ss;
    __syncthreads();
    if (active && nw != nullptr) {
        float total = 0.f;
        for (int i = 0; i < tpu; ++i) total += partial[u * tpu + i];      // the same order in every thread
        const float scale = 1.0f / sqrtf(total / (float)d + eps);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = scale * v[j] * (add_one ? 1.0f + gw[j] : gw[j]);
    }
    if (active) {
#pragma unroll
        for (int j = 0; j < 8; ++j) rows[threadIdx.x * 8 + j] = v[j];
    }
    __syncthreads();
    if (!active) return;
    if (kind == 2) {
        // values are kept transposed inside a page: [dim][slot]
        const int slot = slots[tok];
        const int page = slot / page_size, off = slot - page * page_size;
        bf16_t* vt = v_cache + ((size_t)page * nkv + (hh - nq - nkv)) * d * page_size + off;
#pragma unroll
        for (int j = 0; j < 8; ++j) st(vt + (size_t)(t * 8 + j) * page_size, v[j]);
        return;
    }
    if (cos_t != nullptr) {
        const float* row = rows + (size_t)u * tpu * 8;
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int e = t * 8 + j;
            o[j] = v[j];
            if (e < rot) {
                const int i = interleaved ? e >> 1 : (e < half ? e : e - half);
                const bool first = interleaved ? (e & 1) == 0 : e < half;
                const int partner = interleaved ? e ^ 1 : (first ? e + half : e - half);
                const float c = vec_angles ? cs[j] : cos_t[(size_t)tok * half + i];
                const float s = vec_angles ? sn[j] : sin_t[(size_t)tok * half + i];
                o[j] = first ? v[j] * c - row[partner] * s : row[partner] * s + v[j] * c;
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = o[j];
    }
    bf16_t* dst;
    if (kind == 0) {
        dst = q_out + ((size_t)tok * nq + hh) * d;
    } else {
        const int slot = slots[tok];
        const int page = slot / page_size, off = slot - page * page_size;
        dst = k_cache + (((size_t)page * nkv + (hh - nq)) * page_size + off) * d;
    }
    *(uint4*)(dst + t * 8) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]),
                                        pack_bf16x2(v[6], v[7]));
}

// Steps with prompt portions, where the head size is a power of two and the whole head rotates in
// halves: the threads of a head (d / 8 of them, neighbours in one wave) walk up to QKV_HEADS heads
// of one token.  The token's angles and the norm weights are read once for all of them, the heads'
// rows are all asked for before the first is used, and the sum of squares and the rotation partners
// go from lane to lane without shared memory.  The sum runs in the order of the kernel above, so
// that both give the same bits.
#define QKV_HEADS 8
template <int TPU>
__global__ __launch_bounds__(QKV_THREADS) void qk_rope_kv_bf16_rows_kernel(
    bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    const bf16_t* __restrict__ qkv, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ slots,
    int n, int nq, int nkv, int page_size, float eps, int add_one, int v_from) {
    constexpr int D = TPU * 8, HALF = D / 2;
    __shared__ uint16_t tile[QKV_THREADS * 8];
    if ((int)blockIdx.x >= v_from) {
        values_in_groups(tile, v_cache, qkv, slots, (int)blockIdx.x - v_from, n, nq, nkv, D, page_size);
        return;
    }
    const int rg = threadIdx.x / TPU, t = threadIdx.x % TPU;
    const int chunks = (nq + nkv + QKV_HEADS - 1) / QKV_HEADS;
    const long long item = (long long)blockIdx.x * (QKV_THREADS / TPU) + rg;
    if (item >= (long long)n * chunks) return;
    const int tok = (int)(item / chunks), h0 = (int)(item % chunks) * QKV_HEADS;
    const int hn = nq + nkv - h0 < QKV_HEADS ? nq + nkv - h0 : QKV_HEADS;
    const int e0 = t * 8;
    const bool first = e0 < HALF;
    const bf16_t* src = qkv + ((size_t)tok * (nq + 2 * nkv) + h0) * D + e0;
    uint4 raw[QKV_HEADS];
#pragma unroll
    for (int i = 0; i < QKV_HEADS; ++i)
        if (i < hn) raw[i] = *(const uint4*)(src + (size_t)i * D);
    const size_t at = (size_t)tok * HALF + (first ? e0 : e0 - HALF);
    const float4 c0 = *(const float4*)(cos_t + at), c1 = *(const float4*)(cos_t + at + 4);
    const float4 s0 = *(const float4*)(sin_t + at), s1 = *(const float4*)(sin_t + at + 4);
    const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
    float gq[8], gk[8];
    if (q_norm_w != nullptr && h0 < nq) {
        const float4 g0 = *(const float4*)(q_norm_w + e0), g1 = *(const float4*)(q_norm_w + e0 + 4);
        gq[0] = g0.x; gq[1] = g0.y; gq[2] = g0.z; gq[3] = g0.w; gq[4] = g1.x; gq[5] = g1.y; gq[6] = g1.z; gq[7] = g1.w;
    }
    if (k_norm_w != nullptr && h0 + hn > nq) {
        const float4 g0 = *(const float4*)(k_norm_w + e0), g1 = *(const float4*)(k_norm_w + e0 + 4);
        gk[0] = g0.x; gk[1] = g0.y; gk[2] = g0.z; gk[3] = g0.w; gk[4] = g1.x; gk[5] = g1.y; gk[6] = g1.z; gk[7] = g1.w;
    }
    bf16_t* k_row = nullptr;
    if (h0 + hn > nq) {
        const int slot = slots[tok];
        const int page = slot / page_size, off = slot - page * page_size;
        k_row = k_cache + ((size_t)page * nkv * page_size + off) * D + e0;      // + head * page_size * D
    }
#pragma unroll
    for (int i = 0; i < QKV_HEADS; ++i) {
        if (i >= hn) break;
        const int hh = h0 + i;
        const bool is_q = hh < nq;
        const uint32_t w[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = __uint_as_float(w[j] << 16);
            v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
        if ((is_q ? q_norm_w : k_norm_w) != nullptr) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
            float total = 0.f;
#pragma unroll
            for (int j = 0; j < TPU; ++j) total += __shfl(ss, j, TPU);
            const float scale = 1.0f / sqrtf(total / (float)D + eps);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float g = is_q ? gq[j] : gk[j];
                v[j] = scale * v[j] * (add_one ? 1.0f + g : g);
            }
        }
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float partner = __shfl_xor(v[j], TPU / 2, TPU);
            o[j] = first ? v[j] * cs[j] - partner * sn[j] : partner * sn[j] + v[j] * cs[j];
        }
        bf16_t* dst = is_q ? q_out + ((size_t)tok * nq + hh) * D + e0 : k_row + (size_t)(hh - nq) * page_size * D;
        *(uint4*)dst = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]),
                                  pack_bf16x2(o[6], o[7]));
    }
}

template <int TPU>
static void launch_rows(bf16_t* q_out, bf16_t* k_cache, bf16_t* v_cache, const bf16_t* qkv, const float* q_norm_w,
                        const float* k_norm_w, const float* cos_t, const float* sin_t, const int* slots, int n,
                        int nq, int nkv, int page_size, float eps, int add_one, long long v_blocks,
                        hipStream_t stream) {
    const long long chunks = (nq + nkv + QKV_HEADS - 1) / QKV_HEADS;
    const long long qk_blocks = ((long long)n * chunks + QKV_THREADS / TPU - 1) / (QKV_THREADS / TPU);
    qk_rope_kv_bf16_rows_kernel<TPU><<<(unsigned)(qk_blocks + v_blocks), QKV_THREADS, 0, stream>>>(
        q_out, k_cache, v_cache, qkv, q_norm_w, k_norm_w, cos_t, sin_t, slots, n, nq, nkv, page_size, eps, add_one,
        (int)qk_blocks);
}

static int g_group_values = 1, g_rows = 1;
// Measurement switches: group_values 0 writes the values token by token in every step; rows 0 keeps
// steps with prompt portions on the kernel that gives a thread one head.
extern "C" void ia_qk_rope_kv_tune(int group_values, int rows) { g_group_values = group_values; g_rows = rows; }

extern "C" int ia_qk_rope_kv(void* q_out, void* k_cache, void* v_cache, const void* qkv,
                             const float* q_norm_w, const float* k_norm_w, const float* cos_t,
                             const float* sin_t, const int* slots, int n, int nq, int nkv, int d,
                             int rot, int interleaved, int page_size, float eps, int add_one,
                             int dtype, hipStream_t stream) {
    IA_CHECK(n >= 0 && nq > 0 && nkv > 0, "qk_rope_kv: bad sizes n=%d nq=%d nkv=%d", n, nq, nkv);
    IA_CHECK(d > 0 && d <= QK_MAX_HEAD_DIM, "qk_rope_kv: head_dim %d is outside 1..%d", d, QK_MAX_HEAD_DIM);
    IA_CHECK(rot >= 0 && rot <= d && rot % 2 == 0, "qk_rope_kv: rot_dim %d must be even and <= head_dim %d", rot, d);
    IA_CHECK((cos_t == nullptr) == (sin_t == nullptr), "qk_rope_kv: cos and sin tables must come together");
    IA_CHECK(cos_t == nullptr || rot > 0, "qk_rope_kv: a rotary table needs rot_dim > 0");
    IA_CHECK(slots == nullptr || (k_cache && v_cache && page_size > 0), "qk_rope_kv: slots given without a cache");
    if (n == 0) return 0;
    const long long units = (long long)n * (slots ? nq + 2 * nkv : nq);
    const unsigned grid = (unsigned)((units + QK_WAVES - 1) / QK_WAVES);
    const uintptr_t ptrs = (uintptr_t)q_out | (uintptr_t)qkv | (uintptr_t)(slots ? k_cache : nullptr) |
                           (uintptr_t)q_norm_w | (uintptr_t)k_norm_w | (uintptr_t)cos_t | (uintptr_t)sin_t;
    if (dtype == IA_BF16 && d % 8 == 0 && d / 8 <= QKV_THREADS && (ptrs & 15) == 0) {
        const int units_per_block = QKV_THREADS / (d / 8);
        // values in groups of eight tokens: where a block's threads cover eight rows, pages hold whole
        // groups, and the step has prompt portions in it (single decoded tokens have no neighbours)
        const bool grouped = g_group_values && slots != nullptr && units_per_block >= QKV_GROUP &&
                             page_size % QKV_GROUP == 0 && n >= 2 * QKV_GROUP && ((uintptr_t)v_cache & 15) == 0;
        long long qk_units = units, v_blocks = 0;
        if (grouped) {
            const int hpb = units_per_block / QKV_GROUP;
            qk_units = (long long)n * (nq + nkv);
            v_blocks = (long long)((n + QKV_GROUP - 1) / QKV_GROUP) * ((nkv + hpb - 1) / hpb);
        }
        const long long qk_blocks = (qk_units + units_per_block - 1) / units_per_block;
        IA_CHECK(qk_blocks + v_blocks < (1ll << 31), "qk_rope_kv: %d tokens are too many for one launch", n);
        const int tpu = d / 8;
        if (grouped && g_rows && cos_t != nullptr && rot == d && !interleaved && tpu >= 2 && tpu <= 64 &&
            (tpu & (tpu - 1)) == 0) {
#define ROWS_CASE(T) case T: launch_rows<T>((bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, (const bf16_t*)qkv, \
                     q_norm_w, k_norm_w, cos_t, sin_t, slots, n, nq, nkv, page_size, eps, add_one, v_blocks, stream); break;
            switch (tpu) { ROWS_CASE(2) ROWS_CASE(4) ROWS_CASE(8) ROWS_CASE(16) ROWS_CASE(32) ROWS_CASE(64) }
#undef ROWS_CASE
            IA_LAUNCH_CHECK("qk_rope_kv");
            return 0;
        }
        qk_rope_kv_bf16_vec_kernel<<<(unsigned)(qk_blocks + v_blocks), QKV_THREADS, 0, stream>>>(
            (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, (const bf16_t*)qkv, q_norm_w, k_norm_w,
            cos_t, sin_t, slots, n, nq, nkv, d, rot, interleaved, page_size, eps, add_one,
            grouped ? (int)qk_blocks : -1);
        IA_LAUNCH_CHECK("qk_rope_kv");
        return 0;
    }
    if (dtype == IA_F32)
        qk_rope_kv_kernel<float><<<grid, QK_WAVES * IA_WAVE, 0, stream>>>(
            (float*)q_out, (float*)k_cache, (float*)v_cache, (const float*)qkv, q_norm_w, k_norm_w,
            cos_t, sin_t, slots, n, nq, nkv, d, rot, interleaved, page_size, eps, add_one);
    else if (dtype == IA_BF16)
        qk_rope_kv_kernel<bf16_t><<<grid, QK_WAVES * IA_WAVE, 0, stream>>>(
            (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, (const bf16_t*)qkv, q_norm_w, k_norm_w,
            cos_t, sin_t, slots, n, nq, nkv, d, rot, interleaved, page_size, eps, add_one);
    else
        IA_CHECK(false, "qk_rope_kv: unknown dtype %d", dtype);
    IA_LAUNCH_CHECK("qk_rope_kv");
    return 0;
}
