// Token selection on the device.
//
// ia_argmax: greedy choice, the lowest index among equal maxima (the reference's CPU argmax
// keeps the first maximum, candle-core/src/cpu_backend/mod.rs:150-157; its CUDA reduction
// leaves ties unspecified, inferrs-kernels/candle-kernels/src/reduce.cu:500-520).
//
// ia_penalize: logit bias, repetition penalty (z >= 0 ? z / p : z * p, once per distinct token
// of the window), frequency and presence penalties (z -= f * count + p), in the reference's
// order (inferrs/src/sampler.rs:186-229), in place on 32-bit logits.
//
// ia_sample: the rest of the reference's sampler (sampler.rs:232-335) for a row of logits:
// divide by the temperature, softmax, order by probability (descending, equal values by
// index), keep the first top_k, cut where the running sum reaches top_p, drop what is below
// min_p times the largest probability, renormalise, and walk the kept list until the running
// sum exceeds the row's random number u.  Every one of these filters keeps a prefix of the
// ordered list, so no sort is needed: a prefix is named by a threshold key K and a count m of
// the tokens equal to K (taken by ascending index), and the threshold for "the shortest
// prefix whose weight reaches a target" is found by bisection over the 32 bits of the key,
// one block-wide sum per bit.  Sums are tree sums in a fixed order; they differ from the
// reference's sequential sums by rounding only.  Rows with a top_k of up to 1,024 take a
// shorter way (sample_top_k): their first top_k tokens are picked out and sorted, and the
// reference's steps run on that list as it runs them.  Rows without a top_k try that way with
// the first 1,024 tokens of their list and take the long one when the list does not end there.
// Probabilities, keys and each stretch's candidates for that list are the work of many blocks
// a row (two kernels); one block a row then makes the choice.
#include <mutex>

#include "common.h"
#include "api.h"

// ---- greedy ---------------------------------------------------------------------------------
// every thread's best (value, index; 0x7fffffff: none) -> the block's, the lowest index among equal maxima, in *out
__device__ __forceinline__ void argmax_block(float best, int idx, float* sv, int* si, int* out) {
#pragma unroll
    for (int o = IA_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, IA_WAVE);
        const int oi = __shfl_xor(idx, o, IA_WAVE);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    const int lane = threadIdx.x & (IA_WAVE - 1), wave = threadIdx.x / IA_WAVE;
    __syncthreads();
    if (lane == 0) { sv[wave] = best; si[wave] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nw = (blockDim.x + IA_WAVE - 1) / IA_WAVE;
        for (int w = 1; w < nw; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < idx)) { best = sv[w]; idx = si[w]; }
        *out = idx == 0x7fffffff ? 0 : idx;       // a row of NaN or -inf
    }
}

__device__ __forceinline__ void argmax_row(const float* __restrict__ row, int vocab, float* sv, int* si, int* out) {
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int c = threadIdx.x; c < vocab; c += blockDim.x) {
        const float v = row[c];
        if (v > best || (v == best && c < idx)) { best = v; idx = c; }
    }
    argmax_block(best, idx, sv, si, out);
}

__global__ __launch_bounds__(1024) void argmax_kernel(int* __restrict__ out, const float* __restrict__ logits, int vocab) {
    __shared__ float sv[16];
    __shared__ int si[16];
    argmax_row(logits + (size_t)blockIdx.x * vocab, vocab, sv, si, out + blockIdx.x);
}

// Long rows in two steps: blocks of a row take a stretch each, then one block a row picks among
// their candidates (lowest index among equal maxima in both steps).
#define ARGMAX_STRETCH 8192
__global__ __launch_bounds__(256) void argmax_stretch_kernel(float* __restrict__ cand_v, int* __restrict__ cand_i,
                                                             const float* __restrict__ logits, int vocab) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const int row = blockIdx.y, stretch = blockIdx.x;
    const int lo = stretch * ARGMAX_STRETCH;
    const int len = vocab - lo < ARGMAX_STRETCH ? vocab - lo : ARGMAX_STRETCH;
    int idx;
    if ((vocab & 3) == 0 && ((uintptr_t)logits & 15) == 0) {
        // four neighbours a load and all of a thread's loads under way together (one after the other, each waiting for
        // its own, a stretch took 16 us)
        constexpr int PER = ARGMAX_STRETCH / 4 / 256;
        const float4* src = (const float4*)(logits + (size_t)row * vocab + lo);
        float4 v[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int c = (j * 256 + (int)threadIdx.x) * 4;
            v[j] = c < len ? src[c / 4] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        }
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int c = (j * 256 + (int)threadIdx.x) * 4;
            const float e[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (c + i < len && (e[i] > best || (e[i] == best && c + i < at))) { best = e[i]; at = c + i; }
        }
        argmax_block(best, at, sv, si, &idx);
    } else {
        argmax_row(logits + (size_t)row * vocab + lo, len, sv, si, &idx);
    }
    if (threadIdx.x == 0) {
        cand_i[(size_t)row * gridDim.x + stretch] = lo + idx;
        cand_v[(size_t)row * gridDim.x + stretch] = logits[(size_t)row * vocab + lo + idx];
    }
}

__global__ __launch_bounds__(IA_WAVE) void argmax_pick_kernel(int* __restrict__ out, const float* __restrict__ cand_v,
                                                              const int* __restrict__ cand_i, int stretches) {
    const int row = blockIdx.x;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int c = threadIdx.x; c < stretches; c += IA_WAVE) {
        float v = cand_v[(size_t)row * stretches + c];
        v = v != v ? -INFINITY : v;                      // a stretch of NaN never wins over a number
        const int i = cand_i[(size_t)row * stretches + c];
        if (v > best || (v == best && i < idx) || idx == 0x7fffffff) { best = v; idx = i; }
    }
#pragma unroll
    for (int o = IA_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, IA_WAVE);
        const int oi = __shfl_xor(idx, o, IA_WAVE);
        if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) { best = ov; idx = oi; }
    }
    if (threadIdx.x == 0) out[row] = idx == 0x7fffffff ? 0 : idx;
}

extern "C" long long ia_argmax_workspace(int rows, int vocab) {
    return vocab > 2 * ARGMAX_STRETCH ? 2LL * rows * ((vocab + ARGMAX_STRETCH - 1) / ARGMAX_STRETCH) : 0;
}

// `workspace`: ia_argmax_workspace(rows, vocab) words, or null for the one-block-a-row kernel.
extern "C" int ia_argmax(int* out, const float* logits, void* workspace, int rows, int vocab, hipStream_t stream) {
    IA_CHECK(rows >= 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    if (workspace != nullptr && vocab > 2 * ARGMAX_STRETCH) {
        const int stretches = (vocab + ARGMAX_STRETCH - 1) / ARGMAX_STRETCH;
        IA_CHECK(rows <= 65535, "argmax: %d rows exceed the grid", rows);
        float* cand_v = (float*)workspace;
        int* cand_i = (int*)workspace + (size_t)rows * stretches;
        argmax_stretch_kernel<<<dim3(stretches, rows), 256, 0, stream>>>(cand_v, cand_i, logits, vocab);
        IA_LAUNCH_CHECK("argmax");
        argmax_pick_kernel<<<rows, IA_WAVE, 0, stream>>>(out, cand_v, cand_i, stretches);
        IA_LAUNCH_CHECK("argmax");
        return 0;
    }
    argmax_kernel<<<rows, 1024, 0, stream>>>(out, logits, vocab);
    IA_LAUNCH_CHECK("argmax");
    return 0;
}

// ---- greedy, for callers that cannot allocate -----------------------------------------------
// The two-step arg max needs a place for the stretches' candidates.  ia_argmax takes it from the caller; this
// entry point keeps one of a fixed size in the library's own device memory instead, so that nothing is
// allocated on the way (declared in api.h with the reasons).  Each GPU holds its own copy of the array at its
// own address: the address is asked for once per device, with that device current, and only that pointer
// (never the array's name, which on the host is a stand-in and no device address) goes to the kernels.
#define ARGMAX_STATIC_WORDS 16384                  // 64 KiB a GPU, held until the process ends
#define ARGMAX_STATIC_DEVICES 64
static __device__ __align__(256) int argmax_scratch[ARGMAX_STATIC_WORDS];
static void* g_argmax_scratch_ptr[ARGMAX_STATIC_DEVICES];    // per device; written once, under the lock
static std::mutex g_argmax_scratch_lock;

extern "C" long long ia_argmax_static_capacity(void) { return ARGMAX_STATIC_WORDS; }

extern "C" int ia_argmax_static(int* out, const float* logits, int rows, int vocab, hipStream_t stream) {
    IA_CHECK(rows >= 0 && vocab > 0, "argmax_static: bad sizes rows=%d vocab=%d", rows, vocab);
    IA_CHECK(out != nullptr && logits != nullptr, "argmax_static: null operand");
    if (rows == 0) return 0;
    const long long words = ia_argmax_workspace(rows, vocab);
    IA_CHECK(words <= ARGMAX_STATIC_WORDS, "argmax_static: %d rows of %d logits need %lld words of scratch, the "
             "library's array holds %d (use ia_argmax with a workspace of your own)", rows, vocab, words, ARGMAX_STATIC_WORDS);
    if (words == 0) {                              // short rows: one block a row, no scratch at all
        argmax_kernel<<<rows, 1024, 0, stream>>>(out, logits, vocab);
        IA_LAUNCH_CHECK("argmax_static");
        return 0;
    }
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    IA_CHECK(e == hipSuccess && device >= 0 && device < ARGMAX_STATIC_DEVICES,
             "argmax_static: cannot tell the current device (%s, device %d)", hipGetErrorString(e), device);
    void* scratch = nullptr;
    {
        std::lock_guard<std::mutex> hold(g_argmax_scratch_lock);
        if (g_argmax_scratch_ptr[device] == nullptr) {
            void* ptr = nullptr;
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(argmax_scratch));
            IA_CHECK(e == hipSuccess && ptr != nullptr, "argmax_static: no address for the scratch array on device %d: %s",
                     device, hipGetErrorString(e));
            g_argmax_scratch_ptr[device] = ptr;
        }
        scratch = g_argmax_scratch_ptr[device];
    }
    IA_CHECK(rows <= 65535, "argmax_static: %d rows exceed the grid", rows);
    const int stretches = (vocab + ARGMAX_STRETCH - 1) / ARGMAX_STRETCH;
    // (every candidate that the second kernel reads is written by the first in this call: nothing has to start at zero)
    float* cand_v = (float*)scratch;
    int* cand_i = (int*)scratch + (size_t)rows * stretches;
    argmax_stretch_kernel<<<dim3(stretches, rows), 256, 0, stream>>>(cand_v, cand_i, logits, vocab);
    IA_LAUNCH_CHECK("argmax_static");
    argmax_pick_kernel<<<rows, IA_WAVE, 0, stream>>>(out, cand_v, cand_i, stretches);
    IA_LAUNCH_CHECK("argmax_static");
    return 0;
}

// ---- penalties ------------------------------------------------------------------------------
// window [rows, w]: the last tokens of prompt and output, -1 where a row has fewer.
// bias_ids / bias_vals [rows, nb]: -1 ends a row's list.
__global__ void penalize_kernel(float* __restrict__ logits, int vocab, const int* __restrict__ window, int w,
                                const float* __restrict__ rep, const float* __restrict__ freq,
                                const float* __restrict__ pres, const int* __restrict__ bias_ids,
                                const float* __restrict__ bias_vals, int nb) {
    const int rowi = blockIdx.x;
    float* row = logits + (size_t)rowi * vocab;
    for (int j = threadIdx.x; j < nb; j += blockDim.x) {
        const int id = bias_ids[(size_t)rowi * nb + j];
        if (id >= 0 && id < vocab) atomicAdd(row + id, bias_vals[(size_t)rowi * nb + j]);
    }
    __syncthreads();
    const int* win = window + (size_t)rowi * w;
    const float rp = rep[rowi], fp = freq[rowi], pp = pres[rowi];
    // one thread per distinct token: the one holding its first occurrence
    for (int j = threadIdx.x; j < w; j += blockDim.x) {
        const int id = win[j];
        if (id < 0 || id >= vocab) continue;
        bool first = true;
        int count = 0;
        for (int i = 0; i < w; ++i) {
            if (win[i] == id) {
                if (i < j) { first = false; break; }
                ++count;
            }
        }
        if (!first) continue;
        float v = row[id];
        if (rp != 1.0f && rp != 0.0f) v = v >= 0.f ? v / rp : v * rp;
        if (fp != 0.0f || pp != 0.0f) {
            v -= fp * (float)count;
            v -= pp;
        }
        row[id] = v;
    }
}

extern "C" int ia_penalize(float* logits, int rows, int vocab, const int* window, int w, const float* rep,
                           const float* freq, const float* pres, const int* bias_ids, const float* bias_vals,
                           int nb, hipStream_t stream) {
    IA_CHECK(rows >= 0 && vocab > 0 && w >= 0 && nb >= 0, "penalize: bad sizes rows=%d vocab=%d window=%d bias=%d", rows, vocab, w, nb);
    IA_CHECK(w == 0 || window != nullptr, "penalize: a window of %d tokens without its array", w);
    IA_CHECK(nb == 0 || (bias_ids != nullptr && bias_vals != nullptr), "penalize: %d bias entries without their arrays", nb);
    if (rows == 0 || (w == 0 && nb == 0)) return 0;
    penalize_kernel<<<rows, 256, 0, stream>>>(logits, vocab, window, w, rep, freq, pres, bias_ids, bias_vals, nb);
    IA_LAUNCH_CHECK("penalize");
    return 0;
}

// A row's window after it has drawn `tokens[row]`: the last `caps[row]` tokens of its prompt and output
// (entries from caps[row] on stay -1; caps[row] = 0: the row has no window).  For runs of decode steps that
// are queued without the host in between.
__global__ void window_push_kernel(int* __restrict__ window, int w, const int* __restrict__ caps,
                                   const int* __restrict__ tokens, int rows) {
    const int row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    int* win = window + (size_t)row * w;
    const int cap = caps[row] < w ? caps[row] : w;
    if (cap <= 0) return;
    int held = 0;
    while (held < cap && win[held] >= 0) ++held;
    if (held < cap) {
        win[held] = tokens[row];
        return;
    }
    for (int i = 0; i + 1 < cap; ++i) win[i] = win[i + 1];
    win[cap - 1] = tokens[row];
}

// The same for windows of up to 64 entries (the reference's default, `repeat_last_n`), a wave a row and a lane an
// entry: one thread that moves 64 entries one after the other took 17 us.
__global__ __launch_bounds__(IA_WAVE) void window_push_wave_kernel(int* __restrict__ window, int w, const int* __restrict__ caps,
                                                                   const int* __restrict__ tokens) {
    const int row = blockIdx.x, lane = threadIdx.x;
    int* win = window + (size_t)row * w;
    const int cap = caps[row] < w ? caps[row] : w;
    if (cap <= 0) return;
    const int mine = lane < cap ? win[lane] : -1;
    const unsigned long long empty = __ballot(lane < cap && mine < 0);
    const int held = empty ? __ffsll((long long)empty) - 1 : cap;
    const int next = __shfl_down(mine, 1, IA_WAVE);
    if (held < cap) {
        if (lane == held) win[lane] = tokens[row];
    } else if (lane < cap) {
        win[lane] = lane + 1 < cap ? next : tokens[row];
    }
}

extern "C" int ia_window_push(int* window, int rows, int w, const int* caps, const int* tokens, hipStream_t stream) {
    IA_CHECK(rows >= 0 && w > 0, "window_push: bad sizes rows=%d w=%d", rows, w);
    if (rows == 0) return 0;
    if (w <= IA_WAVE) window_push_wave_kernel<<<rows, IA_WAVE, 0, stream>>>(window, w, caps, tokens);
    else window_push_kernel<<<(rows + 63) / 64, 64, 0, stream>>>(window, w, caps, tokens, rows);
    IA_LAUNCH_CHECK("window_push");
    return 0;
}

// ---- sampling -------------------------------------------------------------------------------
#define SAMPLE_THREADS 1024

// Keys order like the values they come from; NaN sorts below everything.
__device__ __forceinline__ uint32_t order_key(float z) {
    if (z != z) return 0u;
    const uint32_t u = __float_as_uint(z);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct Sums { float w; float n; };

__device__ __forceinline__ Sums block_sums(float w, float n, float* scratch) {
    Sums s;
    s.w = block_sum(w, scratch);
    s.n = block_sum(n, scratch + 16);
    return s;
}

// Weight (probability, or 1 when `by_count`) and number of the tokens with key >= t.
__device__ __forceinline__ Sums at_least(const uint32_t* __restrict__ keys, const float* __restrict__ probs,
                                         int vocab, uint32_t t, bool by_count, float* scratch) {
    float w = 0.f, n = 0.f;
    for (int c = threadIdx.x; c < vocab; c += blockDim.x)
        if (keys[c] >= t) { w += by_count ? 1.0f : probs[c]; n += 1.0f; }
    return block_sums(w, n, scratch);
}

struct Prefix { uint32_t key; int above; int ties; int take; float w_above; float p_key; };

// The shortest prefix of the ordered list whose weight reaches `target` (strictly exceeds it
// when `strict`): every token with a key above `key` and the first `take` of the `ties` tokens
// equal to it.  When even the whole list does not reach the target, the whole list.
__device__ Prefix shortest_prefix(const uint32_t* __restrict__ keys, const float* __restrict__ probs, int vocab,
                                  float target, bool by_count, bool strict, float* scratch) {
    uint32_t k = 0u;
    for (int bit = 31; bit >= 0; --bit) {
        const uint32_t t = k | (1u << bit);
        const float w = at_least(keys, probs, vocab, t, by_count, scratch).w;
        if (strict ? w > target : w >= target) k = t;
    }
    // k is the largest key whose "at least" weight reaches the target (0 if none does).
    float wa = 0.f, na = 0.f, ne = 0.f, pk = 0.f;
    for (int c = threadIdx.x; c < vocab; c += blockDim.x) {
        const uint32_t key = keys[c];
        if (key > k) { wa += by_count ? 1.0f : probs[c]; na += 1.0f; }
        else if (key == k) { ne += 1.0f; pk = by_count ? 1.0f : probs[c]; }
    }
    Prefix r;
    r.key = k;
    r.w_above = block_sum(wa, scratch);
    r.above = (int)block_sum(na, scratch + 16);
    r.ties = (int)block_sum(ne, scratch);
    // every token with this key has the same probability: take it from any thread that saw one
    __shared__ float s_pk;
    if (threadIdx.x == 0) s_pk = 0.f;
    __syncthreads();
    if (ne > 0.f) s_pk = pk;
    __syncthreads();
    r.p_key = s_pk;
    int take = r.ties;
    if (r.ties > 0 && r.p_key > 0.f) {
        float run = r.w_above;
        take = 0;
        while (take < r.ties) {
            run += r.p_key;
            ++take;
            if (strict ? run > target : run >= target) break;
        }
    }
    r.take = take < 1 ? (r.ties > 0 ? 1 : 0) : take;
    return r;
}

// Index of the `rank`-th (1-based, ascending index) token whose key equals `key` (-1: there are fewer).  A thread
// counts a run of neighbouring tokens; the counts are scanned in the wave and over the waves, and the thread in
// whose run the rank falls walks it.  `s_counts`: an entry a wave.
__device__ int nth_with_key(const uint32_t* __restrict__ keys, int vocab, uint32_t key, int rank, int* s_counts) {
    const int per = (vocab + blockDim.x - 1) / blockDim.x;
    const int lo = threadIdx.x * per, hi = lo + per < vocab ? lo + per : vocab;
    int mine = 0;
    for (int c = lo; c < hi; ++c) mine += keys[c] == key;
    const int lane = threadIdx.x & (IA_WAVE - 1), wave = threadIdx.x / IA_WAVE;
    int upto = mine;
#pragma unroll
    for (int o = 1; o < IA_WAVE; o <<= 1) {
        const int other = __shfl_up(upto, o, IA_WAVE);
        if (lane >= o) upto += other;
    }
    __shared__ int s_index;
    __syncthreads();
    if (lane == IA_WAVE - 1) s_counts[wave] = upto;
    if (threadIdx.x == 0) s_index = -1;
    __syncthreads();
    int before = upto - mine;
    for (int w = 0; w < wave; ++w) before += s_counts[w];
    if (before < rank && rank <= before + mine) {
        int seen = before;
        for (int c = lo; c < hi; ++c)
            if (keys[c] == key && ++seen == rank) { s_index = c; break; }
    }
    __syncthreads();
    return s_index;
}

// The first token after (prev_key, prev_idx) in the order of the reference's sorted list: keys
// descending, equal keys by ascending index (its sort is stable).  Returns the index, or -1.
__device__ int next_in_order(const uint32_t* __restrict__ keys, int vocab, uint32_t prev_key, int prev_idx,
                             uint32_t* s_key, int* s_idx) {
    uint32_t bk = 0u;
    int bi = -1;
    for (int c = threadIdx.x; c < vocab; c += blockDim.x) {
        const uint32_t k = keys[c];
        if (!(k < prev_key || (k == prev_key && c > prev_idx))) continue;
        if (bi < 0 || k > bk || (k == bk && c < bi)) { bk = k; bi = c; }
    }
#pragma unroll
    for (int o = IA_WAVE / 2; o > 0; o >>= 1) {
        const uint32_t ok = (uint32_t)__shfl_xor((int)bk, o, IA_WAVE);
        const int oi = __shfl_xor(bi, o, IA_WAVE);
        if (oi >= 0 && (bi < 0 || ok > bk || (ok == bk && oi < bi))) { bk = ok; bi = oi; }
    }
    __syncthreads();
    if ((threadIdx.x & (IA_WAVE - 1)) == 0) { s_key[threadIdx.x / IA_WAVE] = bk; s_idx[threadIdx.x / IA_WAVE] = bi; }
    __syncthreads();
    bk = 0u; bi = -1;
    for (int w = 0; w < (int)(blockDim.x / IA_WAVE); ++w) {
        const uint32_t ok = s_key[w];
        const int oi = s_idx[w];
        if (oi >= 0 && (bi < 0 || ok > bk || (ok == bk && oi < bi))) { bk = ok; bi = oi; }
    }
    __syncthreads();
    return bi;
}

#define SAMPLE_MAX_TOP 20

// With a top_k of up to SAMPLE_FAST_K every filter works on the first top_k entries of the ordered list, so
// the row's top_k tokens are picked out first (three histograms over the key's bits find the k-th largest
// key; equal keys are taken by ascending index), sorted in shared memory, and one thread then does what the
// reference does with its sorted list, in its order and with its sums (sampler.rs:256-335): six passes over
// the row instead of the hundred of the bisections below (16 rows of 152 k: 2.5 ms -> 0.16 ms).
#define SAMPLE_FAST_K 1024
// f(index, key) for all keys of a row, this thread's share, four loads under way at a time.
template <typename F>
__device__ __forceinline__ void for_each_key(const uint32_t* __restrict__ keys, int vocab, F f) {
    for (int c0 = threadIdx.x; c0 < vocab; c0 += 4 * blockDim.x) {
        uint32_t k[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + j * (int)blockDim.x;
            k[j] = c < vocab ? keys[c] : 0u;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + j * (int)blockDim.x;
            if (c < vocab) f(c, k[j]);
        }
    }
}
// The first k entries of the ordered list of `n` keys (keys descending, equal keys by ascending place): every
// key above `kth`, and the keys equal to it up to place `last_tie`.  0 < k < n.  Three histograms over the
// key's bits, 11 + 11 + 10 at a time, find the k-th largest key.
struct Cut { uint32_t kth; int last_tie; };
__device__ Cut top_k_cut(const uint32_t* __restrict__ keys, int n, int k, int* s_counts) {
    __shared__ int hist[2048];
    __shared__ int s_bin, s_above;
    uint32_t prefix = 0u;
    int prefix_bits = 0, need = k;
    for (int level = 0; level < 3; ++level) {
        const int bits = level < 2 ? 11 : 10;
        const int shift = 32 - prefix_bits - bits;
        for (int i = threadIdx.x; i < 2048; i += blockDim.x) hist[i] = 0;
        __syncthreads();
        for_each_key(keys, n, [&](int, uint32_t key) {
            if (prefix_bits == 0 || (key >> (32 - prefix_bits)) == prefix)
                atomicAdd(&hist[(key >> shift) & ((1u << bits) - 1u)], 1);
        });
        __syncthreads();
        // the highest bin at which the count from the top reaches `need`: lane l of the first wave adds up
        // bins top - 32 l - 31 .. top - 32 l, the lanes' sums are scanned, and the lane where the count is
        // reached walks its own bins
        if (threadIdx.x < IA_WAVE) {
            const int n_bins = 1 << bits, per = n_bins / IA_WAVE;
            const int top = n_bins - 1 - (int)threadIdx.x * per;
            int mine = 0;
            for (int i = 0; i < per; ++i) mine += hist[top - i];
            int upto = mine;                                   // inclusive scan over the lanes
#pragma unroll
            for (int o = 1; o < IA_WAVE; o <<= 1) {
                const int other = __shfl_up(upto, o, IA_WAVE);
                if ((int)threadIdx.x >= o) upto += other;
            }
            const unsigned long long reached = __ballot(upto >= need);
            const int first = reached ? __ffsll((long long)reached) - 1 : IA_WAVE - 1;
            if ((int)threadIdx.x == first) {
                int cum = upto - mine, b = top;
                for (; b > top - per + 1; --b) {
                    if (cum + hist[b] >= need) break;
                    cum += hist[b];
                }
                s_bin = b;
                s_above = cum;
            }
        }
        __syncthreads();
        need -= s_above;
        prefix = (prefix << bits) | (uint32_t)s_bin;
        prefix_bits += bits;
        __syncthreads();
    }
    Cut cut;
    cut.kth = prefix;                                       // `need` (>= 1) of the tokens with this key belong to the list
    const int ties = hist[cut.kth & 1023u];
    __syncthreads();
    cut.last_tie = n;                                       // ties up to this place are taken
    if (ties > need) cut.last_tie = nth_with_key(keys, n, cut.kth, need, s_counts);
    return cut;
}

// The reference's steps on the first k entries of a row's ordered list.  `keys` [n] holds the row's candidates in
// the order of their tokens' indices (every stretch of the row has left its own first k there, so the row's first
// k are among them), `token_of` [n] their tokens, `probs` the whole row's probabilities by token.
// `open`: the row has no top_k; k tokens are only the beginning of its list, whose weight is `total`.  The steps
// then succeed if top_p or min_p end the list within these k, or else the walk ends there; if not, nothing is
// written and false comes back (the caller goes the long way).
__device__ bool sample_top_k(int* __restrict__ out, const uint32_t* __restrict__ keys, const int* __restrict__ token_of,
                             const float* __restrict__ probs, int n_keys, int rowi, int k, bool open, float total,
                             float tp, float mp, float u, int want_top, float* __restrict__ lp_out,
                             int* __restrict__ lp_ids, int* s_counts) {
    __shared__ unsigned long long cand[SAMPLE_FAST_K];      // (key, ~place): larger is earlier in the list
    __shared__ int s_n, s_done;
    Cut cut;
    if (k < n_keys) cut = top_k_cut(keys, n_keys, k, s_counts);
    else { cut.kth = 0u; cut.last_tie = n_keys; }
    const uint32_t kth = cut.kth;
    const int last_tie = cut.last_tie;
    if (threadIdx.x == 0) s_n = 0;
    __syncthreads();
    for_each_key(keys, n_keys, [&](int c, uint32_t key) {
        if (key > kth || (key == kth && c <= last_tie)) {
            const int slot = atomicAdd(&s_n, 1);
            if (slot < SAMPLE_FAST_K) cand[slot] = ((unsigned long long)key << 32) | (uint32_t)~(uint32_t)c;
        }
    });
    __syncthreads();
    const int n = s_n < k ? s_n : k;                        // = k
    int padded = 2;
    while (padded < n) padded <<= 1;
    for (int i = n + threadIdx.x; i < padded; i += blockDim.x) cand[i] = 0ull;
    // ---- bitonic sort, descending
    for (int size = 2; size <= padded; size <<= 1)
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int t = threadIdx.x; t < padded / 2; t += blockDim.x) {
                const int i = 2 * t - (t & (stride - 1)), j = i + stride;
                const bool down = (i & size) == 0;
                const unsigned long long a = cand[i], b = cand[j];
                if ((a < b) == down) { cand[i] = b; cand[j] = a; }
            }
        }
    __syncthreads();
    __shared__ float cprob[SAMPLE_FAST_K];
    for (int i = threadIdx.x; i < n; i += blockDim.x) cprob[i] = probs[token_of[(int)~(uint32_t)(cand[i] & 0xffffffffull)]];
    __syncthreads();
    if (threadIdx.x == 0) {
        // ---- the reference's steps 7 to 12 on its sorted list
        auto index_of = [&](int i) { return token_of[(int)~(uint32_t)(cand[i] & 0xffffffffull)]; };
        bool ended = !open, done = true;                    // ended: the list's end lies within these n tokens
        int len = n;
        if (tp < 1.0f) {
            float cumsum = 0.f;
            bool found = false;
            for (int i = 0; i < len; ++i) {
                cumsum += cprob[i];
                if (cumsum >= tp) { len = i + 1; found = true; break; }
            }
            if (found) ended = true;
            else if (open) done = false;                    // the nucleus is longer than what was picked out
        }
        if (done && mp > 0.0f && len > 0) {
            const float threshold = cprob[0] * mp;
            int cut = 0;
            while (cut < len && cprob[cut] >= threshold) ++cut;
            if (cut < len) { if (cut > 0) len = cut; ended = true; }
            else if (!ended) done = false;                  // every picked token passes: the cut lies further on
        }
        float filtered = total;
        if (done && ended) {
            filtered = 0.f;
            for (int i = 0; i < len; ++i) filtered += cprob[i];
        }
        int at = -1;
        if (done && filtered > 0.f) {
            float rng = u;
            for (int i = 0; i < len; ++i) {
                const float norm = cprob[i] / filtered;
                if (rng < norm) { at = i; break; }
                rng -= norm;
            }
            if (at < 0) {
                if (ended) at = len - 1;
                else done = false;                          // the walk goes on beyond what was picked out
            }
        }
        if (done) {
            const float denom = filtered > 0.f ? filtered : 1.0f;
            if (want_top >= 0)
                for (int i = 0; i < want_top && i < SAMPLE_MAX_TOP && i < len; ++i) {
                    const float pi = cprob[i];
                    lp_ids[(size_t)rowi * SAMPLE_MAX_TOP + i] = index_of(i);
                    lp_out[(size_t)rowi * (1 + SAMPLE_MAX_TOP) + 1 + i] = pi > 0.f ? logf(pi / denom) : -INFINITY;
                }
            if (!(filtered > 0.f)) {
                out[rowi] = len > 0 ? index_of(0) : 0;
                if (want_top >= 0) lp_out[(size_t)rowi * (1 + SAMPLE_MAX_TOP)] = -INFINITY;
            } else {
                out[rowi] = index_of(at);
                if (want_top >= 0) {
                    const float pt = cprob[at] / filtered;
                    lp_out[(size_t)rowi * (1 + SAMPLE_MAX_TOP)] = pt > 0.f ? logf(pt) : -INFINITY;
                }
            }
        }
        s_done = done ? 1 : 0;
    }
    __syncthreads();
    return s_done != 0;
}

// ---- a row's workspace and the two passes that fill it --------------------------------------
// Temperature, softmax and the ordering keys of a row are the work of many blocks (a row of 152 k logits kept one
// block busy for 150 us, whatever the batch): the row is cut into stretches of up to SAMPLE_STRETCH tokens, a block each
// (a stretch's keys fit the block's shared memory).
//   pass 1 (sample_partials_kernel): the stretch's maximum of z / temperature and its sum of exp(. - that maximum);
//   pass 2 (sample_stretch_kernel): the row's maximum and sum from the stretches' (every block adds them up in the
//     same order), probabilities and keys of the stretch, the sum of its probabilities, and the stretch's own
//     first k entries of the ordered list (k: the row's top_k, or SAMPLE_FAST_K for a row without one), written
//     in the order of their tokens at a place that follows from k and the stretches' lengths alone;
//   then one block a row (sample_kernel) picks the row's first k among those candidates and walks them.
// A row's words: keys [vocab], probabilities [vocab], the candidates' keys and tokens [stretches * SAMPLE_FAST_K]
// each, and the stretches' maxima, sums and sums of probabilities [stretches] each.
#define SAMPLE_STRETCH 4096
#define SAMPLE_STAGED 8192              // candidates of a row that its last block keeps in shared memory
#define SAMPLE_MAX_STRETCHES 1024       // the stretches' sums meet in a block's shared memory: 4 M tokens a row
struct RowLayout {
    int vocab, stretches, stretch;      // stretch: tokens a stretch (the last one may be shorter), a multiple of 4
    long long words;                    // of a row
    __host__ __device__ int length(int b) const { const int left = vocab - b * stretch; return left < stretch ? left : stretch; }
    // candidates that the stretches before b leave when every stretch leaves its first k (or all it has)
    __host__ __device__ int candidates_before(int b, int k) const {
        const int each = k < stretch ? k : stretch;     // every stretch before the last is a whole one
        return b * each;
    }
    __host__ __device__ int candidates(int k) const {
        const int last = length(stretches - 1);
        return candidates_before(stretches - 1, k) + (k < last ? k : last);
    }
    __device__ uint32_t* keys(uint32_t* ws, int row) const { return ws + (size_t)row * words; }
    __device__ float* probs(uint32_t* ws, int row) const { return (float*)(keys(ws, row) + vocab); }
    __device__ uint32_t* cand_keys(uint32_t* ws, int row) const { return keys(ws, row) + 2 * (size_t)vocab; }
    __device__ int* cand_tokens(uint32_t* ws, int row) const { return (int*)(cand_keys(ws, row) + (size_t)stretches * SAMPLE_FAST_K); }
    __device__ float* part_max(uint32_t* ws, int row) const { return (float*)(cand_tokens(ws, row) + (size_t)stretches * SAMPLE_FAST_K); }
    __device__ float* part_sum(uint32_t* ws, int row) const { return part_max(ws, row) + stretches; }
    __device__ float* part_total(uint32_t* ws, int row) const { return part_sum(ws, row) + stretches; }
};

static RowLayout row_layout(int vocab) {
    RowLayout l;
    l.vocab = vocab;
    l.stretches = (vocab + SAMPLE_STRETCH - 1) / SAMPLE_STRETCH;
    l.stretch = ((vocab + l.stretches - 1) / l.stretches + 3) & ~3;
    const long long words = 2LL * vocab + 2LL * l.stretches * SAMPLE_FAST_K + 3LL * l.stretches;
    l.words = (words + 3) & ~3LL;
    return l;
}

// The temperature a row is sampled at; false: the row is a greedy one and has no use for probabilities.
__device__ __forceinline__ bool row_temperature(const float* temperature, const int* n_top, int rowi, float& temp) {
    temp = temperature[rowi];
    if (temp < 1e-5f) {
        if (n_top == nullptr || n_top[rowi] < 0) return false;
        temp = 1e-5f;           // with log-probabilities the reference takes no shortcut (sampler.rs:176, :232-239)
    }
    return true;
}

// The row's maximum, the sum of exp(z / temperature - maximum) and (with `with_total`) the sum of the probabilities
// from the stretches' (a stretch of nothing but -inf adds nothing to the sum); every block that asks gets the same bits.
// `s_parts`: 3 * stretches floats of shared memory.  All threads of the block call it.
struct RowSums { float mx, sum, total; };
__device__ RowSums row_sums(const RowLayout& l, uint32_t* ws, int rowi, bool with_total, float* s_parts) {
    const float* parts = l.part_max(ws, rowi);               // maxima, sums, totals: one after the other
    const int n = (with_total ? 3 : 2) * l.stretches;
    for (int i = threadIdx.x; i < n; i += blockDim.x) s_parts[i] = parts[i];
    __syncthreads();
    RowSums r;
    r.mx = -INFINITY;
    for (int b = 0; b < l.stretches; ++b) r.mx = fmaxf(r.mx, s_parts[b]);
    r.sum = 0.f;
    for (int b = 0; b < l.stretches; ++b)
        if (s_parts[b] > -INFINITY) r.sum += s_parts[l.stretches + b] * expf(s_parts[b] - r.mx);
    r.total = 0.f;
    if (with_total)
        for (int b = 0; b < l.stretches; ++b) r.total += s_parts[2 * l.stretches + b];
    __syncthreads();
    return r;
}

__global__ __launch_bounds__(256) void sample_partials_kernel(const float* __restrict__ logits, uint32_t* __restrict__ workspace,
                                                              const RowLayout l, const float* __restrict__ temperature,
                                                              const int* __restrict__ n_top) {
    __shared__ float scratch[32];
    const int rowi = blockIdx.y, b = blockIdx.x;
    float temp;
    if (!row_temperature(temperature, n_top, rowi, temp)) return;
    const float* row = logits + (size_t)rowi * l.vocab + (size_t)b * l.stretch;
    const int n = l.length(b);
    // temperature, and the softmax's two sums (sampler.rs:232-249); four loads under way
    float mx = -INFINITY;
    for (int c0 = threadIdx.x; c0 < n; c0 += 4 * blockDim.x) {
        float z[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + j * (int)blockDim.x;
            z[j] = c < n ? row[c] : -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (c0 + j * (int)blockDim.x < n) mx = fmaxf(mx, z[j] / temp);
    }
    mx = wave_max(mx);
    if ((threadIdx.x & (IA_WAVE - 1)) == 0) scratch[16 + threadIdx.x / IA_WAVE] = mx;
    __syncthreads();
    for (int w = 0; w < (int)(blockDim.x / IA_WAVE); ++w) mx = fmaxf(mx, scratch[16 + w]);
    float sum = 0.f;
    if (mx > -INFINITY)
        for (int c0 = threadIdx.x; c0 < n; c0 += 4 * blockDim.x) {
            float z[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = c0 + j * (int)blockDim.x;
                z[j] = c < n ? row[c] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (c0 + j * (int)blockDim.x < n) sum += expf(z[j] / temp - mx);
        }
    sum = block_sum(sum, scratch);
    if (threadIdx.x == 0) {
        l.part_max(workspace, rowi)[b] = mx;
        l.part_sum(workspace, rowi)[b] = sum;
    }
}

// How many entries of a row's ordered list are picked out before the reference's steps run on them: the row's
// top_k, SAMPLE_FAST_K for a row without one, 0 for a row that goes the long way (a top_k beyond SAMPLE_FAST_K, a
// vocabulary within it, or the switch off).
__device__ __forceinline__ int picked_out(int k, int vocab, int fast_top_k) {
    if (!fast_top_k) return 0;
    if (k > 0 && k < vocab) return k <= SAMPLE_FAST_K ? k : 0;
    return vocab > SAMPLE_FAST_K ? SAMPLE_FAST_K : 0;
}

#define STRETCH_THREADS 256
__global__ __launch_bounds__(STRETCH_THREADS) void sample_stretch_kernel(
    const float* __restrict__ logits, uint32_t* __restrict__ workspace, const RowLayout l,
    const float* __restrict__ temperature, const int* __restrict__ top_k, const int* __restrict__ n_top, int fast_top_k) {
    __shared__ float scratch[32];
    __shared__ int s_counts[STRETCH_THREADS];
    __shared__ int s_waves[STRETCH_THREADS / IA_WAVE];
    __shared__ uint32_t s_keys[SAMPLE_STRETCH];             // the stretch's keys: the choice below reads them several times
    __shared__ float s_parts[2 * SAMPLE_MAX_STRETCHES];
    const int rowi = blockIdx.y, b = blockIdx.x;
    float temp;
    if (!row_temperature(temperature, n_top, rowi, temp)) return;
    const int lo = b * l.stretch, n = l.length(b);
    const float* row = logits + (size_t)rowi * l.vocab + lo;
    uint32_t* keys = l.keys(workspace, rowi) + lo;
    float* probs = l.probs(workspace, rowi) + lo;
    const RowSums rs = row_sums(l, workspace, rowi, false, s_parts);
    // The list is ordered by the probabilities themselves, as the reference sorts them: logits whose
    // probabilities round to the same number (or vanish together) are ties, taken in index order.
    float t = 0.f;
    for (int c0 = threadIdx.x; c0 < n; c0 += 4 * blockDim.x) {
        float z[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + j * (int)blockDim.x;
            z[j] = c < n ? row[c] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + j * (int)blockDim.x;
            if (c < n) {
                const float e = expf(z[j] / temp - rs.mx);
                const float pr = rs.sum > 0.f ? e / rs.sum : e;
                const uint32_t key = order_key(pr);
                probs[c] = pr;
                keys[c] = key;
                s_keys[c] = key;
                t += pr;
            }
        }
    }
    t = block_sum(t, scratch);
    if (threadIdx.x == 0) l.part_total(workspace, rowi)[b] = t;
    const int k = picked_out(top_k[rowi], l.vocab, fast_top_k);
    if (k == 0) return;
    __syncthreads();
    // ---- the stretch's own first k, in the order of their tokens
    uint32_t* ck = l.cand_keys(workspace, rowi) + l.candidates_before(b, k);
    int* ct = l.cand_tokens(workspace, rowi) + l.candidates_before(b, k);
    if (k >= n) {
        for (int c = threadIdx.x; c < n; c += blockDim.x) { ck[c] = s_keys[c]; ct[c] = lo + c; }
        return;
    }
    const Cut cut = top_k_cut(s_keys, n, k, s_counts);
    // a thread takes a run of neighbouring tokens, counts those of the list, and writes them behind what the
    // threads before it have counted
    const int per = (n + blockDim.x - 1) / blockDim.x;
    const int first = threadIdx.x * per, last = first + per < n ? first + per : n;
    int mine = 0;
    for (int c = first; c < last; ++c) {
        const uint32_t key = s_keys[c];
        mine += (key > cut.kth || (key == cut.kth && c <= cut.last_tie)) ? 1 : 0;
    }
    int upto = mine;                                        // inclusive scan over the wave's lanes
    const int lane = threadIdx.x & (IA_WAVE - 1), wave = threadIdx.x / IA_WAVE;
#pragma unroll
    for (int o = 1; o < IA_WAVE; o <<= 1) {
        const int other = __shfl_up(upto, o, IA_WAVE);
        if (lane >= o) upto += other;
    }
    if (lane == IA_WAVE - 1) s_waves[wave] = upto;
    __syncthreads();
    int at = upto - mine;
    for (int w = 0; w < wave; ++w) at += s_waves[w];
    for (int c = first; c < last; ++c) {
        const uint32_t key = s_keys[c];
        if (key > cut.kth || (key == cut.kth && c <= cut.last_tie)) {
            if (at < k) { ck[at] = key; ct[at] = lo + c; }
            ++at;
        }
    }
}

// n_top (may be null): per row -1 = no log-probabilities, else how many of the list's first entries are
// reported besides the drawn token's (sampler.rs:285-352).  lp_out [rows, 1 + SAMPLE_MAX_TOP]: the drawn
// token's log-probability within the kept list, then the entries'; lp_ids [rows, SAMPLE_MAX_TOP]: their ids (-1: none).
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    int* __restrict__ out, const float* __restrict__ logits, uint32_t* __restrict__ workspace, const RowLayout l,
    const float* __restrict__ temperature, const int* __restrict__ top_k, const float* __restrict__ top_p,
    const float* __restrict__ min_p, const float* __restrict__ u, const int* __restrict__ n_top,
    float* __restrict__ lp_out, int* __restrict__ lp_ids, int fast_top_k) {
    __shared__ float scratch[32];
    __shared__ int s_counts[SAMPLE_THREADS];
    __shared__ float sv[16];
    __shared__ int si[16];
    const int rowi = blockIdx.x;
    const int vocab = l.vocab;
    const float* row = logits + (size_t)rowi * vocab;
    const int want_top = n_top != nullptr ? n_top[rowi] : -1;
    if (want_top >= 0 && threadIdx.x < SAMPLE_MAX_TOP) {
        lp_ids[(size_t)rowi * SAMPLE_MAX_TOP + threadIdx.x] = -1;
        lp_out[(size_t)rowi * (1 + SAMPLE_MAX_TOP) + 1 + threadIdx.x] = -INFINITY;
    }
    float temp;
    if (!row_temperature(temperature, n_top, rowi, temp)) {
        argmax_row(row, vocab, sv, si, out + rowi);
        return;
    }
    const uint32_t* keys = l.keys(workspace, rowi);
    const float* probs = l.probs(workspace, rowi);
    __shared__ float s_parts[3 * SAMPLE_MAX_STRETCHES];
    const RowSums rs = row_sums(l, workspace, rowi, true, s_parts);
    const float sum = rs.sum, total = rs.total;             // total: the weight of the whole list

    const int k = top_k[rowi];
    const int picked = picked_out(k, vocab, fast_top_k);
    if (picked > 0) {
        // the list's first entries: the row's top_k, or, without one, 1,024 tokens, which hold the nucleus, the min_p
        // cut or the walk's end for all but flat distributions
        const bool open = !(k > 0 && k < vocab);
        // (few candidates are read from shared memory: the choice among them reads them several times)
        __shared__ uint32_t s_cand[SAMPLE_STAGED];
        const int n_cand = l.candidates(picked);
        const uint32_t* cand_keys = l.cand_keys(workspace, rowi);
        if (n_cand <= SAMPLE_STAGED) {
            for (int i = threadIdx.x; i < n_cand; i += blockDim.x) s_cand[i] = cand_keys[i];
            __syncthreads();
            cand_keys = s_cand;
        }
        if (sample_top_k(out, cand_keys, l.cand_tokens(workspace, rowi), probs, n_cand, rowi,
                         picked, open, total, top_p[rowi], min_p[rowi], u[rowi], want_top, lp_out, lp_ids, s_counts))
            return;
    }
    // how long the kept prefix is (sampler.rs:256-283)
    int keep = vocab;
    if (k > 0 && k < keep) keep = k;
    const float tp = top_p[rowi];
    if (tp < 1.0f) {
        const Prefix p = shortest_prefix(keys, probs, vocab, tp, false, false, scratch);
        const int n = p.above + p.take;
        if (n < keep) keep = n;
    }
    const float mp = min_p[rowi];
    if (mp > 0.0f) {
        const float thr = (sum > 0.f ? 1.0f / sum : 1.0f) * mp;       // the largest probability is exp(0) / sum
        float n = 0.f;
        for (int c = threadIdx.x; c < vocab; c += blockDim.x) n += probs[c] >= thr ? 1.0f : 0.0f;
        const int cnt = (int)block_sum(n, scratch);
        if (cnt > 0 && cnt < keep) keep = cnt;
    }

    // the kept prefix by key and tie count, and its weight (sampler.rs:286-292)
    Prefix kept;
    float filtered;
    if (keep < vocab) {
        kept = shortest_prefix(keys, probs, vocab, (float)keep, true, false, scratch);
        float wa = 0.f;
        float pk = 0.f, seen = 0.f;
        for (int c = threadIdx.x; c < vocab; c += blockDim.x) {
            if (keys[c] > kept.key) wa += probs[c];
            else if (keys[c] == kept.key) { pk = probs[c]; seen = 1.f; }
        }
        wa = block_sum(wa, scratch);
        __shared__ float s_pk2;
        if (threadIdx.x == 0) s_pk2 = 0.f;
        __syncthreads();
        if (seen > 0.f) s_pk2 = pk;
        __syncthreads();
        filtered = wa + (float)kept.take * s_pk2;
    } else {
        kept.key = 0u; kept.above = 0; kept.ties = 0; kept.take = 0;
        filtered = total;
    }

    // the walk (sampler.rs:323-335): the first place where the running sum of p / filtered exceeds u
    int token;
    if (!(filtered > 0.f)) {
        argmax_row(row, vocab, sv, si, out + rowi);
        if (want_top >= 0 && threadIdx.x == 0) lp_out[(size_t)rowi * (1 + SAMPLE_MAX_TOP)] = -INFINITY;
        return;
    }
    const Prefix hit = shortest_prefix(keys, probs, vocab, u[rowi] * filtered, false, true, scratch);
    if (keep < vocab && (hit.ties == 0 || hit.above + hit.take > keep)) {
        token = nth_with_key(keys, vocab, kept.key, kept.take, s_counts);          // the last kept token
    } else if (hit.ties == 0) {
        // u * filtered is not exceeded even by the whole list (rounding): the last of the list,
        // that is the last token with the smallest key
        uint32_t lowest = 0xffffffffu;
        for (int c = threadIdx.x; c < vocab; c += blockDim.x) lowest = keys[c] < lowest ? keys[c] : lowest;
#pragma unroll
        for (int o = IA_WAVE / 2; o > 0; o >>= 1) {
            const uint32_t other = (uint32_t)__shfl_xor((int)lowest, o, IA_WAVE);
            lowest = other < lowest ? other : lowest;
        }
        __syncthreads();
        if ((threadIdx.x & (IA_WAVE - 1)) == 0) si[threadIdx.x / IA_WAVE] = (int)lowest;
        __syncthreads();
        for (int w = 0; w < SAMPLE_THREADS / IA_WAVE; ++w) lowest = (uint32_t)si[w] < lowest ? (uint32_t)si[w] : lowest;
        float n = 0.f;
        for (int c = threadIdx.x; c < vocab; c += blockDim.x) n += keys[c] == lowest ? 1.0f : 0.0f;
        token = nth_with_key(keys, vocab, lowest, (int)block_sum(n, scratch), s_counts);
    } else {
        token = nth_with_key(keys, vocab, hit.key, hit.take, s_counts);
    }
    if (threadIdx.x == 0) out[rowi] = token;
    if (want_top < 0) return;
    // log-probabilities within the kept list: the drawn token's, then the list's first entries
    if (threadIdx.x == 0) {
        const float pt = probs[token];
        lp_out[(size_t)rowi * (1 + SAMPLE_MAX_TOP)] = pt > 0.f ? logf(pt / filtered) : -INFINITY;
    }
    const int n_list = keep < vocab ? keep : vocab;
    uint32_t prev_key = 0xffffffffu;
    int prev_idx = -1;
    uint32_t* s_key = (uint32_t*)scratch;
    for (int i = 0; i < want_top && i < SAMPLE_MAX_TOP && i < n_list; ++i) {
        const int idx = next_in_order(keys, vocab, prev_key, prev_idx, s_key, si);
        if (idx < 0) break;
        if (threadIdx.x == 0) {
            const float pi = probs[idx];
            lp_ids[(size_t)rowi * SAMPLE_MAX_TOP + i] = idx;
            lp_out[(size_t)rowi * (1 + SAMPLE_MAX_TOP) + 1 + i] = pi > 0.f ? logf(pi / filtered) : -INFINITY;
        }
        prev_key = keys[idx];
        prev_idx = idx;
    }
}

// Words of workspace for `rows` rows (see the layout of a row above).
extern "C" long long ia_sample_workspace(int rows, int vocab) {
    return vocab > 0 && rows > 0 ? (long long)rows * row_layout(vocab).words : 0;
}

static int g_sample_fast = 1;
// Measurement and test switch: 0 sends rows with a top_k through the bisections as well.
extern "C" void ia_sample_tune(int fast_top_k) { g_sample_fast = fast_top_k; }

extern "C" int ia_sample_max_top(void) { return SAMPLE_MAX_TOP; }

// n_top, lp_out, lp_ids: all null, or all given (see sample_kernel).
extern "C" int ia_sample(int* out, const float* logits, void* workspace, int rows, int vocab,
                         const float* temperature, const int* top_k, const float* top_p, const float* min_p,
                         const float* u, const int* n_top, float* lp_out, int* lp_ids, hipStream_t stream) {
    IA_CHECK(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    IA_CHECK(workspace != nullptr || rows == 0, "sample: needs a workspace of ia_sample_workspace(rows, vocab) words");
    IA_CHECK((n_top == nullptr) == (lp_out == nullptr) && (n_top == nullptr) == (lp_ids == nullptr),
             "sample: the arrays of the log-probabilities come together");
    IA_CHECK(rows <= 65535, "sample: at most 65535 rows a call, not %d", rows);
    IA_CHECK(vocab <= SAMPLE_STRETCH * SAMPLE_MAX_STRETCHES, "sample: at most %d tokens a row, not %d", SAMPLE_STRETCH * SAMPLE_MAX_STRETCHES, vocab);
    if (rows == 0) return 0;
    const RowLayout l = row_layout(vocab);
    const dim3 grid((unsigned)l.stretches, (unsigned)rows);
    sample_partials_kernel<<<grid, 256, 0, stream>>>(logits, (uint32_t*)workspace, l, temperature, n_top);
    sample_stretch_kernel<<<grid, STRETCH_THREADS, 0, stream>>>(logits, (uint32_t*)workspace, l, temperature, top_k, n_top,
                                                               g_sample_fast);
    sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(out, logits, (uint32_t*)workspace, l, temperature,
                                                       top_k, top_p, min_p, u, n_top, lp_out, lp_ids, g_sample_fast);
    IA_LAUNCH_CHECK("sample");
    return 0;
}
