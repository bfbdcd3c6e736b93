// Next-token choice on the GPU: the reference's logits processors in their order, then argmax or
// a draw from the softmax, one workgroup per row of 32-bit logits.
//
// Order (src/transformers/generation/utils.py:898-1097): additive biases on tokens, repetition penalty, banned
// tokens, EOS suppression (minimum length), a forced last token, removal of invalid values, the growing bonus on
// EOS, then for sampling temperature, top-k, top-p, min-p;
// then softmax and a draw (:3274-3279) or argmax.  Formulas: src/transformers/generation/logits_process.py
// :1112-1140 (biases), :337-343 (penalty), :144-151 (EOS), :1590-1596 (forced token), :1618-1626 (invalid),
// :1716-1727 (bonus on EOS), :286-289 (temperature), :505-518 (top-k),
// :452-465 (top-p), :578-595 (min-p), :1762-1764 (renormalise).
//
// Thresholds are found without sorting: the k-th largest score by a radix search on counts, the
// top-p cut by a radix search on probability mass held in 40-bit fixed point, so that both are
// sums of integers and do not depend on the order in which threads add.  The searches run over short
// candidate lists where they can (LDS atomics of 65,000 scores that share a few exponent bytes take
// tens of microseconds a pass): the k-th largest of the threads' maxima is a lower bound of the k-th
// largest score, so the scores at or above it are few and hold the threshold; the top-p cut lies among
// the scores that still have mass after top-k, or among those above the 512th largest thread maximum
// if the mass below them fits into 1 - p.  Where a list would overflow, or the cut lies below it, the
// same searches run over the whole row.  The draw inverts the cumulative distribution in index order
// with a fixed summation order (a wave per sixteenth of the row, sums of lanes, then of waves), from
// a uniform number of a counter-based generator keyed by (seed, sequence, step): a sequence draws the
// same token alone or in any batch.
#include "common.h"
#include "pta_kernels.h"

#include <float.h>

#define S_THREADS 1024

// a key that orders like the score; the two zeros are one score and get one key
__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = f == 0.f ? 0u : __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Philox4x32-10 (Salmon et al. 2011), one block of four 32-bit words
__device__ __forceinline__ void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

__device__ __forceinline__ float uniform_of(uint64_t seed, uint32_t seq, uint32_t step) {
    uint32_t c[4] = {seq, step, 0u, 0u};
    philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
    return (float)(c[0] >> 8) * (1.0f / 16777216.0f);  // 24 bits, [0, 1)
}

extern "C" float pta_philox_uniform(uint64_t seed, uint32_t seq, uint32_t step);

struct ArgBest { float v; int i; };

// largest value, lowest index among equals; every thread gets the result
__device__ __forceinline__ ArgBest block_argmax(float v, int i, float* red_v, int* red_i) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, 64);
        const int oi = __shfl_xor(i, o, 64);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) { red_v[wave] = v; red_i[wave] = i; }
    __syncthreads();
    ArgBest b = {red_v[0], red_i[0]};
    for (int w = 1; w < nw; ++w)
        if (red_v[w] > b.v || (red_v[w] == b.v && red_i[w] < b.i)) { b.v = red_v[w]; b.i = red_i[w]; }
    return b;
}

// Greedy choice with no processor in the way: the largest logit of each row, lowest index among equals,
// read sixteen bytes at a time and never written back.
__global__ __launch_bounds__(S_THREADS) void argmax_kernel(int* __restrict__ out_tok, const float* __restrict__ logits,
                                                           int V) {
    __shared__ float red[16];
    __shared__ int red_i[16];
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* l = logits + (long)row * V;
    float mx = -INFINITY;
    int mi = 0x7fffffff;
    const int head = (int)((16 - ((uintptr_t)l & 15)) & 15) / 4;  // elements before the first 16-byte boundary
    const int first = min(head, V), quads = (V - first) / 4;
    if (tid < first && l[tid] > mx) { mx = l[tid]; mi = tid; }
    const float4* l4 = reinterpret_cast<const float4*>(l + first);
    auto four = [&](int q, const float4& v) {
        const int i = first + q * 4;
        if (v.x > mx) { mx = v.x; mi = i; }
        if (v.y > mx) { mx = v.y; mi = i + 1; }
        if (v.z > mx) { mx = v.z; mi = i + 2; }
        if (v.w > mx) { mx = v.w; mi = i + 3; }
    };
    int q = tid;
    for (; q + 3 * S_THREADS < quads; q += 4 * S_THREADS) {  // four loads in flight
        const float4 a = l4[q], b = l4[q + S_THREADS], c = l4[q + 2 * S_THREADS], d = l4[q + 3 * S_THREADS];
        four(q, a); four(q + S_THREADS, b); four(q + 2 * S_THREADS, c); four(q + 3 * S_THREADS, d);
    }
    for (; q < quads; q += S_THREADS) four(q, l4[q]);
    for (int i = first + quads * 4 + tid; i < V; i += S_THREADS)
        if (l[i] > mx) { mx = l[i]; mi = i; }
    // a thread meets its candidates in index order and keeps the first of equals; so does the reduction
    const ArgBest best = block_argmax(mx, mi, red, red_i);
    if (tid == 0) out_tok[row] = best.i;
}

extern "C" int pta_argmax(int* out_tok, const float* logits, int R, int V, void* stream) {
    PTA_REQUIRE(R > 0 && V > 0, "argmax: R=%d V=%d must be positive", R, V);
    PTA_REQUIRE(out_tok && logits, "argmax: null pointer");
    hipLaunchKernelGGL(argmax_kernel, dim3(R), dim3(S_THREADS), 0, (hipStream_t)stream, out_tok, logits, V);
    return pta_check_launch("argmax");
}

#define MASS_ONE 1099511627776.0f /* 2^40 */
#define S_CAP 2048  // candidates a list holds
#define S_SHORT 256  // candidates of the short way, which sorts them by counting

struct SampleShared {
    float red[16];
    int red_i[16];
    unsigned long long red_q[16];
    float seg[S_THREADS / 64];
    uint32_t cnt[256];
    unsigned long long mass[256];
    uint32_t tkey[S_THREADS];  // the threads' largest scores as keys
    uint32_t cand_key[S_CAP];
    unsigned long long cand_q[S_CAP];
    uint32_t bin, remaining, all, n_cand;
    unsigned long long cum;
    // the short way (sample_short): scores seen before, scores that are left, and the survivors in index order
    uint32_t seen[2048], left[2048], banned[2048];
    uint32_t cand_idx[S_SHORT];
    uint32_t s_key[S_SHORT], s_idx[S_SHORT], s_alive[S_SHORT];
    uint32_t pick, last_mass;
};

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// every thread gets the sum; integers, so any order gives the same bits
__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* red) {
    v = wave_sum_u64(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    unsigned long long t = 0;
    for (int i = 0; i < S_THREADS / 64; ++i) t += red[i];
    return t;
}

// inclusive sums over the block's threads in thread order (integers)
__device__ __forceinline__ unsigned long long block_scan_u64(unsigned long long v, unsigned long long* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const unsigned long long up = __shfl_up(v, o, 64);
        if (lane >= o) v += up;
    }
    __syncthreads();
    if (lane == 63) red[wave] = v;
    __syncthreads();
    for (int w = 0; w < wave; ++w) v += red[w];
    return v;
}

// Key of the `want`-th largest (1-based, want <= n) of the n keys of a list in LDS: one byte of the key at a
// time from the top, counts per byte value, the bin picked by all threads together.  Every thread gets it.
__device__ __forceinline__ uint32_t list_kth_largest(SampleShared& sh, const uint32_t* keys, int n, uint32_t want) {
    const int tid = threadIdx.x;
    uint32_t prefix = 0, maskbits = 0, rem = want;
    for (int shift = 24; shift >= 0; shift -= 8) {
        __syncthreads();
        if (tid < 256) sh.cnt[tid] = 0;
        __syncthreads();
        for (int c = tid; c < n; c += S_THREADS) {
            const uint32_t k = keys[c];
            if ((k & maskbits) == prefix) atomicAdd(&sh.cnt[(k >> shift) & 255u], 1u);
        }
        __syncthreads();
        // thread t < 256 stands for bin 255 - t: the inclusive sum counts the keys in its bin and above
        const uint32_t mine = tid < 256 ? sh.cnt[255 - tid] : 0u;
        const uint32_t from_top = (uint32_t)block_scan_u64(mine, sh.red_q);
        if (tid < 256 && from_top >= rem && from_top - mine < rem) {
            sh.bin = (uint32_t)(255 - tid);
            sh.remaining = rem - (from_top - mine);
        }
        __syncthreads();
        prefix |= sh.bin << shift;
        maskbits |= 255u << shift;
        rem = sh.remaining;
    }
    __syncthreads();
    return prefix;
}

// The top-p cut over the list of (key, mass) in LDS, `low` being the mass of the scores below every key of
// the list (low <= T): the lowest key whose mass, with everything below it, passes T.  Returns false if none
// does (everything could go); else `key` is that key and `below` the mass below it.
__device__ __forceinline__ bool list_mass_cut(SampleShared& sh, int n, unsigned long long low, unsigned long long T,
                                              uint32_t& key, unsigned long long& below) {
    const int tid = threadIdx.x;
    uint32_t prefix = 0, maskbits = 0;
    unsigned long long cum = low;
    for (int shift = 24; shift >= 0; shift -= 8) {
        __syncthreads();
        if (tid < 256) sh.mass[tid] = 0ull;
        if (tid == 0) sh.bin = 256u;
        __syncthreads();
        for (int c = tid; c < n; c += S_THREADS) {
            const uint32_t k = sh.cand_key[c];
            const unsigned long long q = sh.cand_q[c];
            if ((k & maskbits) == prefix && q) atomicAdd(&sh.mass[(k >> shift) & 255u], q);
        }
        __syncthreads();
        const unsigned long long mine = tid < 256 ? sh.mass[tid] : 0ull;
        const unsigned long long upto = block_scan_u64(mine, sh.red_q);  // mass of bins 0 .. tid
        if (tid < 256 && cum + upto > T && cum + upto - mine <= T) {      // the first bin that passes T
            sh.bin = (uint32_t)tid;
            sh.cum = cum + upto - mine;
        }
        __syncthreads();
        if (sh.bin == 256u) return false;
        prefix |= sh.bin << shift;
        maskbits |= 255u << shift;
        cum = sh.cum;
    }
    __syncthreads();
    key = prefix;
    below = cum;
    return true;
}

// inclusive sums over the block's threads in thread order, with a fixed tree: inside a wave by doubling
// steps, then the waves' totals in order
__device__ __forceinline__ float block_scan_f32(float v, float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(v, o, 64);
        if (lane >= o) v += up;
    }
    __syncthreads();
    if (lane == 63) red[wave] = v;
    __syncthreads();
    float before = 0.f;
    for (int w = 0; w < wave; ++w) before += red[w];
    return before + v;
}

__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// The processed score of a token before the thresholds: the row's additive biases (a short list of (token,
// value), searched for every score), repetition penalty (tokens seen before are marked in a bitmap in LDS, so
// vocabularies up to 65,536), the row's banned tokens (a second bitmap), EOS suppression, a forced token (every
// other score gone, its own 0; a banned token stays gone), invalid values, the bonus |score| * decay_m on the EOS
// tokens, temperature, in this order.
struct Processed {
    const float* l;
    const uint32_t* seen;  // null: no penalty
    const uint32_t* banned;  // null: no token of this row is banned
    const int* eos;
    int n_eos;  // 0: no suppression
    float penalty, temperature;
    int remove_invalid;
    const int* bias_tok;  // this row's biased tokens, each once, and their values
    const float* bias_val;
    int n_bias;
    const int* forced;
    int n_forced;  // 0: nothing is forced in this step
    int n_eos_all;  // the EOS tokens, whether suppressed or not
    int decay_on;
    float decay_m;
    __device__ __forceinline__ float operator()(int i) const { return of(i, l[i]); }
    __device__ __forceinline__ float of(int i, float x) const {
        for (int t = 0; t < n_bias; ++t)
            if (bias_tok[t] == i) x += bias_val[t];
        if (seen && ((seen[i >> 5] >> (i & 31)) & 1u)) x = x < 0.f ? x * penalty : x / penalty;
        const bool gone = banned && ((banned[i >> 5] >> (i & 31)) & 1u);
        if (gone) x = -INFINITY;
        for (int e = 0; e < n_eos; ++e)
            if (eos[e] == i) x = -INFINITY;
        if (n_forced) {
            bool is = false;
            for (int e = 0; e < n_forced; ++e) is = is || forced[e] == i;
            x = is && !gone ? 0.f : -INFINITY;
        }
        if (remove_invalid) {
            if (x != x) x = 0.f;
            else if (x == INFINITY) x = FLT_MAX;
            else if (x == -INFINITY) x = -FLT_MAX;
        }
        if (decay_on)
            for (int e = 0; e < n_eos_all; ++e)
                if (eos[e] == i) { x += fabsf(x) * decay_m; break; }
        if (temperature != 1.0f) x = x / temperature;
        return x;
    }
};

// marks the tokens of the row's history in sh.seen; returns the bitmap, or null if there is no penalty
__device__ __forceinline__ const uint32_t* mark_seen(SampleShared& sh, int row, int V, float penalty,
                                                     const int* __restrict__ hist, const int* __restrict__ hist_off) {
    if (!(hist_off && penalty != 1.0f)) return nullptr;
    const int tid = threadIdx.x;
    for (int w = tid; w < 2048; w += S_THREADS) sh.seen[w] = 0u;
    __syncthreads();
    for (int t = hist_off[row] + tid; t < hist_off[row + 1]; t += S_THREADS) {
        const int tok = hist[t];
        if (tok >= 0 && tok < V) atomicOr(&sh.seen[tok >> 5], 1u << (tok & 31));
    }
    __syncthreads();
    return sh.seen;
}

// marks the row's banned tokens in sh.banned; returns the bitmap, or null if the row has none
__device__ __forceinline__ const uint32_t* mark_banned(SampleShared& sh, int row, int V, const int* __restrict__ ban,
                                                       const int* __restrict__ ban_off) {
    if (!ban_off || ban_off[row + 1] == ban_off[row]) return nullptr;
    const int tid = threadIdx.x;
    for (int w = tid; w < 2048; w += S_THREADS) sh.banned[w] = 0u;
    __syncthreads();
    for (int t = ban_off[row] + tid; t < ban_off[row + 1]; t += S_THREADS) {
        const int tok = ban[t];
        if (tok >= 0 && tok < V) atomicOr(&sh.banned[tok >> 5], 1u << (tok & 31));
    }
    __syncthreads();
    return sh.banned;
}

// f(i, l[i]) for every score of a row, each thread in ascending order of i.  Sixteen bytes a load and four
// loads in flight per thread: one load at a time leaves a pass waiting for memory most of its time.
template <typename F>
__device__ __forceinline__ void for_each_score(const float* __restrict__ l, int V, F&& f) {
    const int tid = threadIdx.x;
    if ((((uintptr_t)l) & 15) != 0) {
        for (int i = tid; i < V; i += S_THREADS) f(i, l[i]);
        return;
    }
    const float4* l4 = reinterpret_cast<const float4*>(l);
    const int quads = V >> 2;
    auto four = [&](int q, const float4& a) { f(4 * q, a.x); f(4 * q + 1, a.y); f(4 * q + 2, a.z); f(4 * q + 3, a.w); };
    int q = tid;
    for (; q + 3 * S_THREADS < quads; q += 4 * S_THREADS) {
        const float4 a = l4[q], b = l4[q + S_THREADS], c = l4[q + 2 * S_THREADS], d = l4[q + 3 * S_THREADS];
        four(q, a); four(q + S_THREADS, b); four(q + 2 * S_THREADS, c); four(q + 3 * S_THREADS, d);
    }
    for (; q < quads; q += S_THREADS) four(q, l4[q]);
    for (int i = quads * 4 + tid; i < V; i += S_THREADS) f(i, l[i]);
}

// The short way for a draw with top-k, up to 65,536 scores: two passes over the row (one for the threads'
// maxima, one that lists the scores at or above the bound they give), then everything on that list: the
// k-th largest, the survivors in index order, the top-p cut by integer masses, min-p, the draw.  The row is
// never written unless the processed scores are wanted.  Sums of exponentials run over the survivors in
// index order with a fixed tree, so they can round differently from the sums over the whole row (whose
// other terms are zero), but never depend on the batch.  Returns false, having written nothing, if the list
// would have more than S_SHORT entries (many equal scores, or a large k): then the long way runs.
__device__ __forceinline__ bool sample_short(
    SampleShared& sh, int* __restrict__ out_tok, float* __restrict__ work, const Processed& score, int row, int V,
    int top_k, float top_p, float min_p, int renorm, float u) {
    const int tid = threadIdx.x;
    float m = -INFINITY, mx = -INFINITY;
    int mi = 0x7fffffff;
    bool any = false;
    for_each_score(score.l, V, [&](int i, float raw) {
        const float x = score.of(i, raw);
        m = fmaxf(m, x);
        if (x > mx) { mx = x; mi = i; }
        any = true;
    });
    sh.tkey[tid] = any ? order_key(m) : 0u;
    const ArgBest best = block_argmax(mx, mi, sh.red, sh.red_i);
    const uint32_t bound = list_kth_largest(sh, sh.tkey, S_THREADS, (uint32_t)top_k);
    if (tid == 0) sh.n_cand = 0u;
    __syncthreads();
    for_each_score(score.l, V, [&](int i, float raw) {
        const uint32_t k = order_key(score.of(i, raw));
        if (k >= bound) {
            const uint32_t at = atomicAdd(&sh.n_cand, 1u);
            if (at < S_SHORT) { sh.cand_key[at] = k; sh.cand_idx[at] = (uint32_t)i; }
        }
    });
    __syncthreads();
    const int n = (int)sh.n_cand;
    if (n > S_SHORT) return false;
    const uint32_t kth = list_kth_largest(sh, sh.cand_key, n, (uint32_t)top_k);
    // survivors in index order: a survivor's place is the number of survivors before it
    if (tid == 0) sh.n_cand = 0u;
    __syncthreads();
    if (tid < n && sh.cand_key[tid] >= kth) {
        uint32_t place = 0;
        for (int o = 0; o < n; ++o) place += (sh.cand_key[o] >= kth && sh.cand_idx[o] < sh.cand_idx[tid]) ? 1u : 0u;
        sh.s_key[place] = sh.cand_key[tid];
        sh.s_idx[place] = sh.cand_idx[tid];
        sh.s_alive[place] = 1u;
        atomicAdd(&sh.n_cand, 1u);
    }
    __syncthreads();
    const int ns = (int)sh.n_cand;  // at least top_k
    const bool mine = tid < ns;
    const float x = mine ? key_value(sh.s_key[tid]) : -INFINITY;
    if (top_p < 1.0f) {
        const float e = mine ? expf(x - best.v) : 0.f;
        const float incl = block_scan_f32(e, sh.red);
        __syncthreads();
        if (tid == ns - 1) sh.seg[0] = incl;
        __syncthreads();
        const float Z = sh.seg[0];
        const unsigned long long T = (unsigned long long)((double)(1.0f - top_p) * (double)MASS_ONE);
        if (mine) {
            sh.cand_key[tid] = sh.s_key[tid];
            sh.cand_q[tid] = (unsigned long long)(e / Z * MASS_ONE + 0.5f);
        }
        uint32_t cut = 0;
        unsigned long long below = 0ull;
        const bool found = list_mass_cut(sh, ns, 0ull, T, cut, below);
        const uint32_t keep_from = found ? cut : order_key(best.v);  // if everything could go, the largest stays
        __syncthreads();
        if (mine && sh.s_key[tid] < keep_from) sh.s_alive[tid] = 0u;
        if (found) {
            // equal scores at the cut: in index order the first of them go while they fit, never the last
            const unsigned long long q = (unsigned long long)(expf(key_value(cut) - best.v) / Z * MASS_ONE + 0.5f);
            const unsigned long long r = q ? (T - below) / q : 0ull;
            if (r > 0 && mine && sh.s_key[tid] == cut) {
                uint32_t before = 0, ties = 0;
                for (int o = 0; o < ns; ++o) {
                    const bool tie = sh.s_key[o] == cut;
                    ties += tie ? 1u : 0u;
                    before += (tie && o < tid) ? 1u : 0u;
                }
                if (before < r && before != ties - 1) sh.s_alive[tid] = 0u;
            }
        }
        __syncthreads();
    }
    if (min_p > 0.0f) {
        const float e = (mine && sh.s_alive[tid]) ? expf(x - best.v) : 0.f;
        const float incl = block_scan_f32(e, sh.red);
        __syncthreads();
        if (tid == ns - 1) sh.seg[0] = incl;
        __syncthreads();
        const float Z = sh.seg[0];
        const float thr = min_p * (1.0f / Z);
        if (mine && x != best.v && e / Z < thr) sh.s_alive[tid] = 0u;
        __syncthreads();
    }
    // the draw over the survivors in index order
    const float e = (mine && sh.s_alive[tid]) ? expf(x - best.v) : 0.f;
    const float incl = block_scan_f32(e, sh.red);
    __syncthreads();
    if (tid == ns - 1) sh.seg[0] = incl;
    if (tid == 0) { sh.pick = 0xffffffffu; sh.last_mass = 0u; }
    __syncthreads();
    const float total = sh.seg[0];
    const float target = u * total;
    if (mine && incl > target) atomicMin(&sh.pick, (uint32_t)tid);
    if (mine && e > 0.f) atomicMax(&sh.last_mass, (uint32_t)tid);
    __syncthreads();
    if (tid == 0) out_tok[row] = (int)sh.s_idx[sh.pick != 0xffffffffu ? sh.pick : sh.last_mass];
    if (work) {
        // the processed scores: the survivors keep theirs, everything else is gone
        for (int w = tid; w < 2048; w += S_THREADS) sh.left[w] = 0u;
        __syncthreads();
        if (mine && sh.s_alive[tid]) atomicOr(&sh.left[sh.s_idx[tid] >> 5], 1u << (sh.s_idx[tid] & 31));
        __syncthreads();
        const float lse = renorm ? best.v + logf(total) : 0.f;
        float* w = work + (long)row * V;
        for_each_score(score.l, V, [&](int i, float raw) {
            w[i] = ((sh.left[i >> 5] >> (i & 31)) & 1u) ? score.of(i, raw) - lse : -INFINITY;
        });
    }
    return true;
}

__global__ __launch_bounds__(S_THREADS) void sample_kernel(
    int* __restrict__ out_tok, float* __restrict__ work, const float* __restrict__ logits, int V, int do_sample,
    float temperature, int top_k, float top_p, float min_p, float typical_p, float epsilon_cutoff, float eta_cutoff,
    float penalty, const int* __restrict__ hist, const int* __restrict__ hist_off, const int* __restrict__ ban,
    const int* __restrict__ ban_off, const int* __restrict__ eos, int n_eos, const int* __restrict__ suppress,
    int remove_invalid, int renorm, uint64_t seed, const int* __restrict__ rng_seq,
    const int* __restrict__ rng_step, const float* __restrict__ uniforms, int want_scores,
    const int* __restrict__ bias_tok, const float* __restrict__ bias_val, const int* __restrict__ bias_off,
    const int* __restrict__ forced, int n_forced, int decay_on, float decay_m) {
    __shared__ SampleShared sh;
    float* const red = sh.red;
    int* const red_i = sh.red_i;
    uint32_t* const cnt = sh.cnt;
    unsigned long long* const mass = sh.mass;
    uint32_t& sh_bin = sh.bin;
    uint32_t& sh_remaining = sh.remaining;
    uint32_t& sh_all = sh.all;
    unsigned long long& sh_cum = sh.cum;
    const int n_holding = min(V, S_THREADS);  // threads that hold scores

    const int row = blockIdx.x, tid = threadIdx.x;
    float* w = work + (long)row * V;
    const float* l = logits + (long)row * V;

    const bool suppress_eos = suppress && suppress[row];
    const int bias_lo = bias_off ? bias_off[row] : 0, n_bias = bias_off ? bias_off[row + 1] - bias_lo : 0;
    ArgBest first_best = {-INFINITY, 0x7fffffff};
    unsigned long long first_finite = 0ull;
    float first_max = -INFINITY;  // the largest of the scores this thread saw in the first pass
    bool have_first = false;
    if (V <= 65536) {
        const Processed score{l, mark_seen(sh, row, V, penalty, hist, hist_off), mark_banned(sh, row, V, ban, ban_off), eos,
                              suppress_eos ? n_eos : 0, penalty,
                              do_sample ? temperature : 1.0f, remove_invalid, bias_tok + bias_lo, bias_val + bias_lo, n_bias,
                              forced, n_forced, n_eos, decay_on, decay_m};
        const bool later_warpers = typical_p < 1.0f || epsilon_cutoff > 0.0f || eta_cutoff > 0.0f;  // the long way has them
        if (do_sample && top_k > 0 && top_k < V && top_k <= n_holding && top_k <= S_SHORT && !later_warpers) {
            const float u = uniforms ? uniforms[row] : uniform_of(seed, (uint32_t)rng_seq[row], (uint32_t)rng_step[row]);
            if (sample_short(sh, out_tok, want_scores ? work : nullptr, score, row, V, top_k, top_p, min_p, renorm, u)) return;
            __syncthreads();
        }
        // every processor before the thresholds in one pass, which also finds the largest score (no threshold
        // ever removes it) and counts the scores that are not gone
        float mx = -INFINITY;
        int mi = 0x7fffffff;
        for_each_score(l, V, [&](int i, float raw) {
            const float x = score.of(i, raw);
            w[i] = x;
            if (x > mx) { mx = x; mi = i; }
            first_finite += x != -INFINITY ? 1ull : 0ull;
        });
        first_best = block_argmax(mx, mi, red, red_i);
        first_max = mx;
        have_first = true;
        __syncthreads();
    } else {
        for (int i = tid; i < V; i += S_THREADS) w[i] = l[i];
        __syncthreads();
        auto biased = [&](int tok) {  // the score with the row's bias for this token (a token is listed once)
            float v = l[tok];
            for (int t = 0; t < n_bias; ++t)
                if (bias_tok[bias_lo + t] == tok) v += bias_val[bias_lo + t];
            return v;
        };
        if (n_bias) {
            for (int t = tid; t < n_bias; t += S_THREADS) {
                const int tok = bias_tok[bias_lo + t];
                if (tok >= 0 && tok < V) w[tok] = biased(tok);
            }
            __syncthreads();
        }
        if (hist_off && penalty != 1.0f) {
            for (int t = hist_off[row] + tid; t < hist_off[row + 1]; t += S_THREADS) {
                const int tok = hist[t];
                if (tok >= 0 && tok < V) {
                    const float v = biased(tok);
                    w[tok] = v < 0.f ? v * penalty : v / penalty;
                }
            }
            __syncthreads();
        }
        if (ban_off) {
            for (int t = ban_off[row] + tid; t < ban_off[row + 1]; t += S_THREADS)
                if (ban[t] >= 0 && ban[t] < V) w[ban[t]] = -INFINITY;
            __syncthreads();
        }
        if (suppress_eos) {
            for (int e = tid; e < n_eos; e += S_THREADS)
                if (eos[e] >= 0 && eos[e] < V) w[eos[e]] = -INFINITY;
            __syncthreads();
        }
        if (n_forced) {
            for (int i = tid; i < V; i += S_THREADS) {
                bool is = false;
                for (int e = 0; e < n_forced; ++e) is = is || forced[e] == i;
                w[i] = is ? 0.f : -INFINITY;
            }
            __syncthreads();
            if (ban_off) {  // a banned token stays gone
                for (int t = ban_off[row] + tid; t < ban_off[row + 1]; t += S_THREADS)
                    if (ban[t] >= 0 && ban[t] < V) w[ban[t]] = -INFINITY;
                __syncthreads();
            }
        }
        if (remove_invalid) {
            for (int i = tid; i < V; i += S_THREADS) {
                float v = w[i];
                if (v != v) v = 0.f;
                else if (v == INFINITY) v = FLT_MAX;
                else if (v == -INFINITY) v = -FLT_MAX;
                w[i] = v;
            }
            __syncthreads();
        }
        if (decay_on) {
            if (tid == 0)
                for (int e = 0; e < n_eos; ++e) {
                    bool again = false;  // an id listed twice counts once
                    for (int o = 0; o < e; ++o) again = again || eos[o] == eos[e];
                    if (!again && eos[e] >= 0 && eos[e] < V) w[eos[e]] += fabsf(w[eos[e]]) * decay_m;
                }
            __syncthreads();
        }
        if (do_sample && temperature != 1.0f) {
            for (int i = tid; i < V; i += S_THREADS) w[i] = w[i] / temperature;
            __syncthreads();
        }
    }

    if (do_sample) {
        if (top_k > 0 && top_k < V) {
            uint32_t prefix = 0, maskbits = 0;
            bool found = false;
            if (top_k <= n_holding) {
                // the k-th largest of the threads' maxima bounds the k-th largest score from below: the scores
                // at or above it are few, and the k-th largest of those is the threshold
                float m = -INFINITY;
                for (int i = tid; i < V; i += S_THREADS) m = fmaxf(m, w[i]);
                sh.tkey[tid] = tid < V ? order_key(m) : 0u;
                const uint32_t bound = list_kth_largest(sh, sh.tkey, S_THREADS, (uint32_t)top_k);
                if (tid == 0) sh.n_cand = 0u;
                __syncthreads();
                for (int i = tid; i < V; i += S_THREADS) {
                    const uint32_t k = order_key(w[i]);
                    if (k >= bound) {
                        const uint32_t at = atomicAdd(&sh.n_cand, 1u);
                        if (at < S_CAP) sh.cand_key[at] = k;
                    }
                }
                __syncthreads();
                if (sh.n_cand <= S_CAP) {
                    prefix = list_kth_largest(sh, sh.cand_key, (int)sh.n_cand, (uint32_t)top_k);
                    found = true;
                }
            }
            if (!found) {
                // key of the k-th largest score over the whole row, one byte at a time from the top
                __syncthreads();
                if (tid == 0) sh_remaining = (uint32_t)top_k;
                for (int shift = 24; shift >= 0; shift -= 8) {
                    if (tid < 256) cnt[tid] = 0;
                    __syncthreads();
                    for (int i = tid; i < V; i += S_THREADS) {
                        const uint32_t k = order_key(w[i]);
                        if ((k & maskbits) == prefix) atomicAdd(&cnt[(k >> shift) & 255u], 1u);
                    }
                    __syncthreads();
                    if (tid == 0) {
                        uint32_t rem = sh_remaining;
                        int b = 255;
                        while (b > 0 && cnt[b] < rem) { rem -= cnt[b]; --b; }
                        sh_bin = (uint32_t)b;
                        sh_remaining = rem;
                    }
                    __syncthreads();
                    prefix |= sh_bin << shift;
                    maskbits |= 255u << shift;
                }
            }
            for (int i = tid; i < V; i += S_THREADS)
                if (order_key(w[i]) < prefix) w[i] = -INFINITY;
            __syncthreads();
        }
        if (top_p < 1.0f) {
            float mx = -INFINITY;
            int mi = 0x7fffffff;
            unsigned long long finite = first_finite;
            const bool counted = have_first && !(top_k > 0 && top_k < V);  // nothing has gone since the first pass
            if (!counted) {
                finite = 0ull;
                for (int i = tid; i < V; i += S_THREADS) {
                    const float x = w[i];
                    if (x > mx) { mx = x; mi = i; }
                    finite += x != -INFINITY ? 1ull : 0ull;
                }
            }
            const ArgBest best = have_first ? first_best : block_argmax(mx, mi, red, red_i);
            float s = 0.f;
            for (int i = tid; i < V; i += S_THREADS) s += expf(w[i] - best.v);
            const float Z = block_sum(s, red);
            const unsigned long long T = (unsigned long long)((double)(1.0f - top_p) * (double)MASS_ONE);
            // The candidates: every score that is left if those are few (after top-k), else the scores from the
            // 512th largest thread maximum up, if the mass of all the others fits into 1 - p.
            const unsigned long long n_finite = block_sum_u64(finite, sh.red_q);
            uint32_t from = order_key(-INFINITY) + 1u;
            if (n_finite > S_CAP) {
                // (a thread that saw no score has the key of minus infinity, which is below every candidate)
                sh.tkey[tid] = order_key(counted ? first_max : mx);
                from = list_kth_largest(sh, sh.tkey, S_THREADS, (uint32_t)min(512, n_holding));
            }
            __syncthreads();
            if (tid == 0) sh.n_cand = 0u;
            __syncthreads();
            unsigned long long others = 0ull;
            for (int i = tid; i < V; i += S_THREADS) {
                const uint32_t k = order_key(w[i]);
                if (k >= from) {
                    const uint32_t at = atomicAdd(&sh.n_cand, 1u);
                    if (at < S_CAP) {
                        sh.cand_key[at] = k;
                        sh.cand_q[at] = (unsigned long long)(expf(w[i] - best.v) / Z * MASS_ONE + 0.5f);
                    }
                } else if (n_finite > S_CAP) {
                    others += (unsigned long long)(expf(w[i] - best.v) / Z * MASS_ONE + 0.5f);
                }
            }
            const unsigned long long low = block_sum_u64(others, sh.red_q);
            uint32_t prefix = 0, maskbits = 0;
            if (sh.n_cand <= S_CAP && low <= T) {
                unsigned long long below = 0ull;
                const bool cut = list_mass_cut(sh, (int)sh.n_cand, low, T, prefix, below);
                __syncthreads();
                if (tid == 0) { sh_all = cut ? 0u : 1u; sh_cum = below; }
                __syncthreads();
            } else {
                // the cut by mass over the whole row, one byte of the key at a time
                __syncthreads();
                if (tid == 0) { sh_cum = 0ull; sh_all = 0u; }
                for (int shift = 24; shift >= 0; shift -= 8) {
                    if (tid < 256) mass[tid] = 0ull;
                    __syncthreads();
                    for (int i = tid; i < V; i += S_THREADS) {
                        const uint32_t k = order_key(w[i]);
                        if ((k & maskbits) == prefix) {
                            const unsigned long long q = (unsigned long long)(expf(w[i] - best.v) / Z * MASS_ONE + 0.5f);
                            if (q) atomicAdd(&mass[(k >> shift) & 255u], q);
                        }
                    }
                    __syncthreads();
                    if (tid == 0) {
                        unsigned long long cum = sh_cum;
                        int b = 0;
                        while (b < 256 && cum + mass[b] <= T) { cum += mass[b]; ++b; }
                        if (b == 256) { sh_all = 1u; b = 255; }
                        sh_bin = (uint32_t)b;
                        sh_cum = cum;
                    }
                    __syncthreads();
                    if (sh_all) break;
                    prefix |= sh_bin << shift;
                    maskbits |= 255u << shift;
                }
            }
            // prefix: the lowest key that stays.  If everything could go, the largest score stays.
            const uint32_t keep_from = sh_all ? order_key(best.v) : prefix;
            for (int i = tid; i < V; i += S_THREADS)
                if (order_key(w[i]) < keep_from) w[i] = -INFINITY;
            __syncthreads();
            if (!sh_all) {
                // equal scores at the cut: in index order the first of them go while they fit, never the last one
                // (one token at least stays).  Tiles of consecutive tokens, the tied ones numbered by a scan.
                const float vcut = key_value(prefix);
                const unsigned long long q = (unsigned long long)(expf(vcut - best.v) / Z * MASS_ONE + 0.5f);
                const unsigned long long r = q ? (T - sh_cum) / q : 0ull;
                if (r > 0) {
                    unsigned long long mine = 0ull;
                    for (int i = tid; i < V; i += S_THREADS) mine += order_key(w[i]) == prefix ? 1ull : 0ull;
                    const unsigned long long ties = block_sum_u64(mine, sh.red_q);
                    unsigned long long before = 0ull;
                    for (int i0 = 0; i0 < V && before < r; i0 += S_THREADS) {
                        const int i = i0 + tid;
                        const bool tie = i < V && order_key(w[i]) == prefix;
                        const unsigned long long upto = block_scan_u64(tie ? 1ull : 0ull, sh.red_q);
                        const unsigned long long place = before + upto - 1;  // of a tied score, from 0
                        if (tie && place < r && place != ties - 1) w[i] = -INFINITY;
                        __syncthreads();
                        if (tid == S_THREADS - 1) sh_cum = upto;
                        __syncthreads();
                        before += sh_cum;
                    }
                }
            }
            __syncthreads();
        }
        if (min_p > 0.0f) {
            float mx = -INFINITY;
            for (int i = tid; i < V; i += S_THREADS) mx = fmaxf(mx, w[i]);
            mx = block_max(mx, red);
            float s = 0.f;
            for (int i = tid; i < V; i += S_THREADS) s += expf(w[i] - mx);
            const float Z = block_sum(s, red);
            const float thr = min_p * (1.0f / Z);
            for (int i = tid; i < V; i += S_THREADS)
                if (w[i] != mx && expf(w[i] - mx) / Z < thr) w[i] = -INFINITY;
            __syncthreads();
        }
        if (typical_p < 1.0f) {
            // Locally typical sampling: the scores whose information content -log p lies nearest to the entropy
            // stay, as many as it takes for their mass to reach typical_p.  The key of a score is its distance
            // from the entropy (the smaller the better); the cut by mass goes over the keys one byte at a time,
            // and equal distances at the cut all stay.  The most probable score is not safe here.
            float mx = -INFINITY;
            for (int i = tid; i < V; i += S_THREADS) mx = fmaxf(mx, w[i]);
            mx = block_max(mx, red);
            float s = 0.f;
            for (int i = tid; i < V; i += S_THREADS) s += expf(w[i] - mx);
            const float Z = block_sum(s, red);
            const float logZ = logf(Z);
            float h = 0.f;
            for (int i = tid; i < V; i += S_THREADS)
                if (w[i] != -INFINITY) h -= (w[i] - mx - logZ) * expf(w[i] - mx - logZ);
            const float ent = block_sum(h, red);
            auto typical_key = [&](float x) { return order_key(-fabsf(-(x - mx - logZ) - ent)); };
            uint32_t kbest = 0u;
            for (int i = tid; i < V; i += S_THREADS)
                if (w[i] != -INFINITY) kbest = max(kbest, typical_key(w[i]));
            __syncthreads();
            if (tid == 0) { sh.pick = 0u; sh_cum = 0ull; sh_all = 0u; }
            __syncthreads();
            atomicMax(&sh.pick, kbest);
            const unsigned long long T = (unsigned long long)((double)(1.0f - typical_p) * (double)MASS_ONE);
            uint32_t prefix = 0, maskbits = 0;
            for (int shift = 24; shift >= 0; shift -= 8) {
                if (tid < 256) mass[tid] = 0ull;
                __syncthreads();
                for (int i = tid; i < V; i += S_THREADS) {
                    if (w[i] == -INFINITY) continue;
                    const uint32_t k = typical_key(w[i]);
                    if ((k & maskbits) == prefix) {
                        const unsigned long long q = (unsigned long long)(expf(w[i] - mx) / Z * MASS_ONE + 0.5f);
                        if (q) atomicAdd(&mass[(k >> shift) & 255u], q);
                    }
                }
                __syncthreads();
                if (tid == 0) {
                    unsigned long long cum = sh_cum;
                    int b = 0;
                    while (b < 256 && cum + mass[b] <= T) { cum += mass[b]; ++b; }
                    if (b == 256) { sh_all = 1u; b = 255; }
                    sh_bin = (uint32_t)b;
                    sh_cum = cum;
                }
                __syncthreads();
                if (sh_all) break;
                prefix |= sh_bin << shift;
                maskbits |= 255u << shift;
            }
            // prefix: the lowest key that stays.  If everything could go, the most typical score stays.
            const uint32_t keep_from = sh_all ? sh.pick : prefix;
            for (int i = tid; i < V; i += S_THREADS)
                if (w[i] != -INFINITY && typical_key(w[i]) < keep_from) w[i] = -INFINITY;
            have_first = false;
            __syncthreads();
        }
        if (epsilon_cutoff > 0.0f || eta_cutoff > 0.0f) {
            // probabilities below a bound go, the largest score always stays: the bound is epsilon itself, then
            // min(eta, sqrt(eta) * exp(-entropy)) with the entropy of what epsilon left
            for (int pass = 0; pass < 2; ++pass) {
                const float eps = pass == 0 ? epsilon_cutoff : eta_cutoff;
                if (!(eps > 0.0f)) continue;
                float mx = -INFINITY;
                for (int i = tid; i < V; i += S_THREADS) mx = fmaxf(mx, w[i]);
                mx = block_max(mx, red);
                float s = 0.f;
                for (int i = tid; i < V; i += S_THREADS) s += expf(w[i] - mx);
                const float Z = block_sum(s, red);
                float bound = eps;
                if (pass == 1) {
                    const float logZ = logf(Z);
                    float h = 0.f;
                    for (int i = tid; i < V; i += S_THREADS)
                        if (w[i] != -INFINITY) h -= (w[i] - mx - logZ) * (expf(w[i] - mx) / Z);
                    const float ent = block_sum(h, red);
                    bound = fminf(eps, sqrtf(eps) * expf(-ent));
                }
                for (int i = tid; i < V; i += S_THREADS)
                    if (w[i] != mx && expf(w[i] - mx) / Z < bound) w[i] = -INFINITY;
                __syncthreads();
            }
        }
    }

    // choose
    float mx = -INFINITY;
    int mi = 0x7fffffff;
    if (!have_first)
        for (int i = tid; i < V; i += S_THREADS)
            if (w[i] > mx) { mx = w[i]; mi = i; }
    const ArgBest best = have_first ? first_best : block_argmax(mx, mi, red, red_i);
    int chosen = best.i;
    float Z = 0.f;
    if (do_sample || renorm) {
        // A wave per sixteenth of the row (a multiple of 64 scores): its lanes add every 64th exponential, the
        // wave adds its lanes, and every thread adds the sixteen sums in order.
        const int lane = tid & 63, wave = tid >> 6, n_waves = S_THREADS / 64;
        const int span = ((V + n_waves - 1) / n_waves + 63) & ~63;
        const int lo = min(V, wave * span), hi = min(V, lo + span);
        float s = 0.f;
        if ((((uintptr_t)(w + lo)) & 15) == 0) {
            // sixteen bytes a load, four loads in flight per lane
            const float4* w4 = reinterpret_cast<const float4*>(w + lo);
            const int quads = (hi - lo) >> 2;
            auto add4 = [&](const float4& a) {
                s += expf(a.x - best.v); s += expf(a.y - best.v); s += expf(a.z - best.v); s += expf(a.w - best.v);
            };
            int q = lane;
            for (; q + 192 < quads; q += 256) {
                const float4 a = w4[q], b = w4[q + 64], c = w4[q + 128], d = w4[q + 192];
                add4(a); add4(b); add4(c); add4(d);
            }
            for (; q < quads; q += 64) add4(w4[q]);
            for (int i = lo + quads * 4 + lane; i < hi; i += 64) s += expf(w[i] - best.v);
        } else {
            for (int i = lo + lane; i < hi; i += 64) s += expf(w[i] - best.v);
        }
        s = wave_sum(s);
        __syncthreads();
        if (lane == 0) sh.seg[wave] = s;
        __syncthreads();
        float total = 0.f;
        for (int k = 0; k < n_waves; ++k) total += sh.seg[k];
        Z = total;
        if (do_sample) {
            const float u = uniforms ? uniforms[row] : uniform_of(seed, (uint32_t)rng_seq[row], (uint32_t)rng_step[row]);
            const float target = u * total;
            // the sixteenth in which the cumulative sum passes the target, and what is left of the target there;
            // if rounding leaves none, the last one that has mass, to its last token with mass
            float acc = 0.f, left = INFINITY;
            int pick = -1, last_nonzero = 0;
            for (int k = 0; k < n_waves; ++k) {
                if (sh.seg[k] > 0.f) last_nonzero = k;
                if (pick < 0 && acc + sh.seg[k] > target) { pick = k; left = target - acc; }
                if (pick < 0) acc += sh.seg[k];
            }
            if (pick < 0) pick = last_nonzero;
            if (wave == pick) {
                float before = 0.f;
                int tok = -1, last = lo;
                for (int i0 = lo; i0 < hi && tok < 0; i0 += 256) {
                    float x[4];  // four times 64 scores are loaded before the first of them is used
#pragma unroll
                    for (int k = 0; k < 4; ++k) x[k] = i0 + 64 * k + lane < hi ? w[i0 + 64 * k + lane] : -INFINITY;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (tok >= 0) break;
                        const float e = expf(x[k] - best.v);
                        float incl = e;
#pragma unroll
                        for (int o = 1; o < 64; o <<= 1) {
                            const float up = __shfl_up(incl, o, 64);
                            if (lane >= o) incl += up;
                        }
                        const unsigned long long has_mass = __ballot(e > 0.f);
                        const unsigned long long passed = __ballot(before + incl > left);
                        if (has_mass) last = i0 + 64 * k + 63 - __clzll(has_mass);
                        if (passed) tok = i0 + 64 * k + __ffsll((long long)passed) - 1;
                        before += __shfl(incl, 63, 64);
                    }
                }
                if (lane == 0) out_tok[row] = tok >= 0 ? tok : last;
            }
        }
    }
    if (!do_sample && tid == 0) out_tok[row] = chosen < V ? chosen : 0;  // every score -inf: token 0, as an argmax gives
    if (renorm) {
        __syncthreads();
        const float lse = best.v + logf(Z);
        for (int i = tid; i < V; i += S_THREADS) w[i] = w[i] - lse;
    }
}

extern "C" int pta_sample(int* out_tok, float* work, const float* logits, int R, int V, int do_sample,
                          float temperature, int top_k, float top_p, float min_p, float typical_p,
                          float epsilon_cutoff, float eta_cutoff, float penalty, const int* hist,
                          const int* hist_off, const int* ban, const int* ban_off, const int* eos, int n_eos,
                          const int* suppress, int remove_invalid,
                          int renorm, uint64_t seed, const int* rng_seq, const int* rng_step, const float* uniforms,
                          int want_scores, const int* bias_tok, const float* bias_val, const int* bias_off,
                          const int* forced, int n_forced, int decay_on, float decay_m, void* stream) {
    PTA_REQUIRE(R > 0 && V > 0, "sample: rows=%d vocab=%d must be positive", R, V);
    PTA_REQUIRE(out_tok && work && logits, "sample: null pointer");
    PTA_REQUIRE(!do_sample || temperature > 0.f, "sample: temperature must be > 0, got %g", (double)temperature);
    PTA_REQUIRE(top_p >= 0.f && top_p <= 1.f, "sample: top_p must be in [0, 1], got %g", (double)top_p);
    PTA_REQUIRE(min_p >= 0.f && min_p <= 1.f, "sample: min_p must be in [0, 1], got %g", (double)min_p);
    PTA_REQUIRE(typical_p > 0.f && typical_p <= 1.f, "sample: typical_p must be in (0, 1] (1: off), got %g", (double)typical_p);
    PTA_REQUIRE(epsilon_cutoff >= 0.f && epsilon_cutoff < 1.f, "sample: epsilon_cutoff must be in [0, 1) (0: off), got %g",
                (double)epsilon_cutoff);
    PTA_REQUIRE(eta_cutoff >= 0.f && eta_cutoff < 1.f, "sample: eta_cutoff must be in [0, 1) (0: off), got %g", (double)eta_cutoff);
    PTA_REQUIRE(penalty > 0.f, "sample: repetition penalty must be > 0, got %g", (double)penalty);
    PTA_REQUIRE(!do_sample || uniforms || (rng_seq && rng_step), "sample: sampling needs uniforms or rng counters");
    PTA_REQUIRE(n_eos == 0 || eos, "sample: eos ids missing");
    PTA_REQUIRE(!ban_off || ban, "sample: banned ids missing");
    PTA_REQUIRE(!bias_off || (bias_tok && bias_val), "sample: biased ids or their values missing");
    PTA_REQUIRE(n_forced == 0 || forced, "sample: forced ids missing");
    PTA_REQUIRE(!decay_on || n_eos > 0, "sample: a bonus on the EOS tokens needs their ids");
    hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(S_THREADS), 0, (hipStream_t)stream, out_tok, work, logits, V,
                       do_sample, temperature, top_k, top_p, min_p, typical_p, epsilon_cutoff, eta_cutoff, penalty, hist,
                       hist_off, ban, ban_off, eos, n_eos, suppress, remove_invalid, renorm, seed, rng_seq, rng_step, uniforms, want_scores,
                       bias_tok, bias_val, bias_off, forced, n_forced, decay_on, decay_m);
    return pta_check_launch("sample");
}

// the same generator on the host, for tests and for callers that want the number itself
extern "C" float pta_philox_uniform(uint64_t seed, uint32_t seq, uint32_t step) {
    uint32_t c[4] = {seq, step, 0u, 0u};
    uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return (float)(c[0] >> 8) * (1.0f / 16777216.0f);
}
