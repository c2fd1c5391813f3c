// Token sampling on the GPU, one block per row of logits.
//
// Algorithm of the reference's sampler (crates/mach-model/src/sampling.rs:113-402 and its
// CPU mirror 1169-1274): one SplitMix64 draw per row per call, also when greedy
// (finalizer of the state, then state += golden ratio; u = top 24 bits / 2^24);
// temperature <= 0 -> smallest index among the maxima; else p = exp((x - max) / T),
// top-k as a threshold on the raw logit found by 30 bisection steps between the row's
// minimum and maximum, top-p as a probability cut found by 30 bisection steps so that the
// kept mass is >= p * total, then target = u * allowed mass and a walk in index order to
// the first token whose cumulative mass exceeds the target.
//
// The walk here is in true index order: thread i owns the contiguous segment i of the row,
// the segment masses are scanned in order, and the owner of the segment that holds the
// target walks it.
#include "common.cuh"

namespace ms {

constexpr int ST = 1024;

__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

struct SampleArgs {
    const float* logits;  // [W, vocab]
    const float* temperature;
    const int* top_k;
    const float* top_p;
    unsigned long long* state;  // [W], advanced by one step
    int* out_token;
    float* out_logprob;
    int vocab;
    // per-row partial maxima of ARGMAX_CHUNKS chunks of the row, or null: a greedy row scans itself
    const float* part_val;
    const int* part_idx;
    int* also_token;  // [W] or null: a second place for the tokens (the next step's input, on the device)
};

constexpr int ARGMAX_CHUNKS = 64;

// Stage one of greedy sampling: the row is cut into ARGMAX_CHUNKS contiguous chunks, one block each;
// a block writes the maximum of its chunk and the smallest index that holds it.
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits, int vocab,
                                                             float* __restrict__ part_val, int* __restrict__ part_idx) {
    arguments_now(logits, vocab, part_val, part_idx);
    __shared__ float s_v[4];
    __shared__ int s_i[4];
    const int r = blockIdx.x, ch = blockIdx.y, tid = threadIdx.x;
    const float* row = logits + (size_t)r * vocab;
    // chunks of a multiple of four entries: where the rows are 16-byte aligned (a vocabulary that is a multiple of four),
    // a thread reads four entries at a time (512 rows of 151,936: 131 -> 90 us; the chunks' borders do not change
    // the result, which is the row's maximum at its smallest index)
    const int len = ceil_div(ceil_div(vocab, ARGMAX_CHUNKS), 4) * 4, i0 = min(vocab, ch * len), i1 = min(vocab, i0 + len);
    float best = -INFINITY;
    int bi = 0x7fffffff;
    if (vocab % 4 == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
        for (int i = i0 + 4 * tid; i < i1; i += 4 * 256) {  // i1 - i0 is a multiple of four here
            const float4 x = *reinterpret_cast<const float4*>(row + i);
            const float xs[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (bi == 0x7fffffff || xs[u] > best) { best = xs[u]; bi = i + u; }
        }
    } else {
        for (int i = i0 + tid; i < i1; i += 256) {
            const float x = row[i];
            if (bi == 0x7fffffff || x > best) { best = x; bi = i; }
        }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, WAVE);
        const int oi = __shfl_xor(bi, o, WAVE);
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
    }
    if ((tid & 63) == 0) { s_v[tid >> 6] = best; s_i[tid >> 6] = bi; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 4; ++w)
            if (s_i[w] != 0x7fffffff && (bi == 0x7fffffff || s_v[w] > best || (s_v[w] == best && s_i[w] < bi))) { best = s_v[w]; bi = s_i[w]; }
        part_val[r * ARGMAX_CHUNKS + ch] = best;
        part_idx[r * ARGMAX_CHUNKS + ch] = bi;
    }
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = scratch[0];
    for (int i = 1; i < ST / WAVE; ++i) t = fmaxf(t, scratch[i]);
    return t;
}

__global__ __launch_bounds__(ST) void sample_kernel(SampleArgs a) {
    arguments_now(a.logits, a.temperature, a.top_k, a.top_p, a.state, a.out_token, a.out_logprob, a.vocab, a.part_val, a.part_idx,
                  a.also_token);
    __shared__ float scratch[ST / WAVE];
    __shared__ float seg[ST], seg_pref[ST];
    __shared__ float s_u;
    __shared__ int s_idx[ST / WAVE];
    __shared__ float s_val[ST / WAVE];
    __shared__ int s_found;
    const int r = blockIdx.x, tid = threadIdx.x, V = a.vocab;
    const float* row = a.logits + (size_t)r * V;
    const float T = a.temperature[r];

    if (tid == 0) {
        unsigned long long st = a.state[r];
        const unsigned long long z = mix64(st);
        a.state[r] = st + 0x9E3779B97F4A7C15ULL;
        s_u = (float)(z >> 40) * (1.0f / 16777216.0f);
        s_found = -1;
    }
    __syncthreads();

    const int seg_len = ceil_div(V, ST);
    const int i0 = min(V, tid * seg_len), i1 = min(V, i0 + seg_len);

    if (T <= 0.0f && a.part_val) {
        // stage two: the chunks' maxima, smallest index first among equals
        if (tid < WAVE) {
            float best = tid < ARGMAX_CHUNKS ? a.part_val[r * ARGMAX_CHUNKS + tid] : -INFINITY;
            int bi = tid < ARGMAX_CHUNKS ? a.part_idx[r * ARGMAX_CHUNKS + tid] : 0x7fffffff;
            for (int o = 32; o > 0; o >>= 1) {
                const float ov = __shfl_xor(best, o, WAVE);
                const int oi = __shfl_xor(bi, o, WAVE);
                if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
            }
            if (tid == 0) {
                a.out_token[r] = bi;
                if (a.also_token) a.also_token[r] = bi;
                a.out_logprob[r] = 0.0f;
            }
        }
        return;
    }
    if (T <= 0.0f) {
        // smallest index among the maxima.  A thread walks its strided indices in ascending
        // order and keeps the first maximum; ties between threads go to the smaller index.
        float best = -INFINITY;
        int bi = 0x7fffffff;
        for (int i = tid; i < V; i += ST) {
            const float x = row[i];
            if (bi == 0x7fffffff || x > best) { best = x; bi = i; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, WAVE);
            const int oi = __shfl_xor(bi, o, WAVE);
            if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
        }
        if ((tid & 63) == 0) { s_val[tid >> 6] = best; s_idx[tid >> 6] = bi; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < ST / WAVE; ++w) {
                const int oi = s_idx[w];
                if (oi != 0x7fffffff && (bi == 0x7fffffff || s_val[w] > best || (s_val[w] == best && oi < bi))) {
                    best = s_val[w];
                    bi = oi;
                }
            }
            a.out_token[r] = bi;
            if (a.also_token) a.also_token[r] = bi;
            a.out_logprob[r] = 0.0f;
        }
        return;
    }

    float mx = -INFINITY, mn = INFINITY;
    for (int i = tid; i < V; i += ST) {
        const float x = row[i];
        mx = fmaxf(mx, x);
        mn = fminf(mn, x);
    }
    const float maxv = block_max(mx, scratch);
    const float minv = -block_max(-mn, scratch);
    const float inv_t = 1.0f / T;
    const int k = a.top_k[r];
    const int k_eff = (k > 0 && k < V) ? k : 0;

    float topk_thr = -INFINITY;
    if (k_eff > 0) {
        float lo = minv, hi = maxv;
        for (int it = 0; it < 30; ++it) {
            const float mid = (lo + hi) * 0.5f;
            float cnt = 0.f;
            for (int i = tid; i < V; i += ST) cnt += row[i] > mid ? 1.f : 0.f;
            cnt = block_sum<ST>(cnt, scratch);
            if (cnt >= (float)k_eff) lo = mid; else hi = mid;
        }
        topk_thr = hi;
    }

    // total mass, summed segment by segment in index order
    float part = 0.f;
    for (int i = i0; i < i1; ++i) part += expf((row[i] - maxv) * inv_t);
    const float s_tot = block_sum<ST>(part, scratch);

    const float top_p = a.top_p[r];
    const bool use_topp = top_p < 1.0f;
    float cut = 0.f;
    if (use_topp) {
        float lo = 0.f, hi = 1.f;
        for (int it = 0; it < 30; ++it) {
            const float mid = (lo + hi) * 0.5f;
            float acc = 0.f;
            for (int i = i0; i < i1; ++i) {
                const float pr = expf((row[i] - maxv) * inv_t);
                if (pr >= mid) acc += pr;
            }
            acc = block_sum<ST>(acc, scratch);
            if (acc >= top_p * s_tot) lo = mid; else hi = mid;
        }
        cut = lo;
    }

    auto allowed = [&](float x, float pr) { return (k_eff == 0 || x >= topk_thr) && (!use_topp || pr >= cut); };

    float mass = 0.f;
    for (int i = i0; i < i1; ++i) {
        const float pr = expf((row[i] - maxv) * inv_t);
        if (allowed(row[i], pr)) mass += pr;
    }
    seg[tid] = mass;
    __syncthreads();
    if (tid == 0) {
        float acc = 0.f;
        for (int j = 0; j < ST; ++j) { seg_pref[j] = acc; acc += seg[j]; }
        scratch[0] = acc;
    }
    __syncthreads();
    const float tot = scratch[0];
    const float target = s_u * tot;
    if (seg_pref[tid] <= target && target < seg_pref[tid] + seg[tid]) {
        float acc = seg_pref[tid];
        for (int i = i0; i < i1; ++i) {
            const float pr = expf((row[i] - maxv) * inv_t);
            if (allowed(row[i], pr)) {
                acc += pr;
                if (acc > target) { s_found = i; break; }  // segments are disjoint: one owner
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        int found = s_found;
        if (found < 0) {
            // rounding at the top of the mass: no segment's walk went past the target.  As the reference
            // (crates/mach-model/src/sampling.rs:385-400): the first allowed token, else the row's maximum
            for (int i = 0; i < V && found < 0; ++i) {
                const float pr = expf((row[i] - maxv) * inv_t);
                if (allowed(row[i], pr)) found = i;
            }
            if (found < 0) {
                found = 0;
                for (int i = 1; i < V; ++i)
                    if (row[i] > row[found]) found = i;
            }
        }
        a.out_token[r] = found;
        if (a.also_token) a.also_token[r] = found;
        a.out_logprob[r] = (row[found] - maxv) * inv_t - logf(tot);
    }
}

// logits[row_of[e], token[e]] += delta[e]: penalties and biases, merged per (row, token) on the host
__global__ void logit_edit_kernel(float* logits, int vocab, const int* row_of, const int* token, const float* delta,
                                  int n) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n && token[e] >= 0 && token[e] < vocab) logits[(size_t)row_of[e] * vocab + token[e]] += delta[e];
}

constexpr int TOPLP_MAX = 20;

// The k most probable tokens of every row and their log-probabilities under the row's temperature
// (`inv_t`; the host passes 1 for temperature <= 0), ties to the smaller token id:
// logprob = (x - max) * inv_t - log(sum exp((x - max) * inv_t)).
// Role in the reference: topk_batched (crates/mach-model/src/sampling.rs:411-539).  k rounds, each
// a search for the best token after the previous pick in the order (logit descending, id ascending).
__global__ __launch_bounds__(ST) void top_logprobs_kernel(const float* __restrict__ logits, const float* __restrict__ inv_t,
                                                          int* __restrict__ out_tok, float* __restrict__ out_lp, int vocab,
                                                          int k) {
    __shared__ float scratch[ST / WAVE];
    __shared__ float s_val[ST / WAVE];
    __shared__ int s_idx[ST / WAVE];
    __shared__ float s_last_v;
    __shared__ int s_last_i;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * vocab;
    const float it = inv_t[r];
    float mx = -INFINITY;
    for (int i = tid; i < vocab; i += ST) mx = fmaxf(mx, row[i]);
    const float maxv = block_max(mx, scratch);
    const int seg_len = ceil_div(vocab, ST);
    const int i0 = min(vocab, tid * seg_len), i1 = min(vocab, i0 + seg_len);
    float part = 0.f;
    for (int i = i0; i < i1; ++i) part += expf((row[i] - maxv) * it);
    const float logz = logf(block_sum<ST>(part, scratch));
    float last_v = INFINITY;
    int last_i = -1;
    for (int round = 0; round < k; ++round) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
        for (int i = tid; i < vocab; i += ST) {
            const float x = row[i];
            const bool after = x < last_v || (x == last_v && i > last_i);
            if (after && (bi == 0x7fffffff || x > best)) { best = x; bi = i; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, WAVE);
            const int oi = __shfl_xor(bi, o, WAVE);
            if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
        }
        __syncthreads();
        if ((tid & 63) == 0) { s_val[tid >> 6] = best; s_idx[tid >> 6] = bi; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < ST / WAVE; ++w)
                if (s_idx[w] != 0x7fffffff && (bi == 0x7fffffff || s_val[w] > best || (s_val[w] == best && s_idx[w] < bi))) {
                    best = s_val[w];
                    bi = s_idx[w];
                }
            const bool found = bi != 0x7fffffff;
            out_tok[(size_t)r * TOPLP_MAX + round] = found ? bi : -1;
            out_lp[(size_t)r * TOPLP_MAX + round] = found ? (best - maxv) * it - logz : -INFINITY;
            s_last_v = best;
            s_last_i = found ? bi : 0x7fffffff;
        }
        __syncthreads();
        last_v = s_last_v;
        last_i = s_last_i;
    }
}

}  // namespace ms

using namespace ms;

extern "C" int ms_top_logprobs_max() { return TOPLP_MAX; }

// out_tok / out_lp: [rows, ms_top_logprobs_max()], the first k entries of a row are written.
extern "C" int ms_top_logprobs(const float* logits, const float* inv_t, int* out_tok, float* out_lp, int rows, int vocab,
                               int k, hipStream_t stream) {
    MS_REQUIRE(rows > 0 && vocab > 0, "top_logprobs: empty problem rows=%d vocab=%d", rows, vocab);
    MS_REQUIRE(k >= 1 && k <= TOPLP_MAX, "top_logprobs: k=%d must be in 1..%d", k, TOPLP_MAX);
    hipLaunchKernelGGL(top_logprobs_kernel, dim3(rows), dim3(ST), 0, stream, logits, inv_t, out_tok, out_lp, vocab, k);
    return check_launch("top_logprobs");
}

// part_val / part_idx: float / int workspaces [rows, ms_sample_chunks()] for the two-stage greedy
// search, or null (every row scans itself in one block).
extern "C" int ms_sample_chunks() { return ARGMAX_CHUNKS; }

extern "C" int ms_sample(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                         unsigned long long* state, int* out_token, float* out_logprob, float* part_val, int* part_idx,
                         int* also_token, int rows, int vocab, hipStream_t stream) {
    MS_REQUIRE(rows > 0 && vocab > 0, "sample: empty problem rows=%d vocab=%d", rows, vocab);
    static_assert(ARGMAX_CHUNKS <= WAVE, "stage two is one wave");
    if (part_val && part_idx) {
        hipLaunchKernelGGL(argmax_partial_kernel, dim3(rows, ARGMAX_CHUNKS), dim3(256), 0, stream, logits, vocab, part_val,
                           part_idx);
        if (int rc = check_launch("argmax_partial")) return rc;
    } else {
        part_val = nullptr;
        part_idx = nullptr;
    }
    SampleArgs a{logits, temperature, top_k, top_p, state, out_token, out_logprob, vocab, part_val, part_idx, also_token};
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(ST), 0, stream, a);
    return check_launch("sample");
}

extern "C" int ms_logit_edit(float* logits, int vocab, const int* row_of, const int* token, const float* delta, int n,
                             hipStream_t stream) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(logit_edit_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, stream, logits, vocab, row_of, token,
                       delta, n);
    return check_launch("logit_edit");
}
