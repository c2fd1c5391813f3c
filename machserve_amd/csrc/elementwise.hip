// Memory-bound kernels around the matrix products: embedding gather, RMS norm (optionally
// of gathered rows), and rotation of q and k fused with the write of k and v into pages.
//
// Role in the reference: embed_batched, rms_norm, rope_batched, kv_store_paged
// (crates/mach-model/src/kernels.rs:578-585, 63-80, 589-660, 1148-1168).
// Norm statistics, rotation angles and the rotation itself are 32-bit in both builds.
#include "common.cuh"

namespace ms {

// x[t, :] = float(table[tokens[t], :]) * scale
__global__ __launch_bounds__(256) void embed_kernel(const int* __restrict__ tokens, const elem_t* __restrict__ table,
                                                    float* __restrict__ x, int d, float scale) {
    arguments_now(tokens, table, x, d, scale);
    const int t = blockIdx.x;
    const elem_t* src = table + (size_t)tokens[t] * d;
    float* dst = x + (size_t)t * d;
    for (int c = threadIdx.x; c < d; c += 256) dst[c] = to_f32(src[c]) * scale;
}

// tokens[rows[i]] = sampled[src[i]] for the i with 0 <= rows[i] < n_tokens and 0 <= src[i] < n_sampled: the input of
// those rows of a step that the step before it sampled, taken on the device (the host has not seen them yet)
__global__ __launch_bounds__(256) void feed_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ sampled,
                                                          const int* __restrict__ rows, const int* __restrict__ src, int n,
                                                          int n_tokens, int n_sampled) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int r = rows[i], s = src[i];
    if (r >= 0 && r < n_tokens && s >= 0 && s < n_sampled) tokens[r] = sampled[s];
}

// r = rows ? rows[i] : i;  v = x[r, :] + sum_p partials[p, r, :] (in order);  if partials are given
// and no rows are gathered, x[r, :] = v is written back (the residual stream takes the pending
// sums);  out[i, :] = v * rsqrt(mean(v^2) + eps) * w.
template <typename OutT>
__global__ __launch_bounds__(256) void rmsnorm_kernel(float* __restrict__ x, const float* __restrict__ partials,
                                                      int n_partials, size_t partial_stride,
                                                      const int* __restrict__ rows, const float* __restrict__ w,
                                                      OutT* __restrict__ out, int d, float eps) {
    __shared__ float scratch[4];
    extern __shared__ float vals[];  // d floats: the summed row
    const int i = blockIdx.x;
    const size_t r = rows ? rows[i] : i;
    float* src = x + r * d;
    float ss = 0.f;
    for (int c = threadIdx.x; c < d; c += 256) {
        const float wc = w[c];  // requested with the row, not after the reduction
        float v = src[c];
        for (int p = 0; p < n_partials; ++p) v += partials[p * partial_stride + r * d + c];
        if (n_partials > 0 && !rows) src[c] = v;
        vals[c] = v * wc;
        ss += v * v;
    }
    ss = block_sum<256>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    OutT* dst = out + (size_t)i * d;
    for (int c = threadIdx.x; c < d; c += 256) dst[c] = from_f32<OutT>(vals[c] * inv);
}

// The same for widths that are a multiple of four and at most 1024 * G.  A thread owns G groups of
// four consecutive columns (group t, t + 256, ...) and asks for all of the row it needs - stream,
// weights and the NP pending sums - before it uses the first value, so the kernel pays one memory
// round trip instead of one per column and pending sum.  The sums are added in the same order.
// With more than eight pending sums (MORE, NP = 8) the rest, up to eight again, follows in a second
// round of loads.
template <typename OutT, int G, int NP, bool MORE = false>
__global__ __launch_bounds__(256) void rmsnorm_wide_kernel(float* __restrict__ x, const float* __restrict__ partials,
                                                           size_t partial_stride, const int* __restrict__ rows,
                                                           const float* __restrict__ w, OutT* __restrict__ out, int d,
                                                           float eps, int n_more) {
    arguments_now(x, partials, partial_stride, rows, w, out, d, eps, n_more);
    __shared__ float scratch[4];
    const int i = blockIdx.x, ng = d / 4;
    const size_t r = rows ? rows[i] : i;
    f32x4* src = reinterpret_cast<f32x4*>(x + r * d);
    const f32x4* w4 = reinterpret_cast<const f32x4*>(w);
    f32x4 v[G], wv[G], pend[NP > 0 ? NP : 1][G];
    int at[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int c4 = threadIdx.x + g * 256;
        at[g] = c4 < ng ? c4 : 0;  // a group beyond the row reads group 0 and is dropped
        v[g] = src[at[g]];
        wv[g] = w4[at[g]];
    }
#pragma unroll
    for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int g = 0; g < G; ++g) pend[p][g] = reinterpret_cast<const f32x4*>(partials + p * partial_stride + r * d)[at[g]];
    if constexpr (MORE) {
        static_assert(NP == 8, "a second round follows a full first one");
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int p = 0; p < NP; ++p) v[g] += pend[p][g];
        // sums beyond the last one read the last one again and count for nothing
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int g = 0; g < G; ++g)
                pend[p][g] = reinterpret_cast<const f32x4*>(partials + (size_t)(NP + min(p, n_more - 1)) * partial_stride + r * d)[at[g]];
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                const float keep = p < n_more ? 1.f : 0.f;
                v[g] += pend[p][g] * keep;
            }
    }
    float ss = 0.f;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if constexpr (!MORE) {
#pragma unroll
            for (int p = 0; p < NP; ++p) v[g] += pend[p][g];
        }
        if (threadIdx.x + g * 256 < ng) {
            if ((NP > 0 || MORE) && !rows) src[at[g]] = v[g];
            ss += v[g].x * v[g].x + v[g].y * v[g].y + v[g].z * v[g].z + v[g].w * v[g].w;
        }
    }
    ss = block_sum<256>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    OutT* dst = out + (size_t)i * d;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if (threadIdx.x + g * 256 >= ng) continue;
        const f32x4 o = v[g] * wv[g] * inv;
        typedef OutT out4_t __attribute__((ext_vector_type(4)));  // the group's four values in one store
        const out4_t o4 = {from_f32<OutT>(o.x), from_f32<OutT>(o.y), from_f32<OutT>(o.z), from_f32<OutT>(o.w)};
        *reinterpret_cast<out4_t*>(dst + (size_t)at[g] * 4) = o4;
    }
}

// x[t, :] += sum_p partials[p, t, :] (in order): pending sums folded in without a norm
__global__ __launch_bounds__(256) void add_partials_kernel(float* __restrict__ x, const float* __restrict__ partials,
                                                           int n_partials, size_t partial_stride, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v = x[i];
    for (int p = 0; p < n_partials; ++p) v += partials[p * partial_stride + i];
    x[i] = v;
}

struct RopeArgs {
    const float* qkv;       // [n_partials, T, stride] partial sums of: q heads, then (if written) k heads, v heads
    const float* bias;      // [stride] or null, added to the sum
    int n_partials;
    size_t partial_stride;
    const int* positions;   // [T]
    const float* inv_freq;  // [hd / 2] or null: no rotation
    const int* slot_map;    // [T] page * ps + offset of the row's key, or null: nothing is written
    elem_t* q_out;          // [T, H * hd]
    elem_t* kpool;          // [pages, KV, ps, hd]
    elem_t* vpool;          // [pages, KV, hd, ps]
    int stride, H, KV, hd, ps;
};

__global__ __launch_bounds__(256) void rope_kv_write_kernel(RopeArgs a) {
    __shared__ float cs[128], sn[128];
    extern __shared__ float row[];  // stride floats: this row's sums with the bias added
    const int t = blockIdx.x, half = a.hd / 2;
    const int width = a.H * a.hd + (a.slot_map ? 2 * a.KV * a.hd : 0);
    for (int c = threadIdx.x; c < width; c += 256) {
        float v = a.bias ? a.bias[c] : 0.f;
        for (int p = 0; p < a.n_partials; ++p) v += a.qkv[p * a.partial_stride + (size_t)t * a.stride + c];
        row[c] = v;
    }
    if (threadIdx.x < half) {
        float c = 1.f, s = 0.f;
        if (a.inv_freq) {
            const float ang = (float)a.positions[t] * a.inv_freq[threadIdx.x];
            sincosf(ang, &s, &c);
        }
        cs[threadIdx.x] = c;
        sn[threadIdx.x] = s;
    }
    __syncthreads();
    // q: pairs (j, j + half) of every head
    for (int p = threadIdx.x; p < a.H * half; p += 256) {
        const int h = p / half, j = p % half;
        const float x0 = row[h * a.hd + j], x1 = row[h * a.hd + j + half];
        elem_t* o = a.q_out + ((size_t)t * a.H + h) * a.hd;
        o[j] = from_f32<elem_t>(x0 * cs[j] - x1 * sn[j]);
        o[j + half] = from_f32<elem_t>(x0 * sn[j] + x1 * cs[j]);
    }
    if (!a.slot_map) return;
    const int slot = a.slot_map[t];
    if (slot < 0) return;
    const int page = slot / a.ps, off = slot % a.ps;
    const float* krow = row + a.H * a.hd;
    const float* vrow = krow + a.KV * a.hd;
    for (int p = threadIdx.x; p < a.KV * half; p += 256) {
        const int h = p / half, j = p % half;
        const float x0 = krow[h * a.hd + j], x1 = krow[h * a.hd + j + half];
        elem_t* o = a.kpool + (((size_t)page * a.KV + h) * a.ps + off) * a.hd;
        o[j] = from_f32<elem_t>(x0 * cs[j] - x1 * sn[j]);
        o[j + half] = from_f32<elem_t>(x0 * sn[j] + x1 * cs[j]);
    }
    for (int p = threadIdx.x; p < a.KV * a.hd; p += 256) {
        const int h = p / a.hd, dd = p % a.hd;
        a.vpool[(((size_t)page * a.KV + h) * a.hd + dd) * a.ps + off] = from_f32<elem_t>(vrow[p]);
    }
}

// cs[t, j] = (cos, sin) of positions[t] * inv_freq[j]: the angles of a step's rows, once for every layer that rotates
// by these frequencies, for the product that rotates in its own epilogue (it cannot share a row's sines among its
// lanes as the kernels here do).  The same expression as above: the same values.
__global__ __launch_bounds__(256) void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                                         float* __restrict__ cs, int n, int half) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int t = i / half, j = i - t * half;
    float c, s;
    sincosf((float)positions[t] * inv_freq[j], &s, &c);
    cs[2 * (size_t)i] = c;
    cs[2 * (size_t)i + 1] = s;
}

// The same in quads: head sizes that are multiples of 8, rows whose stride is a multiple of 4 and
// 16-byte aligned buffers.  A thread takes four neighbouring pairs (j .. j + 3, j + half .. + 3) of one
// head: two 16-byte loads per partial sum, all asked for before the first is used, and two 8-byte
// (bfloat16) or 16-byte stores.  Nothing is staged in LDS but the row's cosines and sines.
template <int NP>
__global__ __launch_bounds__(256) void rope_kv_write_quads_kernel(RopeArgs a) {
    __shared__ float cs[128], sn[128];
    const int t = blockIdx.x, half = a.hd / 2, hq = half / 4;
    if (threadIdx.x < half) {
        float c = 1.f, s = 0.f;
        if (a.inv_freq) {
            const float ang = (float)a.positions[t] * a.inv_freq[threadIdx.x];
            sincosf(ang, &s, &c);
        }
        cs[threadIdx.x] = c;
        sn[threadIdx.x] = s;
    }
    const bool writes = a.slot_map != nullptr;
    const int slot = writes ? a.slot_map[t] : -1;
    const int page = slot >= 0 ? slot / a.ps : 0, off = slot >= 0 ? slot % a.ps : 0;
    const float* rowp = a.qkv + (size_t)t * a.stride;
    auto summed = [&](int c) {  // bias + the partial sums of columns c .. c + 3, in order
        f32x4 v[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) v[p] = *reinterpret_cast<const f32x4*>(rowp + p * a.partial_stride + c);
        f32x4 r = a.bias ? *reinterpret_cast<const f32x4*>(a.bias + c) : (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < NP; ++p) r += v[p];
        return r;
    };
    auto store_quad = [](elem_t* o, const f32x4& v) {
#ifdef MS_ELEM_HALF
        half4_t b = {(elem_t)v[0], (elem_t)v[1], (elem_t)v[2], (elem_t)v[3]};
        *reinterpret_cast<half4_t*>(o) = b;
#else
        *reinterpret_cast<f32x4*>(o) = v;
#endif
    };
    // q heads, then k heads: pairs (j, j + half)
    const int rot_heads = a.H + (writes ? a.KV : 0);
    const int n_rot = rot_heads * hq;
    // v heads: quads of the head's elements
    const int n_v = writes ? a.KV * (a.hd / 4) : 0;
    __syncthreads();
    for (int it = threadIdx.x; it < n_rot + n_v; it += 256) {
        if (it < n_rot) {
            const int h = it / hq, j = (it % hq) * 4;
            const f32x4 x0 = summed(h * a.hd + j), x1 = summed(h * a.hd + half + j);
            f32x4 lo, hi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[e] = x0[e] * cs[j + e] - x1[e] * sn[j + e];
                hi[e] = x0[e] * sn[j + e] + x1[e] * cs[j + e];
            }
            elem_t* o;
            if (h < a.H) o = a.q_out + ((size_t)t * a.H + h) * a.hd;
            else if (slot >= 0) o = a.kpool + (((size_t)page * a.KV + (h - a.H)) * a.ps + off) * a.hd;
            else continue;
            store_quad(o + j, lo);
            store_quad(o + half + j, hi);
        } else if (slot >= 0) {
            const int q = it - n_rot, h = q / (a.hd / 4), dd = (q % (a.hd / 4)) * 4;
            const f32x4 v = summed((a.H + a.KV + h) * a.hd + dd);
            elem_t* o = a.vpool + (((size_t)page * a.KV + h) * a.hd + dd) * a.ps + off;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[(size_t)e * a.ps] = from_f32<elem_t>(v[e]);
        }
    }
}

}  // namespace ms

using namespace ms;

// The widest row that the norm and the rotation kernels hold in a block's LDS (floats); a model asks for these
// when it is put together, so that a wider one is refused then, with the size's name, not at its first step.
constexpr int MAX_ROW_FLOATS = 15000;
extern "C" int ms_max_norm_width() { return MAX_ROW_FLOATS; }
extern "C" int ms_max_rope_row() { return MAX_ROW_FLOATS; }

// cs [T, half, 2] (float) = cosine and sine of positions[t] * inv_freq[j].
extern "C" int ms_rope_table(const int* positions, const float* inv_freq, float* cs, int T, int half, hipStream_t stream) {
    MS_REQUIRE(T > 0 && half > 0 && positions && inv_freq && cs, "rope table: T=%d, %d frequencies", T, half);
    MS_REQUIRE((long)T * half < 2147483647L, "rope table: %d rows of %d frequencies", T, half);
    const int n = T * half;
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, stream, positions, inv_freq, cs, n, half);
    return check_launch("rope_table");
}

extern "C" int ms_embed(const int* tokens, const void* table, float* x, int T, int d, float scale, hipStream_t stream) {
    MS_REQUIRE(T > 0 && d > 0, "embed: empty problem T=%d d=%d", T, d);
    hipLaunchKernelGGL(embed_kernel, dim3(T), dim3(256), 0, stream, tokens, (const elem_t*)table, x, d, scale);
    return check_launch("embed");
}

extern "C" int ms_feed_tokens(int* tokens, const int* sampled, const int* rows, const int* src, int n, int n_tokens, int n_sampled,
                              hipStream_t stream) {
    MS_REQUIRE(n > 0 && n_tokens > 0 && n_sampled > 0, "feed_tokens: empty problem n=%d tokens=%d sampled=%d", n, n_tokens, n_sampled);
    MS_REQUIRE(tokens && sampled && rows && src, "feed_tokens: a buffer is missing");
    hipLaunchKernelGGL(feed_tokens_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, stream, tokens, sampled, rows, src, n, n_tokens, n_sampled);
    return check_launch("feed_tokens");
}

// rows may be null (identity).  out is float when out_f32 != 0, else the element type.
// partials [n_partials, T, d] are pending sums of the stream x [T, d] (n_partials may be 0); see the
// kernel for what is written back.
extern "C" int ms_rmsnorm(float* x, const float* partials, int n_partials, int T, const int* rows, const float* w,
                          void* out, int out_f32, int n, int d, float eps, hipStream_t stream) {
    MS_REQUIRE(n > 0 && d > 0, "rmsnorm: empty problem n=%d d=%d", n, d);
    MS_REQUIRE(d <= MAX_ROW_FLOATS, "rmsnorm: width %d exceeds the row buffer of %d", d, MAX_ROW_FLOATS);
    MS_REQUIRE(n_partials == 0 || partials, "rmsnorm: %d partial sums without a buffer", n_partials);
    const size_t ps = (size_t)T * d, smem = (size_t)d * sizeof(float);
    const bool f32_out = out_f32 || !kHalf;
    const int groups = d % 4 == 0 ? (d <= 1024 ? 1 : (d <= 2048 ? 2 : (d <= 4096 ? 4 : 0))) : 0;
    const bool aligned = (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(partials)) % 16 == 0;
    if (groups && aligned && n_partials <= 16) {
#define MS_NORM(OUT_, G_, NP_)                                                                                   \
    hipLaunchKernelGGL((rmsnorm_wide_kernel<OUT_, G_, NP_>), dim3(n), dim3(256), 0, stream, x, partials, ps, rows, w, \
                       (OUT_*)out, d, eps, 0)
#define MS_NORM_MORE(OUT_, G_)                                                                                          \
    hipLaunchKernelGGL((rmsnorm_wide_kernel<OUT_, G_, 8, true>), dim3(n), dim3(256), 0, stream, x, partials, ps, rows, w, \
                       (OUT_*)out, d, eps, n_partials - 8)
#define MS_NORM_NP(OUT_, G_)                                    \
    switch (n_partials) {                                       \
        case 0: MS_NORM(OUT_, G_, 0); break;                    \
        case 1: MS_NORM(OUT_, G_, 1); break;                    \
        case 2: MS_NORM(OUT_, G_, 2); break;                    \
        case 3: MS_NORM(OUT_, G_, 3); break;                    \
        case 4: MS_NORM(OUT_, G_, 4); break;                    \
        case 5: MS_NORM(OUT_, G_, 5); break;                    \
        case 6: MS_NORM(OUT_, G_, 6); break;                    \
        case 7: MS_NORM(OUT_, G_, 7); break;                    \
        case 8: MS_NORM(OUT_, G_, 8); break;                    \
        default: MS_NORM_MORE(OUT_, G_); break;                 \
    }
#define MS_NORM_G(OUT_)                                         \
    if (groups == 1) { MS_NORM_NP(OUT_, 1) }                    \
    else if (groups == 2) { MS_NORM_NP(OUT_, 2) }               \
    else { MS_NORM_NP(OUT_, 4) }
        if (f32_out) { MS_NORM_G(float) } else { MS_NORM_G(elem_t) }
#undef MS_NORM_G
#undef MS_NORM_NP
#undef MS_NORM_MORE
#undef MS_NORM
        return check_launch("rmsnorm");
    }
    if (f32_out)
        hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(n), dim3(256), smem, stream, x, partials, n_partials, ps, rows, w,
                           (float*)out, d, eps);
    else
        hipLaunchKernelGGL(rmsnorm_kernel<elem_t>, dim3(n), dim3(256), smem, stream, x, partials, n_partials, ps, rows, w,
                           (elem_t*)out, d, eps);
    return check_launch("rmsnorm");
}

extern "C" int ms_add_partials(float* x, const float* partials, int n_partials, int T, int d, hipStream_t stream) {
    MS_REQUIRE(T > 0 && d > 0 && n_partials > 0, "add_partials: empty problem");
    const size_t n = (size_t)T * d;
    hipLaunchKernelGGL(add_partials_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, partials,
                       n_partials, n, n);
    return check_launch("add_partials");
}

// Sum the partial sums of the q/k/v projection, add the bias, rotate q (and k) by the rows'
// positions and write k, v into their pages.  inv_freq null: no
// rotation.  slot_map null: the rows hold q only and nothing is written (a layer that reads
// another layer's cache).
extern "C" int ms_rope_kv_write(const float* qkv, int n_partials, const float* bias, int stride, const int* positions,
                                const float* inv_freq,
                                const int* slot_map, void* q_out, void* kpool, void* vpool, int T, int H, int KV,
                                int hd, int ps, hipStream_t stream) {
    MS_REQUIRE(T > 0, "rope: no rows");
    MS_REQUIRE(hd % 2 == 0 && hd >= 2 && hd <= 256, "rope: head size %d must be even and at most 256", hd);
    MS_REQUIRE(stride >= H * hd + (slot_map ? 2 * KV * hd : 0), "rope: row stride %d too small for %d+2*%d heads of %d",
               stride, H, KV, hd);
    MS_REQUIRE(!slot_map || (kpool && vpool && ps > 0), "rope: cache write without pools");
    MS_REQUIRE(n_partials >= 1, "rope: %d partial sums", n_partials);
    MS_REQUIRE(stride <= MAX_ROW_FLOATS, "rope: a row of %d values exceeds the row buffer of %d", stride, MAX_ROW_FLOATS);
    RopeArgs a{qkv, bias, n_partials, (size_t)T * stride, positions, inv_freq, slot_map, (elem_t*)q_out, (elem_t*)kpool,
               (elem_t*)vpool, stride, H, KV, hd, ps};
    const bool aligned = ((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(bias) | reinterpret_cast<uintptr_t>(q_out) |
                           reinterpret_cast<uintptr_t>(kpool)) & 15) == 0;
    // (up to eight partial sums: a portion of 65 to 128 rows cuts the projection's K seven times)
    if (hd % 8 == 0 && stride % 4 == 0 && a.partial_stride % 4 == 0 && aligned && n_partials <= 8) {
        switch (n_partials) {
            case 1: hipLaunchKernelGGL(rope_kv_write_quads_kernel<1>, dim3(T), dim3(256), 0, stream, a); break;
            case 2: hipLaunchKernelGGL(rope_kv_write_quads_kernel<2>, dim3(T), dim3(256), 0, stream, a); break;
            case 3: hipLaunchKernelGGL(rope_kv_write_quads_kernel<3>, dim3(T), dim3(256), 0, stream, a); break;
            case 4: hipLaunchKernelGGL(rope_kv_write_quads_kernel<4>, dim3(T), dim3(256), 0, stream, a); break;
            case 5: hipLaunchKernelGGL(rope_kv_write_quads_kernel<5>, dim3(T), dim3(256), 0, stream, a); break;
            case 6: hipLaunchKernelGGL(rope_kv_write_quads_kernel<6>, dim3(T), dim3(256), 0, stream, a); break;
            case 7: hipLaunchKernelGGL(rope_kv_write_quads_kernel<7>, dim3(T), dim3(256), 0, stream, a); break;
            default: hipLaunchKernelGGL(rope_kv_write_quads_kernel<8>, dim3(T), dim3(256), 0, stream, a); break;
        }
        return check_launch("rope_kv_write");
    }
    hipLaunchKernelGGL(rope_kv_write_kernel, dim3(T), dim3(256), (size_t)stride * sizeof(float), stream, a);
    return check_launch("rope_kv_write");
}
