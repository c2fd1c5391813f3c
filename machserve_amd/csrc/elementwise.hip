// Memory-bound kernels around the matrix products: embedding gather, RMS norm (optionally
// of gathered rows), and rotation of q and k fused with the write of k and v into pages.
//
// Role in the reference: embed_batched, rms_norm, rope_batched, kv_store_paged
// (crates/mach-model/src/kernels.rs:578-585, 63-80, 589-660, 1148-1168).
// Norm statistics, rotation angles and the rotation itself are 32-bit in both builds.
#include "common.cuh"

namespace ms {

// x[t, :] = float(table[tokens[t], :])
__global__ __launch_bounds__(256) void embed_kernel(const int* __restrict__ tokens, const elem_t* __restrict__ table,
                                                    float* __restrict__ x, int d) {
    const int t = blockIdx.x;
    const elem_t* src = table + (size_t)tokens[t] * d;
    float* dst = x + (size_t)t * d;
    for (int c = threadIdx.x; c < d; c += 256) dst[c] = to_f32(src[c]);
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

}  // namespace ms

using namespace ms;

extern "C" int ms_embed(const int* tokens, const void* table, float* x, int T, int d, hipStream_t stream) {
    MS_REQUIRE(T > 0 && d > 0, "embed: empty problem T=%d d=%d", T, d);
    hipLaunchKernelGGL(embed_kernel, dim3(T), dim3(256), 0, stream, tokens, (const elem_t*)table, x, d);
    return check_launch("embed");
}

// rows may be null (identity).  out is float when out_f32 != 0, else the element type.
// partials [n_partials, T, d] are pending sums of the stream x [T, d] (n_partials may be 0); see the
// kernel for what is written back.
extern "C" int ms_rmsnorm(float* x, const float* partials, int n_partials, int T, const int* rows, const float* w,
                          void* out, int out_f32, int n, int d, float eps, hipStream_t stream) {
    MS_REQUIRE(n > 0 && d > 0, "rmsnorm: empty problem n=%d d=%d", n, d);
    MS_REQUIRE(d * sizeof(float) <= 60000, "rmsnorm: width %d exceeds the row buffer", d);
    MS_REQUIRE(n_partials == 0 || partials, "rmsnorm: %d partial sums without a buffer", n_partials);
    const size_t ps = (size_t)T * d, smem = (size_t)d * sizeof(float);
    if (out_f32 || !kBf16)
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
    MS_REQUIRE(stride * sizeof(float) <= 60000, "rope: a row of %d values exceeds the row buffer", stride);
    RopeArgs a{qkv, bias, n_partials, (size_t)T * stride, positions, inv_freq, slot_map, (elem_t*)q_out, (elem_t*)kpool,
               (elem_t*)vpool, stride, H, KV, hd, ps};
    hipLaunchKernelGGL(rope_kv_write_kernel, dim3(T), dim3(256), (size_t)stride * sizeof(float), stream, a);
    return check_launch("rope_kv_write");
}
