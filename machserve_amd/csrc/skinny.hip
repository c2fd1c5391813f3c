// Matrix products with few rows (a decode step: M <= 64): out[M, N] = A[M, K] W[N, K]^T.
// The weights are read exactly once, straight from memory into MFMA fragments (no LDS
// staging: nothing of W is reused), and the work is cut so that thousands of waves stream
// at once whatever N is.
//
// Role in the reference: gemv_f16 / gemv_f16_qkv (crates/mach-model/src/kernels.rs:2665-2808),
// one 32-lane warp per output with shuffles; here a 64-lane wave owns 16 * NT output columns
// and up to 64 rows at once on the matrix cores.
//
// A block is WN x KSI waves: WN groups of output columns, KSI slices of K.  The KSI slices
// of a block are summed through LDS in slice order; gridDim.y further slices write partial
// sums out[ks][M][N] that the consumer adds in order (the norm that follows a residual, the
// rotation that follows the q/k/v projection).  How K is cut depends on N and K only, never
// on M, so a row's result does not depend on what else is in the batch.
#include "common.cuh"

namespace ms {

constexpr int KSTEP = 128;  // K elements per wave iteration: four fragments per lane; fragment c of the wave is the
                            // contiguous chunk c of 32 elements (the four key groups side by side: 64 bytes a row in bf16)

enum SkinnyEpi { SK_STORE_F32 = 0, SK_SWIGLU = 1 };

struct SkinnyArgs {
    const elem_t* A;  // [M, K]
    const elem_t* W;  // [N, K]
    void* out;        // SK_STORE_F32: float [gridDim.y, M, N]; SK_SWIGLU: elem [M, n_out]
    int M, N, K;
    int k_per_wave;   // multiple of 32
    int n_out;        // SK_SWIGLU: intermediate size
};

__device__ __forceinline__ float silu_sk(float g) {
#ifdef MS_ELEM_BF16
    return g / (1.0f + __expf(-g));
#else
    return g / (1.0f + expf(-g));
#endif
}

template <int MT, int NT, int WN, int KSI, int EPI>
__global__ __launch_bounds__(64 * WN * KSI) void gemm_skinny_kernel(SkinnyArgs a) {
    __shared__ float red[(KSI > 1 ? (KSI - 1) : 1) * WN * NT * 4 * 64];  // one row tile of every slice at a time
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wn = wave % WN, wk = wave / WN;
    const int r16 = lane & 15, grp = lane >> 4;
    const int n0 = (blockIdx.x * WN + wn) * 16 * NT;
    const int k0 = (blockIdx.y * KSI + wk) * a.k_per_wave;
    const int k1 = min(a.K, k0 + a.k_per_wave);

    f32x4 acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    if (n0 < a.N) {
        // Every load is unconditional, so that all of a slice's fragments are in flight at once and
        // one wait serves them: a row or column beyond the matrix reads row 0 instead (what it adds
        // to is never stored), and elements beyond the end of K are read from the last eight of the
        // row and dropped from A, so that they add nothing whatever W holds there.
        const elem_t* wrow[NT];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int n = n0 + j * 16 + r16;
            wrow[j] = a.W + (size_t)(n < a.N ? n : 0) * a.K;
        }
        const elem_t* arow[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int m = i * 16 + r16;
            arow[i] = a.A + (size_t)(m < a.M ? m : 0) * a.K;
        }
        // `spread` 0 makes every lane of a row read the same 16 bytes: a load that is only there to
        // keep the loop's shape (after the last step) then costs one line per row
        auto load = [&](int kk, int spread, Frag (&fw)[NT][4], Frag (&fa)[MT][4]) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int k = min(kk + (c * 4 + grp) * 8 * spread, a.K - 8);
#pragma unroll
                for (int j = 0; j < NT; ++j) fw[j][c] = frag_load(wrow[j] + k);
#pragma unroll
                for (int i = 0; i < MT; ++i) fa[i][c] = frag_load(arow[i] + k);
            }
        };
        auto multiply = [&](int kk, Frag (&fw)[NT][4], Frag (&fa)[MT][4]) {
            if (kk + KSTEP > k1) {  // the slice ends inside this step (the same for the whole wave)
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (kk + (c * 4 + grp) * 8 >= k1) {
#pragma unroll
                        for (int i = 0; i < MT; ++i) fa[i][c] = frag_zero();
                    }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j) mma_16x16x32(acc[i][j], fa[i][c], fw[j][c]);
        };
        constexpr bool PREFETCH = MT * NT <= 8;  // a second set of fragments fits the registers
        Frag fw0[NT][4], fa0[MT][4];
        if (!PREFETCH || k1 - k0 <= KSTEP) {
            for (int kk = k0; kk < k1; kk += KSTEP) {
                load(kk, 1, fw0, fa0);
                multiply(kk, fw0, fa0);
            }
        } else {
            // two sets of fragments take turns: the next step is in flight while this one is multiplied
            Frag fw1[NT][4], fa1[MT][4];
            load(k0, 1, fw0, fa0);
            for (int kk = k0; kk < k1; kk += 2 * KSTEP) {
                const bool more1 = kk + KSTEP < k1;
                load(more1 ? kk + KSTEP : k0, more1, fw1, fa1);
                multiply(kk, fw0, fa0);
                if (!more1) break;
                const bool more2 = kk + 2 * KSTEP < k1;
                load(more2 ? kk + 2 * KSTEP : k0, more2, fw0, fa0);
                multiply(kk + KSTEP, fw1, fa1);
            }
        }
    }

    // sum the K slices of the block in slice order: slice 0 keeps its sums and adds 1, 2, ...;
    // one 16-row tile per round keeps the LDS buffer small
    if constexpr (KSI > 1) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            if (i > 0) __syncthreads();
            if (wk > 0) {
                float* dst = red + ((size_t)((wk - 1) * WN + wn) * NT * 4) * 64;
#pragma unroll
                for (int j = 0; j < NT; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[(j * 4 + e) * 64 + lane] = acc[i][j][e];
            }
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int s = 1; s < KSI; ++s) {
                    const float* src = red + ((size_t)((s - 1) * WN + wn) * NT * 4) * 64;
#pragma unroll
                    for (int j = 0; j < NT; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][e] += src[(j * 4 + e) * 64 + lane];
                }
            }
        }
    }
    const bool owner = wk == 0 && n0 < a.N;  // this wave holds the finished sums of its columns

    if constexpr (EPI == SK_SWIGLU) {
        static_assert(NT % 2 == 0, "gate and up tiles come in pairs");
        if (!owner) return;
        elem_t* out = reinterpret_cast<elem_t*>(a.out);
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; j += 2) {
                const int col = (n0 + j * 16) / 2 + r16;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = i * 16 + grp * 4 + e;
                    if (row < a.M && col < a.n_out)
                        out[(size_t)row * a.n_out + col] = from_f32<elem_t>(silu_sk(acc[i][j][e]) * acc[i][j + 1][e]);
                }
            }
    } else {
        if (owner) {
            float* out = reinterpret_cast<float*>(a.out) + (size_t)blockIdx.y * a.M * a.N;
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const int col = n0 + j * 16 + r16;
                    if (col >= a.N) continue;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = i * 16 + grp * 4 + e;
                        if (row < a.M) out[(size_t)row * a.N + col] = acc[i][j][e];
                    }
                }
        }
    }
}

// How K is cut for a product of N columns over K: (slices inside a block, blocks along K,
// K per wave).  A function of N and K alone.
struct SkinnyPlan { int wn, ksi, ksb, k_per_wave; };

// Columns per wave in units of 16: with more than 32 rows and enough columns to keep every CU busy,
// a wave takes 64 columns, so that the rows it re-reads (from L2, they are shared by all waves)
// weigh no more than the weights it streams.
static int skinny_nt(int M, int N) { return (M > 32 && N >= 4096) ? 4 : 2; }

static int g_force_ksi = 0;  // measurements only: waves along K inside a block (1 = four column waves)
static int g_max_ksb = 0;    // measurements only: most blocks along K

static SkinnyPlan plan_skinny(int M, int N, int K, bool allow_partials) {
    const int NT = skinny_nt(M, N);
    const int col_waves = ceil_div(N, 16 * NT);
    const int slices = ceil_div(K, KSTEP);  // slices of 128 along K: one wave iteration each
    int want = max(1, min(ceil_div(4096, col_waves), slices));  // waves wanted along K
    if (g_force_ksi > 0) want = min(g_force_ksi, slices);
    SkinnyPlan p;
    if (want == 1) {
        p = {4, 1, 1, slices * KSTEP};
        return p;
    }
    p.wn = 1;
    p.ksi = want > 4 ? 8 : (want > 2 ? 4 : 2);
    p.ksb = (allow_partials && want > p.ksi) ? ceil_div(want, p.ksi) : 1;
    if (g_max_ksb > 0) p.ksb = min(p.ksb, g_max_ksb);
    p.k_per_wave = ceil_div(slices, p.ksi * p.ksb) * KSTEP;
    return p;
}

template <int MT, int NT, int EPI>
static int launch_skinny_mt(const SkinnyArgs& a0, const SkinnyPlan& p, hipStream_t stream) {
    SkinnyArgs a = a0;
    a.k_per_wave = p.k_per_wave;
    const dim3 grid((unsigned)ceil_div(a.N, 16 * NT * p.wn), (unsigned)p.ksb);
#define MS_SK(WN_, KSI_)                                                                                          \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT, WN_, KSI_, EPI>), grid, dim3(64 * WN_ * KSI_), 0, stream, a); \
    return check_launch("gemm_skinny")
    if (p.wn == 4) { MS_SK(4, 1); }
    if (p.ksi == 8) { MS_SK(1, 8); }
    if (p.ksi == 4) { MS_SK(1, 4); }
    if (p.ksi == 2) { MS_SK(1, 2); }
    MS_SK(1, 1);
#undef MS_SK
}

template <int EPI>
static int launch_skinny(const SkinnyArgs& a, const SkinnyPlan& p, hipStream_t stream) {
    MS_REQUIRE(a.M > 0 && a.M <= 64, "skinny product: M=%d must be in 1..64", a.M);
    MS_REQUIRE(a.K % 8 == 0, "skinny product: the reduction size K=%d must be a multiple of 8", a.K);
    if (a.M <= 16) return launch_skinny_mt<1, 2, EPI>(a, p, stream);
    if (a.M <= 32) return launch_skinny_mt<2, 2, EPI>(a, p, stream);
    if (skinny_nt(a.M, a.N) == 4) {
        if (a.M <= 48) return launch_skinny_mt<3, 4, EPI>(a, p, stream);
        return launch_skinny_mt<4, 4, EPI>(a, p, stream);
    }
    if (a.M <= 48) return launch_skinny_mt<3, 2, EPI>(a, p, stream);
    return launch_skinny_mt<4, 2, EPI>(a, p, stream);
}

}  // namespace ms

using namespace ms;

extern "C" void ms_skinny_force_ksi(int ksi) { g_force_ksi = ksi; }
extern "C" void ms_skinny_max_ksb(int ksb) { g_max_ksb = ksb; }

// Number of partial sums ms_linear_skinny writes for M rows of this N and K (1 = the complete product).
extern "C" int ms_skinny_partials(int M, int N, int K, int allow_partials) { return plan_skinny(M, N, K, allow_partials != 0).ksb; }

// out[ks, M, N] (float) = partial sums of a w^T; ks = ms_skinny_partials(N, K, allow_partials).
extern "C" int ms_linear_skinny(const void* a, const void* w, float* out, int M, int N, int K, int allow_partials,
                                hipStream_t stream) {
    SkinnyArgs args{(const elem_t*)a, (const elem_t*)w, out, M, N, K, 0, 0};
    return launch_skinny<SK_STORE_F32>(args, plan_skinny(M, N, K, allow_partials != 0), stream);
}

// out[M, I] = silu(a g^T) * (a u^T), gate and up rows interleaved in blocks of 16 (see ms_linear_swiglu).
extern "C" int ms_linear_swiglu_skinny(const void* a, const void* w, void* out, int M, int I, int K, hipStream_t stream) {
    const int n = 2 * ceil_div(I, 16) * 16;
    SkinnyArgs args{(const elem_t*)a, (const elem_t*)w, out, M, n, K, 0, I};
    return launch_skinny<SK_SWIGLU>(args, plan_skinny(M, n, K, false), stream);
}
