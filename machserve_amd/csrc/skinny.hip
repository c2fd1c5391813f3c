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
// rotation that follows the q/k/v projection).  How K is cut depends on N, K and on whether the
// step has more than 32 rows (then a wave takes 64 columns instead of 32 under a wide output, which
// changes how many waves share K); within either range a row's sums do not depend on what else is
// in the batch, and between them they differ in the order of summation only.
#include "common.cuh"

namespace ms {

constexpr int KSTEP = 128;  // K elements per wave iteration: four fragments per lane; fragment c of the wave is the
                            // contiguous chunk c of 32 elements (the four key groups side by side: 64 bytes a row in bf16)

enum SkinnyEpi { SK_STORE_F32 = 0, SK_SWIGLU = 1, SK_RESIDUAL = 2, SK_RESIDUAL_PRENORM = 3 };

struct SkinnyArgs {
    const elem_t* A;  // [M, K]
    const elem_t* W;  // [N, K]
    void* out;        // SK_STORE_F32: float [gridDim.y, M, N]; SK_SWIGLU: elem [M, n_out]; SK_RESIDUAL: float [M, N], added to
    int M, N, K;
    int k_per_wave;   // multiple of 32
    int n_out;        // SK_SWIGLU: intermediate size
    // SK_RESIDUAL_PRENORM: beside the sum, what the norm that follows needs from it
    const float* norm_w;  // [N]
    elem_t* hn;           // [M, N]: (stream + product) * norm_w, not yet divided by the root mean square
    float* ss_part;       // [column waves, M]: each column wave's share of the rows' sums of squares
    // SK_SWIGLU of rows that came in multiplied by a norm's weight only (at most 16 rows): both products of a
    // row are multiplied by 1 / sqrt(sum over parts of row_ss[part, row] / K + ss_eps) before the activation
    const float* row_ss;  // [ss_parts, M] or null
    int ss_parts;
    float ss_eps;
    int act;          // SK_SWIGLU: the activation on the gate (GateActivation)
};

// A block of eight waves puts two on every SIMD; with more than 128 registers a wave a CU then holds one
// block, and a grid of more blocks than CUs (the gated product: 304 for 9,728 columns) runs in two rounds
// although every block only waits for its one trip to memory.  One row tile under at most 32 columns a wave
// fits 128 registers where nothing of the residual stream is held beside the sums: two blocks a CU.
template <int MT, int NT, int WN, int KSI, int EPI>
constexpr int skinny_waves_per_simd() { return (WN * KSI == 8 && MT == 1 && NT <= 2 && EPI <= SK_SWIGLU) ? 4 : 1; }

template <int MT, int NT, int WN, int KSI, int EPI>
__global__ __launch_bounds__(64 * WN * KSI, (skinny_waves_per_simd<MT, NT, WN, KSI, EPI>())) void gemm_skinny_kernel(SkinnyArgs a) {
    arguments_now(a.A, a.W, a.out, a.M, a.N, a.K, a.k_per_wave);
    if constexpr (EPI == SK_SWIGLU) arguments_now(a.n_out, a.row_ss, a.ss_parts, a.ss_eps, a.act);
    if constexpr (EPI == SK_RESIDUAL_PRENORM) arguments_now(a.norm_w, a.hn, a.ss_part);
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

    // SK_SWIGLU with row factors: the rows' sums of squares come in parts (written by the kernel before this
    // one).  The block's waves share them out: lane (row, q) of wave w adds parts 4 w + q, 4 w + q + 4 W, ...
    // (W waves), the first two of them asked for here with everything else; the four q of a row are added by
    // shuffles, the waves' shares through LDS in wave order.  The order depends on the number of parts only.
    constexpr bool FACTORS = EPI == SK_SWIGLU && MT == 1;
    __shared__ float ss_red[FACTORS ? WN * KSI : 1][16];
    float ss_early[2] = {0.f, 0.f};
    if constexpr (FACTORS) {
        if (a.row_ss) {
            const int share = wave * 4 + grp, row = min(r16, a.M - 1);
#pragma unroll
            for (int u = 0; u < 2; ++u)
                ss_early[u] = a.row_ss[(size_t)min(share + u * 4 * WN * KSI, a.ss_parts - 1) * a.M + row];
        }
    }

    // SK_RESIDUAL: the stream's values are asked for now, with everything else, not after the sums
    constexpr bool ADDS = EPI == SK_RESIDUAL || EPI == SK_RESIDUAL_PRENORM;
    static_assert(EPI != SK_RESIDUAL_PRENORM || MT <= 2, "the form that prepares the norm is for at most 32 rows");
    constexpr bool PRIOR_EARLY = ADDS && MT <= 2;  // with more row tiles the registers are needed elsewhere
    float prior[PRIOR_EARLY ? MT : 1][NT][4];
    if constexpr (PRIOR_EARLY) {
        const float* xs = reinterpret_cast<const float*>(a.out);
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = min(i * 16 + grp * 4 + e, a.M - 1), col = min(n0 + j * 16 + r16, a.N - 1);
                    prior[i][j][e] = xs[(size_t)row * a.N + col];
                }
    }
    // SK_RESIDUAL_PRENORM: the norm's weights of this wave's columns, asked for with everything else
    float nw_early[EPI == SK_RESIDUAL_PRENORM ? NT : 1];
    if constexpr (EPI == SK_RESIDUAL_PRENORM) {
#pragma unroll
        for (int j = 0; j < NT; ++j) nw_early[j] = a.norm_w[min(n0 + j * 16 + r16, a.N - 1)];
    }
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
        // a second set of fragments, if it fits the registers of a wave in a block of eight
        constexpr int FRAG_REGS = (int)sizeof(Frag) / 4;
        constexpr bool PREFETCH = 2 * (MT + NT) * 4 * FRAG_REGS + MT * NT * 4 <= 176;
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

    if constexpr (FACTORS) {
        if (a.row_ss) {
            constexpr int W = WN * KSI;
            const int share = wave * 4 + grp, row = min(r16, a.M - 1);
            float sq = (share < a.ss_parts ? ss_early[0] : 0.f) + (share + 4 * W < a.ss_parts ? ss_early[1] : 0.f);
            for (int p = share + 8 * W; p < a.ss_parts; p += 4 * W) sq += a.row_ss[(size_t)p * a.M + row];  // a very wide stream
            sq += __shfl_xor(sq, 16, WAVE);
            sq += __shfl_xor(sq, 32, WAVE);
            if (grp == 0) ss_red[wave][r16] = sq;
            if constexpr (KSI == 1) __syncthreads();  // with slices of K the barrier of their sum serves
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
        float f[4] = {1.f, 1.f, 1.f, 1.f};  // of the rows this lane holds
        if constexpr (FACTORS) {
            if (a.row_ss) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float sq = 0.f;
#pragma unroll
                    for (int w = 0; w < WN * KSI; ++w) sq += ss_red[w][grp * 4 + e];
                    f[e] = 1.0f / sqrtf(sq / (float)a.K + a.ss_eps);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; j += 2) {
                const int col = (n0 + j * 16) / 2 + r16;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = i * 16 + grp * 4 + e;
                    if (row < a.M && col < a.n_out)
                        out[(size_t)row * a.n_out + col] = from_f32<elem_t>(gate_activation(acc[i][j][e] * f[e], a.act) * (acc[i][j + 1][e] * f[e]));
                }
            }
    } else if constexpr (EPI == SK_RESIDUAL_PRENORM) {
        // The stream takes the sum as in SK_RESIDUAL.  The RMS norm that reads it next is prepared here: the new
        // values times the norm's weight in the element type, and this wave's columns' share of every row's sum
        // of squares (a lane's column of each tile, then the sixteen lanes by shuffles); the reader adds the
        // shares in column order and applies the factor to its finished sums.
        if (!owner) return;  // the same for a whole wave
        float* out = reinterpret_cast<float*>(a.out);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            float ss[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const int col = n0 + j * 16 + r16;
                const float nw = nw_early[j];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = i * 16 + grp * 4 + e;
                    const bool on = col < a.N && row < a.M;
                    const float v = prior[i][j][e] + acc[i][j][e];
                    if (on) {
                        out[(size_t)row * a.N + col] = v;
                        a.hn[(size_t)row * a.N + col] = from_f32<elem_t>(v * nw);
                    }
                    ss[e] += on ? v * v : 0.f;  // this lane's column of each tile, the tiles in order
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float sq = ss[e];
#pragma unroll
                for (int o = 1; o < 16; o <<= 1) sq += __shfl_xor(sq, o, WAVE);
                const int row = i * 16 + grp * 4 + e;
                if (r16 == 0 && row < a.M) a.ss_part[(size_t)(blockIdx.x * WN + wn) * a.M + row] = sq;
            }
        }
    } else {
        if (owner) {
            // SK_RESIDUAL: all of K lies in this block (gridDim.y == 1), so every element has one writer
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
                        if (row >= a.M) continue;
                        if constexpr (PRIOR_EARLY) out[(size_t)row * a.N + col] = prior[i][j][e] + acc[i][j][e];
                        else if constexpr (EPI == SK_RESIDUAL) out[(size_t)row * a.N + col] += acc[i][j][e];
                        else out[(size_t)row * a.N + col] = acc[i][j][e];
                    }
                }
        }
    }
}

// The same product for at most 16 rows with the RMS norm of the residual stream folded in:
//   v = x + sum_p partials[p] (in order);  out = ((v * norm_w) W^T) / sqrt(mean(v^2) + eps).
// The norm's factor is one number a row, so it is applied to the finished sums instead of to the
// rows: a wave builds its A fragments from v * norm_w (rounded to the element type as a norm kernel's
// output would be), sums v^2 over its slice of K, and the slices' sums of squares ride along with
// the reduction of the products through LDS.  The whole of K lies inside one block.  The blocks of
// the first columns also write v to x_out (another buffer than x, which other blocks still read):
// the stream with its pending sums added.  This saves the norm's own launch, a memory round trip
// on the critical path of a decode step.
struct SkinnyNormArgs {
    const float* x;         // [M, K] residual stream
    const float* partials;  // [NP, M, K] pending sums
    size_t partial_stride;
    const float* norm_w;    // [K]
    float* x_out;           // [M, K] or null (nothing pending)
    const elem_t* W;        // [N, K]
    void* out;              // SK_STORE_F32: float [M, N]; SK_SWIGLU: elem [M, n_out]
    int M, N, K, k_per_wave, n_out;
    float eps;
    int act;                // SK_SWIGLU: the activation on the gate (GateActivation)
};

template <int NT, int KSI, int EPI, int NP>
__global__ __launch_bounds__(64 * KSI) void gemm_skinny_norm_kernel(SkinnyNormArgs a) {
    arguments_now(a.x, a.partials, a.partial_stride, a.norm_w, a.x_out, a.W, a.out, a.M, a.N, a.K, a.k_per_wave, a.n_out, a.eps, a.act);
    static_assert(KSI > 1, "the slices of K are waves of one block");
    __shared__ float red[(KSI - 1) * NT * 4 * 64];
    __shared__ float ss_part[KSI][16];
    const int lane = threadIdx.x & 63, wk = threadIdx.x >> 6;
    const int r16 = lane & 15, grp = lane >> 4;
    const int n0 = blockIdx.x * 16 * NT;
    const int k0 = wk * a.k_per_wave, k1 = min(a.K, k0 + a.k_per_wave);
    const bool row_on = r16 < a.M;
    const size_t row = row_on ? r16 : 0;
    const float* xrow = a.x + row * a.K;
    const float* prow = a.partials + row * a.K;
    float* orow = a.x_out + row * a.K;
    const bool writer = blockIdx.x == 0 && a.x_out != nullptr && row_on;
    const elem_t* wrow[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        const int n = n0 + j * 16 + r16;
        wrow[j] = a.W + (size_t)(n < a.N ? n : 0) * a.K;
    }
    f32x4 acc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float ss = 0.f;
    for (int kk = k0; kk < k1; kk += KSTEP) {
        // Every load first (unconditional, clamped as in the plain kernel), then the sums.  With many
        // pending sums the registers hold only half a step's loads at a time.
        constexpr int HALVES = NP >= 3 ? 2 : 1, CPH = 4 / HALVES;
#pragma unroll
        for (int half = 0; half < HALVES; ++half) {
            Frag fw[NT][CPH];
            f32x4 xv[CPH][2], wn[CPH][2], pv[NP > 0 ? NP : 1][CPH][2];
#pragma unroll
            for (int cc = 0; cc < CPH; ++cc) {
                const int c = half * CPH + cc;
                const int k = min(kk + (c * 4 + grp) * 8, a.K - 8);
#pragma unroll
                for (int j = 0; j < NT; ++j) fw[j][cc] = frag_load(wrow[j] + k);
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    xv[cc][h] = *reinterpret_cast<const f32x4*>(xrow + k + 4 * h);
                    wn[cc][h] = *reinterpret_cast<const f32x4*>(a.norm_w + k + 4 * h);
#pragma unroll
                    for (int p = 0; p < NP; ++p)
                        pv[p][cc][h] = *reinterpret_cast<const f32x4*>(prow + p * a.partial_stride + k + 4 * h);
                }
            }
#pragma unroll
            for (int cc = 0; cc < CPH; ++cc) {
                const int k = kk + ((half * CPH + cc) * 4 + grp) * 8;
                const bool on = k < k1;  // beyond the slice: nothing (K is a multiple of 8, so a chunk is in or out)
                Frag fa;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    f32x4 v = xv[cc][h];
#pragma unroll
                    for (int p = 0; p < NP; ++p) v += pv[p][cc][h];
                    if (!on) v = (f32x4){0.f, 0.f, 0.f, 0.f};
                    if (writer && on && NP > 0) *reinterpret_cast<f32x4*>(orow + k + 4 * h) = v;
                    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
                    const f32x4 t = v * wn[cc][h];
                    fa.v[4 * h + 0] = from_f32<elem_t>(t.x);
                    fa.v[4 * h + 1] = from_f32<elem_t>(t.y);
                    fa.v[4 * h + 2] = from_f32<elem_t>(t.z);
                    fa.v[4 * h + 3] = from_f32<elem_t>(t.w);
                }
#pragma unroll
                for (int j = 0; j < NT; ++j) mma_16x16x32(acc[j], fa, fw[j][cc]);
            }
        }
    }
    // the row's sum of squares over this wave's slice: the four key groups of a row, then the slices
    ss += __shfl_xor(ss, 16, WAVE);
    ss += __shfl_xor(ss, 32, WAVE);
    if (grp == 0) ss_part[wk][r16] = ss;
    if (wk > 0) {
        float* dst = red + ((size_t)(wk - 1) * NT * 4) * 64;
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[(j * 4 + e) * 64 + lane] = acc[j][e];
    }
    __syncthreads();
    if (wk > 0 || n0 >= a.N) return;
#pragma unroll
    for (int s = 1; s < KSI; ++s) {
        const float* src = red + ((size_t)(s - 1) * NT * 4) * 64;
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[j][e] += src[(j * 4 + e) * 64 + lane];
    }
    float total = 0.f;
#pragma unroll
    for (int s = 0; s < KSI; ++s) total += ss_part[s][r16];  // in slice order
    const float inv_own = 1.0f / sqrtf(total / (float)a.K + a.eps);  // of row r16
    float inv[4];  // of the rows this lane holds: grp * 4 + e
#pragma unroll
    for (int e = 0; e < 4; ++e) inv[e] = __shfl(inv_own, grp * 4 + e, WAVE);

    if constexpr (EPI == SK_SWIGLU) {
        static_assert(NT % 2 == 0, "gate and up tiles come in pairs");
        elem_t* out = reinterpret_cast<elem_t*>(a.out);
#pragma unroll
        for (int j = 0; j < NT; j += 2) {
            const int col = (n0 + j * 16) / 2 + r16;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = grp * 4 + e;
                if (r < a.M && col < a.n_out)
                    out[(size_t)r * a.n_out + col] = from_f32<elem_t>(gate_activation(acc[j][e] * inv[e], a.act) * (acc[j + 1][e] * inv[e]));
            }
        }
    } else {
        float* out = reinterpret_cast<float*>(a.out);
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int col = n0 + j * 16 + r16;
            if (col >= a.N) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = grp * 4 + e;
                if (r < a.M) out[(size_t)r * a.N + col] = acc[j][e] * inv[e];
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
// Under at most 32 rows and a narrow output a wave takes 16 columns only: a CU that streams a weight alone gets
// little more than its share of the chip's rate, so a small weight wants as many blocks as it can be cut into
// (`pairs`: the gated product needs gate and up tiles side by side).
static int skinny_nt(int M, int N, bool pairs = false) {
    if (kHalf && M > 32 && N >= 4096) return 4;  // 32-bit fragments are twice as large
    if (!pairs && M <= 32 && N <= 2048) return 1;
    return 2;
}

#ifdef MS_MEASURE  // switches for measurements, in no library that serves
static int g_force_ksi = 0;  // waves along K inside a block (1 = four column waves)
static int g_max_ksb = 0;    // most blocks along K
#else
static constexpr int g_force_ksi = 0, g_max_ksb = 0;
#endif

static SkinnyPlan plan_skinny(int M, int N, int K, bool allow_partials, bool pairs = false) {
    const int NT = skinny_nt(M, N, pairs);
    const int col_waves = ceil_div(N, 16 * NT);
    const int slices = ceil_div(K, KSTEP);  // slices of 128 along K: one wave iteration each
    int want = max(1, min(ceil_div(16 * compute_units(), col_waves), slices));  // waves wanted along K: sixteen a CU in all
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
    if constexpr (EPI != SK_SWIGLU) {
        if (skinny_nt(a.M, a.N) == 1) {
            if (a.M <= 16) return launch_skinny_mt<1, 1, EPI>(a, p, stream);
            return launch_skinny_mt<2, 1, EPI>(a, p, stream);
        }
    }
    if (a.M <= 16) return launch_skinny_mt<1, 2, EPI>(a, p, stream);
    if (a.M <= 32) return launch_skinny_mt<2, 2, EPI>(a, p, stream);
    if constexpr (kHalf) {
        if (skinny_nt(a.M, a.N) == 4) {
            if (a.M <= 48) return launch_skinny_mt<3, 4, EPI>(a, p, stream);
            return launch_skinny_mt<4, 4, EPI>(a, p, stream);
        }
    }
    if (a.M <= 48) return launch_skinny_mt<3, 2, EPI>(a, p, stream);
    return launch_skinny_mt<4, 2, EPI>(a, p, stream);
}


// Waves along K for the product with the norm folded in (all of K inside a block), or 0 if this
// shape is not taken: more than 16 rows, so few columns that one wave would do all of K, or more
// pending sums than the kernel has variants for.
static int plan_skinny_norm(int M, int N, int K, int n_partials) {
    if (M > 16 || n_partials > 6 || K % 8) return 0;
    const int col_waves = ceil_div(N, 32);
    const int slices = ceil_div(K, KSTEP);
    const int want = max(1, min(ceil_div(16 * compute_units(), col_waves), slices));
    if (want == 1) return 0;
    return want > 4 ? 8 : (want > 2 ? 4 : 2);
}

template <int EPI>
static int launch_skinny_norm(SkinnyNormArgs a, int n_partials, hipStream_t stream) {
    const int ksi = plan_skinny_norm(a.M, a.N, a.K, n_partials);
    MS_REQUIRE(ksi > 0, "product with the norm folded in: M=%d N=%d K=%d with %d pending sums is not taken", a.M, a.N, a.K, n_partials);
    MS_REQUIRE(((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.partials) | reinterpret_cast<uintptr_t>(a.norm_w) |
                 reinterpret_cast<uintptr_t>(a.x_out)) & 15) == 0, "product with the norm folded in: operands must be 16-byte aligned");
    MS_REQUIRE(n_partials == 0 || (a.x_out && a.x_out != a.x), "product with the norm folded in: pending sums need another buffer for the stream");
    a.k_per_wave = ceil_div(ceil_div(a.K, KSTEP), ksi) * KSTEP;
    const dim3 grid((unsigned)ceil_div(a.N, 32));
#define MS_SKN(KSI_, NP_)                                                                                     \
    hipLaunchKernelGGL((gemm_skinny_norm_kernel<2, KSI_, EPI, NP_>), grid, dim3(64 * KSI_), 0, stream, a); \
    return check_launch("gemm_skinny_norm")
#define MS_SKN_NP(KSI_)                          \
    switch (n_partials) {                        \
        case 0: MS_SKN(KSI_, 0);                 \
        case 1: MS_SKN(KSI_, 1);                 \
        case 2: MS_SKN(KSI_, 2);                 \
        case 3: MS_SKN(KSI_, 3);                 \
        case 4: MS_SKN(KSI_, 4);                 \
        case 5: MS_SKN(KSI_, 5);                 \
        default: MS_SKN(KSI_, 6);                \
    }
    if (ksi == 8) { MS_SKN_NP(8) }
    if (ksi == 4) { MS_SKN_NP(4) }
    MS_SKN_NP(2)
#undef MS_SKN_NP
#undef MS_SKN
}

}  // namespace ms

using namespace ms;

#ifdef MS_MEASURE
extern "C" void ms_skinny_force_ksi(int ksi) { g_force_ksi = ksi; }
extern "C" void ms_skinny_max_ksb(int ksb) { g_max_ksb = ksb; }
#endif

// Number of partial sums ms_linear_skinny writes for M rows of this N and K (1 = the complete product).
extern "C" int ms_skinny_partials(int M, int N, int K, int allow_partials) { return plan_skinny(M, N, K, allow_partials != 0).ksb; }

// out[ks, M, N] (float) = partial sums of a w^T; ks = ms_skinny_partials(N, K, allow_partials).
extern "C" int ms_linear_skinny(const void* a, const void* w, float* out, int M, int N, int K, int allow_partials,
                                hipStream_t stream) {
    SkinnyArgs args{(const elem_t*)a, (const elem_t*)w, out, M, N, K, 0, 0};
    return launch_skinny<SK_STORE_F32>(args, plan_skinny(M, N, K, allow_partials != 0), stream);
}

// out[M, I] = act(a g^T) * (a u^T), gate and up rows interleaved in blocks of 16 (see ms_linear_swiglu).
extern "C" int ms_linear_swiglu_skinny(const void* a, const void* w, void* out, int M, int I, int K, int act, hipStream_t stream) {
    MS_REQUIRE(act >= 0 && act < ACT_COUNT, "gated product: no activation %d", act);
    const int n = 2 * ceil_div(I, 16) * 16;
    SkinnyArgs args{(const elem_t*)a, (const elem_t*)w, out, M, n, K, 0, I, nullptr, nullptr, nullptr, nullptr, 0, 0.f, act};
    return launch_skinny<SK_SWIGLU>(args, plan_skinny(M, n, K, false, true), stream);
}

// Whether ms_linear_swiglu_scaled_skinny takes this shape, and is the faster of the two forms for it: one
// tile of rows, and so few waves that all of them are on the chip at once (sixteen a CU), each
// waiting for its one trip to memory.  (0.5B gate/up, 304 blocks: 9.9 us tiled with three K steps in flight,
// which multiplies 64-row tiles of padding and ends in a long epilogue; the walk over K there is bound by
// its own instructions, not by memory.)
extern "C" int ms_swiglu_scaled_skinny_takes(int M, int I, int K) {
    if (!kHalf || !kRoundsBeforeTheNormIsSafe || M < 1 || M > 16 || K % 8) return 0;
    const int n = 2 * ceil_div(I, 16) * 16;
    const SkinnyPlan p = plan_skinny(M, n, K, false, true);
    return ceil_div(n, 32 * p.wn) * p.wn * p.ksi <= 16 * compute_units();  // sixteen waves a CU
}

// ms_linear_swiglu_skinny for rows that came in multiplied by a norm's weight only: both products of a row are
// divided by the row's root mean square, 1 / sqrt(sum_p row_ss[p, row] / K + eps), before the activation.
extern "C" int ms_linear_swiglu_scaled_skinny(const void* a, const float* row_ss, int ss_parts, float eps, const void* w, void* out,
                                              int M, int I, int K, int act, hipStream_t stream) {
    MS_REQUIRE(act >= 0 && act < ACT_COUNT, "gated product: no activation %d", act);
    MS_REQUIRE(ms_swiglu_scaled_skinny_takes(M, I, K), "few-rows gated product with row factors: M=%d I=%d K=%d is not taken", M, I, K);
    MS_REQUIRE(row_ss && ss_parts >= 1, "few-rows gated product with row factors: the rows' sums of squares are missing");
    const int n = 2 * ceil_div(I, 16) * 16;
    SkinnyArgs args{(const elem_t*)a, (const elem_t*)w, out, M, n, K, 0, I, nullptr, nullptr, nullptr, row_ss, ss_parts, eps, act};
    return launch_skinny<SK_SWIGLU>(args, plan_skinny(M, n, K, false, true), stream);
}

// Whether ms_linear_norm_skinny / ms_linear_swiglu_norm_skinny should be given this shape.
// Every block reads the stream and its pending sums for itself, which pays only while there is little
// to read (measured: with nothing pending it saves a microsecond or two over the norm's own launch;
// with one pending sum it breaks even at four rows; with five it costs twice as much).
extern "C" int ms_skinny_norm_takes(int M, int N, int K, int n_partials) {
    if (!kRoundsBeforeTheNormIsSafe) return 0;  // the kernel rounds x * norm_w before it knows the row's root mean square
    if (n_partials > 1 || (n_partials == 1 && M > 4)) return 0;
    return plan_skinny_norm(M, N, K, n_partials) > 0;
}

// out[M, N] (float) = rmsnorm(x + sum partials; norm_w, eps) w^T, and x_out = x + sum partials (if any are pending).
extern "C" int ms_linear_norm_skinny(const float* x, const float* partials, int n_partials, int T, const float* norm_w, float eps,
                                     float* x_out, const void* w, float* out, int M, int N, int K, hipStream_t stream) {
    SkinnyNormArgs a{x, partials ? partials : x, (size_t)T * K, norm_w, n_partials ? x_out : nullptr, (const elem_t*)w, out, M, N, K, 0, 0, eps};
    return launch_skinny_norm<SK_STORE_F32>(a, n_partials, stream);
}

// out[M, I] = act(h g^T) * (h u^T) with h = rmsnorm(x + sum partials), gate and up rows interleaved in blocks of 16.
extern "C" int ms_linear_swiglu_norm_skinny(const float* x, const float* partials, int n_partials, int T, const float* norm_w,
                                            float eps, float* x_out, const void* w, void* out, int M, int I, int K, int act,
                                            hipStream_t stream) {
    MS_REQUIRE(act >= 0 && act < ACT_COUNT, "gated product: no activation %d", act);
    const int n = 2 * ceil_div(I, 16) * 16;
    SkinnyNormArgs a{x, partials ? partials : x, (size_t)T * K, norm_w, n_partials ? x_out : nullptr, (const elem_t*)w, out, M, n, K, 0, I, eps, act};
    return launch_skinny_norm<SK_SWIGLU>(a, n_partials, stream);
}

// x[M, N] += a w^T for a product whose K lies inside one block (ms_skinny_partials(..., 1) == 1): the
// stream takes the sum in the product's epilogue and nothing stays pending.
extern "C" int ms_linear_residual_skinny(const void* a, const void* w, float* x, int M, int N, int K, hipStream_t stream) {
    const SkinnyPlan p = plan_skinny(M, N, K, true);
    MS_REQUIRE(p.ksb == 1, "few-rows product into the stream: K=%d is cut over %d blocks", K, p.ksb);
    SkinnyArgs args{(const elem_t*)a, (const elem_t*)w, x, M, N, K, 0, 0};
    return launch_skinny<SK_RESIDUAL>(args, p, stream);
}

// Column waves of ms_linear_residual_prenorm_skinny for this shape (the first size of its ss_part), or 0 if the
// shape is not taken: more than 32 rows, or a K that is cut over several blocks.
extern "C" int ms_skinny_prenorm_parts(int M, int N, int K) {
    if (!kRoundsBeforeTheNormIsSafe) return 0;  // hn = x * norm_w is rounded before the division
    if (M < 1 || M > 32 || K % 8) return 0;
    const SkinnyPlan p = plan_skinny(M, N, K, true);
    return p.ksb == 1 ? ceil_div(N, 16 * skinny_nt(M, N)) : 0;
}

// x[M, N] += a w^T as ms_linear_residual_skinny does, and beside it hn[M, N] = x * norm_w in the element type and
// ss_part[parts, M], whose sum over parts is the rows' sums of squares of x (parts = ms_skinny_prenorm_parts).
extern "C" int ms_linear_residual_prenorm_skinny(const void* a, const void* w, float* x, const float* norm_w, void* hn, float* ss_part,
                                                 int M, int N, int K, hipStream_t stream) {
    MS_REQUIRE(ms_skinny_prenorm_parts(M, N, K) > 0, "few-rows product that prepares the norm: M=%d N=%d K=%d is not taken", M, N, K);
    MS_REQUIRE(norm_w && hn && ss_part, "few-rows product that prepares the norm: its outputs are missing");
    const SkinnyPlan p = plan_skinny(M, N, K, true);
    SkinnyArgs args{(const elem_t*)a, (const elem_t*)w, x, M, N, K, 0, 0, norm_w, (elem_t*)hn, ss_part};
    if (skinny_nt(M, N) == 1) {
        if (M <= 16) return launch_skinny_mt<1, 1, SK_RESIDUAL_PRENORM>(args, p, stream);
        return launch_skinny_mt<2, 1, SK_RESIDUAL_PRENORM>(args, p, stream);
    }
    if (M <= 16) return launch_skinny_mt<1, 2, SK_RESIDUAL_PRENORM>(args, p, stream);
    return launch_skinny_mt<2, 2, SK_RESIDUAL_PRENORM>(args, p, stream);
}
