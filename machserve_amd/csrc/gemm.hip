// out[M, N] = A[M, K] * W[N, K]^T on the matrix cores, with the epilogue fused:
// bias add, residual accumulation into the 32-bit stream, or SiLU(gate) * up.
//
// Role in the reference: hipBLAS Sgemm / GemmEx plus separate add_bias, add and silu_mul
// kernels (crates/mach-model/src/kernels.rs:5772-5798, 6416-6455, 131-160).
//
// Both operands are contiguous along K, so a 16x32 MFMA fragment of either is "row
// l % 16, elements (l / 16) * 8 .. + 8".  Two LDS buffers, one barrier per K step.  LDS has 64 banks
// of 4 bytes; the 16-byte fragment reads of a wave are free of bank conflicts when the row pitch is
// 32 modulo 64 bytes (measured: pitches of 80 or 144 bytes take twice as long), or, with unpadded
// rows of 128 bytes, when chunk c of row r lies at position c ^ (r & 7).
// bfloat16 with K steps of 64: tiles go global -> LDS directly (global_load_lds_dwordx4, a wave's
// 64 lanes fill 1 KB = 8 unpadded rows in lane order, so the swizzle is applied to the global
// address), and the next step's tile is in flight while this one is multiplied; only a partial last
// step goes through registers, where what lies beyond K is masked.  The 32-bit build and K steps of
// 32 go global -> registers -> LDS (padded rows).
// Every output element is the sum over K in steps of 32 in ascending order whatever the
// tile shape or the number of rows, so a row's result does not depend on its batch.
#include <type_traits>

#include "common.cuh"

namespace ms {

#ifdef MS_ELEM_HALF
constexpr int EPC = 8;   // elements per 16-byte chunk
constexpr int KPAD = 16;  // row padding in elements: rows of 96 (BK 32) or 160 (BK 64) bytes
#else
constexpr int EPC = 4;
constexpr int KPAD = 8;  // rows of 160 bytes (BK 32)
#endif

enum EpiKind { EPI_STORE_F32 = 0, EPI_STORE_ELEM = 1, EPI_RESIDUAL = 2, EPI_SWIGLU = 3, EPI_QKV_ROPE = 4 };

struct EpiArgs {
    void* out;          // [M, ldo]
    const float* bias;  // [N] or null
    int ldo;
    int n_out;          // SWIGLU: number of output columns (intermediate size)
    int k_per_split;    // K range of one blockIdx.y slice (multiple of 32); K itself without split
    size_t split_stride;  // STORE_F32 with gridDim.y > 1: elements between the slices' outputs
    // a factor a row for the finished sums (the RMS norm of rows that came in multiplied by the norm's weight only):
    // 1 / sqrt(sum over parts of row_ss[part, row] / K + ss_eps)
    const float* row_ss;  // [ss_parts, M] or null
    int ss_parts;
    float ss_eps;
    int act;            // SWIGLU: the activation on the gate (GateActivation)
    // QKV_ROPE: the columns are H query heads, KV key heads and KV value heads of the tile's width; bias added, queries
    // and keys rotated by the rows' angles (pairs (j, j + half a head)), queries to `out` [M, H * hd], keys and values
    // into their pages
    const float* rope_cs;  // [M, hd / 2, 2]: cosine and sine of each row's angles
    const int* slot_map;   // [M]: page * ps + offset of each row's key and value, or negative: not written
    elem_t* kpool;         // [pages, KV, ps, hd]
    elem_t* vpool;         // [pages, KV, hd, ps]
    int H, KV, ps;
};

template <int BM, int BN, int WM, int WN, int BK, int EPI, int STAGES = 2, bool SCALED = false>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(const elem_t* __restrict__ A, const elem_t* __restrict__ W,
                                                   int M, int N, int K, EpiArgs ep) {
    static_assert(WM * WN == 4 || WM * WN == 8, "four waves, or eight for the widest tiles");
    constexpr int NT = 64 * WM * WN;  // threads of the block
    arguments_now(A, W, M, N, K, ep.out, ep.bias, ep.ldo, ep.n_out, ep.k_per_split, ep.split_stride);
    if constexpr (SCALED) arguments_now(ep.row_ss, ep.ss_parts, ep.ss_eps);
    static_assert(BK % 32 == 0, "K step in MFMA steps of 32");
#ifdef MS_ELEM_HALF
    constexpr bool DIRECT = BK == 64;
#else
    constexpr bool DIRECT = false;
#endif
    constexpr int LDS_LD = DIRECT ? BK : BK + KPAD;
    constexpr int CPR = BK / EPC;  // chunks per tile row
    // where chunk `chunk` of tile row `row` lies in a buffer
    auto at = [](int row, int chunk) { return row * LDS_LD + (DIRECT ? (chunk ^ (row & 7)) : chunk) * EPC; };
    constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
    constexpr int A_CHUNKS = BM * CPR / NT, W_CHUNKS = BN * CPR / NT;
    static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "tile loads divide over the block");
    static_assert(NT == 256 || !SCALED, "the row factors' shares are dealt to four waves");
    static_assert(STAGES == 2 || DIRECT, "more than two LDS buffers only with direct loads");
    static_assert(!SCALED || (STAGES > 2 && EPI == EPI_SWIGLU), "row factors: built for the gated product with several steps in flight");
    static_assert(256 % BM == 0 || !SCALED, "threads are dealt to the rows");
    __shared__ float ss_q[SCALED ? 256 / BM : 1][SCALED ? BM : 1];  // the rows' sums of squares, in 256 / BM interleaved shares
    float ss_v[SCALED ? 8 : 1];
    int ss_r = 0;
    __shared__ __attribute__((aligned(16))) elem_t As[STAGES][BM * LDS_LD];
    __shared__ __attribute__((aligned(16))) elem_t Ws[STAGES][BN * LDS_LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int tiles_m = ceil_div(M, BM);
    const int m0 = (blockIdx.x % tiles_m) * BM, n0 = (blockIdx.x / tiles_m) * BN;
    const int r16 = lane & 15, grp = lane >> 4;

    const int split = blockIdx.y;
    const int k_end = min(K, (split + 1) * ep.k_per_split);
    // Loads are unconditional, on one straight path: a row beyond the operand reads the last row
    // (its results are never stored), and only the last K step of a slice, if it is a partial one,
    // masks what lies beyond the slice.
    u32x4 ra[A_CHUNKS], rw[W_CHUNKS];
    const elem_t* pa[A_CHUNKS];
    const elem_t* pw[W_CHUNKS];
    // Thread t owns position (t + i * NT) % CPR of tile row (t + i * NT) / CPR; with swizzled rows that
    // position holds another chunk of K, the same one for every i (NT / CPR rows on is a multiple of 8).
    const int my_chunk = DIRECT ? (tid % CPR) ^ ((tid / CPR) & 7) : tid % CPR;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        const int c = tid + i * NT;
        pa[i] = A + (size_t)min(m0 + c / CPR, M - 1) * K + my_chunk * EPC;
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
        const int c = tid + i * NT;
        pw[i] = W + (size_t)min(n0 + c / CPR, N - 1) * K + my_chunk * EPC;
    }
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) ra[i] = *reinterpret_cast<const u32x4*>(pa[i] + k0);
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) rw[i] = *reinterpret_cast<const u32x4*>(pw[i] + k0);
    };
    auto load_global_tail = [&](int k0) {
        const int kk = k0 + my_chunk * EPC;  // the same K chunk for all of a thread's loads
        const bool in = kk < k_end;
        const uint32_t keep = opaque(in ? 0xffffffffu : 0u);
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            u32x4 v = *reinterpret_cast<const u32x4*>(in ? pa[i] + k0 : A);  // the operand's start when beyond the slice
            ra[i] = (u32x4){v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            u32x4 v = *reinterpret_cast<const u32x4*>(in ? pw[i] + k0 : W);
            rw[i] = (u32x4){v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + i * NT, row = c / CPR;
            *reinterpret_cast<u32x4*>(&As[buf][at(row, my_chunk)]) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + i * NT, row = c / CPR;
            *reinterpret_cast<u32x4*>(&Ws[buf][at(row, my_chunk)]) = rw[i];
        }
    };
#ifdef MS_ELEM_HALF
    // One K step of both tiles straight into LDS buffer `buf`: lane l of a wave's load lands at the wave's
    // base + 16 l.  Written in assembly: of a load that it knows to write LDS the compiler makes every later
    // LDS read wait (vmcnt(0)), and nothing would be in flight during the multiplications; the waits are
    // explicit instead (`step_barrier`).
    auto load_direct = [&](int k0, int buf) {
        auto issue = [](const elem_t* g, const elem_t* l) {
            const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)l);
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(base) : "memory", "m0");
        };
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) issue(pa[i] + k0, &As[buf][(i * NT + wave * 64) * EPC]);
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) issue(pw[i] + k0, &Ws[buf][(i * NT + wave * 64) * EPC]);
    };
#endif
    // End of a K step: this wave's loads and LDS accesses have completed, then everybody's.
    auto step_barrier = [&]() {
        if constexpr (DIRECT) {
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        } else {
            __syncthreads();
        }
    };

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // a slice of K per blockIdx.y: partial sums that the consumer adds in slice order
    const int k_begin = split * ep.k_per_split;
    const int nk = ceil_div(k_end - k_begin, BK);
    const bool partial = (k_end - k_begin) % BK != 0;  // the last step is a partial one
    auto multiply = [&](int buf) {
#pragma unroll
        for (int kk = 0; kk < BK; kk += 32) {
            Frag fa[TM], fb[TN];
            if constexpr (DIRECT) {
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[i] = frag_load(&As[buf][at(wm * (BM / WM) + i * 16 + r16, kk / EPC + grp)]);
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[j] = frag_load(&Ws[buf][at(wn * (BN / WN) + j * 16 + r16, kk / EPC + grp)]);
            } else {
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[i] = frag_load(&As[buf][(wm * (BM / WM) + i * 16 + r16) * LDS_LD + kk + grp * 8]);
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[j] = frag_load(&Ws[buf][(wn * (BN / WN) + j * 16 + r16) * LDS_LD + kk + grp * 8]);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) mma_16x16x32(acc[i][j], fa[i], fb[j]);
        }
    };
    if constexpr (DIRECT && STAGES > 2) {
#ifdef MS_ELEM_HALF
        // A block that is alone on its CU (few tiles: one tile of rows under a weight of a few hundred column
        // tiles) has nobody to hide its loads behind, and with one step in flight every step costs a trip to
        // memory.  Here STAGES - 1 steps are in flight: the loads of step kt + STAGES - 1 go out before step
        // kt is multiplied, and the step's end waits only for the loads of step kt + 1 (a wave's loads
        // complete in order, so "all but the last (STAGES - 2) steps' loads" is a count).  The launcher
        // gives this variant whole K steps only.
        constexpr int PER_STEP = A_CHUNKS + W_CHUNKS;
        static_assert(PER_STEP * (STAGES - 2) <= 63, "the wait count is a 6-bit field");
        for (int s = 0; s < STAGES - 1; ++s)
            if (s < nk) load_direct(k_begin + s * BK, s);
        if constexpr (SCALED) {
            // The rows' sums of squares, asked for behind the first K steps and not used before the last one is
            // multiplied: what they are made of was written by the kernel before this one, a slow read that the
            // walk over K covers.  Thread (row, q) takes parts q, q + 256 / BM, ...
            ss_r = min(m0 + tid % BM, M - 1);
#pragma unroll
            for (int u = 0; u < 8; ++u) ss_v[u] = ep.row_ss[(size_t)min(tid / BM + u * (256 / BM), ep.ss_parts - 1) * M + ss_r];
        }
        // the first step's loads: the earliest of up to STAGES - 1 steps' loads
        __builtin_amdgcn_sched_barrier(0);
        if (nk >= STAGES - 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER_STEP * (STAGES - 2)) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        for (int kt = 0; kt < nk; ++kt) {
            const bool more = kt + STAGES - 1 < nk;
            if (more) load_direct(k_begin + (kt + STAGES - 1) * BK, (kt + STAGES - 1) % STAGES);
            multiply(kt % STAGES);
            __builtin_amdgcn_sched_barrier(0);
            // towards the end fewer steps are in flight behind step kt + 1: wait for everything
            if (more) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(PER_STEP * (STAGES - 2)) : "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (SCALED) {
            constexpr int Q = 256 / BM;
            const int q = tid / BM;
            float ssum = 0.f;
#pragma unroll
            for (int u = 0; u < 8; ++u) ssum += q + u * Q < ep.ss_parts ? ss_v[u] : 0.f;
            for (int p = q + 8 * Q; p < ep.ss_parts; p += Q) ssum += ep.row_ss[(size_t)p * M + ss_r];  // more than 8 * Q parts: a very wide stream
            ss_q[q][tid % BM] = ssum;
            __syncthreads();
        }
#endif
    } else if constexpr (DIRECT) {
#ifdef MS_ELEM_HALF
        if (nk == 1 && partial) {
            load_global_tail(k_begin);
            store_lds(0);
        } else {
            load_direct(k_begin, 0);
        }
        step_barrier();
        for (int kt = 0; kt < nk; ++kt) {
            const int buf = kt & 1;
            // the next step: a whole one straight into the other buffer, a partial one into registers
            const bool tail_next = kt + 2 == nk && partial;
            if (kt + 1 < nk) {
                if (tail_next) load_global_tail(k_begin + (kt + 1) * BK);
                else load_direct(k_begin + (kt + 1) * BK, buf ^ 1);
            }
            multiply(buf);
            if (tail_next) store_lds(buf ^ 1);
            step_barrier();
        }
#endif
    } else {
        if (nk == 1 && partial) load_global_tail(k_begin);
        else load_global(k_begin);
        store_lds(0);
        __syncthreads();
        for (int kt = 0; kt < nk; ++kt) {
            const int buf = kt & 1;
            if (kt + 2 < nk || (kt + 2 == nk && !partial)) load_global(k_begin + (kt + 1) * BK);
            else if (kt + 1 < nk) load_global_tail(k_begin + (kt + 1) * BK);
            multiply(buf);
            if (kt + 1 < nk) store_lds(buf ^ 1);
            __syncthreads();
        }
    }

    // Epilogue.  Lane holds rows grp * 4 + e of column r16 in each 16x16 tile: sixteen lanes write
    // sixteen consecutive elements of a row.  (Four consecutive columns a lane - transposed tiles,
    // one 8-byte store - measured slower: neighbouring lanes then write to different rows, which
    // the memory pipeline does not merge.)  A tile wholly inside the output stores without checks:
    // sixty-four guarded stores cost a third of a whole 2,048 x 9,728 x 896 product.
    const int row_base = m0 + wm * (BM / WM) + grp * 4;
    const int col_base = n0 + wn * (BN / WN) + r16;
    const bool whole = m0 + BM <= M && n0 + BN <= N && (EPI != EPI_SWIGLU || (n0 + BN) / 2 <= ep.n_out);
    // A tile at the lower edge of an output whose rows come in whole groups of sixteen (a decode step
    // of 48 requests in a 64-row tile) skips the groups beyond the last row and stores the others
    // without checks as well.
    auto emit = [&](auto checked, auto row_groups) {
        constexpr bool CHECKED = decltype(checked)::value, ROW_GROUPS = decltype(row_groups)::value;
        if constexpr (EPI == EPI_SWIGLU) {
            static_assert(TN % 2 == 0, "gate and up tiles come in pairs");
            elem_t* out = reinterpret_cast<elem_t*>(ep.out);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                if (ROW_GROUPS && m0 + wm * (BM / WM) + i * 16 >= M) continue;
                float f[4] = {1.f, 1.f, 1.f, 1.f};  // SCALED: of the rows this lane holds
                if constexpr (SCALED) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int lr = wm * (BM / WM) + i * 16 + grp * 4 + e;
                        float ssum = 0.f;
#pragma unroll
                        for (int qq = 0; qq < 256 / BM; ++qq) ssum += ss_q[qq][lr];
                        f[e] = 1.0f / sqrtf(ssum / (float)K + ep.ss_eps);
                    }
                }
#pragma unroll
                for (int j = 0; j < TN; j += 2) {
                    const int col = (col_base + j * 16 - r16) / 2 + r16;  // tiles 2t, 2t+1 -> output tile t
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = row_base + i * 16 + e;
                        if (CHECKED && !(row < M && col < ep.n_out)) continue;
                        float gv = acc[i][j][e], uv = acc[i][j + 1][e];
                        if constexpr (SCALED) {
                            gv *= f[e];
                            uv *= f[e];
                        }
                        out[(size_t)row * ep.ldo + col] = from_f32<elem_t>(gate_activation(gv, ep.act) * uv);
                    }
                }
            }
        } else if constexpr (EPI == EPI_QKV_ROPE) {
            // The tile's columns are one head (the launcher sees to it), and a wave holds all of them: lane (r16, grp)
            // has columns r16 + 16 j of rows grp * 4 + e, so both elements of a pair (j, j + TN / 2) are its own.
            static_assert(WN == 1 && TN % 2 == 0, "a wave holds whole heads");
            constexpr int HT = TN / 2, hd = BN, half = BN / 2;
            const int head = n0 / hd;
            const int kind = head < ep.H ? 0 : (head < ep.H + ep.KV ? 1 : 2);  // query, key or value head
            float bias_j[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) bias_j[j] = ep.bias ? ep.bias[n0 + j * 16 + r16] : 0.f;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = row_base + i * 16 + e;
                    if (row >= M) continue;
                    float x[TN];
#pragma unroll
                    for (int j = 0; j < TN; ++j) x[j] = bias_j[j] + acc[i][j][e];
                    if (kind < 2) {
                        const float* cs = ep.rope_cs + (size_t)row * (2 * half);
#pragma unroll
                        for (int j = 0; j < HT; ++j) {
                            const float c = cs[2 * (j * 16 + r16)], sn = cs[2 * (j * 16 + r16) + 1];
                            const float x0 = x[j], x1 = x[j + HT];
                            x[j] = x0 * c - x1 * sn;
                            x[j + HT] = x0 * sn + x1 * c;
                        }
                    }
                    if (kind == 0) {
                        elem_t* o = reinterpret_cast<elem_t*>(ep.out) + ((size_t)row * ep.H + head) * hd + r16;
#pragma unroll
                        for (int j = 0; j < TN; ++j) o[j * 16] = from_f32<elem_t>(x[j]);
                    } else {
                        const int slot = ep.slot_map[row];
                        if (slot < 0) continue;
                        const int page = slot / ep.ps, off = slot - page * ep.ps;
                        if (kind == 1) {
                            elem_t* o = ep.kpool + (((size_t)page * ep.KV + (head - ep.H)) * ep.ps + off) * hd + r16;
#pragma unroll
                            for (int j = 0; j < TN; ++j) o[j * 16] = from_f32<elem_t>(x[j]);
                        } else {
                            elem_t* o = ep.vpool + (((size_t)page * ep.KV + (head - ep.H - ep.KV)) * hd + r16) * ep.ps + off;
#pragma unroll
                            for (int j = 0; j < TN; ++j) o[(size_t)(j * 16) * ep.ps] = from_f32<elem_t>(x[j]);
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                if (ROW_GROUPS && m0 + wm * (BM / WM) + i * 16 >= M) continue;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int col = col_base + j * 16;
                    const float b = ep.bias ? ep.bias[min(col, N - 1)] : 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = row_base + i * 16 + e;
                        if (CHECKED && !(row < M && col < N)) continue;
                        const size_t o = (size_t)row * ep.ldo + col;
                        const float v = acc[i][j][e] + b;
                        if constexpr (EPI == EPI_STORE_F32) reinterpret_cast<float*>(ep.out)[split * ep.split_stride + o] = v;
                        else if constexpr (EPI == EPI_STORE_ELEM) reinterpret_cast<elem_t*>(ep.out)[o] = from_f32<elem_t>(v);
                        else reinterpret_cast<float*>(ep.out)[o] += v;  // residual stream, 32-bit
                    }
                }
            }
        }
    };
    const bool cols_whole = n0 + BN <= N && (EPI != EPI_SWIGLU || (n0 + BN) / 2 <= ep.n_out);
    if (whole) emit(std::false_type{}, std::false_type{});
    else if (cols_whole && M % 16 == 0) emit(std::false_type{}, std::true_type{});
    else emit(std::true_type{}, std::false_type{});
}

#ifdef MS_MEASURE  // switches for measurements, in no library that serves
static int g_gemm_config = 0;  // 0: chosen by shape; else a fixed tile
#else
static constexpr int g_gemm_config = 0;
#endif

template <int EPI>
static int launch_gemm(const elem_t* A, const elem_t* W, int M, int N, int K, EpiArgs ep, hipStream_t stream,
                       int nsplit = 1) {
    MS_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: empty problem M=%d N=%d K=%d", M, N, K);
    MS_REQUIRE(K % 8 == 0, "gemm: the reduction size K=%d must be a multiple of 8", K);
    MS_REQUIRE((reinterpret_cast<uintptr_t>(A) & 15) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0,
               "gemm: operands must be 16-byte aligned");
    MS_REQUIRE(nsplit >= 1 && (nsplit == 1 || EPI == EPI_STORE_F32), "gemm: %d K slices need the float store", nsplit);
    // slices of a multiple of 64; rounding up may leave fewer slices than asked for
    ep.k_per_split = ceil_div(ceil_div(K, nsplit), 64) * 64;
    ep.split_stride = (size_t)M * N;
    const unsigned ns = (unsigned)ceil_div(K, ep.k_per_split);
    MS_REQUIRE(nsplit == 1 || (int)ns == nsplit, "gemm: %d K slices asked for, %u fit", nsplit, ns);
#define MS_GEMM_DEEP(BM_, BN_, WM_, WN_, BK_, ST_)                                                                         \
    do {                                                                                                                  \
        const long nb = (long)ceil_div(M, BM_) * ceil_div(N, BN_);                                                        \
        hipLaunchKernelGGL((gemm_kernel<BM_, BN_, WM_, WN_, BK_, EPI, ST_>), dim3((unsigned)nb, ns), dim3(64 * WM_ * WN_), 0, stream, \
                           A, W, M, N, K, ep);                                                                            \
        return check_launch("gemm " #BM_ "x" #BN_ "x" #BK_ " deep");                                                      \
    } while (0)
#define MS_GEMM(BM_, BN_, WM_, WN_, BK_)                                                                              \
    do {                                                                                                              \
        const long nb = (long)ceil_div(M, BM_) * ceil_div(N, BN_);                                                    \
        hipLaunchKernelGGL((gemm_kernel<BM_, BN_, WM_, WN_, BK_, EPI>), dim3((unsigned)nb, ns), dim3(64 * WM_ * WN_), 0, stream, \
                           A, W, M, N, K, ep);                                                                        \
        return check_launch("gemm " #BM_ "x" #BN_ "x" #BK_);                                                          \
    } while (0)
#ifdef MS_ELEM_HALF
    const int forced = g_gemm_config;
    if (forced == 1) MS_GEMM(128, 128, 2, 2, 32);
    if (forced == 2) MS_GEMM(128, 128, 2, 2, 64);
    if (forced == 5) MS_GEMM(128, 64, 2, 2, 64);
    if (forced == 6) MS_GEMM(64, 64, 2, 2, 64);
    const bool whole_steps = ep.k_per_split % 64 == 0 && K % 64 == 0;
    if (forced == 8 && whole_steps) MS_GEMM_DEEP(64, 64, 2, 2, 64, 4);
    if (forced == 9) MS_GEMM(256, 256, 2, 4, 64);
    // The largest tile that still gives every CU of the chip a block or two, with K steps of 64 (half
    // the barriers of steps of 32).  Measured on M = 512..8192 of the 0.5B shapes; larger tiles under
    // four waves (256x128) lose: their accumulators no longer fit the registers of two blocks a CU.
    // two 128x128 blocks a CU are a round of the chip (512 on 256 CUs); a tile is taken when its blocks fill
    // six tenths of a round
    const long round_blocks = 2L * compute_units(), enough = round_blocks * 300 / 512;
    if (M > 64 && (ns == 1 || K >= 16384) && ep.k_per_split >= 128 && forced == 0) {
        // Tiles of 256x256 under eight waves (each 128 rows by 64 columns: 128 accumulator registers, 220 in all, two
        // waves a SIMD; 128 KB of LDS: one block a CU) bring half the bytes of two 128x128 tiles from the L2 into the CUs,
        // which is what bounds the large products (every variant of the 128x128 loop pulls 13 to 15 TB/s).  They pay
        // where the last of their rounds of one block a CU is well filled: measured against the choice below at the
        // 0.5B, 1.5B and 7B layer sizes with 1,024 to 8,192 rows, +4 to +18 % from 0.72 of the rounds' blocks upwards
        // (7B gate/up at 2,048 rows 604 -> 511 us, at 8,192 rows 2,167 -> 1,818 us = 1.22 PFLOP/s; 7B down at 4,096
        // rows 588 -> 496), -15 to -44 % below 0.63; a short K (the 0.5B model's 896: fourteen steps between a tile's
        // start and its 256x256 stores) wants the rounds fuller (0.95: +16 %; 0.89 - 1,536 and 3,072 rows of the 0.5B
        // gate/up product - +24 and +7 %; 0.79: -5 to +6 %; 0.59: -20 %).  Three LDS stages
        // (256x128, 128x256), four of K = 32 (256x256: 1.13 against 1.22 PFLOP/s) and four waves of 128x128 each with
        // their sums in the accumulation registers (1.06) were slower than this.
        // (with K cut over `ns` blocks - a very long K under few tiles, see plan_tiled_splits - the slices fill the round)
        const long t256 = (long)ceil_div(M, 256) * ceil_div(N, 256) * ns, cus = compute_units();
        const long rounds = ceil_div(t256, cus);
        if (t256 * 100 >= rounds * cus * (K >= 1536 ? 72 : 85)) MS_GEMM(256, 256, 2, 4, 64);
    }
    if (M > 64) {
        const long b128 = (long)ceil_div(M, 128) * ceil_div(N, 128), b12864 = (long)ceil_div(M, 128) * ceil_div(N, 64);
        // The chip holds a round of such blocks at a time and a round that is nearly empty takes as long as a full one:
        // the time is rounds times the tile's width.  Where tiles a quarter wider save more in rounds than they
        // cost, they are taken (0.5B gate/up product at 2,048 rows: 1,216 tiles of 128x128 are two rounds and three
        // eighths, 976 of 128x160 two rounds less a twentieth: 55 -> 45 us).  Tiles of 128x96 save rounds by the
        // same count but lose more in themselves (8,192 rows: 16.3 against 15.7 ms for the whole prompt).
        if (ns == 1 && ep.k_per_split >= 128 && b128 >= enough) {
            const long rounds128 = ceil_div(b128, round_blocks), rounds160 = ceil_div((long)ceil_div(M, 128) * ceil_div(N, 160), round_blocks);
            if (rounds160 * 160 < rounds128 * 128) MS_GEMM(128, 160, 4, 1, 64);
        }
        if (b128 * ns >= enough) {
            if (ep.k_per_split >= 128) MS_GEMM(128, 128, 2, 2, 64);
            MS_GEMM(128, 128, 2, 2, 32);
        }
        if (b12864 * ns >= enough) {
            if (ep.k_per_split >= 128) MS_GEMM(128, 64, 2, 2, 64);
            MS_GEMM(128, 64, 2, 2, 32);
        }
    }
    // At most two blocks a CU, each a chain of K steps: four LDS buffers keep three steps in flight (0.5B
    // gate/up product at 64 rows, 152 blocks of 14 steps: 10.5 -> 7.8 us; 1.5B: 23.7 -> 21.1; with more
    // blocks than that the blocks hide each other's loads and the two-buffer kernel is as fast).
    if ((long)ceil_div(M, 64) * ceil_div(N, 64) * ns <= round_blocks && whole_steps && ep.k_per_split >= 256) MS_GEMM_DEEP(64, 64, 2, 2, 64, 4);
    MS_GEMM(64, 64, 2, 2, 64);
#else
    MS_GEMM(64, 64, 2, 2, 32);
#endif
#undef MS_GEMM
#undef MS_GEMM_DEEP
}

// K slices for a product whose consumer adds partial sums: enough 128x128 blocks to fill the chip,
// at least 512 of K each.  The 32-bit build never slices: its sums keep one order.
#ifdef MS_MEASURE
static int g_force_splits = 0;
#else
static constexpr int g_force_splits = 0;
#endif

static int plan_tiled_splits(int M, int N, int K) {
#ifdef MS_ELEM_HALF
    const long b128 = (long)ceil_div(M, 128) * ceil_div(N, 128);
    const long round_blocks = 2L * compute_units();  // two 128x128 blocks a CU
    // A very long K under few output tiles (the 7B down projection: K = 18,944, 14 column tiles of 256): tiles of 256x256
    // bring half the bytes of 128x128 tiles from the L2, but one or two thousand rows of them do not fill the chip's round of
    // one block a CU; with K cut in two to four they do, and the norm that follows adds the slices.  Measured with that
    // norm: 2,048 rows 374 -> 330 us in two slices (320 in four), 1,024 rows 198 -> 158 in four; shorter K (the 1.5B down
    // projection, 8,960) and the 0.5B sizes lose by it, and from 4,096 rows on the uncut tiles fill the round themselves.
    if (M > 64 && K >= 16384 && g_force_splits == 0) {
        const long t256 = (long)ceil_div(M, 256) * ceil_div(N, 256), cus = compute_units();
        if (t256 * 100 < 72 * cus)
            for (int sl = 2; sl <= 4; ++sl)
                if (t256 * sl * 100 >= 85 * cus && t256 * sl <= cus) return ceil_div(K, ceil_div(ceil_div(K, sl), 64) * 64);
    }
    if (b128 >= round_blocks * 300 / 512 && g_force_splits == 0) return 1;
    // More than six slices cost more in the consumer's sums than they gain here (with very few tiles - a
    // portion of a few hundred rows - slices of 256 still pay).  With few rows the partial sums are small
    // and the weight is all the traffic: a long K is then cut up to 16 times (7B down projection at 64
    // rows: 49 us with 6 slices, 33 with 12 to 16).
    // (measured again at 33 and 64 rows of the three layer sizes: 1.5B down projection, K = 8,960, 9.0 us in 10
    // slices, 10.0 in 16, and its consumer sums fewer planes)
    // (and again once few blocks ran with four LDS buffers in turn: with its 56 column tiles in four slices the 7B down
    // projection stays within a round of blocks and takes that kernel, 30 to 34 us at 16 to 64 rows with the sum of its
    // planes, against 31 to 36 in thirteen; the 7B decode step at 16 to 64 requests 0.5 to 1 % shorter)
    const int most = M <= 128 ? (K >= 16384 ? (M <= 64 ? 4 : 16) : (K >= 8192 ? 10 : 8)) : 6;
    // (a handful of tiles under few rows - a small projection in a decode step of 33 to 64 requests:
    // slices of 128, or the step's few blocks leave the chip idle)
    // (from K = 1,536 on slices of 256, which run with four LDS buffers in turn: 1.5B output projection at 64
    // rows 5.1 us in 6 slices, 5.5 in 8)
    const int shortest = b128 <= 16 && M <= 128 ? (K >= 1536 ? 256 : 128) : (b128 <= 32 ? 256 : 512);
    const int limit = max(1, min(K / shortest, most));
    // The chip holds two of the 128x128 blocks a CU at a time (512 on 256 CUs), and a last round that is nearly
    // empty takes as long as a full one: the fewest slices that fill their rounds to 70 %, else the
    // count that fills them best (1.5B down projection at 2,048 rows, 192 tiles: 3 slices make a
    // full round and an eighth, 118 us; 2 slices one round three quarters full, 97 us).
    int want = 1;
    double best = 0.0;
    for (int sl = 1; sl <= limit; ++sl) {
        const long blocks = b128 * sl, rounds = ceil_div(blocks, round_blocks);
        const double filled = (double)blocks / (double)(rounds * round_blocks);
        if (filled > best + 1e-9) {
            best = filled;
            want = sl;
        }
        if (filled >= 0.7) break;
    }
    if (g_force_splits > 0) want = g_force_splits;
    // what the launcher's rounding of a slice to a multiple of 64 really yields
    const int k_per_split = ceil_div(ceil_div(K, want), 64) * 64;
    return ceil_div(K, k_per_split);
#else
    (void)M; (void)N; (void)K;
    return 1;
#endif
}

}  // namespace ms

using namespace ms;

// out[M, N] = a[M, K] w[N, K]^T (+ bias[N]); out is float when out_f32 != 0, else the element type.
extern "C" int ms_linear(const void* a, const void* w, const float* bias, void* out, int out_f32, int M, int N, int K,
                         hipStream_t stream) {
    EpiArgs ep{out, bias, N, N, 0, 0};
    if (out_f32) return launch_gemm<EPI_STORE_F32>((const elem_t*)a, (const elem_t*)w, M, N, K, ep, stream);
    return launch_gemm<EPI_STORE_ELEM>((const elem_t*)a, (const elem_t*)w, M, N, K, ep, stream);
}

// x[M, N] += a[M, K] w[N, K]^T, x being the 32-bit residual stream.
extern "C" int ms_linear_residual(const void* a, const void* w, float* x, int M, int N, int K, hipStream_t stream) {
    EpiArgs ep{x, nullptr, N, N, 0, 0};
    return launch_gemm<EPI_RESIDUAL>((const elem_t*)a, (const elem_t*)w, M, N, K, ep, stream);
}

// out[M, I] = act(a g^T) * (a u^T) where w holds gate and up rows interleaved in blocks of 16:
// rows [32 t, 32 t + 16) are gate rows [16 t, 16 t + 16), rows [32 t + 16, 32 t + 32) the same
// up rows; w has 2 * ceil16(I) rows, the padding rows being zero.
extern "C" int ms_linear_swiglu(const void* a, const void* w, void* out, int M, int I, int K, int act, hipStream_t stream) {
    MS_REQUIRE(act >= 0 && act < ACT_COUNT, "gated product: no activation %d", act);
    const int n = 2 * ceil_div(I, 16) * 16;
    EpiArgs ep{out, nullptr, I, I, 0, 0, nullptr, 0, 0.f, act};
    return launch_gemm<EPI_SWIGLU>((const elem_t*)a, (const elem_t*)w, M, n, K, ep, stream);
}

// Whether ms_linear_swiglu_scaled takes this shape: bfloat16, one tile of rows, whole K steps of 64.
extern "C" int ms_swiglu_scaled_takes(int M, int I, int K) {
#ifdef MS_ELEM_HALF
    (void)I;
    return kRoundsBeforeTheNormIsSafe && M >= 1 && M <= 64 && K % 64 == 0 && K >= 256;
#else
    (void)M; (void)I; (void)K;
    return 0;
#endif
}

// ms_linear_swiglu for rows that came in multiplied by a norm's weight only: both products of a row are
// divided by the row's root mean square, 1 / sqrt(sum_p row_ss[p, row] / K + eps), before the activation.
extern "C" int ms_linear_swiglu_scaled(const void* a, const float* row_ss, int ss_parts, float eps, const void* w, void* out, int M, int I,
                                       int K, int act, hipStream_t stream) {
#ifdef MS_ELEM_HALF
    MS_REQUIRE(act >= 0 && act < ACT_COUNT, "gated product: no activation %d", act);
    MS_REQUIRE(ms_swiglu_scaled_takes(M, I, K), "gated product with row factors: M=%d K=%d is not taken", M, K);
    MS_REQUIRE(row_ss && ss_parts >= 1, "gated product with row factors: the rows' sums of squares are missing");
    MS_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0, "gemm: operands must be 16-byte aligned");
    const int n = 2 * ceil_div(I, 16) * 16;
    EpiArgs ep{out, nullptr, I, I, K, 0, row_ss, ss_parts, eps, act};
    hipLaunchKernelGGL((gemm_kernel<64, 64, 2, 2, 64, EPI_SWIGLU, 4, true>), dim3((unsigned)ceil_div(n, 64), 1), dim3(256), 0, stream,
                       (const elem_t*)a, (const elem_t*)w, M, n, K, ep);
    return check_launch("gemm 64x64x64 deep, row factors");
#else
    (void)a; (void)row_ss; (void)ss_parts; (void)eps; (void)w; (void)out; (void)M; (void)I; (void)K; (void)act; (void)stream;
    MS_REQUIRE(false, "gated product with row factors: built for bfloat16 only");
#endif
}

// Whether ms_linear_qkv_rope takes this shape: two-byte elements, more rows than the few-rows kernels take, heads of
// 64 (a tile's columns are one head, so that both elements of a rotated pair lie in one lane), K in whole chunks.
// Heads of 128 are left to the plain product and the rotation kernel: tiles of one head's width, four waves above one
// another, give those shapes a worse count of blocks and less reuse in a wave than the plain product's wider tiles
// (7B layer sizes, 2,048 rows: 133 us in one launch against 81 + 17 in two; 1.5B, 512 rows: the step 6 % longer).
// So are steps of up to 256 rows: their few tiles are each a chain of all K steps, which takes 10 us whatever the
// number of LDS buffers, while the plain product cuts K over several blocks (0.5B sizes, 128 rows: 8.9 us in two
// kernels, 9.7 to 11.8 in one; from 384 rows on the one kernel is ahead: 10.0 against 10.9).
extern "C" int ms_qkv_rope_takes(int M, int H, int KV, int hd, int K) {
#ifdef MS_ELEM_HALF
    return M > 256 && H > 0 && KV > 0 && hd == 64 && K % 8 == 0 && K >= 128;
#else
    (void)M; (void)H; (void)KV; (void)hd; (void)K;
    return 0;
#endif
}

// The q/k/v projection of a step of many rows with what follows it in its epilogue: w [(H + 2 KV) * hd, K] holds the
// query heads, the key heads and the value heads; bias [(H + 2 KV) * hd] or null is added, queries and keys are rotated
// by the rows' angles (rope_cs [M, hd / 2, 2], cosine and sine, as ms_rope_table makes them), queries go to q_out
// [M, H * hd], keys and values into their pages at slot_map[row] (a negative slot is not written).  The same values as
// ms_linear (32-bit output) followed by ms_rope_kv_write, without the 32-bit sums' trip through memory and without
// the second launch.
extern "C" int ms_linear_qkv_rope(const void* a, const void* w, const float* bias, const float* rope_cs, const int* slot_map,
                                  void* q_out, void* kpool, void* vpool, int M, int H, int KV, int hd, int ps, int K,
                                  hipStream_t stream) {
#ifdef MS_ELEM_HALF
    MS_REQUIRE(ms_qkv_rope_takes(M, H, KV, hd, K), "q/k/v product with rotation: M=%d, %d + 2 x %d heads of %d, K=%d is not taken", M, H, KV, hd, K);
    MS_REQUIRE(rope_cs && slot_map && q_out && kpool && vpool && ps > 0, "q/k/v product with rotation: a buffer is missing");
    MS_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0, "gemm: operands must be 16-byte aligned");
    const int N = (H + 2 * KV) * hd;
    EpiArgs ep{q_out, bias, H * hd, N, K, 0, nullptr, 0, 0.f, 0, rope_cs, slot_map, (elem_t*)kpool, (elem_t*)vpool, H, KV, ps};
    const long round_blocks = 2L * compute_units();
#define MS_QKV(BM_, BN_)                                                                                                 \
    do {                                                                                                                 \
        const long nb = (long)ceil_div(M, BM_) * (N / BN_);                                                              \
        hipLaunchKernelGGL((gemm_kernel<BM_, BN_, 4, 1, 64, EPI_QKV_ROPE>), dim3((unsigned)nb, 1), dim3(256), 0, stream, \
                           (const elem_t*)a, (const elem_t*)w, M, N, K, ep);                                             \
        return check_launch("gemm q/k/v with rotation " #BM_ "x" #BN_);                                                  \
    } while (0)
    // rows in tiles of 128 where that still gives the chip a round of blocks, else of 64
    const bool tall = (long)ceil_div(M, 128) * (N / hd) >= round_blocks * 300 / 512;
    if (tall) MS_QKV(128, 64);
    if (K % 64 == 0 && K >= 256) {
        // three LDS buffers in turn (two K steps in flight, three blocks a CU): 0.5B, 2,048 rows, 17.0 -> 16.4 us; tiles of
        // 128x64 take 20.3 (288 blocks, barely one a CU, each step a trip to the L2); four buffers where the blocks are
        // at most two a CU (512 to 1,536 rows: 10.6 -> 10.0, 11.8 -> 11.4 us; at 2,048 rows 13.4 -> 17.9)
        const long nb = (long)ceil_div(M, 64) * (N / 64);
        if (nb <= round_blocks) {
            hipLaunchKernelGGL((gemm_kernel<64, 64, 4, 1, 64, EPI_QKV_ROPE, 4>), dim3((unsigned)nb, 1), dim3(256), 0, stream,
                               (const elem_t*)a, (const elem_t*)w, M, N, K, ep);
            return check_launch("gemm q/k/v with rotation 64x64 deeper");
        }
        hipLaunchKernelGGL((gemm_kernel<64, 64, 4, 1, 64, EPI_QKV_ROPE, 3>), dim3((unsigned)nb, 1), dim3(256), 0, stream,
                           (const elem_t*)a, (const elem_t*)w, M, N, K, ep);
        return check_launch("gemm q/k/v with rotation 64x64 deep");
    }
    MS_QKV(64, 64);
#undef MS_QKV
#else
    (void)a; (void)w; (void)bias; (void)rope_cs; (void)slot_map; (void)q_out; (void)kpool; (void)vpool; (void)M; (void)H; (void)KV;
    (void)hd; (void)ps; (void)K; (void)stream;
    MS_REQUIRE(false, "q/k/v product with rotation: built for two-byte elements only");
#endif
}

// Number of partial sums ms_linear_split_tiled writes for this problem (1 = the complete product).
extern "C" int ms_tiled_partials(int M, int N, int K) { return plan_tiled_splits(M, N, K); }

// Whether a product of M rows is better served by the tiled kernel than by the few-rows kernel (which
// takes at most 64 rows).  The few-rows kernel reads its rows again for every 32 or 64 columns; with
// many rows and a large weight that traffic outweighs the weight itself, and the tiled kernel, which
// shares the rows of a block through LDS, streams the weight faster (measured at the 0.5B, 1.5B and 7B
// layer sizes, 8 to 64 rows).  The choice changes the order of the sums, so results differ in rounding.
extern "C" int ms_prefers_tiled(int M, int N, int K) {
    if (M > 64) return 1;
#ifdef MS_ELEM_HALF
    // Above 32 rows the tiled kernel, with K cut over enough blocks, beats the few-rows kernel for every
    // weight (0.5B q/k/v projection at 64 rows: 9.7 us few-rows, 4.9 us tiled in seven slices).
    if (M > 32) return 1;
    const double nk = (double)N * (double)K;
    if (N >= 2048) {
        // A large weight under a wide output: the tiled kernel's blocks each stream their columns' rows of the
        // weight step after step, several steps in flight, while every wave of the few-rows kernel asks for its
        // whole share at once and then waits.  From one row on (decode steps of the 1.5B and 7B layer sizes at
        // batch 1, 2, 4, 8: 7 to 12 % shorter; the vocabulary-sized head of every shape); a smaller weight
        // (0.5B gate/up) from 17 rows on, where the few-rows kernel can no longer apply the norm itself and
        // re-reads its rows for every 32 columns (batch 32: 1.53 -> 1.40 ms a step); from 9 rows on where the output
        // is wide (0.5B gate/up, 9,728 columns), together with the narrow projections below: the norm between them
        // then runs by itself and adds the K slices (0.5B decode step at batch 12 and 16: 1.085 -> 1.056 ms; a
        // 2,048-wide output, the 1.5B q/k/v projection, loses 1 % by it and keeps the few-rows kernel up to 16 rows).
        return nk >= 10e6 || M >= 17 || (M >= 9 && N >= 4096);
    }
    if (N >= 1024) {
        // a projection of the width (q/k/v, output): from 16 rows, or 8 if it is not small (batch 32: 1.40 ->
        // 1.36 ms a step; 0.5B q/k/v at 8 rows is faster in the few-rows kernel); a large weight (the 1.5B down
        // projection: 27 MB) from one row on (1.5B decode step at batch 1 and 4: 1.5 % shorter)
        return M >= 16 || (M >= 8 && nk >= 2e6) || nk >= 10e6;
    }
    // a narrow output (the 0.5B output and down projections, 896 columns): from 9 rows on the tiled kernel with K cut
    // over many blocks (0.5B decode step at batch 24 and 32: 1.195 -> 1.129 and 1.200 -> 1.138 ms, all of it from the
    // output projection; at 9 to 16 rows only together with the gate/up product above)
    return M >= 9;
#else
    return 0;
#endif
}

// out[ks, M, N] (float) = partial sums of a w^T over ms_tiled_partials(M, N, K) slices of K.
extern "C" int ms_linear_split_tiled(const void* a, const void* w, float* out, int M, int N, int K, hipStream_t stream) {
    EpiArgs ep{out, nullptr, N, N, 0, 0};
    return launch_gemm<EPI_STORE_F32>((const elem_t*)a, (const elem_t*)w, M, N, K, ep, stream, plan_tiled_splits(M, N, K));
}

// Measurements only: force one tile configuration (0 = choose by shape).
#ifdef MS_MEASURE
extern "C" void ms_gemm_force_config(int c) { g_gemm_config = c; }
extern "C" void ms_gemm_force_splits(int n) { g_force_splits = n; }
#endif
