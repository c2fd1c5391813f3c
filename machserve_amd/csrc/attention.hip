// Causal grouped-query attention of a mixed batch over a paged cache, on the matrix cores.
//
// Role in the reference: attn_paged_tiled_*_gqa and *_gqa_runs
// (crates/mach-model/src/kernels.rs:1367-1496, 1650-1885): K/V tiles staged in LDS and
// shared by the query heads of one KV head, online softmax with
// m' = max(m, tile_max), acc = acc * exp(m - m') + sum exp(s - m') V.
//
// One block = 64 "flat rows" of one request and one KV head.  Flat row r of a request is
// (token r / g, query head kvh * g + r % g), g = heads per KV head: a prompt portion of n
// tokens has n * g rows, a decoded token g rows, and any g works the same way.  Each of the
// four waves owns 16 flat rows.  Scores are computed transposed, S^T = K Q^T, so that a lane
// holds four consecutive keys of one query row: row maxima and sums stay in the lane (plus
// two cross-lane steps), and the probabilities are already laid out as the B operand of
// O^T = V^T P^T.  V is stored transposed in its pages ([head_dim][page_size]) so that V^T
// tiles load with contiguous 16-byte reads.
//
// Key tiles start at absolute multiples of BKV from key 0, whatever the portion, so a
// row's result does not depend on how its request was cut into steps.
//
// Compiled once per MS_ATTN_ND (tile head size / 16); a smaller head size runs in the next
// larger tile with the unused columns zero.
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "common.cuh"
#include "no_alloc.h"

#ifndef MS_ATTN_ND
#error "MS_ATTN_ND: head-size tile in units of 16"
#endif

namespace ms {

constexpr int ND = MS_ATTN_ND;
constexpr int HDT = ND * 16;             // head size of the tile
constexpr int NKS = (HDT + 31) / 32;     // K steps of 32 over the head size
#ifdef MS_ELEM_HALF
constexpr int BKV = ND <= 8 ? 64 : 32;
constexpr int EPC = 8;
// LDS has 64 banks of 4 bytes: the 16-byte reads of K fragments (row l % 16, chunk l / 16) are free of
// conflicts at a row pitch of 32 modulo 64 bytes, the 8-byte reads of V^T fragments at 16 modulo 32.
constexpr int KPAD = (ND * 16 * 2) % 64 == 0 ? 16 : 0, VPAD = 8;
#else
constexpr int BKV = ND <= 4 ? 64 : (ND <= 8 ? 32 : 16);
constexpr int EPC = 4;
constexpr int KPAD = 4, VPAD = 4;
#endif
constexpr int NT = BKV / 16;             // 16-key score tiles per key tile
constexpr int NTP = (NT + 1) / 2;        // pairs of score tiles = K steps of the PV product
constexpr int K_LD = HDT + KPAD, V_LD = BKV + VPAD;
// Flat rows of a work item.  The kernel of 32-row tiles (two-byte elements, head size 64) takes 128 a block; the
// general kernel takes 64, and where a library has both, two of its blocks share an item.
#if defined(MS_ELEM_HALF) && MS_ATTN_ND == 4
#define MS_HAS_ROWS32 1
constexpr int ROWS_PER_BLOCK = 128;
#else
constexpr int ROWS_PER_BLOCK = 64;
#endif
constexpr int SUB_BLOCKS = ROWS_PER_BLOCK / 64;  // blocks of the general kernel per work item
constexpr float NEG_BIG = -1e30f;
#ifdef MS_ELEM_HALF
constexpr int MAX_KEY_GROUPS = ND <= 4 ? 4 : 2;  // groups of four waves that may share a block's keys
#else
constexpr int MAX_KEY_GROUPS = 2;
#endif

struct AttnArgs {
    const elem_t* q;         // [T, H, hd]
    const elem_t* kpool;     // [pages, KV, ps, hd]
    const elem_t* vpool;     // [pages, KV, hd, ps]
    elem_t* out;             // [T, H * hd]
    const int* block_table;  // [S, table_stride]
    const int* seq_q_start;  // [S] first row of the request in this step
    const int* seq_q_len;    // [S] rows of the request in this step
    const int* seq_pos0;     // [S] position of its first row
    const int* work;         // [W, 2] (request index, first flat row), best with the longest contexts first
    int table_stride, H, KV, hd, ps, window;
    float scale;
    int n_work;     // W
    int pair_span;  // work items per round of blocks over the chip when two blocks share a CU, else 0
    // the keys of a block cut over gridDim.y blocks (few blocks of rows, long contexts): each writes
    // its unnormalised output and (max, sum) per row, and decode_merge_kernel adds them up
    int nsplit;
    float* part_o;   // [T, H, nsplit, hd]
    float* part_ml;  // [T, H, nsplit, 2]
};

__device__ __forceinline__ float exp_f(float x) {
#ifdef MS_ELEM_HALF
    return __expf(x);
#else
    return expf(x);
#endif
}

__device__ __forceinline__ float exp2_f(float x) {
#ifdef MS_ELEM_HALF
    return __builtin_amdgcn_exp2f(x);
#else
    return exp2f(x);
#endif
}

// KG "key groups" of four waves each share a block: group kg takes the key tiles whose absolute
// index is kg modulo KG, with its own staging buffers, and the groups' running (max, sum, output)
// are merged through LDS at the end.  A block's time is the length of its serial chain of tiles,
// and a causal prompt's last rows see every key: more groups cut that chain.
// Waves per SIMD the compiler has to leave room for: with the small bfloat16 tiles two blocks of a CU
// overlap one's LDS traffic with the other's arithmetic, if the registers allow them.
#ifdef MS_ELEM_HALF
template <int KG> constexpr int attention_waves_per_simd() { return ND <= 4 ? (KG == 1 ? 3 : 4) : 1; }
#else
template <int KG> constexpr int attention_waves_per_simd() { return 1; }
#endif

template <int KG>
__global__ __launch_bounds__(256 * KG, attention_waves_per_simd<KG>()) void paged_attention_kernel(AttnArgs a) {
    constexpr int KS_ELEMS = BKV * K_LD, VS_ELEMS = HDT * V_LD;
    constexpr int STAGE_BYTES = (KS_ELEMS + VS_ELEMS) * (int)sizeof(elem_t);
    constexpr int MERGE_FLOATS = 4 * 64 * (4 * ND + 2);  // per group: four waves, per lane the output and (max, sum)
    // two stages per group: a tile is multiplied out of one while the next is written into the other
    constexpr int SMEM_BYTES = 2 * KG * STAGE_BYTES > (KG - 1) * MERGE_FLOATS * 4 ? 2 * KG * STAGE_BYTES : (KG - 1) * MERGE_FLOATS * 4;
    static_assert(SMEM_BYTES <= 160 * 1024, "the tiles of a block exceed the LDS of a CU");
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];

    const int kg = threadIdx.x >> 8, tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
    auto stage_k = [&](int b) { return reinterpret_cast<elem_t*>(smem + (2 * kg + b) * STAGE_BYTES); };
    auto stage_v = [&](int b) { return stage_k(b) + KS_ELEMS; };
    const int r16 = lane & 15, grp = lane >> 4;
    // Blocks are numbered item by item, the KV heads of an item side by side.  A block's work grows
    // with its context, and blocks go to the CUs in turn: with two blocks a CU, block b shares its
    // CU with block b + (number of CUs).  So the list's heaviest `pair_span` items come first, then
    // its lightest ones, lightest first (each beside one of the heaviest), then the middle.
    // (a work item of ROWS_PER_BLOCK rows is SUB_BLOCKS blocks of 64 rows here, side by side)
    const int kvh = blockIdx.x % a.KV, sub = (blockIdx.x / a.KV) % SUB_BLOCKS, turn = blockIdx.x / (a.KV * SUB_BLOCKS);
    int item = turn;
    if (a.pair_span > 0 && turn >= a.pair_span)
        item = turn < 2 * a.pair_span ? a.n_work - 1 - (turn - a.pair_span) : turn - a.pair_span;
    const int s = a.work[item * 2], r0 = a.work[item * 2 + 1] + 64 * sub;
    if (s < 0) return;  // an item that only fills the list up to a size that many steps share (the same for the whole block)
    const int g = a.H / a.KV;
    const int q_start = a.seq_q_start[s], q_len = a.seq_q_len[s], pos0 = a.seq_pos0[s];
    const int R = q_len * g;
    if (r0 >= R) return;  // the item's rows end in the block beside this one (the same for the whole block)
    const int hd = a.hd, ps = a.ps;
    const int* table = a.block_table + (size_t)s * a.table_stride;

    // this lane's query row
    const int row = r0 + wave * 16 + r16;
    const bool valid = row < R;
    const int tok = valid ? row / g : 0;
    const int head = kvh * g + (valid ? row % g : 0);
    const int pos = pos0 + tok;
    const bool wave_active = r0 + wave * 16 < R;

    // keys any row of the block may see, and of those the rounds of tiles that are this split's
    constexpr int ROUND = KG * BKV;  // keys per round of the block
    const int last_row = min(r0 + 64, R) - 1;
    int kv_hi = pos0 + last_row / g + 1;
    int kv_lo = 0;
    if (a.window > 0) kv_lo = max(0, pos0 + r0 / g - a.window + 1);
    const int lo_key = a.window > 0 ? pos - a.window + 1 : 0;
    const int sp = blockIdx.y;
    if (a.nsplit > 1) {
        const int first = (kv_lo / ROUND) * ROUND;
        const int per = ceil_div(ceil_div(kv_hi - first, ROUND), a.nsplit) * ROUND;
        kv_lo = max(kv_lo, first + sp * per);
        kv_hi = min(kv_hi, first + (sp + 1) * per);
    }
    // a row's partial result of this split (group 0 writes, after the groups have been merged)
    auto write_partial = [&](const f32x4* o, float m, float l) {
        const size_t base = (((size_t)(q_start + tok)) * a.H + head) * a.nsplit + sp;
        float* po = a.part_o + base * hd;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            const int d0 = dt * 16 + grp * 4;
            if (d0 < hd) {
#pragma unroll
                for (int i = 0; i < 4; ++i) po[d0 + i] = o[dt][i];
            }
        }
        // the merge takes maxima in natural-logarithm units of the scaled scores
        if (grp == 0) { a.part_ml[base * 2] = m * a.scale; a.part_ml[base * 2 + 1] = l; }
    };
    if (kv_lo >= kv_hi) {  // nothing for this split (the same for every thread of the block)
        if (a.nsplit > 1 && threadIdx.x < 256 && valid) {
            f32x4 zero[ND];
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) zero[dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
            write_partial(zero, NEG_BIG, 0.f);
        }
        return;
    }

    Frag qf[NKS];
    {
        const elem_t* qrow = a.q + ((size_t)(q_start + tok) * a.H + head) * hd;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const int d0 = ks * 32 + grp * 8;
            qf[ks] = (valid && d0 < hd) ? frag_load(qrow + d0) : frag_zero();
        }
    }

    f32x4 acc_o[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i) acc_o[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // running maximum in units of the raw score; exponentials are taken in base 2 with the scale
    // folded in: exp(scale * (s - m)) = exp2(s * sl - m * sl)
    float m_run = NEG_BIG, l_run = 0.f;
    const float sl = a.scale * 1.4426950408889634f;

    // Tiles go global -> registers -> LDS.  PF tiles per group are in flight at any time: a tile's
    // loads are requested PF rounds before it is multiplied, which covers the memory latency even
    // when few blocks share a CU.  Where a tile's 16-key groups lie in the pools is looked up once
    // per tile by NT threads and shared through LDS (offsets in units of 16 elements).
    constexpr int CPRK = HDT / EPC, CPRV = BKV / EPC;
    constexpr int NCK = (BKV * CPRK + 255) / 256, NCV = (HDT * CPRV + 255) / 256;
    constexpr int PF = KG == 1 ? (ND <= 4 ? 4 : (ND <= 8 ? 2 : 1)) : (ND <= 8 ? 2 : 1);
    constexpr unsigned ABSENT = 0xffffffffu;
    __shared__ unsigned kofs[KG][PF][NT], vofs[KG][PF][NT];
    u32x4 rk[PF][NCK], rv[PF][NCV];
    // what does not change from tile to tile: where in a 16-key group this thread's chunks lie (an
    // unused chunk, beyond the head size or the tile, reads the start of the pool)
    const elem_t* k_base[NCK];
    const elem_t* v_base[NCV];
    bool k_on[NCK], v_on[NCV];
#pragma unroll
    for (int i = 0; i < NCK; ++i) {
        const int c = tid + i * 256, kl = c / CPRK, d0 = (c % CPRK) * EPC;
        k_on[i] = c < BKV * CPRK && d0 < hd;
        k_base[i] = a.kpool + (k_on[i] ? (kl % 16) * hd + d0 : 0);
    }
#pragma unroll
    for (int i = 0; i < NCV; ++i) {
        const int c = tid + i * 256, d = c / CPRV, k0 = (c % CPRV) * EPC;
        v_on[i] = c < HDT * CPRV && d < hd;
        v_base[i] = a.vpool + (v_on[i] ? d * ps + (k0 % 16) : 0);
    }
    // Every load below is unconditional (an absent or unused chunk reads the start of the pool and is
    // zeroed when it is stored to LDS, PF rounds later): with loads on one straight path, and no use
    // of the loaded values before that, the compiler counts the loads and waits only for the tile it
    // is about to use, and the younger tiles stay in flight.  The page of a tile's 16-key group is
    // read one round before its offsets are needed; which logical page that is, is stepped from
    // round to round rather than divided out.
    const int tsub = tid % NT;
    const int round_pages = ROUND / ps, round_rem = ROUND % ps;
    int key_next, lp_next, off_next;  // this thread's 16-key group of the next tile to look up
    auto start_lookup = [&](int kt0) {
        key_next = kt0 + tsub * 16;
        lp_next = key_next / ps;
        off_next = key_next % ps;
    };
    struct Entry { int page, off; };
    auto lookup = [&]() {  // page (or -1) and offset in it of the group; moves on by one round
        Entry e{table[min(lp_next, a.table_stride - 1)] | (key_next < kv_hi ? 0 : -1), off_next};
        key_next += ROUND;
        lp_next += round_pages;
        off_next += round_rem;
        if (off_next >= ps) {
            off_next -= ps;
            ++lp_next;
        }
        return e;
    };
    auto fill_offsets = [&](int slot, Entry e) {
        if (tid < NT) {
            const size_t pk = (size_t)max(e.page, 0) * a.KV + kvh;
            kofs[kg][slot][tid] = e.page >= 0 ? (unsigned)(((pk * ps + e.off) * hd) >> 4) : ABSENT;
            vofs[kg][slot][tid] = e.page >= 0 ? (unsigned)((pk * hd * ps + e.off) >> 4) : ABSENT;
        }
    };
    unsigned live[PF];  // bit i: chunk i of the slot's tile was really read (K chunks first, then V)
    auto load_tile = [&](int slot, u32x4* pk, u32x4* pv) {
        unsigned bits = 0;
#pragma unroll
        for (int i = 0; i < NCK; ++i) {
            const int kl = (tid + i * 256) / CPRK;
            const unsigned o = kofs[kg][slot][(kl / 16) % NT];
            const bool on = k_on[i] && o != ABSENT;
            pk[i] = *reinterpret_cast<const u32x4*>(k_base[i] + ((size_t)(on ? o : 0u) << 4));
            bits |= (on ? 1u : 0u) << i;
        }
#pragma unroll
        for (int i = 0; i < NCV; ++i) {
            const int k0 = ((tid + i * 256) % CPRV) * EPC;
            const unsigned o = vofs[kg][slot][(k0 / 16) % NT];
            const bool on = v_on[i] && o != ABSENT;
            pv[i] = *reinterpret_cast<const u32x4*>(v_base[i] + ((size_t)(on ? o : 0u) << 4));
            bits |= (on ? 1u : 0u) << (NCK + i);
        }
        live[slot] = bits;
    };
    auto store_tile = [&](int slot, int b, const u32x4* pk, const u32x4* pv) {
        elem_t* Ks = stage_k(b);
        elem_t* Vs = stage_v(b);
        const unsigned bits = live[slot];
        // nearly always every chunk of every thread was really read: then nothing is masked
        if (__all(bits == (1u << (NCK + NCV)) - 1)) {
#pragma unroll
            for (int i = 0; i < NCK; ++i) {
                const int c = tid + i * 256;
                if (c < BKV * CPRK) *reinterpret_cast<u32x4*>(&Ks[(c / CPRK) * K_LD + (c % CPRK) * EPC]) = pk[i];
            }
#pragma unroll
            for (int i = 0; i < NCV; ++i) {
                const int c = tid + i * 256;
                if (c < HDT * CPRV) *reinterpret_cast<u32x4*>(&Vs[(c / CPRV) * V_LD + (c % CPRV) * EPC]) = pv[i];
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < NCK; ++i) {
            const int c = tid + i * 256;
            const unsigned keep = (bits >> i & 1) ? 0xffffffffu : 0u;
            if (c < BKV * CPRK)
                *reinterpret_cast<u32x4*>(&Ks[(c / CPRK) * K_LD + (c % CPRK) * EPC]) = pk[i] & (u32x4){keep, keep, keep, keep};
        }
#pragma unroll
        for (int i = 0; i < NCV; ++i) {
            const int c = tid + i * 256;
            const unsigned keep = (bits >> (NCK + i) & 1) ? 0xffffffffu : 0u;
            if (c < HDT * CPRV)
                *reinterpret_cast<u32x4*>(&Vs[(c / CPRV) * V_LD + (c % CPRV) * EPC]) = pv[i] & (u32x4){keep, keep, keep, keep};
        }
    };
    // rows of this wave: the first and the last position decide which tiles need no mask at all
    const int pos_first = pos0 + (r0 + wave * 16) / g;
    const int pos_last = pos0 + min(r0 + wave * 16 + 15, max(R - 1, 0)) / g;
    const int lo_last = a.window > 0 ? pos_last - a.window + 1 : 0;

    // Round r: group kg has the tile of absolute index round_first * KG + r * KG + kg.  Its loads are
    // asked for PF rounds ahead into register slot r % PF, it is written into LDS stage r % 2 while
    // round r - 1 is multiplied out of the other stage, and one barrier a round separates the two.
    const int kt_first = (kv_lo / ROUND) * ROUND;
    start_lookup(kt_first + kg * BKV);
#pragma unroll
    for (int j = 0; j < PF; ++j) fill_offsets(j, lookup());
    Entry ahead = lookup();
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PF; ++j) load_tile(j, rk[j], rv[j]);
    __syncthreads();  // slot 0's offsets have been read by everyone
    fill_offsets(0, ahead);  // of round PF, which the first round asks for
    ahead = lookup();
    store_tile(0, 0, rk[0], rv[0]);
    __syncthreads();
    constexpr int UNROLL = PF > 2 ? PF : 2;
    for (int kt_base = kt_first; kt_base < kv_hi; kt_base += UNROLL * ROUND) {
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (kt_base + u * ROUND >= kv_hi) break;  // the same for every thread of the block
        const int j = u % PF, jn = (u + 1) % PF, b = u & 1;
        const int kt0 = kt_base + u * ROUND + kg * BKV;
        const elem_t* Ks = stage_k(b);
        const elem_t* Vs = stage_v(b);
        load_tile(j, rk[j], rv[j]);  // round r + PF into the slot that round r left
        const bool busy = wave_active && kt0 < kv_hi;

        // S^T = K Q^T: lane holds keys grp * 4 + i of tile nt for query row r16
        f32x4 sc[NT];
        if (busy) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                sc[nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    const int d0 = ks * 32 + grp * 8;
                    Frag kf = (d0 < HDT) ? frag_load(&Ks[(nt * 16 + r16) * K_LD + d0]) : frag_zero();
                    mma_16x16x32(sc[nt], kf, qf[ks]);
                }
            }
        }
        // the next round's tile goes into the other stage, which the round before this one has left
        if (kt_base + (u + 1) * ROUND < kv_hi) {
            store_tile(jn, b ^ 1, rk[jn], rv[jn]);
            fill_offsets(jn, ahead);
            ahead = lookup();
        }
        if (busy) {
        // a tile that every row of the wave sees whole needs no mask
        const bool whole = kt0 + BKV - 1 <= pos_first && kt0 >= lo_last;
        float tmax = NEG_BIG;
        if (whole) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) tmax = fmaxf(tmax, sc[nt][i]);
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = kt0 + nt * 16 + grp * 4 + i;
                    const bool ok = valid && key <= pos && key >= lo_key;
                    const float v = ok ? sc[nt][i] : -INFINITY;
                    sc[nt][i] = v;
                    tmax = fmaxf(tmax, v);
                }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
        const float m_new = fmaxf(m_run, tmax);
        const float mb = m_new * sl;
        float psum = 0.f;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = exp2_f(fmaf(sc[nt][i], sl, -mb));
                sc[nt][i] = p;
                psum += p;
            }
        psum += __shfl_xor(psum, 16, WAVE);
        psum += __shfl_xor(psum, 32, WAVE);
        // where no row's maximum rose the factor is exactly one: after the first tiles that is the rule
        if (__any(m_new > m_run)) {
            const float alpha = exp2_f((m_run - m_new) * sl);
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc_o[dt][i] *= alpha;
        }
        l_run += psum;
        m_run = m_new;

        // O^T += V^T P^T: the probabilities of two score tiles form one B fragment
#pragma unroll
        for (int pp = 0; pp < NTP; ++pp) {
            Frag pf;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pf.v[i] = from_f32<elem_t>(sc[2 * pp][i]);
                pf.v[4 + i] = from_f32<elem_t>((2 * pp + 1 < NT) ? sc[(2 * pp + 1) % NT][i] : 0.f);
            }
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                Frag vf;
                const elem_t* v0 = &Vs[(dt * 16 + r16) * V_LD + (2 * pp) * 16 + grp * 4];
#pragma unroll
                for (int i = 0; i < 4; ++i) vf.v[i] = v0[i];
                if (2 * pp + 1 < NT) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) vf.v[4 + i] = v0[16 + i];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) vf.v[4 + i] = from_f32<elem_t>(0.f);
                }
                mma_16x16x32(acc_o[dt], vf, pf);
            }
        }
        }
        __syncthreads();  // this round's stage has been read, the next round's written
      }
    }

    if constexpr (KG > 1) {
        // groups 1.. hand (output, max, sum) to group 0 through LDS, which adds them in group order
        // (the rounds end with a barrier: the stages are free)
        float* mg = reinterpret_cast<float*>(smem);
        if (kg > 0) {
            float* mine = mg + ((size_t)(kg - 1) * 4 + wave) * 64 * (4 * ND + 2);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) mine[(dt * 4 + i) * 64 + lane] = acc_o[dt][i];
            mine[(4 * ND) * 64 + lane] = m_run;
            mine[(4 * ND + 1) * 64 + lane] = l_run;
        }
        __syncthreads();
        if (kg > 0) return;
#pragma unroll
        for (int o = 0; o < KG - 1; ++o) {
            const float* other = mg + ((size_t)o * 4 + wave) * 64 * (4 * ND + 2);
            const float m_o = other[(4 * ND) * 64 + lane], l_o = other[(4 * ND + 1) * 64 + lane];
            const float m_new = fmaxf(m_run, m_o);
            const float c0 = exp2_f((m_run - m_new) * sl), c1 = exp2_f((m_o - m_new) * sl);
            l_run = l_run * c0 + l_o * c1;
            m_run = m_new;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc_o[dt][i] = acc_o[dt][i] * c0 + other[(dt * 4 + i) * 64 + lane] * c1;
        }
    }

    if (valid && a.nsplit > 1) {
        write_partial(acc_o, m_run, l_run);
    } else if (valid) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        elem_t* orow = a.out + ((size_t)(q_start + tok) * a.H + head) * hd;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            const int d0 = dt * 16 + grp * 4;
            if (d0 < hd) {
#pragma unroll
                for (int i = 0; i < 4; ++i) orow[d0 + i] = from_f32<elem_t>(acc_o[dt][i] * inv);
            }
        }
    }
}


// ---------------------------------------------------------------------------------------
// The same attention in tiles of 32 query rows by 32 keys (`mfma_f32_32x32x16`), for the two-byte element
// types and a head size of 64.  The counters of the kernel above say that it spends fifteen vector instructions
// on every matrix instruction, and its blocks of 64 rows read the keys and values of a long prompt so often
// (a block of 64 flat rows is nine tokens of seven heads) that the traffic from the L2 comes within sight of that
// path's ceiling.  Here a block is 128 flat rows, four waves of 32 rows under each of four key groups (sixteen waves,
// a whole CU), so a tile that was brought into LDS feeds twice the rows; a lane holds sixteen keys of one query row
// (one step across lanes instead of two) and a fragment read from LDS feeds twice the arithmetic; the
// accumulator is rescaled only when a row's maximum has risen by more than a factor of 2^8 (a probability then
// reaches 256 at most, which neither the 32-bit sums nor the rounded probabilities mind); tiles go from memory
// straight into one of four LDS stages, three rounds before they are multiplied (no staging registers, no
// stores); and the block's share of the block table is copied into LDS once, so that no round waits for a page
// number.  Key tiles start at absolute multiples of 32, tile t belongs to group t mod 4, and every decision is a
// row's own, so a row's result depends neither on the step's cut nor on the rows beside it.
//
// Operands (K = 16): A is 32 rows x 16, lane l holds row l % 32, elements (l / 32) * 8 .. + 8; B likewise by
// column; the result has column l % 32 and, in register v, row 8 * (v / 4) + 4 * (l / 32) + v % 4.  With
// S^T = K Q^T a lane's registers 8c .. 8c + 7 are therefore rows 16c + {0..3, 8..11} + 4 * (l / 32) of the key
// tile: if row R of the tile holds key R with bits 2 and 3 exchanged, they are the eight consecutive keys
// 16c + 8 * (l / 32) .., which is a B fragment of P^T as it stands and one 16-byte read of V^T.
//
// A tile that is loaded straight into LDS cannot be zeroed on its way: keys that are not there (beyond the
// rows' positions, in pages given back behind a window, in tiles past the block's range) read the start of the
// pool instead, and are masked in the scores; the pools hold finite values everywhere, so a value that meets a
// zero probability adds nothing.
#ifdef MS_HAS_ROWS32
namespace r32 {
constexpr int KG = 4, RW = 4, TK = 32;  // key groups, waves of rows, keys of a group's tile
constexpr int GT = RW * 64;             // threads of a key group
constexpr int ROUND = KG * TK;          // keys of a round of the block
constexpr int NS = 4;                   // LDS stages: a tile is asked for NS - 1 rounds before it is multiplied
constexpr int NC = HDT / 16;            // steps of the score product
constexpr int NDT = HDT / 32;           // 32-row tiles of the output's head dimension
// LDS rows are unpadded; 16-byte chunk q of row r sits at q ^ f(r), with f such that the rows a fragment read takes
// in one pass (0..7 with 16..23, 8..15 with 24..31) fall on different banks.
constexpr int K_BYTES = TK * HDT * 2, V_BYTES = HDT * TK * 2;
constexpr int STAGE = K_BYTES + V_BYTES;
constexpr int PER_LANE = 16 * NDT + 2;  // what a group hands over per lane: the output, the reference, the sum
constexpr int MERGE_BYTES = (KG - 1) * RW * 64 * PER_LANE * 4;
constexpr int SMEM = NS * KG * STAGE > MERGE_BYTES ? NS * KG * STAGE : MERGE_BYTES;
constexpr int MAX_TABLE = 2048;  // pages of a block's share of the block table (in LDS)
constexpr float RISE = 8.0f;     // a row's reference maximum follows its maximum when that has risen by more (in powers of two)
static_assert(ROWS_PER_BLOCK == RW * 32, "a work item is what one block of this kernel takes");
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ void mma_32x32x16(f32x16& acc, const Frag& a, const Frag& b) {
#if defined(MS_ELEM_BF16)
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc, 0, 0, 0);
#else
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.v, b.v, acc, 0, 0, 0);
#endif
}
// The largest of three, as one instruction (from `fmaxf` the compiler makes two for every operand it cannot prove to be
// no signalling NaN; scores are sums of products of finite values, or -inf where masked).
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ int swap_bits_2_3(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }
__device__ __forceinline__ int k_swizzle(int r) { return ((r >> 1) & 3) | (((r >> 4) & 1) << 2); }  // rows of 8 chunks
__device__ __forceinline__ int v_swizzle(int d) { return ((d >> 2) & 1) | (((d >> 4) & 1) << 1); }  // rows of 4 chunks
}  // namespace r32

__global__ __launch_bounds__(r32::KG * r32::GT, 4) void paged_attention_rows32_kernel(AttnArgs a) {
    using namespace r32;
    static_assert(HDT == 64 && TK == 32 && RW == 4, "the swizzles and the tiles' split over a group's waves are written for this shape");
    static_assert(SMEM + MAX_TABLE * 4 + 1024 <= 160 * 1024, "the tiles of a block exceed the LDS of a CU");
    __shared__ __attribute__((aligned(1024))) unsigned char smem[SMEM];
    __shared__ int tab[MAX_TABLE];
    __shared__ unsigned kofs[KG][NS][2], vofs[KG][NS][2];  // [group][round % NS][16-key group of the tile]

    const int kg = threadIdx.x >> 8, tg = threadIdx.x & 255, lane = tg & 63, rw = tg >> 6;
    const int n32 = lane & 31, h = lane >> 5;
    auto stage = [&](int b) { return smem + (KG * b + kg) * STAGE; };
    const int kvh = blockIdx.x % a.KV, item = blockIdx.x / a.KV;
    const int s = a.work[item * 2], r0 = a.work[item * 2 + 1];
    if (s < 0) return;  // an item that only fills the list up (the same for the whole block)
    const int g = a.H / a.KV;
    const int q_start = a.seq_q_start[s], q_len = a.seq_q_len[s], pos0 = a.seq_pos0[s];
    const int R = q_len * g;
    constexpr int hd = HDT;
    const int ps = a.ps;
    const int* table = a.block_table + (size_t)s * a.table_stride;

    // this lane's query row (both halves of the wave hold the same 32 rows)
    const int row = r0 + rw * 32 + n32;
    const bool valid = row < R;
    const int tok = valid ? row / g : 0;
    const int head = kvh * g + (valid ? row % g : 0);
    const int pos = pos0 + tok;
    const bool wave_active = __builtin_amdgcn_readfirstlane((int)(r0 + rw * 32 < R)) != 0;  // the same for the whole wave

    const int last_row = min(r0 + ROWS_PER_BLOCK, R) - 1;
    int kv_hi = pos0 + last_row / g + 1;
    int kv_lo = 0;
    if (a.window > 0) kv_lo = max(0, pos0 + r0 / g - a.window + 1);
    const int lo_key = a.window > 0 ? pos - a.window + 1 : 0;
    const int sp = blockIdx.y;
    if (a.nsplit > 1) {
        const int first = (kv_lo / ROUND) * ROUND;
        const int per = ceil_div(ceil_div(kv_hi - first, ROUND), a.nsplit) * ROUND;
        kv_lo = max(kv_lo, first + sp * per);
        kv_hi = min(kv_hi, first + (sp + 1) * per);
    }
    // a row's partial result of this split: d = 32 dt + 8 (v / 4) + 4 h + v % 4 in register v of tile dt
    auto write_partial = [&](const f32x16* o, float m, float l) {
        const size_t base = (((size_t)(q_start + tok)) * a.H + head) * a.nsplit + sp;
        float* po = a.part_o + base * hd;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int d0 = 32 * dt + 8 * qd + 4 * h;
#pragma unroll
                for (int i = 0; i < 4; ++i) po[d0 + i] = o[dt][4 * qd + i];
            }
        if (h == 0) { a.part_ml[base * 2] = m * a.scale; a.part_ml[base * 2 + 1] = l; }
    };
    if (kv_lo >= kv_hi) {  // nothing for this split (the same for every thread of the block)
        if (a.nsplit > 1 && kg == 0 && valid) {
            f32x16 zero[NDT];
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) zero[dt][i] = 0.f;
            write_partial(zero, NEG_BIG, 0.f);
        }
        return;
    }
    // the pages of the block's keys, once: those of [kt_first, kv_hi), at most MAX_TABLE of them (the launcher sees to it)
    kv_hi = __builtin_amdgcn_readfirstlane(kv_hi);
    const int kt_first = __builtin_amdgcn_readfirstlane((kv_lo / ROUND) * ROUND);
    const int page_first = kt_first / ps, n_tab = min(ceil_div(kv_hi, ps), a.table_stride) - page_first;
    for (int i = threadIdx.x; i < n_tab; i += KG * GT) tab[i] = table[page_first + i];

    Frag qf[NC];
    {
        const elem_t* qrow = a.q + ((size_t)(q_start + tok) * a.H + head) * hd;
#pragma unroll
        for (int c = 0; c < NC; ++c) qf[c] = valid ? frag_load(qrow + c * 16 + h * 8) : frag_zero();
    }
    f32x16 acc[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[dt][i] = 0.f;
    // m_ref: the maximum that the exponentials refer to (a row's own running maximum, followed lazily)
    float m_ref = NEG_BIG, l_run = 0.f;
    const float sl = a.scale * 1.4426950408889634f;

    // A group's four waves bring the group's tile, a quarter of K and a quarter of V^T each: a wave's load lands at the
    // wave's LDS base + 16 * lane, so the chunk that belongs at place p = 64 * wave + lane of the K tile (row p / 8,
    // chunk p % 8 ^ swizzle) is the one this lane asks for; likewise the V^T tile (row p / 4).  Which 16-key group of
    // the tile a chunk lies in picks the page offset, which the group's first two threads leave in LDS a round before.
    const int p_own = 64 * rw + lane;
    const int Rk = p_own >> 3, kq = (p_own & 7) ^ k_swizzle(Rk), kl = swap_bits_2_3(Rk);  // row Rk of the tile holds key kl
    const elem_t* k_src = a.kpool + (kl & 15) * hd + kq * 8;
    const int k_grp = kl >> 4;
    const int dv = p_own >> 2, vq = (p_own & 3) ^ v_swizzle(dv);  // keys 8 vq .. + 8 of row dv of V^T
    const elem_t* v_src = a.vpool + (size_t)dv * ps + (vq & 1) * 8;
    const int v_grp = vq >> 1;
    // Offsets of the group's tile of the next round to be looked up, by the group's first two threads (one 16-key group of
    // the tile each), stepped from round to round rather than divided out.  Keys that are not there (past the
    // block's range, in a page given back) get offset 0: the first rows of the pool, finite and masked.
    int key_next = kt_first + kg * TK + (tg & 1) * 16, lp_next = key_next / ps, off_next = key_next - lp_next * ps;
    const int round_pages = ROUND / ps, round_rem = ROUND % ps;
    auto fill_offsets = [&](int r) {
        if (tg < 2) {
            const bool there = key_next < kv_hi && lp_next < a.table_stride;
            const int page = there ? tab[min(lp_next - page_first, n_tab - 1)] : -1;
            const size_t pk = (size_t)max(page, 0) * a.KV + kvh;
            kofs[kg][r % NS][tg] = page >= 0 ? (unsigned)(((pk * ps + off_next) * hd) >> 4) : 0u;
            vofs[kg][r % NS][tg] = page >= 0 ? (unsigned)((pk * hd * ps + off_next) >> 4) : 0u;
            key_next += ROUND;
            lp_next += round_pages;
            off_next += round_rem;
            if (off_next >= ps) {
                off_next -= ps;
                ++lp_next;
            }
        }
    };
    // the group's tile of round r straight into stage r % NS (in assembly: of a load that it knows to write LDS the
    // compiler would make every later LDS read wait; the waits are written by hand at the rounds' ends)
    const uint32_t lds_own = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)(smem + kg * STAGE + 1024 * rw));
    auto load_direct = [&](int r) {
        const int b = r % NS;
        const elem_t* gk = k_src + ((size_t)kofs[kg][b][k_grp] << 4);
        const elem_t* gv = v_src + ((size_t)vofs[kg][b][v_grp] << 4);
        const uint32_t kb = lds_own + b * (KG * STAGE), vb = kb + K_BYTES;
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gk), "s"(kb) : "memory", "m0");
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gv), "s"(vb) : "memory", "m0");
    };
    // rows of this wave: the first and the last position decide which tiles need no mask at all
    const int pos_first = pos0 + (r0 + rw * 32) / g;
    const int pos_last = pos0 + min(r0 + rw * 32 + 31, max(R - 1, 0)) / g;
    const int lo_last = a.window > 0 ? pos_last - a.window + 1 : 0;
    // where this lane reads its fragments in a stage: row n32 of the K tile, row 32 dt + n32 of V^T, chunk 2c + h
    const int k_row = n32 * (HDT * 2), k_sw = k_swizzle(n32), v_row = K_BYTES + n32 * (TK * 2), v_sw = v_swizzle(n32);

    // Round r: group kg has the tile of absolute index (kt_first / 32) + r * KG + kg.  Its page offsets are written a
    // round before its loads go out, its loads NS - 1 rounds before it is multiplied, and one barrier a round
    // separates the steps.
    // (the same for the whole block: kept in scalar registers, so that the rounds' branches are scalar ones)
    const int n_rounds = __builtin_amdgcn_readfirstlane(ceil_div(kv_hi - kt_first, ROUND));
    // the queries and the table are here before the first tile is asked for, so that no later wait of the compiler's
    // for them takes the tiles' loads with it
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int c = 0; c < NC; ++c) asm volatile("" : "+v"(qf[c].v));
    __syncthreads();  // the table is in LDS
    for (int r = 0; r < NS - 1; ++r) fill_offsets(r);
    __syncthreads();
    for (int r = 0; r < NS - 1; ++r)
        if (r < n_rounds) load_direct(r);
    fill_offsets(NS - 1);
    // End of a round: the tiles of all rounds but the youngest one asked for have landed (a wave's loads complete in
    // order, two a round), and this wave's LDS accesses are done; then everybody's.
    auto round_end = [&](bool one_behind) {
        __builtin_amdgcn_sched_barrier(0);
        if (one_behind) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    round_end(n_rounds >= NS - 1);  // rounds 0 and 1 are here
    // S^T = K Q^T of the group's tile of round r: register v of this lane is key kt0 + 16 (v / 8) + 8 h + v % 8 for query
    // row n32.  The scores of round r + 1 are asked for at the end of round r, behind the products of round r: the
    // matrix cores work on them while other waves take their exponentials.
    f32x16 sc;
    auto scores = [&](int r) {
        const unsigned char* st = stage(r % NS);
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
        auto k_frag = [&](int c) { return frag_load(reinterpret_cast<const elem_t*>(st + k_row + (((2 * c + h) ^ k_sw) << 4))); };
        Frag kf[2] = {k_frag(0), k_frag(1)};  // two fragments in flight
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            mma_32x32x16(sc, kf[c & 1], qf[c]);
            if (c + 2 < NC) kf[c & 1] = k_frag(c + 2);
        }
    };
    const int kg_keys = __builtin_amdgcn_readfirstlane(kg * TK);
    auto busy_in = [&](int r) { return wave_active && kt_first + r * ROUND + kg_keys < kv_hi; };
    if (busy_in(0)) scores(0);
    for (int r = 0; r < n_rounds; ++r) {
        const int kt0 = kt_first + r * ROUND + kg * TK;
        const unsigned char* st = stage(r % NS);
        const bool more = r + NS - 1 < n_rounds;
        if (more) load_direct(r + NS - 1);  // into the stage that round r - 1 has left
        if (busy_in(r)) {
            // the values of the first sixteen keys, which the step after next multiplies by: asked for before the exponentials
            auto v_frag = [&](int c, int dt) {
                return frag_load(reinterpret_cast<const elem_t*>(st + v_row + dt * (32 * TK * 2) + (((2 * c + h) ^ v_sw) << 4)));
            };
            Frag vf[NDT];
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) vf[dt] = v_frag(0, dt);
            const bool whole = kt0 + TK - 1 <= pos_first && kt0 >= lo_last;
            if (!whole) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int key = kt0 + 16 * (i / 8) + 8 * h + (i % 8);
                    const bool ok = valid && key <= pos && key >= lo_key;
                    sc[i] = ok ? sc[i] : -INFINITY;
                }
            }
            // this lane's half of the row's keys
            const float tmax = max3(max3(max3(sc[0], sc[1], sc[2]), max3(sc[3], sc[4], sc[5]), max3(sc[6], sc[7], sc[8])),
                                    max3(max3(sc[9], sc[10], sc[11]), sc[12], sc[13]), max3(sc[14], sc[15], sc[15]));
            // A row's reference follows its maximum only when that has risen far (the two lanes of a row keep the same
            // reference: where either's half has risen far they exchange their maxima); for every other row the factor
            // is exactly one and nothing changes.  After a prompt's first tiles this is rare.
            if (__any((tmax - m_ref) * sl > RISE)) {
                const float row_max = max3(tmax, __shfl_xor(tmax, 32, WAVE), tmax);
                const float m_new = (row_max - m_ref) * sl > RISE ? row_max : m_ref;
                const float alpha = exp2_f((m_ref - m_new) * sl);
                l_run *= alpha;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[dt][i] *= alpha;
                m_ref = m_new;
            }
            const float mb = m_ref * sl;
#pragma unroll
            for (int i = 0; i < 16; ++i) sc[i] = exp2_f(fmaf(sc[i], sl, -mb));
            float t8[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) t8[i] = sc[i] + sc[i + 8];
            l_run += ((t8[0] + t8[1]) + (t8[2] + t8[3])) + ((t8[4] + t8[5]) + (t8[6] + t8[7]));  // of this lane's half of the keys
            // O^T += V^T P^T: registers 8c .. 8c + 7 are the probabilities of keys 16c + 8h .. + 8, a B fragment as they stand
            Frag pf[2];
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int i = 0; i < 8; ++i) pf[c].v[i] = from_f32<elem_t>(sc[8 * c + i]);
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    mma_32x32x16(acc[dt], vf[dt], pf[c]);
                    if (c == 0) vf[dt] = v_frag(1, dt);
                }
        }
        if (r + 1 < n_rounds && busy_in(r + 1)) scores(r + 1);
        if (r + NS < n_rounds) fill_offsets(r + NS);  // read when that round's loads go out, at the top of the next round
        round_end(more);
    }

    l_run += __shfl_xor(l_run, 32, WAVE);  // the row's two halves (they were scaled alike all along)
    // groups 1.. hand (output, reference, sum) to group 0 through LDS, which adds them in group order
    float* mg = reinterpret_cast<float*>(smem);
    if (kg > 0) {
        float* mine = mg + ((size_t)(kg - 1) * RW + rw) * 64 * PER_LANE;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) mine[(dt * 16 + i) * 64 + lane] = acc[dt][i];
        mine[(16 * NDT) * 64 + lane] = m_ref;
        mine[(16 * NDT + 1) * 64 + lane] = l_run;
    }
    __syncthreads();
    if (kg > 0) return;
    for (int o = 0; o < KG - 1; ++o) {
        const float* other = mg + ((size_t)o * RW + rw) * 64 * PER_LANE;
        const float m_o = other[(16 * NDT) * 64 + lane], l_o = other[(16 * NDT + 1) * 64 + lane];
        const float m_new = fmaxf(m_ref, m_o);
        const float c0 = exp2_f((m_ref - m_new) * sl), c1 = exp2_f((m_o - m_new) * sl);
        l_run = l_run * c0 + l_o * c1;
        m_ref = m_new;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[dt][i] = acc[dt][i] * c0 + other[(dt * 16 + i) * 64 + lane] * c1;
    }
    if (valid && a.nsplit > 1) {
        write_partial(acc, m_ref, l_run);
    } else if (valid) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        elem_t* orow = a.out + ((size_t)(q_start + tok) * a.H + head) * hd;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int d0 = 32 * dt + 8 * qd + 4 * h;
                half4_t o4 = {from_f32<elem_t>(acc[dt][4 * qd] * inv), from_f32<elem_t>(acc[dt][4 * qd + 1] * inv),
                              from_f32<elem_t>(acc[dt][4 * qd + 2] * inv), from_f32<elem_t>(acc[dt][4 * qd + 3] * inv)};
                *reinterpret_cast<half4_t*>(orow + d0) = o4;
            }
    }
}
#endif  // MS_HAS_ROWS32

// ---------------------------------------------------------------------------------------
// Decode attention: every request of the step has one row.  The g query heads of one KV
// head are the rows of one MFMA tile (g <= 16), so each key and value is read once per KV
// head.  The keys of a request are cut into `nsplit` contiguous ranges (grid z), and inside
// a block each of the four waves takes every fourth key tile, reading K and V^T straight
// from the pages into fragments (nothing is shared between waves, so nothing is staged in
// LDS).  Waves combine through LDS; blocks write (max, sum, unnormalised output) per split,
// and a second kernel merges the splits.
// Role in the reference: attn_decode_batched_f16_gqa (crates/mach-model/src/kernels.rs:2905-3036).

struct DecodeArgs {
    const elem_t* q;         // [S, H, hd]
    const elem_t* kpool;
    const elem_t* vpool;
    elem_t* out;             // [S, H * hd] (written when nsplit == 1)
    float* part_o;           // [S, H, nsplit, hd]
    float* part_ml;          // [S, H, nsplit, 2]
    const int* block_table;  // [S, table_stride]
    const int* seq_pos0;     // [S] position of the row = number of keys before it
    int table_stride, H, KV, hd, ps, window, nsplit;
    float scale;
    // fused form: q, k, v of the step come as partial sums of the projection; the kernel adds
    // them and the bias, rotates q and k, writes k and v into their page and merges the splits
    const float* qkv;        // [n_partials, S, stride]: q heads, k heads, v heads
    const float* bias;       // [stride] or null
    const float* inv_freq;   // [hd / 2] or null: no rotation
    const int* slot_map;     // [S] page * ps + offset of the row's key
    int n_partials, stride;
};

constexpr int MAX_SPLITS = 64;
// The decode kernel's key tile: a wave holds two tiles in registers (one being multiplied, one in
// flight), and smaller tiles leave room for more waves on a CU, which is what keeps memory busy.
#ifndef MS_DECODE_BKV
#define MS_DECODE_BKV (BKV >= 32 ? 32 : BKV)
#endif
constexpr int DBKV = MS_DECODE_BKV;
constexpr int DNT = DBKV / 16, DNTP = (DNT + 1) / 2;

// Fragments of one key tile for one lane: keys (K rows) for the scores, V^T groups for the output.
struct DecodeTile {
    Frag kf[DNT][NKS];
    Frag vf[DNTP][ND];
};

template <bool FUSED>
__global__ __launch_bounds__(256) void decode_attention_kernel(DecodeArgs a) {
    arguments_now(a.q, a.kpool, a.vpool, a.out, a.part_o, a.part_ml, a.block_table, a.seq_pos0, a.table_stride, a.H, a.KV, a.hd,
                  a.ps, a.window, a.nsplit, a.scale, a.qkv, a.bias, a.inv_freq, a.slot_map, a.n_partials, a.stride);
    __shared__ __align__(32) float sm_o[3][HDT][16];  // also the staging area of the fused prologue: (g + 2) * hd sums and g * hd elements
    __shared__ float sm_m[3][16], sm_l[3][16];
    __shared__ float cs[HDT / 2], sn[HDT / 2], knew[HDT], vnew[HDT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, grp = lane >> 4;
    const int s = blockIdx.x, kvh = blockIdx.y, sp = blockIdx.z;
    const int g = a.H / a.KV, hd = a.hd, ps = a.ps;
    const int pos = a.seq_pos0[s];
    // keys read from the pages: all of them, or (fused) those before the row's own position,
    // whose key and value are still in registers and enter as one extra term
    const int kv_len = FUSED ? pos : pos + 1;
    const int lo_key = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const int* table = a.block_table + (size_t)s * a.table_stride;
    const bool valid = r16 < g;
    const int head = kvh * g + (valid ? r16 : 0);

    const int t_lo = lo_key / DBKV, t_hi = ceil_div(kv_len, DBKV);
    const int tps = max(1, ceil_div(t_hi - t_lo, a.nsplit));
    const int t0 = t_lo + sp * tps, t1 = min(t_hi, t0 + tps);

    // Where the keys of a tile sit in the MFMA rows is free, as long as the probabilities meet the
    // values of the same keys.  With an even number of 16-key score tiles, the pair (2pp, 2pp + 1)
    // covers 32 keys so that the lane of key group `grp` ends up with the probabilities of the eight
    // consecutive keys pp * 32 + grp * 8 ..: its V^T fragment is then one contiguous read.  Row r16 of
    // score tile 2pp + j holds key pp * 32 + (r16 / 4) * 8 + j * 4 + r16 % 4.
    constexpr bool PAIRED = DNT % 2 == 0;
    auto k_row = [&](int nt) { return PAIRED ? (nt / 2) * 32 + (r16 >> 2) * 8 + (nt & 1) * 4 + (r16 & 3) : nt * 16 + r16; };
    auto score_key = [&](int nt, int i) { return PAIRED ? (nt / 2) * 32 + grp * 8 + (nt & 1) * 4 + i : nt * 16 + grp * 4 + i; };
    // Loads are unconditional and on one straight path, so that the compiler counts them and a wait
    // for one tile leaves the next in flight: a key that is not there (beyond the row, in a page
    // given back, in a tile past the split) is read from the start of the pool instead and masked in
    // the scores.  The pools hold finite values everywhere, so a value that meets a zero probability
    // adds nothing.  The pages of a tile's 16-key groups are looked up one tile ahead.
    const float inv_gpp = 1.0f / (float)(ps >> 4);  // 1 / (16-key groups per page)
    // of this lane's groups: page as the table has it, -1 if the group is not to be read (else 0), offset in the page
    struct Pages { int kp[DNTP], kx[DNTP], ko[DNTP], vp[DNTP], vx[DNTP], vo[DNTP]; };
    auto lookup = [&](int t) {
        Pages pg;
        const int kt0 = t * DBKV;
#pragma unroll
        for (int pp = 0; pp < DNTP; ++pp) {
            // 16-key groups of this lane: of its K rows of score tiles 2pp and 2pp + 1, and of its V keys
            const int gk = (kt0 >> 4) + (PAIRED ? 2 * pp + (r16 >> 3) : pp), gv = (kt0 >> 4) + (PAIRED ? 2 * pp + (grp >> 1) : pp);
            const int lk = (int)(((float)gk + 0.5f) * inv_gpp), lv = (int)(((float)gv + 0.5f) * inv_gpp);
            const int pk = table[min(lk, a.table_stride - 1)], pv = table[min(lv, a.table_stride - 1)];
            // The loaded pages are not touched here (a use would wait for them), and are later "or"-ed with
            // a mask the compiler cannot see through: it would turn a select (and an "or" with a known
            // 0 / -1, which it reads as one) into a branch around the load.
            pg.kp[pp] = pk;
            pg.kx[pp] = opaque((t < t1 && gk * 16 < kv_len) ? 0 : -1);
            pg.ko[pp] = gk * 16 - lk * ps;
            pg.vp[pp] = pv;
            pg.vx[pp] = opaque((t < t1 && gv * 16 < kv_len) ? 0 : -1);
            pg.vo[pp] = gv * 16 - lv * ps;
        }
        return pg;
    };
    const size_t page_elems = (size_t)ps * hd;
    auto load_tile = [&](const Pages& pg, DecodeTile& td) {
#pragma unroll
        for (int nt = 0; nt < DNT; ++nt) {
            // the row of (page, kvh, offset of the row's 16-key group + place in the group) in [pages, KV, ps, hd]
            const int pp = PAIRED ? nt / 2 : nt;
            const int page = pg.kp[pp] | pg.kx[pp], off = pg.ko[pp] + (k_row(nt) & 15);
            const elem_t* krow = page >= 0 ? a.kpool + ((size_t)page * a.KV + kvh) * page_elems + (size_t)off * hd : a.kpool;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const int d0 = ks * 32 + grp * 8;
                td.kf[nt][ks] = frag_load(krow + (d0 < hd ? d0 : 0));  // beyond the head size q is zero
            }
        }
#pragma unroll
        for (int pp = 0; pp < DNTP; ++pp) {
            const int page = pg.vp[pp] | pg.vx[pp], off = pg.vo[pp] + (PAIRED ? (grp & 1) * 8 : grp * 4);
            const elem_t* vcol = page >= 0 ? a.vpool + ((size_t)page * a.KV + kvh) * page_elems + off : a.vpool;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const int d = dt * 16 + r16;
                const elem_t* v0 = vcol + (page >= 0 && d < hd ? (size_t)d * ps : 0);
                if constexpr (PAIRED) {
                    td.vf[pp][dt] = frag_load(v0);
                } else {
                    Frag vf = frag_zero();
#pragma unroll
                    for (int i = 0; i < 4; ++i) vf.v[i] = v0[i];
                    td.vf[pp][dt] = vf;
                }
            }
        }
    };
    // The fused prologue stages this KV head's share of the step's row: its g query heads, its key, its
    // value, (g + 2) * hd columns, four per thread at a time.  What the first four need from memory
    // (the bias and the first two partial sums) is asked for here, before anything else: nothing of it
    // depends on the row's position, and the row's query is what the block waits for in the end.
    const int width = FUSED ? (g + 2) * hd : 0;
    const size_t pstride = FUSED ? (size_t)gridDim.x * a.stride : 0;
    const float* row0 = FUSED ? a.qkv + (size_t)s * a.stride : nullptr;
    const float* bias = FUSED && a.bias ? a.bias : row0;  // without a bias: finite values, times zero
    const float bias_on = FUSED && a.bias ? 1.f : 0.f;
    auto column = [&](int c) {
        c = min(c, width - 1);
        const int qcol = kvh * g * hd, kcol = a.H * hd + kvh * hd, vcol = (a.H + a.KV) * hd + kvh * hd;
        return c < g * hd ? qcol + c : (c < (g + 1) * hd ? kcol + c - g * hd : vcol + c - (g + 1) * hd);
    };
    int col_e[4];
    float bias_e[4], part_e[2][4], freq_e = 0.f;
    int slot = -1;
    if constexpr (FUSED) {
        const size_t p1 = (size_t)min(1, a.n_partials - 1) * pstride;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            col_e[u] = column(tid + u * 256);
            bias_e[u] = bias[col_e[u]];
            part_e[0][u] = row0[col_e[u]];
            part_e[1][u] = row0[p1 + col_e[u]];
        }
        freq_e = (a.inv_freq ? a.inv_freq : row0)[min(tid, hd / 2 - 1)];
        slot = a.slot_map[s];
        __builtin_amdgcn_sched_barrier(0);  // the loads stay up here
    }

    // The first tile depends on nothing the prologue computes: it is requested before the prologue
    // so that its latency hides behind it.
    DecodeTile next;
    Pages ahead = lookup(t0 + wave);
    load_tile(ahead, next);
    ahead = lookup(t0 + wave + 4);

    Frag qf[NKS];
    if constexpr (FUSED) {
        const int half = hd / 2;
        float* rowv = &sm_o[0][0][0];                                   // (g + 2) * hd sums, then ...
        elem_t* qrot = reinterpret_cast<elem_t*>(rowv + (g + 2) * hd);  // ... the g rotated queries, rounded
        // the angles, while the sums are on their way
        if (tid < half) {
            float c = 1.f, sv = 0.f;
            if (a.inv_freq) sincosf((float)pos * freq_e, &sv, &c);
            cs[tid] = c;
            sn[tid] = sv;
        }
        // Further partial sums, eight at a time, all of their loads asked for before the first is added: the
        // sums were written by the kernel before this one, and one load after the other would be as many trips
        // to them (beyond the last partial sum: the last one again, not added).
        auto add_partials = [&](int first, const int (&col)[4], float (&v)[4]) {
            constexpr int NB = 8;
            for (int p0 = first; p0 < a.n_partials; p0 += NB) {
                float t[NB][4];
#pragma unroll
                for (int q = 0; q < NB; ++q) {
                    const size_t po = (size_t)min(p0 + q, a.n_partials - 1) * pstride;
#pragma unroll
                    for (int u = 0; u < 4; ++u) t[q][u] = row0[po + col[u]];
                }
#pragma unroll
                for (int q = 0; q < NB; ++q)
                    if (p0 + q < a.n_partials) {
#pragma unroll
                        for (int u = 0; u < 4; ++u) v[u] += t[q][u];
                    }
            }
        };
        {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = bias_e[u] * bias_on + part_e[0][u] + (a.n_partials > 1 ? part_e[1][u] : 0.f);
            add_partials(2, col_e, v);
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (tid + u * 256 < width) rowv[tid + u * 256] = v[u];
        }
        for (int c0 = tid + 4 * 256; c0 < width; c0 += 4 * 256) {  // more than 1,024 columns: many large heads
            int col[4];
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                col[u] = column(c0 + u * 256);
                v[u] = bias[col[u]] * bias_on;
            }
            add_partials(0, col, v);
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (c0 + u * 256 < width) rowv[c0 + u * 256] = v[u];
        }
        __syncthreads();
        // Rotation, one pair (d, d + hd / 2) of a query head or of the key per thread at a time; the row's
        // own key and value are rounded as the page holds them, and one block writes them there (nobody
        // reads them in this launch).
        {
            const int page = slot >= 0 ? slot / ps : 0, off = slot >= 0 ? slot % ps : 0;
            const bool writes = sp == 0 && slot >= 0;
            elem_t* kdst = const_cast<elem_t*>(a.kpool) + (((size_t)page * a.KV + kvh) * ps + off) * hd;
            elem_t* vdst = const_cast<elem_t*>(a.vpool) + ((size_t)page * a.KV + kvh) * hd * ps + off;
            const float inv_half = 1.0f / (float)half;
            for (int i = tid; i < (g + 1) * half; i += 256) {
                const int row = (int)(((float)i + 0.5f) * inv_half), j = i - row * half;  // i < 17 * 128: exact
                const float x0 = rowv[row * hd + j], x1 = rowv[row * hd + j + half];
                const elem_t r0 = from_f32<elem_t>(x0 * cs[j] - x1 * sn[j]), r1 = from_f32<elem_t>(x0 * sn[j] + x1 * cs[j]);
                if (row < g) {
                    qrot[row * hd + j] = r0;
                    qrot[row * hd + j + half] = r1;
                } else {
                    knew[j] = to_f32(r0);
                    knew[j + half] = to_f32(r1);
                    if (writes) {
                        kdst[j] = r0;
                        kdst[j + half] = r1;
                    }
                }
            }
            const float* vv_ = rowv + (g + 1) * hd;
            for (int d = tid; d < hd; d += 256) {
                const elem_t ve = from_f32<elem_t>(vv_[d]);
                vnew[d] = to_f32(ve);
                if (writes) vdst[(size_t)d * ps] = ve;
            }
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const int d0 = ks * 32 + grp * 8;
            qf[ks] = (valid && d0 < hd) ? frag_load(qrot + r16 * hd + d0) : frag_zero();
        }
        __syncthreads();  // the staging area is free again: the waves hand their results over through it
    } else {
        const elem_t* qrow = a.q + ((size_t)s * a.H + head) * hd;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const int d0 = ks * 32 + grp * 8;
            qf[ks] = (valid && d0 < hd) ? frag_load(qrow + d0) : frag_zero();
        }
    }

    f32x4 acc_o[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i) acc_o[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run = NEG_BIG, l_run = 0.f;

    auto process = [&](const DecodeTile& cur, int t) {
        const int kt0 = t * DBKV;
        f32x4 sc[DNT];
#pragma unroll
        for (int nt = 0; nt < DNT; ++nt) {
            sc[nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) mma_16x16x32(sc[nt], cur.kf[nt][ks], qf[ks]);
        }
        float tmax = NEG_BIG;
#pragma unroll
        for (int nt = 0; nt < DNT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = kt0 + score_key(nt, i);
                const bool ok = valid && key < kv_len && key >= lo_key;
                const float v = ok ? sc[nt][i] * a.scale : -INFINITY;
                sc[nt][i] = v;
                tmax = fmaxf(tmax, v);
            }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = exp_f(m_run - m_new);
        float psum = 0.f;
#pragma unroll
        for (int nt = 0; nt < DNT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = exp_f(sc[nt][i] - m_new);
                sc[nt][i] = p;
                psum += p;
            }
        psum += __shfl_xor(psum, 16, WAVE);
        psum += __shfl_xor(psum, 32, WAVE);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_o[dt][i] *= alpha;
#pragma unroll
        for (int pp = 0; pp < DNTP; ++pp) {
            Frag pf;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pf.v[i] = from_f32<elem_t>(sc[2 * pp][i]);
                pf.v[4 + i] = from_f32<elem_t>((2 * pp + 1 < DNT) ? sc[(2 * pp + 1) % DNT][i] : 0.f);
            }
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) mma_16x16x32(acc_o[dt], cur.vf[pp][dt], pf);
        }
    };
    // Two tile buffers take turns, so that no tile is copied.  The loads of the tile after next are
    // issued before the current tile is multiplied, and the scheduler may not move them below it:
    // it would, to keep fewer registers live, and the loads' latency would then lie open.
    DecodeTile other;
    for (int t = t0 + wave; t < t1; t += 8) {
        load_tile(ahead, other);  // of tile t + 4; past the split it reads one line of the pool's start
        ahead = lookup(t + 8);
        __builtin_amdgcn_sched_barrier(0);
        process(next, t);
        if (t + 4 >= t1) break;
        load_tile(ahead, next);
        ahead = lookup(t + 12);
        __builtin_amdgcn_sched_barrier(0);
        process(other, t + 4);
    }

    if constexpr (FUSED) {
        // the row's own key: one more term of the online softmax, in wave 0 of split 0
        if (sp == 0 && wave == 0) {
            float dot = 0.f;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const int d0 = ks * 32 + grp * 8;
                if (d0 < hd) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) dot += to_f32(qf[ks].v[e]) * knew[d0 + e];
                }
            }
            dot += __shfl_xor(dot, 16, WAVE);
            dot += __shfl_xor(dot, 32, WAVE);
            const float sv = valid ? dot * a.scale : -INFINITY;
            const float m_new = fmaxf(m_run, sv);
            const float alpha = exp_f(m_run - m_new), p = exp_f(sv - m_new);
            l_run = l_run * alpha + p;
            m_run = m_new;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = dt * 16 + grp * 4 + i;
                    acc_o[dt][i] = acc_o[dt][i] * alpha + (d < hd ? p * vnew[d] : 0.f);
                }
        }
    }

    // waves 1..3 hand their state to wave 0
    if (wave > 0) {
        if (grp == 0) { sm_m[wave - 1][r16] = m_run; sm_l[wave - 1][r16] = l_run; }
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) sm_o[wave - 1][dt * 16 + grp * 4 + i][r16] = acc_o[dt][i];
    }
    __syncthreads();
    if (wave > 0) return;
    float m_all = m_run;
#pragma unroll
    for (int w = 0; w < 3; ++w) m_all = fmaxf(m_all, sm_m[w][r16]);
    const float c0 = exp_f(m_run - m_all);
    float l_all = l_run * c0;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc_o[dt][i] *= c0;
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        const float c = exp_f(sm_m[w][r16] - m_all);
        l_all += sm_l[w][r16] * c;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_o[dt][i] += sm_o[w][dt * 16 + grp * 4 + i][r16] * c;
    }
    if (!valid) return;
    if (a.nsplit == 1) {
        const float inv = l_all > 0.f ? 1.0f / l_all : 0.f;
        elem_t* orow = a.out + ((size_t)s * a.H + head) * hd;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            const int d0 = dt * 16 + grp * 4;
            if (d0 < hd) {
#pragma unroll
                for (int i = 0; i < 4; ++i) orow[d0 + i] = from_f32<elem_t>(acc_o[dt][i] * inv);
            }
        }
    } else {
        const size_t base = ((size_t)s * a.H + head) * a.nsplit + sp;
        float* po = a.part_o + base * hd;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            const int d0 = dt * 16 + grp * 4;
            if (d0 < hd) {
#pragma unroll
                for (int i = 0; i < 4; ++i) po[d0 + i] = acc_o[dt][i];
            }
        }
        if (grp == 0) { a.part_ml[base * 2] = m_all; a.part_ml[base * 2 + 1] = l_all; }
    }
}

// out[row, :] = sum_sp o_sp exp(m_sp - m) / sum_sp l_sp exp(m_sp - m), splits in order.
// One wave per (request, head); lane = element of the head (in chunks of 64).  The splits' outputs are
// asked for eight at a time, the first eight together with the (max, sum) pairs and before anything
// is computed from those, so that the kernel waits for memory once.
__global__ __launch_bounds__(64) void decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                          elem_t* __restrict__ out, int hd, int nsplit) {
    arguments_now(part_o, part_ml, out, hd, nsplit);
    constexpr int BATCH = 8;
    const size_t row = blockIdx.x;  // (request, head)
    const int lane = threadIdx.x;
    const float* ml = part_ml + row * nsplit * 2;
    const float* po = part_o + row * nsplit * hd;
    auto fetch = [&](int d, int sp0, float (&v)[BATCH]) {
#pragma unroll
        for (int u = 0; u < BATCH; ++u) v[u] = po[(size_t)min(sp0 + u, nsplit - 1) * hd + min(d, hd - 1)];
    };
    float first[BATCH];
    fetch(lane, 0, first);
    // every lane holds one split's (max, sum); nsplit <= 64
    const int own = min(lane, nsplit - 1);
    const float m_ld = ml[own * 2], l_ld = ml[own * 2 + 1];
    const float m_own = lane < nsplit ? m_ld : NEG_BIG;
    const float l_own = lane < nsplit ? l_ld : 0.f;
    const float m = wave_max(m_own);
    const float c = lane < nsplit ? exp_f(m_own - m) : 0.f;
    float l = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) l += __shfl(l_own * c, sp, WAVE);  // in split order
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const float coef = c * inv;  // of split `lane`; zero beyond the last split
    for (int d = lane; d - lane < hd; d += 64) {
        float o = 0.f;
        for (int sp0 = 0; sp0 < nsplit; sp0 += BATCH) {
            float v[BATCH];
            if (d == lane && sp0 == 0) {
#pragma unroll
                for (int u = 0; u < BATCH; ++u) v[u] = first[u];
            } else {
                fetch(d, sp0, v);
            }
#pragma unroll
            for (int u = 0; u < BATCH; ++u) o += v[u] * __shfl(coef, min(sp0 + u, 63), WAVE);  // zero beyond the last split
        }
        if (d < hd) out[row * hd + d] = from_f32<elem_t>(o);
    }
}

}  // namespace ms

using namespace ms;

#define MS_CAT2(a, b) a##b
#define MS_CAT(a, b) MS_CAT2(a, b)

// Attention of a mixed batch.  `work` lists (request index, first flat row) for every ROWS_PER_BLOCK
// flat rows of a request (ms_attention_rows_per_block_nd<N>() tells the caller the number; the general kernel
// takes an item as SUB_BLOCKS blocks of 64 rows, the kernel of 32-row tiles as one block); an item of
// request -1 only fills a list up and is skipped; see the file comment.  window = 0 means all keys.  max_key_groups = 0 lets the
// launcher choose how many key groups share a block (1, 2 or 4) from the width of the block tables;
// a positive value asks for that many (as far as this tile has them).  nsplit > 1 cuts every block's
// keys over that many blocks (few blocks of rows over long contexts would leave most of the chip idle
// and run as long as their chain of tiles); T is the number of rows, part_o [T, H, nsplit, hd] and
// part_ml [T, H, nsplit, 2] are float workspaces.
// Whether a launch with these sizes runs in the kernel of 32-row tiles: where the block tables allow contexts of
// 2,048 keys and more (measured on one prompt of the 0.5B head shape: 512 tokens 13.9 against 11.9 us, 2,048 32.2
// against 34.4, 4,096 60 against 83, 8,192 194 against 252), the head size is the tile's, and a block's share of the
// block table fits its place in LDS (asked for by name with max_key_groups = 32).
static bool takes_rows32(int hd, int ps, int table_stride, int window, int max_key_groups) {
#ifdef MS_HAS_ROWS32
    const long span = window > 0 ? (long)window + BKV : (long)table_stride * ps;
    const long pages_of_span = window > 0 ? ((long)window + 2 * ROWS_PER_BLOCK + r32::ROUND) / ps + 2 : (long)table_stride;
    return hd == HDT && pages_of_span <= r32::MAX_TABLE && (max_key_groups == 32 || (max_key_groups == 0 && span >= 2048));
#else
    (void)hd; (void)ps; (void)table_stride; (void)window; (void)max_key_groups;
    return false;
#endif
}

static int attention_compute_units() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        (void)hipGetLastError();
        cus = n;
    }
    return cus;
}

// Into how many blocks ms_paged_attention should cut the keys of every block of rows (its `nsplit`) when the caller
// leaves the choice to the library: n_work items of the work list, T rows in the step.  Few blocks of rows over long
// contexts leave most of the chip idle and run as long as their chain of tiles; cutting the chain fills the chip, at
// the price of the partial results' trip through memory and the merge's launch.  Block tables no wider than twice the
// step's rows are (or may be) those of prompts that run whole, whose blocks walk half the keys on average and whose
// longest block decides: cutting those only adds (0.5B heads, one prompt of 1,024 tokens 18.9 us uncut, 22.8 in two,
// 31.9 in four; 1,536 tokens 24.4 / 32.3 / 36.8).  The kernel of 32-row tiles holds one block a CU: it is cut so that
// blocks x splits stay within one round of the chip, at least 1,024 keys a split (256 rows behind 7,936 keys: 91 us
// uncut, 25.8 in eight, 35.2 in sixteen; 512 rows behind 7,680: 90.6, 36.2 in four, 50.4 in six; 1,024 rows behind
// 3,072: 49.4, 38.9 in two, 44.7 in four).  The cut depends on the batch, so results differ in rounding between batches.
extern "C" int MS_CAT(ms_attention_splits_nd, MS_ATTN_ND)(int n_work, int KV, int T, int hd, int ps, int table_stride, int window) {
    if (n_work < 1 || KV < 1 || ps < 1 || table_stride < 1) return 1;
    const long blocks = (long)n_work * KV;
    long span = (long)table_stride * ps;
    if (window > 0 && span > (long)window + 64) span = (long)window + 64;
    if (span <= 2L * T) return 1;
    long n;
    if (takes_rows32(hd, ps, table_stride, window, 0)) {
        n = std::min((long)attention_compute_units() / blocks, span / 1024);
    } else {
        if (blocks >= 192) return 1;
        n = std::min((384 + blocks - 1) / blocks, span / 512);
    }
    return (int)std::max(1L, std::min(n, (long)MAX_SPLITS));
}

extern "C" int MS_CAT(ms_paged_attention_nd, MS_ATTN_ND)(
    const void* q, const void* kpool, const void* vpool, void* out, const int* block_table, int table_stride,
    const int* seq_q_start, const int* seq_q_len, const int* seq_pos0, const int* work, int n_work, int H, int KV,
    int hd, int ps, int n_pages, int window, float scale, int max_key_groups, int T, int nsplit, float* part_o,
    float* part_ml, hipStream_t stream) {
    MS_REQUIRE(n_work > 0, "attention: no work");
    MS_REQUIRE(nsplit >= 1 && nsplit <= MAX_SPLITS && (nsplit == 1 || (part_o && part_ml && T > 0)),
               "attention: %d key splits (at most %d, with their workspaces)", nsplit, MAX_SPLITS);
    MS_REQUIRE(hd % 16 == 0 && hd > 0 && hd <= HDT, "attention: head size %d does not fit this tile of %d", hd, HDT);
    MS_REQUIRE(KV > 0 && H % KV == 0, "attention: %d heads are not a multiple of %d key/value heads", H, KV);
    MS_REQUIRE(ps % 16 == 0 && ps > 0, "attention: page size %d must be a multiple of 16", ps);
    MS_REQUIRE(window >= 0, "attention: window %d", window);
    MS_REQUIRE((double)n_pages * KV * ps * hd < 68719476736.0, "attention: a pool of %d pages exceeds 2^36 elements", n_pages);
    AttnArgs a{(const elem_t*)q, (const elem_t*)kpool, (const elem_t*)vpool, (elem_t*)out, block_table, seq_q_start,
               seq_q_len, seq_pos0, work, table_stride, H, KV, hd, ps, window, scale, n_work, 0, nsplit, part_o, part_ml};
    // key groups per block by the longest context the block tables allow (the lengths themselves
    // are on the device): short contexts have no chain worth cutting
    const long span = window > 0 ? (long)window + BKV : (long)table_stride * ps;
    // measured at 512 to 8,192 keys: two groups beat one by a quarter, four gain nothing over two
    int groups = 2;
    if (max_key_groups > 0) {
        groups = max_key_groups < MAX_KEY_GROUPS ? max_key_groups : MAX_KEY_GROUPS;
    } else if (span < 4 * BKV) {
        groups = 1;
    }
    MS_REQUIRE((long)n_work * KV * SUB_BLOCKS < 2147483647L, "attention: %d blocks of rows times %d key/value heads", n_work, KV);
    const dim3 grid((unsigned)(n_work * KV * SUB_BLOCKS), (unsigned)nsplit);
    // how many blocks of each variant a CU holds, and how many CUs there are: asked once
    static int cus = 0, resident[4] = {0, 0, 0, 0};
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1)
            n = 256;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident[0], paged_attention_kernel<1>, 256, 0) != hipSuccess) resident[0] = 1;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident[1], paged_attention_kernel<2>, 512, 0) != hipSuccess) resident[1] = 1;
        if constexpr (MAX_KEY_GROUPS >= 4) {
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident[2], paged_attention_kernel<4>, 1024, 0) != hipSuccess) resident[2] = 1;
        }
        (void)hipGetLastError();
        cus = n;
    }
    auto span_for = [&](int variant) { return resident[variant] == 2 ? (cus / (KV * SUB_BLOCKS) > 0 ? cus / (KV * SUB_BLOCKS) : 1) : 0; };
#ifdef MS_HAS_ROWS32
    {
        // tiles of 32 rows by 32 keys under four key groups, a block a CU (the list's order, longest contexts first, is
        // the order the blocks start in)
        if (takes_rows32(hd, ps, table_stride, window, max_key_groups)) {
            a.pair_span = 0;
            const dim3 grid32((unsigned)(n_work * KV), (unsigned)nsplit);
            hipLaunchKernelGGL(paged_attention_rows32_kernel, grid32, dim3(r32::KG * r32::GT), 0, stream, a);
            int rc32 = check_launch("paged_attention (32-row tiles)");
            if (rc32 || nsplit == 1) return rc32;
            hipLaunchKernelGGL(decode_merge_kernel, dim3((unsigned)((size_t)T * H)), dim3(64), 0, stream, part_o, part_ml, (elem_t*)out, hd, nsplit);
            return check_launch("attention_merge");
        }
    }
#endif
    if (groups >= 4 && MAX_KEY_GROUPS >= 4) {
        // sixteen waves leave each 128 registers, which only the small bfloat16 tiles fit into
        a.pair_span = span_for(2);
        if constexpr (MAX_KEY_GROUPS >= 4) hipLaunchKernelGGL(paged_attention_kernel<4>, grid, dim3(1024), 0, stream, a);
    } else if (groups >= 2) {
        a.pair_span = span_for(1);
        hipLaunchKernelGGL(paged_attention_kernel<2>, grid, dim3(512), 0, stream, a);
    } else {
        a.pair_span = span_for(0);
        hipLaunchKernelGGL(paged_attention_kernel<1>, grid, dim3(256), 0, stream, a);
    }
    int rc = check_launch("paged_attention");
    if (rc || nsplit == 1) return rc;
    hipLaunchKernelGGL(decode_merge_kernel, dim3((unsigned)((size_t)T * H)), dim3(64), 0, stream, part_o, part_ml, (elem_t*)out, hd, nsplit);
    return check_launch("attention_merge");
}

extern "C" int MS_CAT(ms_attention_rows_per_block_nd, MS_ATTN_ND)() { return ROWS_PER_BLOCK; }

// Attention of a step in which every request has exactly one row (row s = request s).
// part_o [S, H, nsplit, hd] and part_ml [S, H, nsplit, 2] are float workspaces (unused when
// nsplit == 1).  Needs H / KV <= 16.
extern "C" int MS_CAT(ms_decode_attention_nd, MS_ATTN_ND)(
    const void* q, const void* kpool, const void* vpool, void* out, float* part_o, float* part_ml, const int* block_table,
    int table_stride, const int* seq_pos0, int S, int H, int KV, int hd, int ps, int window, int nsplit, float scale,
    hipStream_t stream) {
    MS_REQUIRE(S > 0, "decode attention: no rows");
    MS_REQUIRE(hd % 16 == 0 && hd > 0 && hd <= HDT, "decode attention: head size %d does not fit this tile of %d", hd, HDT);
    MS_REQUIRE(KV > 0 && H % KV == 0 && H / KV <= 16, "decode attention: %d heads over %d key/value heads (at most 16 each)", H, KV);
    MS_REQUIRE(ps % 16 == 0 && ps > 0, "decode attention: page size %d must be a multiple of 16", ps);
    MS_REQUIRE(nsplit >= 1 && nsplit <= MAX_SPLITS && (nsplit == 1 || (part_o && part_ml)), "decode attention: %d splits (at most %d)", nsplit, MAX_SPLITS);
    DecodeArgs a{(const elem_t*)q, (const elem_t*)kpool, (const elem_t*)vpool, (elem_t*)out, part_o, part_ml, block_table,
                 seq_pos0, table_stride, H, KV, hd, ps, window, nsplit, scale, nullptr, nullptr, nullptr, nullptr, 0, 0};
    hipLaunchKernelGGL(decode_attention_kernel<false>, dim3((unsigned)S, (unsigned)KV, (unsigned)nsplit), dim3(256), 0, stream, a);
    int rc = check_launch("decode_attention");
    if (rc || nsplit == 1) return rc;
    hipLaunchKernelGGL(decode_merge_kernel, dim3((unsigned)(S * H)), dim3(64), 0, stream, part_o, part_ml, (elem_t*)out, hd, nsplit);
    return check_launch("decode_merge");
}

// Scratch memory of ms_decode_attention_noalloc_nd*: the splits' partial outputs, then their (max, sum)
// pairs.  Each GPU on which the library runs holds its own copy of this array, at its own address, until
// the process ends.  In host code the name is only a handle for hipGetSymbolAddress; the address that
// kernels and copies take is looked up once per device and kept in g_scratch_ptr.
constexpr size_t NOALLOC_SCRATCH_FLOATS = (size_t)1 << 20;  // 4 MiB
static __device__ __align__(256) float scratch[NOALLOC_SCRATCH_FLOATS];
constexpr int NOALLOC_MAX_DEVICES = 64;
static float* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};
static std::mutex g_scratch_mutex;

// The device address of `scratch` on the current device (null and an error message if it cannot be had).
static float* scratch_of_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= NOALLOC_MAX_DEVICES) {
        ms::set_error("decode attention (no allocation): device %d (%s); at most %d devices", dev, hipGetErrorString(e),
                      NOALLOC_MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            ms::set_error("decode attention (no allocation): hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

// ms_decode_attention_nd* for callers that cannot allocate (declared in no_alloc.h): the same kernels, with the
// workspace of the splits in `scratch` instead of two buffers of the caller.  It calls no hipMalloc, hipFree or
// allocating library routine.  S * H * nsplit * (hd + 2) floats must fit NOALLOC_SCRATCH_FLOATS.  Nothing in
// the scratch has to start at zero (every block writes its split's partial result, an empty split a sum
// of zero); it keeps the last call's contents, and all calls on one GPU share it, so two calls that
// overlap on one GPU (two streams, two threads) race: the caller orders them.
extern "C" int MS_CAT(ms_decode_attention_noalloc_nd, MS_ATTN_ND)(
    const void* q, const void* kpool, const void* vpool, void* out, const int* block_table, int table_stride,
    const int* seq_pos0, int S, int H, int KV, int hd, int ps, int window, int nsplit, float scale, hipStream_t stream) {
    MS_REQUIRE(S > 0 && H > 0 && hd > 0 && nsplit >= 1, "decode attention (no allocation): %d rows, %d heads, head size %d, %d splits",
               S, H, hd, nsplit);
    float* part_o = nullptr;
    float* part_ml = nullptr;
    if (nsplit > 1) {
        const double need = (double)S * H * nsplit * (hd + 2);
        MS_REQUIRE(need <= (double)NOALLOC_SCRATCH_FLOATS,
                   "decode attention (no allocation): %d rows x %d heads x %d splits x (%d + 2) floats = %.0f exceed the scratch of %zu floats",
                   S, H, nsplit, hd, need, NOALLOC_SCRATCH_FLOATS);
        float* base = scratch_of_current_device();
        if (!base) return 1;
        part_o = base;
        part_ml = base + (size_t)S * H * nsplit * hd;
    }
    return MS_CAT(ms_decode_attention_nd, MS_ATTN_ND)(q, kpool, vpool, out, part_o, part_ml, block_table, table_stride,
                                                      seq_pos0, S, H, KV, hd, ps, window, nsplit, scale, stream);
}
// The most floats of scratch a step may need.  The call also looks up the scratch's address on the current device
// (the set-up that the entry point would otherwise do at its first call there): a caller that is about to capture
// a stream calls this first, on each device it uses, and the entry point itself then makes nothing but launches.
extern "C" long MS_CAT(ms_decode_attention_noalloc_max_floats_nd, MS_ATTN_ND)() {
    (void)scratch_of_current_device();
    return (long)NOALLOC_SCRATCH_FLOATS;
}

// The same from the partial sums of the q/k/v projection: adds them and the bias, rotates q and k
// by the row's position, writes k and v into the row's page, and attends; a second launch merges
// the splits.  (Merging in the block that finishes last needs a device-wide fence in every block,
// which on this chip writes back a whole L2 and costs more than the launch it saves.)
// qkv is float [n_partials, S, stride] with the q heads, then the k heads, then the v heads.
extern "C" int MS_CAT(ms_decode_attention_fused_nd, MS_ATTN_ND)(
    const float* qkv, int n_partials, int stride, const float* bias, const float* inv_freq, const int* slot_map,
    void* kpool, void* vpool, void* out, float* part_o, float* part_ml, const int* block_table,
    int table_stride, const int* seq_pos0, int S, int H, int KV, int hd, int ps, int window, int nsplit, float scale,
    hipStream_t stream) {
    MS_REQUIRE(S > 0 && n_partials >= 1, "decode attention: no rows");
    MS_REQUIRE(hd % 16 == 0 && hd > 0 && hd <= HDT, "decode attention: head size %d does not fit this tile of %d", hd, HDT);
    MS_REQUIRE(KV > 0 && H % KV == 0 && H / KV <= 16, "decode attention: %d heads over %d key/value heads (at most 16 each)", H, KV);
    MS_REQUIRE(ps % 16 == 0 && ps > 0, "decode attention: page size %d must be a multiple of 16", ps);
    MS_REQUIRE(stride >= (H + 2 * KV) * hd, "decode attention: row stride %d too small", stride);
    MS_REQUIRE(nsplit >= 1 && nsplit <= MAX_SPLITS && (nsplit == 1 || (part_o && part_ml)), "decode attention: %d splits (at most %d)", nsplit, MAX_SPLITS);
    MS_REQUIRE(slot_map && kpool && vpool, "decode attention: the fused form writes the cache");
    DecodeArgs a{nullptr, (const elem_t*)kpool, (const elem_t*)vpool, (elem_t*)out, part_o, part_ml, block_table, seq_pos0,
                 table_stride, H, KV, hd, ps, window, nsplit, scale, qkv, bias, inv_freq, slot_map, n_partials, stride};
    hipLaunchKernelGGL(decode_attention_kernel<true>, dim3((unsigned)S, (unsigned)KV, (unsigned)nsplit), dim3(256), 0, stream, a);
    int rc = check_launch("decode_attention_fused");
    if (rc || nsplit == 1) return rc;
    hipLaunchKernelGGL(decode_merge_kernel, dim3((unsigned)(S * H)), dim3(64), 0, stream, part_o, part_ml, (elem_t*)out, hd, nsplit);
    return check_launch("decode_merge");
}

extern "C" int MS_CAT(ms_attention_key_tile_nd, MS_ATTN_ND)() { return DBKV; }  // of the decode kernel
