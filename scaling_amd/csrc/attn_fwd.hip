// Attention forward for gfx950 (bf16 MFMA, fp32 online softmax, causal / packed-document masks, GQA).
//
// Workgroup = NW wavefronts (4 or 8); every wavefront owns 32 consecutive query tokens of one head.
// With 8 wavefronts, wavefronts w and w + 4 share a SIMD and run half a tile out of phase (enforced by
// the barriers), so one issues MFMAs while the other runs its softmax on the VALU.
// Keys/values stream through LDS in tiles of 64 tokens, loaded global -> LDS directly (no staging
// registers) two tile-steps ahead into a ring of three swizzled stages.
// Per tile:
//     S^T = K * Q^T            A = K tile rows from LDS, B = Q fragment held in registers
//     online softmax           each lane owns ONE query (C column): the row max / sum are in-lane
//                              reductions plus a single exchange with lane ^ 32.  The running max is
//                              only raised (and O rescaled) when it grows by more than 2^8, so the
//                              rescale of the 64 accumulator registers is skipped on most tiles.
//     O^T += V^T * P^T         B = P^T taken straight from the S^T accumulators (no LDS round trip),
//                              A = V^T obtained with LDS transpose reads from the token-major V tile
// The mask is a per-lane key interval [klo, khi) derived from the cumulative sequence lengths; tiles
// outside the union of the intervals are never loaded, tiles inside every interval skip the compare.
#include "attn_common.h"

#include <type_traits>

namespace {

constexpr int BN = 64;               // keys per tile
constexpr float kRescaleGap = 8.0f;  // log2 units by which a row max may lag before O is rescaled

// ROTM: 0 = q / k are used as they are; 1 = rotate-half rotary applied to q and k on load (tables in the I/O dtype),
// 2 = interleaved-pair rotary applied to q and k on load (fp32 tables); 3 / 4 = the same two rotations applied to q
// only (k arrives rotated: the training path rotates it once with the stand-alone kernel, because every K tile is
// loaded by each query block of each head of its group and would be rotated a few hundred times over in here, whereas
// a Q row is loaded exactly once).  With p.q_rot the rotated q is also written out (the backward kernels stream it).
// SPLIT: the probabilities enter the P V product as two bf16 terms (P = hi + lo, lo = bf16(P - hi)), i.e. with 16
// mantissa bits instead of 8, at the price of a second pass of P V MFMAs (accuracy mode, MI_ATTN_SPLIT_P).
template <int D, int NW, int ROTM, bool DROP, bool SPLIT>
__global__ __launch_bounds__(64 * NW, 2) void attn_fwd_kernel(const AttnParams p) {
    constexpr int ROT = (ROTM == 1 || ROTM == 2) ? ROTM : 0;        // rotation of K inside the tile loaders
    constexpr int QROT = ROTM == 0 ? 0 : ((ROTM & 1) ? 1 : 2);      // rotation of the Q fragment
    constexpr int BM = 32 * NW;
    constexpr int KS = D / 16;            // contraction steps of Q K^T
    constexpr int DT = D / 32;            // 32-row tiles of O^T
    constexpr int NS = 4;                 // LDS stages per operand
    using Tile = LdsTile<D>;
    constexpr int RB = Tile::RB;
    constexpr int TILE = Tile::kBytes;
    constexpr int IPW = Tile::kInstrs / 4;   // direct-load instructions per loader wavefront and tile
    constexpr int KV_VECS = D / 32;       // 128-bit vectors per loader thread and tile (register-staged K, fused rotary)
    static_assert(D % 32 == 0 && D <= 128, "head_dim must be 32, 64, 96 or 128");
    static_assert(NW == 4 || NW == 8, "4 or 8 wavefronts");

    __shared__ __attribute__((aligned(1024))) char k_lds[NS * TILE];
    __shared__ __attribute__((aligned(1024))) char v_lds[NS * TILE];
    __shared__ int range_lds[2 * NW];
    __shared__ int lpt_lds[2 * kLptMax];  // work estimates and hand-out order of the query blocks (packed documents)

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: role and phase branches stay uniform
    const int lane = tid & 63, l32 = lane & 31, g = lane >> 5;

    // ---- work items --------------------------------------------------------------------------
    // The grid holds at most one workgroup per compute unit (its LDS rings leave room for no second one) and every
    // workgroup walks through several (head, query block) items: item lists are cut into passes of gridDim.x items,
    // heaviest first, and a workgroup takes the items at its own index in even passes and at the mirrored index in
    // odd ones, so that its heavy and light items add up to the same work as everybody else's (the mirror keeps
    // index mod 8, i.e. the XCD, so an XCD still sees a fixed set of heads).  This saves the few microseconds it takes
    // to retire a 128 KB workgroup and dispatch the next one onto the compute unit, once per item.
    const int nqb = (p.total_q + BM - 1) / BM;
    const int n_items = nqb * p.nq;
    const int G = gridDim.x;
    if (p.lpt_q) lpt_order<false>(p, nqb, BM, lpt_lds, lpt_lds + kLptMax);   // documents of different lengths, once per workgroup
    for (int pass = 0; pass * G < n_items; ++pass) {
    int idx = blockIdx.x;
    if (pass & 1) idx = (G & 7) == 0 ? ((idx & 7) | (((G >> 3) - 1 - (idx >> 3)) << 3)) : G - 1 - idx;
    const int item = pass * G + idx;
    if (item >= n_items) continue;        // the same for the whole workgroup
    int head, q_rank;
    head_and_rank(item, p.nq, head, q_rank);
    const int kvh = head / p.n_rep;
    const int qb = p.lpt_q ? lpt_lds[kLptMax + q_rank]                        // long query blocks first: by their real work,
                           : block_for_rank(q_rank, nqb, p.n_docs, p.across_q, true);   // or by position

    // ---- per-lane query, mask interval, Q fragment ---------------------------------------------
    const int tq = qb * BM + wave * 32 + l32;
    int klo, khi;
    key_range(p, tq, klo, khi);
    int wmin = khi > klo ? klo : 0x7fffffff, wmax = khi > klo ? khi : 0;
    elem8_t qf[KS];
    {
        const int tl = tq < p.total_q ? tq : p.total_q - 1;
        const elem_t* qrow = p.q + (int64_t)tl * p.q_st + (int64_t)head * p.q_sh + 8 * g;
        uint4 raw[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) raw[ks] = *reinterpret_cast<const uint4*>(qrow + 16 * ks);
        if constexpr (QROT == 1) {
            int64_t pos = p.pos_q[tl];
            pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
            const elem_t* cr = p.cos + pos * D + 8 * g;
            const elem_t* sr = p.sin + pos * D + 8 * g;
#pragma unroll
            for (int ks = 0; ks < KS / 2; ++ks) {
                const uint4 c = *reinterpret_cast<const uint4*>(cr + 16 * ks);
                const uint4 s = *reinterpret_cast<const uint4*>(sr + 16 * ks);
                rotate_pair(raw[ks], raw[ks + KS / 2], c, s, 1.0f);
            }
        } else if constexpr (QROT == 2) {
            int64_t pos = p.pos_q[tl];
            pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
            const float* cr = p.cos32 + pos * (D / 2) + 4 * g;   // features 16 ks + 8 g .. + 8 = pairs 8 ks + 4 g .. + 4
            const float* sr = p.sin32 + pos * (D / 2) + 4 * g;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                rotate_interleaved(raw[ks], ld128(cr + 8 * ks), ld128(sr + 8 * ks), 1.0f);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = __builtin_bit_cast(elem8_t, raw[ks]);
        if constexpr (QROT != 0) {
            if (p.q_rot != nullptr && tq < p.total_q) {
                elem_t* qo = p.q_rot + (int64_t)tq * p.q_st + (int64_t)head * p.q_sh + 8 * g;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) st128(qo + 16 * ks, raw[ks]);
            }
        }
    }
    // Consume the Q registers here: otherwise their loads count as possibly outstanding at the loop
    // entry, and every use inside the loop waits for the K/V prefetch issued just before it.
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]));
    wmin = group_min<64>(wmin);           // DPP lane reductions: no trips through the LDS crossbar
    wmax = group_max<64>(wmax);
    if (lane == 0) { range_lds[wave] = wmin; range_lds[NW + wave] = wmax; }
    __syncthreads();
    int bmin = 0x7fffffff, bmax = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) { bmin = min(bmin, range_lds[w]); bmax = max(bmax, range_lds[NW + w]); }
    if (bmax <= bmin) { bmin = 0; bmax = 0; }
    // the same in every lane; made scalar so that loop control and tile addresses stay on the scalar unit
    const int kt0 = __builtin_amdgcn_readfirstlane(bmin & ~(BN - 1));
    const int n_tiles = __builtin_amdgcn_readfirstlane((bmax - kt0 + BN - 1) / BN);

    // ---- accumulators ----------------------------------------------------------------------
    f32x16_t o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;

    // ---- tile loaders: with 8 wavefronts the first four stage V, the last four stage K ----------
    // V (and K unless the rotary embedding is fused) goes global -> LDS directly, two tile-steps ahead of
    // its use; with fused rotary K passes through registers to be rotated.
    const bool v_role = (NW == 4) || (wave < 4);
    const bool k_role = (NW == 4) || (wave >= 4);
    const int lw = wave & 3;                                         // loader index within the role
    const int ltid = (NW == 4) ? tid : (tid & 255);
    uint4 kraw[ROT ? KV_VECS : 1];
    constexpr int TAB_VECS = ROT == 2 ? KV_VECS : (ROT == 1 ? KV_VECS / 2 : 1);
    uint4 craw[TAB_VECS], sraw[TAB_VECS];                            // rotary table rows of the K tile
    int64_t kpos[ROT ? KV_VECS / 2 : 1];                             // their positions, fetched a tile ahead
    const elem_t* kbase = p.k + (int64_t)kvh * p.k_sh;
    const elem_t* vbase = p.v + (int64_t)kvh * p.v_sh;
    const int last_k = p.total_k - 1;

    auto load_kpos = [&](int kt) {
        if constexpr (ROT) {
#pragma unroll
            for (int j = 0; j < KV_VECS / 2; ++j) {
                const int row = (ltid + 256 * j) / (D / 16);
                kpos[j] = p.pos_k[min(kt + row, last_k)];
            }
        }
    };
    auto load_k = [&](int kt) {
        if constexpr (ROT) {
#pragma unroll
            for (int j = 0; j < KV_VECS / 2; ++j) {
                const int idx = ltid + 256 * j;
                const int row = idx / (D / 16), c = idx % (D / 16);
                const int tok = min(kt + row, last_k);
                const elem_t* kr = kbase + (int64_t)tok * p.k_st + 8 * c;
                kraw[2 * j] = ld128(kr);
                kraw[2 * j + 1] = ld128(kr + D / 2);
                int64_t pos = kpos[j];
                pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
                if constexpr (ROT == 1) {
                    craw[j] = ld128(p.cos + pos * D + 8 * c);
                    sraw[j] = ld128(p.sin + pos * D + 8 * c);
                } else {                          // pairs 4 c .. + 4 of the first vector, D / 4 further on for the second
                    craw[2 * j] = ld128(p.cos32 + pos * (D / 2) + 4 * c);
                    sraw[2 * j] = ld128(p.sin32 + pos * (D / 2) + 4 * c);
                    craw[2 * j + 1] = ld128(p.cos32 + pos * (D / 2) + 4 * c + D / 4);
                    sraw[2 * j + 1] = ld128(p.sin32 + pos * (D / 2) + 4 * c + D / 4);
                }
            }
        }
    };
    auto store_k = [&](int stage) {
        if constexpr (ROT) {
            char* ks = k_lds + stage * TILE;
#pragma unroll
            for (int j = 0; j < KV_VECS / 2; ++j) {
                const int idx = ltid + 256 * j;
                const int row = idx / (D / 16), c = idx % (D / 16);
                if constexpr (ROT == 1) {
                    rotate_pair(kraw[2 * j], kraw[2 * j + 1], craw[j], sraw[j], 1.0f);
                } else {
                    rotate_interleaved(kraw[2 * j], craw[2 * j], sraw[2 * j], 1.0f);
                    rotate_interleaved(kraw[2 * j + 1], craw[2 * j + 1], sraw[2 * j + 1], 1.0f);
                }
                st128(ks + Tile::unit_offset(row, c), kraw[2 * j]);
                st128(ks + Tile::unit_offset(row, c + D / 16), kraw[2 * j + 1]);
            }
        }
    };
    DmaPlan<D, IPW> k_plan, v_plan;
    k_plan.init(lw * IPW, lane, p.k_st);
    v_plan.init(lw * IPW, lane, p.v_st);
    // this wavefront's share of the direct loads of K / V tile `tile_idx`
    auto dma_k_tile = [&](int tile_idx) {
        if (tile_idx < n_tiles) k_plan.issue(kbase, p.k_st, kt0 + tile_idx * BN, last_k, k_lds + (tile_idx % NS) * TILE);
    };
    auto dma_v_tile = [&](int tile_idx) {
        if (tile_idx < n_tiles) v_plan.issue(vbase, p.v_st, kt0 + tile_idx * BN, last_k, v_lds + (tile_idx % NS) * TILE);
    };
    // ---- main loop ---------------------------------------------------------------------------
    // Each wavefront alternates an MFMA phase (O^T += V^T P^T of the previous tile, then S^T of the
    // current one) and a VALU phase (softmax of the current tile), with a workgroup barrier after each.
    // The second group of four wavefronts runs one phase behind the first, so on every SIMD one
    // wavefront is in its MFMA phase while the other is in its VALU phase.
    //   K tile n is read in phases 2n (group 0) and 2n+1 (group 1); V tile n in phases 2n+2 and 2n+3.
    //   At the end of its VALU phase i the V loader group (0) issues V tile i+2 and the K loader group (1)
    //   issues K tile i+3, each into the stage (of four) whose last reader finished two phases earlier; a
    //   loader waits for a tile right before the barrier that precedes its first read.
    // wave-uniform by construction: the extra barriers below must sit behind scalar branches
    const int grp = (NW == 8) ? wave >> 2 : 0;
    // number of direct-load instructions a loader issues for tiles [a, b)
    auto n_issued = [&](int a, int b) { return IPW * max(0, min(b, n_tiles) - a); };
    if (n_tiles > 0) {
        if (k_role) {
            if constexpr (ROT) {
                load_kpos(kt0);
                load_k(kt0);
                if (n_tiles > 1) load_kpos(kt0 + BN);
                store_k(0);
                if (n_tiles > 1) {
                    load_k(kt0 + BN);
                    if (n_tiles > 2) load_kpos(kt0 + 2 * BN);
                }
            } else {
                dma_k_tile(0);
                dma_k_tile(1);
                dma_k_tile(2);
            }
        }
        if (v_role) {
            dma_v_tile(0);
            dma_v_tile(1);
        }
        // K tile 0 must have landed; whatever was issued after it may still be in flight
        if (!ROT && k_role) wait_vmcnt_dyn(n_issued(1, 3) + (NW == 4 ? n_issued(0, 2) : 0));
    }
    __syncthreads();
    if (grp == 1) __syncthreads();

    const float c2 = p.scale_log2;
    int v_h0, v_h1;
    Tile::tr_bases(lane, v_h0, v_h1);
    const int k_row = Tile::row_base(l32, g);
    // dropout: hash input of this lane's query row at key pair 2 g, and the bit offset of its row of a 2 x 2 block
    uint32_t drop_xr = 0, drop_sel = 0;
    if constexpr (DROP) {
        drop_xr = drop_head_base(p.drop_seed, head) + (uint32_t)(tq >> 1) * kDropC1 + (uint32_t)(2 * g) * kDropC2;
        drop_sel = 16u * (uint32_t)(tq & 1);
    }
    f32x16_t s_acc[2];
    elem8_t pf[4];
    elem8_t pl[SPLIT ? 4 : 1];           // low-order terms of the probabilities
    bool pending = false;                 // pf holds the probabilities of the previous tile

    // One MFMA phase = up to 16 steps of O^T += V^T P^T (previous tile) followed by up to 16 steps of
    // S^T = K Q^T (current tile).  The A operands come from LDS through a ring of kDepth registers
    // filled kDepth steps ahead, so a wavefront that has its SIMD's matrix core to itself keeps it fed
    // in spite of the LDS latency; sched_barrier pins that order.
    constexpr int PV_STEPS = 4 * DT, S_STEPS = 2 * KS;
    constexpr int kDepth = 3;
    auto mfma_phase = [&](auto mode, const char* vt, const char* ks) {
        constexpr bool kPV = (decltype(mode)::value & 1) != 0, kS = (decltype(mode)::value & 2) != 0;
        constexpr int first = kPV ? 0 : PV_STEPS, last = kS ? PV_STEPS + S_STEPS : PV_STEPS;
        elem8_t ring[kDepth];
        auto fetch = [&](int i) -> elem8_t {
            if (i < PV_STEPS) {
                const int m = i / DT, dt = i % DT;
                return tr_pair(vt + (v_h0 ^ (dt << 6)) + 16 * m * RB, vt + (v_h1 ^ (dt << 6)) + 16 * m * RB);
            }
            const int ksi = (i - PV_STEPS) >> 1, t = (i - PV_STEPS) & 1;
            return *reinterpret_cast<const elem8_t*>(ks + (k_row ^ (ksi << 5)) + 32 * t * RB);
        };
        if constexpr (kS) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) s_acc[t][r] = 0.f;
        }
#pragma unroll
        for (int i = first; i < first + kDepth && i < last; ++i) ring[(i - first) % kDepth] = fetch(i);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = first; i < last; ++i) {
            const elem8_t a = ring[(i - first) % kDepth];
            if (i < PV_STEPS) {
                const int m = i / DT, dt = i % DT;
                o_acc[dt] = mfma_32x32x16(a, pf[m], o_acc[dt]);
                if constexpr (SPLIT) o_acc[dt] = mfma_32x32x16(a, pl[m], o_acc[dt]);
            } else {
                const int ksi = (i - PV_STEPS) >> 1, t = (i - PV_STEPS) & 1;
                s_acc[t] = mfma_32x32x16(a, qf[ksi], s_acc[t]);
            }
            if (i + kDepth < last) ring[(i - first) % kDepth] = fetch(i + kDepth);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for (int it = 0; it <= n_tiles; ++it) {
        const int kt = kt0 + it * BN;
        // ---- staging (register path of the fused rotary only) ----
        if constexpr (ROT) {
            if (k_role && it + 1 < n_tiles) {
                store_k((it + 1) % NS);
                if (it + 2 < n_tiles) {
                    load_k(kt + 2 * BN);
                    if (it + 3 < n_tiles) load_kpos(kt + 3 * BN);
                }
            }
        }
        // ---- MFMA phase ----
        const bool wave_active = it < n_tiles && (kt < wmax) && (kt + BN > wmin);
        {
            const char* vt = v_lds + ((it + NS - 1) % NS) * TILE;
            const char* ks = k_lds + (it % NS) * TILE;
            if (pending && wave_active) mfma_phase(std::integral_constant<int, 3>{}, vt, ks);
            else if (pending) mfma_phase(std::integral_constant<int, 1>{}, vt, ks);
            else if (wave_active) mfma_phase(std::integral_constant<int, 2>{}, vt, ks);
        }
        if (it == n_tiles) break;
        // K tile it+1 is read after this barrier (by group 0): the K loaders of group 1 make sure it
        // has landed; only K tile it+2 was issued after it
        if (NW == 8 && !ROT && k_role) wait_vmcnt_dyn(n_issued(it + 2, it + 3));
        __syncthreads();

        // ---- VALU phase ----
        pending = wave_active;
        if (wave_active) {
            // tiles that cross an interval boundary of some lane get the compare; the others skip it
            if (__any((kt < klo) || (kt + BN > khi))) {
                int rel0 = kt + 4 * g - klo;
                asm volatile("" : "+v"(rel0));   // opaque: keeps the 32 compares inside this branch
                const unsigned len = (unsigned)(khi - klo);
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const unsigned rel = (unsigned)(rel0 + 32 * t + 8 * (r >> 2) + (r & 3));
                        if (rel >= len) s_acc[t][r] = -INFINITY;
                    }
            }
            float mx = fmaxf(s_acc[0][0], s_acc[1][0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(mx, fmaxf(s_acc[0][r], s_acc[1][r]));
            mx = pair_max(mx);
            const float m_cand = mx * c2;
            if (__any(m_cand > m_i + kRescaleGap)) {
                const float m_new = fmaxf(m_i, m_cand);
                float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_i - m_new);
                // opaque to the optimiser: keeps the 64 multiplies below inside this rarely taken
                // branch instead of being speculated onto every tile
                asm volatile("" : "+v"(alpha));
                m_i = m_new;
                l_i *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_acc[dt][r] *= alpha;
            }
            const float m_use = (m_i == -INFINITY) ? 0.f : m_i;
            float rs0 = 0.f, rs1 = 0.f;
            const uint32_t drop_xt = drop_xr + (uint32_t)(kt >> 1) * kDropC2;   // used with DROP only
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const int t = m >> 1, r0 = 8 * (m & 1);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float ev = fast_exp2(s_acc[t][r0 + e] * c2 - m_use);
                    if (e & 1) rs1 += ev; else rs0 += ev;
                    pf[m][e] = (elem_t)ev;
                    if constexpr (SPLIT) pl[m][e] = (elem_t)(ev - (float)pf[m][e]);
                }
                if constexpr (DROP) {
                    // the row sum above stays that of the full softmax; only the P that multiplies V is masked
                    // (register r0 + e holds key kt + 32 t + 8 a + 4 g + c with 4 a + c = r0 + e)
#pragma unroll
                    for (int pi = 0; pi < 4; ++pi) {
                        const int a = 2 * (m & 1) + (pi >> 1), j = pi & 1;
                        const uint32_t h = lowbias32(drop_xt + (uint32_t)(16 * t + 4 * a + j) * kDropC2);
                        if (drop_byte(h, drop_sel) < p.drop_thr) { pf[m][2 * pi] = (elem_t)0.f; if constexpr (SPLIT) pl[m][2 * pi] = (elem_t)0.f; }
                        if (drop_byte(h, drop_sel + 8) < p.drop_thr) { pf[m][2 * pi + 1] = (elem_t)0.f; if constexpr (SPLIT) pl[m][2 * pi + 1] = (elem_t)0.f; }
                    }
                }
            }
            l_i += rs0 + rs1;
        }
        // Direct loads are issued here, at the end of the shorter phase: the texture path takes a few
        // hundred cycles to accept a tile's worth of them, and this wavefront would otherwise idle at
        // the barrier while its SIMD neighbour finishes the MFMA phase.
        if (v_role) dma_v_tile(it + 2);
        if (!ROT && k_role) dma_k_tile(it + 3);
        // V tile it (and with one group K tile it+1) is read after this barrier
        if (NW == 8) {
            if (v_role) wait_vmcnt_dyn(n_issued(it + 1, it + 3));
        } else {
            wait_vmcnt_dyn(n_issued(it + 1, it + 3) + (ROT ? 0 : n_issued(it + 2, it + 4)));
        }
        __syncthreads();
    }
    if (grp == 0) __syncthreads();

    // ---- epilogue ------------------------------------------------------------------------------
    const float l_tot = pair_sum(l_i);
    const float inv = (l_tot > 0.f ? 1.0f / l_tot : 0.f) * (DROP ? p.drop_rscale : 1.0f);
    if (tq < p.total_q) {
        elem_t* orow = p.o + (int64_t)tq * p.o_st + (int64_t)head * p.o_sh + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const uint32_t w0 = pack_elem2(o_acc[dt][4 * a] * inv, o_acc[dt][4 * a + 1] * inv);
                const uint32_t w1 = pack_elem2(o_acc[dt][4 * a + 2] * inv, o_acc[dt][4 * a + 3] * inv);
                *reinterpret_cast<uint2*>(orow + 32 * dt + 8 * a) = make_uint2(w0, w1);
            }
        if (g == 0 && p.lse != nullptr) {
            const float lse = l_tot > 0.f ? (m_i + __log2f(l_tot)) * 0.6931471805599453f : INFINITY;
            p.lse[(int64_t)head * p.total_q + tq] = lse;
        }
    }
    __syncthreads();                      // the LDS rings and range_lds are free for the next item
    }   // items
}

template <int D, int NW, int ROT, bool DROP, bool SPLIT = false> int launch(const AttnParams& p, hipStream_t st) {
    constexpr int BM = 32 * NW;
    const int64_t nqb = ((int64_t)p.total_q + BM - 1) / BM;
    const int64_t items = nqb * p.nq;
    if (items > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "attn_fwd: too many work items");
    const int cus = mi_compute_units();
    const int64_t grid = items < cus ? items : cus;
    attn_fwd_kernel<D, NW, ROT, DROP, SPLIT><<<dim3((unsigned)grid), dim3(64 * NW), 0, st>>>(p);
    return mi_check_launch("attn_fwd");
}

// rot: 0 = none, 1 = rotate-half, 2 = interleaved pairs; q_only: k arrives rotated
template <int D> int launch_d(const AttnParams& p, int rot, bool q_only, int nw, bool split, hipStream_t st) {
    if (split) {      // accuracy mode: 256-query workgroups, no dropout, rotary on q only
        if (p.drop_thr != 0 || (rot && !q_only)) return mi_fail(MI_E_SHAPE, "attn_fwd: MI_ATTN_SPLIT_P takes no dropout and rotary on q only");
        if constexpr (D == 64 || D == 128) {
            if (rot == 2) return launch<D, 8, 4, false, true>(p, st);
            if (rot == 1) return launch<D, 8, 3, false, true>(p, st);
        } else {
            if (rot) return mi_fail(MI_E_SHAPE, "attn_fwd: fused rotary needs head_dim 64 or 128");
        }
        return launch<D, 8, 0, false, true>(p, st);
    }
    if (rot) {
        if constexpr (D == 64 || D == 128) {
            if (p.drop_thr != 0) {           // dropout: one tiling per head_dim (256-query workgroups), rotary on q only
                if (!q_only) return mi_fail(MI_E_SHAPE, "attn_fwd: with dropout the fused rotary covers q only (pass rotated k and position_ids_k = NULL)");
                return rot == 2 ? launch<D, 8, 4, true>(p, st) : launch<D, 8, 3, true>(p, st);
            }
            if (q_only) {
                if (rot == 2) return nw == 8 ? launch<D, 8, 4, false>(p, st) : launch<D, 4, 4, false>(p, st);
                return nw == 8 ? launch<D, 8, 3, false>(p, st) : launch<D, 4, 3, false>(p, st);
            }
            if (rot == 2) return nw == 8 ? launch<D, 8, 2, false>(p, st) : launch<D, 4, 2, false>(p, st);
            return nw == 8 ? launch<D, 8, 1, false>(p, st) : launch<D, 4, 1, false>(p, st);
        } else {
            return mi_fail(MI_E_SHAPE, "attn_fwd: fused rotary needs head_dim 64 or 128");
        }
    }
    if (p.drop_thr != 0) return launch<D, 8, 0, true>(p, st);
    return nw == 8 ? launch<D, 8, 0, false>(p, st) : launch<D, 4, 0, false>(p, st);
}

}  // namespace

int MI_ENTRY(mi_attn_fwd_impl)(const mi_attn_args* a) {
    int rc = mi_attn_validate(a, "attn_fwd");
    if (rc != MI_OK) return rc;
    if (!a->o) return mi_fail(MI_E_NULL, "attn_fwd: o is null");
    if (!mi_aligned16(a->o) || a->o_stride_token % 8 || a->o_stride_head % 8)
        return mi_fail(MI_E_ALIGN, "attn_fwd: o must be 16-byte aligned with strides multiple of 8");
    if (a->total_q == 0) return MI_OK;
    AttnParams p;
    mi_attn_fill_params(a, &p);
    const int rot = a->rotary_cos == nullptr ? 0 : (a->rotary_interleaved ? 2 : 1);
    const bool q_only = a->position_ids_k == nullptr;
    if (a->q_rot_out) {
        if (!rot) return mi_fail(MI_E_NULL, "attn_fwd: q_rot_out needs the fused rotary");
        if (!mi_aligned16(a->q_rot_out)) return mi_fail(MI_E_ALIGN, "attn_fwd: q_rot_out must be 16-byte aligned");
        p.q_rot = (elem_t*)a->q_rot_out;
    }
    // 256-query workgroups (two groups of wavefronts a phase apart) beat 128-query ones at every size measured,
    // also when they leave most compute units without work (1 x 512 tokens x 32 heads: 22 against 25 us,
    // 1 x 2048: 65 against 93 us); the smaller tiling only serves inputs that do not fill one workgroup
    int nw = p.total_q > 128 ? 8 : 4;
    if (a->flags & MI_ATTN_QG1) nw = 4;
    if (a->flags & MI_ATTN_QG2) nw = 8;
    const bool split = (a->flags & MI_ATTN_SPLIT_P) != 0;
    if (split) nw = 8;
    // equal-length documents: across them only when every query head has its own K / V; documents of different lengths:
    // longest-processing-time first also with shared K / V (measured at 7 documents of 545 - 2023 tokens, 32 / 8 heads:
    // forward -2 %, dQ -3 %; the query heads of a group still run the same block together)
    const int per_doc = mi_blocks_per_doc(a->total_q, a->n_docs, 32 * nw);
    if (p.n_rep == 1) p.across_q = per_doc;
    p.lpt_q = mi_use_lpt(a->total_q, a->n_docs, 32 * nw, per_doc);
    hipStream_t st = (hipStream_t)a->stream;
    switch (a->head_dim) {
        case 32: return launch_d<32>(p, rot, q_only, nw, split, st);
        case 64: return launch_d<64>(p, rot, q_only, nw, split, st);
        case 96: return launch_d<96>(p, rot, q_only, nw, split, st);
        case 128: return launch_d<128>(p, rot, q_only, nw, split, st);
        default: return mi_fail(MI_E_SHAPE, "attn_fwd: head_dim %d unsupported (32, 64, 96, 128)", a->head_dim);
    }
}
