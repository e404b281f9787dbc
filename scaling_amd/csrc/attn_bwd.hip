// Attention backward for gfx950 (bf16 MFMA, fp32 softmax recomputation from the saved log-sum-exp).
//
// Three kernels (four with fewer than 8 KV heads), no atomics, fixed summation order (bit-reproducible):
//   1. delta[h][t] = sum_d dO[t][h][d] * O[t][h][d]
//   2. dK/dV: a workgroup owns 128 keys of one KV head (K and V rows stay in LDS), loops over the query
//      heads of the group and over 64-query tiles staged in LDS:
//          S = Q K^T,  P = exp2(S*c - lse),  dP = dO V^T,  dS = P * (dP - delta)
//          dV^T += dO^T P        dK^T += Q^T dS         (P / dS feed the MFMA straight from registers)
//      With fewer than 8 KV heads the query heads of a group are split over workgroups, which write fp32 partial
//      dK / dV that a small reduce kernel sums in a fixed order (enough workgroups for all compute units).
//   3. dQ: a workgroup owns 256 queries of one head (32 per wavefront, Q and dO fragments in registers),
//      loops over 64-key tiles:  S^T = K Q^T, dP^T = V dO^T, dS^T, dQ^T += K^T dS^T.
// Tiles whose rows are needed both as row operands and transposed (Q / dO in kernel 2, K in kernel 3) are
// loaded once, global -> LDS directly, token-major, in a swizzled layout that serves plain 128-bit reads and
// LDS transpose reads without bank conflicts (LdsTile in attn_common.h); score tiles are consumed in their
// accumulator layout.
#include "attn_common.h"

#include <type_traits>

namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------------------------
// 1. delta
// ---------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(kThreads) void attn_bwd_delta_kernel(const AttnParams p) {
    constexpr int LPR = 16;  // lanes per (token, head) row, 8 elements each
    const int64_t row = ((int64_t)blockIdx.x * kThreads + threadIdx.x) / LPR;
    const int c = threadIdx.x % LPR;
    const int64_t n_rows = (int64_t)p.total_q * p.nq;
    float acc = 0.f;
    const bool ok = row < n_rows && c < D / 8;
    const int64_t t = ok ? row / p.nq : 0;
    const int h = ok ? (int)(row % p.nq) : 0;
    if (ok) {
        const uint4 a = *reinterpret_cast<const uint4*>(p.o + t * p.o_st + (int64_t)h * p.o_sh + 8 * c);
        const uint4 b = *reinterpret_cast<const uint4*>(p.d_o + t * p.o_st + (int64_t)h * p.o_sh + 8 * c);
        float fa[8], fb[8];
        Elem<elem_t>::unpack(a, fa);
        Elem<elem_t>::unpack(b, fb);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc += fa[i] * fb[i];
    }
    acc = group_sum<LPR>(acc);
    if (ok && c == 0) p.delta[(int64_t)h * p.total_q + t] = acc;
}

// ---------------------------------------------------------------------------------------------
// 2. dK / dV
// ---------------------------------------------------------------------------------------------
// 8 wavefronts, two per SIMD.  The workgroup owns 128 keys of one KV head whose K and V rows stay in
// LDS for its lifetime; wavefront w works on key group (w & 3) (32 keys) and on query sub-tile (w >> 2)
// (32 of the 64 queries staged per iteration), so the pair (w, w + 4) accumulates the same dK / dV
// rows and is summed once at the end.  The first four wavefronts stage Q, the last four dO; the staged
// tiles are double buffered (one barrier per iteration).
// __launch_bounds__(512, 2): the second argument is wavefronts per SIMD, i.e. the two that one 512-thread workgroup
// brings; the kernel takes 250 - 254 of the 256 registers each of them can have (no AGPRs, no scratch).
template <int D, bool DROP, bool SPLIT>
__global__ __launch_bounds__(512, 2) void attn_bwd_dkdv_kernel(const AttnParams p) {
    constexpr int BNK = 128;              // keys per workgroup
    constexpr int BQ = 64;                // queries per tile
    constexpr int KS = D / 16;
    constexpr int DT = D / 32;
    using Tile = LdsTile<D>;
    constexpr int RB = Tile::RB;
    constexpr int TILE = Tile::kBytes;    // one 64-token tile
    constexpr int IPW = Tile::kInstrs / 4;   // direct-load instructions per loader wavefront and 64-token tile
    constexpr int STAGE_BYTES = 4 * TILE + 4 * TILE;  // K, V (two tiles each) + Q, dO (two stages each)
    constexpr int RED_BYTES = 8 * 16 * DT * 64 * 4;   // the pair exchange: one accumulator set (dK or dV) of each of the 8 wavefronts
    constexpr int SMEM_BYTES = STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES;

    __shared__ __attribute__((aligned(1024))) char smem[SMEM_BYTES];
    __shared__ __attribute__((aligned(16))) float lse_lds[2][BQ];
    __shared__ __attribute__((aligned(16))) float delta_lds[2][BQ];
    __shared__ int range_lds[16];
    __shared__ int lpt_lds[2 * kLptMax];  // work estimates and hand-out order of the key blocks (packed documents)
    // The streamed tiles come first: with the stage index a compile-time constant (the tile loop is unrolled by two)
    // their LDS addresses are a per-lane register plus an immediate offset, which reaches 64 KB.
    char* q_t = smem;                     // [2 stages]
    char* do_t = smem + 2 * TILE;         // [2 stages]
    char* k_t = smem + 4 * TILE;          // [2 tiles of 64 keys]
    char* v_t = smem + 6 * TILE;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    const int kgp = wave & 3, sub = wave >> 2;

    const int nkb = (p.total_k + BNK - 1) / BNK;
    // (KV head, head split) groups x key-block ranks.  With a multiple of 8 groups every XCD receives whole groups
    // with all their key blocks (the same Q / dO stream through its L2, equal work per XCD); otherwise a contiguous
    // slice per XCD would give one XCD a group's heavy key blocks and another its light ones, so the items go out
    // rank-major and every XCD sees every rank.
    const int n_groups = p.nkv * p.hsplit;
    int kb_rank, group;
    if ((n_groups & 7) == 0) {
        const int work = xcd_remap(blockIdx.x, gridDim.x);
        kb_rank = work % nkb;
        group = work / nkb;
    } else {
        kb_rank = blockIdx.x / n_groups;
        group = blockIdx.x - kb_rank * n_groups;
    }
    int kb = block_for_rank(kb_rank, nkb, p.n_docs, p.across_k, false);   // key blocks with the most queries first
    if (p.lpt_k) {                        // documents of different lengths: by the work each key block really has
        lpt_order<true>(p, nkb, BNK, lpt_lds, lpt_lds + kLptMax);
        kb = lpt_lds[kLptMax + kb_rank];
    }
    const int hpw = p.n_rep / p.hsplit;   // query heads of this workgroup: hs * hpw .. + hpw of the group
    const int kvh = group / p.hsplit;
    const int hs = group - kvh * p.hsplit;
    const int key = kb * BNK + kgp * 32 + l32;

    int qlo, qhi;
    query_range(p, key, qlo, qhi);
    int wmin = qhi > qlo ? qlo : 0x7fffffff, wmax = qhi > qlo ? qhi : 0;
    wmin = group_min<64>(wmin);           // DPP lane reductions: no trips through the LDS crossbar
    wmax = group_max<64>(wmax);
    if (lane == 0) { range_lds[wave] = wmin; range_lds[8 + wave] = wmax; }

    // K / V rows of this key block: loaded once, global -> LDS directly; wavefronts 0-3 fetch K, 4-7 fetch V
    const bool q_role = wave < 4;         // later: wavefronts 0-3 stage Q, 4-7 stage dO
    const int lw = wave & 3;
    {
        DmaPlan<D, IPW> plan;
        plan.init(lw * IPW, lane, q_role ? p.k_st : p.v_st);
        const elem_t* base = q_role ? p.k + (int64_t)kvh * p.k_sh : p.v + (int64_t)kvh * p.v_sh;
        const int64_t st = q_role ? p.k_st : p.v_st;
        char* dst = q_role ? k_t : v_t;
#pragma unroll
        for (int half = 0; half < 2; ++half) plan.issue(base, st, kb * BNK + 64 * half, p.total_k - 1, dst + half * TILE);
    }
    __syncthreads();                      // publishes range_lds (the loads are waited for below)
    int bmin = 0x7fffffff, bmax = 0;
#pragma unroll
    for (int w = 0; w < 8; ++w) { bmin = min(bmin, range_lds[w]); bmax = max(bmax, range_lds[8 + w]); }
    if (bmax <= bmin) { bmin = 0; bmax = 0; }
    const int qt0 = __builtin_amdgcn_readfirstlane(bmin & ~(BQ - 1));
    const int n_tiles = __builtin_amdgcn_readfirstlane((bmax - qt0 + BQ - 1) / BQ);

    f32x16_t dk_acc[DT], dv_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk_acc[dt][r] = 0.f; dv_acc[dt][r] = 0.f; }

    // Query tiles are visited from the last one downwards, the group's query heads innermost: under a causal mask
    // every key block of a document needs the document's last queries, so the workgroups that share an XCD start on
    // the same tile and walk down in step, streaming the same Q / dO rows through that XCD's L2 once.
    const int total_iters = n_tiles * hpw;
    const int last_q = p.total_q - 1;
    const elem_t* src_base = q_role ? p.q : p.d_o;
    const int64_t src_head_stride = q_role ? p.q_sh : p.o_sh;
    const int64_t src_tok_stride = q_role ? p.q_st : p.o_st;
    char* dst_tile = q_role ? q_t : do_t;
    DmaPlan<D, IPW> plan;
    plan.init(lw * IPW, lane, src_tok_stride);
    // log-sum-exp (to the exp2 domain) and delta rows of a tile pass through one register of threads 0..127
    const float* stat_base = (tid < BQ) ? p.lse : p.delta;
    const float stat_scale = (tid < BQ) ? 1.4426950408889634f : 1.0f;
    float stat = 0.f;
    // (query head of the group, query tile) of the current and of the next iteration, stepped without divisions
    int cur_rep = 0, cur_tile = 0, nxt_rep = 0, nxt_tile = 0;
    auto issue_tile = [&](int iter) {     // Q / dO tile of iteration `iter` (= the next one) -> stage iter & 1
        const int head = kvh * p.n_rep + hs * hpw + nxt_rep;
        const int qt = qt0 + (n_tiles - 1 - nxt_tile) * BQ;
        plan.issue(src_base + (int64_t)head * src_head_stride, src_tok_stride, qt, last_q, dst_tile + (iter & 1) * TILE);
        if (tid < 2 * BQ) {
            const int tok = min(qt + (tid & (BQ - 1)), last_q);
            stat = stat_base[(int64_t)head * p.total_q + tok];
        }
    };
    auto store_stat = [&](int iter) {
        if (tid < BQ) lse_lds[iter & 1][tid] = stat * stat_scale;
        else if (tid < 2 * BQ) delta_lds[iter & 1][tid - BQ] = stat * stat_scale;
    };

    if (total_iters > 0) {
        issue_tile(0);
        store_stat(0);
    }
    wait_vmcnt<0>();
    __syncthreads();

    int tr_h0, tr_h1;
    Tile::tr_bases(lane, tr_h0, tr_h1);
    tr_h0 += 32 * sub * RB;
    tr_h1 += 32 * sub * RB;
    const int a_row = Tile::row_base(32 * sub + l32, g);                       // Q / dO rows of this wavefront's sub-tile
    const int b_row = (kgp >> 1) * TILE + Tile::row_base(32 * (kgp & 1) + l32, g);   // its K / V rows
    const float c2 = p.scale_log2;
    // dropout: hash input of this lane's key column at query pair 2 g, bit offset of its column of a 2 x 2 block
    uint32_t drop_xc = 0, drop_sel = 0;
    if constexpr (DROP) {
        drop_xc = (uint32_t)(key >> 1) * kDropC2 + (uint32_t)(2 * g) * kDropC1;
        drop_sel = 8u * (uint32_t)(key & 1);
    }

    auto tile_step = [&](auto buf_c, int iter) {
        constexpr int buf = decltype(buf_c)::value;
        const int qs = qt0 + (n_tiles - 1 - cur_tile) * BQ + 32 * sub;
        if (++nxt_rep == hpw) { nxt_rep = 0; ++nxt_tile; }
        if (iter + 1 < total_iters) issue_tile(iter + 1);

        if ((qs < wmax) && (qs + 32 > wmin)) {
            const char* qt_ = q_t + buf * TILE;
            const char* dt_ = do_t + buf * TILE;
            f32x16_t s_acc, dp_acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) { s_acc[r] = 0.f; dp_acc[r] = 0.f; }
            // 2 KS products whose operands come from LDS through rings of kDepth registers filled kDepth products ahead
            // (sched_barrier pins that order): left to the compiler, the four reads of a contraction step are issued right
            // before its two products, which then wait out the LDS latency KS times per tile (measured: 1330 -> 810 cycles
            // for this stage, -3 % on the kernel)
            {
                constexpr int kSteps = 2 * KS, kDepth = 3;
                elem8_t ra[kDepth], rb[kDepth];
                auto fetch = [&](int i, elem8_t& a, elem8_t& b) {
                    const int ks = i >> 1;
                    const int ao = a_row ^ (ks << 5), bo = b_row ^ (ks << 5);
                    a = *reinterpret_cast<const elem8_t*>(((i & 1) ? dt_ : qt_) + ao);
                    b = *reinterpret_cast<const elem8_t*>(((i & 1) ? v_t : k_t) + bo);
                };
#pragma unroll
                for (int i = 0; i < kDepth; ++i) fetch(i, ra[i], rb[i]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < kSteps; ++i) {
                    const elem8_t a = ra[i % kDepth], b = rb[i % kDepth];
                    if (i & 1) dp_acc = mfma_32x32x16(a, b, dp_acc);
                    else s_acc = mfma_32x32x16(a, b, s_acc);
                    if (i + kDepth < kSteps) fetch(i + kDepth, ra[i % kDepth], rb[i % kDepth]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // rows of the accumulators are queries qs + 8a + 4g + c, the column is this lane's key
            if (__any((qs < qlo) || (qs + 32 > qhi))) {
                int rel0 = qs + 4 * g - qlo;
                asm volatile("" : "+v"(rel0));   // opaque: keeps the compares inside this branch
                const unsigned len = (unsigned)(qhi - qlo);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const unsigned rel = (unsigned)(rel0 + 8 * (r >> 2) + (r & 3));
                    if (rel >= len) s_acc[r] = -INFINITY;
                }
            }
            elem8_t pf[2], dsf[2];
            elem8_t pl[SPLIT ? 2 : 1], dsl[SPLIT ? 2 : 1];   // accuracy mode: low-order terms of P and dS
            uint32_t drop_xb = 0;
            if constexpr (DROP) {
                const int head_i = kvh * p.n_rep + hs * hpw + cur_rep;
                drop_xb = drop_head_base(p.drop_seed, head_i) + drop_xc + (uint32_t)(qs >> 1) * kDropC1;
            }
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4_t l4 = *reinterpret_cast<const f32x4_t*>(&lse_lds[buf][32 * sub + 8 * a + 4 * g]);
                const f32x4_t d4 = *reinterpret_cast<const f32x4_t*>(&delta_lds[buf][32 * sub + 8 * a + 4 * g]);
                bool keep[4] = {true, true, true, true};
                if constexpr (DROP) {
                    // register 4 a + c holds query qs + 8 a + 4 g + c: two query pairs per a
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const uint32_t h = lowbias32(drop_xb + (uint32_t)(4 * a + j) * kDropC1);
                        keep[2 * j] = drop_byte(h, drop_sel) >= p.drop_thr;
                        keep[2 * j + 1] = drop_byte(h, drop_sel + 16) >= p.drop_thr;
                    }
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int r = 4 * a + c;
                    const float pv = fast_exp2(s_acc[r] * c2 - l4[c]);
                    const float dpv = DROP ? (keep[c] ? dp_acc[r] * p.drop_rscale : 0.f) : dp_acc[r];
                    const float ds = pv * (dpv - d4[c]);
                    const float pk = (DROP && !keep[c]) ? 0.f : pv;
                    pf[a >> 1][4 * (a & 1) + c] = (elem_t)pk;
                    dsf[a >> 1][4 * (a & 1) + c] = (elem_t)ds;
                    if constexpr (SPLIT) {
                        pl[a >> 1][4 * (a & 1) + c] = (elem_t)(pk - (float)pf[a >> 1][4 * (a & 1) + c]);
                        dsl[a >> 1][4 * (a & 1) + c] = (elem_t)(ds - (float)dsf[a >> 1][4 * (a & 1) + c]);
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < 2; ++m) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const int o0 = (tr_h0 ^ (dt << 6)) + 16 * m * RB, o1 = (tr_h1 ^ (dt << 6)) + 16 * m * RB;
                    const elem8_t adt = tr_pair(dt_ + o0, dt_ + o1);
                    const elem8_t aqt = tr_pair(qt_ + o0, qt_ + o1);
                    dv_acc[dt] = mfma_32x32x16(adt, pf[m], dv_acc[dt]);
                    dk_acc[dt] = mfma_32x32x16(aqt, dsf[m], dk_acc[dt]);
                    if constexpr (SPLIT) {
                        dv_acc[dt] = mfma_32x32x16(adt, pl[m], dv_acc[dt]);
                        dk_acc[dt] = mfma_32x32x16(aqt, dsl[m], dk_acc[dt]);
                    }
                }
            }
        }
        if (iter + 1 < total_iters) store_stat(iter + 1);
        cur_rep = nxt_rep;
        cur_tile = nxt_tile;
        wait_vmcnt<0>();                  // the next Q / dO tile has landed
        __syncthreads();
    };
    for (int iter = 0; iter < total_iters; iter += 2) {
        tile_step(std::integral_constant<int, 0>{}, iter);
        if (iter + 1 < total_iters) tile_step(std::integral_constant<int, 1>{}, iter + 1);
    }

    // ---- sum the two wavefronts of each key group (fixed order), then store -------------------------
    // One exchange: the second wavefront of a pair hands its dK to the first and receives the first's dV, so each of them
    // sums and stores one of the two tensors (half the LDS traffic and half the stores per wavefront of a one-way sum).
    constexpr int kAccFloats = 16 * DT * 64;          // one accumulator set of one wavefront
    static_assert(2 * 4 * kAccFloats * 4 <= SMEM_BYTES, "the exchange reuses the tile stages");
    float* red_k = reinterpret_cast<float*>(smem) + (size_t)kgp * kAccFloats + lane;
    float* red_v = reinterpret_cast<float*>(smem) + (size_t)(4 + kgp) * kAccFloats + lane;
    {
        const f32x16_t* mine = sub == 1 ? dk_acc : dv_acc;
        float* out = sub == 1 ? red_k : red_v;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) out[(dt * 16 + r) * 64] = mine[dt][r];
    }
    __syncthreads();
    if (sub == 0) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dk_acc[dt][r] += red_k[(dt * 16 + r) * 64];
    } else {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dv_acc[dt][r] = red_v[(dt * 16 + r) * 64] + dv_acc[dt][r];
    }
    if (key >= p.total_k) return;

    if (p.hsplit > 1) {
        const int64_t prow = (((int64_t)hs * p.total_k + key) * p.nkv + kvh) * D + 4 * g;
        const float sc = sub == 0 ? p.scale : (DROP ? p.drop_rscale : 1.0f);
        const f32x16_t* acc = sub == 0 ? dk_acc : dv_acc;
        float* part = sub == 0 ? p.dk_part : p.dv_part;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                f32x4_t x4;
#pragma unroll
                for (int c = 0; c < 4; ++c) x4[c] = acc[dt][4 * a + c] * sc;
                *reinterpret_cast<f32x4_t*>(part + prow + 32 * dt + 8 * a) = x4;
            }
    } else if (sub == 0) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dk_acc[dt][r] *= p.scale;
        if constexpr (D == 64 || D == 128) {
            if (p.unrotate != 0) unrotate_acc<D>(dk_acc, p, p.pos_k[key], g);   // k was the rotated tensor
        }
        elem_t* dkr = p.dk + (int64_t)key * p.dk_st + (int64_t)kvh * p.dk_sh + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const uint32_t k0 = pack_elem2(dk_acc[dt][4 * a], dk_acc[dt][4 * a + 1]);
                const uint32_t k1 = pack_elem2(dk_acc[dt][4 * a + 2], dk_acc[dt][4 * a + 3]);
                *reinterpret_cast<uint2*>(dkr + 32 * dt + 8 * a) = make_uint2(k0, k1);
            }
    } else {
        const float vs = DROP ? p.drop_rscale : 1.0f;   // dV = (P * mask / (1 - p))^T dO
        elem_t* dvr = p.dv + (int64_t)key * p.dv_st + (int64_t)kvh * p.dv_sh + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const uint32_t v0 = pack_elem2(dv_acc[dt][4 * a] * vs, dv_acc[dt][4 * a + 1] * vs);
                const uint32_t v1 = pack_elem2(dv_acc[dt][4 * a + 2] * vs, dv_acc[dt][4 * a + 3] * vs);
                *reinterpret_cast<uint2*>(dvr + 32 * dt + 8 * a) = make_uint2(v0, v1);
            }
    }
}

// Sum of the hsplit partial dK / dV of a split launch, in a fixed order; one thread per (key, KV head) and two groups
// of 4 features, D / 2 apart (the two halves of rotate-half pairs), so that the summed dK can be rotated back in place.
template <int D>
__global__ __launch_bounds__(kThreads) void attn_bwd_dkdv_reduce_kernel(const AttnParams p) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const int64_t n = (int64_t)p.total_k * p.nkv * (D / 8);
    if (idx >= n) return;
    const int c = (int)(idx % (D / 8));
    const int kvh = (int)((idx / (D / 8)) % p.nkv);
    const int64_t key = idx / ((int64_t)(D / 8) * p.nkv);
    const int64_t stride = (int64_t)p.total_k * p.nkv * D;
    const int64_t off = (key * p.nkv + kvh) * D + 4 * c;
    f32x4_t k4[2], v4[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        k4[h] = *reinterpret_cast<const f32x4_t*>(p.dk_part + off + h * (D / 2));
        v4[h] = *reinterpret_cast<const f32x4_t*>(p.dv_part + off + h * (D / 2));
    }
    for (int s = 1; s < p.hsplit; ++s)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            k4[h] += *reinterpret_cast<const f32x4_t*>(p.dk_part + s * stride + off + h * (D / 2));
            v4[h] += *reinterpret_cast<const f32x4_t*>(p.dv_part + s * stride + off + h * (D / 2));
        }
    if (p.unrotate != 0) {
        int64_t pos = p.pos_k[key];
        pos = pos < 0 ? 0 : (pos >= p.table_rows ? p.table_rows - 1 : pos);
        if (p.unrotate == 1) {               // features 4 c + i pair with 4 c + i + D / 2
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float cs = (float)p.cos[pos * D + 4 * c + i], sn = (float)p.sin[pos * D + 4 * c + i];
                const float x0 = k4[0][i], x1 = k4[1][i];
                k4[0][i] = x0 * cs + x1 * sn;
                k4[1][i] = x1 * cs - x0 * sn;
            }
        } else {                             // pairs (4 c, 4 c + 1), (4 c + 2, 4 c + 3) of either half
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int pair = (4 * c + h * (D / 2)) / 2 + i;
                    float x0 = k4[h][2 * i], x1 = k4[h][2 * i + 1];
                    rotate_complex_pair(x0, x1, p.cos32[pos * (D / 2) + pair], -p.sin32[pos * (D / 2) + pair]);
                    k4[h][2 * i] = x0;
                    k4[h][2 * i + 1] = x1;
                }
        }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        *reinterpret_cast<uint2*>(p.dk + key * p.dk_st + (int64_t)kvh * p.dk_sh + 4 * c + h * (D / 2)) =
            make_uint2(pack_elem2(k4[h][0], k4[h][1]), pack_elem2(k4[h][2], k4[h][3]));
        *reinterpret_cast<uint2*>(p.dv + key * p.dv_st + (int64_t)kvh * p.dv_sh + 4 * c + h * (D / 2)) =
            make_uint2(pack_elem2(v4[h][0], v4[h][1]), pack_elem2(v4[h][2], v4[h][3]));
    }
}

// ---------------------------------------------------------------------------------------------
// 3. dQ
// ---------------------------------------------------------------------------------------------
// 8 wavefronts, two per SIMD, 32 queries each (256 per workgroup); the first four stage K (one
// token-major tile read both as row operand and transposed), the last four stage V.  Double-buffered
// LDS, one barrier per 64-key tile.
template <int D, bool DROP, bool SPLIT>
__global__ __launch_bounds__(512, 2) void attn_bwd_dq_kernel(const AttnParams p) {
    constexpr int BM = 256;
    constexpr int BN = 64;
    constexpr int KS = D / 16;
    constexpr int DT = D / 32;
    constexpr int NS = 4;                 // LDS stages per operand
    using Tile = LdsTile<D>;
    constexpr int RB = Tile::RB;
    constexpr int TILE = Tile::kBytes;
    constexpr int IPW = Tile::kInstrs / 4;   // direct-load instructions per loader wavefront and tile

    __shared__ __attribute__((aligned(1024))) char k_t[NS * TILE];   // row operand and transposed operand
    __shared__ __attribute__((aligned(1024))) char v_t[NS * TILE];   // row operand
    __shared__ int range_lds[16];
    __shared__ int lpt_lds[2 * kLptMax];  // work estimates and hand-out order of the query blocks (packed documents)

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, l32 = lane & 31, g = lane >> 5;

    const int nqb = (p.total_q + BM - 1) / BM;
    int head, q_rank;
    head_and_rank(blockIdx.x, p.nq, head, q_rank);
    const int kvh = head / p.n_rep;
    int qb = block_for_rank(q_rank, nqb, p.n_docs, p.across_q, true);
    if (p.lpt_q) {                        // documents of different lengths: by the work each query block really has
        lpt_order<false>(p, nqb, BM, lpt_lds, lpt_lds + kLptMax);
        qb = lpt_lds[kLptMax + q_rank];
    }
    const int tq = qb * BM + wave * 32 + l32;

    int klo, khi;
    key_range(p, tq, klo, khi);
    int wmin = khi > klo ? klo : 0x7fffffff, wmax = khi > klo ? khi : 0;
    wmin = group_min<64>(wmin);           // DPP lane reductions: no trips through the LDS crossbar
    wmax = group_max<64>(wmax);
    if (lane == 0) { range_lds[wave] = wmin; range_lds[8 + wave] = wmax; }

    const int tl = tq < p.total_q ? tq : p.total_q - 1;
    elem8_t qf[KS], dof[KS];
    {
        const elem_t* qr = p.q + (int64_t)tl * p.q_st + (int64_t)head * p.q_sh + 8 * g;
        const elem_t* dr = p.d_o + (int64_t)tl * p.o_st + (int64_t)head * p.o_sh + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qf[ks] = *reinterpret_cast<const elem8_t*>(qr + 16 * ks);
            dof[ks] = *reinterpret_cast<const elem8_t*>(dr + 16 * ks);
        }
    }
    const float lse_nat = p.lse[(int64_t)head * p.total_q + tl];
    float delta = p.delta[(int64_t)head * p.total_q + tl];
    float lse2 = lse_nat * 1.4426950408889634f;
    // Consume the loaded registers here: otherwise their loads count as possibly outstanding at the
    // loop entry and their uses inside the loop wait for them again.
    asm volatile("" : "+v"(lse2), "+v"(delta));
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]), "+v"(dof[ks]));

    __syncthreads();
    int bmin = 0x7fffffff, bmax = 0;
#pragma unroll
    for (int w = 0; w < 8; ++w) { bmin = min(bmin, range_lds[w]); bmax = max(bmax, range_lds[8 + w]); }
    if (bmax <= bmin) { bmin = 0; bmax = 0; }
    const int kt0 = __builtin_amdgcn_readfirstlane(bmin & ~(BN - 1));
    const int n_tiles = __builtin_amdgcn_readfirstlane((bmax - kt0 + BN - 1) / BN);

    f32x16_t dq_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq_acc[dt][r] = 0.f;

    // wavefronts 0-3 fetch K tiles, 4-7 fetch V tiles: global -> LDS directly, two tiles ahead, into the
    // stage whose readers passed the previous barrier
    const bool k_role = wave < 4;
    const int lw = wave & 3;
    const elem_t* src_base = k_role ? p.k + (int64_t)kvh * p.k_sh : p.v + (int64_t)kvh * p.v_sh;
    const int64_t src_tok_stride = k_role ? p.k_st : p.v_st;
    char* dst_ring = k_role ? k_t : v_t;
    const int last_k = p.total_k - 1;
    DmaPlan<D, IPW> plan;
    plan.init(lw * IPW, lane, src_tok_stride);
    auto issue_tile = [&](int t) {
        if (t < n_tiles) plan.issue(src_base, src_tok_stride, kt0 + t * BN, last_k, dst_ring + (t % NS) * TILE);
    };
    issue_tile(0);
    issue_tile(1);
    issue_tile(2);
    if (n_tiles > 2) wait_vmcnt<2 * IPW>(); else if (n_tiles > 1) wait_vmcnt<IPW>(); else wait_vmcnt<0>();
    __syncthreads();

    const float c2 = p.scale_log2;
    int tr_h0, tr_h1;
    Tile::tr_bases(lane, tr_h0, tr_h1);
    const int a_row = Tile::row_base(l32, g);
    // dropout: hash input of this lane's query row at key pair 2 g, bit offset of its row of a 2 x 2 block
    uint32_t drop_xr = 0, drop_sel = 0;
    if constexpr (DROP) {
        drop_xr = drop_head_base(p.drop_seed, head) + (uint32_t)(tq >> 1) * kDropC1 + (uint32_t)(2 * g) * kDropC2;
        drop_sel = 16u * (uint32_t)(tq & 1);
    }
    for (int it = 0; it < n_tiles; ++it) {
        const int kt = kt0 + it * BN;
        issue_tile(it + 3);

        if ((kt < wmax) && (kt + BN > wmin)) {
            const char* kt_ = k_t + (it % NS) * TILE;
            const char* vt_ = v_t + (it % NS) * TILE;
            f32x16_t s_acc[2], dp_acc[2];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) { s_acc[t][r] = 0.f; dp_acc[t][r] = 0.f; }
            // 4 KS products whose A operands come from LDS through a ring of kDepth registers filled kDepth products ahead
            {
                constexpr int kSteps = 4 * KS, kDepth = 3;
                elem8_t ring[kDepth];
                auto fetch = [&](int i) -> elem8_t {
                    const int ks = i >> 2, t = (i >> 1) & 1;
                    return *reinterpret_cast<const elem8_t*>(((i & 1) ? vt_ : kt_) + (a_row ^ (ks << 5)) + 32 * t * RB);
                };
#pragma unroll
                for (int i = 0; i < kDepth; ++i) ring[i] = fetch(i);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < kSteps; ++i) {
                    const int ks = i >> 2, t = (i >> 1) & 1;
                    const elem8_t a = ring[i % kDepth];
                    if (i & 1) dp_acc[t] = mfma_32x32x16(a, dof[ks], dp_acc[t]);
                    else s_acc[t] = mfma_32x32x16(a, qf[ks], s_acc[t]);
                    if (i + kDepth < kSteps) ring[i % kDepth] = fetch(i + kDepth);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (__any((kt < klo) || (kt + BN > khi))) {
                int rel0 = kt + 4 * g - klo;
                asm volatile("" : "+v"(rel0));   // opaque: keeps the compares inside this branch
                const unsigned len = (unsigned)(khi - klo);
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const unsigned rel = (unsigned)(rel0 + 32 * t + 8 * (r >> 2) + (r & 3));
                        if (rel >= len) s_acc[t][r] = -INFINITY;
                    }
            }
            // dS of accumulator register 8 (m & 1) + e of key sub-tile m >> 1 (m = 16-key chunk, e = 0..7), compile-time indices
            const uint32_t drop_xt = DROP ? drop_xr + (uint32_t)(kt >> 1) * kDropC2 : 0u;
            auto ds_element = [&](auto m_c, auto e_c, elem8_t& dsf, elem8_t& dsl) {
                constexpr int m = decltype(m_c)::value, e = decltype(e_c)::value, t = m >> 1, r = 8 * (m & 1) + e;
                float dpv = dp_acc[t][r];
                if constexpr (DROP) {
                    // dP of a dropped probability is zero, that of a kept one carries the 1 / (1 - p) scale
                    constexpr int pi = e >> 1, a = 2 * (m & 1) + (pi >> 1), j = pi & 1;
                    const uint32_t h = lowbias32(drop_xt + (uint32_t)(16 * t + 4 * a + j) * kDropC2);
                    dpv = drop_byte(h, drop_sel + 8 * (e & 1)) >= p.drop_thr ? dpv * p.drop_rscale : 0.f;
                }
                const float pv = fast_exp2(s_acc[t][r] * c2 - lse2);
                const float ds = pv * (dpv - delta);
                dsf[e] = (elem_t)ds;
                if constexpr (SPLIT) dsl[e] = (elem_t)(ds - (float)dsf[e]);
            };
            // dQ^T += K^T dS^T: 4 DT products, chunk by chunk of 16 keys; the transposed K operands come through a ring filled
            // kDepth products ahead and the dS of chunk m + 1 are computed between the products of chunk m, so neither the LDS
            // latency nor the softmax arithmetic sits between two products (sched_barrier pins the order)
            {
                constexpr int kSteps = 4 * DT, kDepth = 3;
                elem8_t ring[kDepth];
                elem8_t d[2], dl[2];
                auto fetch = [&](int i) -> elem8_t {
                    const int m = i / DT, dt = i % DT;
                    const int o0 = (tr_h0 ^ (dt << 6)) + 16 * m * RB, o1 = (tr_h1 ^ (dt << 6)) + 16 * m * RB;
                    return tr_pair(kt_ + o0, kt_ + o1);
                };
#pragma unroll
                for (int i = 0; i < kDepth; ++i) ring[i] = fetch(i);
                __builtin_amdgcn_sched_barrier(0);
                static_for<8>([&](auto e_c) { ds_element(std::integral_constant<int, 0>{}, e_c, d[0], dl[0]); });
                __builtin_amdgcn_sched_barrier(0);
                static_for<kSteps>([&](auto i_c) {
                    constexpr int i = decltype(i_c)::value, m = i / DT, dt = i % DT;
                    const elem8_t a = ring[i % kDepth];
                    dq_acc[dt] = mfma_32x32x16(a, d[m & 1], dq_acc[dt]);
                    if constexpr (SPLIT) dq_acc[dt] = mfma_32x32x16(a, dl[m & 1], dq_acc[dt]);
                    if constexpr (i + kDepth < kSteps) ring[i % kDepth] = fetch(i + kDepth);
                    if constexpr (m < 3) {
                        static_for<8>([&](auto e_c) {
                            constexpr int e = decltype(e_c)::value;
                            if constexpr ((e * DT) / 8 == dt) ds_element(std::integral_constant<int, m + 1>{}, e_c, d[(m + 1) & 1], dl[(m + 1) & 1]);
                        });
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            }
        }
        // tile it+1 must have landed; tiles it+2 and it+3 (just issued) may still be in flight
        if (it + 3 < n_tiles) wait_vmcnt<2 * IPW>(); else if (it + 2 < n_tiles) wait_vmcnt<IPW>(); else wait_vmcnt<0>();
        __syncthreads();
    }

    if (tq < p.total_q) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dq_acc[dt][r] *= p.scale;
        if constexpr (D == 64 || D == 128) {
            // q was the rotated tensor: the gradient of the unrotated one is the row rotated back (rotary.py:117-139)
            if (p.unrotate != 0) unrotate_acc<D>(dq_acc, p, p.pos_q[tq], g);
        }
        elem_t* dqr = p.dq + (int64_t)tq * p.q_st + (int64_t)head * p.q_sh + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const uint32_t w0 = pack_elem2(dq_acc[dt][4 * a], dq_acc[dt][4 * a + 1]);
                const uint32_t w1 = pack_elem2(dq_acc[dt][4 * a + 2], dq_acc[dt][4 * a + 3]);
                *reinterpret_cast<uint2*>(dqr + 32 * dt + 8 * a) = make_uint2(w0, w1);
            }
    }
}

template <int D> int launch_bwd(const AttnParams& p, int flags, hipStream_t st) {
    const int stages = flags & (MI_ATTN_BWD_DELTA | MI_ATTN_BWD_DKDV | MI_ATTN_BWD_DQ);
    const bool split = (flags & MI_ATTN_SPLIT_P) != 0;     // accuracy mode (no dropout: checked by the entry point)
    const bool all = stages == 0;
    if (all || (stages & MI_ATTN_BWD_DELTA)) {
        const int64_t rows = (int64_t)p.total_q * p.nq;
        const int64_t blocks = (rows * 16 + kThreads - 1) / kThreads;
        if (blocks > 0x7fffffffLL) return mi_fail(MI_E_SHAPE, "attn_bwd: grid too large");
        attn_bwd_delta_kernel<D><<<dim3((unsigned)blocks), dim3(kThreads), 0, st>>>(p);
        int rc = mi_check_launch("attn_bwd_delta");
        if (rc != MI_OK) return rc;
    }
    if (all || (stages & MI_ATTN_BWD_DKDV)) {
        const int64_t grid = (((int64_t)p.total_k + 127) / 128) * p.nkv * p.hsplit;
        if (split) attn_bwd_dkdv_kernel<D, false, true><<<dim3((unsigned)grid), dim3(512), 0, st>>>(p);
        else if (p.drop_thr != 0) attn_bwd_dkdv_kernel<D, true, false><<<dim3((unsigned)grid), dim3(512), 0, st>>>(p);
        else attn_bwd_dkdv_kernel<D, false, false><<<dim3((unsigned)grid), dim3(512), 0, st>>>(p);
        int rc = mi_check_launch("attn_bwd_dkdv");
        if (rc != MI_OK) return rc;
        if (p.hsplit > 1) {
            const int64_t n = (int64_t)p.total_k * p.nkv * (D / 8);
            attn_bwd_dkdv_reduce_kernel<D><<<dim3((unsigned)((n + kThreads - 1) / kThreads)), dim3(kThreads), 0, st>>>(p);
            rc = mi_check_launch("attn_bwd_dkdv_reduce");
            if (rc != MI_OK) return rc;
        }
    }
    if (all || (stages & MI_ATTN_BWD_DQ)) {
        const int64_t grid = (((int64_t)p.total_q + 255) / 256) * p.nq;
        if (split) attn_bwd_dq_kernel<D, false, true><<<dim3((unsigned)grid), dim3(512), 0, st>>>(p);
        else if (p.drop_thr != 0) attn_bwd_dq_kernel<D, true, false><<<dim3((unsigned)grid), dim3(512), 0, st>>>(p);
        else attn_bwd_dq_kernel<D, false, false><<<dim3((unsigned)grid), dim3(512), 0, st>>>(p);
        return mi_check_launch("attn_bwd_dq");
    }
    return MI_OK;
}

}  // namespace

#ifndef MI_ELEM_F16
extern "C" size_t mi_attn_bwd_workspace_bytes(int64_t total_q, int32_t n_q_heads, int32_t head_dim) {
    (void)head_dim;
    if (total_q <= 0 || n_q_heads <= 0) return 0;
    return (size_t)total_q * (size_t)n_q_heads * sizeof(float);
}
#else
extern "C" size_t mi_attn_bwd_workspace_bytes(int64_t total_q, int32_t n_q_heads, int32_t head_dim);
#endif

namespace {
// query-head split of the dK/dV launch: enough workgroup groups for the 8 XCDs when there are fewer than 8 KV heads
int dkdv_head_split(int nq, int nkv) {
    const int n_rep = nq / nkv;
    int h = 1;
    while (nkv * h < 8 && n_rep % (2 * h) == 0) h *= 2;
    return h;
}
size_t delta_bytes_aligned(int64_t total_q, int nq) { return ((size_t)total_q * (size_t)nq * sizeof(float) + 255) & ~(size_t)255; }
}  // namespace

#ifndef MI_ELEM_F16
extern "C" size_t mi_attn_bwd_workspace_bytes_kv(int64_t total_q, int64_t total_k, int32_t n_q_heads, int32_t n_kv_heads,
                                                 int32_t head_dim) {
    if (total_q <= 0 || total_k <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || n_q_heads % n_kv_heads != 0 || head_dim <= 0)
        return mi_attn_bwd_workspace_bytes(total_q, n_q_heads, head_dim);
    const int h = dkdv_head_split(n_q_heads, n_kv_heads);
    if (h == 1) return mi_attn_bwd_workspace_bytes(total_q, n_q_heads, head_dim);
    return delta_bytes_aligned(total_q, n_q_heads) + (size_t)2 * h * (size_t)total_k * n_kv_heads * head_dim * sizeof(float);
}
#endif

int MI_ENTRY(mi_attn_bwd_impl)(const mi_attn_bwd_args* b) {
    if (!b) return mi_fail(MI_E_NULL, "attn_bwd: args is null");
    const mi_attn_args* a = &b->fwd;
    int rc = mi_attn_validate(a, "attn_bwd");
    if (rc != MI_OK) return rc;
    if (a->rotary_cos && !a->position_ids_k) return mi_fail(MI_E_NULL, "attn_bwd: rotary needs the position ids of q and k");
    if (!a->o || !a->lse || !b->d_o || !b->dq || !b->dk || !b->dv)
        return mi_fail(MI_E_NULL, "attn_bwd: o, lse, d_o, dq, dk, dv are required");
    if (!mi_aligned16(a->o) || !mi_aligned16(b->d_o) || !mi_aligned16(b->dq) || !mi_aligned16(b->dk) || !mi_aligned16(b->dv))
        return mi_fail(MI_E_ALIGN, "attn_bwd: tensors must be 16-byte aligned");
    if (a->o_stride_token % 8 || a->o_stride_head % 8 || b->dk_stride_token % 8 || b->dk_stride_head % 8 ||
        b->dv_stride_token % 8 || b->dv_stride_head % 8)
        return mi_fail(MI_E_ALIGN, "attn_bwd: strides must be multiples of 8 elements");
    if ((a->flags & MI_ATTN_SPLIT_P) && a->dropout_p > 0.f) return mi_fail(MI_E_SHAPE, "attn_bwd: MI_ATTN_SPLIT_P takes no dropout");
    if (a->total_q == 0) return MI_OK;
    const size_t need = mi_attn_bwd_workspace_bytes(a->total_q, a->n_q_heads, a->head_dim);
    if (!b->workspace || b->workspace_bytes < need || !mi_aligned16(b->workspace))
        return mi_fail(MI_E_WORKSPACE, "attn_bwd: workspace needs %zu bytes (16-byte aligned), got %zu", need, b->workspace_bytes);
    AttnParams p;
    mi_attn_fill_params(a, &p);
    p.d_o = (const elem_t*)b->d_o; p.dq = (elem_t*)b->dq; p.dk = (elem_t*)b->dk; p.dv = (elem_t*)b->dv;
    p.dk_st = b->dk_stride_token; p.dk_sh = b->dk_stride_head;
    p.dv_st = b->dv_stride_token; p.dv_sh = b->dv_stride_head;
    p.delta = (float*)b->workspace;
    p.unrotate = a->rotary_cos == nullptr ? 0 : (a->rotary_interleaved ? 2 : 1);
    p.hsplit = 1;
    {   // fewer than 8 KV heads: split the query heads of a group over workgroups if the workspace has room for the partials
        const int h = dkdv_head_split(a->n_q_heads, a->n_kv_heads);
        const size_t part = (size_t)h * (size_t)a->total_k * a->n_kv_heads * a->head_dim * sizeof(float);
        const size_t base = delta_bytes_aligned(a->total_q, a->n_q_heads);
        if (h > 1 && b->workspace_bytes >= base + 2 * part) {
            p.hsplit = h;
            p.dk_part = (float*)((char*)b->workspace + base);
            p.dv_part = (float*)((char*)b->workspace + base + part);
        }
    }
    {                                                                                               // dQ: 256-query blocks
        const int per_doc = mi_blocks_per_doc(a->total_q, a->n_docs, 256);
        if (p.n_rep == 1) p.across_q = per_doc;
        p.lpt_q = mi_use_lpt(a->total_q, a->n_docs, 256, per_doc);      // documents of different lengths, any head grouping
    }
    if (((a->total_k + 127) / 128) * p.nkv * p.hsplit <= 1024) {                                    // dK/dV: 128-key blocks
        p.across_k = mi_blocks_per_doc(a->total_k, a->n_docs, 128);
        p.lpt_k = mi_use_lpt(a->total_k, a->n_docs, 128, p.across_k);
    }
    hipStream_t st = (hipStream_t)a->stream;
    switch (a->head_dim) {
        case 32: return launch_bwd<32>(p, a->flags, st);
        case 64: return launch_bwd<64>(p, a->flags, st);
        case 96: return launch_bwd<96>(p, a->flags, st);
        case 128: return launch_bwd<128>(p, a->flags, st);
        default: return mi_fail(MI_E_SHAPE, "attn_bwd: head_dim %d unsupported", a->head_dim);
    }
}
