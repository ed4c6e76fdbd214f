// Block-sparse prefill attention for gfx950, 16-bit inputs: the narrow-wave instance of the streaming kernel.
//
// Same computation, same request plan, same work items, same K/V staging and the same partials layout as the kernel
// of br_prefill_mfma_impl.h (reference: sdpa_blockrank_attention_forward, blockrank_std_attention.py:503-650); what
// differs is how a query tile's 128 rows are cut into waves.  There a wave owns 32 rows of one head and needs the
// whole register file of its SIMD lane pair (two waves per SIMD); a BlockRank document's key walk is three or four
// tiles long, so an item is mostly a chain of waits (Q rows, first tile, barrier, store drain) that two waves per
// SIMD cannot hide.  Here a wave owns 16 rows, on v_mfma_f32_16x16x32: half the accumulators, half the Q fragments,
// 128 registers, four waves per SIMD - twice as many independent instruction streams over the same chain.  The price
// is LDS operand traffic: every wave still reads the whole K and V tile, for half the rows.
//
// Workgroup: 8 waves = 4 row blocks of 32 rows (the plan's geometry) x 2 halves.  Per wave and 64-key tile:
//   S^T = K Q^T      16 MFMAs 16x16x32: A = 16 K rows x 32 dims from LDS, B = Q^T (32 dims x 16 rows) in registers;
//                    lane (lr = lane & 15, lg = lane >> 4) ends up with row lr, keys 4 lg + 0..3 of every 16-row block
//   online softmax   a query row's 64 logits sit in four lanes (lg = 0..3): row maximum with one permlane16 and one
//                    permlane32 exchange; the rescale factor is a per-lane scalar
//   O^T += V^T P^T   16 MFMAs: A = V^T (16 dims x 32 keys) by transposing LDS reads, B = P^T straight from the S^T
//                    accumulators: LDS row R of a K tile holds key (R & 32) | ((R >> 2) & 3) << 3 | ((R >> 4) & 1) << 2
//                    | (R & 3), so that the eight values a lane holds for two adjacent 16-row blocks are the eight
//                    consecutive keys 8 lg + 0..7 of the 32-key chunk, which is what the B operand wants.
// LDS layouts (rows of 2 D bytes, 16-byte pieces, D = 128):
//   K    piece c of LDS row R sits at piece c ^ (R & 15): the 16 rows one operand read touches fall into 16 bank groups
//   V    row = key; piece c of row r sits at c ^ (((r & 3) | ((r & 8) >> 1)) << 1): the eight key rows that half a
//        wave's transposing read touches (r, r+1, r+2, r+3 and the same +8) fall into eight different 32-byte groups
#pragma once
#include "br_prefill_mfma_impl.h"

namespace {

#ifdef BR_E16_IS_F16
__device__ inline f32x4 br_mma16n(e16x8 a, e16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
#else
__device__ inline f32x4 br_mma16n(e16x8 a, e16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
#endif

// Maximum over the four lanes lane, lane ^ 16, lane ^ 32, lane ^ 48: v_permlane16_swap exchanges the odd 16-lane
// rows of its first operand with the even rows of its second, v_permlane32_swap the halves.
__device__ inline float max_quad(float x) {
    const unsigned u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return max_xor32(fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1])));
}
__device__ inline float sum_quad(float x) {
    x += __shfl_xor(x, 16);
    return x + __shfl_xor(x, 32);
}

// Key held by LDS row R of a K tile (see the file comment).
__device__ inline int keyperm16(int R) { return (R & 32) | (((R >> 2) & 3) << 3) | (((R >> 4) & 1) << 2) | (R & 3); }

// SC: the instance that can leave score partials and the log-sum-exp (exact probability sums); the plain instance
// carries none of their registers, scalars or code.
template <int D, bool SC>
struct PrefillNarrow {
    static_assert(D == 128, "the narrow-wave kernel is laid out for head dim 128");
    using SM = Smem<D, false>;
    static constexpr int NW = 8;                           // waves per workgroup
    static constexpr int RW = 16;                          // query rows per wave
    static constexpr int CPR = D / 8;                      // 16-byte pieces per row
    static constexpr int NI = BR_BN * CPR / 64;            // DMA instructions per K (or V) tile
    static constexpr int JK = NI / NW;                     // per wave
    static constexpr int STEP_ROWS = NW * 64 / CPR;        // rows between consecutive pieces of a wave
    static constexpr int KA = 2, VA = 2;                   // LDS operand reads in flight ahead of their MFMAs
    static constexpr int eRow = D + 8;                     // epilogue tile: [16 rows][eRow] per wave
    static constexpr int eBytesPerWave = RW * eRow * 2;
    static_assert(NW * eBytesPerWave <= 2 * SM::stageBytes, "epilogue tiles must fit the K/V stages");

    struct Lane {
        int koff, voff;    // global byte offsets inside a tile of this lane's first DMA piece (the next is STEP_ROWS rows on)
        int krd;           // LDS byte offset of the K operand read of block 0, chunk 0; chunk c is krd ^ (c << 6)
        int vrd;           // LDS byte offset of the V^T operand read of dim block 0; block d is vrd ^ (d << 5)
    };

    static __device__ inline Lane make_lane(const BrPrefillParams& p, int wave, int lane) {
        Lane L;
        const int slot = wave * 64 + lane;
        const int prow = slot / CPR, cp = slot - prow * CPR;
        L.koff = keyperm16(prow) * (int)p.k32_t * 2 + ((cp ^ (prow & 15)) << 4);
        L.voff = prow * (int)p.v32_t * 2 + ((cp ^ (((prow & 3) | ((prow & 8) >> 1)) << 1)) << 4);
        const int lr = lane & 15, lg = lane >> 4;
        L.krd = lr * SM::rowB + ((lg ^ lr) << 4);
        // transposing read: lane lr of a 16-lane group points at key 8 lg + (lr >> 2), dims 4 (lr & 3) .. + 3
        const int f = (lr >> 2) | ((lg & 1) << 2);
        L.vrd = SM::kBytes + (8 * lg + (lr >> 2)) * SM::rowB + (f << 5) + (((lr & 3) >> 1) << 4) + (lr & 1) * 8;
        return L;
    }

    // Start the DMA of one K/V tile into a stage (kt / vt: the tile's first row, uniform).  Rows past a partial tile's
    // real keys are not fetched: the LDS rows keep older (finite) data, which the kernel masks (K) or multiplies by
    // exact zeros (V).
    static __device__ inline void issue_tile(const Lane& L, int wave, int lane_l, const char* kt, const char* vt, int sk_bytes,
                                             int sv_bytes, int nvalid, unsigned stage_lds) {
        if (nvalid == BR_BN) {
#pragma unroll
            for (int j = 0; j < JK; ++j) dma16(kt + j * STEP_ROWS * sk_bytes, L.koff, stage_lds + (wave + NW * j) * 1024);
#pragma unroll
            for (int j = 0; j < JK; ++j) dma16(vt + j * STEP_ROWS * sv_bytes, L.voff, stage_lds + SM::kBytes + (wave + NW * j) * 1024);
            return;
        }
#pragma unroll
        for (int j = 0; j < JK; ++j) {
            const int prow = ((wave + NW * j) * 64 + lane_l) / CPR;
            if (keyperm16(prow) < nvalid) dma16(kt + j * STEP_ROWS * sk_bytes, L.koff, stage_lds + (wave + NW * j) * 1024);
        }
#pragma unroll
        for (int j = 0; j < JK; ++j) {
            const int prow = ((wave + NW * j) * 64 + lane_l) / CPR;
            if (prow < nvalid) dma16(vt + j * STEP_ROWS * sv_bytes, L.voff, stage_lds + SM::kBytes + (wave + NW * j) * 1024);
        }
    }

    // K operand of 16-row block j, 32-dim chunk c
    static __device__ inline e16x8 read_k(const char* stage, const Lane& L, int j, int c) {
        return as_e16x8(ld16(stage + j * 16 * SM::rowB + (L.krd ^ (c << 6))));
    }
    // V^T operand for dims 16 db + (lane & 15), keys 32 c2 + 8 lg + 0..7: two transposing reads
    static __device__ inline e16x8 read_vt(const char* stage, const Lane& L, int db, int c2) {
        const char* vp = stage + (L.vrd ^ (db << 5)) + c2 * 32 * SM::rowB;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(__attribute__((address_space(3))) const char*)vp);
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(__attribute__((address_space(3))) const char*)(vp + 4 * SM::rowB));
        union { s16x8 s8; e16x8 b8; } a;
        a.s8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return a.b8;
    }

    // One wave, one 64-key tile already in LDS.  NKB 32-key chunks are computed (the second is skipped when no row
    // of the wave can see it); with MASK, keys >= lim (per row: the tile's real keys and the diagonal) are excluded.
    template <int NKB, bool MASK, bool EXACT>
    static __device__ inline void compute_tile(const char* stage, const Lane& L, const e16x8 (&qf)[D / 32], f32x4 (&o)[D / 16],
                                               float& m_run, float& l_run, float& lt_run, float scale_log2, int lim, int lg, float& psum_out) {
        constexpr int NC = D / 32, ND = D / 16, NJ = 2 * NKB, NR = NJ * NC, NP = NKB * ND;
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        f32x4 s[NJ];
        {
            // read i: block i % NJ, chunk i / NJ - the blocks alternate so that consecutive MFMAs are independent;
            // reads run KA ahead (with four waves per SIMD the other waves cover the rest of the LDS latency)
            e16x8 ka[KA];
#pragma unroll
            for (int i = 0; i < KA; ++i) ka[i] = read_k(stage, L, i % NJ, i / NJ);
#pragma unroll
            for (int j = 0; j < NJ; ++j) s[j] = zero;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const e16x8 a = ka[i % KA];
                if (i + KA < NR) ka[i % KA] = read_k(stage, L, (i + KA) % NJ, (i + KA) / NJ);
                s[i % NJ] = br_mma16n(a, qf[i / NJ], s[i % NJ]);
            }
            BR_SCHED_DSREAD(KA);
#pragma unroll
            for (int i = 0; i + KA < NR; ++i) {
                BR_SCHED_MFMA(1);
                BR_SCHED_DSREAD(1);
            }
            BR_SCHED_MFMA(KA);
            BR_SCHED_FENCE();
        }
        if (MASK) {
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int key = 32 * (j >> 1) + 8 * lg + 4 * (j & 1) + v;
                    if (key >= lim) s[j][v] = -INFINITY;
                }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) mx = fmaxf(mx, s[j][v]);
        mx = max_quad(mx);
        // Lazy rescale: the running max is only raised (and O, l rescaled) when some row's max grew by more than 2^8
        const float m_new = fmaxf(m_run, mx * scale_log2);
        if (__builtin_amdgcn_ballot_w64(m_new - m_run > 8.f) != 0) {
            const float m_sub = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_sub);
            m_run = m_new;
            l_run *= alpha;
            lt_run *= alpha;
#pragma unroll
            for (int d = 0; d < ND; ++d)
#pragma unroll
                for (int v = 0; v < 4; ++v) o[d][v] *= alpha;
        }
        const float m_sub = m_run == -INFINITY ? 0.f : m_run;
        // Two sums of the probabilities (both over this lane's keys only; the four lanes of a row are added up at the
        // end of the item): the exact one (log-sum-exp, score partials) and the sum of the values as rounded for the
        // P V product, which normalises the output.
        float psum = 0.f, psum_t = 0.f;
        const e16x2 ones2 = {(BR_E16)1.0f, (BR_E16)1.0f};
        e16x8 pf[NKB];
#pragma unroll
        for (int c2 = 0; c2 < NKB; ++c2) {
            f32x8 t;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                t[e] = __builtin_amdgcn_exp2f(s[2 * c2 + (e >> 2)][e & 3] * scale_log2 - m_sub);
                if (EXACT) psum += t[e];
            }
            pf[c2] = __builtin_convertvector(t, e16x8);
            psum_t = br_dot2(__builtin_shufflevector(pf[c2], pf[c2], 0, 1), ones2, psum_t);
            psum_t = br_dot2(__builtin_shufflevector(pf[c2], pf[c2], 2, 3), ones2, psum_t);
            psum_t = br_dot2(__builtin_shufflevector(pf[c2], pf[c2], 4, 5), ones2, psum_t);
            psum_t = br_dot2(__builtin_shufflevector(pf[c2], pf[c2], 6, 7), ones2, psum_t);
        }
        l_run += psum;
        lt_run += psum_t;
        psum_out = psum;
        e16x8 va[VA];
#pragma unroll
        for (int i = 0; i < VA; ++i) va[i] = read_vt(stage, L, i % ND, i / ND);
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const e16x8 a = va[i % VA];
            if (i + VA < NP) va[i % VA] = read_vt(stage, L, (i + VA) % ND, (i + VA) / ND);
            o[i % ND] = br_mma16n(a, pf[i / ND], o[i % ND]);
        }
    }

    static __device__ void run_item(const BrPrefillParams& p, const BrPlanView& pv, const BrItem& it, int hg, char* smem,
                                    const Lane& L, BrPrefetch& pf, bool padded_layout) {
        const int tid = threadIdx.x;
        const int wave = uni(tid >> 6), lane = tid & 63, lr = lane & 15, lg = lane >> 4;
        const BrGeom& ge = p.geom;
        const int T = ge.tpb * BR_RB;
        const int b = it.b, m = it.m;
        const int kvh = ge.HGS == 1 ? hg : hg / ge.HGS, hsub = hg - kvh * ge.HGS;
        const int tsh = ge.tpb == 1 ? 0 : (ge.tpb == 2 ? 1 : 2);
        const int ww = wave >> 1, half = wave & 1;         // the 32-row block of the plan's geometry, and which half of it
        const int g = ww >> tsh, sub = ww & (ge.tpb - 1);
        const int hpos = hsub * ge.Gw + g;
        const bool head_ok = hpos < ge.G;
        const int head = kvh * ge.G + (head_ok ? hpos : ge.G - 1);
        const int len_m = it.len_m;
        const int len_w = head_ok ? len_m : 0;
        const int row0 = it.t0 + sub * BR_RB + half * RW;  // first query row of this wave, valid-relative
        const bool rb_active = row0 < len_w;
        const int self_end = it.t0 + T < len_m ? it.t0 + T : len_m;
        const int qtok0 = it.tok_m;
        const unsigned smem_lds = lds_addr_of(smem);
        const int sk_bytes = (int)p.k32_t * 2, sv_bytes = (int)p.v32_t * 2;
        const char* kbase = reinterpret_cast<const char*>(p.k) + ((unsigned long long)p.k32_b * (unsigned)b + (unsigned long long)p.k32_h * (unsigned)kvh) * 2;
        const char* vbase = reinterpret_cast<const char*>(p.v) + ((unsigned long long)p.v32_b * (unsigned)b + (unsigned long long)p.v32_h * (unsigned)kvh) * 2;
        const float sc2 = p.scale_log2;

        // The walk over the item's key tiles (see the wide kernel: a document's only earlier block is the prefix,
        // described by the item; a query-block item keeps its earlier-block tile descriptors in lane registers).
        const int2* tiles_b = pv.tiles + (size_t)b * pv.tps;
        const bool table = it.pe > 1;
        bool emit_scores = false, lse_out = false;
        if constexpr (SC) {
            emit_scores = p.score_part != nullptr && table && m == p.M - 1;
            lse_out = p.lse != nullptr;
        }
        const int first_doc_tile = (it.len0 + BR_BN - 1) / BR_BN;
        const int nprev = it.nprev;
        const int f_end = it.ntiles > 0x3fffffff ? 0x7fffffff : it.f_lo + it.ntiles;
        const int own_tok0 = it.tok_m;
        int wf = it.f_lo;
        int dbase = it.f_lo;
        int2 dreg = make_int2(0, 0);
        if (table) {
            if (dbase + lane < nprev) dreg = tiles_b[dbase + lane];
            asm volatile("" : "+v"(dreg.x), "+v"(dreg.y));     // wait for the table here, before the Q loads are issued
        }
        // Q^T fragments: lane (lr, lg) holds row row0 + lr, dims 32 c + 8 lg .. + 7 for every chunk c
        e16x8 qf[D / 32];
        {
            const char* qrow = reinterpret_cast<const char*>(p.q) +
                               ((unsigned long long)p.q32_b * (unsigned)b + (unsigned long long)p.q32_h * (unsigned)head +
                                (unsigned long long)p.q32_t * (unsigned)(qtok0 + row0)) * 2;
            // rows past the block's end load its last row instead: what such rows compute is never stored
            const int last = len_m - 1 - row0;
            const int qoff = ((lr < last ? lr : last) * (int)p.q32_t + lg * 8) * 2;
            if (rb_active) {
#pragma unroll
                for (int c = 0; c < D / 32; ++c) qf[c] = as_e16x8(ld16(qrow + qoff + c * 64));
            } else {
#pragma unroll
                for (int c = 0; c < D / 32; ++c) qf[c] = as_e16x8(uint4{0u, 0u, 0u, 0u});
            }
        }
        int c_f = 0, c_tok0 = 0, c_nvalid = 0;
        int n_f = 0, n_tok0 = 0, n_nvalid = 0;
        auto fetch = [&]() -> bool {
            const int f = wf;
            const bool prev = f < nprev;
            const int k0 = (f - nprev) * BR_BN;
            if (f >= f_end || (!prev && k0 >= self_end)) return false;
            if (prev && table && f - dbase >= 64) {
                dbase = f;
                dreg = dbase + lane < nprev ? tiles_b[dbase + lane] : make_int2(0, 0);
                asm volatile("" : "+v"(dreg.x), "+v"(dreg.y));
            }
            const int li = (prev && table) ? f - dbase : 0;
            const int t_tok0 = __builtin_amdgcn_readlane(dreg.x, li), t_nv = __builtin_amdgcn_readlane(dreg.y, li);
            const int p_nv = it.len0 - f * BR_BN < BR_BN ? it.len0 - f * BR_BN : BR_BN;
            const int o_nv = self_end - k0 < BR_BN ? self_end - k0 : BR_BN;
            n_f = f;
            n_tok0 = prev ? (table ? t_tok0 : it.tok0 + f * BR_BN) : own_tok0 + k0;
            n_nvalid = prev ? (table ? t_nv : p_nv) : o_nv;
            wf = f + 1;
            return true;
        };
        bool have = fetch();
        c_f = n_f; c_tok0 = n_tok0; c_nvalid = n_nvalid;
        if (have) {
            int lane_l = lane;
            asm volatile("" : "+v"(lane_l));
            issue_tile(L, wave, lane_l, kbase + (long long)c_tok0 * sk_bytes, vbase + (long long)c_tok0 * sv_bytes, sk_bytes, sv_bytes, c_nvalid,
                       smem_lds);
        }

        f32x4 o[D / 16];
#pragma unroll
        for (int d = 0; d < D / 16; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};
        float m_run = -INFINITY, l_run = 0.f, lt_run = 0.f;

        vm_wait_all();
        // tell the compiler the Q fragments are in registers now (otherwise it waits for every outstanding load,
        // the next tile's DMA included, in front of the first MFMA of each iteration)
#pragma unroll
        for (int c = 0; c < D / 32; ++c) asm volatile("" : "+v"(qf[c]));
        __syncthreads();
        int bufi = 0;

        while (have) {
            int lane_l = lane;
            asm volatile("" : "+v"(lane_l));
            const bool have_next = fetch();
            if (have_next)
                issue_tile(L, wave, lane_l, kbase + (long long)n_tok0 * sk_bytes, vbase + (long long)n_tok0 * sv_bytes, sk_bytes, sv_bytes,
                           n_nvalid, smem_lds + (bufi ^ 1) * SM::stageBytes);
            const char* stage = smem + bufi * SM::stageBytes;

            // 32-key chunks of the tile this wave needs: limited by the real keys in the tile and, on the block's own
            // keys, by the diagonal (last row of the wave is row0 + 15).  Tile quantities go to the arithmetic as
            // per-lane values (scalar ones make the variant selection need far more registers).
            int v_nvalid = c_nvalid, v_f = c_f;
            asm volatile("" : "+v"(v_nvalid), "+v"(v_f));
            int nkb = (v_nvalid + 31) >> 5;
            const bool c_self = v_f >= nprev;
            const int key0 = (v_f - nprev) * BR_BN;
            if (c_self) {
                const int vis = row0 + RW - key0;
                const int c = vis <= 0 ? 0 : (vis + 31) >> 5;
                nkb = c < nkb ? c : nkb;
            }
            if (!rb_active) nkb = 0;
            const bool need_mask = (v_nvalid < nkb * 32) || (c_self && key0 + nkb * 32 - 1 > row0);
            float psum = 0.f;
            if (nkb > 0) {
                const int lim_causal = c_self ? row0 + lr - key0 + 1 : BR_BN;
                const int lim = v_nvalid < lim_causal ? v_nvalid : lim_causal;
                // (the instance with score partials / log-sum-exp keeps the exact sums in every tile: one set of variants)
                if (nkb == 2 && !need_mask) compute_tile<2, false, SC>(stage, L, qf, o, m_run, l_run, lt_run, sc2, 0, lg, psum);
                else if (nkb == 2) compute_tile<2, true, SC>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lg, psum);
                else if (need_mask) compute_tile<1, true, SC>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lg, psum);
                else compute_tile<1, false, SC>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lg, psum);
            }
            if constexpr (SC) {
                // Score partials: this tile's probability mass (against the running max) for the query block's last rows
                if (emit_scores && nkb > 0 && !c_self && c_f >= first_doc_tile) {
                    const float tot = sum_quad(psum);
                    const int lr_l = lane_l & 15;
                    const int r16 = it.start_m + row0 + lr_l - (p.H - p.score_R);
                    if (lane_l < 16 && r16 >= 0 && row0 + lr_l < len_w) {
                        float2 ms = make_float2(m_run == -INFINITY ? 0.f : m_run, tot);
                        *reinterpret_cast<float2*>(p.score_part + ((((long long)b * p.Nq + head) * p.score_R + r16) * pv.tps + c_f) * 2) = ms;
                    }
                }
            }

            if (wave == 0) pf.step();
            vm_wait_all();
            __syncthreads();
            bufi ^= 1;
            c_f = n_f; c_tok0 = n_tok0; c_nvalid = n_nvalid;
            have = have_next;
        }

        // ---- epilogue: lane (lr, lg) holds row row0 + lr, dims 16 d + 4 lg + 0..3 ----
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        const float lt_tot = sum_quad(lt_run);              // sum of the rounded probabilities: normalises the output
        if (it.slot >= 0) {
            if (row0 + lr < len_w) {
                const long long slot = (long long)it.slot * ge.NHG + hg;
                const long long prow = slot * (NW / 2 * BR_RB) + ww * BR_RB + half * RW + lr;
                float* po = p.part_o + prow * D;
#pragma unroll
                for (int d = 0; d < D / 16; ++d) *reinterpret_cast<f32x4*>(po + d * 16 + 4 * lg) = o[d];
                if constexpr (SC) {
                    if (lse_out) {
                        const float l_tot = sum_quad(l_run);
                        if (lg == 0) p.part_lx[prow] = l_tot;
                    }
                }
                if (lg == 0) {
                    p.part_ml[prow * 2] = m_run;
                    p.part_ml[prow * 2 + 1] = lt_tot;
                }
            }
        } else {
            // the last loop iteration ended with a barrier, so the K/V buffers are free: transpose through LDS so
            // that every output row is written as full 16-byte pieces
            BR_E16* Es = reinterpret_cast<BR_E16*>(smem + wave * eBytesPerWave);
            const float inv = lt_tot > 0.f ? __builtin_amdgcn_rcpf(lt_tot) : 0.f;
            if constexpr (SC) {
                if (lse_out) {
                    const float l_tot = sum_quad(l_run);    // exact sum: log-sum-exp
                    if (lane_e < 16 && row0 + lane_e < len_w)
                        p.lse[(long long)b * p.lse_b + (long long)head * p.lse_h + qtok0 + row0 + lane_e] = m_run + __builtin_amdgcn_logf(l_tot);
                }
            }
            if (rb_active) {
#pragma unroll
                for (int d = 0; d < D / 16; ++d) {
                    const f32x4 t = o[d] * inv;
                    *reinterpret_cast<e16x4*>(Es + lr * eRow + d * 16 + 4 * lg) = __builtin_convertvector(t, e16x4);
                }
                __threadfence_block();      // same wave wrote and reads: keeps the compiler from moving the reads up
                constexpr int RPI = 64 / CPR, NIT = RW / RPI;
                const unsigned le = (unsigned)lane_e;
                const unsigned rsub = le / CPR, c8 = le % CPR;
                uint4 vals[NIT];
#pragma unroll
                for (int i = 0; i < NIT; ++i) vals[i] = ld16(Es + (rsub + i * RPI) * eRow + c8 * 8);
                const unsigned long long row_first = (unsigned)(qtok0 + row0);
                char* optr = reinterpret_cast<char*>(p.out) +
                             2 * ((unsigned long long)p.o32_b * (unsigned)b + (unsigned long long)p.o32_h * (unsigned)head +
                                  (unsigned long long)p.o32_t * (row_first + rsub) + c8 * 8);
                const long long stepb = 2LL * RPI * p.o32_t;
                if (row0 + RW <= len_m) {
#pragma unroll
                    for (int i = 0; i < NIT; ++i) *reinterpret_cast<uint4*>(optr + i * stepb) = vals[i];
                } else {
#pragma unroll
                    for (int i = 0; i < NIT; ++i)
                        if (row0 + (int)rsub + i * RPI < len_m) *reinterpret_cast<uint4*>(optr + i * stepb) = vals[i];
                }
            }
        }
        // a document's padded slots get zeros from the item that holds its first query tile (see the wide kernel)
        if (it.t0 == 0 && m > 0 && m < p.M - 1 && padded_layout)
            zero_padded_rows<D>(p, b, kvh * ge.G + hsub * ge.Gw, ge.G - hsub * ge.Gw < ge.Gw ? ge.G - hsub * ge.Gw : ge.Gw,
                                it.tok_m - it.start_m, it.start_m, len_m, tid, NW * 64);
    }
};

template <int D, bool SC>
__global__ __launch_bounds__(512, 4) void br_prefill_narrow_kernel(BrPrefillParams p) {
    using PF = PrefillNarrow<D, SC>;
    __shared__ __attribute__((aligned(1024))) char smem[2 * PF::SM::stageBytes + 2 * sizeof(BrDescMail)];
    BrDescMail* mail = reinterpret_cast<BrDescMail*>(smem + 2 * PF::SM::stageBytes);
    const int NHG = p.geom.NHG;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, p.geom.tpb * BR_RB);
    int* hdr = const_cast<int*>(p.plan);
    const int wave = uni(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const typename PF::Lane L = PF::make_lane(p, wave, lane);
    // DMA pieces of partial tiles are skipped, so whatever sits in LDS must be finite: start from zero
    for (int i = threadIdx.x * 16; i < 2 * PF::SM::stageBytes; i += PF::NW * 64 * 16) *reinterpret_cast<uint4*>(smem + i) = uint4{0u, 0u, 0u, 0u};
    const bool padded_layout = uni(hdr[BR_PH_PACKED]) == 0;
    BrPrefetch pf;
    pf.init(hdr, &pv, NHG, lane);
    if (wave == 0) pf.publish(&mail[0]);
    __syncthreads();
    for (int cur = 0;; cur ^= 1) {
        const int mw = reinterpret_cast<const int*>(&mail[cur])[lane < BR_ITEM_INTS + 2 ? lane : 0];
#define BR_W(i) __builtin_amdgcn_readlane(mw, i)
        if (BR_W(BR_ITEM_INTS + 1) == 0) break;     // .valid
        BrItem it;
        it.b = BR_W(0); it.m = BR_W(1); it.t0 = BR_W(2); it.f_lo = BR_W(3); it.nprev = BR_W(4); it.ntiles = BR_W(5); it.slot = BR_W(6);
        it.pe = BR_W(7); it.len_m = BR_W(8); it.start_m = BR_W(9); it.len0 = BR_W(10); it.start0 = BR_W(11); it.tok_m = BR_W(12);
        it.tok0 = BR_W(13);
        it.pad[0] = it.pad[1] = 0;
        const int hg = BR_W(BR_ITEM_INTS);          // .hg
#undef BR_W
        if (wave == 0) pf.draw();
        PF::run_item(p, pv, it, hg, smem, L, pf, padded_layout);
        if (wave == 0) pf.publish(&mail[cur ^ 1]);
        __syncthreads();
    }
    if (threadIdx.x == 0) br_leave(hdr);
}

}  // namespace
