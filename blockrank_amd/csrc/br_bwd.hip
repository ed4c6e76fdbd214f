// Backward of the block-sparse prefill attention for gfx950 (bf16 inputs, fp32 arithmetic and accumulation).
//
// The reference has no hand-written backward: its trainable hooks (blockrank_std_attention.py:96-262, :472-650,
// used by trainer.py:79-101) are differentiated by torch autograd over dense masked tensors, and its Triton
// hook refuses (blockrank_triton_kernel_attention.py:759-761).  These kernels compute the same gradients
//     P = softmax(S),  dV = P^T dO,  dP = dO V^T,  dS = P * (dP - rowsum(dO * O)),
//     dQ = scale * dS K,  dK = scale * dS^T Q        (dK, dV summed over the query heads of a kv head)
// over exactly the (query row, key) pairs the forward visits.  P is rebuilt from the log-sum-exp the forward
// saved.  Two kernels, so that every sum that has one owner is kept in that owner's registers:
//
//   br_bwd_dq_kernel   query-major: walks the forward's own work items, one
//                      workgroup per (item, head group), a wave per 32 rows of one query head.  Per 64-key tile
//                      (K, V staged in LDS):  S^T = K Q^T, dP^T = V dO^T  (lane = query row, registers = keys)
//                      -> dS^T in bf16 is directly the A operand of dQ += dS K (K through transposing LDS reads).
//                      An item that owns its rows stores dQ; the items that share the query block's rows (its key
//                      walk is split) add into a small fp32 buffer that a finishing kernel converts.  Also writes
//                      delta = rowsum(dO * O) for the second kernel.
//   br_bwd_dkv_kernel  key-major: one workgroup per (64-key tile, kv head); a wave owns 32 of the keys and walks,
//                      for half of the group's query heads, every 32-row block that sees them (the rest of the
//                      key's own block from the diagonal on; for prefix keys all later blocks; for document keys
//                      the query block).  S = Q K^T, dP = dO V^T (lane = key, registers = rows) -> P and dS in
//                      bf16 are directly the A operands of dV += P^T dO and dK += dS^T Q, with dO and Q as
//                      "lane = dim, registers = rows" operands obtained by transposing LDS reads of the wave's
//                      own copy of the rows.  dK and dV never leave the registers until the walk ends: no atomics.
#include "br_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

__device__ inline uint4 ld16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline bf16x8 as_bf16x8(uint4 u) {
    union { uint4 u; bf16x8 v; } c;
    c.u = u;
    return c.v;
}
// Workgroup barrier that waits for this wave's LDS operations only.  __syncthreads() also waits for its outstanding
// global loads, which would make every barrier wait for the rows requested ahead for the next step.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ inline f32x16 mma(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
__device__ inline f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    return z;
}
// accumulator registers 8s .. 8s+7 as one bf16 operand
__device__ inline bf16x8 pack8(const f32x16& x, int s) {
    f32x8 t;
#pragma unroll
    for (int e = 0; e < 8; ++e) t[e] = x[8 * s + e];
    return __builtin_convertvector(t, bf16x8);
}

template <int D>
struct Bwd {
    static constexpr int RS = 2 * D + 32;          // LDS row stride in bytes: the 32 bytes of padding put the four rows of a transposing read in different banks
    static constexpr int CPR = D / 8;              // 16-byte pieces per row
    static constexpr int NC = D / 16, ND = D / 32;
    static constexpr int tileBytes = BR_BN * RS;
    static constexpr int rowsBytes = BR_RB * RS;

    // Row (r0 + lane % 32), dims 16c + 8 * (lane / 32) .. +7 of a row-major LDS tile: the operand layout of a
    // product that contracts over the head dim.
    static __device__ inline bf16x8 read_row(const char* tile, int r0, int c, int ln, int lh) {
        return as_bf16x8(ld16(tile + (r0 + ln) * RS + c * 32 + lh * 16));
    }
    // Column (32 db + lane % 32), rows r0 + 4 lh + {0..3, 8..11} of a row-major LDS tile: the operand layout of a
    // product that contracts over rows, in the order in which a 32x32 accumulator's registers 8s .. 8s+7 hold
    // them (r0 = 16 s).  Two transposing reads: in each group of 16 lanes, lane s points at row (s >> 2),
    // dims 4 (s & 3) .. +3 of the group's 16 dims and receives the four rows of dim s.
    static __device__ inline bf16x8 read_col(const char* tile, int r0, int db, int lane) {
        const int s = lane & 15, hi = (lane >> 4) & 1, lh = lane >> 5;
        const char* p = tile + (r0 + 4 * lh + (s >> 2)) * RS + (32 * db + 16 * hi + 4 * (s & 3)) * 2;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(__attribute__((address_space(3))) const char*)p);
        s16x4 up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(__attribute__((address_space(3))) const char*)(p + 8 * RS));
        union { s16x8 s8; bf16x8 b8; } a;
        a.s8 = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
        return a.b8;
    }

    // ---------------------------------------------------------------------------------------------------------
    // dQ (and delta) of one work item
    // ---------------------------------------------------------------------------------------------------------
    static constexpr int dqLdsBytes = 2 * tileBytes;

    static __device__ __forceinline__ void dq_item(const BrBwdParams& p, const BrPlanView& pv, const BrItem& it, int hg, char* smem, int NW) {
        const int tid = threadIdx.x, NT = NW * 64;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, ln = lane & 31, lh = lane >> 5;
        const BrGeom& ge = p.geom;
        const int T = ge.tpb * BR_RB;
        const int b = it.b;
        const int kvh = hg / ge.HGS, hsub = hg - kvh * ge.HGS;
        const int g = wave / ge.tpb, sub = wave - g * ge.tpb;
        const int head = kvh * ge.G + hsub * ge.Gw + g;
        const int len_m = it.len_m;
        const int row0 = it.t0 + sub * BR_RB;
        const bool rb_active = row0 < len_m;
        const int self_end = it.t0 + T < len_m ? it.t0 + T : len_m;
        const int qtok0 = it.tok_m;
        char* Ks = smem;
        char* Vs = smem + tileBytes;
        const char* kbase = reinterpret_cast<const char*>(p.k) + 2 * ((unsigned long long)p.k32_b * (unsigned)b + (unsigned long long)p.k32_h * (unsigned)kvh);
        const char* vbase = reinterpret_cast<const char*>(p.v) + 2 * ((unsigned long long)p.v32_b * (unsigned)b + (unsigned long long)p.v32_h * (unsigned)kvh);

        // Q and dO of this wave's rows (lane = row, registers = dims), the rows' log-sum-exp and delta
        bf16x8 qf[NC], dof[NC];
        float lse_l = 0.f, delta_l = 0.f;
        if (rb_active) {
            const int last = len_m - 1 - row0;
            const int r = ln < last ? ln : last;       // rows past the block's end repeat its last row; they are masked below
            const unsigned tok = (unsigned)(qtok0 + row0 + r);
            const char* qrow = reinterpret_cast<const char*>(p.q) +
                               2 * ((unsigned long long)p.q32_b * (unsigned)b + (unsigned long long)p.q32_h * (unsigned)head + (unsigned long long)p.q32_t * tok);
            const char* grow = reinterpret_cast<const char*>(p.dout) +
                               2 * ((unsigned long long)p.g32_b * (unsigned)b + (unsigned long long)p.g32_h * (unsigned)head + (unsigned long long)p.g32_t * tok);
            const char* orow = reinterpret_cast<const char*>(p.out) +
                               2 * ((unsigned long long)p.o32_b * (unsigned)b + (unsigned long long)p.o32_h * (unsigned)head + (unsigned long long)p.o32_t * tok);
            float dsum = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                qf[c] = as_bf16x8(ld16(qrow + c * 32 + lh * 16));
                dof[c] = as_bf16x8(ld16(grow + c * 32 + lh * 16));
                const bf16x8 o8 = as_bf16x8(ld16(orow + c * 32 + lh * 16));
#pragma unroll
                for (int e = 0; e < 8; ++e) dsum += (float)o8[e] * (float)dof[c][e];
            }
            delta_l = dsum + __shfl_xor(dsum, 32);
            const long long li = (long long)b * p.lse_b + (long long)head * p.lse_h + tok;
            lse_l = p.lse[li];
            // every item of a row block computes the same delta; the one that starts the key walk publishes it
            if (it.f_lo == 0 && lh == 0 && ln <= last) p.delta[li] = delta_l;
        } else {
#pragma unroll
            for (int c = 0; c < NC; ++c) qf[c] = dof[c] = as_bf16x8(uint4{0u, 0u, 0u, 0u});
        }

        f32x16 dq[ND];
#pragma unroll
        for (int db = 0; db < ND; ++db) dq[db] = zero16();

        // the item's key walk: the earlier blocks' tiles it covers, then its own block's up to the diagonal
        const int2* tiles_b = pv.tiles + (size_t)b * pv.tps;
        const bool table = it.pe > 1;
        const int nprev = it.nprev;
        const int f_end = it.ntiles > 0x3fffffff ? 0x7fffffff : it.f_lo + it.ntiles;
        // The walk is software-pipelined: a thread's pieces of the next tile are loaded into registers while the
        // current tile (in LDS) is computed.
        struct Tile {
            int tok0, nvalid, key0, self;
        };
        int f = it.f_lo;
        auto next_tile = [&](Tile& t) -> bool {
            while (f < f_end) {
                const int fi = f++;
                t.self = fi >= nprev;
                t.key0 = 0;
                if (!t.self) {
                    if (table) {
                        const int2 d = tiles_b[fi];
                        t.tok0 = d.x;
                        t.nvalid = d.y;
                    } else {
                        t.tok0 = it.tok0 + fi * BR_BN;
                        t.nvalid = it.len0 - fi * BR_BN < BR_BN ? it.len0 - fi * BR_BN : BR_BN;
                    }
                } else {
                    t.key0 = (fi - nprev) * BR_BN;
                    if (t.key0 >= self_end) {
                        f = f_end;
                        return false;
                    }
                    t.tok0 = it.tok_m + t.key0;
                    t.nvalid = self_end - t.key0 < BR_BN ? self_end - t.key0 : BR_BN;
                }
                if (t.nvalid > 0) return true;
            }
            return false;
        };
        constexpr int NPC = BR_BN * CPR / 256;     // 16-byte pieces of K (and of V) per thread and tile (at least 256 threads)
        uint4 kreg[NPC], vreg[NPC];
        auto load_tile = [&](const Tile& t) {      // rows past the tile's real keys are zero
#pragma unroll
            for (int i = 0; i < NPC; ++i) {
                const int idx = tid + i * NT;
                const int r = idx / CPR, c = idx - r * CPR;
                kreg[i] = vreg[i] = uint4{0u, 0u, 0u, 0u};
                if (idx < BR_BN * CPR && r < t.nvalid) {
                    kreg[i] = ld16(kbase + 2 * ((long long)(t.tok0 + r) * p.k32_t + c * 8));
                    vreg[i] = ld16(vbase + 2 * ((long long)(t.tok0 + r) * p.v32_t + c * 8));
                }
            }
        };
        Tile cur, nxt;
        bool have = next_tile(cur);
        if (have) load_tile(cur);
        // Everything requested so far (Q, dO, O, the first tile) is needed before the first product anyway: wait here,
        // so that the loop is entered with no load pending.  Otherwise the compiler's wait-count bookkeeping keeps
        // partial waits in front of every use of Q and dO inside the loop, and those waits count the tile requested
        // ahead - the look-ahead would wait for itself.
        __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0); expcnt and lgkmcnt not waited for
        while (have) {
            const bool self = cur.self;
            const int nvalid = cur.nvalid, key0 = cur.key0;
            lds_barrier();                         // every wave has finished with the previous tile
#pragma unroll
            for (int i = 0; i < NPC; ++i) {
                const int idx = tid + i * NT;
                const int r = idx / CPR, c = idx - r * CPR;
                if (idx < BR_BN * CPR) {
                    *reinterpret_cast<uint4*>(Ks + r * RS + c * 16) = kreg[i];
                    *reinterpret_cast<uint4*>(Vs + r * RS + c * 16) = vreg[i];
                }
            }
            const bool have_next = next_tile(nxt);
            if (have_next) load_tile(nxt);
            lds_barrier();

            // 32-key halves this wave needs: limited by the real keys and, on the block's own keys, by the diagonal
            int nkb = (nvalid + 31) >> 5;
            if (self) {
                const int vis = row0 + BR_RB - key0;
                const int c = vis <= 0 ? 0 : (vis + 31) >> 5;
                nkb = c < nkb ? c : nkb;
            }
            if (!rb_active) nkb = 0;
            for (int kb = 0; kb < nkb; ++kb) {
                f32x16 st = zero16(), dpt = zero16();
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    st = mma(read_row(Ks, kb * 32, c, ln, lh), qf[c], st);
                    dpt = mma(read_row(Vs, kb * 32, c, ln, lh), dof[c], dpt);
                }
                const int lim_c = self ? row0 + ln - key0 + 1 : BR_BN;                 // keys [0, lim) of the tile are visible
                int lim = nvalid < lim_c ? nvalid : lim_c;
                if (row0 + ln >= len_m) lim = 0;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int key = kb * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                    // hidden pairs get exponent -inf, i.e. probability 0, without a branch (every operand is finite)
                    const float pr = __builtin_amdgcn_exp2f(key < lim ? st[v] * p.scale_log2 - lse_l : -INFINITY);
                    st[v] = pr * (dpt[v] - delta_l) * p.scale;
                }
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const bf16x8 a = pack8(st, s);
                    // K as "lane = dim" operand of this 16-key step: the transposing reads are issued together, ahead of the products
                    bf16x8 kc[ND];
#pragma unroll
                    for (int db = 0; db < ND; ++db) kc[db] = read_col(Ks, kb * 32 + 16 * s, db, lane);
#pragma unroll
                    for (int db = 0; db < ND; ++db) dq[db] = mma(a, kc[db], dq[db]);
                }
            }
            cur = nxt;
            have = have_next;
        }
        // dQ of this wave's rows: lane = dim 32 db + ln, register v = row 8 (v/4) + 4 lh + v%4
        if (!rb_active) return;
        if (it.slot < 0) {
            __bf16* dst = reinterpret_cast<__bf16*>(p.dq) + (long long)b * p.dq_b + (long long)head * p.dq_h +
                          (long long)(qtok0 + row0 + 4 * lh) * p.dq_t + ln;
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = 8 * (v >> 2) + (v & 3);
                    if (row0 + 4 * lh + r < len_m) dst[(long long)r * p.dq_t + db * 32] = (__bf16)dq[db][v];
                }
        } else {
            // shared rows (the query block): [b][head][row of the block][D] fp32
            float* dqp = p.dq32 + (((long long)b * p.Nq + head) * p.H + row0 + 4 * lh) * D + ln;
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = 8 * (v >> 2) + (v & 3);
                    if (row0 + 4 * lh + r < len_m) unsafeAtomicAdd(dqp + r * D + db * 32, dq[db][v]);
                }
        }
    }

    // ---------------------------------------------------------------------------------------------------------
    // dK, dV of one 32-key half (kb) of a 64-key tile of one kv head.  128 threads: wave = side dh.
    // The two waves work on the same step - 32 query rows of one head - and split it: the dh = 0
    // wave loads the Q rows and computes S = Q K^T, the dh = 1 wave loads the dO rows and computes dP = dO V^T;
    // they exchange the two 32x32 results through LDS, and then each owns one half of the head dim of dV and dK
    // (dims [dh D/2, (dh+1) D/2)), whose "lane = dim" operands are transposing reads of the rows the pair has
    // copied to LDS.  16 MFMAs per wave and step, nothing computed twice; per wave 64 accumulator registers, 32 of
    // K or V operands, 32 of rows in flight: about 200 in all, so four workgroups share a CU.
    // ---------------------------------------------------------------------------------------------------------
    static constexpr int xBytes = 2 * 4 * 64 * 16;                        // the pair's two 32x32 fp32 results
    static constexpr int pairBytes = 2 * rowsBytes + xBytes + 256;        // 32 rows of Q, of dO, the exchange, lse and delta
    static constexpr int dkvLdsBytes = pairBytes;

    // mq_only < 0: the tile's main workgroup - viewers are the rest of the keys' own block and, for document keys,
    // the query block; mq_only >= 1 (prefix keys only): the rows of block mq_only.  Prefix keys have a workgroup
    // per viewing block, so their sums meet in fp32 buffers (atomic adds); all other keys have one owner, which
    // stores bf16.
    static __device__ __forceinline__ void dkv_tile(const BrBwdParams& p, const BrPlanView& pv, int b, int m, int kt, int kb, int kvh, int mq_only, char* smem) {
        constexpr int NH = ND / 2 > 0 ? ND / 2 : 1;                    // 32-dim blocks a wave owns
        static_assert(ND % 2 == 0, "the head dim is split in two halves of whole 32-dim blocks");
        const int tid = threadIdx.x;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, ln = lane & 31, lh = lane >> 5;
        const int dh = wave;
        const int G = p.geom.G, M = p.M;
        const int len_m = pv.len[b * M + m], tok_m = pv.tok[b * M + m];
        const int key0 = kt * BR_BN;
        const int nvalid = len_m - key0 < BR_BN ? len_m - key0 : BR_BN;      // > kb * 32: checked by the caller
        char* Wq = smem;
        char* Wd = Wq + rowsBytes;
        uint4* X = reinterpret_cast<uint4*>(Wd + rowsBytes);              // [2 sides][4][64 lanes] x 16 bytes
        float* Wl = reinterpret_cast<float*>(Wd + rowsBytes + xBytes);    // [32] log-sum-exp, [32] delta

        // this wave's side: Q rows against K (dh = 0) or dO rows against V (dh = 1)
        const char* kv_t = reinterpret_cast<const char*>(dh == 0 ? p.k : p.v);
        const unsigned kv_b = dh == 0 ? p.k32_b : p.v32_b, kv_h = dh == 0 ? p.k32_h : p.v32_h, kv_s = dh == 0 ? p.k32_t : p.v32_t;
        const char* row_t = reinterpret_cast<const char*>(dh == 0 ? p.q : p.dout);
        const unsigned row_b = dh == 0 ? p.q32_b : p.g32_b, row_h = dh == 0 ? p.q32_h : p.g32_h, row_s = dh == 0 ? p.q32_t : p.g32_t;
        const float* stat = dh == 0 ? p.lse : p.delta;
        char* Wmine = dh == 0 ? Wq : Wd;

        // the wave's 32 keys as operands (lane = key, registers = dims); rows past the real keys are zero
        bf16x8 ks[NC];
        {
            const int key = kb * 32 + ln;
            const bool on = key < nvalid;
            const unsigned tok = (unsigned)(tok_m + key0 + (on ? key : 0));
            const char* row = kv_t + 2 * ((unsigned long long)kv_b * (unsigned)b + (unsigned long long)kv_h * (unsigned)kvh + (unsigned long long)kv_s * tok);
#pragma unroll
            for (int c = 0; c < NC; ++c) ks[c] = as_bf16x8(on ? ld16(row + c * 32 + lh * 16) : uint4{0u, 0u, 0u, 0u});
        }
        f32x16 dk[NH], dv[NH];      // lane = dim 32 (dh NH + j) + ln, register v = key kb*32 + 8 (v/4) + 4 lh + v%4
#pragma unroll
        for (int j = 0; j < NH; ++j) dk[j] = dv[j] = zero16();
        const bool half_on = kb * 32 < nvalid;

        // The workgroup's steps: (32-row block that sees these keys, head of the group).  Row blocks come from up to
        // two blocks: the keys' own block from the diagonal on, then the query block (document keys) - or, for a
        // prefix-key workgroup of a viewing block, that block alone.  The step sequence is the same for both waves
        // (they meet at barriers).
        struct Step {
            int r0, nrows, tok, head, self;
        };
        const int blk0 = mq_only < 0 ? m : mq_only;
        const int blk1 = (mq_only < 0 && m > 0 && m < M - 1) ? M - 1 : -1;
        int seg = 0;                                                 // 2 = exhausted
        int cur_blk = blk0, cur_len = pv.len[b * M + blk0], cur_tok = pv.tok[b * M + blk0];
        int rb = mq_only < 0 ? key0 / BR_RB : 0, hl = 0;
        auto next_step = [&](Step& st) -> bool {
            while (seg < 2) {
                if (rb * BR_RB >= cur_len) {
                    seg = (seg == 0 && blk1 >= 0) ? 1 : 2;
                    if (seg == 1) {
                        cur_blk = blk1;
                        cur_len = pv.len[b * M + blk1];
                        cur_tok = pv.tok[b * M + blk1];
                        rb = 0;
                    }
                    continue;
                }
                const int r0 = rb * BR_RB;
                st.r0 = r0;
                st.nrows = cur_len - r0 < BR_RB ? cur_len - r0 : BR_RB;
                st.tok = cur_tok + r0;
                st.head = kvh * G + hl;
                st.self = cur_blk == m;
                if (++hl >= G) {
                    hl = 0;
                    ++rb;
                }
                return true;
            }
            return false;
        };
        // the pair's key half has a pair to compute in this step (causal rule on the block's own keys: nothing if even
        // the last row precedes the half's first key)
        auto has_work = [&](const Step& st) { return half_on && !(st.self && st.r0 + st.nrows - 1 < key0 + kb * 32); };
        // this side's rows of a step (lane = row, registers = dims; rows past the block's end repeat its last row and
        // are masked later) and the rows' log-sum-exp (dh = 0) or delta (dh = 1); lane ln holds row ln's
        auto load_step = [&](const Step& st, uint4 (&rv)[NC], float& stat_l) {
            const int r = ln < st.nrows ? ln : st.nrows - 1;
            const unsigned tok = (unsigned)(st.tok + r);
            const char* row = row_t + 2 * ((unsigned long long)row_b * (unsigned)b + (unsigned long long)row_h * (unsigned)st.head + (unsigned long long)row_s * tok);
#pragma unroll
            for (int c = 0; c < NC; ++c) rv[c] = ld16(row + c * 32 + lh * 16);
            stat_l = stat[(long long)b * p.lse_b + (long long)st.head * p.lse_h + tok];
        };
        {
            // Per step: barrier (every wave is done with the previous rows); copy this side's rows to LDS; this side's
            // product from the registers, result to the exchange - after which the registers are free, so the next
            // step's loads are issued into them; barrier (rows and both products are in LDS); the other side's
            // product; softmax terms; dV and dK products of this wave's half of the head dim.
            Step cur, nxt;
            uint4 rv[NC], rn[NC];
            float stat_c = 0.f, stat_n = 0.f;
            bool have = next_step(cur);
            if (have && has_work(cur)) load_step(cur, rv, stat_c);
            // Wait for the first step's rows here.  Entering the loop with loads still pending makes the compiler's
            // wait-count bookkeeping treat the current rows as "loaded a few requests ago" in every iteration: it
            // then puts partial waits in front of each use, and those waits count the rows requested ahead for
            // the next step - the look-ahead would wait for itself.
            __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0); expcnt and lgkmcnt not waited for
            while (have) {
                const bool have_next = next_step(nxt);
                const bool work = has_work(cur);
                if (have_next && has_work(nxt)) load_step(nxt, rn, stat_n);
                lds_barrier();
                f32x16 mine = zero16();
                if (work) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) *reinterpret_cast<uint4*>(Wmine + ln * RS + c * 32 + lh * 16) = rv[c];
                    if (lh == 0) Wl[dh * 32 + ln] = stat_c;
#pragma unroll
                    for (int c = 0; c < NC; ++c) mine = mma(as_bf16x8(rv[c]), ks[c], mine);
#pragma unroll
                    for (int v4 = 0; v4 < 4; ++v4) {
                        const f32x4 t = {mine[4 * v4], mine[4 * v4 + 1], mine[4 * v4 + 2], mine[4 * v4 + 3]};
                        *reinterpret_cast<f32x4*>(X + (dh * 4 + v4) * 64 + lane) = t;
                    }
                }
                lds_barrier();
                if (work) {
                    f32x16 other;
#pragma unroll
                    for (int v4 = 0; v4 < 4; ++v4) {
                        const f32x4 t = *reinterpret_cast<const f32x4*>(X + ((1 - dh) * 4 + v4) * 64 + lane);
                        other[4 * v4] = t[0]; other[4 * v4 + 1] = t[1]; other[4 * v4 + 2] = t[2]; other[4 * v4 + 3] = t[3];
                    }
                    const int key = kb * 32 + ln;
                    f32x16 pr16, ds16;
                    // most steps see every pair (whole key half, whole row block, nothing above the diagonal): they
                    // skip the per-pair visibility test.  sa / da are S and dP whichever side computed them.
                    const bool all_visible = nvalid - kb * 32 >= 32 && cur.nrows == BR_RB && (!cur.self || key0 + kb * 32 + 31 <= cur.r0);
                    auto terms = [&](const f32x16& sa, const f32x16& da) {
#pragma unroll
                        for (int v4 = 0; v4 < 4; ++v4) {
                            // accumulator registers 4 v4 .. 4 v4 + 3 hold rows r0 + 8 v4 + 4 lh + 0..3
                            const f32x4 l4 = *reinterpret_cast<const f32x4*>(Wl + 8 * v4 + 4 * lh);
                            const f32x4 d4 = *reinterpret_cast<const f32x4*>(Wl + 32 + 8 * v4 + 4 * lh);
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int v = 4 * v4 + e, i = 8 * v4 + 4 * lh + e;
                                float x = sa[v] * p.scale_log2 - l4[e];
                                if (!all_visible) {
                                    // hidden pairs get exponent -inf, i.e. probability 0, without a branch (every operand is finite)
                                    const bool vis = key < nvalid && i < cur.nrows && (!cur.self || key0 + key <= cur.r0 + i);
                                    x = vis ? x : -INFINITY;
                                }
                                const float pr = __builtin_amdgcn_exp2f(x);
                                pr16[v] = pr;
                                ds16[v] = pr * (da[v] - d4[e]) * p.scale;
                            }
                        }
                    };
                    if (dh == 0) terms(mine, other);
                    else terms(other, mine);
                    // the "lane = dim" operands of one 16-row step at a time: its reads are issued together, ahead of its products
#pragma unroll
                    for (int s2 = 0; s2 < 2; ++s2) {
                        const bf16x8 pa = pack8(pr16, s2), da = pack8(ds16, s2);
                        bf16x8 cd[NH], cq[NH];
#pragma unroll
                        for (int j = 0; j < NH; ++j) {
                            cd[j] = read_col(Wd, 16 * s2, dh * NH + j, lane);
                            cq[j] = read_col(Wq, 16 * s2, dh * NH + j, lane);
                        }
#pragma unroll
                        for (int j = 0; j < NH; ++j) {
                            dv[j] = mma(pa, cd[j], dv[j]);
                            dk[j] = mma(da, cq[j], dk[j]);
                        }
                    }
                }
                cur = nxt;
                stat_c = stat_n;
#pragma unroll
                for (int c = 0; c < NC; ++c) rv[c] = rn[c];
                have = have_next;
            }
        }

        if (!half_on) return;
        if (m == 0 && M > 1) {
            // prefix keys: add into the fp32 buffers [b][kv head][key][D]
            const long long base = (((long long)b * p.Nkv + kvh) * p.H + key0 + kb * 32 + 4 * lh) * D + dh * NH * 32 + ln;
#pragma unroll
            for (int j = 0; j < NH; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int kr = 8 * (v >> 2) + (v & 3);
                    if (kb * 32 + 4 * lh + kr < nvalid) {
                        unsafeAtomicAdd(p.dk32 + base + kr * D + j * 32, dk[j][v]);
                        unsafeAtomicAdd(p.dv32 + base + kr * D + j * 32, dv[j][v]);
                    }
                }
            return;
        }
        // every other key has this one owner: store bf16
        __bf16* dkp = reinterpret_cast<__bf16*>(p.dk) + (long long)b * p.dk_b + (long long)kvh * p.dk_h +
                      (long long)(tok_m + key0 + kb * 32 + 4 * lh) * p.dk_t + dh * NH * 32 + ln;
        __bf16* dvp = reinterpret_cast<__bf16*>(p.dv) + (long long)b * p.dv_b + (long long)kvh * p.dv_h +
                      (long long)(tok_m + key0 + kb * 32 + 4 * lh) * p.dv_t + dh * NH * 32 + ln;
#pragma unroll
        for (int j = 0; j < NH; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int kr = 8 * (v >> 2) + (v & 3);
                if (kb * 32 + 4 * lh + kr < nvalid) {
                    dkp[(long long)kr * p.dk_t + j * 32] = (__bf16)dk[j][v];
                    dvp[(long long)kr * p.dv_t + j * 32] = (__bf16)dv[j][v];
                }
            }
    }
};

template <int D, int MAXW>
__global__ __launch_bounds__(MAXW * 64, MAXW <= 4 ? (D == 64 ? 3 : 2) : 1) void br_bwd_dq_kernel(BrBwdParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const BrGeom& ge = p.geom;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, ge.tpb * BR_RB);
    const int item = blockIdx.x / ge.NHG, hg = blockIdx.x - item * ge.NHG;
    if (item >= pv.hdr[BR_PH_NITEMS]) return;
    const BrItem it = pv.items[item];
    Bwd<D>::dq_item(p, pv, it, hg, smem, blockDim.x >> 6);
}

// Work is enumerated as (group, slot): a group is one (block m, sequence, kv head) and holds every workgroup that
// reads that block's Q and dO rows - for each 64-key tile of the block and each 32-key half its main workgroup,
// plus (m >= 1) the workgroups that take the block's rows to the prefix keys.  The hardware deals workgroups
// round robin to the 8 XCDs by index, and each XCD has its own L2: group g is therefore laid out on indices
// congruent to g mod 8, so that all its workgroups run on one XCD and the rows are fetched from HBM into one L2
// only (measured at the Mistral-7B shape with 20 documents: 0.39 GB of HBM reads per launch against 1.25 GB with
// a plain enumeration, where every row block was fetched by up to eight workgroups on different XCDs; 0.27 GB
// is the algorithmic minimum).
template <int D>
__global__ __launch_bounds__(128, D == 64 ? 3 : 2) void br_bwd_dkv_kernel(BrBwdParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, p.geom.tpb * BR_RB);
    const int KT = (p.H + BR_BN - 1) / BR_BN;
    const int S = 4 * KT;                                    // slots per group
    const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int g = (j / S) * 8 + x, slot = j % S;
    if (g >= p.M * p.B * p.Nkv) return;
    const int kvh = g % p.Nkv, b = (g / p.Nkv) % p.B, mg = g / (p.Nkv * p.B);
    const bool extra = slot >= 2 * KT;
    const int kt = (extra ? slot - 2 * KT : slot) >> 1, kb = slot & 1;
    if (extra && mg == 0) return;
    const int m = extra ? 0 : mg, mq_only = extra ? mg : -1;
    const int len_m = pv.len[b * p.M + m];
    // padded slots of this block (dk and dv of this kv head): zeros, written by the block's first workgroup
    if (kt == 0 && kb == 0 && mq_only < 0 && !pv.hdr[BR_PH_PACKED]) {
        const int st = pv.start[b * p.M + m], npad = p.H - len_m;
        constexpr int CP8 = D / 8;
        const uint4 z = {0u, 0u, 0u, 0u};
        __bf16* kb_ = reinterpret_cast<__bf16*>(p.dk) + (long long)b * p.dk_b + (long long)kvh * p.dk_h;
        __bf16* vb_ = reinterpret_cast<__bf16*>(p.dv) + (long long)b * p.dv_b + (long long)kvh * p.dv_h;
        for (int i = threadIdx.x; i < npad * CP8; i += blockDim.x) {
            const int r = i / CP8, c8 = i - r * CP8;
            const long long pos = (long long)m * p.H + (r < st ? r : r + len_m);
            *reinterpret_cast<uint4*>(kb_ + pos * p.dk_t + c8 * 8) = z;
            *reinterpret_cast<uint4*>(vb_ + pos * p.dv_t + c8 * 8) = z;
        }
    }
    if (kt * BR_BN + kb * 32 >= len_m) return;           // no real key in this half
    Bwd<D>::dkv_tile(p, pv, b, m, kt, kb, kvh, mq_only, smem);
}

__global__ __launch_bounds__(256) void br_fill_zero_kernel(uint4* p, size_t n16) {
    const uint4 z = {0u, 0u, 0u, 0u};
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) p[i] = z;
}

// dQ of the rows whose key walk was split (the plan's combine list names their query tiles): fp32 sums -> bf16;
// and zeros for the padded slots of dq.
template <int D>
__global__ __launch_bounds__(256) void br_bwd_dq_finish_kernel(BrBwdParams p) {
    const BrGeom& ge = p.geom;
    const int T = ge.tpb * BR_RB;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, T);
    constexpr int C4 = D / 4;
    const int m = p.M - 1;
    const long long n = (long long)pv.hdr[BR_PH_NCOMB] * p.Nq * T * C4;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(i % C4);
        long long r = i / C4;
        const int row_in = (int)(r % T);
        r /= T;
        const int head = (int)(r % p.Nq), ci = (int)(r / p.Nq);
        const BrComb cb = pv.comb[ci];
        const int row = cb.t0 + row_in;
        if (row >= pv.len[cb.b * p.M + m]) continue;
        const f32x4 x = *reinterpret_cast<const f32x4*>(p.dq32 + (((long long)cb.b * p.Nq + head) * p.H + row) * D + c * 4);
        __bf16* dst = reinterpret_cast<__bf16*>(p.dq) + (long long)cb.b * p.dq_b + (long long)head * p.dq_h +
                      (long long)(pv.tok[cb.b * p.M + m] + row) * p.dq_t + c * 4;
        *reinterpret_cast<bf16x4*>(dst) = __builtin_convertvector(x, bf16x4);
    }
    // dK, dV of the prefix keys (summed over the workgroups of every viewing block)
    if (p.M > 1) {
        const long long nk = (long long)p.B * p.Nkv * p.H * C4;
        for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < nk; i += (long long)gridDim.x * blockDim.x) {
            const int c = (int)(i % C4);
            long long r = i / C4;
            const int key = (int)(r % p.H);
            r /= p.H;
            const int kvh = (int)(r % p.Nkv), b = (int)(r / p.Nkv);
            if (key >= pv.len[b * p.M]) continue;
            const long long src = (((long long)b * p.Nkv + kvh) * p.H + key) * D + c * 4;
            const long long tokk = pv.tok[b * p.M] + key;
            *reinterpret_cast<bf16x4*>(reinterpret_cast<__bf16*>(p.dk) + (long long)b * p.dk_b + (long long)kvh * p.dk_h + tokk * p.dk_t + c * 4) =
                __builtin_convertvector(*reinterpret_cast<const f32x4*>(p.dk32 + src), bf16x4);
            *reinterpret_cast<bf16x4*>(reinterpret_cast<__bf16*>(p.dv) + (long long)b * p.dv_b + (long long)kvh * p.dv_h + tokk * p.dv_t + c * 4) =
                __builtin_convertvector(*reinterpret_cast<const f32x4*>(p.dv32 + src), bf16x4);
        }
    }
    if (pv.hdr[BR_PH_PACKED]) return;
    constexpr int CP8 = D / 8;
    const uint4 z = {0u, 0u, 0u, 0u};
    for (int w = blockIdx.x; w < p.B * p.M * p.Nq; w += gridDim.x) {
        const int bm = w / p.Nq, head = w - bm * p.Nq;
        const int b = bm / p.M, mm = bm - b * p.M;
        const int st = pv.start[bm], ln = pv.len[bm], npad = p.H - ln;
        __bf16* base = reinterpret_cast<__bf16*>(p.dq) + (long long)b * p.dq_b + (long long)head * p.dq_h;
        for (int idx = threadIdx.x; idx < npad * CP8; idx += blockDim.x) {
            const int r = idx / CP8, c8 = idx - r * CP8;
            const long long pos = (long long)mm * p.H + (r < st ? r : r + ln);
            *reinterpret_cast<uint4*>(base + pos * p.dq_t + c8 * 8) = z;
        }
    }
}

template <int D, int MAXW>
int launch_dq(const BrBwdParams& p, int NW, hipStream_t stream) {
    constexpr int lds = Bwd<D>::dqLdsBytes;
    static_assert(lds <= 65536, "dynamic LDS above 64 KiB would need hipFuncSetAttribute");
    hipLaunchKernelGGL((br_bwd_dq_kernel<D, MAXW>), dim3(p.max_items * p.geom.NHG), dim3(NW * 64), lds, stream, p);
    return 0;
}

template <int D>
int launch_all(const BrBwdParams& p, int NW, int n_cu, hipStream_t stream) {
    const size_t n16 = (size_t)p.B * (p.Nq + 2 * p.Nkv) * p.H * D / 4;      // dq32, dk32, dv32 are contiguous
    hipLaunchKernelGGL(br_fill_zero_kernel, dim3(n_cu * 4), dim3(256), 0, stream, reinterpret_cast<uint4*>(p.dq32), n16);
    const int rc = NW <= 4 ? launch_dq<D, 4>(p, NW, stream) : launch_dq<D, 8>(p, NW, stream);
    if (rc) return rc;
    constexpr int lds = Bwd<D>::dkvLdsBytes;
    static_assert(lds <= 65536, "dynamic LDS above 64 KiB would need hipFuncSetAttribute");
    const int KT = (p.H + BR_BN - 1) / BR_BN;
    hipLaunchKernelGGL((br_bwd_dkv_kernel<D>), dim3((p.M * p.B * p.Nkv + 7) / 8 * 8 * 4 * KT), dim3(128), lds, stream, p);
    hipLaunchKernelGGL((br_bwd_dq_finish_kernel<D>), dim3(n_cu * 4), dim3(256), 0, stream, p);
    return 0;
}

}  // namespace

// Returns 0 on success, -1 if D has no instance.
int br_launch_bwd(const BrBwdParams& p, int D, int NW, int n_cu, hipStream_t stream) {
    if (D == 128) return launch_all<128>(p, NW, n_cu, stream);
    if (D == 64) return launch_all<64>(p, NW, n_cu, stream);
    return -1;
}
