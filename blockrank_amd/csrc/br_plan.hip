// Request plan: turns the (B, M, H) block mask into the block table (start, len per block) and the
// work-item list the persistent prefill kernel consumes.  Built on the device with no host
// synchronisation, once per forward pass (the block structure is the same for every layer).
//
// The additive 5-D mask of the reference (blockrank_std_attention.py:293-309) carries exactly this
// information: which keys of each block are real.  Everything else (causality inside a block, which
// earlier blocks a block may see) follows from the block index, so the kernels never read a mask.
#include "br_common.h"

namespace {

constexpr int kPlanThreads = 1024;

// One wave per block: count real tokens, find the first and the last.  len is written negated
// (-1 - count) when the real tokens are not one contiguous span; the plan kernel repairs the sign
// and raises the header flag.
__global__ __launch_bounds__(256) void br_block_table_kernel(const uint8_t* __restrict__ valid, int BM, int H,
                                                             int* __restrict__ start, int* __restrict__ len) {
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (wave >= BM) return;
    const uint8_t* row = valid + (size_t)wave * H;
    int cnt = 0, first = H, last = -1;
    for (int j = lane; j < H; j += 64) {
        if (row[j]) {
            ++cnt;
            first = j < first ? j : first;
            last = j > last ? j : last;
        }
    }
    for (int o = 32; o > 0; o >>= 1) {
        cnt += __shfl_xor(cnt, o);
        int f = __shfl_xor(first, o);
        int l = __shfl_xor(last, o);
        first = f < first ? f : first;
        last = l > last ? l : last;
    }
    if (lane == 0) {
        bool contiguous = cnt == 0 || (last - first + 1 == cnt);
        start[wave] = cnt == 0 ? 0 : first;
        len[wave] = contiguous ? cnt : -1 - cnt;
    }
}

__device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Exclusive scan of one int per thread over the workgroup (kPlanThreads entries): wave-level scan with
// lane shuffles, then the 16 wave totals.  Returns the exclusive prefix, leaves the total in *total.
__device__ int block_exclusive_scan(int x, int* sh, int* total) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int incl = x;
    for (int o = 1; o < 64; o <<= 1) {
        int y = __shfl_up(incl, o);
        if (lane >= o) incl += y;
    }
    if (lane == 63) sh[wave] = incl;
    __syncthreads();
    int base = 0, tot = 0;
    for (int w = 0; w < kPlanThreads / 64; ++w) {
        int v = sh[w];
        if (w < wave) base += v;
        tot += v;
    }
    __syncthreads();
    *total = tot;
    return base + incl - x;
}

// Split count for query tile tt of the query block: enough splits that each covers about
// BR_MIN_CHUNK key tiles, limited so that all tiles of the block fit the sequence's slot budget.
__device__ inline int splits_for(int ntiles, int ns_cap) {
    int ns = ceil_div(ntiles, BR_MIN_CHUNK);
    ns = ns < 1 ? 1 : ns;
    return ns > ns_cap ? ns_cap : ns;
}

__global__ __launch_bounds__(kPlanThreads) void br_plan_kernel(int* __restrict__ plan, int B, int M, int H, int T, int packed) {
    __shared__ int sh[kPlanThreads / 64];
    __shared__ int s_bad;
    const int tid = threadIdx.x;
    int* hdr = plan;
    int* start = plan + br_plan_off_start();
    int* len = plan + br_plan_off_len(B, M);
    int* tok = plan + br_plan_off_tok(B, M);
    int* prev_tiles = plan + br_plan_off_prev(B, M);
    int* tbase = plan + br_plan_off_tbase(B, M);
    int2* tiles = reinterpret_cast<int2*>(plan + br_plan_off_tiles(B, M));
    const int tps = br_plan_tps(M, H);
    const int max_items = br_plan_max_items(B, M, H, T);
    BrItem* items = reinterpret_cast<BrItem*>(plan + br_plan_off_items(B, M, H, T));
    BrComb* comb = reinterpret_cast<BrComb*>(plan + br_plan_off_comb(B, M, H, T));
    int* fused = plan + br_plan_off_fused(B, M, H, T);

    if (tid < BR_PLAN_HDR) hdr[tid] = 0;
    if (tid == 0) s_bad = 0;
    __syncthreads();
    const int BM = B * M;
    for (int p = tid; p < BM; p += kPlanThreads) {
        int l = len[p];
        if (l < 0) {
            len[p] = -1 - l;
            s_bad = 1;
        }
    }
    __syncthreads();
    // where each block's first real token sits on the token axis
    if (!packed) {
        for (int p = tid; p < BM; p += kPlanThreads) tok[p] = (p % M) * H + start[p];
    } else {
        int base = 0;
        for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
            const int p = p0 + tid;
            int tot;
            const int ex = block_exclusive_scan(p < BM ? len[p] : 0, sh, &tot);
            if (p < BM) tok[p] = base + ex;
            base += tot;
        }
    }
    __syncthreads();
    for (int b = tid; b < B; b += kPlanThreads) {
        int s = 0;
        for (int m = 0; m < M - 1; ++m) {
            tbase[b * M + m] = s;
            s += ceil_div(len[b * M + m], BR_BN);
        }
        prev_tiles[b] = s;
    }
    __syncthreads();
    // tile descriptors of blocks 0..M-2, one thread per block
    for (int p = tid; p < BM; p += kPlanThreads) {
        const int b = p / M, m = p - b * M;
        if (m == M - 1) continue;
        const int L = len[p];
        for (int kt = 0; kt * BR_BN < L; ++kt)
            tiles[(size_t)b * tps + tbase[p] + kt] = make_int2(tok[p] + kt * BR_BN, L - kt * BR_BN < BR_BN ? L - kt * BR_BN : BR_BN);
    }
    __syncthreads();

    // Work distribution, in two views.
    // View 0 (every kernel but the bf16 one): the query-block items (long walks, split) form the global
    // queue, drained first.  All other items keep their natural order (sequence, block, query tile) and
    // that list is cut into eight contiguous runs of equal estimated work, one per XCD queue: an XCD
    // then works on a few adjacent blocks at a time (their K/V stay in its L2), and the runs end
    // together, so that no workgroup has to go looking for work in other queues at the end of the
    // kernel (polling the ticket counters there slows the memory accesses of every workgroup still
    // working).  Estimated work of an item: its key tiles plus a constant for set-up and epilogue.
    // View 1 (bf16): the same for the sequences that are not "fused".  A sequence is fused when all the
    // keys any of its blocks 0..M-2 sees (the prefix's tiles and its own) fit into BR_RES_TILES tiles
    // and its query block is at most two query tiles long.  Each block of a fused sequence is one
    // resident item: the resident kernel keeps the block's keys in LDS for the block's own rows and for
    // the query block's rows, whose partial result against this block goes into partial slot
    // (query tile * M + block); the combine entries of a fused sequence merge those M slots.
    constexpr int kItemOverhead = 2;
    auto item_weight = [&](int nprev_t, int tt, int L) {
        int e = (tt + 1) * T < L ? (tt + 1) * T : L;
        return nprev_t + ceil_div(e, BR_BN) + kItemOverhead;
    };
    for (int b = tid; b < B; b += kPlanThreads) {
        const int n0 = M > 1 ? ceil_div(len[b * M], BR_BN) : 0;
        const int Lq = len[b * M + M - 1];
        bool ok = M > 1 && Lq > 0 && ceil_div(Lq, T) <= 2 && ceil_div(Lq, BR_BN) <= BR_RES_TILES && n0 <= BR_RES_TILES;
        for (int m = 1; ok && m < M - 1; ++m) ok = n0 + ceil_div(len[b * M + m], BR_BN) <= BR_RES_TILES;
        fused[b] = ok ? 1 : 0;
    }
    __shared__ int s_qfirst[2][8];
    if (tid < 16) s_qfirst[tid >> 3][tid & 7] = 0x7fffffff;
    __syncthreads();

    struct Counts {
        int glob[2], x[2], w[2], comb[2], res;
    };
    // what one (sequence, block) pair contributes; pairs are visited sequence by sequence, the query block first
    auto count_pair = [&](int p, Counts& c, int& b, int& m, int& L, int& nq, int& ns_cap, int& pt, int& npt, bool& is_last, bool& fz) {
        c = Counts{{0, 0}, {0, 0}, {0, 0}, {0, 0}, 0};
        b = p / M;
        const int jj = p - b * M;
        m = jj == 0 ? M - 1 : jj - 1;
        is_last = jj == 0;
        fz = fused[b] != 0;
        L = len[b * M + m];
        nq = ceil_div(L, T);
        if (is_last) {
            pt = M > 1 ? prev_tiles[b] : 0;
            ns_cap = nq > 0 ? BR_SLOTS_PER_SEQ / nq : 1;
            ns_cap = ns_cap < 1 ? 1 : ns_cap;
            for (int tt = 0; tt < nq; ++tt) {
                int e = (tt + 1) * T < L ? (tt + 1) * T : L;
                int ns = splits_for(pt + ceil_div(e, BR_BN), ns_cap);
                c.glob[0] += ns;
                c.comb[0] += ns > 1;
            }
        } else {
            c.x[0] = nq;
            npt = br_prev_blocks(m, M) > 0 ? ceil_div(len[b * M], BR_BN) : 0;
            for (int tt = 0; tt < nq; ++tt) c.w[0] += item_weight(npt, tt, L);
        }
        if (fz) {
            c.res = 1;
            c.comb[1] = is_last ? nq : 0;
        } else {
            c.glob[1] = c.glob[0]; c.x[1] = c.x[0]; c.w[1] = c.w[0]; c.comb[1] = c.comb[0];
        }
    };

    // Pass 1: totals.
    int n_glob_total[2] = {0, 0}, n_x_total[2] = {0, 0}, n_comb0_total = 0;
    long long w_total[2] = {0, 0};
    for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
        const int p = p0 + tid;
        Counts c = Counts{{0, 0}, {0, 0}, {0, 0}, {0, 0}, 0};
        if (p < BM) {
            int b, m, L, nq, ns_cap, pt, npt;
            bool is_last, fz;
            count_pair(p, c, b, m, L, nq, ns_cap, pt, npt, is_last, fz);
        }
        int tot;
        for (int v = 0; v < 2; ++v) {
            block_exclusive_scan(c.glob[v], sh, &tot);
            n_glob_total[v] += tot;
            block_exclusive_scan(c.x[v], sh, &tot);
            n_x_total[v] += tot;
            block_exclusive_scan(c.w[v], sh, &tot);
            w_total[v] += tot;
        }
        block_exclusive_scan(c.comb[0], sh, &tot);
        n_comb0_total += tot;
    }

    // Pass 2: the items array is [global 0][XCD 0][global 1][XCD 1][resident], the combine array [view 0][view 1].
    const int goff[2] = {0, n_glob_total[0] + n_x_total[0]};
    const int xoff[2] = {n_glob_total[0], goff[1] + n_glob_total[1]};
    const int res_off = xoff[1] + n_x_total[1];
    const int coff[2] = {0, n_comb0_total};
    int base_glob[2] = {goff[0], goff[1]}, base_x[2] = {xoff[0], xoff[1]}, base_comb[2] = {coff[0], coff[1]}, base_res = res_off;
    long long base_w[2] = {0, 0};
    for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
        const int p = p0 + tid;
        Counts c = Counts{{0, 0}, {0, 0}, {0, 0}, {0, 0}, 0};
        int b = 0, m = 0, L = 0, nq = 0, ns_cap = 1, pt = 0, npt = 0;
        bool is_last = false, fz = false;
        if (p < BM) count_pair(p, c, b, m, L, nq, ns_cap, pt, npt, is_last, fz);
        int off_g[2], off_x[2], off_c[2];
        long long off_w[2];
        int tot;
        for (int v = 0; v < 2; ++v) {
            off_g[v] = base_glob[v] + block_exclusive_scan(c.glob[v], sh, &tot);
            base_glob[v] += tot;
            off_x[v] = base_x[v] + block_exclusive_scan(c.x[v], sh, &tot);
            base_x[v] += tot;
            off_c[v] = base_comb[v] + block_exclusive_scan(c.comb[v], sh, &tot);
            base_comb[v] += tot;
            off_w[v] = base_w[v] + block_exclusive_scan(c.w[v], sh, &tot);
            base_w[v] += tot;
        }
        const int off_res = base_res + block_exclusive_scan(c.res, sh, &tot);
        base_res += tot;
        if (p < BM) {
            const int pe = br_prev_blocks(m, M);
            BrItem it;
            it.b = b; it.m = m; it.pe = pe;
            it.len_m = L; it.start_m = start[b * M + m]; it.len0 = len[b * M]; it.start0 = start[b * M];
            it.tok_m = tok[b * M + m]; it.tok0 = tok[b * M];
            it.pad[0] = it.pad[1] = 0;
            if (!is_last) {
                it.nprev = npt;
                for (int tt = 0; tt < nq; ++tt) {
                    it.t0 = tt * T; it.f_lo = 0;
                    it.ntiles = 0x7fffffff; it.slot = -1;
                    for (int v = 0; v < 2; ++v) {
                        if (c.x[v] == 0) continue;
                        items[off_x[v] + tt] = it;
                        int q = w_total[v] > 0 ? (int)(off_w[v] * 8 / w_total[v]) : 0;
                        q = q > 7 ? 7 : q;
                        atomicMin(&s_qfirst[v][q], off_x[v] + tt);
                        off_w[v] += item_weight(npt, tt, L);
                    }
                }
            } else {
                it.nprev = pt;
                int slot = 0;
                int off_i[2] = {off_g[0], off_g[1]};
                for (int tt = 0; tt < nq; ++tt) {
                    int e = (tt + 1) * T < L ? (tt + 1) * T : L;
                    int nself = ceil_div(e, BR_BN);
                    int nt = pt + nself;
                    int ns = splits_for(nt, ns_cap);
                    if (ns > 1) {
                        BrComb cb;
                        cb.b = b; cb.t0 = tt * T; cb.slot0 = slot; cb.nsplit = ns;
                        comb[off_c[0]++] = cb;
                        if (!fz) comb[off_c[1]++] = cb;
                    }
                    for (int s = 0; s < ns; ++s) {
                        int lo = (int)((long long)s * nt / ns);
                        int hi = (int)((long long)(s + 1) * nt / ns);
                        it.t0 = tt * T; it.f_lo = lo;
                        it.ntiles = ns > 1 ? hi - lo : 0x7fffffff; it.slot = ns > 1 ? slot + s : -1;
                        items[off_i[0]++] = it;
                        if (!fz) items[off_i[1]++] = it;
                    }
                    if (ns > 1) slot += ns;
                    if (fz) {
                        BrComb cb;
                        cb.b = b; cb.t0 = tt * T; cb.slot0 = tt * M; cb.nsplit = M;
                        comb[off_c[1]++] = cb;
                    }
                }
            }
            if (fz) {
                // resident item: the fields a resident block does not need carry the query block's span and
                // the block's place in the sequence's tile table
                const int pq = b * M + M - 1;
                it.nprev = is_last ? 0 : npt;
                it.t0 = len[pq];                  // real tokens of the query block
                it.f_lo = tok[pq];                // its first token on the token axis
                it.slot = start[pq];              // ... and inside its H slots
                it.ntiles = is_last ? 0 : tbase[b * M + m];
                it.pe = ceil_div(len[pq], T);     // query tiles
                items[off_res] = it;
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        for (int v = 0; v < 2; ++v) {
            // a queue that received no item starts where the next one starts
            const int end = xoff[v] + n_x_total[v];
            int nxt = end;
            const int qc = v == 0 ? BR_PH_QCOUNT : BR_PH_QCOUNT2, qo = v == 0 ? BR_PH_QOFF : BR_PH_QOFF2;
            for (int g = 7; g >= 0; --g) {
                int f = s_qfirst[v][g];
                if (f == 0x7fffffff) f = nxt;
                hdr[qo + g] = f;
                hdr[qc + g] = nxt - f;
                nxt = f;
            }
            hdr[qo + BR_GLOBAL_QUEUE] = goff[v];
            hdr[qc + BR_GLOBAL_QUEUE] = n_glob_total[v];
        }
        hdr[BR_PH_NITEMS] = base_res;
        hdr[BR_PH_NCOMB] = n_comb0_total;
        hdr[BR_PH_NCOMB2] = base_comb[1] - coff[1];
        hdr[BR_PH_COMB_OFF2] = coff[1];
        hdr[BR_PH_RES_OFF] = res_off;
        hdr[BR_PH_NRES] = base_res - res_off;
        hdr[BR_PH_SLOTS2] = br_slots_view1(M);
        hdr[BR_PH_PACKED] = packed;
        hdr[BR_PH_NONCONTIG] = s_bad;
        hdr[BR_PH_MAX_ITEMS] = max_items;
        hdr[BR_PH_MAX_COMB] = br_plan_max_comb(B);
        hdr[BR_PH_T] = T;
    }
}

// Block table straight from per-block lengths (left- or right-aligned spans): the packed-layout
// entry, where the caller already knows the lengths and there is no (B, M, H) mask to scan.
__global__ void br_block_table_from_len_kernel(const int* __restrict__ lens, int BM, int H, int left_padded,
                                               int* __restrict__ start, int* __restrict__ len) {
    int p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= BM) return;
    int l = lens[p];
    l = l < 0 ? 0 : (l > H ? H : l);
    len[p] = l;
    start[p] = left_padded ? H - l : 0;
}

}  // namespace

void br_launch_plan(const uint8_t* valid, const int* lens, int left_padded, int packed, int B, int M, int H, int T, int* plan,
                    hipStream_t stream) {
    int* start = plan + br_plan_off_start();
    int* len = plan + br_plan_off_len(B, M);
    const int BM = B * M;
    if (valid) {
        int waves_per_wg = 4;
        hipLaunchKernelGGL(br_block_table_kernel, dim3((BM + waves_per_wg - 1) / waves_per_wg), dim3(256), 0, stream, valid,
                           BM, H, start, len);
    } else {
        hipLaunchKernelGGL(br_block_table_from_len_kernel, dim3((BM + 255) / 256), dim3(256), 0, stream, lens, BM, H,
                           left_padded, start, len);
    }
    hipLaunchKernelGGL(br_plan_kernel, dim3(1), dim3(kPlanThreads), 0, stream, plan, B, M, H, T, packed);
}
