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

// Split count for a query tile of the query block: enough splits that each covers about ``chunk`` key tiles.
__device__ inline int splits_for(int ntiles, int chunk) {
    const int ns = ceil_div(ntiles, chunk);
    return ns < 1 ? 1 : ns;
}

// par: workgroups of the prefill grid per head group, i.e. how many of a plan's items run side by side.
// pool: split-KV partial slots the caller's workspace has room for (br_split_pool(par)).
__global__ __launch_bounds__(kPlanThreads) void br_plan_kernel(int* __restrict__ plan, int B, int M, int H, int T, int packed, int par, int pool) {
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

    // Work distribution.
    // The query-block items (long walks, split) form the global queue, drained first.  All other items keep
    // their natural order (sequence, block, query tile) and that list is cut into eight contiguous runs of
    // equal estimated work, one per XCD queue: an XCD then works on a few adjacent blocks at a time (their
    // K/V stay in its L2), and the runs end together, so that no workgroup has to go looking for work in other
    // queues at the end of the kernel (polling the ticket counters there slows the memory accesses of every
    // workgroup still working).  Estimated work of an item: its key tiles plus a constant for set-up and
    // epilogue.
    constexpr int kItemOverhead = 2;
    auto item_weight = [&](int nprev_t, int tt, int L) {
        int e = (tt + 1) * T < L ? (tt + 1) * T : L;
        return nprev_t + ceil_div(e, BR_BN) + kItemOverhead;
    };
    __shared__ int s_qfirst[8];
    if (tid < 8) s_qfirst[tid] = 0x7fffffff;
    __syncthreads();

    // Length of a split of the query block's key walk.  The walk is cut so that the batch has enough items to fill
    // the grid, and no further: every split costs a set-up, an epilogue and a set of partials to write and merge,
    // while a long split still ends with the others because the split items are handed out first.  So: the estimated
    // work per workgroup (all items' key tiles plus their constant, over the workgroups that run side by side) less
    // one ordinary item - the workgroup that takes a split still has to fit one of those before the kernel ends, which
    // is what decides at a batch of one - and at least BR_MIN_CHUNK.
    long long w_all = 0, w_ord = 0;
    int n_ord = 0;
    for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
        const int p = p0 + tid;
        int w = 0, nq = 0;
        bool last = false;
        if (p < BM) {
            const int b = p / M, m = p - b * M;
            const int L = len[p];
            nq = ceil_div(L, T);
            last = m == M - 1;
            const int np = last ? (M > 1 ? prev_tiles[b] : 0) : (br_prev_blocks(m, M) > 0 ? ceil_div(len[b * M], BR_BN) : 0);
            for (int tt = 0; tt < nq; ++tt) w += item_weight(np, tt, L);
        }
        int tot;
        block_exclusive_scan(w, sh, &tot);
        w_all += tot;
        block_exclusive_scan(last ? 0 : w, sh, &tot);
        w_ord += tot;
        block_exclusive_scan(last ? 0 : nq, sh, &tot);
        n_ord += tot;
    }
    int chunk = (int)(w_all / (par > 0 ? par : 1)) - (n_ord > 0 ? (int)(w_ord / n_ord) : 0);
    chunk = chunk < BR_MIN_CHUNK ? BR_MIN_CHUNK : chunk;
    // ... and long enough that the batch's splits fit the pool of partial slots: lengthen until they do (a chunk
    // longer than every walk means no split at all, so this ends)
    for (;;) {
        int need = 0;
        for (int b0 = 0; b0 < B; b0 += kPlanThreads) {
            const int b = b0 + tid;
            int mine = 0;
            if (b < B) {
                const int L = len[b * M + M - 1], pt = M > 1 ? prev_tiles[b] : 0;
                for (int tt = 0; tt * T < L; ++tt) {
                    const int e = (tt + 1) * T < L ? (tt + 1) * T : L;
                    const int ns = splits_for(pt + ceil_div(e, BR_BN), chunk);
                    mine += ns > 1 ? ns : 0;
                }
            }
            int tot;
            block_exclusive_scan(mine, sh, &tot);
            need += tot;
        }
        if (need <= pool) break;
        chunk += (chunk + 1) / 2;
    }

    struct Counts {
        int glob, x, w, comb, slots;
    };
    // what one (sequence, block) pair contributes; pairs are visited sequence by sequence, the query block first
    auto count_pair = [&](int p, Counts& c, int& b, int& m, int& L, int& nq, int& pt, int& npt, bool& is_last) {
        c = Counts{0, 0, 0, 0, 0};
        b = p / M;
        const int jj = p - b * M;
        m = jj == 0 ? M - 1 : jj - 1;
        is_last = jj == 0;
        L = len[b * M + m];
        nq = ceil_div(L, T);
        if (is_last) {
            pt = M > 1 ? prev_tiles[b] : 0;
            for (int tt = 0; tt < nq; ++tt) {
                int e = (tt + 1) * T < L ? (tt + 1) * T : L;
                int ns = splits_for(pt + ceil_div(e, BR_BN), chunk);
                c.glob += ns;
                c.comb += ns > 1;
                c.slots += ns > 1 ? ns : 0;
            }
        } else {
            c.x = nq;
            npt = br_prev_blocks(m, M) > 0 ? ceil_div(len[b * M], BR_BN) : 0;
            for (int tt = 0; tt < nq; ++tt) c.w += item_weight(npt, tt, L);
        }
    };

    // Pass 1: totals.
    int n_glob_total = 0, n_x_total = 0, n_comb_total = 0;
    long long w_total = 0;
    for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
        const int p = p0 + tid;
        Counts c = Counts{0, 0, 0, 0, 0};
        if (p < BM) {
            int b, m, L, nq, pt, npt;
            bool is_last;
            count_pair(p, c, b, m, L, nq, pt, npt, is_last);
        }
        int tot;
        block_exclusive_scan(c.glob, sh, &tot);
        n_glob_total += tot;
        block_exclusive_scan(c.x, sh, &tot);
        n_x_total += tot;
        block_exclusive_scan(c.w, sh, &tot);
        w_total += tot;
        block_exclusive_scan(c.comb, sh, &tot);
        n_comb_total += tot;
    }

    // Pass 2: the items array is [global queue][XCD queues].
    const int xoff = n_glob_total;
    int base_glob = 0, base_x = xoff, base_comb = 0, base_slot = 0;
    long long base_w = 0;
    for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
        const int p = p0 + tid;
        Counts c = Counts{0, 0, 0, 0, 0};
        int b = 0, m = 0, L = 0, nq = 0, pt = 0, npt = 0;
        bool is_last = false;
        if (p < BM) count_pair(p, c, b, m, L, nq, pt, npt, is_last);
        int tot;
        int off_g = base_glob + block_exclusive_scan(c.glob, sh, &tot);
        base_glob += tot;
        const int off_x = base_x + block_exclusive_scan(c.x, sh, &tot);
        base_x += tot;
        int off_c = base_comb + block_exclusive_scan(c.comb, sh, &tot);
        base_comb += tot;
        const int off_s = base_slot + block_exclusive_scan(c.slots, sh, &tot);
        base_slot += tot;
        long long off_w = base_w + block_exclusive_scan(c.w, sh, &tot);
        base_w += tot;
        if (p < BM) {
            const int pe = br_prev_blocks(m, M);
            BrItem it;
            it.b = b; it.m = m; it.pe = pe;
            it.len_m = L; it.start_m = start[b * M + m]; it.len0 = len[b * M]; it.start0 = start[b * M];
            it.tok_m = tok[b * M + m]; it.tok0 = tok[b * M];
            it.pad[0] = it.pad[1] = 0;
            if (!is_last) {
                it.nprev = npt;
                // a block's query tiles are handed out from the last (the longest walk) to the first: what a queue
                // ends on are short items
                for (int k = 0; k < nq; ++k) {
                    const int tt = nq - 1 - k;
                    it.t0 = tt * T; it.f_lo = 0;
                    it.ntiles = 0x7fffffff; it.slot = -1;
                    items[off_x + k] = it;
                    int q = w_total > 0 ? (int)(off_w * 8 / w_total) : 0;
                    q = q > 7 ? 7 : q;
                    atomicMin(&s_qfirst[q], off_x + k);
                    off_w += item_weight(npt, tt, L);
                }
            } else {
                it.nprev = pt;
                int slot = off_s;                            // slots of the batch's pool, in item order
                for (int tt = 0; tt < nq; ++tt) {
                    int e = (tt + 1) * T < L ? (tt + 1) * T : L;
                    int nself = ceil_div(e, BR_BN);
                    int nt = pt + nself;
                    int ns = splits_for(nt, chunk);
                    if (ns > 1) {
                        BrComb cb;
                        cb.b = b; cb.t0 = tt * T; cb.slot0 = slot; cb.nsplit = ns;
                        comb[off_c++] = cb;
                    }
                    for (int s = 0; s < ns; ++s) {
                        int lo = (int)((long long)s * nt / ns);
                        int hi = (int)((long long)(s + 1) * nt / ns);
                        it.t0 = tt * T; it.f_lo = lo;
                        it.ntiles = ns > 1 ? hi - lo : 0x7fffffff; it.slot = ns > 1 ? slot + s : -1;
                        items[off_g++] = it;
                    }
                    if (ns > 1) slot += ns;
                }
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        // a queue that received no item starts where the next one starts
        int nxt = xoff + n_x_total;
        for (int g = 7; g >= 0; --g) {
            int f = s_qfirst[g];
            if (f == 0x7fffffff) f = nxt;
            hdr[BR_PH_QOFF + g] = f;
            hdr[BR_PH_QCOUNT + g] = nxt - f;
            nxt = f;
        }
        hdr[BR_PH_QOFF + BR_GLOBAL_QUEUE] = 0;
        hdr[BR_PH_QCOUNT + BR_GLOBAL_QUEUE] = n_glob_total;
        hdr[BR_PH_NITEMS] = xoff + n_x_total;
        hdr[BR_PH_NCOMB] = n_comb_total;
        hdr[BR_PH_PACKED] = packed;
        hdr[BR_PH_NONCONTIG] = s_bad;
        hdr[BR_PH_MAX_ITEMS] = max_items;
        hdr[BR_PH_MAX_COMB] = br_plan_max_comb(B);
        hdr[BR_PH_T] = T;
        hdr[BR_PH_POOL] = pool;
        hdr[BR_PH_NSLOTS] = base_slot;
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

void br_launch_plan(const uint8_t* valid, const int* lens, int left_padded, int packed, int B, int M, int H, int T, int par, int pool,
                    int* plan, hipStream_t stream) {
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
    hipLaunchKernelGGL(br_plan_kernel, dim3(1), dim3(kPlanThreads), 0, stream, plan, B, M, H, T, packed, par, pool);
}
