// Request plan: turns the (B, M, H) block mask into the block table (start, len per block) and the
// work-item list the persistent prefill kernel consumes.  Built on the device with no host
// synchronisation, once per forward pass (the block structure is the same for every layer).
//
// The additive 5-D mask of the reference (blockrank_std_attention.py:293-309) carries exactly this
// information: which keys of each block are real.  Everything else (causality inside a block, which
// earlier blocks a block may see) follows from the block index, so the kernels never read a mask.
#include "br_common.h"

namespace {

constexpr int kPlanThreads = 512;

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

// The same for N values per thread at once (one pair of barriers for all of them): x[i] becomes the exclusive
// prefix of x[i] over the workgroup, tot[i] the total.
template <int N>
__device__ void block_exclusive_scan_n(int (&x)[N], int (&tot)[N], int* shn /* N * kPlanThreads / 64 ints */) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int incl[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        incl[i] = x[i];
        for (int o = 1; o < 64; o <<= 1) {
            int y = __shfl_up(incl[i], o);
            if (lane >= o) incl[i] += y;
        }
        if (lane == 63) shn[i * (kPlanThreads / 64) + wave] = incl[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        int base = 0, t = 0;
        for (int w = 0; w < kPlanThreads / 64; ++w) {
            const int v = shn[i * (kPlanThreads / 64) + w];
            if (w < wave) base += v;
            t += v;
        }
        tot[i] = t;
        x[i] = base + incl[i] - x[i];
    }
    __syncthreads();
}

// Split count for a query tile of the query block: enough splits that each covers about ``chunk`` key tiles.
__device__ inline int splits_for(int ntiles, int chunk) {
    const int ns = ceil_div(ntiles, chunk);
    return ns < 1 ? 1 : ns;
}

// par: workgroups of the prefill grid per head group, i.e. how many of a plan's items run side by side.
// pool: split-KV partial slots the caller's workspace has room for (br_split_pool).
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
    // All items but the query blocks' keep their natural order (sequence, block, query tile) and that list is cut
    // into eight contiguous runs of equal estimated work, one per XCD queue: an XCD then works on a few adjacent
    // blocks at a time (their K/V stay in its L2), and the runs end together, so that no workgroup has to go looking
    // for work in other queues at the end of the kernel (polling the ticket counters there slows the memory accesses
    // of every workgroup still working).  Estimated work of an item: its key tiles plus a constant for set-up and
    // epilogue.  A query block reads the K/V of every earlier block of its sequence: its key walk is cut where those
    // blocks pass from one XCD's run to the next and each stretch is handed to that XCD (at the front of its queue:
    // long items first), so that the walk finds the tiles in the L2 that the blocks' own items fill anyway instead of
    // pulling all K/V of the sequence into a second L2.
    constexpr int kItemOverhead = 2;
    auto item_weight = [&](int nprev_t, int tt, int L) {
        int e = (tt + 1) * T < L ? (tt + 1) * T : L;
        return nprev_t + ceil_div(e, BR_BN) + kItemOverhead;
    };
    int* bq = plan + br_plan_off_bq(B, M);
    __shared__ int s_qfirst[8];
    __shared__ int s_base[BR_NQUEUES], s_nsplit[BR_NQUEUES];
    if (tid < 8) s_qfirst[tid] = 0x7fffffff;
    __syncthreads();

    // Ordinary (not query-block) items of the pair p = (b, m): how many, their weight, the prefix tiles they walk.
    auto ordinary = [&](int p, int& nq, int& npt, int& L) -> int {
        nq = 0; npt = 0; L = 0;
        if (p >= BM) return 0;
        const int b = p / M, m = p - b * M;
        if (m == M - 1) return 0;
        L = len[p];
        nq = ceil_div(L, T);
        npt = br_prev_blocks(m, M) > 0 ? ceil_div(len[b * M], BR_BN) : 0;
        int w = 0;
        for (int tt = 0; tt < nq; ++tt) w += item_weight(npt, tt, L);
        return w;
    };

    // Totals: all items' weight (with the query blocks'), the ordinary items' weight and number.
    long long w_all = 0, w_ord = 0;
    int n_ord = 0;
    for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
        const int p = p0 + tid;
        int nq, npt, L;
        int w = ordinary(p, nq, npt, L), wq = 0;
        if (p < BM && p % M == M - 1) {
            const int b = p / M, Lq = len[p], pt = M > 1 ? prev_tiles[b] : 0;
            for (int tt = 0; tt * T < Lq; ++tt) wq += item_weight(pt, tt, Lq);
        }
        int tot;
        block_exclusive_scan(w + wq, sh, &tot);
        w_all += tot;
        block_exclusive_scan(w, sh, &tot);
        w_ord += tot;
        block_exclusive_scan(nq, sh, &tot);
        n_ord += tot;
    }
    const long long w_total = w_ord;

    // Queue of every ordinary item (by the weight before it), first item of every queue, queue of every block (that of
    // its first item).
    {
        int base_x = 0;
        long long base_w = 0;
        for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
            const int p = p0 + tid;
            int nq, npt, L;
            const int w = ordinary(p, nq, npt, L);
            int tot;
            const int off_x = base_x + block_exclusive_scan(nq, sh, &tot);
            base_x += tot;
            long long off_w = base_w + block_exclusive_scan(w, sh, &tot);
            base_w += tot;
            if (p < BM) bq[p] = -1;
            for (int k = 0; k < nq; ++k) {
                int q = w_total > 0 ? (int)(off_w * 8 / w_total) : 0;
                q = q > 7 ? 7 : q;
                if (k == 0) bq[p] = q;
                atomicMin(&s_qfirst[q], off_x + k);
                off_w += item_weight(npt, nq - 1 - k, L);
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        // a queue that received no item starts where the next one starts
        int nxt = n_ord;
        for (int g = 7; g >= 0; --g) {
            if (s_qfirst[g] == 0x7fffffff) s_qfirst[g] = nxt;
            nxt = s_qfirst[g];
        }
    }
    __syncthreads();

    // What the walks below read about every block - its key tiles and its queue - staged in LDS once: a walk is a
    // serial loop over a sequence's blocks run by a single thread, and from global memory every step of it is a
    // round trip of its own.
    constexpr int kStage = 8192;
    __shared__ unsigned short s_nt[kStage];
    __shared__ signed char s_bq[kStage];
    const bool staged = BM <= kStage;
    if (staged) {
        for (int p = tid; p < BM; p += kPlanThreads) {
            const int nt = ceil_div(len[p], BR_BN);
            s_nt[p] = (unsigned short)(nt > 0xffff ? 0xffff : nt);
            s_bq[p] = (signed char)bq[p];
        }
    }
    __syncthreads();
    auto blk_tiles = [&](int p) -> int { return staged ? (int)s_nt[p] : ceil_div(len[p], BR_BN); };
    auto blk_queue = [&](int p) -> int { return staged ? (int)s_bq[p] : bq[p]; };

    // The stretches of a sequence's earlier blocks that one XCD's queue owns: first tile, tiles, queue.  The queues
    // follow the blocks' order, so there are at most eight; a stretch shorter than min_seg tiles stays with the next
    // one.  (Small fixed arrays indexed through unrolled loops: they live in registers - a dynamically indexed local
    // array is scratch memory, a round trip of microseconds per access for the single thread that walks a sequence.)
    struct Segs {
        int n;
        int lo[8], cnt[8], q[8];
    };
    auto build_segs = [&](int b, int min_seg, Segs& S) {
        S.n = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) S.lo[i] = S.cnt[i] = S.q[i] = 0;
        int seg_lo = 0, seg_n = 0, seg_q = -1;
        auto push = [&]() {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i == S.n) {
                    S.lo[i] = seg_lo; S.cnt[i] = seg_n; S.q[i] = seg_q;
                }
            ++S.n;
        };
        for (int m = 0; m < M - 1; ++m) {
            const int nt = blk_tiles(b * M + m);
            if (nt == 0) continue;
            const int q = blk_queue(b * M + m);
            if (seg_q >= 0 && q != seg_q && seg_n >= min_seg && S.n < 7) {
                push();
                seg_lo += seg_n;
                seg_n = 0;
                seg_q = q;
            }
            if (seg_q < 0) seg_q = q;
            seg_n += nt;
        }
        if (seg_q >= 0) push();
    };
    // The pieces of the key walk of query tile tt of sequence b's query block, in walk order: fn(index, first tile,
    // tiles, queue).  Every stretch is cut into pieces of at most `chunk` tiles; the query block's own tiles go with the
    // last stretch (a sequence without earlier keys has them alone, in the global queue).  Returns the number of pieces.
    auto walk_pieces = [&](int b, int tt, int chunk, const Segs& S, auto&& fn) -> int {
        const int L = len[b * M + M - 1];
        const int e = (tt + 1) * T < L ? (tt + 1) * T : L;
        const int nself = ceil_div(e, BR_BN);
        int count = 0;
        auto close = [&](int lo, int n, int q) {
            int parts = ceil_div(n, chunk);
            parts = parts < 1 ? 1 : parts;
            for (int s = 0; s < parts; ++s) {
                const int a = lo + (int)((long long)s * n / parts), z = lo + (int)((long long)(s + 1) * n / parts);
                fn(count, a, z - a, q);
                ++count;
            }
        };
        if (S.n == 0) {
            close(0, nself, BR_GLOBAL_QUEUE);
            return count;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i < S.n) close(S.lo[i], S.cnt[i] + (i == S.n - 1 ? nself : 0), S.q[i]);
        return count;
    };
    auto no_op = [](int, int, int, int) {};
    // a[q] += 1 for a register-resident array of the nine queues; returns the value before
    auto bump = [](int (&a)[BR_NQUEUES], int q) -> int {
        int r = 0;
#pragma unroll
        for (int i = 0; i < BR_NQUEUES; ++i)
            if (i == q) {
                r = a[i];
                a[i] = r + 1;
            }
        return r;
    };

    // Length of a piece.  The walks are cut so that the batch has enough items to fill the grid, and no further: every
    // piece costs a set-up, an epilogue and a set of partials to write and merge, while a long piece still ends with the
    // others because the pieces are handed out first.  So: the estimated work per workgroup (all items' key tiles plus
    // their constant, over the workgroups that run side by side) less one ordinary item - the workgroup that takes a
    // piece still has to fit one of those before the kernel ends, which is what decides at a batch of one - and at
    // least BR_MIN_CHUNK; and long enough that the batch's pieces fit the pool of partial slots: lengthen until they
    // do, and where longer pieces no longer help (what remains are the cuts between XCDs) join short stretches to
    // their neighbours; with both beyond every walk's length nothing is split at all, so this ends.
    int chunk = (int)(w_all / (par > 0 ? par : 1)) - (n_ord > 0 ? (int)(w_ord / n_ord) : 0);
    chunk = chunk < BR_MIN_CHUNK ? BR_MIN_CHUNK : chunk;
    int min_seg = BR_MIN_CHUNK, need_before = 0x7fffffff;
    // Thread tid walks the sequences tid, tid + kPlanThreads, ...  With one sequence per thread (every batch but
    // the largest) its stretch list is built once and kept in registers; otherwise it is rebuilt at every visit.
    Segs segs;
    segs.n = 0;
    const bool one_each = B <= kPlanThreads;
    if (one_each && tid < B) build_segs(tid, min_seg, segs);
    auto for_my_sequences = [&](auto&& fn) {
        for (int b = tid; b < B; b += kPlanThreads) {
            if (!one_each) build_segs(b, min_seg, segs);
            fn(b, len[b * M + M - 1]);
        }
    };
    for (;;) {
        int mine = 0;
        for_my_sequences([&](int b, int Lq) {
            for (int tt = 0; tt * T < Lq; ++tt) {
                const int ns = walk_pieces(b, tt, chunk, segs, no_op);
                mine += ns > 1 ? ns : 0;
            }
        });
        int need;
        block_exclusive_scan(mine, sh, &need);
        if (need <= pool) break;
        if (need >= need_before) {
            min_seg *= 2;
            if (one_each && tid < B) build_segs(tid, min_seg, segs);
        }
        need_before = need;
        if (chunk < (1 << 24)) chunk += (chunk + 1) / 2;
    }

    // Layout of the items array: [global queue][queue 0: its pieces, its ordinary items][queue 1: ...] ...
    // Every thread counts the pieces of its sequences' query blocks per queue; scans give it its offsets.
    int my_cnt[BR_NQUEUES], my_off[BR_NQUEUES], my_comb = 0, my_slots = 0;
#pragma unroll
    for (int q = 0; q < BR_NQUEUES; ++q) my_cnt[q] = 0;
    for_my_sequences([&](int b, int Lq) {
        for (int tt = 0; tt * T < Lq; ++tt) {
            const int ns = walk_pieces(b, tt, chunk, segs, [&](int, int, int, int q) { bump(my_cnt, q); });
            my_comb += ns > 1;
            my_slots += ns > 1 ? ns : 0;
        }
    });
    // (all eleven counts through one scan)
    __shared__ int s_scan[(BR_NQUEUES + 2) * (kPlanThreads / 64)];
    int sc[BR_NQUEUES + 2], sc_tot[BR_NQUEUES + 2];
#pragma unroll
    for (int q = 0; q < BR_NQUEUES; ++q) sc[q] = my_cnt[q];
    sc[BR_NQUEUES] = my_comb;
    sc[BR_NQUEUES + 1] = my_slots;
    block_exclusive_scan_n<BR_NQUEUES + 2>(sc, sc_tot, s_scan);
#pragma unroll
    for (int q = 0; q < BR_NQUEUES; ++q) {
        my_off[q] = sc[q];
        if (tid == 0) s_nsplit[q] = sc_tot[q];
    }
    const int off_comb = sc[BR_NQUEUES], off_slot = sc[BR_NQUEUES + 1];
    const int n_comb_total = sc_tot[BR_NQUEUES], n_slot_total = sc_tot[BR_NQUEUES + 1];
    __syncthreads();
    if (tid == 0) {
        int nxt = s_nsplit[BR_GLOBAL_QUEUE];
        for (int g = 0; g < 8; ++g) {
            s_base[g] = nxt;
            const int ord = (g < 7 ? s_qfirst[g + 1] : n_ord) - s_qfirst[g];
            hdr[BR_PH_QOFF + g] = nxt;
            hdr[BR_PH_QCOUNT + g] = s_nsplit[g] + ord;
            nxt += s_nsplit[g] + ord;
        }
        s_base[BR_GLOBAL_QUEUE] = 0;
        hdr[BR_PH_QOFF + BR_GLOBAL_QUEUE] = 0;
        hdr[BR_PH_QCOUNT + BR_GLOBAL_QUEUE] = s_nsplit[BR_GLOBAL_QUEUE];
        hdr[BR_PH_NITEMS] = nxt;
        hdr[BR_PH_NCOMB] = n_comb_total;
        hdr[BR_PH_PACKED] = packed;
        hdr[BR_PH_NONCONTIG] = s_bad;
        hdr[BR_PH_MAX_ITEMS] = max_items;
        hdr[BR_PH_MAX_COMB] = br_plan_max_comb(B);
        hdr[BR_PH_T] = T;
        hdr[BR_PH_POOL] = pool;
        hdr[BR_PH_NSLOTS] = n_slot_total;
    }
    __syncthreads();

    // Ordinary items: queue g's start at s_base[g] + its pieces, in their natural order.
    {
        int base_x = 0;
        long long base_w = 0;
        for (int p0 = 0; p0 < BM; p0 += kPlanThreads) {
            const int p = p0 + tid;
            int nq, npt, L;
            const int w = ordinary(p, nq, npt, L);
            int tot;
            const int off_x = base_x + block_exclusive_scan(nq, sh, &tot);
            base_x += tot;
            long long off_w = base_w + block_exclusive_scan(w, sh, &tot);
            base_w += tot;
            if (nq > 0) {
                const int b = p / M, m = p - b * M;
                BrItem it;
                it.b = b; it.m = m; it.pe = br_prev_blocks(m, M);
                it.len_m = L; it.start_m = start[p]; it.len0 = len[b * M]; it.start0 = start[b * M];
                it.tok_m = tok[p]; it.tok0 = tok[b * M];
                it.pad[0] = it.pad[1] = 0;
                it.nprev = npt;
                it.f_lo = 0; it.ntiles = 0x7fffffff; it.slot = -1;
                // a block's query tiles are handed out from the last (the longest walk) to the first: what a queue
                // ends on are short items
                for (int k = 0; k < nq; ++k) {
                    const int tt = nq - 1 - k;
                    int q = w_total > 0 ? (int)(off_w * 8 / w_total) : 0;
                    q = q > 7 ? 7 : q;
                    it.t0 = tt * T;
                    items[s_base[q] + s_nsplit[q] + (off_x + k - s_qfirst[q])] = it;
                    off_w += item_weight(npt, tt, L);
                }
            }
        }
    }
    // The query blocks' pieces (the thread of every sequence, in the order and at the offsets of the counting pass above).
    int pos[BR_NQUEUES];
#pragma unroll
    for (int q = 0; q < BR_NQUEUES; ++q) pos[q] = s_base[q] + my_off[q];
    int slot = off_slot, ci = off_comb;
    for_my_sequences([&](int b, int L) {
        const int pq = b * M + M - 1;
        BrItem it;
        it.b = b; it.m = M - 1; it.pe = br_prev_blocks(M - 1, M);
        it.len_m = L; it.start_m = start[pq]; it.len0 = len[b * M]; it.start0 = start[b * M];
        it.tok_m = tok[pq]; it.tok0 = tok[b * M];
        it.pad[0] = it.pad[1] = 0;
        it.nprev = M > 1 ? prev_tiles[b] : 0;
        for (int tt = 0; tt * T < L; ++tt) {
            const int ns = walk_pieces(b, tt, chunk, segs, no_op);
            if (ns > 1) {
                BrComb cb;
                cb.b = b; cb.t0 = tt * T; cb.slot0 = slot; cb.nsplit = ns;
                comb[ci++] = cb;
            }
            it.t0 = tt * T;
            walk_pieces(b, tt, chunk, segs, [&](int i, int lo, int n, int q) {
                it.f_lo = lo;
                it.ntiles = ns > 1 ? n : 0x7fffffff;
                it.slot = ns > 1 ? slot + i : -1;
                items[bump(pos, q)] = it;
            });
            if (ns > 1) slot += ns;
        }
    });
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

// Ticket counters and the count of workgroups that have left back to zero (what the last workgroup of a launch that
// ran to its end does itself).
__global__ void br_plan_rearm_kernel(int* __restrict__ plan) {
    const int i = threadIdx.x;
    if (i < BR_NQUEUES) plan[BR_PH_QTICKET + i] = 0;
    if (i == BR_NQUEUES) plan[BR_PH_DONE] = 0;
}

}  // namespace

void br_launch_plan_rearm(int* plan, hipStream_t stream) {
    hipLaunchKernelGGL(br_plan_rearm_kernel, dim3(1), dim3(64), 0, stream, plan);
}

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
