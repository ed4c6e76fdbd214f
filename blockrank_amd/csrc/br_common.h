// Shared definitions for the BlockRank gfx950 kernels: the block table, the request plan (work
// items for the persistent prefill kernel), the key/value tile walk and the row mapping that the
// bf16 MFMA kernel, the fp32 kernel and the combine kernel all use.
//
// Vocabulary (the reference's): a sequence is M blocks of padded length H; block 0 is the
// instruction prefix, blocks 1..M-2 are documents, block M-1 is the query.  Each block holds one
// contiguous span of real tokens [start, start+len) inside its H slots (left padding puts it at the
// end).  Every position used by the kernels is "valid-relative": 0 is the block's first real token.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define BR_BN 64              // keys per key/value tile
#define BR_RB 32              // query rows per wave (one 32x32 MFMA row block)
// Split-KV partial slots of the query blocks' key walks: one pool for the whole batch, handed out by the plan in
// item order.  Splitting exists to give every workgroup of the grid something to do, so the pool is a fraction of
// the workgroups that share a head group's items (par) and does not grow with the batch: br_split_pool(par, nhg) slots,
// at most BR_SPLIT_POOL_MAX.  The plan lengthens the splits until the batch fits the pool.
#define BR_SPLIT_POOL_MAX 160
#ifndef BR_MIN_CHUNK
#define BR_MIN_CHUNK 4        // a split of the query block's key walk covers at least this many tiles
#endif

// Plan buffer (int32):
//   [header BR_PLAN_HDR][start B*M][len B*M][tok B*M][prev_tiles B][tile base B*M][block queue B*M]
//   [tile descriptors 2*B*TPS][items 16*max_items][comb 4*max_comb]
// The items array holds the global queue's items followed by the items of the eight XCD queues.
// Tile descriptors: for each sequence, the 64-key tiles of blocks 0..M-2 in order, as (token index of
// the tile's first key, number of real keys); TPS = (M-1) * ceil(H/64) slots per sequence.
// Work is handed out through 9 queues.  Queues 0..7 belong to the 8 XCDs: all query tiles of one (sequence,
// block) go to one queue, so the block's K/V for all heads are fetched into one XCD's L2 only; the query
// block's key walk is cut where the blocks it reads change from one XCD's run to the next, and every piece is
// put at the front of the queue of the XCD whose L2 holds those blocks (the long items go first, and the K/V
// they walk over are the ones that XCD's other items fetch anyway).  Queue 8, drained first by every workgroup,
// holds what has no such preference: the items of sequences that are one block only.  The items array is grouped by queue (queue g's items
// start at QOFF[g]); a ticket t of queue g is (item QOFF[g] + t / NHG, head group t % NHG):
// consecutive tickets cover all kv heads, which keeps every L2 channel busy.
#define BR_PLAN_HDR 96
#define BR_NQUEUES 9
#define BR_GLOBAL_QUEUE 8
enum BrPlanHeader {
    BR_PH_NITEMS = 0,     // number of work items (per head group)
    BR_PH_NCOMB = 1,      // number of combine entries (per head group)
    BR_PH_PACKED = 2,     // 1: tokens are packed (no padded slots between blocks), see tok[] below
    BR_PH_NONCONTIG = 4,  // set to 1 if some block's real tokens are not one contiguous span
    BR_PH_MAX_ITEMS = 5,
    BR_PH_MAX_COMB = 6,
    BR_PH_T = 7,          // tokens per query tile the plan was built for
    BR_PH_POOL = 26,      // split-KV slots the plan was built for
    BR_PH_NSLOTS = 27,    // ... and how many of them it uses
    BR_PH_QCOUNT = 8,     // [9] items in each queue
    BR_PH_QOFF = 17,      // [9] index of each queue's first item
    // second cache line: everything the running kernels update
    BR_PH_QTICKET = 32,   // [9] ticket counters (zero between launches)
    BR_PH_DONE = 48,      // workgroups that have left the persistent loop (zero between launches)
};

// One unit of prefill work: query tile [t0, t0+T) of block m of sequence b, restricted to a range
// of its key/value tile walk.  The walk is: the nprev tiles of the earlier blocks the block may see
// (the sequence's first nprev tile descriptors), then the tiles of its own block up to the diagonal.
// f_lo is the first tile of the range in that order, ntiles how many to process (INT_MAX = to the
// end).  slot < 0: the item owns its rows and writes the final output; slot >= 0: it writes an
// unnormalised partial into that slot of the batch's pool.  The item also carries what the kernel would otherwise have
// to look up before it can issue its first load: the block's own span and the prefix block's span.
struct BrItem {
    int b, m, t0, f_lo, nprev, ntiles, slot, pe;
    int len_m, start_m, len0, start0;
    int tok_m, tok0;      // index on the token axis of the first real token of block m / of block 0
    int pad[2];
};
#define BR_ITEM_WORDS_USED 14
#define BR_ITEM_INTS 16
struct BrComb {
    int b, t0, slot0, nsplit;
};

struct BrPlanView {
    const int* hdr;
    const int* start;      // B*M: position of the block's first real token inside its H slots
    const int* len;        // B*M
    const int* tok;        // B*M: index of that token on the token axis of q/k/v/out.  Padded layout:
                           // m*H + start (per sequence); packed layout: running sum of the lengths
                           // over the whole batch (the batch stride of the tensors is then 0)
    const int2* tiles;     // B * TPS tile descriptors
    int tps;
    const BrItem* items;
    const BrComb* comb;
};

__host__ __device__ inline size_t br_plan_off_start() { return BR_PLAN_HDR; }
__host__ __device__ inline size_t br_plan_off_len(int B, int M) { return BR_PLAN_HDR + (size_t)B * M; }
__host__ __device__ inline size_t br_plan_off_tok(int B, int M) { return BR_PLAN_HDR + 2 * (size_t)B * M; }
__host__ __device__ inline size_t br_plan_off_prev(int B, int M) { return BR_PLAN_HDR + 3 * (size_t)B * M; }
// par / 4 pieces to fill the grid with, plus room for the cuts at the XCD queues' boundaries (up to eight per query
// tile of a sequence that is spread over all XCDs; nhg: head groups, each of which has its own set of slots).
__host__ __device__ inline int br_split_pool(int par, int nhg) {
    const int n = par / 4 + 2 + 128 / (nhg > 0 ? nhg : 1);
    return n > BR_SPLIT_POOL_MAX ? BR_SPLIT_POOL_MAX : n;
}
__host__ __device__ inline int br_plan_max_items(int B, int M, int H, int T) {
    int qt = (H + T - 1) / T;
    // every query tile of every block once, plus one more item per slot a split query tile takes
    return B * (M > 1 ? M : 1) * qt + BR_SPLIT_POOL_MAX;
}
// (a split query tile takes at least two slots)
__host__ __device__ inline int br_plan_max_comb(int B) { return BR_SPLIT_POOL_MAX / 2; }
__host__ __device__ inline int br_plan_tps(int M, int H) { return (M > 1 ? M - 1 : 0) * ((H + BR_BN - 1) / BR_BN); }
__host__ __device__ inline size_t br_plan_off_tbase(int B, int M) { return BR_PLAN_HDR + 3 * (size_t)B * M + (size_t)B; }
__host__ __device__ inline size_t br_plan_off_bq(int B, int M) { return br_plan_off_tbase(B, M) + (size_t)B * M; }
__host__ __device__ inline size_t br_plan_off_tiles(int B, int M) { return (br_plan_off_bq(B, M) + (size_t)B * M + 1) & ~(size_t)1; }
__host__ __device__ inline size_t br_plan_off_items(int B, int M, int H, int T) {
    size_t o = br_plan_off_tiles(B, M) + 2 * (size_t)B * br_plan_tps(M, H);
    return (o + 15) & ~(size_t)15;   // 64-byte aligned items
}
__host__ __device__ inline size_t br_plan_off_comb(int B, int M, int H, int T) {
    return br_plan_off_items(B, M, H, T) + BR_ITEM_INTS * (size_t)br_plan_max_items(B, M, H, T);
}
__host__ __device__ inline size_t br_plan_total_ints(int B, int M, int H, int T) {
    return br_plan_off_comb(B, M, H, T) + 4 * (size_t)br_plan_max_comb(B);
}

__device__ inline BrPlanView br_plan_view(const int* plan, int B, int M, int H, int T) {
    BrPlanView v;
    v.hdr = plan;
    v.start = plan + br_plan_off_start();
    v.len = plan + br_plan_off_len(B, M);
    v.tok = plan + br_plan_off_tok(B, M);
    v.tiles = reinterpret_cast<const int2*>(plan + br_plan_off_tiles(B, M));
    v.tps = br_plan_tps(M, H);
    v.items = reinterpret_cast<const BrItem*>(plan + br_plan_off_items(B, M, H, T));
    v.comb = reinterpret_cast<const BrComb*>(plan + br_plan_off_comb(B, M, H, T));
    return v;
}

// ---- work distribution of the persistent kernels -------------------------------------------------
// The XCD this wave runs on (0..7).
__device__ inline int br_xcc_id() {
    // s_getreg_b32 HW_REG_XCC_ID (id 20), bits [3:0]
    return __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7;
}

// Queue visited at step k of a workgroup on XCD x: the global queue, its own, then the others.
__device__ inline int br_queue_at(int k, int x) { return k == 0 ? BR_GLOBAL_QUEUE : ((x + k - 1) & 7); }

// Called by one thread: take the next ticket from the queue at step *k, moving on once a queue is
// empty (so that an XCD that runs dry helps the others).  Returns queue << 24 | ticket, or -1 when
// every queue is exhausted.  first_ticket is a ticket already drawn from the current queue, or -1.
__device__ inline int br_take_ticket(int* hdr, int NHG, int x, int* k, int first_ticket) {
    int t = first_ticket;
    while (*k < BR_NQUEUES) {
        const int q = br_queue_at(*k, x);
        if (t < 0) t = atomicAdd(&hdr[BR_PH_QTICKET + q], 1);
        if (t < hdr[BR_PH_QCOUNT + q] * NHG) return (q << 24) | t;
        ++*k;
        t = -1;
    }
    return -1;
}

// Decode queue << 24 | ticket into (item index, head group).  Uniform across the workgroup.
__device__ inline void br_decode_ticket(const BrPlanView& pv, int qt, int NHG, int& item, int& hg) {
    const int q = qt >> 24, t = qt & 0xffffff;
    const int li = t / NHG;
    hg = t - li * NHG;
    item = pv.hdr[BR_PH_QOFF + q] + li;
}

// Leave the persistent loop: the last workgroup re-arms the counters for the next launch.
__device__ inline void br_leave(int* hdr) {
    int d = atomicAdd(&hdr[BR_PH_DONE], 1);
    if (d == (int)gridDim.x - 1) {
        for (int i = 0; i < BR_NQUEUES; ++i) atomicExch(&hdr[BR_PH_QTICKET + i], 0);
        atomicExch(&hdr[BR_PH_DONE], 0);
    }
}

// Number of earlier blocks a query block m attends to in full: none for the prefix, the prefix for
// a document, every earlier block for the query block (which is also block 0 when M == 1).
__host__ __device__ inline int br_prev_blocks(int m, int M) {
    if (m == 0) return 0;
    return m == M - 1 ? M - 1 : 1;
}

// Walk over the key/value tiles one query tile sees.  Every field is uniform across the workgroup.
struct BrTile {
    int flat;     // index among the sequence's earlier-block tile descriptors, -1 for the block's own tiles
    int tok0;     // token index (inside the sequence) of the tile's first key
    int kt;       // for the block's own tiles: tile index inside the block (first key is kt*BR_BN)
    int nvalid;   // real keys in the tile (1..BR_BN)
    int self;     // 1 if the keys belong to the query tile's own block (causal rule applies)
};

// Index part of the walk: which tile comes next and whether it is one of the nprev earlier-block
// tiles (flat index returned in *prev_index, descriptor to be supplied by the caller) or one of the
// block's own.
struct BrWalk {
    int f, f_end, nprev, self_end, own_tok0;

    __device__ void init(const BrItem& it, int self_end_, int H) {
        f = it.f_lo;
        f_end = it.ntiles > 0x3fffffff ? 0x7fffffff : it.f_lo + it.ntiles;
        nprev = it.nprev;
        self_end = self_end_;
        own_tok0 = it.tok_m;
    }
    // returns 0: exhausted, 1: earlier-block tile *prev_index, 2: own tile filled into t
    __device__ int next(BrTile& t, int* prev_index) {
        if (f >= f_end) return 0;
        if (f < nprev) {
            *prev_index = f++;
            return 1;
        }
        const int kt = f - nprev, k0 = kt * BR_BN;
        if (k0 >= self_end) return 0;
        t.flat = -1;
        t.tok0 = own_tok0 + k0;
        t.kt = kt;
        t.nvalid = self_end - k0 < BR_BN ? self_end - k0 : BR_BN;
        t.self = 1;
        ++f;
        return 2;
    }
};

// Descriptor of earlier-block tile i of a document (the only earlier block is the prefix).
__device__ inline void br_prefix_tile(const BrItem& it, int i, BrTile& t) {
    t.flat = i;
    t.tok0 = it.tok0 + i * BR_BN;
    t.kt = i;
    t.nvalid = it.len0 - i * BR_BN < BR_BN ? it.len0 - i * BR_BN : BR_BN;
    t.self = 0;
}

// Row mapping shared by every kernel that touches a work item: a workgroup of NW "row blocks" of 32
// query rows covers Gw = NW / tpb heads x T = 32 * tpb tokens.  Row block r is head r / tpb of the
// group and token sub-block r % tpb.  hg enumerates (kv head, head sub-group).
struct BrGeom {
    int G;      // query heads per kv head
    int Gw;     // heads one workgroup covers
    int tpb;    // 32-token sub-blocks per query tile
    int HGS;    // head sub-groups per kv head = G / Gw
    int NHG;    // head groups in total = Nkv * HGS
};

__host__ __device__ inline int br_tokens_per_tile(const BrGeom& g) { return g.tpb * BR_RB; }

struct BrPrefillParams {
    const void* q;
    const void* k;
    const void* v;
    void* out;
    const int* plan;
    float* part_o;    // split-KV partial outputs: [slot][NW*32 rows][D] fp32, unnormalised
    float* part_ml;   // [slot][NW*32 rows][2]: running max (log2 domain) and denominator (the sum of the probabilities as
                      // rounded for the P V product: what normalises the merged output)
    float* part_lx;   // [slot][NW*32 rows]: the exact sum of the probabilities, written and read only when the
                      // log-sum-exp is asked for (lse below)
    long long sq_b, sq_h, sq_t;   // element strides of q for (batch, head, token); the last dim is dense
    long long sk_b, sk_h, sk_t;
    long long sv_b, sv_h, sv_t;
    long long so_b, so_h, so_t;
    // the same strides as 32-bit values (the entry points reject strides of 2^31 elements or more): the
    // MFMA kernels use these - half the registers, and 32 x 32 -> 64 bit multiplies for the addresses
    unsigned q32_b, q32_h, q32_t, k32_b, k32_h, k32_t, v32_b, v32_h, v32_t, o32_b, o32_h, o32_t;
    int B, Nq, Nkv, M, H;
    BrGeom geom;
    float scale_log2;  // softmax scale * log2(e)
    // Optional score partials of the query block's last score_R rows (padded positions H-score_R..H-1):
    // [B][Nq][score_R][TPS][2] = (reference max in the log2 domain, sum of 2^(logit - max)) per earlier-block
    // key tile, in the order of the sequence's tile descriptors.  Null: not wanted.
    float* score_part;
    int score_R;
    // fp8 Q K^T variant: k8 is the e4m3 copy of K ((batch, head) strides k8_b, k8_h in bytes, token stride D) and
    // qk_scales its dequantisation scales (powers of two), [B][Nkv] (Q is converted in registers by the attention
    // kernel, one scale per query row).  Null otherwise.
    const float* qk_scales;
    const void* k8;
    unsigned k8_b, k8_h;
    // Optional: rotary position embedding of Q applied by the attention kernel to the rows it loads (bf16 kernel
    // only): cos and sin tables (batch or 1, tokens, D) on the same token axis as q, element strides rope_b (0: one
    // table for the whole batch) and rope_t; q then holds the projection's output as it is.  Null: q is used as given.
    const void* rope_cos;
    const void* rope_sin;
    unsigned rope_b, rope_t;
    // Optional: the log-sum-exp of every real query row, in base-2 units (log2 of the sum over the visible keys
    // of 2^(scale * log2(e) * q.k)), at lse[b * lse_b + head * lse_h + token]; the backward pass starts from it.
    // Null: not wanted.  Written by the streaming bf16 kernel and the finish kernel only.
    float* lse;
    long long lse_b, lse_h;
};

// Arguments of the backward kernels (bf16).
struct BrBwdParams {
    const void* q;
    const void* k;
    const void* v;
    const void* out;
    const void* dout;
    const int* plan;
    const float* lse;          // base-2 log-sum-exp of every real row, as the forward wrote it
    float* delta;              // rowsum(dO * O) of every real row, same indexing as lse (written by the dQ kernel)
    long long lse_b, lse_h;
    float* dq32;               // [B][Nq][H][D] fp32: dQ sums of the query block's rows when several items share them
    float* dk32;               // [B][Nkv][H][D] fp32: dK, dV sums of the prefix keys (one workgroup per viewing block adds to them)
    float* dv32;
    void* dq;
    void* dk;
    void* dv;
    long long dq_b, dq_h, dq_t, dk_b, dk_h, dk_t, dv_b, dv_h, dv_t;
    unsigned q32_b, q32_h, q32_t, k32_b, k32_h, k32_t, v32_b, v32_h, v32_t, o32_b, o32_h, o32_t, g32_b, g32_h, g32_t;
    int B, Nq, Nkv, M, H;
    BrGeom geom;
    float scale, scale_log2;
    int max_items;
};
