// Block-sparse prefill attention for gfx950, 16-bit inputs (bf16), fp32 softmax and accumulation.
//
// What it computes (reference: sdpa_blockrank_attention_forward, blockrank_std_attention.py:503-650):
// for every real query token, softmax(scale * q.k) over the keys it may see, times V, where the
// prefix block sees itself causally, a document sees the prefix in full plus itself causally, and
// the query block sees every earlier block in full plus itself causally.  Padded slots are neither
// read nor computed (the reference leaves an unspecified average there and never consumes it); the
// finish kernel sets them to zero.
//
// How: a persistent grid pulls work items (query tile x key-walk range) from the request plan.  A
// workgroup of NW waves stages each 64-key K tile and V^T tile in LDS once and every wave - one
// 32-row block of one query head of the kv head's group - consumes them, so K/V are read once per
// head group, not once per query head.  Per wave and tile:
//   S^T = K Q^T      v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q^T held in registers
//   online softmax   each lane owns one query row and half of the tile's keys, so the row max / sum
//                    need one cross-lane exchange (lane ^ 32) and the O rescale is a per-lane scalar
//   O^T += V^T P^T   A = V^T rows from LDS, B = P^T straight from the S^T accumulators: the K rows
//                    are assigned to MFMA rows in a permuted order chosen so that the accumulator
//                    registers a lane ends up holding are exactly the 8 consecutive keys the next
//                    MFMA's B operand wants, so P never travels through LDS.
//
// Data movement: K/V tiles go from global memory straight into LDS (global_load_lds_dwordx4, 64
// lanes x 16 bytes per instruction, no staging registers); which 16-byte piece of which row a lane
// fetches is free, and that freedom provides both the row permutation and the swizzles below.  V is
// kept row-major ([key][dim]) and read with ds_read_b64_tr_b16, which hands each lane four
// consecutive keys of one dim - the MFMA A-operand layout of V^T - so V is never transposed by ALU code.
//
// LDS layouts (row = 2*D bytes, 16-byte chunks; reads are bank-conflict free):
//   K    row r of each 32-row half holds key swap23(r) (bits 2 and 3 of the index exchanged) so that
//        MFMA row = LDS row; chunk c of row r sits at chunk c ^ (r & 7).
//   V    row = key; chunk c of row r sits at chunk c ^ ((r & 3) << 1).
#pragma once
#include "br_common.h"
#include "br_score_tiles.h"

namespace {

// The 16-bit element type of Q, K, V and the output is a property of the translation unit: BR_E16 is __bf16 unless the
// including file defines it as _Float16 (with BR_E16_IS_F16).  Same layouts, same kernels; the matrix and dot-product
// instructions are the ones of that type.
#ifndef BR_E16
#define BR_E16 __bf16
#endif
typedef float br_f32x16 __attribute__((ext_vector_type(16)));
typedef BR_E16 e16x8 __attribute__((ext_vector_type(8)));
typedef BR_E16 e16x4 __attribute__((ext_vector_type(4)));
typedef BR_E16 e16x2 __attribute__((ext_vector_type(2)));
#ifdef BR_E16_IS_F16
__device__ inline br_f32x16 br_mma16(e16x8 a, e16x8 b, br_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
__device__ inline float br_dot2(e16x2 a, e16x2 b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }
#else
__device__ inline br_f32x16 br_mma16(e16x8 a, e16x8 b, br_f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
__device__ inline float br_dot2(e16x2 a, e16x2 b, float c) { return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false); }
#endif
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// F8: K (and Q) are fp8 e4m3 (one byte per element, dequantisation scales folded into the softmax
// scale); V, P and the output stay bf16.
template <int D, bool F8>
struct Smem {
    static constexpr int rowB = D * 2;                     // bytes per V row (and per bf16 K row)
    static constexpr int rowKB = F8 ? D : D * 2;           // bytes per K row
    static constexpr int kBytes = BR_BN * rowB;            // room of the K tile (an fp8 tile fills half of it): the V tile
                                                           // sits at the same offset whatever the K element type, so that
                                                           // items of both kinds can follow each other in one kernel and
                                                           // the V rows never hold anything but bf16 V data
    static constexpr int vBytes = BR_BN * rowB;
    static constexpr int stageBytes = kBytes + vBytes;     // K tile then V tile
    static constexpr int eRow = D + 8;                     // epilogue tile: [32 rows][eRow] per wave
    static constexpr int eBytesPerWave = BR_RB * eRow * 2;
    static constexpr int total(int nw) {
        int a = 2 * stageBytes, b = nw * eBytesPerWave;
        return a > b ? a : b;
    }
};

__device__ inline uint4 ld16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline e16x8 as_e16x8(uint4 u) {
    union { uint4 u; e16x8 v; } c;
    c.u = u;
    return c.v;
}
__device__ inline int uni(int x) { return __builtin_amdgcn_readfirstlane(x); }
// The value of lane ^ 32 combined with the lane's own: one v_permlane32_swap (which exchanges the upper half of its
// first operand with the lower half of its second) instead of a trip through the LDS crossbar.
__device__ inline float max_xor32(float x) {
    const unsigned u = __float_as_uint(x);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
// Scheduling directives for the compiler's instruction scheduler: a group of `n` instructions of one kind, placed in
// the order the directives are written; unmatched instructions go where their dependencies allow.
#define BR_SCHED_MFMA(n) __builtin_amdgcn_sched_group_barrier(0x008, n, 0)
#define BR_SCHED_DSREAD(n) __builtin_amdgcn_sched_group_barrier(0x100, n, 0)
#define BR_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// 64 lanes x 16 bytes from global memory (uniform base + per-lane byte offset) into LDS at
// lds_addr + lane * 16.  Issued through asm so that the compiler does not make later LDS reads of
// other buffers wait for it; completion is awaited explicitly (vm_wait_all) before the barrier that
// publishes the tile.
__device__ inline void dma16(const void* base, int byte_off, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(byte_off), "s"(base), "s"(lds_addr) : "memory", "m0");
}
__device__ inline void vm_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ inline unsigned lds_addr_of(const void* p) {
    return (unsigned)(size_t)(__attribute__((address_space(3))) const void*)p;
}

// Zero the output rows of a block's padded token slots (padded layout: the block's H slots start at token
// slot0; its real tokens are [start, start + len)), for heads head0 .. head0 + nheads - 1.  Called by
// all nthreads threads of a workgroup; plain 16-byte stores, nothing waits for them.
template <int D>
__device__ inline void zero_padded_rows(const BrPrefillParams& p, int b, int head0, int nheads, int slot0, int start, int len, int tid,
                                        int nthreads) {
    constexpr int CP8 = D / 8;                    // 16-byte pieces per row (a power of two)
    const int npad = p.H - len;
    if (npad <= 0) return;
    const uint4 z = {0u, 0u, 0u, 0u};
    for (int g = 0; g < nheads; ++g) {
        char* obase = reinterpret_cast<char*>(p.out) +
                      2 * ((unsigned long long)p.o32_b * (unsigned)b + (unsigned long long)p.o32_h * (unsigned)(head0 + g) +
                           (unsigned long long)p.o32_t * (unsigned)slot0);
        for (int idx = tid; idx < npad * CP8; idx += nthreads) {
            const int r = idx / CP8, c8 = idx - r * CP8;
            const int pos = r < start ? r : r + len;
            *reinterpret_cast<uint4*>(obase + 2 * ((long long)pos * p.o32_t + c8 * 8)) = z;
        }
    }
}

// Exchange bits 2 and 3.  MFMA row r of a 32-key half tile carries key swap23(r): with the 32x32
// accumulator layout (lane = column + 32*h; register v is row 8*(v/4) + 4*h + v%4) registers
// 8*jp .. 8*jp+7 of lane half h then hold keys 16*jp + 8*h + 0..7, which is the B-operand layout of
// the P^T V product.
__device__ inline int swap23(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

// Descriptor prefetch, run by wave 0 while the workgroup computes an item: the ticket for the next
// item is drawn at the start of the current one; after the first key tile the 64-byte item it names
// is requested, and at the end of the item it is published through LDS.  Each step consumes a value
// whose load was issued a whole tile earlier, so the chain ticket -> item costs the item's critical
// path nothing (an item with a single tile finishes the chain at its end, waiting as needed).
//
// A workgroup draws from the global queue, then from the queue of its XCD (by workgroup index: the
// hardware deals workgroups round robin to the XCDs), and is done when both are dry.  It does not look into the other XCDs' queues: the plan cuts the work into eight runs of
// equal estimated size, and polling other queues' counters at the end of the kernel (with atomics
// or with loads) was measured to stretch the memory waits of every workgroup still working from
// 0.1 to 5-15 us.
struct BrDescMail {      // layout of one LDS mailbox
    int word[BR_ITEM_INTS];
    int hg;
    int valid;
    int pad[2];
};

struct BrPrefetch {
    int* hdr;
    const BrPlanView* pv;
    int NHG, lane;
    int xq, ng;    // this workgroup serves the XCD queues xq, xq + ng, ... (ng = 8 unless the grid is smaller)
    int qk, qend;  // step in the queue order: 0 global queue, 1.. own queues, qend done
    int counts;    // lane j: tickets of queue j
    int qoffs;     // lane j: index of queue j's first item
    int scounts;   // lane j: tickets of queue j handed out statically (one per workgroup, see init)
    int t_next;    // ticket drawn from the queue at step qk (lane 0), or -1
    int stage;     // 0 ticket drawn, 2 item requested, 9 nothing in flight
    int word, hg;

    // The first ticket of every workgroup is fixed by its index, with no atomic (512 workgroups
    // drawing from one counter at the same moment queue up for microseconds): workgroups 0..SG-1
    // take the global queue's tickets 0..SG-1; the others take, in index order, the first tickets of
    // the queue blockIdx & 7 (workgroups are dealt round robin to the XCDs, so this is normally the
    // queue of the XCD they run on; if it is not, only locality is lost).  The counters therefore
    // count the tickets drawn after the static ones.
    __device__ void init(int* hdr_, const BrPlanView* pv_, int NHG_, int lane_) {
        hdr = hdr_; pv = pv_; NHG = NHG_; lane = lane_;
        counts = lane < BR_NQUEUES ? hdr[BR_PH_QCOUNT + lane] * NHG : 0;
        qoffs = lane < BR_NQUEUES ? hdr[BR_PH_QOFF + lane] : 0;
        const int grid = gridDim.x, me = blockIdx.x;
        // Queue ownership goes by workgroup index, not by the XCD id the hardware reports: every queue
        // then has its workgroups whatever the placement is, so all work is done in any case.
        ng = grid < 8 ? grid : 8;
        xq = me % ng;
        qend = 1 + (8 - xq + ng - 1) / ng;
        const int cg = __builtin_amdgcn_readlane(counts, BR_GLOBAL_QUEUE);
        const int SG = grid < 8 ? 0 : (cg < grid ? cg : grid);      // (no static tickets on a tiny grid)
        const int first = SG + ((lane - SG) & 7);                   // lane j < 8: first workgroup of queue j
        const int nwg = first < grid ? (grid - 1 - first) / 8 + 1 : 0;
        scounts = lane < 8 ? (nwg < counts ? nwg : counts) : (lane == BR_GLOBAL_QUEUE ? SG : 0);
        if (grid < 8) scounts = 0;
        qk = SG == cg ? 1 : 0;      // every global ticket handed out already: start at the XCD's own queue
        t_next = -1;
        stage = 9;
        word = hg = 0;
        int q = -1, t = 0;
        if (me < SG) {
            q = BR_GLOBAL_QUEUE;
            t = me;
        } else if (grid >= 8) {
            const int x = me & 7;
            const int r = (me - __builtin_amdgcn_readlane(first, x)) >> 3;
            if (r < __builtin_amdgcn_readlane(scounts, x)) {
                q = x;
                t = r;
            }
        }
        if (q >= 0) request(q, t);
    }
    __device__ int queue_now() const { return qk == 0 ? BR_GLOBAL_QUEUE : xq + (qk - 1) * ng; }
    __device__ void request(int q, int t) {   // ask for the item that ticket t of queue q names
        const int li = t / NHG;
        hg = t - li * NHG;
        const int idx = __builtin_amdgcn_readlane(qoffs, q) + li;
        word = reinterpret_cast<const int*>(pv->items + idx)[lane & (BR_ITEM_INTS - 1)];
        stage = 2;
    }
    __device__ void draw() {   // at the start of an item
        t_next = -1;
        stage = 9;
        if (qk < qend) {
            if (lane == 0) t_next = atomicAdd(&hdr[BR_PH_QTICKET + queue_now()], 1);
            stage = 0;
        }
    }
    __device__ void step() {   // once per key tile, after the tile's arithmetic
        if (stage == 0) {
            const int q = queue_now();
            const int t = __builtin_amdgcn_readfirstlane(t_next) + __builtin_amdgcn_readlane(scounts, q);
            if (t < __builtin_amdgcn_readlane(counts, q)) {
                request(q, t);
            } else {
                stage = 9;
                ++qk;          // that queue is dry for good
            }
        }
    }
    // Nothing in flight: draw now, from the global queue and then the own one.
    __device__ bool find_work() {
        while (qk < qend) {
            const int q = queue_now();
            if (__builtin_amdgcn_readlane(counts, q) <= __builtin_amdgcn_readlane(scounts, q)) {   // nothing to hand out: no atomic
                ++qk;
                continue;
            }
            int t = 0;
            if (lane == 0) t = atomicAdd(&hdr[BR_PH_QTICKET + q], 1);
            t = __builtin_amdgcn_readfirstlane(t) + __builtin_amdgcn_readlane(scounts, q);
            if (t < __builtin_amdgcn_readlane(counts, q)) {
                request(q, t);
                return true;
            }
            ++qk;
        }
        return false;
    }
    __device__ void publish(BrDescMail* mail) {   // at the end of an item (and once before the first)
        if (stage == 0) step();
        if (stage == 9 && !find_work()) {
            if (lane == 0) mail->valid = 0;
            return;
        }
        if (lane < BR_ITEM_INTS) mail->word[lane] = word;
        if (lane == 0) {
            mail->hg = hg;
            mail->valid = 1;
        }
    }
};

// Power-of-two quantisation scale of a group whose largest magnitude is amax: 2^(floor(log2(amax)) - 7), which
// puts that magnitude into [128, 256) of e4m3's range (up to 448), and its inverse.  Multiplying by a power of two
// is exact, so every implementation of the quantiser rounds the same values the same way.  A group whose maximum
// is below 2^-119 (or not a number) counts as zero: both results are 0.
__device__ inline void br_pow2_scale(float amax, float& scale, float& inv) {
    const unsigned eb = __float_as_uint(fminf(amax, 3.0e38f)) & 0x7f800000u;
    const bool ok = eb >= (8u << 23);
    const unsigned sb = eb - (7u << 23);
    scale = ok ? __uint_as_float(sb) : 0.f;
    inv = ok ? __uint_as_float((254u << 23) - sb) : 0.f;
}

typedef long k8x8;   // eight fp8 values: one MFMA operand of v_mfma_f32_32x32x16_fp8_fp8

template <bool F8> struct QKFrag { typedef e16x8 type; };
template <> struct QKFrag<true> { typedef k8x8 type; };

// SC: the instance that can leave score partials and the log-sum-exp (exact probability sums); ROPE: the instance
// that rotates the Q rows it loads.  An instance without them carries none of their registers, scalars or code
// (the plain layers of a ranking forward use neither).
template <int D, int NW, bool F8, bool SC = true, bool ROPE = true>
struct Prefill {
    using SM = Smem<D, F8>;
    using Frag = typename QKFrag<F8>::type;                // K and Q operand of one 16-dim chunk
    static constexpr int ESZ = F8 ? 1 : 2;                 // bytes per K/Q element
    static constexpr int CPR = D / 8;                      // 16-byte chunks per V (and output) row
    static constexpr int CPRK = SM::rowKB / 16;            // 16-byte chunks per K row
    static constexpr int NI = BR_BN * CPR / 64;            // DMA instructions per V tile
    static constexpr int NIK = BR_BN * CPRK / 64;          // ... per K tile
    static constexpr int JK = (NI + NW - 1) / NW;          // per wave
    static constexpr int JKK = (NIK + NW - 1) / NW;

    // Per-lane constants, fixed for the whole kernel.
    // With 4 or 8 waves the DMA pieces of one lane are a whole number of 16-row groups apart, so one
    // offset plus a uniform step describes them all; otherwise each piece keeps its own offset.
    static constexpr bool UNIFORM_STEP = (NW == 4 || NW == 8);
    static constexpr int JO = UNIFORM_STEP ? 1 : JK;
    static constexpr int JOK = UNIFORM_STEP ? 1 : JKK;
    static constexpr int STEP_ROWS = NW * 64 / CPR;        // rows between consecutive V pieces of a wave
    // V swizzle: LDS piece = global piece ^ ((row & 3) << VSW).  One transposing read touches eight key rows
    // (rows r, r+1, r+2, r+3 and the same eight rows further), 64 bytes of each: with 256-byte rows the four
    // rows must land in four different 64-byte bank groups (shift 2); with 128-byte rows two rows share a bank
    // line and the shift that separates them is 1.
    static constexpr int VSW = CPR == 16 ? 2 : 1;
    static constexpr int STEP_ROWSK = NW * 64 / CPRK;      // ... K pieces
    // K swizzle: LDS piece = global piece ^ (row & KSW).  An operand read takes one 16-byte piece of each of 32 rows;
    // the 16 lanes that go through the banks together (16 x 16 bytes = one pass over all 64 banks) must hit 16
    // different pieces, so with 16 pieces per row the whole row index's low four bits take part (with 8 pieces per
    // row two rows share a 256-byte bank line and three bits do).
#ifndef BR_K_SWIZZLE_MASK
#define BR_K_SWIZZLE_MASK 15
#endif
    static constexpr int KSW = CPRK >= 16 ? BR_K_SWIZZLE_MASK : (CPRK < 8 ? CPRK - 1 : 7);
    struct Lane {
        int koff[JOK], voff[JO];   // global byte offsets inside a tile of this lane's DMA pieces
        int krd;                   // LDS byte offset of the K operand read of chunk 0; chunk c is krd ^ (c << (F8 ? 4 : 5))
        int vrd[D / 32];           // LDS byte offsets of the V^T operand reads, one per 32-dim block
    };

    static __device__ inline Lane make_lane(const BrPrefillParams& p, int wave, int lane) {
        Lane L;
#pragma unroll
        for (int j = 0; j < JOK; ++j) {
            const int slot = (wave + NW * j) * 64 + lane;
            const int prow = slot / CPRK, cp = slot - prow * CPRK;
            const int kkey = (prow & 32) | swap23(prow & 31);
            L.koff[j] = kkey * (F8 ? D : (int)p.k32_t * 2) + ((cp ^ (prow & KSW)) << 4);
        }
#pragma unroll
        for (int j = 0; j < JO; ++j) {
            const int slot = (wave + NW * j) * 64 + lane;
            const int prow = slot / CPR, cp = slot - prow * CPR;
            L.voff[j] = prow * (int)p.v32_t * 2 + ((cp ^ ((prow & 3) << VSW)) << 4);
        }
        const int ln = lane & 31, lh = lane >> 5;
        if (F8) L.krd = ln * SM::rowKB + ((ln & KSW) << 4) + lh * 8;   // 8 bytes: dims 16c + 8lh .. +7
        else L.krd = ln * SM::rowKB + ((lh ^ (ln & KSW)) << 4);
        // transposing read: within a group of 16 lanes, lane s points at key (s >> 2), dims 4 * (s & 3)
        const int s = lane & 15, ln_hi = (lane >> 4) & 1;
#pragma unroll
        for (int d = 0; d < D / 32; ++d)
            L.vrd[d] = SM::kBytes + (8 * lh + (s >> 2)) * SM::rowB + (((4 * d + 2 * ln_hi + ((s & 3) >> 1)) ^ ((s >> 2) << VSW)) << 4) + (s & 1) * 8;
        return L;
    }

    // Start the DMA of one K/V tile into a stage.  kt / vt point at the tile's first row (uniform).
    // lane_l is the lane index as an opaque value of the current loop iteration: the row arithmetic of
    // the partial-tile path is then redone where it is needed (it is rare) instead of being kept in
    // registers across the whole key loop.
    static __device__ inline void issue_tile(const Lane& L, int wave, int lane_l, const char* kt, const char* vt, int sk_bytes,
                                             int sv_bytes, int nvalid, unsigned stage_lds) {
        // rows past a partial tile's real keys are not fetched: the LDS rows keep older (finite) data,
        // which the kernel masks (K) or multiplies by exact zeros (V)
        if (nvalid == BR_BN) {
            // whole tile: straight-line issue, no per-piece predicate
#pragma unroll
            for (int j = 0; j < JKK; ++j) {
                const int q = wave + NW * j;
                if (NIK % NW == 0 || q < NIK) {
                    if (UNIFORM_STEP) dma16(kt + j * STEP_ROWSK * sk_bytes, L.koff[0], stage_lds + q * 1024);
                    else dma16(kt, L.koff[j], stage_lds + q * 1024);
                }
            }
#pragma unroll
            for (int j = 0; j < JK; ++j) {
                const int q = wave + NW * j;
                if (NI % NW == 0 || q < NI) {
                    if (UNIFORM_STEP) dma16(vt + j * STEP_ROWS * sv_bytes, L.voff[0], stage_lds + SM::kBytes + q * 1024);
                    else dma16(vt, L.voff[j], stage_lds + SM::kBytes + q * 1024);
                }
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < JKK; ++j) {
            const int q = wave + NW * j;
            if (NIK % NW == 0 || q < NIK) {
                const int prow = (q * 64 + lane_l) / CPRK;
                if (((prow & 32) | swap23(prow & 31)) < nvalid) {                  // K row of this piece
                    if (UNIFORM_STEP) dma16(kt + j * STEP_ROWSK * sk_bytes, L.koff[0], stage_lds + q * 1024);
                    else dma16(kt, L.koff[j], stage_lds + q * 1024);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < JK; ++j) {
            const int q = wave + NW * j;
            if (NI % NW == 0 || q < NI) {
                if ((q * 64 + lane_l) / CPR < nvalid) {                            // V row of this piece
                    if (UNIFORM_STEP) dma16(vt + j * STEP_ROWS * sv_bytes, L.voff[0], stage_lds + SM::kBytes + q * 1024);
                    else dma16(vt, L.voff[j], stage_lds + SM::kBytes + q * 1024);
                }
            }
        }
    }

    // Eight bf16 values times inv (the inverse of their row's power-of-two scale) as eight e4m3 values, in the
    // element order of the input (round to nearest even, the conversion instruction's rule).
    static __device__ inline k8x8 quantize_q8(u32x4 u, float inv) {
        const unsigned w[4] = {u[0], u[1], u[2], u[3]};
        int lo = 0, hi = 0;
        float x[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            x[2 * j] = __uint_as_float(w[j] << 16) * inv;               // below 256 in magnitude: no clamp needed
            x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u) * inv;
        }
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(x[0], x[1], lo, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(x[2], x[3], lo, true);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(x[4], x[5], hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(x[6], x[7], hi, true);
        return (k8x8)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
    }

    static __device__ inline Frag read_k(const char* stage, const Lane& L, int kb, int c) {
        if constexpr (F8) {
            return *reinterpret_cast<const k8x8*>(stage + kb * 32 * SM::rowKB + (L.krd ^ (c << 4)));
        } else {
            return as_e16x8(ld16(stage + kb * 32 * SM::rowKB + (L.krd ^ (c << 5))));
        }
    }
    static __device__ inline f32x16 mma_qk(Frag a, Frag b, f32x16 c) {
        if constexpr (F8) {
            return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a, b, c, 0, 0, 0);
        } else {
            return br_mma16(a, b, c);
        }
    }
    // V^T operand for dims 32d + (lane & 31), keys 16*c2 + 8*lh + 0..7: two transposing reads
    static __device__ inline e16x8 read_vt(const char* stage, const Lane& L, int d, int c2) {
        const char* vp = stage + L.vrd[d] + c2 * 16 * SM::rowB;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(__attribute__((address_space(3))) const char*)vp);
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(__attribute__((address_space(3))) const char*)(vp + 4 * SM::rowB));
        union { s16x8 s8; e16x8 b8; } a;
        a.s8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return a.b8;
    }

    // One wave, one 64-key tile already in LDS: S^T = K Q^T, online softmax, O^T += V^T P^T.
    // NKB 32-key halves are computed (the second half is skipped when no row of the wave can see it);
    // with MASK, keys >= lim (per row: the tile's real keys and the diagonal) are excluded.  Every
    // variant is one straight-line block with the LDS operand reads issued ahead of their use.
    template <int NKB, bool MASK, bool EXACT>
    static __device__ inline void compute_tile(const char* stage, const Lane& L, const Frag (&qf)[D / 16], f32x16 (&o)[D / 32],
                                               float& m_run, float& l_run, float& lt_run, float scale_log2, int lim, int lh, float& psum_out) {
        constexpr int NC = D / 16, ND = D / 32, NR = NKB * NC;
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        f32x16 s[NKB];
        {
            // read i: half i % NKB, chunk i / NKB - the halves alternate so that consecutive MFMAs are
            // independent; reads run 4 ahead
            Frag ka[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) ka[i] = read_k(stage, L, i % NKB, i / NKB);
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) s[kb] = zero;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const Frag a = ka[i & 3];
                if (i + 4 < NR) ka[i & 3] = read_k(stage, L, (i + 4) % NKB, (i + 4) / NKB);
                s[i % NKB] = mma_qk(a, qf[i / NKB], s[i % NKB]);
            }
            // keep that order: four operand reads in flight ahead of every product (left alone, the scheduler
            // shortens the live ranges until every product waits for its own read)
            BR_SCHED_DSREAD(4);
#pragma unroll
            for (int i = 0; i + 4 < NR; ++i) {
                BR_SCHED_MFMA(1);
                BR_SCHED_DSREAD(1);
            }
            BR_SCHED_MFMA(4);
            BR_SCHED_FENCE();
        }
        // first V^T operands: their LDS latency passes under the softmax arithmetic
        e16x8 va[ND];
#pragma unroll
        for (int d = 0; d < ND; ++d) va[d] = read_vt(stage, L, d, 0);
        if (MASK) {
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int key = kb * 32 + 16 * (v >> 3) + 8 * lh + (v & 7);
                    if (key >= lim) s[kb][v] = -INFINITY;
                }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[kb][v]);
        mx = max_xor32(mx);
        // Lazy rescale: the running max is only raised (and O, l rescaled) when some row's max grew by
        // more than 2^8; otherwise exponentials are taken against the older max, which changes nothing
        // in the final quotient and keeps them below 2^8.
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
                for (int v = 0; v < 16; ++v) o[d][v] *= alpha;
        }
        const float m_sub = m_run == -INFINITY ? 0.f : m_run;
        // Two sums of the probabilities: the exact one (log-sum-exp, score partials) and the sum of the values
        // as rounded to bf16 for the P V product.  The output is normalised by the second: numerator and
        // denominator then carry the same rounding, and a row whose mass sits on one key reproduces that key's
        // V row exactly instead of V * (rounded p / p).
        float psum = 0.f, psum_t = 0.f;
        const e16x2 ones2 = {(BR_E16)1.0f, (BR_E16)1.0f};
        e16x8 pf[2 * NKB];
#pragma unroll
        for (int c2 = 0; c2 < 2 * NKB; ++c2) {
            f32x8 t;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                t[e] = __builtin_amdgcn_exp2f(s[c2 >> 1][8 * (c2 & 1) + e] * scale_log2 - m_sub);
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
#pragma unroll
        for (int c2 = 0; c2 < 2 * NKB; ++c2) {
#pragma unroll
            for (int d = 0; d < ND; ++d) {
                o[d] = br_mma16(va[d], pf[c2], o[d]);
                if (c2 + 1 < 2 * NKB) va[d] = read_vt(stage, L, d, c2 + 1);
            }
        }
    }

    static __device__ void run_item(const BrPrefillParams& p, const BrPlanView& pv, const BrItem& it, int hg, char* smem,
                                    const Lane& L, BrPrefetch& pf, bool padded_layout) {
        const int tid = threadIdx.x;
        const int wave = uni(tid >> 6), lane = tid & 63, ln = lane & 31, lh = lane >> 5;
        const BrGeom& ge = p.geom;
        const int T = ge.tpb * BR_RB;
        const int b = it.b, m = it.m;
        // (tpb is 1, 2 or 4 and a kv head usually has one sub-group: no integer divisions on the way to the first load)
        const int kvh = ge.HGS == 1 ? hg : hg / ge.HGS, hsub = hg - kvh * ge.HGS;
        const int tsh = ge.tpb == 1 ? 0 : (ge.tpb == 2 ? 1 : 2);
        const int g = wave >> tsh, sub = wave & (ge.tpb - 1);
        // (a kv head's group need not be a multiple of Gw: the last sub-group then has waves without a head, which
        // stay with the workgroup - barriers, DMA - and neither load rows nor store anything)
        const int hpos = hsub * ge.Gw + g;
        const bool head_ok = hpos < ge.G;
        const int head = kvh * ge.G + (head_ok ? hpos : ge.G - 1);
        const int len_m = it.len_m;
        const int len_w = head_ok ? len_m : 0;             // the block's length as far as this wave's rows go
        const int row0 = it.t0 + sub * BR_RB;              // first query row of this wave, valid-relative
        const bool rb_active = row0 < len_w;
        const int self_end = it.t0 + T < len_m ? it.t0 + T : len_m;
        const int qtok0 = it.tok_m;                        // token index of the block's first real token
        const unsigned smem_lds = lds_addr_of(smem);
        const int sk_bytes = F8 ? D : (int)p.k32_t * 2, sv_bytes = (int)p.v32_t * 2;

        // fp8: K comes from the quantised copy (token stride D bytes); Q is read as bf16 and converted in registers
        const char* kbase = F8 ? reinterpret_cast<const char*>(p.k8) + ((unsigned long long)p.k8_b * (unsigned)b + (unsigned long long)p.k8_h * (unsigned)kvh)
                               : reinterpret_cast<const char*>(p.k) + ((unsigned long long)p.k32_b * (unsigned)b + (unsigned long long)p.k32_h * (unsigned)kvh) * 2;
        const char* vbase = reinterpret_cast<const char*>(p.v) + ((unsigned long long)p.v32_b * (unsigned)b + (unsigned long long)p.v32_h * (unsigned)kvh) * 2;
        // fp8: every query row is quantised in registers with its own scale (absmax of the row / 448: each lane owns
        // one row, so the scale is a per-lane factor of the softmax scale); K carries one scale per (sequence, kv head)
        float sc2 = p.scale_log2;
        if constexpr (F8) {
            float f = 0.f;
            if (lane == 0) f = p.qk_scales[(long long)b * p.Nkv + kvh];
            sc2 *= __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, f)));
        }

        // The walk over the item's key tiles needs no memory lookups inside the loop: a document's only
        // earlier block is the prefix (described by the item itself); a query-block item keeps the
        // descriptors of its earlier-block tiles in lane registers (lane i = tile dbase + i) and reads
        // them with readlane.  Every quantity is a scalar computed with selects (no tile structs: they
        // would end up in scratch memory, and a scratch load waits for the tile DMAs in flight).
        const int2* tiles_b = pv.tiles + (size_t)b * pv.tps;
        const bool table = it.pe > 1;
        // only query-block items of a sequence with documents emit score partials, for document tiles
        bool emit_scores = false, exact = false;
        if constexpr (SC) {
            emit_scores = p.score_part != nullptr && table && m == p.M - 1;
            exact = emit_scores || p.lse != nullptr;
        }
        const int first_doc_tile = (it.len0 + BR_BN - 1) / BR_BN;
        const int nprev = it.nprev;
        const int f_end = it.ntiles > 0x3fffffff ? 0x7fffffff : it.f_lo + it.ntiles;
        const int own_tok0 = it.tok_m;
        int wf = it.f_lo;                                  // next tile of the walk
        int dbase = it.f_lo;
        int2 dreg = make_int2(0, 0);
        if (table) {
            if (dbase + lane < nprev) dreg = tiles_b[dbase + lane];
            // wait for the table here: a wait placed later would also cover the Q loads issued below
            asm volatile("" : "+v"(dreg.x), "+v"(dreg.y));
        }
        // Q^T fragments: lane (ln, lh) holds row row0+ln, dims 16c + 8lh .. +7 for every chunk c.  Requested
        // early (they come from HBM; only the tile table's load, which the walk needs first, goes before them):
        // the rest of the set-up runs under their latency.
        Frag qf[D / 16];
        u32x4 qraw[F8 ? D / 16 : 1];       // fp8: the bf16 rows as loaded, converted once they have arrived
        // rotary embedding applied here: the row's cos / sin values for the lane's dims (both halves of the tables)
        constexpr bool DO_ROPE = ROPE && !F8;
        constexpr int NRC = DO_ROPE ? D / 32 : 1;
        e16x8 rcos[2][DO_ROPE ? NRC : 0], rsin[2][DO_ROPE ? NRC : 0];
        bool rope = false;
        if constexpr (DO_ROPE) rope = p.rope_cos != nullptr && rb_active;
        {
            const char* qrow = reinterpret_cast<const char*>(p.q) +
                               ((unsigned long long)p.q32_b * (unsigned)b + (unsigned long long)p.q32_h * (unsigned)head +
                                (unsigned long long)p.q32_t * (unsigned)(qtok0 + row0)) * 2;
            // rows past the block's end load its last row instead (no per-lane branches around the loads):
            // what such rows compute is never stored
            const int last = len_m - 1 - row0;
            const int qoff = ((ln < last ? ln : last) * (int)p.q32_t + lh * 8) * 2;
            if (rb_active) {
#pragma unroll
                for (int c = 0; c < D / 16; ++c) {
                    if constexpr (F8) qraw[c] = *reinterpret_cast<const u32x4*>(qrow + qoff + c * 32);
                    else qf[c] = as_e16x8(ld16(qrow + qoff + c * 32));
                }
            } else {
                // a wave without rows computes no tile (nkb is 0 below): its fragments are never read, so they are
                // only declared defined (clearing them cost every item 32 moves ahead of the branch)
#pragma unroll
                for (int c = 0; c < D / 16; ++c) {
                    if constexpr (F8) asm volatile("" : "=v"(qraw[c]));
                    else asm volatile("" : "=v"(qf[c]));
                }
            }
            if constexpr (DO_ROPE) {
                if (rope) {
                    const long long tbl = ((long long)p.rope_b * b + (long long)p.rope_t * (qtok0 + row0 + (ln < last ? ln : last))) * 2 + lh * 16;
                    const char* crow = reinterpret_cast<const char*>(p.rope_cos) + tbl;
                    const char* srow = reinterpret_cast<const char*>(p.rope_sin) + tbl;
#pragma unroll
                    for (int c = 0; c < NRC; ++c) {
                        rcos[0][c] = as_e16x8(ld16(crow + c * 32));
                        rcos[1][c] = as_e16x8(ld16(crow + (c + NRC) * 32));
                        rsin[0][c] = as_e16x8(ld16(srow + c * 32));
                        rsin[1][c] = as_e16x8(ld16(srow + (c + NRC) * 32));
                    }
                }
            }
        }
        // tile state: index in the walk (earlier-block tiles come first, f < nprev; then the block's
        // own tiles), first token, real keys
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
                asm volatile("" : "+v"(dreg.x), "+v"(dreg.y));   // wait here, not at every later use
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

        f32x16 o[D / 32];
#pragma unroll
        for (int d = 0; d < D / 32; ++d)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[d][v] = 0.f;
        float m_run = -INFINITY, l_run = 0.f, lt_run = 0.f;

        vm_wait_all();
        // tell the compiler the Q fragments are in registers now: otherwise it would put its own
        // "wait for every outstanding load" in front of the first MFMA of each iteration, which would
        // also wait for the next tile's DMA and undo the overlap
        if constexpr (F8) {
            float amax = 0.f;
#pragma unroll
            for (int c = 0; c < D / 16; ++c) {
                asm volatile("" : "+v"(qraw[c]));
                const unsigned w[4] = {qraw[c][0], qraw[c][1], qraw[c][2], qraw[c][3]};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(w[j] << 16)), fabsf(__uint_as_float(w[j] & 0xffff0000u))));
            }
            amax = fmaxf(amax, __shfl_xor(amax, 32));      // the other half of the row's dims
            float q_scale, q_inv;
            br_pow2_scale(amax, q_scale, q_inv);
            sc2 *= q_scale;
#pragma unroll
            for (int c = 0; c < D / 16; ++c) qf[c] = quantize_q8(qraw[c], q_inv);
        }
        if constexpr (DO_ROPE) {
            // out = x cos + rotate_half(x) sin: dim d < D/2 pairs with d + D/2, which the same lane holds D/32 chunks
            // further on; fp32 arithmetic, one rounding (what the stand-alone rotary kernel computes)
            if (rope) {
#pragma unroll
                for (int c = 0; c < NRC; ++c) {
                    e16x8 lo = qf[c], hi = qf[c + NRC];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float x1 = (float)lo[j], x2 = (float)hi[j];
                        const float o1 = x1 * (float)rcos[0][c][j] - x2 * (float)rsin[0][c][j];
                        const float o2 = x2 * (float)rcos[1][c][j] + x1 * (float)rsin[1][c][j];
                        lo[j] = (BR_E16)o1;
                        hi[j] = (BR_E16)o2;
                    }
                    qf[c] = lo;
                    qf[c + NRC] = hi;
                }
            }
        }
#pragma unroll
        for (int c = 0; c < D / 16; ++c) asm volatile("" : "+v"(qf[c]));
        __syncthreads();
        int bufi = 0;

        while (have) {
            // the lane index as a value the compiler cannot trace back: what the rare paths below derive
            // from it (partial tiles, score partials) is computed there, not kept in registers
            int lane_l = lane;
            asm volatile("" : "+v"(lane_l));
            const bool have_next = fetch();
            if (have_next)
                issue_tile(L, wave, lane_l, kbase + (long long)n_tok0 * sk_bytes, vbase + (long long)n_tok0 * sv_bytes, sk_bytes, sv_bytes,
                           n_nvalid, smem_lds + (bufi ^ 1) * SM::stageBytes);
            const char* stage = smem + bufi * SM::stageBytes;

            // 32-key halves of the tile this wave needs: limited by the real keys in the tile and, on
            // the block's own keys, by the diagonal (last row of the wave is row0 + 31).
            // (the tile quantities are handed to the arithmetic below as per-lane values: with scalar ones
            // the compiler's code for the four tile variants needs far more registers than there are)
            int v_nvalid = c_nvalid, v_f = c_f;
            asm volatile("" : "+v"(v_nvalid), "+v"(v_f));
            int nkb = (v_nvalid + 31) >> 5;
            const bool c_self = v_f >= nprev;              // the block's own keys: the causal rule applies
            const int key0 = (v_f - nprev) * BR_BN;        // then: position of the tile's first key in the block
            if (c_self) {
                int vis = row0 + BR_RB - key0;             // keys [0, vis) of the tile are visible to some row
                int c = vis <= 0 ? 0 : (vis + 31) >> 5;
                nkb = c < nkb ? c : nkb;
            }
            if (!rb_active) nkb = 0;
            const bool need_mask = (v_nvalid < nkb * 32) || (c_self && key0 + nkb * 32 - 1 > row0);
            float psum = 0.f;
            // (the exact sum of the probabilities is only kept where something reads it: the log-sum-exp output and
            // the score partials; everything else normalises by the sum of the rounded values alone)
            if (nkb > 0) {
                const int lim_causal = c_self ? row0 + ln - key0 + 1 : BR_BN;   // keys [0, lim) visible
                const int lim = v_nvalid < lim_causal ? v_nvalid : lim_causal;
                bool done = false;
                if constexpr (SC) {
                    int v_exact = exact ? 1 : 0;             // (a per-lane value, like the tile quantities above)
                    asm volatile("" : "+v"(v_exact));
                    if (v_exact != 0) {
                        if (nkb == 2 && !need_mask) compute_tile<2, false, true>(stage, L, qf, o, m_run, l_run, lt_run, sc2, 0, lh, psum);
                        else if (nkb == 2) compute_tile<2, true, true>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lh, psum);
                        else if (need_mask) compute_tile<1, true, true>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lh, psum);
                        else compute_tile<1, false, true>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lh, psum);
                        done = true;
                    }
                }
                if (!done) {
                    if (nkb == 2 && !need_mask) compute_tile<2, false, false>(stage, L, qf, o, m_run, l_run, lt_run, sc2, 0, lh, psum);
                    else if (nkb == 2) compute_tile<2, true, false>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lh, psum);
                    else if (need_mask) compute_tile<1, true, false>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lh, psum);
                    else compute_tile<1, false, false>(stage, L, qf, o, m_run, l_run, lt_run, sc2, lim, lh, psum);
                }
            }
            // Score partials: this tile's probability mass (against the running max) for the query block's
            // last rows, per head - everything the per-document scores need, with no second pass over K.
            if (SC && emit_scores && nkb > 0 && !c_self && c_f >= first_doc_tile) {
                const float tot = psum + __shfl_xor(psum, 32);
                const int ln_l = lane_l & 31;
                const int r16 = it.start_m + row0 + ln_l - (p.H - p.score_R);
                if (lane_l < 32 && r16 >= 0 && row0 + ln_l < len_w) {
                    float2 ms = make_float2(m_run == -INFINITY ? 0.f : m_run, tot);
                    *reinterpret_cast<float2*>(p.score_part + ((((long long)b * p.Nq + head) * p.score_R + r16) * pv.tps + c_f) * 2) = ms;
                }
            }

            if (wave == 0) pf.step();
            vm_wait_all();
            __syncthreads();
            bufi ^= 1;
            c_f = n_f; c_tok0 = n_tok0; c_nvalid = n_nvalid;
            have = have_next;
        }

        // ---- epilogue: lane (ln, lh) holds row row0+ln, dims 32d + 8(v/4) + 4lh + v%4 ----
        // (the lane index is laundered so that the output addresses are computed here, not hoisted
        // to the top of the item where they would have to be spilled across the key loop)
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        const float l_tot = l_run + __shfl_xor(l_run, 32);       // exact sum: log-sum-exp
        const float lt_tot = lt_run + __shfl_xor(lt_run, 32);    // sum of the rounded probabilities: normalises the output
        if (it.slot >= 0) {
            if (row0 + ln < len_w) {
                const long long slot = (long long)it.slot * ge.NHG + hg;
                const long long prow = slot * (NW * BR_RB) + wave * BR_RB + ln;
                float* po = p.part_o + prow * D;
#pragma unroll
                for (int d = 0; d < D / 32; ++d)
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        f32x4 t = {o[d][4 * q4], o[d][4 * q4 + 1], o[d][4 * q4 + 2], o[d][4 * q4 + 3]};
                        *reinterpret_cast<f32x4*>(po + d * 32 + 8 * q4 + 4 * lh) = t;
                    }
                if (lh == 0) {
                    p.part_ml[prow * 2] = m_run;
                    p.part_ml[prow * 2 + 1] = lt_tot;
                    if (SC && p.lse != nullptr) p.part_lx[prow] = l_tot;
                }
            }
        } else {
            // the last loop iteration ended with a barrier, so the K/V buffers are free: transpose
            // through LDS so that every output row is written as full 16-byte pieces
            BR_E16* Es = reinterpret_cast<BR_E16*>(smem + wave * SM::eBytesPerWave);
            const float inv = lt_tot > 0.f ? __builtin_amdgcn_rcpf(lt_tot) : 0.f;
            if (SC && p.lse != nullptr && lane_e < 32 && row0 + lane_e < len_w)
                p.lse[(long long)b * p.lse_b + (long long)head * p.lse_h + qtok0 + row0 + lane_e] = m_run + __builtin_amdgcn_logf(l_tot);
            if (rb_active) {
#pragma unroll
                for (int d = 0; d < D / 32; ++d)
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        f32x4 t = {o[d][4 * q4] * inv, o[d][4 * q4 + 1] * inv, o[d][4 * q4 + 2] * inv,
                                   o[d][4 * q4 + 3] * inv};
                        e16x4 h4 = __builtin_convertvector(t, e16x4);
                        *reinterpret_cast<e16x4*>(Es + ln * SM::eRow + d * 32 + 8 * q4 + 4 * lh) = h4;
                    }
                // same wave wrote and reads: LDS operations of one wave complete in order; the fence
                // keeps the compiler from moving the reads above the writes
                __threadfence_block();
                // lane -> (row rsub of each group of RPI rows, 16-byte piece c8); all reads first, then
                // the stores, whose addresses differ by a uniform step
                constexpr int RPI = 64 / CPR, NIT = BR_RB / RPI;
                const unsigned le = (unsigned)lane_e;
                const unsigned rsub = le / CPR, c8 = le % CPR;
                uint4 vals[NIT];
#pragma unroll
                for (int i = 0; i < NIT; ++i) vals[i] = ld16(Es + (rsub + i * RPI) * SM::eRow + c8 * 8);
                const unsigned long long row_first = (unsigned)(qtok0 + row0);
                char* optr = reinterpret_cast<char*>(p.out) +
                             2 * ((unsigned long long)p.o32_b * (unsigned)b + (unsigned long long)p.o32_h * (unsigned)head +
                                  (unsigned long long)p.o32_t * (row_first + rsub) + c8 * 8);
                const long long stepb = 2LL * RPI * p.o32_t;
                if (row0 + BR_RB <= len_m) {
#pragma unroll
                    for (int i = 0; i < NIT; ++i) *reinterpret_cast<uint4*>(optr + i * stepb) = vals[i];
                } else {
#pragma unroll
                    for (int i = 0; i < NIT; ++i)
                        if (row0 + (int)rsub + i * RPI < len_m) *reinterpret_cast<uint4*>(optr + i * stepb) = vals[i];
                }
            }
        }
        // A document's padded slots get zeros from the item that holds its first query tile (one such item per
        // document and head group; a packed layout has no padded slots).  The prefix's and the query block's
        // are left to the finish kernel: their items are the ones the others wait for.
        if (it.t0 == 0 && m > 0 && m < p.M - 1 && padded_layout)
            zero_padded_rows<D>(p, b, kvh * ge.G + hsub * ge.Gw, ge.G - hsub * ge.Gw < ge.Gw ? ge.G - hsub * ge.Gw : ge.Gw,
                                it.tok_m - it.start_m, it.start_m, len_m, tid, NW * 64);
    }
};

template <int D, int NW, bool F8, bool SC, bool ROPE>
__global__ __launch_bounds__(NW * 64, 2) void br_prefill_mfma_kernel(BrPrefillParams p) {
    // one LDS object, so that it starts at LDS address 0 and every DMA target stays below 64 KiB;
    // the two descriptor mailboxes sit behind the tile stages
    __shared__ __attribute__((aligned(1024))) char smem[Smem<D, F8>::total(NW) + 2 * sizeof(BrDescMail)];
    BrDescMail* mail = reinterpret_cast<BrDescMail*>(smem + Smem<D, F8>::total(NW));
    using PF = Prefill<D, NW, F8, SC, ROPE>;
    using PF16 = Prefill<D, NW, false, SC, ROPE>;
    const int NHG = p.geom.NHG;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, p.geom.tpb * BR_RB);
    int* hdr = const_cast<int*>(p.plan);
    const int wave = uni(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const typename PF::Lane L = PF::make_lane(p, wave, lane);
    // fp8 kernel: the query block's items (the rows the document scores are read from, and the single block of a
    // sequence without documents) run on the bf16 Q and K, every other item on the e4m3 copies
    typename PF16::Lane L16;
    if constexpr (F8) {
        // only the K pieces differ between the two element types: the V offsets are shared registers
        const typename PF16::Lane t = PF16::make_lane(p, wave, lane);
#pragma unroll
        for (int j = 0; j < PF16::JOK; ++j) L16.koff[j] = t.koff[j];
        L16.krd = t.krd;
#pragma unroll
        for (int j = 0; j < PF16::JO; ++j) L16.voff[j] = L.voff[j];
#pragma unroll
        for (int d = 0; d < D / 32; ++d) L16.vrd[d] = L.vrd[d];
    }
    // DMA pieces of partial tiles are skipped, so whatever sits in LDS must be finite: start from zero
    for (int i = threadIdx.x * 16; i < Smem<D, F8>::total(NW); i += NW * 64 * 16) *reinterpret_cast<uint4*>(smem + i) = uint4{0u, 0u, 0u, 0u};
    const bool padded_layout = uni(hdr[BR_PH_PACKED]) == 0;
    BrPrefetch pf;
    pf.init(hdr, &pv, NHG, lane);
    if (wave == 0) pf.publish(&mail[0]);
    __syncthreads();
    for (int cur = 0;; cur ^= 1) {
        // one LDS read per lane (lane i: word i of the mailbox), then the words are taken from the lanes
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
        if constexpr (F8) {
            if (it.m == p.M - 1) PF16::run_item(p, pv, it, hg, smem, L16, pf, padded_layout);
            else PF::run_item(p, pv, it, hg, smem, L, pf, padded_layout);
        } else {
            PF::run_item(p, pv, it, hg, smem, L, pf, padded_layout);
        }
        if (wave == 0) pf.publish(&mail[cur ^ 1]);
        __syncthreads();
    }
    if (threadIdx.x == 0) br_leave(hdr);
}

// Finish: (1) merge the split-KV partials of the query block,
// out = sum_s O_s 2^(m_s - m) / sum_s l_s 2^(m_s - m); one workgroup per (query tile, head group, row
// block); (2) set the rows of padded token slots to zero.
// THREADS: workgroup size.  PATH >= 0 (with score_wgs > 0): the first score_wgs workgroups (one per sequence) turn
// the score partials the prefill kernel left into per-document scores instead (sp, reduction PATH of
// br_doc_final_tiles_body with sp_waves accumulator rows of LDS), the others share the merge as if they were the
// whole grid.  PATH < 0: the merge alone.
template <int D, int THREADS, int PATH>
__global__ __launch_bounds__(THREADS) void br_finish_kernel(BrPrefillParams p, int NW, BrTileScoreParams sp, int score_wgs, int sp_waves) {
    if constexpr (PATH >= 0) {
        extern __shared__ float br_finish_dyn[];
        if ((int)blockIdx.x < score_wgs) {
            br_doc_final_tiles_body<PATH>(sp, blockIdx.x, br_finish_dyn, sp_waves);
            return;
        }
    } else {
        score_wgs = 0;
    }
    const int bid = blockIdx.x - score_wgs, nblk = gridDim.x - score_wgs;
    const BrGeom& ge = p.geom;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, ge.tpb * BR_RB);
    constexpr int CPR = D / 4;                    // float4 chunks per row = threads per row
    constexpr int RPW = THREADS / CPR;            // rows one workgroup merges at a time
    const int rows = NW * BR_RB;                  // rows of one (combine entry, head group): NW query-tile waves of 32
    const int subs = (rows + RPW - 1) / RPW;      // such row groups
    const int n_units = pv.hdr[BR_PH_NCOMB] * ge.NHG * subs;
    const BrComb* combs = pv.comb;
    const int m = p.M - 1;
    const int rr = threadIdx.x / CPR, cc = threadIdx.x % CPR;
    for (int u = bid; u < n_units; u += nblk) {
        const int subu = u % subs;
        const int w = u / subs;
        const int ci = w / ge.NHG, hg = w - ci * ge.NHG;
        const int r = subu * RPW + rr;                               // row inside the slot
        if (r >= rows) continue;
        const int wave = r / BR_RB, rloc = r - wave * BR_RB;         // the prefill wave that owned it, row of its 32
        const BrComb c = combs[ci];
        const int kvh = hg / ge.HGS, hsub = hg - kvh * ge.HGS;
        const int len_m = pv.len[c.b * p.M + m];
        const int qtok0 = pv.tok[c.b * p.M + m];
        const int g = wave / ge.tpb, sub = wave - g * ge.tpb;
        const int row = c.t0 + sub * BR_RB + rloc;
        if (row >= len_m || hsub * ge.Gw + g >= ge.G) continue;     // (the second: a wave without a head, ragged group)
        const int head = kvh * ge.G + hsub * ge.Gw + g;
        const long long slot0 = (long long)c.slot0 * ge.NHG + hg;
        const long long sstride = (long long)ge.NHG * rows;          // rows between consecutive splits
        const float2* ml = reinterpret_cast<const float2*>(p.part_ml) + slot0 * rows + r;
        const float* lx = p.part_lx + slot0 * rows + r;
        const bool want_lse = p.lse != nullptr && cc == 0;
        const float* po = p.part_o + (slot0 * rows + r) * D + cc * 4;
        // all loads of up to eight splits are in flight together; a thread owns one float4 of the row
        float mmax = -INFINITY, l = 0.f, lex = 0.f;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int s0 = 0; s0 < c.nsplit; s0 += 8) {
            float2 mls[8];
            float lxs[8];
            f32x4 ov[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const bool on = s0 + j < c.nsplit;
                mls[j] = on ? ml[(s0 + j) * sstride] : make_float2(-INFINITY, 0.f);
                ov[j] = on ? *reinterpret_cast<const f32x4*>(po + (s0 + j) * sstride * D) : f32x4{0.f, 0.f, 0.f, 0.f};
                lxs[j] = (on && want_lse) ? lx[(s0 + j) * sstride] : 0.f;
            }
            float mnew = mmax;
#pragma unroll
            for (int j = 0; j < 8; ++j) mnew = fmaxf(mnew, mls[j].x);
            const float resc = mmax == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mmax - mnew);
            l *= resc;
            lex *= resc;
            acc *= resc;
            mmax = mnew;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float w8 = mls[j].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mls[j].x - mmax);
                l += mls[j].y * w8;
                lex += lxs[j] * w8;
                acc += ov[j] * w8;
            }
        }
        const float inv = l > 0.f ? 1.f / l : 0.f;
        // (the log-sum-exp from the exact sums, as the rows the prefill kernel finishes itself get it)
        if (want_lse) p.lse[(long long)c.b * p.lse_b + (long long)head * p.lse_h + qtok0 + row] = mmax + __builtin_amdgcn_logf(lex);
        BR_E16* dst = reinterpret_cast<BR_E16*>(p.out) + (long long)c.b * p.so_b + (long long)head * p.so_h +
                      (long long)(qtok0 + row) * p.so_t;
        e16x4 h4 = __builtin_convertvector(acc * inv, e16x4);
        *reinterpret_cast<e16x4*>(dst + cc * 4) = h4;
    }
    // Padded token slots: no kernel computes them, so give them a defined value (zero).  The prefill kernel
    // does that for the documents it has items for; what is left here are the prefix, the query block and
    // documents with no real token at all (a packed layout has no padded slots).
    // One (block, head) per wave and step: the loop is a chain of dependent loads (block table, then the stores'
    // addresses), so what counts is how many of them are in flight.
    const int n_pad_work = pv.hdr[BR_PH_PACKED] ? 0 : p.B * p.M * p.Nq;
    constexpr int WAVES = THREADS / 64;
    const int lane = threadIdx.x & 63;
    for (int w = bid * WAVES + (threadIdx.x >> 6); w < n_pad_work; w += nblk * WAVES) {
        const int bm = w / p.Nq, head = w - bm * p.Nq;
        const int b = bm / p.M, mm = bm - b * p.M;
        const int st = pv.start[bm], ln = pv.len[bm];
        if (ln != 0 && mm > 0 && mm < p.M - 1) continue;
        const int npad = p.H - ln;
        constexpr int CP8 = D / 8;
        BR_E16* obase = reinterpret_cast<BR_E16*>(p.out) + (long long)b * p.so_b + (long long)head * p.so_h;
        for (int idx = lane; idx < npad * CP8; idx += 64) {
            int r = idx / CP8, c8 = idx - r * CP8;
            int pos = r < st ? r : r + ln;
            uint4 z = {0u, 0u, 0u, 0u};
            *reinterpret_cast<uint4*>(obase + (long long)(mm * p.H + pos) * p.so_t + c8 * 8) = z;
        }
    }
}

// Launch of the finish kernel after a prefill kernel.  sp: the per-document score reduction to run in the same
// launch (its partials are those the prefill kernel just wrote), or nullptr.  Returns 1 when the reduction's
// accumulator rows do not fit the LDS (too many documents), with nothing launched.
template <int D>
inline int br_launch_finish(const BrPrefillParams& p, int NW, int combine_grid, const BrTileScoreParams* sp, hipStream_t stream) {
    BrTileScoreParams none = {};
    if (!sp) {
        hipLaunchKernelGGL((br_finish_kernel<D, 256, -1>), dim3(combine_grid), dim3(256), 0, stream, p, NW, none, 0, 0);
        return 0;
    }
    const int docs = sp->M - 2;
    const int path = br_doc_final_path(docs, sp->H);
    int nwaves = path == 0 ? 16 : 8;
    while (nwaves > 1 && (size_t)nwaves * docs * sizeof(float) > 48 * 1024) nwaves >>= 1;
    const size_t lds = (size_t)nwaves * docs * sizeof(float);
    if (lds > 60 * 1024) return 1;
    const int grid = sp->B + (path == 0 ? (combine_grid + 3) / 4 : (combine_grid + 1) / 2);
    if (path == 0)
        hipLaunchKernelGGL((br_finish_kernel<D, 1024, 0>), dim3(grid), dim3(1024), lds, stream, p, NW, *sp, sp->B, nwaves);
    else if (path == 1)
        hipLaunchKernelGGL((br_finish_kernel<D, 512, 1>), dim3(grid), dim3(512), lds, stream, p, NW, *sp, sp->B, nwaves);
    else
        hipLaunchKernelGGL((br_finish_kernel<D, 512, 2>), dim3(grid), dim3(512), lds, stream, p, NW, *sp, sp->B, nwaves);
    return 0;
}

}  // namespace
