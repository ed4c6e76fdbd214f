// Backward of the block-sparse prefill attention for gfx950 (bf16 inputs, fp32 arithmetic and accumulation).
//
// The reference has no hand-written backward: its trainable hooks (blockrank_std_attention.py:96-262, :472-650,
// used by trainer.py:79-101) are differentiated by torch autograd over dense masked tensors, and its Triton
// hook refuses (blockrank_triton_kernel_attention.py:759-761).  This kernel computes the same gradients
//     P = softmax(S),  dV = P^T dO,  dP = dO V^T,  dS = P * (dP - rowsum(dO * O)),
//     dQ = scale * dS K,  dK = scale * dS^T Q        (dK, dV summed over the query heads of a kv head)
// over exactly the (query tile, key tile) pairs the forward visits: it walks the forward's own work items
// (view 0 of the request plan), one workgroup per (item, head group), a wave per 32 rows of one query head.
// P is rebuilt from the log-sum-exp the forward saved, so an item needs nothing from the items that share
// its rows (the query block's key walk is split over several).
//
// Per wave and 64-key tile (K, V tile staged in LDS by the whole workgroup):
//   S^T = K Q^T, dP^T = V dO^T     accumulators: lane = query row, registers = keys
//        -> dS^T (bf16) is directly the A operand of   dQ += dS K      (K read with transposing LDS reads)
//   S = Q K^T, dP = dO V^T         the same products with the operands exchanged: lane = key, registers = rows
//        -> P, dS (bf16) are directly the A operands of dV += P^T dO,  dK += dS^T Q
//           (dO and Q as "lane = dim, registers = rows" operands, transposed once per item through LDS)
// Recomputing S and dP in the second orientation costs 32 of the 112 MFMAs per tile and saves moving P
// and dS through LDS.
// dQ stays in registers over the item's walk; dK and dV contributions of a tile leave as fp32 atomic adds
// into accumulation buffers (several items and the heads of a group add to the same key rows), and so
// does dQ at the end of the item.  A last kernel converts the three buffers to bf16 tensors.
#include "br_common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

}  // namespace


namespace {

__device__ inline uint4 ld16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline bf16x8 as_bf16x8(uint4 u) {
    union { uint4 u; bf16x8 v; } c;
    c.u = u;
    return c.v;
}
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
    static constexpr int RS = 2 * D + 16;          // LDS row stride in bytes (16 bytes of padding spread the banks)
    static constexpr int CPR = D / 8;              // 16-byte pieces per row
    static constexpr int NC = D / 16, ND = D / 32;
    static constexpr int tileBytes = BR_BN * RS;
    static constexpr int waveBytes = BR_RB * RS;
    static constexpr int ldsBytes(int nw) { return 2 * tileBytes + nw * waveBytes; }

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

    static __device__ void run_item(const BrBwdParams& p, const BrPlanView& pv, const BrItem& it, int hg, char* smem, int NW) {
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
        char* Ws = smem + 2 * tileBytes + wave * waveBytes;
        const char* kbase = reinterpret_cast<const char*>(p.k) + 2 * ((unsigned long long)p.k32_b * (unsigned)b + (unsigned long long)p.k32_h * (unsigned)kvh);
        const char* vbase = reinterpret_cast<const char*>(p.v) + 2 * ((unsigned long long)p.v32_b * (unsigned)b + (unsigned long long)p.v32_h * (unsigned)kvh);

        // ---- per item: Q and dO of this wave's rows in both operand layouts, the rows' log-sum-exp and
        // delta = rowsum(dO * O) ----
        bf16x8 qf[NC], dof[NC];        // lane = row, registers = dims
        bf16x8 qt[ND][2], dot[ND][2];  // lane = dim, registers = rows
        float lse_l = 0.f, delta_l = 0.f;          // of row row0 + ln
        float lse_r[16], delta_r[16];              // of row row0 + 8 (v / 4) + 4 lh + v % 4
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
            lse_l = p.lse[(long long)b * p.lse_b + (long long)head * p.lse_h + tok];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = 8 * (v >> 2) + 4 * lh + (v & 3);
                lse_r[v] = __shfl(lse_l, i);
                delta_r[v] = __shfl(delta_l, i);
            }
            // transposed operands through the wave's own LDS rows (a wave's LDS operations complete in order)
#pragma unroll
            for (int c = 0; c < NC; ++c) *reinterpret_cast<bf16x8*>(Ws + ln * RS + c * 32 + lh * 16) = qf[c];
            __threadfence_block();
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int s = 0; s < 2; ++s) qt[db][s] = read_col(Ws, 16 * s, db, lane);
            __threadfence_block();
#pragma unroll
            for (int c = 0; c < NC; ++c) *reinterpret_cast<bf16x8*>(Ws + ln * RS + c * 32 + lh * 16) = dof[c];
            __threadfence_block();
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int s = 0; s < 2; ++s) dot[db][s] = read_col(Ws, 16 * s, db, lane);
        } else {
#pragma unroll
            for (int c = 0; c < NC; ++c) qf[c] = dof[c] = as_bf16x8(uint4{0u, 0u, 0u, 0u});
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int s = 0; s < 2; ++s) qt[db][s] = dot[db][s] = as_bf16x8(uint4{0u, 0u, 0u, 0u});
#pragma unroll
            for (int v = 0; v < 16; ++v) lse_r[v] = delta_r[v] = 0.f;
        }

        f32x16 dq[ND];
#pragma unroll
        for (int db = 0; db < ND; ++db) dq[db] = zero16();

        // ---- the item's key walk: the earlier blocks' tiles it covers, then its own block's up to the diagonal ----
        const int2* tiles_b = pv.tiles + (size_t)b * pv.tps;
        const bool table = it.pe > 1;
        const int nprev = it.nprev;
        const int f_end = it.ntiles > 0x3fffffff ? 0x7fffffff : it.f_lo + it.ntiles;
        const long long slot_b = (long long)b * p.acc_b;
        for (int f = it.f_lo; f < f_end; ++f) {
            const bool self = f >= nprev;
            int tok0, nvalid, key0 = 0;
            if (!self) {
                if (table) {
                    const int2 d = tiles_b[f];
                    tok0 = d.x;
                    nvalid = d.y;
                } else {
                    tok0 = it.tok0 + f * BR_BN;
                    nvalid = it.len0 - f * BR_BN < BR_BN ? it.len0 - f * BR_BN : BR_BN;
                }
            } else {
                key0 = (f - nprev) * BR_BN;
                if (key0 >= self_end) break;
                tok0 = it.tok_m + key0;
                nvalid = self_end - key0 < BR_BN ? self_end - key0 : BR_BN;
            }
            if (nvalid <= 0) continue;
            // stage the tile: rows past its real keys are zero
            __syncthreads();                       // every wave has finished with the previous tile
            for (int idx = tid; idx < BR_BN * CPR; idx += NT) {
                const int r = idx / CPR, c = idx - r * CPR;
                uint4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
                if (r < nvalid) {
                    kk = ld16(kbase + 2 * ((long long)(tok0 + r) * p.k32_t + c * 8));
                    vv = ld16(vbase + 2 * ((long long)(tok0 + r) * p.v32_t + c * 8));
                }
                *reinterpret_cast<uint4*>(Ks + r * RS + c * 16) = kk;
                *reinterpret_cast<uint4*>(Vs + r * RS + c * 16) = vv;
            }
            __syncthreads();

            // 32-key halves this wave needs: limited by the real keys and, on the block's own keys, by the diagonal
            int nkb = (nvalid + 31) >> 5;
            if (self) {
                const int vis = row0 + BR_RB - key0;
                const int c = vis <= 0 ? 0 : (vis + 31) >> 5;
                nkb = c < nkb ? c : nkb;
            }
            if (!rb_active) nkb = 0;
            for (int kb = 0; kb < nkb; ++kb) {
                // -- lane = query row: dS^T, then dQ += dS K --
                {
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
                        const float pr = __builtin_amdgcn_exp2f(st[v] * p.scale_log2 - lse_l);
                        st[v] = key < lim ? pr * (dpt[v] - delta_l) * p.scale : 0.f;
                    }
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        const bf16x8 a = pack8(st, s);
#pragma unroll
                        for (int db = 0; db < ND; ++db) dq[db] = mma(a, read_col(Ks, kb * 32 + 16 * s, db, lane), dq[db]);
                    }
                }
                // -- lane = key: P and dS, then dV += P^T dO and dK += dS^T Q for this half's 32 keys --
                {
                    f32x16 sn = zero16(), dpn = zero16();
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        sn = mma(qf[c], read_row(Ks, kb * 32, c, ln, lh), sn);
                        dpn = mma(dof[c], read_row(Vs, kb * 32, c, ln, lh), dpn);
                    }
                    const int key = kb * 32 + ln;
                    const bool key_ok = key < nvalid;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int row = row0 + 8 * (v >> 2) + 4 * lh + (v & 3);
                        const bool vis = key_ok && row < len_m && (!self || key0 + key <= row);
                        const float pr = vis ? __builtin_amdgcn_exp2f(sn[v] * p.scale_log2 - lse_r[v]) : 0.f;
                        sn[v] = pr;
                        dpn[v] = vis ? pr * (dpn[v] - delta_r[v]) * p.scale : 0.f;
                    }
                    const bf16x8 p0 = pack8(sn, 0), p1 = pack8(sn, 1), d0 = pack8(dpn, 0), d1 = pack8(dpn, 1);
                    // accumulator: lane = dim 32 db + ln, register v = key kb*32 + 8 (v/4) + 4 lh + v%4
                    const long long rowk = slot_b + tok0 + kb * 32 + 4 * lh;
#pragma unroll
                    for (int db = 0; db < ND; ++db) {
                        f32x16 av = mma(p0, dot[db][0], zero16());
                        av = mma(p1, dot[db][1], av);
                        f32x16 ak = mma(d0, qt[db][0], zero16());
                        ak = mma(d1, qt[db][1], ak);
                        float* dvp = p.dv32 + (rowk * p.Nkv + kvh) * D + db * 32 + ln;
                        float* dkp = p.dk32 + (rowk * p.Nkv + kvh) * D + db * 32 + ln;
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int kr = 8 * (v >> 2) + (v & 3);                       // key row minus 4 lh
                            if (kb * 32 + 4 * lh + kr < nvalid) {
                                unsafeAtomicAdd(dvp + (long long)kr * p.Nkv * D, av[v]);
                                unsafeAtomicAdd(dkp + (long long)kr * p.Nkv * D, ak[v]);
                            }
                        }
                    }
                }
            }
        }
        // ---- dQ of this wave's rows: lane = dim 32 db + ln, register v = row 8 (v/4) + 4 lh + v%4 ----
        if (rb_active) {
            float* dqp = p.dq32 + ((slot_b + qtok0 + row0 + 4 * lh) * p.Nq + head) * D + ln;
#pragma unroll
            for (int db = 0; db < ND; ++db)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = 8 * (v >> 2) + (v & 3);
                    if (row0 + 4 * lh + r < len_m) unsafeAtomicAdd(dqp + (long long)r * p.Nq * D + db * 32, dq[db][v]);
                }
        }
    }
};

template <int D, int MAXW>
__global__ __launch_bounds__(MAXW * 64, 1) void br_bwd_kernel(BrBwdParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const BrGeom& ge = p.geom;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, ge.tpb * BR_RB);
    const int item = blockIdx.x / ge.NHG, hg = blockIdx.x - item * ge.NHG;
    if (item >= pv.hdr[BR_PH_QOFF2 + BR_GLOBAL_QUEUE]) return;      // view 0's items come first in the array; view 1 starts here
    const BrItem it = pv.items[item];
    Bwd<D>::run_item(p, pv, it, hg, smem, blockDim.x >> 6);
}

__global__ __launch_bounds__(256) void br_fill_zero_kernel(uint4* p, size_t n16) {
    const uint4 z = {0u, 0u, 0u, 0u};
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) p[i] = z;
}

// fp32 accumulation buffer [slot][heads][D] -> bf16 tensor with (batch, head, token) strides; slots of padded
// tokens were never added to and come out as zeros.
__global__ __launch_bounds__(256) void br_bwd_store_kernel(const float* acc, __bf16* dst, long long n_slots, long long slots_per_b, int heads,
                                                           int D, long long s_b, long long s_h, long long s_t) {
    const int c4 = D / 4;
    const long long n = n_slots * heads * c4;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const long long row = i / c4;
        const int c = (int)(i - row * c4);
        const long long slot = row / heads;
        const int h = (int)(row - slot * heads);
        const long long b = slots_per_b > 0 ? slot / slots_per_b : 0, t = slots_per_b > 0 ? slot - b * slots_per_b : slot;
        const float4 x = *reinterpret_cast<const float4*>(acc + row * D + c * 4);
        typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const f32x4 f = {x.x, x.y, x.z, x.w};
        *reinterpret_cast<bf16x4*>(dst + b * s_b + h * s_h + t * s_t + c * 4) = __builtin_convertvector(f, bf16x4);
    }
}

template <int D, int MAXW>
int launch_bwd(const BrBwdParams& p, int NW, hipStream_t stream) {
    const int lds = Bwd<D>::ldsBytes(NW);
    static int armed = 0;          // largest dynamic LDS size this instance has been enabled for
    if (lds > armed) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&br_bwd_kernel<D, MAXW>), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
            return -2;
        armed = lds;
    }
    hipLaunchKernelGGL((br_bwd_kernel<D, MAXW>), dim3(p.max_items * p.geom.NHG), dim3(NW * 64), lds, stream, p);
    return 0;
}

}  // namespace

// dq/dk/dv: bf16 tensors with (batch, head, token) element strides.  n_slots = token slots in total
// (B * M * H padded, or the packed token count), slots_per_b = M * H for a padded layout, 0 for a packed one.
// Returns 0 on success, -1 if D has no instance, -2 if the kernel's LDS size could not be set.
int br_launch_bwd(const BrBwdParams& p, int D, int NW, int n_cu, void* dq, void* dk, void* dv, const long long* sdq, const long long* sdk,
                  const long long* sdv, long long n_slots, long long slots_per_b, hipStream_t stream) {
    const size_t n16 = (size_t)n_slots * (p.Nq + 2 * p.Nkv) * D / 4;          // the three buffers are contiguous
    hipLaunchKernelGGL(br_fill_zero_kernel, dim3(n_cu * 8), dim3(256), 0, stream, reinterpret_cast<uint4*>(p.dq32), n16);
    int rc;
    if (D == 128) rc = NW <= 4 ? launch_bwd<128, 4>(p, NW, stream) : launch_bwd<128, 8>(p, NW, stream);
    else if (D == 64) rc = NW <= 4 ? launch_bwd<64, 4>(p, NW, stream) : launch_bwd<64, 8>(p, NW, stream);
    else return -1;
    if (rc) return rc;
    const int grid = n_cu * 8;
    hipLaunchKernelGGL(br_bwd_store_kernel, dim3(grid), dim3(256), 0, stream, p.dq32, static_cast<__bf16*>(dq), n_slots, slots_per_b, p.Nq, D,
                       sdq[0], sdq[1], sdq[2]);
    hipLaunchKernelGGL(br_bwd_store_kernel, dim3(grid), dim3(256), 0, stream, p.dk32, static_cast<__bf16*>(dk), n_slots, slots_per_b, p.Nkv, D,
                       sdk[0], sdk[1], sdk[2]);
    hipLaunchKernelGGL(br_bwd_store_kernel, dim3(grid), dim3(256), 0, stream, p.dv32, static_cast<__bf16*>(dv), n_slots, slots_per_b, p.Nkv, D,
                       sdv[0], sdv[1], sdv[2]);
    return 0;
}
