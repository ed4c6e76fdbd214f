// Block-sparse prefill attention for fp32 inputs: same plan, same tile walk and same row mapping as
// the bf16 MFMA kernel, all arithmetic in fp32 on the vector ALU (an fp32 model is a parity
// configuration, not a throughput one, and 1e-5 agreement with an fp32 reference rules out 16-bit
// products).  Two adjacent lanes share one query row, each owning half of the head dimension: the
// dot product is finished with one lane exchange and each lane accumulates its half of the output.
//
// Reference semantics: sdpa_blockrank_attention_forward, blockrank_std_attention.py:503-650.
#include "br_common.h"

namespace {

template <int D, int NW>
__global__ __launch_bounds__(NW * 64) void br_prefill_f32_kernel(BrPrefillParams p) {
    constexpr int NT = NW * 64;
    constexpr int HD = D / 2;
    __shared__ __attribute__((aligned(16))) float Ks[BR_BN * D];
    __shared__ __attribute__((aligned(16))) float Vs[BR_BN * D];
    __shared__ int s_next;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, n = lane >> 1, half = lane & 1;
    const BrGeom& ge = p.geom;
    const int T = ge.tpb * BR_RB;
    const int NHG = ge.NHG;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, T);
    int* hdr = const_cast<int*>(p.plan);
    const float* Q = reinterpret_cast<const float*>(p.q);
    const float* K = reinterpret_cast<const float*>(p.k);
    const float* V = reinterpret_cast<const float*>(p.v);
    float* O = reinterpret_cast<float*>(p.out);

    const int xcc = br_xcc_id();
    int qk = 0;
    for (;;) {
        if (tid == 0) s_next = br_take_ticket(hdr, NHG, xcc, &qk, -1);
        __syncthreads();
        const int qt = __builtin_amdgcn_readfirstlane(s_next);
        __syncthreads();
        if (qt < 0) break;
        int item, hg;
        br_decode_ticket(pv, qt, NHG, item, hg);
        const BrItem it = pv.items[item];
        const int b = it.b, m = it.m;
        const int kvh = hg / ge.HGS, hsub = hg - kvh * ge.HGS;
        const int g = wave / ge.tpb, sub = wave - g * ge.tpb;
        const int head = kvh * ge.G + hsub * ge.Gw + g;
        const int len_m = it.len_m;
        const int row = it.t0 + sub * BR_RB + n;           // this lane pair's query row, valid-relative
        const bool row_ok = row < len_m;
        const int self_end = it.t0 + T < len_m ? it.t0 + T : len_m;
        const int qtok0 = it.tok_m;

        float q[HD], o[HD];
        {
            const float* qp = Q + (long long)b * p.sq_b + (long long)head * p.sq_h + (long long)(qtok0 + row) * p.sq_t + half * HD;
#pragma unroll
            for (int d = 0; d < HD; ++d) {
                q[d] = row_ok ? qp[d] : 0.f;
                o[d] = 0.f;
            }
        }
        float m_run = -INFINITY, l_run = 0.f;
        const float* kbase = K + (long long)b * p.sk_b + (long long)kvh * p.sk_h;
        const float* vbase = V + (long long)b * p.sv_b + (long long)kvh * p.sv_h;

        BrWalk walk;
        walk.init(it, self_end, p.H);
        const int2* tiles_b = pv.tiles + (size_t)b * pv.tps;
        BrTile t;
        for (;;) {
            int pi = 0;
            const int wr = walk.next(t, &pi);
            if (wr == 0) break;
            if (wr == 1) {
                if (it.pe > 1) {
                    const int2 d = tiles_b[pi];
                    t.tok0 = d.x; t.nvalid = d.y; t.kt = 0; t.self = 0;
                } else {
                    br_prefix_tile(it, pi, t);
                }
            }
            const int tok0 = t.tok0;
            __syncthreads();   // previous tile fully consumed
            for (int ch = tid; ch < BR_BN * (D / 4); ch += NT) {
                int r = ch / (D / 4), c4 = ch - r * (D / 4);
                float4 kz = {0.f, 0.f, 0.f, 0.f}, vz = kz;
                if (r < t.nvalid) {
                    kz = *reinterpret_cast<const float4*>(kbase + (long long)(tok0 + r) * p.sk_t + c4 * 4);
                    vz = *reinterpret_cast<const float4*>(vbase + (long long)(tok0 + r) * p.sv_t + c4 * 4);
                }
                *reinterpret_cast<float4*>(&Ks[r * D + c4 * 4]) = kz;
                *reinterpret_cast<float4*>(&Vs[r * D + c4 * 4]) = vz;
            }
            __syncthreads();
            const int key0 = t.kt * BR_BN;
            int lim = t.nvalid;
            if (t.self) {
                int c = row - key0 + 1;                    // keys [0, c) of the tile are at or before the row
                lim = c < lim ? c : lim;
            }
            // every lane runs the same trip count (the exchange below needs both lanes of a pair, and
            // a pair always agrees on lim); rows that see nothing in this tile run zero iterations
            for (int j = 0; j < lim; ++j) {
                const float* kr = &Ks[j * D + half * HD];
                float s = 0.f;
#pragma unroll
                for (int d = 0; d < HD; ++d) s = fmaf(q[d], kr[d], s);
                s += __shfl_xor(s, 1);
                s *= p.scale_log2;
                const float m_new = fmaxf(m_run, s);
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                const float e = __builtin_amdgcn_exp2f(s - m_new);
                l_run = l_run * alpha + e;
                m_run = m_new;
                const float* vr = &Vs[j * D + half * HD];
#pragma unroll
                for (int d = 0; d < HD; ++d) o[d] = fmaf(o[d], alpha, e * vr[d]);
            }
        }

        if (row_ok) {
            if (it.slot >= 0) {
                const long long slot = (long long)it.slot * ge.NHG + hg;
                const long long prow = slot * (NW * BR_RB) + wave * BR_RB + n;
                float* po = p.part_o + prow * D + half * HD;
#pragma unroll
                for (int d = 0; d < HD; ++d) po[d] = o[d];
                if (half == 0) {
                    p.part_ml[prow * 2] = m_run;
                    p.part_ml[prow * 2 + 1] = l_run;
                }
            } else {
                const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
                float* op = O + (long long)b * p.so_b + (long long)head * p.so_h + (long long)(qtok0 + row) * p.so_t + half * HD;
#pragma unroll
                for (int d = 0; d < HD; ++d) op[d] = o[d] * inv;
            }
        }
    }
    if (tid == 0) br_leave(hdr);
}

template <int D>
__global__ __launch_bounds__(256) void br_combine_f32_kernel(BrPrefillParams p, int NW) {
    const BrGeom& ge = p.geom;
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, ge.tpb * BR_RB);
    const int n_work = pv.hdr[BR_PH_NCOMB] * ge.NHG;
    const int m = p.M - 1;
    float* O = reinterpret_cast<float*>(p.out);
    for (int w = blockIdx.x; w < n_work; w += gridDim.x) {
        const int ci = w / ge.NHG, hg = w - ci * ge.NHG;
        const BrComb c = pv.comb[ci];
        const int kvh = hg / ge.HGS, hsub = hg - kvh * ge.HGS;
        const int len_m = pv.len[c.b * p.M + m];
        const int qtok0 = pv.tok[c.b * p.M + m];
        const int rows = NW * BR_RB;
        for (int idx = threadIdx.x; idx < rows * D; idx += blockDim.x) {
            const int r = idx / D, d = idx - r * D;
            const int wave = r >> 5, n = r & 31;
            const int g = wave / ge.tpb, sub = wave - g * ge.tpb;
            const int row = c.t0 + sub * BR_RB + n;
            if (row >= len_m) continue;
            const int head = kvh * ge.G + hsub * ge.Gw + g;
            float mmax = -INFINITY;
            for (int s = 0; s < c.nsplit; ++s) {
                const long long slot = (long long)(c.slot0 + s) * ge.NHG + hg;
                mmax = fmaxf(mmax, p.part_ml[(slot * rows + r) * 2]);
            }
            float l = 0.f, acc = 0.f;
            for (int s = 0; s < c.nsplit; ++s) {
                const long long slot = (long long)(c.slot0 + s) * ge.NHG + hg;
                const long long prow = slot * rows + r;
                const float ms = p.part_ml[prow * 2];
                const float w8 = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - mmax);
                l += p.part_ml[prow * 2 + 1] * w8;
                acc += p.part_o[prow * D + d] * w8;
            }
            O[(long long)c.b * p.so_b + (long long)head * p.so_h + (long long)(qtok0 + row) * p.so_t + d] = l > 0.f ? acc / l : 0.f;
        }
    }
    // padded token slots: the kernels never touch them, so give them a defined value (zero)
    const int n_pad_work = pv.hdr[BR_PH_PACKED] ? 0 : p.B * p.M * p.Nq;
    for (int w = blockIdx.x; w < n_pad_work; w += gridDim.x) {
        const int bm = w / p.Nq, head = w - bm * p.Nq;
        const int b = bm / p.M, mm = bm - b * p.M;
        const int st = pv.start[bm], ln = pv.len[bm];
        const int npad = p.H - ln;
        float* obase = O + (long long)b * p.so_b + (long long)head * p.so_h;
        for (int idx = threadIdx.x; idx < npad * D; idx += blockDim.x) {
            int r = idx / D, d = idx - r * D;
            int pos = r < st ? r : r + ln;
            obase[(long long)(mm * p.H + pos) * p.so_t + d] = 0.f;
        }
    }
}

}  // namespace

int br_launch_prefill_f32(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                           hipEvent_t ev_start, hipEvent_t ev_stop) {
    const int grid = n_cu;
    if (ev_start) (void)hipEventRecord(ev_start, stream);
#define BR_CASE(DD, WW)                                                                                        \
    if (D == DD && NW == WW) {                                                                                 \
        hipLaunchKernelGGL((br_prefill_f32_kernel<DD, WW>), dim3(grid), dim3(WW * 64), 0, stream, p);          \
        goto launched;                                                                                         \
    }
    BR_CASE(128, 4) BR_CASE(128, 5) BR_CASE(128, 6) BR_CASE(128, 7) BR_CASE(128, 8)
    BR_CASE(64, 4) BR_CASE(64, 5) BR_CASE(64, 6) BR_CASE(64, 7) BR_CASE(64, 8)
#undef BR_CASE
    return -1;
launched:
    if (ev_stop) (void)hipEventRecord(ev_stop, stream);
    if (D == 128)
        hipLaunchKernelGGL((br_combine_f32_kernel<128>), dim3(combine_grid), dim3(256), 0, stream, p, NW);
    else
        hipLaunchKernelGGL((br_combine_f32_kernel<64>), dim3(combine_grid), dim3(256), 0, stream, p, NW);
    return 0;
}
