// Per-document scores from the per-tile score partials of the prefill kernel: the parameter block and the
// workgroup-level reduction, shared by the stand-alone kernel (br_scores.hip) and the kernel that runs it next to
// the merge of the prefill kernel's split partials (br_prefill_mfma_impl.h).
#pragma once
#include "br_common.h"

// Per-document scores from the per-tile partials the prefill kernel leaves for the query block's last
// Rw rows: part[b][n][r][tile] = (max, sum of 2^(logit - max)) over that tile's real keys, tiles in the
// order of the sequence's tile descriptors (document d owns tiles tbase[d+1] .. + ceil(len/64)).
// One workgroup per sequence; every wave takes (head, row) pairs round robin, a lane takes a
// document: joint normalisation over all documents, then the per-document sums are added into the
// wave's own accumulator row in LDS; the rows are added up in a fixed order at the end.
struct BrTileScoreParams {
    const float* part;
    const int* plan;
    const int* rows;        // (B, R) indices into the last Rw positions of the query block
    float* scores;          // (B, docs)
    float* probs;           // optional (B, Nq, R, docs)
    int B, Nq, M, H, R, Rw;
    float out_scale;
};


// One sequence (b) by one workgroup.  dyn: nwaves * docs floats of LDS; the first nwaves waves of the workgroup
// take the (head, row) pairs, the others (a workgroup larger than the accumulator space allows) only join the
// barrier.  Every thread of the workgroup must call this.
//
// PATH selects the reduction (br_doc_final_path picks it on the host): 0 - at most 64 documents of at most 8 key
// tiles, one document per lane with its tiles in registers; 1 - at most 256 such documents, four per lane; 2 - any.
// Each is compiled on its own so that none carries the registers of the others.
__host__ __device__ inline int br_doc_final_path(int docs, int H) {
    if (H > 8 * BR_BN || docs > 256) return 2;
    return docs <= 64 ? 0 : 1;
}

template <int PATH>
__device__ __forceinline__ void br_doc_final_tiles_body(const BrTileScoreParams& p, const int b, float* dyn, const int nwaves) {
    const int docs = p.M - 2;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool idle = wave >= nwaves;           // waves beyond the accumulator rows only join the barrier
    const int* start = p.plan + br_plan_off_start();
    const int* len = p.plan + br_plan_off_len(p.B, p.M);
    const int* tbase = p.plan + br_plan_off_tbase(p.B, p.M);
    const int tps = br_plan_tps(p.M, p.H);
    const int NR = idle ? 0 : p.Nq * p.R;
    const int st_q = start[b * p.M + p.M - 1], len_q = len[b * p.M + p.M - 1];
    float* mine = dyn + (idle ? 0 : wave) * docs;
    for (int d = lane; d < docs && !idle; d += 64) mine[d] = 0.f;
    const float uniform = 1.f / (float)docs;
    constexpr bool small = PATH == 0;
    int t0 = 0, nt = 0;
    if (small && lane < docs) {
        t0 = tbase[b * p.M + lane + 1];
        nt = (len[b * p.M + lane + 1] + BR_BN - 1) / BR_BN;
    }
    if constexpr (small) {
        // four (head, row) pairs of a wave at a time: all their loads are issued before the first reduction
        constexpr int PG = 4;
        for (int j0 = wave; j0 < NR; j0 += PG * nwaves) {
            float2 v[PG][8];
            bool pair_on[PG];
#pragma unroll
            for (int i = 0; i < PG; ++i) {
                const int j = j0 + i * nwaves;
                pair_on[i] = j < NR;
                const int jj = pair_on[i] ? j : 0;
                const int n = jj / p.R, r = jj - n * p.R;
                int r16 = p.rows[b * p.R + r];
                r16 = r16 < 0 ? 0 : (r16 >= p.Rw ? p.Rw - 1 : r16);
                const int pos = p.H - p.Rw + r16;
                const bool row_ok = pair_on[i] && pos >= st_q && pos < st_q + len_q;
                const float2* base = reinterpret_cast<const float2*>(p.part) + (((long long)b * p.Nq + n) * p.Rw + r16) * tps;
#pragma unroll
                for (int t8 = 0; t8 < 8; ++t8) v[i][t8] = (row_ok && t8 < nt) ? base[t0 + t8] : make_float2(-INFINITY, 0.f);
            }
#pragma unroll
            for (int i = 0; i < PG; ++i) {
                if (!pair_on[i]) continue;
                const int j = j0 + i * nwaves;
                float* pr_out = p.probs ? p.probs + ((long long)b * p.Nq * p.R + j) * docs : nullptr;
                float mx = -INFINITY;
#pragma unroll
                for (int t8 = 0; t8 < 8; ++t8) mx = fmaxf(mx, v[i][t8].x);
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
                float sd = 0.f;
#pragma unroll
                for (int t8 = 0; t8 < 8; ++t8)
                    if (v[i][t8].x != -INFINITY) sd += v[i][t8].y * __builtin_amdgcn_exp2f(v[i][t8].x - mx);
                float den = sd;
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
                if (lane < docs) {
                    const float pr = den > 0.f ? sd / den : uniform;
                    if (pr_out) pr_out[lane] = pr;
                    mine[lane] += pr;
                }
            }
        }
    }
    // Up to 256 documents of at most 8 tiles: a lane takes documents lane, lane + 64, ...; each document's
    // tiles are reduced to (max, sum) as they arrive, two (head, row) pairs of a wave at a time.
    constexpr bool medium = PATH == 1;
    if constexpr (medium) {
        constexpr int PG = 4, DPL = 4;
        const int kmax = (docs + 63) >> 6;       // document slots per lane actually in use
        int t0m[DPL], ntm[DPL];
#pragma unroll
        for (int k = 0; k < DPL; ++k) {
            const int d = lane + 64 * k;
            ntm[k] = d < docs ? (len[b * p.M + d + 1] + BR_BN - 1) / BR_BN : 0;
            // (a document without tokens owns no tile: its loads below go to the row's first partial, not to the index
            // one past the documents before it, which for trailing empty documents is one past the row's partials)
            t0m[k] = ntm[k] > 0 ? tbase[b * p.M + d + 1] : 0;
        }
        for (int j0 = wave; j0 < NR; j0 += PG * nwaves) {
            float md[PG][DPL], sdm[PG][DPL];
            bool pair_on[PG];
            const float2* base[PG];
            bool row_ok[PG];
#pragma unroll
            for (int i = 0; i < PG; ++i) {
                const int j = j0 + i * nwaves;
                pair_on[i] = j < NR;
                const int jj = pair_on[i] ? j : 0;
                const int n = jj / p.R, r = jj - n * p.R;
                int r16 = p.rows[b * p.R + r];
                r16 = r16 < 0 ? 0 : (r16 >= p.Rw ? p.Rw - 1 : r16);
                const int pos = p.H - p.Rw + r16;
                row_ok[i] = pair_on[i] && pos >= st_q && pos < st_q + len_q;
                base[i] = reinterpret_cast<const float2*>(p.part) + (((long long)b * p.Nq + n) * p.Rw + r16) * tps;
            }
#pragma unroll
            for (int k = 0; k < DPL; ++k) {
#pragma unroll
                for (int i = 0; i < PG; ++i) {
                    md[i][k] = -INFINITY;
                    sdm[i][k] = 0.f;
                }
                if (k >= kmax) continue;
                float2 v[PG][8];
#pragma unroll
                for (int i = 0; i < PG; ++i)
#pragma unroll
                    for (int t8 = 0; t8 < 8; ++t8) v[i][t8] = base[i][t0m[k] + (t8 < ntm[k] ? t8 : 0)];   // always a valid address
#pragma unroll
                for (int i = 0; i < PG; ++i)
#pragma unroll
                    for (int t8 = 0; t8 < 8; ++t8)
                        if (!(row_ok[i] && t8 < ntm[k])) v[i][t8] = make_float2(-INFINITY, 0.f);
#pragma unroll
                for (int i = 0; i < PG; ++i) {
                    float m = -INFINITY;
#pragma unroll
                    for (int t8 = 0; t8 < 8; ++t8) m = fmaxf(m, v[i][t8].x);
                    float sacc = 0.f;
#pragma unroll
                    for (int t8 = 0; t8 < 8; ++t8)
                        if (v[i][t8].x != -INFINITY) sacc += v[i][t8].y * __builtin_amdgcn_exp2f(v[i][t8].x - m);
                    md[i][k] = m;
                    sdm[i][k] = sacc;
                }
            }
#pragma unroll
            for (int i = 0; i < PG; ++i) {
                if (!pair_on[i]) continue;
                const int j = j0 + i * nwaves;
                float* pr_out = p.probs ? p.probs + ((long long)b * p.Nq * p.R + j) * docs : nullptr;
                float mx = -INFINITY;
#pragma unroll
                for (int k = 0; k < DPL; ++k) mx = fmaxf(mx, md[i][k]);
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
                float den = 0.f;
#pragma unroll
                for (int k = 0; k < DPL; ++k) {
                    sdm[i][k] = md[i][k] == -INFINITY ? 0.f : sdm[i][k] * __builtin_amdgcn_exp2f(md[i][k] - mx);
                    den += sdm[i][k];
                }
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
#pragma unroll
                for (int k = 0; k < DPL; ++k) {
                    const int d = lane + 64 * k;
                    if (d < docs) {
                        const float pr = den > 0.f ? sdm[i][k] / den : uniform;
                        if (pr_out) pr_out[d] = pr;
                        mine[d] += pr;
                    }
                }
            }
        }
    }
    for (int j = wave; j < NR && PATH == 2; j += nwaves) {
        const int n = j / p.R, r = j - n * p.R;
        int r16 = p.rows[b * p.R + r];
        r16 = r16 < 0 ? 0 : (r16 >= p.Rw ? p.Rw - 1 : r16);
        const int pos = p.H - p.Rw + r16;
        const bool row_ok = pos >= st_q && pos < st_q + len_q;
        const float2* base = reinterpret_cast<const float2*>(p.part) + (((long long)b * p.Nq + n) * p.Rw + r16) * tps;
        float* pr_out = p.probs ? p.probs + ((long long)b * p.Nq * p.R + j) * docs : nullptr;
        {
            float mx = -INFINITY;
            if (row_ok)
                for (int d = lane; d < docs; d += 64) {
                    const int f0 = tbase[b * p.M + d + 1], f1 = f0 + (len[b * p.M + d + 1] + BR_BN - 1) / BR_BN;
                    for (int f = f0; f < f1; ++f) mx = fmaxf(mx, base[f].x);
                }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
            float den = 0.f;
            if (mx != -INFINITY)
                for (int d = lane; d < docs; d += 64) {
                    const int f0 = tbase[b * p.M + d + 1], f1 = f0 + (len[b * p.M + d + 1] + BR_BN - 1) / BR_BN;
                    float sd = 0.f;
                    for (int f = f0; f < f1; ++f) {
                        const float2 ms = base[f];
                        sd += ms.y * __builtin_amdgcn_exp2f(ms.x - mx);
                    }
                    den += sd;
                    if (pr_out) pr_out[d] = sd;       // unnormalised for now, only this lane touches it
                }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
            const float inv = den > 0.f ? 1.f / den : 0.f;
            for (int d = lane; d < docs; d += 64) {
                float pr = uniform;
                if (inv != 0.f) {
                    float sd;
                    if (pr_out) {
                        sd = pr_out[d];
                    } else {
                        const int f0 = tbase[b * p.M + d + 1], f1 = f0 + (len[b * p.M + d + 1] + BR_BN - 1) / BR_BN;
                        sd = 0.f;
                        for (int f = f0; f < f1; ++f) {
                            const float2 ms = base[f];
                            sd += ms.y * __builtin_amdgcn_exp2f(ms.x - mx);
                        }
                    }
                    pr = sd * inv;
                }
                if (pr_out) pr_out[d] = pr;
                mine[d] += pr;
            }
        }
    }
    __syncthreads();
    for (int d = threadIdx.x; d < docs; d += blockDim.x) {
        float acc = 0.f;
        for (int w = 0; w < nwaves; ++w) acc += dyn[w * docs + d];
        p.scores[(long long)b * docs + d] = acc * p.out_scale;
    }
}
