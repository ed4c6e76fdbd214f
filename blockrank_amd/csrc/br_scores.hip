// Per-document relevance from the query block's attention, without materialising attention rows.
//
// Reference: compute_auxiliary_attention_loss(answer_ids=None, return_logits=True), losses.py:37-78,
// applied to the logits of blockrank_std_attention.py:233,259 (scaled q.k of chosen rows of the
// query block against every key).  For each (head, chosen row) the reference soft-maxes the logits
// over all document tokens jointly and sums the probabilities per document, then averages heads and
// rows and divides by the temperature.  Here:
//   br_doc_partial_kernel  one workgroup per (document, kv head group, sequence): logits of that
//                          document's real keys for every (head, row) of the group, reduced on the
//                          fly to (max, sum of exp) per (head, row, document);
//   br_doc_final_kernel    one workgroup per sequence: joint normalisation across documents, head /
//                          row reduction, temperature.
// br_last_logits_kernel writes the reference's s_last tensor itself for callers that still want it.
#include "br_common.h"
#include "br_score_tiles.h"

namespace {

constexpr int kQR = 16;            // (head, row) pairs one workgroup carries
constexpr float kLog2e = 1.4426950408889634f;

template <typename T>
struct Load8;
template <>
struct Load8<float> {
    static __device__ inline void ld(const float* p, float* x) {
        float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
};
template <>
struct Load8<__bf16> {
    static __device__ inline void ld(const __bf16* p, float* x) {
        uint4 u = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[2 * i] = __uint_as_float(w[i] << 16);
            x[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
};

struct BrScoreParams {
    const void* q;
    const void* k;
    const int* plan;        // only the block table part is used
    const int* rows;        // (B, R) positions of the chosen rows inside the query block, 0..H-1
    float* part;            // (B, Nq, R, docs, 2): max (log2 domain) and sum of exp per document
    float* scores;          // (B, docs)
    float* probs;           // optional (B, Nq, R, docs) per-head, per-row document probabilities
    float* logits;          // br_last_logits_kernel: (B, Nq, R, S)
    long long sq_b, sq_h, sq_t;
    long long sk_b, sk_h, sk_t;
    int B, Nq, Nkv, M, H, D, R, T;
    int hc;                 // heads per workgroup (hc * R <= kQR)
    float scale;            // softmax scale
    float out_scale;        // head/row reduction factor divided by the temperature
    float neg;              // the reference's finite "masked" value for the model dtype
};

// Stage the (head, row) query vectors of one workgroup into LDS as fp32, pre-multiplied by mult.
// qs is [hc*R][D]; ok[j] says whether that row is a real token.
template <typename T>
__device__ void stage_queries(const BrScoreParams& p, const BrPlanView& pv, int b, int head0, int nheads, float mult, float* qs,
                              int* ok) {
    const int m = p.M - 1;
    const int st = pv.start[b * p.M + m], ln = pv.len[b * p.M + m], tk = pv.tok[b * p.M + m];
    for (int idx = threadIdx.x; idx < nheads * p.R * p.D; idx += blockDim.x) {
        int j = idx / p.D, d = idx - j * p.D;
        int h = j / p.R, r = j - h * p.R;
        int pos = p.rows[b * p.R + r];
        bool v = pos >= st && pos < st + ln;
        float x = 0.f;
        if (v) x = (float)reinterpret_cast<const T*>(p.q)[(long long)b * p.sq_b + (long long)(head0 + h) * p.sq_h +
                                                         (long long)(tk + pos - st) * p.sq_t + d];
        qs[j * p.D + d] = x * mult;
        if (d == 0) ok[j] = v;
    }
}

// Dot products of one key row with the nq staged query vectors.  The head dim is a compile-time
// constant so that the loop unrolls and every load of the key row is in flight before the first use.
template <>
struct Load8<_Float16> {
    static __device__ inline void ld(const _Float16* p, float* x) {
        uint4 u = *reinterpret_cast<const uint4*>(p);
        const _Float16* h = reinterpret_cast<const _Float16*>(&u);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = (float)h[i];
    }
};

template <typename T, int D>
__device__ inline void key_dots(const T* krow, const float* qs, int nq, float* s) {
#pragma unroll
    for (int j = 0; j < kQR; ++j) s[j] = 0.f;
    constexpr int HALF = D / 2;
#pragma unroll
    for (int h0 = 0; h0 < D; h0 += HALF) {
        float x[HALF];
#pragma unroll
        for (int d0 = 0; d0 < HALF; d0 += 8) Load8<T>::ld(krow + h0 + d0, x + d0);
#pragma unroll
        for (int j = 0; j < kQR; ++j) {
            if (j < nq) {
                const float* qv = qs + j * D + h0;
                float a = s[j];
#pragma unroll
                for (int e = 0; e < HALF; ++e) a = fmaf(x[e], qv[e], a);
                s[j] = a;
            }
        }
    }
}

template <typename T, int D>
__global__ __launch_bounds__(256) void br_doc_partial_kernel(BrScoreParams p) {
    extern __shared__ float dyn[];
    float* qs = dyn;                                   // [kQR][D]
    __shared__ int ok[kQR];
    __shared__ float red_m[4][kQR], red_s[4][kQR];
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, p.T);
    const int doc = blockIdx.x, b = blockIdx.z;
    const int G = p.Nq / p.Nkv;
    const int chunks = (G + p.hc - 1) / p.hc;
    const int kvh = blockIdx.y / chunks, hchunk = blockIdx.y - kvh * chunks;
    const int head0 = kvh * G + hchunk * p.hc;
    const int nheads = (hchunk + 1) * p.hc <= G ? p.hc : G - hchunk * p.hc;
    const int nq = nheads * p.R;
    const int docs = p.M - 2;
    stage_queries<T>(p, pv, b, head0, nheads, p.scale * kLog2e, qs, ok);
    __syncthreads();
    const int blk = doc + 1;
    const int st = pv.start[b * p.M + blk], ln = pv.len[b * p.M + blk];
    const T* kbase = reinterpret_cast<const T*>(p.k) + (long long)b * p.sk_b + (long long)kvh * p.sk_h +
                     (long long)pv.tok[b * p.M + blk] * p.sk_t;
    float mx[kQR], sm[kQR];
#pragma unroll
    for (int j = 0; j < kQR; ++j) {
        mx[j] = -INFINITY;
        sm[j] = 0.f;
    }
    for (int key = threadIdx.x; key < ln; key += blockDim.x) {
        float s[kQR];
        key_dots<T, D>(kbase + (long long)key * p.sk_t, qs, nq, s);
#pragma unroll
        for (int j = 0; j < kQR; ++j) {
            float mn = fmaxf(mx[j], s[j]);
            sm[j] = sm[j] * __builtin_amdgcn_exp2f(mx[j] - mn) + __builtin_amdgcn_exp2f(s[j] - mn);
            mx[j] = mn;
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < kQR; ++j) {
        float m1 = mx[j], s1 = sm[j];
        for (int o = 32; o > 0; o >>= 1) {
            float m2 = __shfl_xor(m1, o), s2 = __shfl_xor(s1, o);
            float mn = fmaxf(m1, m2);
            float a = m1 == -INFINITY ? 0.f : s1 * __builtin_amdgcn_exp2f(m1 - mn);
            float c = m2 == -INFINITY ? 0.f : s2 * __builtin_amdgcn_exp2f(m2 - mn);
            m1 = mn;
            s1 = a + c;
        }
        if (lane == 0) {
            red_m[wave][j] = m1;
            red_s[wave][j] = s1;
        }
    }
    __syncthreads();
    if (threadIdx.x < nq) {
        const int j = threadIdx.x;
        float m1 = -INFINITY, s1 = 0.f;
        for (int w = 0; w < 4; ++w) {
            float m2 = red_m[w][j], s2 = red_s[w][j];
            float mn = fmaxf(m1, m2);
            float a = m1 == -INFINITY ? 0.f : s1 * __builtin_amdgcn_exp2f(m1 - mn);
            float c = m2 == -INFINITY ? 0.f : s2 * __builtin_amdgcn_exp2f(m2 - mn);
            m1 = mn;
            s1 = a + c;
        }
        const int h = j / p.R, r = j - h * p.R;
        if (!ok[j]) {   // a padded query row sees nothing; the final kernel turns this into the uniform answer
            m1 = -INFINITY;
            s1 = 0.f;
        }
        float* dst = p.part + ((((long long)b * p.Nq + head0 + h) * p.R + r) * docs + doc) * 2;
        dst[0] = m1;
        dst[1] = s1;
    }
}

__global__ __launch_bounds__(256) void br_doc_final_kernel(BrScoreParams p) {
    extern __shared__ float dyn[];
    const int NR = p.Nq * p.R;
    const int docs = p.M - 2;
    float* gmax = dyn;          // [NR]
    float* ginv = dyn + NR;     // [NR], 0 marks "no visible document key": uniform
    const int b = blockIdx.x;
    const float* part = p.part + (long long)b * NR * docs * 2;
    // one coalesced pass brings this sequence's (max, sum) pairs into LDS when they fit
    if (p.hc) {
        float* stage = dyn + 2 * NR;
        for (int i = threadIdx.x; i < NR * docs * 2; i += blockDim.x) stage[i] = part[i];
        __syncthreads();
        part = stage;
    }
    for (int j = threadIdx.x; j < NR; j += blockDim.x) {
        float mm = -INFINITY;
        for (int d = 0; d < docs; ++d) mm = fmaxf(mm, part[((long long)j * docs + d) * 2]);
        float den = 0.f;
        if (mm != -INFINITY)
            for (int d = 0; d < docs; ++d) {
                float m1 = part[((long long)j * docs + d) * 2];
                if (m1 != -INFINITY) den += part[((long long)j * docs + d) * 2 + 1] * __builtin_amdgcn_exp2f(m1 - mm);
            }
        gmax[j] = mm;
        ginv[j] = den > 0.f ? 1.f / den : 0.f;
    }
    __syncthreads();
    const float uniform = 1.f / (float)docs;
    for (int d = threadIdx.x; d < docs; d += blockDim.x) {
        float acc = 0.f;
        for (int j = 0; j < NR; ++j) {
            float pr;
            if (ginv[j] == 0.f) {
                pr = uniform;
            } else {
                float m1 = part[((long long)j * docs + d) * 2];
                pr = m1 == -INFINITY ? 0.f : part[((long long)j * docs + d) * 2 + 1] * __builtin_amdgcn_exp2f(m1 - gmax[j]) * ginv[j];
            }
            if (p.probs) p.probs[((long long)b * NR + j) * docs + d] = pr;
            acc += pr;
        }
        p.scores[(long long)b * docs + d] = acc * p.out_scale;
    }
}

// MAXT: threads per workgroup the instance is compiled for (1024: sixteen waves of at most 128 registers, for
// the one-document-per-lane case; 512: eight waves of up to 256 registers, whose loads are all in flight together).
template <int MAXT, int PATH>
__global__ __launch_bounds__(MAXT) void br_doc_final_tiles_kernel(BrTileScoreParams p) {
    extern __shared__ float dyn[];      // [nwaves][docs]
    br_doc_final_tiles_body<PATH>(p, blockIdx.x, dyn, blockDim.x >> 6);
}

// s_last[b, n, r, key] = scale * q.k + (0 if the row may see the key else NEG), every key slot of
// the padded sequence included (blockrank_std_attention.py:639-645 with the eager scaling of :154).
template <typename T, int D>
__global__ __launch_bounds__(256) void br_last_logits_kernel(BrScoreParams p) {
    extern __shared__ float dyn[];
    float* qs = dyn;
    __shared__ int ok[kQR];
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, p.T);
    const int b = blockIdx.z;
    const int G = p.Nq / p.Nkv;
    const int chunks = (G + p.hc - 1) / p.hc;
    const int kvh = blockIdx.y / chunks, hchunk = blockIdx.y - kvh * chunks;
    const int head0 = kvh * G + hchunk * p.hc;
    const int nheads = (hchunk + 1) * p.hc <= G ? p.hc : G - hchunk * p.hc;
    const int nq = nheads * p.R;
    const int S = p.M * p.H;
    stage_queries<T>(p, pv, b, head0, nheads, p.scale, qs, ok);
    __syncthreads();
    const int key = blockIdx.x * blockDim.x + threadIdx.x;
    if (key >= S) return;
    const int blk = key / p.H, j = key - blk * p.H;
    const int st = pv.start[b * p.M + blk], ln = pv.len[b * p.M + blk];
    const bool kvalid = j >= st && j < st + ln;
    // (a slot that holds no real token has no key row to read - in a packed layout not even storage;
    // its logit is the masked value whatever the dot product would be)
    const T* krow = reinterpret_cast<const T*>(p.k) + (long long)b * p.sk_b + (long long)kvh * p.sk_h +
                    (long long)(pv.tok[b * p.M + blk] + j - st) * p.sk_t;
    float s[kQR];
    if (kvalid) {
        key_dots<T, D>(krow, qs, nq, s);
    } else {
#pragma unroll
        for (int jq = 0; jq < kQR; ++jq) s[jq] = 0.f;
    }
#pragma unroll
    for (int jq = 0; jq < kQR; ++jq) {
        if (jq < nq) {
            const int h = jq / p.R, r = jq - h * p.R;
            const int pos = p.rows[b * p.R + r];
            bool allow = kvalid && ok[jq] && (blk < p.M - 1 || j <= pos);
            p.logits[(((long long)b * p.Nq + head0 + h) * p.R + r) * S + key] = s[jq] + (allow ? 0.f : p.neg);
        }
    }
}


// ---- gradient of br_last_logits_kernel ----
// s[b,n,r,key] = scale * q[b,n,row_r] . k[b,n/G,key] + constant for real rows and real keys (the additive mask is a
// constant, so disallowed real keys carry gradient like the reference's additive-mask logits do); slots without a token
// and rows that are padding do not depend on q or k at all.
struct BrLogitsBwdParams {
    const float* ds;        // (B, Nq, R, M*H) gradient of the logits
    const void* q;
    const void* k;
    const int* plan;
    const int* rows;        // (B, R) positions inside the query block
    void* dq;               // caller-zeroed; only the chosen rows are written
    void* dk;               // every key token is written
    long long sq_b, sq_h, sq_t, sk_b, sk_h, sk_t;
    long long dq_b, dq_h, dq_t, dk_b, dk_h, dk_t;
    int B, Nq, Nkv, M, H, D, R, T;
    float scale;
};

template <typename T>
__device__ inline void store_row_piece(T* dst, const float* x, int n);
template <>
__device__ inline void store_row_piece<float>(float* dst, const float* x, int n) {
    for (int i = 0; i < n; ++i) dst[i] = x[i];
}
template <>
__device__ inline void store_row_piece<__bf16>(__bf16* dst, const float* x, int n) {
    for (int i = 0; i < n; ++i) dst[i] = (__bf16)x[i];
}
template <>
__device__ inline void store_row_piece<_Float16>(_Float16* dst, const float* x, int n) {
    for (int i = 0; i < n; ++i) dst[i] = (_Float16)x[i];
}

// dk[key] = scale * sum over the kv head's query heads n and rows r of ds[n, r, key] * q[n, row_r].  One thread per key
// slot, the whole row of D sums in its registers; the query vectors go through LDS sixteen (head, row) pairs at a time.
template <typename T, int D>
__global__ __launch_bounds__(256) void br_last_logits_bwd_dk_kernel(BrLogitsBwdParams p) {
    __shared__ float qs[kQR * D];
    __shared__ int ok[kQR];
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, p.T);
    const int b = blockIdx.z, kvh = blockIdx.y;
    const int G = p.Nq / p.Nkv;
    const int S = p.M * p.H;
    const int hc = kQR / p.R;                                  // heads per pass
    const int key = blockIdx.x * blockDim.x + threadIdx.x;
    const bool in_range = key < S;
    const int kk = in_range ? key : 0;
    const int blk = kk / p.H, j = kk - blk * p.H;
    const int st = pv.start[b * p.M + blk], ln = pv.len[b * p.M + blk];
    const bool kvalid = in_range && j >= st && j < st + ln;
    const bool packed = pv.hdr[BR_PH_PACKED] != 0;
    float acc[D];
#pragma unroll
    for (int d = 0; d < D; ++d) acc[d] = 0.f;
    BrScoreParams sp;                                           // what stage_queries reads
    sp.q = p.q; sp.rows = p.rows; sp.sq_b = p.sq_b; sp.sq_h = p.sq_h; sp.sq_t = p.sq_t; sp.M = p.M; sp.R = p.R; sp.D = D;
    for (int h0 = 0; h0 < G; h0 += hc) {
        const int nheads = h0 + hc <= G ? hc : G - h0;
        __syncthreads();
        stage_queries<T>(sp, pv, b, kvh * G + h0, nheads, p.scale, qs, ok);
        __syncthreads();
        if (kvalid) {
            for (int jq = 0; jq < nheads * p.R; ++jq) {
                const int h = jq / p.R, r = jq - h * p.R;
                const float w = p.ds[(((long long)b * p.Nq + kvh * G + h0 + h) * p.R + r) * S + key];
                const float* qv = qs + jq * D;
#pragma unroll
                for (int d = 0; d < D; ++d) acc[d] = fmaf(w, qv[d], acc[d]);
            }
        }
    }
    if (!in_range || (packed && !kvalid)) return;              // a packed layout has no storage for empty slots
    const long long tokn = kvalid ? pv.tok[b * p.M + blk] + j - st : (long long)blk * p.H + j;
    T* dst = reinterpret_cast<T*>(p.dk) + (long long)b * p.dk_b + (long long)kvh * p.dk_h + tokn * p.dk_t;
    store_row_piece<T>(dst, acc, D);
}

// dq[row_r] = scale * sum over the real keys of ds[n, r, key] * k[key].  One workgroup per (sequence, head): thread =
// (key phase, dim), sixteen row sums in registers; the ds values and the slot -> token map of 256 keys at a time in LDS.
template <typename T, int D>
__global__ __launch_bounds__(256) void br_last_logits_bwd_dq_kernel(BrLogitsBwdParams p) {
    constexpr int NPH = 256 / D;                               // key phases
    constexpr int CH = 256;                                    // keys per chunk
    __shared__ float dsl[kQR * CH];
    __shared__ int tokl[CH];
    static_assert(NPH * kQR * D <= kQR * CH, "the phase reduction reuses the ds buffer");
    const BrPlanView pv = br_plan_view(p.plan, p.B, p.M, p.H, p.T);
    const int b = blockIdx.y, n = blockIdx.x;
    const int G = p.Nq / p.Nkv, kvh = n / G;
    const int S = p.M * p.H;
    const int d = threadIdx.x % D, ph = threadIdx.x / D;
    const T* kb = reinterpret_cast<const T*>(p.k) + (long long)b * p.sk_b + (long long)kvh * p.sk_h + d;
    float acc[kQR];
#pragma unroll
    for (int r = 0; r < kQR; ++r) acc[r] = 0.f;
    for (int s0 = 0; s0 < S; s0 += CH) {
        __syncthreads();
        {
            const int key = s0 + threadIdx.x;
            int tk = -1;
            if (key < S) {
                const int blk = key / p.H, j = key - blk * p.H;
                const int st = pv.start[b * p.M + blk], ln = pv.len[b * p.M + blk];
                if (j >= st && j < st + ln) tk = pv.tok[b * p.M + blk] + j - st;
            }
            tokl[threadIdx.x] = tk;
            for (int r = 0; r < p.R; ++r)
                dsl[r * CH + threadIdx.x] = key < S ? p.ds[(((long long)b * p.Nq + n) * p.R + r) * S + key] : 0.f;
        }
        __syncthreads();
        constexpr int U = 8;
        for (int i0 = ph; i0 < CH; i0 += NPH * U) {
            float kv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = i0 + u * NPH;
                const int tk = i < CH ? tokl[i] : -1;
                kv[u] = tk >= 0 ? (float)kb[(long long)tk * p.sk_t] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = i0 + u * NPH;
                if (i < CH) {
#pragma unroll
                    for (int r = 0; r < kQR; ++r)
                        if (r < p.R) acc[r] = fmaf(dsl[r * CH + i], kv[u], acc[r]);
                }
            }
        }
    }
    // add the key phases up (in dsl, free now), then one thread per (row, dim) writes the row - rows named twice are
    // summed into their first occurrence
    __syncthreads();
    float* red2 = dsl;                                          // [NPH][R][D] <= 16 * 256 floats
    for (int r = 0; r < p.R; ++r) red2[(ph * kQR + r) * D + d] = acc[r];
    __syncthreads();
    const int m = p.M - 1;
    const int st = pv.start[b * p.M + m], ln = pv.len[b * p.M + m], tk0 = pv.tok[b * p.M + m];
    for (int idx = threadIdx.x; idx < p.R * D; idx += blockDim.x) {
        const int r = idx / D, dd = idx - r * D;
        const int pos = p.rows[b * p.R + r];
        if (pos < st || pos >= st + ln) continue;              // a padded row: its logits do not depend on q
        bool first = true;
        for (int r2 = 0; r2 < r; ++r2) first = first && p.rows[b * p.R + r2] != pos;
        if (!first) continue;
        float v = 0.f;
        for (int r2 = r; r2 < p.R; ++r2)
            if (p.rows[b * p.R + r2] == pos)
                for (int q = 0; q < NPH; ++q) v += red2[(q * kQR + r2) * D + dd];
        T* dst = reinterpret_cast<T*>(p.dq) + (long long)b * p.dq_b + (long long)n * p.dq_h + (long long)(tk0 + pos - st) * p.dq_t + dd;
        const float out = v * p.scale;
        store_row_piece<T>(dst, &out, 1);
    }
}

}  // namespace

// Launch KERNEL<element type, head dim> for the dtype code (0 fp32, 1 bf16, 2 fp16) and D (64 or 128) in scope, 256
// threads, with the parameter block p.
#define BR_BY_TYPE_AND_DIM(KERNEL, GRID, LDS)                                                                   \
    do {                                                                                                        \
        if (dtype == 0 && D == 64) hipLaunchKernelGGL((KERNEL<float, 64>), GRID, dim3(256), LDS, stream, p);         \
        else if (dtype == 0) hipLaunchKernelGGL((KERNEL<float, 128>), GRID, dim3(256), LDS, stream, p);              \
        else if (dtype == 1 && D == 64) hipLaunchKernelGGL((KERNEL<__bf16, 64>), GRID, dim3(256), LDS, stream, p);   \
        else if (dtype == 1) hipLaunchKernelGGL((KERNEL<__bf16, 128>), GRID, dim3(256), LDS, stream, p);             \
        else if (D == 64) hipLaunchKernelGGL((KERNEL<_Float16, 64>), GRID, dim3(256), LDS, stream, p);               \
        else hipLaunchKernelGGL((KERNEL<_Float16, 128>), GRID, dim3(256), LDS, stream, p);                           \
    } while (0)

// dtype: 0 fp32, 1 bf16
int br_launch_doc_scores(const void* q, const void* k, const int* plan, const int* rows, float* part, float* scores,
                         float* probs, const long long* sq, const long long* sk, int B, int Nq, int Nkv, int M, int H, int D,
                         int R, int T, float scale, float out_scale, int dtype, hipStream_t stream) {
    BrScoreParams p;
    p.q = q; p.k = k; p.plan = plan; p.rows = rows; p.part = part; p.scores = scores; p.probs = probs; p.logits = nullptr;
    p.sq_b = sq[0]; p.sq_h = sq[1]; p.sq_t = sq[2];
    p.sk_b = sk[0]; p.sk_h = sk[1]; p.sk_t = sk[2];
    p.B = B; p.Nq = Nq; p.Nkv = Nkv; p.M = M; p.H = H; p.D = D; p.R = R; p.T = T;
    p.hc = kQR / R; p.scale = scale; p.out_scale = out_scale; p.neg = 0.f;
    const int G = Nq / Nkv;
    const int chunks = (G + p.hc - 1) / p.hc;
    dim3 grid(M - 2, Nkv * chunks, B);
    size_t sh = (size_t)kQR * D * sizeof(float);
    BR_BY_TYPE_AND_DIM(br_doc_partial_kernel, grid, sh);
    // the final kernel reuses hc as "the partials fit in LDS" flag
    size_t fin = (size_t)2 * Nq * R * sizeof(float);
    const size_t stage = (size_t)Nq * R * (M - 2) * 2 * sizeof(float);
    p.hc = stage + fin <= 63 * 1024 ? 1 : 0;   // stays within the default dynamic LDS limit
    if (p.hc) fin += stage;
    hipLaunchKernelGGL(br_doc_final_kernel, dim3(B), dim3(256), fin, stream, p);
    return 0;
}

int br_launch_last_logits(const void* q, const void* k, const int* plan, const int* rows, float* logits, const long long* sq,
                          const long long* sk, int B, int Nq, int Nkv, int M, int H, int D, int R, int T, float scale,
                          float neg, int dtype, hipStream_t stream) {
    BrScoreParams p;
    p.q = q; p.k = k; p.plan = plan; p.rows = rows; p.part = nullptr; p.scores = nullptr; p.probs = nullptr; p.logits = logits;
    p.sq_b = sq[0]; p.sq_h = sq[1]; p.sq_t = sq[2];
    p.sk_b = sk[0]; p.sk_h = sk[1]; p.sk_t = sk[2];
    p.B = B; p.Nq = Nq; p.Nkv = Nkv; p.M = M; p.H = H; p.D = D; p.R = R; p.T = T;
    p.hc = kQR / R; p.scale = scale; p.out_scale = 1.f; p.neg = neg;
    const int G = Nq / Nkv;
    const int chunks = (G + p.hc - 1) / p.hc;
    const int S = M * H;
    dim3 grid((S + 255) / 256, Nkv * chunks, B);
    size_t sh = (size_t)kQR * D * sizeof(float);
    BR_BY_TYPE_AND_DIM(br_last_logits_kernel, grid, sh);
    return 0;
}

int br_launch_doc_scores_tiles(const float* part, const int* plan, const int* rows, float* scores, float* probs, int B, int Nq,
                               int M, int H, int R, int Rw, float out_scale, hipStream_t stream) {
    BrTileScoreParams p;
    p.part = part; p.plan = plan; p.rows = rows; p.scores = scores; p.probs = probs;
    p.B = B; p.Nq = Nq; p.M = M; p.H = H; p.R = R; p.Rw = Rw; p.out_scale = out_scale;
    const int docs = M - 2;
    const int path = br_doc_final_path(docs, H);
    int nwaves = path == 0 ? 16 : 8;
    while (nwaves > 1 && (size_t)nwaves * docs * sizeof(float) > 48 * 1024) nwaves >>= 1;
    if ((size_t)nwaves * docs * sizeof(float) > 60 * 1024) return 1;
    const size_t lds = (size_t)nwaves * docs * sizeof(float);
    if (path == 0)
        hipLaunchKernelGGL((br_doc_final_tiles_kernel<1024, 0>), dim3(B), dim3(nwaves * 64), lds, stream, p);
    else if (path == 1)
        hipLaunchKernelGGL((br_doc_final_tiles_kernel<512, 1>), dim3(B), dim3(nwaves * 64), lds, stream, p);
    else
        hipLaunchKernelGGL((br_doc_final_tiles_kernel<512, 2>), dim3(B), dim3(nwaves * 64), lds, stream, p);
    return 0;
}

int br_launch_last_logits_bwd(const float* ds, const void* q, const void* k, const int* plan, const int* rows, void* dq, void* dk,
                              const long long* sq, const long long* sk, const long long* sdq, const long long* sdk, int B, int Nq,
                              int Nkv, int M, int H, int D, int R, int T, float scale, int dtype, hipStream_t stream) {
    BrLogitsBwdParams p;
    p.ds = ds; p.q = q; p.k = k; p.plan = plan; p.rows = rows; p.dq = dq; p.dk = dk;
    p.sq_b = sq[0]; p.sq_h = sq[1]; p.sq_t = sq[2];
    p.sk_b = sk[0]; p.sk_h = sk[1]; p.sk_t = sk[2];
    p.dq_b = sdq[0]; p.dq_h = sdq[1]; p.dq_t = sdq[2];
    p.dk_b = sdk[0]; p.dk_h = sdk[1]; p.dk_t = sdk[2];
    p.B = B; p.Nq = Nq; p.Nkv = Nkv; p.M = M; p.H = H; p.D = D; p.R = R; p.T = T; p.scale = scale;
    const int S = M * H;
    dim3 gk((S + 255) / 256, Nkv, B), gq(Nq, B);
    BR_BY_TYPE_AND_DIM(br_last_logits_bwd_dk_kernel, gk, 0);
    BR_BY_TYPE_AND_DIM(br_last_logits_bwd_dq_kernel, gq, 0);
    return 0;
}
