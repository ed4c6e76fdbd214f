// extern "C" entry points of libblockrank_hip.so: argument checks, geometry selection, launches.
#include <stdarg.h>
#include <atomic>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/blockrank_hip.h"
#include "br_common.h"
#include "br_score_tiles.h"

void br_launch_plan_rearm(int* plan, hipStream_t stream);
void br_launch_plan(const uint8_t* valid, const int* lens, int left_padded, int packed, int B, int M, int H, int T, int par, int pool,
                    int* plan, hipStream_t stream);
int br_launch_prefill_bf16(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                           hipEvent_t ev_start, hipEvent_t ev_stop, const BrTileScoreParams* rank);
int br_launch_prefill_f16(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                          hipEvent_t ev_start, hipEvent_t ev_stop, const BrTileScoreParams* rank);
int br_launch_prefill_f32(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                           hipEvent_t ev_start, hipEvent_t ev_stop);
int br_launch_doc_scores(const void* q, const void* k, const int* plan, const int* rows, float* part, float* scores,
                         float* probs, const long long* sq, const long long* sk, int B, int Nq, int Nkv, int M, int H, int D,
                         int R, int T, float scale, float out_scale, int dtype, hipStream_t stream);
int br_launch_prefill_fp8qk(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                            hipEvent_t ev_start, hipEvent_t ev_stop, const BrTileScoreParams* rank);
void br_launch_quantize_fp8(const void* k, const int* plan, void* k8, unsigned* amax, float* scales, const long long* sk,
                            long long k8_b, long long k8_h, int B, int Nkv, int M, int H, int D, hipStream_t stream);
int br_launch_rope(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int B, int Nq, int Nkv, int S,
                   int D, const long long* sq, const long long* sk, const long long* sc, int dtype, int n_cu, hipStream_t stream);
int br_launch_doc_scores_tiles(const float* part, const int* plan, const int* rows, float* scores, float* probs, int B, int Nq,
                               int M, int H, int R, int Rw, float out_scale, hipStream_t stream);
int br_launch_last_logits(const void* q, const void* k, const int* plan, const int* rows, float* logits, const long long* sq,
                          const long long* sk, int B, int Nq, int Nkv, int M, int H, int D, int R, int T, float scale,
                          float neg, int dtype, hipStream_t stream);

int br_launch_last_logits_bwd(const float* ds, const void* q, const void* k, const int* plan, const int* rows, void* dq, void* dk,
                              const long long* sq, const long long* sk, const long long* sdq, const long long* sdk, int B, int Nq,
                              int Nkv, int M, int H, int D, int R, int T, float scale, int dtype, hipStream_t stream);
int br_launch_bwd(const BrBwdParams& p, int D, int NW, int n_cu, hipStream_t stream);
int br_launch_rmsnorm(const void* x, const void* w, void* out, long long rows, int hidden, long long sx, long long so, float eps, int dtype,
                      int n_cu, hipStream_t stream);
void br_launch_silu_mul(const void* gate, const void* up, void* out, long long n, int dtype, int n_cu, hipStream_t stream);

// Split-KV partials of br_prefill_fwd_noalloc: device memory that belongs to the library, one copy on every GPU
// the library runs on, held until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress: the address the kernels get is the one that call returns for the current device.
#define BR_NOALLOC_SCRATCH_BYTES ((size_t)32 << 20)
static __device__ __align__(256) unsigned char scratch[BR_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// Head layout -> workgroup shape.  A workgroup carries NW row blocks of 32 query rows: Gw heads of
// one kv head's group times tpb 32-token sub-blocks.
// ragged (the 16-bit MFMA forward kernels only): a group of 7 heads (Qwen2.5-7B's 28/4), which has no divisor but
// itself, is cut into sub-groups of 4 + 3 (the spare wave of the second idles) instead of one workgroup of 7 waves:
// two independent 4-wave workgroups per CU beat one wide one by a little more than the idle wave costs (measured 225
// against 231 us at that shape).  Tokens per query tile are the same either way, so one plan serves both shapes.
bool make_geom(int Nq, int Nkv, BrGeom* g, int* NW, bool ragged = false) {
    if (Nq <= 0 || Nkv <= 0 || Nq % Nkv) return false;
    const int G = Nq / Nkv;
    int Gw = 1;
    for (int d = 1; d <= 8 && d <= G; ++d)
        if (G % d == 0) Gw = d;
    if (ragged && Gw == 7) Gw = 4;
    int nw, tpb;
    switch (Gw) {
        case 1: nw = 4; tpb = 4; break;
        case 2: nw = 4; tpb = 2; break;
        case 3: nw = 6; tpb = 2; break;
        case 4: nw = 4; tpb = 1; break;
        default: nw = Gw; tpb = 1; break;
    }
    g->G = G;
    g->Gw = Gw;
    g->tpb = tpb;
    g->HGS = (G + Gw - 1) / Gw;
    g->NHG = Nkv * g->HGS;
    *NW = nw;
    return true;
}

// Workgroups of the prefill kernel per compute unit (the launchers' choice: two of up to four waves, else one).
int prefill_wgs_per_cu(int nw) { return nw <= 4 ? 2 : 1; }

int n_compute_units() {
    static thread_local int cached_dev = -1, cached_cu = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (dev != cached_dev) {
        int cu = 0;
        if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cached_dev = dev;
        cached_cu = cu;
    }
    return cached_cu;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(BR_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
    return BR_OK;
}

int check_common(int B, int Nq, int Nkv, int M, int H, int D, int dtype) {
    if (B <= 0 || M <= 0 || H <= 0) return fail(BR_ERR_ARG, "B, M and H must be positive (got %d, %d, %d)", B, M, H);
    if (Nq <= 0 || Nkv <= 0 || Nq % Nkv) return fail(BR_ERR_ARG, "Nq=%d must be a positive multiple of Nkv=%d", Nq, Nkv);
    if (D != 64 && D != 128) return fail(BR_ERR_ARG, "head dim %d not supported (64 or 128)", D);
    if (dtype != BR_DTYPE_F32 && dtype != BR_DTYPE_BF16 && dtype != BR_DTYPE_F16) return fail(BR_ERR_ARG, "dtype %d not supported", dtype);
    return BR_OK;
}

int check_strides(const char* name, const int64_t* s, int dtype) {
    if (!s) return fail(BR_ERR_ARG, "%s strides are null", name);
    const int per16 = dtype == BR_DTYPE_F32 ? 4 : 8;
    for (int i = 0; i < 3; ++i)
        if (s[i] < 0 || s[i] % per16) return fail(BR_ERR_ARG, "%s stride %d = %lld is not a multiple of 16 bytes", name, i, (long long)s[i]);
    return BR_OK;
}

// Workgroups of the 16-bit prefill grid that share one head group's items: what the plan balances the split of the
// query blocks' walks against, and what sizes the pool of split-KV partial slots.
int prefill_par(int Nq, int Nkv, int n_cu, int* nhg = nullptr) {
    BrGeom g16;
    int nw16;
    if (!make_geom(Nq, Nkv, &g16, &nw16, true)) return 1;
    if (nhg) *nhg = g16.NHG;
    const int par = n_cu * prefill_wgs_per_cu(nw16) / g16.NHG;
    return par < 1 ? 1 : par;
}

// Slots of the split-KV partial pool for a head layout on the current device.
int prefill_pool(int Nq, int Nkv, int n_cu) {
    int nhg = 1;
    const int par = prefill_par(Nq, Nkv, n_cu, &nhg);
    return br_split_pool(par, nhg);
}

size_t slots_total(int pool, const BrGeom& g) { return (size_t)pool * g.NHG; }

}  // namespace

extern "C" {

int br_version(void) { return 100; }

const char* br_last_error(void) { return g_err; }

int br_tile_tokens(int Nq, int Nkv) {
    BrGeom g;
    int nw;
    if (!make_geom(Nq, Nkv, &g, &nw)) return 0;
    return br_tokens_per_tile(g);
}

size_t br_plan_ints(int B, int M, int H, int Nq, int Nkv) {
    BrGeom g;
    int nw;
    if (!make_geom(Nq, Nkv, &g, &nw) || B <= 0 || M <= 0 || H <= 0) return 0;
    return br_plan_total_ints(B, M, H, br_tokens_per_tile(g));
}

int br_plan_check(const int32_t* plan, void* stream) {
    if (!plan) return fail(BR_ERR_ARG, "null pointer");
    int32_t words[BR_PH_DONE - BR_PH_QTICKET + 1];
    hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (e == hipSuccess) e = hipMemcpy(words, plan + BR_PH_QTICKET, sizeof(words), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return fail(BR_ERR_HIP, "reading the plan header: %s", hipGetErrorString(e));
    for (int i = 0; i < BR_NQUEUES; ++i)
        if (words[i] != 0)
            return fail(BR_ERR_PLAN, "plan not at rest: ticket counter of queue %d is %d (a launch on it did not run to its end); call br_plan_rearm",
                        i, (int)words[i]);
    if (words[BR_PH_DONE - BR_PH_QTICKET] != 0)
        return fail(BR_ERR_PLAN, "plan not at rest: %d workgroups of a launch have left and the others have not; call br_plan_rearm",
                    (int)words[BR_PH_DONE - BR_PH_QTICKET]);
    return BR_OK;
}

int br_plan_rearm(int32_t* plan, void* stream) {
    if (!plan) return fail(BR_ERR_ARG, "null pointer");
    br_launch_plan_rearm(plan, static_cast<hipStream_t>(stream));
    return check_launch("br_plan_rearm");
}

// Address of this device's copy of the scratch array, looked up once per device (with that device current).
static int noalloc_scratch(void** out) {
    constexpr int kMaxDev = 64;
    static std::atomic<void*> ptrs[kMaxDev];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(BR_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDev) return fail(BR_ERR_HIP, "device index %d out of range", dev);
    void* ptr = ptrs[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) return fail(BR_ERR_HIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        ptrs[dev].store(ptr, std::memory_order_release);     // every thread gets the same address for a device
    }
    *out = ptr;
    return BR_OK;
}

static int plan_build(const uint8_t* valid, const int32_t* lens, int left_padded, int packed, int B, int M, int H, int Nq, int Nkv,
                      int32_t* plan, size_t plan_ints, void* stream) {
    if (B <= 0 || M <= 0 || H <= 0) return fail(BR_ERR_ARG, "B, M and H must be positive (got %d, %d, %d)", B, M, H);
    BrGeom g;
    int nw;
    if (!make_geom(Nq, Nkv, &g, &nw)) return fail(BR_ERR_ARG, "Nq=%d must be a positive multiple of Nkv=%d", Nq, Nkv);
    const int T = br_tokens_per_tile(g);
    if (!plan || (!valid && !lens)) return fail(BR_ERR_ARG, "null pointer");
    if (!aligned16(plan)) return fail(BR_ERR_ARG, "plan buffer must be 16-byte aligned");
    const size_t need = br_plan_total_ints(B, M, H, T);
    if (plan_ints < need) return fail(BR_ERR_SPACE, "plan buffer holds %zu ints, %zu needed", plan_ints, need);
    BrGeom g16;
    int nw16;
    make_geom(Nq, Nkv, &g16, &nw16, true);                  // the shape the 16-bit forward kernels run in
    if ((long long)br_plan_max_items(B, M, H, T) * (g16.NHG > g.NHG ? g16.NHG : g.NHG) >= (1 << 24))
        return fail(BR_ERR_ARG, "batch too large for one plan (B=%d, M=%d, H=%d)", B, M, H);
    const int n_cu = n_compute_units();
    if (n_cu <= 0) return fail(BR_ERR_HIP, "no HIP device");
    // (the set-up call of every request: look the no-alloc entry's scratch array up here, so that the entry itself
    // never has to - the first lookup on a device makes the runtime load the code object)
    void* scratch_ptr = nullptr;
    int src = noalloc_scratch(&scratch_ptr);
    if (src) return src;
    const int par = prefill_par(Nq, Nkv, n_cu);
    br_launch_plan(valid, lens, left_padded, packed, B, M, H, T, par, prefill_pool(Nq, Nkv, n_cu), plan, static_cast<hipStream_t>(stream));
    return check_launch("plan launch");
}

int br_plan_build(const uint8_t* valid, int B, int M, int H, int Nq, int Nkv, int32_t* plan, size_t plan_ints, void* stream) {
    if (!valid) return fail(BR_ERR_ARG, "attention mask must be provided");
    return plan_build(valid, nullptr, 1, 0, B, M, H, Nq, Nkv, plan, plan_ints, stream);
}

int br_plan_build_from_lengths(const int32_t* lens, int left_padded, int B, int M, int H, int Nq, int Nkv, int32_t* plan,
                               size_t plan_ints, void* stream) {
    if (!lens) return fail(BR_ERR_ARG, "block lengths must be provided");
    return plan_build(nullptr, lens, left_padded, 0, B, M, H, Nq, Nkv, plan, plan_ints, stream);
}

int br_plan_build_packed(const int32_t* lens, int B, int M, int H, int Nq, int Nkv, int32_t* plan, size_t plan_ints, void* stream) {
    if (!lens) return fail(BR_ERR_ARG, "block lengths must be provided");
    return plan_build(nullptr, lens, 1, 1, B, M, H, Nq, Nkv, plan, plan_ints, stream);
}

size_t br_prefill_workspace_bytes(int B, int Nq, int Nkv, int D) {
    BrGeom g;
    int nw;
    if (!make_geom(Nq, Nkv, &g, &nw) || B <= 0 || D <= 0) return 0;
    const int n_cu = n_compute_units();
    if (n_cu <= 0) return 0;
    const int pool = prefill_pool(Nq, Nkv, n_cu);
    size_t rows = slots_total(pool, g) * (size_t)nw * BR_RB;
    // (the 16-bit kernels may cut a head group differently from the fp32 kernel: enough for either)
    make_geom(Nq, Nkv, &g, &nw, true);
    const size_t rows16 = slots_total(pool, g) * (size_t)nw * BR_RB;
    rows = rows16 > rows ? rows16 : rows;
    return rows * (size_t)(D + 3) * sizeof(float);      // partial outputs, (max, sum) and the exact sum of every row
}

size_t br_score_partials_bytes(int B, int Nq, int M, int H, int score_rows) {
    if (B <= 0 || Nq <= 0 || M < 3 || H <= 0 || score_rows <= 0) return 0;
    return (size_t)B * Nq * score_rows * br_plan_tps(M, H) * 2 * sizeof(float);
}

static size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

size_t br_prefill_fp8qk_workspace_bytes(int B, int Nq, int Nkv, int D, int M, int64_t tokens) {
    const size_t base = br_prefill_workspace_bytes(B, Nq, Nkv, D);
    if (base == 0 || tokens <= 0 || M <= 0) return 0;
    return up256(base) + up256((size_t)Nkv * tokens * D) + up256((size_t)B * M * Nkv * 4) + up256((size_t)B * Nkv * 4);
}

// Everything optional about a forward call, in one place (the entry points below fill in what they expose).
struct PrefillExtras {
    void* ev_start = nullptr;
    void* ev_stop = nullptr;
    int score_rows = 0;                  // with score_part: the query block's last rows whose score partials are left
    float* score_part = nullptr;
    size_t score_part_bytes = 0;
    int64_t fp8_tokens = 0;              // > 0: Q K^T in fp8 (inputs bf16, K quantised into the workspace first); the length of
                                         // the token axis summed over the batch (B*M*H padded slots, or the packed token count)
    float* lse = nullptr;
    const int64_t* lse_strides = nullptr;
    const void* rope_cos = nullptr;
    const void* rope_sin = nullptr;
    const int64_t* rope_strides = nullptr;
    const int32_t* rank_rows = nullptr;  // with rank_scores: per-document scores of these rows, reduced in the finish launch
    int rank_R = 0;
    float rank_scale = 1.f;
    float* rank_scores = nullptr;
};

static PrefillExtras with_events(void* ev_start, void* ev_stop) {
    PrefillExtras x;
    x.ev_start = ev_start; x.ev_stop = ev_stop;
    return x;
}

static int prefill_impl(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv,
                        int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* out_strides, float scale, int dtype, void* workspace, size_t workspace_bytes,
                        void* stream, const PrefillExtras& x) {
    void* const ev_start = x.ev_start;
    void* const ev_stop = x.ev_stop;
    const int score_rows = x.score_part ? x.score_rows : 0;
    float* const score_part = x.score_part;
    const size_t score_part_bytes = x.score_part_bytes;
    const int64_t fp8_tokens = x.fp8_tokens;
    float* const lse = x.lse;
    const int64_t* const lse_strides = x.lse_strides;
    const void* const rope_cos = x.rope_cos;
    const void* const rope_sin = x.rope_sin;
    const int64_t* const rope_strides = x.rope_strides;
    int rc = check_common(B, Nq, Nkv, M, H, D, dtype);
    if (rc) return rc;
    if (rope_cos || rope_sin) {
        if (dtype == BR_DTYPE_F32 || fp8_tokens > 0) return fail(BR_ERR_ARG, "the rotary embedding of Q inside the attention kernel needs the bf16 or fp16 kernel");
        if (!rope_cos || !rope_sin || !rope_strides) return fail(BR_ERR_ARG, "cos, sin and their strides must be given together");
        if (!aligned16(rope_cos) || !aligned16(rope_sin)) return fail(BR_ERR_ARG, "cos and sin must be 16-byte aligned");
        if (rope_strides[0] < 0 || rope_strides[1] < D || rope_strides[0] % 8 || rope_strides[1] % 8 || rope_strides[0] >= (int64_t(1) << 31) ||
            rope_strides[1] >= (int64_t(1) << 31))
            return fail(BR_ERR_ARG, "cos/sin strides (batch, token) must be multiples of 16 bytes below 2^31 elements, rows dense");
    }
    if (lse && (dtype != BR_DTYPE_BF16 || fp8_tokens > 0 || !lse_strides)) return fail(BR_ERR_ARG, "the log-sum-exp output comes from the bf16 kernel only");
    if (score_part) {
        if (dtype == BR_DTYPE_F32) return fail(BR_ERR_ARG, "score partials come from the bf16 / fp16 kernel only; use br_doc_scores");
        if (M < 3) return fail(BR_ERR_ARG, "score partials need at least one document block (M=%d)", M);
        if (score_rows <= 0 || score_rows > H) return fail(BR_ERR_ARG, "score_rows=%d outside 1..H=%d", score_rows, H);
        if (!aligned16(score_part)) return fail(BR_ERR_ARG, "score_part must be 16-byte aligned");
        const size_t sneed = br_score_partials_bytes(B, Nq, M, H, score_rows);
        if (score_part_bytes < sneed) return fail(BR_ERR_SPACE, "score_part holds %zu bytes, %zu needed", score_part_bytes, sneed);
    }
    if (x.rank_rows || x.rank_scores) {
        if (!x.rank_rows || !x.rank_scores) return fail(BR_ERR_ARG, "the rows to score and the scores output must be given together");
        if (!score_part) return fail(BR_ERR_ARG, "per-document scores in the same call need the score partials buffer");
        if (x.rank_R <= 0 || x.rank_R > 16) return fail(BR_ERR_ARG, "R=%d rows not supported (1..16)", x.rank_R);
        if ((size_t)(M - 2) * sizeof(float) > 60 * 1024) return fail(BR_ERR_ARG, "too many documents (%d) for the score reduction", M - 2);
    }
    if (!q || !k || !v || !out || !plan) return fail(BR_ERR_ARG, "null pointer");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || !aligned16(plan) || !aligned16(workspace))
        return fail(BR_ERR_ARG, "q, k, v, out, plan and workspace must be 16-byte aligned");
    if ((rc = check_strides("q", q_strides, dtype)) || (rc = check_strides("k", k_strides, dtype)) ||
        (rc = check_strides("v", v_strides, dtype)) || (rc = check_strides("out", out_strides, dtype)))
        return rc;
    BrGeom g;
    int nw;
    make_geom(Nq, Nkv, &g, &nw, dtype != BR_DTYPE_F32);
    if (fp8_tokens > 0 && (dtype != BR_DTYPE_BF16 || D != 128))
        return fail(BR_ERR_ARG, "the fp8 Q K^T variant takes bf16 inputs with head dim 128");
    const size_t need = fp8_tokens > 0 ? br_prefill_fp8qk_workspace_bytes(B, Nq, Nkv, D, M, fp8_tokens) : br_prefill_workspace_bytes(B, Nq, Nkv, D);
    if (!workspace || workspace_bytes < need) return fail(BR_ERR_SPACE, "workspace holds %zu bytes, %zu needed", workspace_bytes, need);
    const int n_cu = n_compute_units();
    if (n_cu <= 0) return fail(BR_ERR_HIP, "no HIP device");

    BrPrefillParams p;
    p.q = q; p.k = k; p.v = v; p.out = out; p.plan = plan;
    const size_t rows = slots_total(prefill_pool(Nq, Nkv, n_cu), g) * (size_t)nw * BR_RB;
    p.part_o = static_cast<float*>(workspace);
    p.part_ml = p.part_o + rows * D;
    p.part_lx = p.part_ml + rows * 2;
    p.sq_b = q_strides[0]; p.sq_h = q_strides[1]; p.sq_t = q_strides[2];
    p.sk_b = k_strides[0]; p.sk_h = k_strides[1]; p.sk_t = k_strides[2];
    p.sv_b = v_strides[0]; p.sv_h = v_strides[1]; p.sv_t = v_strides[2];
    p.so_b = out_strides[0]; p.so_h = out_strides[1]; p.so_t = out_strides[2];
    for (const int64_t* st : {q_strides, k_strides, v_strides, out_strides})
        for (int i = 0; i < 3; ++i)
            if (st[i] < 0 || st[i] >= (int64_t(1) << 31)) return fail(BR_ERR_ARG, "strides must be below 2^31 elements (got %lld)", (long long)st[i]);
    p.q32_b = (unsigned)q_strides[0]; p.q32_h = (unsigned)q_strides[1]; p.q32_t = (unsigned)q_strides[2];
    p.k32_b = (unsigned)k_strides[0]; p.k32_h = (unsigned)k_strides[1]; p.k32_t = (unsigned)k_strides[2];
    p.v32_b = (unsigned)v_strides[0]; p.v32_h = (unsigned)v_strides[1]; p.v32_t = (unsigned)v_strides[2];
    p.o32_b = (unsigned)out_strides[0]; p.o32_h = (unsigned)out_strides[1]; p.o32_t = (unsigned)out_strides[2];
    p.B = B; p.Nq = Nq; p.Nkv = Nkv; p.M = M; p.H = H;
    p.geom = g;
    p.scale_log2 = scale * 1.4426950408889634f;
    p.score_part = score_part;
    p.score_R = score_part ? score_rows : 0;
    p.qk_scales = nullptr;
    p.rope_cos = rope_cos; p.rope_sin = rope_sin;
    p.rope_b = rope_cos ? (unsigned)rope_strides[0] : 0u;
    p.rope_t = rope_cos ? (unsigned)rope_strides[1] : 0u;
    p.k8 = nullptr;
    p.k8_b = p.k8_h = 0;
    p.lse = lse;
    p.lse_b = lse ? lse_strides[0] : 0;
    p.lse_h = lse ? lse_strides[1] : 0;
    int combine_grid = br_plan_max_comb(B) * g.NHG;
    if (combine_grid < B * M) combine_grid = B * M;
    if (combine_grid > 4 * n_cu) combine_grid = 4 * n_cu;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t e0 = static_cast<hipEvent_t>(ev_start), e1 = static_cast<hipEvent_t>(ev_stop);
    BrTileScoreParams rank = {};
    const BrTileScoreParams* rankp = nullptr;
    if (x.rank_scores) {
        rank.part = score_part; rank.plan = plan; rank.rows = x.rank_rows; rank.scores = x.rank_scores; rank.probs = nullptr;
        rank.B = B; rank.Nq = Nq; rank.M = M; rank.H = H; rank.R = x.rank_R; rank.Rw = score_rows;
        rank.out_scale = x.rank_scale;
        rankp = &rank;
    }
    int lrc;
    if (fp8_tokens > 0) {
        const bool packed = k_strides[0] == 0;
        const long long stot = packed ? fp8_tokens : fp8_tokens / B;        // tokens per batch entry of k8
        const long long k8_h = stot * D;
        const long long k8_b = packed ? 0 : (long long)Nkv * k8_h;
        if (k8_b >= (1LL << 32) || k8_h >= (1LL << 32)) return fail(BR_ERR_ARG, "fp8 staging strides must be below 2^32 bytes");
        char* w = static_cast<char*>(workspace) + up256(br_prefill_workspace_bytes(B, Nq, Nkv, D));
        void* k8 = w;
        w += up256((size_t)Nkv * fp8_tokens * D);
        unsigned* amax = reinterpret_cast<unsigned*>(w);
        w += up256((size_t)B * M * Nkv * 4);
        float* scales = reinterpret_cast<float*>(w);
        const long long sk[3] = {k_strides[0], k_strides[1], k_strides[2]};
        br_launch_quantize_fp8(k, plan, k8, amax, scales, sk, k8_b, k8_h, B, Nkv, M, H, D, s);
        p.k8 = k8;
        p.k8_b = (unsigned)k8_b; p.k8_h = (unsigned)k8_h;
        p.qk_scales = scales;
        lrc = br_launch_prefill_fp8qk(p, D, nw, n_cu, combine_grid, s, e0, e1, rankp);
    } else {
        lrc = dtype == BR_DTYPE_BF16  ? br_launch_prefill_bf16(p, D, nw, n_cu, combine_grid, s, e0, e1, rankp)
              : dtype == BR_DTYPE_F16 ? br_launch_prefill_f16(p, D, nw, n_cu, combine_grid, s, e0, e1, rankp)
                                      : br_launch_prefill_f32(p, D, nw, n_cu, combine_grid, s, e0, e1);
    }
    if (lrc) return fail(BR_ERR_ARG, "no kernel for head dim %d with %d query heads per kv head", D, g.G);
    return check_launch("prefill launch");
}

int br_prefill_fwd_events(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv,
                          int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* out_strides, float scale, int dtype, void* workspace, size_t workspace_bytes,
                          void* stream, void* ev_start, void* ev_stop) {
    return prefill_impl(q, k, v, out, plan, B, Nq, Nkv, M, H, D, q_strides, k_strides, v_strides, out_strides, scale, dtype,
                        workspace, workspace_bytes, stream, with_events(ev_start, ev_stop));
}

int br_prefill_fwd(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv, int M,
                   int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                   const int64_t* out_strides, float scale, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return prefill_impl(q, k, v, out, plan, B, Nq, Nkv, M, H, D, q_strides, k_strides, v_strides, out_strides, scale, dtype,
                        workspace, workspace_bytes, stream, PrefillExtras());
}

size_t br_prefill_noalloc_max_workspace_bytes(void) { return BR_NOALLOC_SCRATCH_BYTES; }

int br_prefill_fwd_noalloc(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv,
                           int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                           const int64_t* out_strides, float scale, int dtype, void* stream) {
    int rc = check_common(B, Nq, Nkv, M, H, D, dtype);
    if (rc) return rc;
    const size_t need = br_prefill_workspace_bytes(B, Nq, Nkv, D);
    if (need == 0) return fail(BR_ERR_HIP, "no HIP device");
    if (need > BR_NOALLOC_SCRATCH_BYTES)
        return fail(BR_ERR_SPACE, "br_prefill_fwd_noalloc: B=%d with %d/%d heads of dim %d needs %zu bytes of partials, the built-in scratch holds %zu; "
                                  "use br_prefill_fwd with a workspace, or a smaller batch", B, Nq, Nkv, D, need, (size_t)BR_NOALLOC_SCRATCH_BYTES);
    void* ws = nullptr;
    if ((rc = noalloc_scratch(&ws))) return rc;
    return prefill_impl(q, k, v, out, plan, B, Nq, Nkv, M, H, D, q_strides, k_strides, v_strides, out_strides, scale, dtype,
                        ws, need, stream, PrefillExtras());
}

int br_prefill_fwd_scores(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv,
                          int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* out_strides, float scale, int dtype, void* workspace, size_t workspace_bytes,
                          int score_rows, float* score_part, size_t score_part_bytes, void* stream, void* ev_start,
                          void* ev_stop) {
    if (!score_part) return fail(BR_ERR_ARG, "score_part must be provided");
    PrefillExtras x = with_events(ev_start, ev_stop);
    x.score_rows = score_rows; x.score_part = score_part; x.score_part_bytes = score_part_bytes;
    return prefill_impl(q, k, v, out, plan, B, Nq, Nkv, M, H, D, q_strides, k_strides, v_strides, out_strides, scale, dtype,
                        workspace, workspace_bytes, stream, x);
}

int br_prefill_fwd_ex(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv,
                      int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                      const int64_t* out_strides, float scale, int dtype, void* workspace, size_t workspace_bytes,
                      const BrPrefillOptions* opt, void* stream) {
    PrefillExtras x;
    if (opt) {
        if (opt->struct_bytes != sizeof(BrPrefillOptions))
            return fail(BR_ERR_ARG, "BrPrefillOptions.struct_bytes is %zu, this library's structure has %zu", opt->struct_bytes, sizeof(BrPrefillOptions));
        if (opt->fp8_tokens < 0) return fail(BR_ERR_ARG, "fp8_tokens must not be negative");
        if ((opt->rope_cos || opt->rope_sin) && !(opt->rope_cos && opt->rope_sin && opt->rope_strides))
            return fail(BR_ERR_ARG, "cos, sin and their strides must be given together");
        if (opt->lse && (!opt->lse_strides || opt->lse_strides[0] < 0 || opt->lse_strides[1] <= 0)) return fail(BR_ERR_ARG, "bad lse strides");
        x.ev_start = opt->ev_start; x.ev_stop = opt->ev_stop;
        x.score_rows = opt->score_rows; x.score_part = opt->score_part; x.score_part_bytes = opt->score_part_bytes;
        x.fp8_tokens = opt->fp8_tokens;
        x.lse = opt->lse; x.lse_strides = opt->lse_strides;
        x.rope_cos = opt->rope_cos; x.rope_sin = opt->rope_sin; x.rope_strides = opt->rope_strides;
        x.rank_rows = opt->rank_rows; x.rank_R = opt->rank_R; x.rank_scale = opt->rank_scale; x.rank_scores = opt->rank_scores;
    }
    return prefill_impl(q, k, v, out, plan, B, Nq, Nkv, M, H, D, q_strides, k_strides, v_strides, out_strides, scale, dtype,
                        workspace, workspace_bytes, stream, x);
}

int br_prefill_fwd_fp8qk(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv,
                         int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                         const int64_t* out_strides, float scale, int64_t tokens, void* workspace, size_t workspace_bytes,
                         int score_rows, float* score_part, size_t score_part_bytes, void* stream, void* ev_start, void* ev_stop) {
    if (tokens <= 0) return fail(BR_ERR_ARG, "tokens must be positive (got %lld)", (long long)tokens);
    PrefillExtras x = with_events(ev_start, ev_stop);
    x.score_rows = score_rows; x.score_part = score_part; x.score_part_bytes = score_part_bytes;
    x.fp8_tokens = tokens;
    return prefill_impl(q, k, v, out, plan, B, Nq, Nkv, M, H, D, q_strides, k_strides, v_strides, out_strides, scale,
                        BR_DTYPE_BF16, workspace, workspace_bytes, stream, x);
}

int br_prefill_fwd_lse(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv, int M,
                       int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                       const int64_t* out_strides, float scale, void* workspace, size_t workspace_bytes, float* lse,
                       const int64_t* lse_strides, void* stream) {
    if (!lse || !lse_strides) return fail(BR_ERR_ARG, "lse and its strides must be provided");
    if (lse_strides[0] < 0 || lse_strides[1] <= 0) return fail(BR_ERR_ARG, "bad lse strides");
    PrefillExtras x;
    x.lse = lse; x.lse_strides = lse_strides;
    return prefill_impl(q, k, v, out, plan, B, Nq, Nkv, M, H, D, q_strides, k_strides, v_strides, out_strides, scale, BR_DTYPE_BF16,
                        workspace, workspace_bytes, stream, x);
}

size_t br_prefill_bwd_workspace_bytes(int B, int Nq, int Nkv, int H, int D, int64_t token_slots) {
    if (B <= 0 || Nq <= 0 || Nkv <= 0 || H <= 0 || D <= 0 || token_slots <= 0) return 0;
    // fp32 dQ sums of the query block's rows and dK, dV sums of the prefix keys, then delta for every token slot and query head
    return up256((size_t)B * (Nq + 2 * Nkv) * H * D * sizeof(float)) + (size_t)token_slots * Nq * sizeof(float);
}

int br_prefill_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                   const int32_t* plan, int B, int Nq, int Nkv, int M, int H, int D, const int64_t* q_strides,
                   const int64_t* k_strides, const int64_t* v_strides, const int64_t* out_strides, const int64_t* dout_strides,
                   const int64_t* lse_strides, void* dq, void* dk, void* dv, const int64_t* dq_strides, const int64_t* dk_strides,
                   const int64_t* dv_strides, float scale, int64_t token_slots, void* workspace, size_t workspace_bytes,
                   void* stream) {
    int rc = check_common(B, Nq, Nkv, M, H, D, BR_DTYPE_BF16);
    if (rc) return rc;
    if (!q || !k || !v || !out || !dout || !lse || !plan || !dq || !dk || !dv || !lse_strides) return fail(BR_ERR_ARG, "null pointer");
    for (const void* ptr : {q, k, v, out, dout, (const void*)plan, (const void*)dq, (const void*)dk, (const void*)dv, (const void*)workspace})
        if (!aligned16(ptr)) return fail(BR_ERR_ARG, "tensors, plan and workspace must be 16-byte aligned");
    const int64_t* all[8] = {q_strides, k_strides, v_strides, out_strides, dout_strides, dq_strides, dk_strides, dv_strides};
    const char* names[8] = {"q", "k", "v", "out", "dout", "dq", "dk", "dv"};
    for (int i = 0; i < 8; ++i) {
        if ((rc = check_strides(names[i], all[i], BR_DTYPE_BF16))) return rc;
        for (int j = 0; j < 3; ++j)
            if (all[i][j] >= (int64_t(1) << 31)) return fail(BR_ERR_ARG, "strides must be below 2^31 elements (got %lld)", (long long)all[i][j]);
    }
    if (lse_strides[0] < 0 || lse_strides[1] <= 0) return fail(BR_ERR_ARG, "bad lse strides");
    const bool packed = q_strides[0] == 0;
    if (!packed && token_slots != (int64_t)B * M * H) return fail(BR_ERR_ARG, "token_slots=%lld, expected B*M*H=%lld", (long long)token_slots, (long long)B * M * H);
    if (token_slots <= 0) return fail(BR_ERR_ARG, "token_slots must be positive");
    // delta is kept in the workspace with lse's indexing: lse must be the dense (batch, head, token) array
    const int64_t per_b = packed ? token_slots : (int64_t)M * H;
    if (lse_strides[1] != per_b || lse_strides[0] != (packed ? 0 : (int64_t)Nq * per_b))
        return fail(BR_ERR_ARG, "lse must be dense: strides (%lld, %lld) expected", (long long)(packed ? 0 : (int64_t)Nq * per_b), (long long)per_b);
    const size_t need = br_prefill_bwd_workspace_bytes(B, Nq, Nkv, H, D, token_slots);
    if (!workspace || workspace_bytes < need) return fail(BR_ERR_SPACE, "workspace holds %zu bytes, %zu needed", workspace_bytes, need);
    const int n_cu = n_compute_units();
    if (n_cu <= 0) return fail(BR_ERR_HIP, "no HIP device");
    BrGeom g;
    int nw;
    make_geom(Nq, Nkv, &g, &nw);
    BrBwdParams p;
    p.q = q; p.k = k; p.v = v; p.out = out; p.dout = dout; p.plan = plan; p.lse = lse;
    p.lse_b = lse_strides[0]; p.lse_h = lse_strides[1];
    p.dq32 = static_cast<float*>(workspace);
    p.dk32 = p.dq32 + (size_t)B * Nq * H * D;
    p.dv32 = p.dk32 + (size_t)B * Nkv * H * D;
    p.delta = reinterpret_cast<float*>(static_cast<char*>(workspace) + up256((size_t)B * (Nq + 2 * Nkv) * H * D * sizeof(float)));
    if (((long long)M * B * Nkv + 7) * 4 * ((H + BR_BN - 1) / BR_BN) >= (1LL << 31)) return fail(BR_ERR_ARG, "batch too large for one backward launch");
    p.dq = dq; p.dk = dk; p.dv = dv;
    p.dq_b = dq_strides[0]; p.dq_h = dq_strides[1]; p.dq_t = dq_strides[2];
    p.dk_b = dk_strides[0]; p.dk_h = dk_strides[1]; p.dk_t = dk_strides[2];
    p.dv_b = dv_strides[0]; p.dv_h = dv_strides[1]; p.dv_t = dv_strides[2];
    p.q32_b = (unsigned)q_strides[0]; p.q32_h = (unsigned)q_strides[1]; p.q32_t = (unsigned)q_strides[2];
    p.k32_b = (unsigned)k_strides[0]; p.k32_h = (unsigned)k_strides[1]; p.k32_t = (unsigned)k_strides[2];
    p.v32_b = (unsigned)v_strides[0]; p.v32_h = (unsigned)v_strides[1]; p.v32_t = (unsigned)v_strides[2];
    p.o32_b = (unsigned)out_strides[0]; p.o32_h = (unsigned)out_strides[1]; p.o32_t = (unsigned)out_strides[2];
    p.g32_b = (unsigned)dout_strides[0]; p.g32_h = (unsigned)dout_strides[1]; p.g32_t = (unsigned)dout_strides[2];
    p.B = B; p.Nq = Nq; p.Nkv = Nkv; p.M = M; p.H = H;
    p.geom = g;
    p.scale = scale;
    p.scale_log2 = scale * 1.4426950408889634f;
    p.max_items = br_plan_max_items(B, M, H, br_tokens_per_tile(g));
    const int lrc = br_launch_bwd(p, D, nw, n_cu, static_cast<hipStream_t>(stream));
    if (lrc) return fail(BR_ERR_ARG, "no backward kernel for head dim %d with %d query heads per kv head (code %d)", D, g.G, lrc);
    return check_launch("backward launch");
}

int br_doc_scores_from_partials(const float* score_part, const int32_t* plan, const int32_t* rows, int R, int score_rows, int B,
                                int Nq, int M, int H, float out_scale, float* scores, float* probs, void* stream) {
    if (B <= 0 || Nq <= 0 || H <= 0) return fail(BR_ERR_ARG, "bad sizes B=%d Nq=%d H=%d", B, Nq, H);
    if (M < 3) return fail(BR_ERR_ARG, "per-document scores need at least one document block (M=%d)", M);
    if (R <= 0 || R > 16) return fail(BR_ERR_ARG, "R=%d rows not supported (1..16)", R);
    if (score_rows <= 0 || score_rows > H) return fail(BR_ERR_ARG, "score_rows=%d outside 1..H=%d", score_rows, H);
    if (!score_part || !plan || !rows || !scores) return fail(BR_ERR_ARG, "null pointer");
    if (br_launch_doc_scores_tiles(score_part, plan, rows, scores, probs, B, Nq, M, H, R, score_rows, out_scale,
                                   static_cast<hipStream_t>(stream)))
        return fail(BR_ERR_ARG, "too many documents (%d) for the score reduction", M - 2);
    return check_launch("score reduction launch");
}

size_t br_doc_scores_workspace_bytes(int B, int Nq, int M, int R) {
    if (B <= 0 || Nq <= 0 || M < 3 || R <= 0) return 0;
    return (size_t)B * Nq * R * (M - 2) * 2 * sizeof(float);
}

static int check_scores(const void* q, const void* k, const int32_t* plan, const int32_t* rows, int R, int B, int Nq, int Nkv,
                        int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, int dtype) {
    int rc = check_common(B, Nq, Nkv, M, H, D, dtype);
    if (rc) return rc;
    if (R <= 0 || R > 16) return fail(BR_ERR_ARG, "R=%d rows not supported (1..16)", R);
    if (!q || !k || !plan || !rows) return fail(BR_ERR_ARG, "null pointer");
    if (!aligned16(q) || !aligned16(k) || !aligned16(plan)) return fail(BR_ERR_ARG, "q, k and plan must be 16-byte aligned");
    if ((rc = check_strides("q", q_strides, dtype)) || (rc = check_strides("k", k_strides, dtype))) return rc;
    return BR_OK;
}

int br_doc_scores(const void* q, const void* k, const int32_t* plan, const int32_t* rows, int R, int B, int Nq, int Nkv, int M,
                  int H, int D, const int64_t* q_strides, const int64_t* k_strides, float scale, float out_scale, int dtype,
                  float* scores, float* probs, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_scores(q, k, plan, rows, R, B, Nq, Nkv, M, H, D, q_strides, k_strides, dtype);
    if (rc) return rc;
    if (M < 3) return fail(BR_ERR_ARG, "per-document scores need at least one document block (M=%d)", M);
    if (!scores) return fail(BR_ERR_ARG, "null pointer");
    const size_t need = br_doc_scores_workspace_bytes(B, Nq, M, R);
    if (!workspace || workspace_bytes < need) return fail(BR_ERR_SPACE, "workspace holds %zu bytes, %zu needed", workspace_bytes, need);
    const long long sq[3] = {q_strides[0], q_strides[1], q_strides[2]};
    const long long sk[3] = {k_strides[0], k_strides[1], k_strides[2]};
    BrGeom g;
    int nw;
    make_geom(Nq, Nkv, &g, &nw);
    br_launch_doc_scores(q, k, plan, rows, static_cast<float*>(workspace), scores, probs, sq, sk, B, Nq, Nkv, M, H, D, R,
                         br_tokens_per_tile(g), scale, out_scale, dtype, static_cast<hipStream_t>(stream));
    return check_launch("score launch");
}

int br_last_block_logits(const void* q, const void* k, const int32_t* plan, const int32_t* rows, int R, int B, int Nq, int Nkv,
                         int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, float scale, float neg,
                         int dtype, float* logits, void* stream) {
    int rc = check_scores(q, k, plan, rows, R, B, Nq, Nkv, M, H, D, q_strides, k_strides, dtype);
    if (rc) return rc;
    if (!logits) return fail(BR_ERR_ARG, "null pointer");
    const long long sq[3] = {q_strides[0], q_strides[1], q_strides[2]};
    const long long sk[3] = {k_strides[0], k_strides[1], k_strides[2]};
    BrGeom g;
    int nw;
    make_geom(Nq, Nkv, &g, &nw);
    br_launch_last_logits(q, k, plan, rows, logits, sq, sk, B, Nq, Nkv, M, H, D, R, br_tokens_per_tile(g), scale, neg,
                          dtype, static_cast<hipStream_t>(stream));
    return check_launch("logits launch");
}

int br_last_block_logits_bwd(const float* dlogits, const void* q, const void* k, const int32_t* plan, const int32_t* rows, int R, int B,
                             int Nq, int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, float scale,
                             int dtype, void* dq, const int64_t* dq_strides, void* dk, const int64_t* dk_strides, void* stream) {
    int rc = check_scores(q, k, plan, rows, R, B, Nq, Nkv, M, H, D, q_strides, k_strides, dtype);
    if (rc) return rc;
    if (!dlogits || !dq || !dk || !dq_strides || !dk_strides) return fail(BR_ERR_ARG, "null pointer");
    const long long sq[3] = {q_strides[0], q_strides[1], q_strides[2]};
    const long long sk[3] = {k_strides[0], k_strides[1], k_strides[2]};
    const long long sdq[3] = {dq_strides[0], dq_strides[1], dq_strides[2]};
    const long long sdk[3] = {dk_strides[0], dk_strides[1], dk_strides[2]};
    for (const long long* st : {sdq, sdk})
        for (int i = 0; i < 3; ++i)
            if (st[i] < 0) return fail(BR_ERR_ARG, "negative gradient stride");
    BrGeom g;
    int nw;
    make_geom(Nq, Nkv, &g, &nw);
    br_launch_last_logits_bwd(dlogits, q, k, plan, rows, dq, dk, sq, sk, sdq, sdk, B, Nq, Nkv, M, H, D, R, br_tokens_per_tile(g), scale,
                              dtype, static_cast<hipStream_t>(stream));
    return check_launch("score-logit gradient launch");
}


int br_rope_qk(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int B, int Nq, int Nkv, int S,
               int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* cs_strides, int dtype, void* stream) {
    if (dtype != BR_DTYPE_F32 && dtype != BR_DTYPE_BF16 && dtype != BR_DTYPE_F16) return fail(BR_ERR_ARG, "dtype must be fp32 (0), bf16 (1) or fp16 (2)");
    if (B <= 0 || Nq < 0 || Nkv <= 0 || S <= 0) return fail(BR_ERR_ARG, "B, Nkv and S must be positive, Nq not negative");
    if (D != 64 && D != 128) return fail(BR_ERR_ARG, "head dim %d not supported (64 or 128)", D);
    const int64_t zero3[3] = {0, 0, 0};
    if (Nq == 0) {       // K alone (Q is rotated by the attention kernel): the q arguments are not used
        q = k; q_out = k_out; q_strides = zero3;
    }
    if (!q || !k || !cos || !sin || !q_out || !k_out || !q_strides || !k_strides || !cs_strides) return fail(BR_ERR_ARG, "null pointer");
    if (!aligned16(q) || !aligned16(k) || !aligned16(cos) || !aligned16(sin) || !aligned16(q_out) || !aligned16(k_out))
        return fail(BR_ERR_ARG, "q, k, cos, sin and the outputs must be 16-byte aligned");
    int rc;
    if ((rc = check_strides("q", q_strides, dtype)) || (rc = check_strides("k", k_strides, dtype))) return rc;
    const int per16 = dtype == BR_DTYPE_F32 ? 4 : 8;
    if (cs_strides[0] % per16 || cs_strides[1] % per16 || cs_strides[0] < 0 || cs_strides[1] < 0)
        return fail(BR_ERR_ARG, "cos/sin strides must be non-negative multiples of 16 bytes");
    const int n_cu = n_compute_units();
    if (n_cu <= 0) return fail(BR_ERR_HIP, "no HIP device");
    const long long sq[3] = {q_strides[0], q_strides[1], q_strides[2]}, sk[3] = {k_strides[0], k_strides[1], k_strides[2]};
    const long long sc[2] = {cs_strides[0], cs_strides[1]};
    br_launch_rope(q, k, cos, sin, q_out, k_out, B, Nq, Nkv, S, D, sq, sk, sc, dtype, n_cu, static_cast<hipStream_t>(stream));
    return check_launch("rotary embedding launch");
}

int br_rmsnorm(const void* x, const void* weight, void* out, int64_t rows, int hidden, int64_t x_row_stride, int64_t out_row_stride,
               float eps, int dtype, void* stream) {
    if (dtype != BR_DTYPE_F32 && dtype != BR_DTYPE_BF16) return fail(BR_ERR_ARG, "dtype must be fp32 (0) or bf16 (1)");
    if (rows < 0 || hidden <= 0) return fail(BR_ERR_ARG, "rows and hidden must be positive");
    const int per16 = dtype == BR_DTYPE_F32 ? 4 : 8;
    if (hidden % per16 || x_row_stride % per16 || out_row_stride % per16 || x_row_stride < hidden || out_row_stride < hidden)
        return fail(BR_ERR_ARG, "hidden size and row strides must be multiples of 16 bytes, rows must not overlap");
    if (!x || !weight || !out) return fail(BR_ERR_ARG, "null pointer");
    if (!aligned16(x) || !aligned16(weight) || !aligned16(out)) return fail(BR_ERR_ARG, "x, weight and out must be 16-byte aligned");
    if (rows == 0) return BR_OK;
    const int n_cu = n_compute_units();
    if (n_cu <= 0) return fail(BR_ERR_HIP, "no HIP device");
    if (br_launch_rmsnorm(x, weight, out, rows, hidden, x_row_stride, out_row_stride, eps, dtype, n_cu, static_cast<hipStream_t>(stream)))
        return fail(BR_ERR_ARG, "hidden size %d too large for the RMSNorm kernel", hidden);
    return check_launch("RMSNorm launch");
}

int br_silu_mul(const void* gate, const void* up, void* out, int64_t n, int dtype, void* stream) {
    if (dtype != BR_DTYPE_F32 && dtype != BR_DTYPE_BF16) return fail(BR_ERR_ARG, "dtype must be fp32 (0) or bf16 (1)");
    const int per16 = dtype == BR_DTYPE_F32 ? 4 : 8;
    if (n < 0 || n % per16) return fail(BR_ERR_ARG, "the element count must be a multiple of 16 bytes");
    if (!gate || !up || !out) return fail(BR_ERR_ARG, "null pointer");
    if (!aligned16(gate) || !aligned16(up) || !aligned16(out)) return fail(BR_ERR_ARG, "gate, up and out must be 16-byte aligned");
    if (n == 0) return BR_OK;
    const int n_cu = n_compute_units();
    if (n_cu <= 0) return fail(BR_ERR_HIP, "no HIP device");
    br_launch_silu_mul(gate, up, out, n, dtype, n_cu, static_cast<hipStream_t>(stream));
    return check_launch("SiLU gate launch");
}

}  // extern "C"
