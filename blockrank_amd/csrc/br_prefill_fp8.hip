// Block-sparse prefill attention with Q K^T in fp8 e4m3 and P V in bf16: the quantisation of K and the fp8
// instances of the prefill kernel (templates in br_prefill_mfma_impl.h).  Inputs stay bf16.
//
//   K   one scale per (sequence, kv head): br_quant_pass_kernel<false> takes max |x| over the real tokens of every block,
//       br_quant_pass_kernel<true> writes x / scale as e4m3 into caller-provided scratch on the same token axis,
//       with scale the power of two that puts the maximum into [128, 256) (e4m3 reaches 448; a power of two
//       makes the division exact), and the scale into the table the attention kernel reads.  K is the small operand (1/4 to 1/7 of Q's volume with grouped heads).
//   Q   never touched here: the attention kernel reads the bf16 rows it reads anyway and converts them in
//       registers, each query row with its own power-of-two scale (a lane owns a row, so the scale is a per-lane
//       factor of the softmax scale).
// The query block's items (the rows the document scores are read from) run on the bf16 Q and K: their
// logits, and so the scores, are those of the bf16 kernel.
#include "br_prefill_mfma_impl.h"

namespace {

struct BrQuantParams {
    const __bf16* k;
    const int* plan;
    unsigned char* k8;
    unsigned* amax;      // [B][M][Nkv]: per block, bit patterns of non-negative floats (ordered like unsigned ints)
    float* scales;       // [B][Nkv]: dequantisation scales
    long long sk_b, sk_h, sk_t;        // input strides (elements)
    long long k8_b, k8_h;              // output strides (bytes); token stride is D
    int B, Nkv, M, H, D;
};

// One workgroup per (block of a sequence, kv head): the block table tells where its real tokens are.
// WRITE = false: max |x| of the block into amax[b][m][h] (every workgroup owns its slot: nothing to clear, no atomics).
// WRITE = true: the sequence's maximum from the M slots, then x / scale as e4m3.
// A thread keeps UNR 16-byte loads in flight: the passes are short chains of dependent memory round trips otherwise.
template <bool WRITE>
__global__ __launch_bounds__(256) void br_quant_pass_kernel(BrQuantParams p) {
    constexpr int UNR = 8;
    __shared__ float s_red[4];
    const int bm = blockIdx.x, h = blockIdx.y;
    const int b = bm / p.M;
    const int* len = p.plan + br_plan_off_len(p.B, p.M);
    const int* tok = p.plan + br_plan_off_tok(p.B, p.M);
    const int L = len[bm], t0 = tok[bm];
    const __bf16* src = p.k + (long long)b * p.sk_b + (long long)h * p.sk_h;
    const long long st = p.sk_t;
    const int c8 = p.D / 8;                               // 16-byte pieces per row
    float inv = 0.f;
    unsigned char* dst = nullptr;
    if (WRITE) {
        // the sequence's maximum: bit patterns of non-negative floats order like unsigned integers
        unsigned am = 0u;
        for (int m = threadIdx.x; m < p.M; m += blockDim.x) {
            const unsigned v = p.amax[((long long)b * p.M + m) * p.Nkv + h];
            am = v > am ? v : am;
        }
        float mx = __uint_as_float(am);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
        float sc;
        br_pow2_scale(mx, sc, inv);
        dst = p.k8 + (long long)b * p.k8_b + (long long)h * p.k8_h;
        if (bm % p.M == 0 && threadIdx.x == 0) p.scales[(long long)b * p.Nkv + h] = sc;
    }
    float mx = 0.f;
    const int n = L * c8;
    for (int i0 = threadIdx.x; i0 < n; i0 += UNR * blockDim.x) {
        uint4 u[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const int i = i0 + k * blockDim.x;
            const int ii = i < n ? i : i0;                  // a valid address for the lanes past the end
            const int r = ii / c8, c = ii - r * c8;
            u[k] = *reinterpret_cast<const uint4*>(src + (long long)(t0 + r) * st + c * 8);
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const int i = i0 + k * blockDim.x;
            if (i >= n) continue;
            const int r = i / c8, c = i - r * c8;
            const unsigned w[4] = {u[k].x, u[k].y, u[k].z, u[k].w};
            float x[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                x[2 * j] = __uint_as_float(w[j] << 16);
                x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
            }
            if (WRITE) {
                int lo = 0, hi = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) x[j] *= inv;           // below 256 in magnitude
                lo = __builtin_amdgcn_cvt_pk_fp8_f32(x[0], x[1], lo, false);
                lo = __builtin_amdgcn_cvt_pk_fp8_f32(x[2], x[3], lo, true);
                hi = __builtin_amdgcn_cvt_pk_fp8_f32(x[4], x[5], hi, false);
                hi = __builtin_amdgcn_cvt_pk_fp8_f32(x[6], x[7], hi, true);
                *reinterpret_cast<int2*>(dst + (long long)(t0 + r) * p.D + c * 8) = make_int2(lo, hi);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) mx = fmaxf(mx, fabsf(x[j]));
            }
        }
    }
    if (!WRITE) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = mx;
        __syncthreads();
        // NaN never wins fmaxf; a non-finite maximum would make every scale useless, so keep it finite
        if (threadIdx.x == 0)
            p.amax[(long long)bm * p.Nkv + h] = __float_as_uint(fminf(fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3])), 3.0e38f));
    }
}

template <int D, int NW>
void launch8(const BrPrefillParams& p, int grid, hipStream_t stream) {
    hipLaunchKernelGGL((br_prefill_mfma_kernel<D, NW, true, true, false>), dim3(grid), dim3(NW * 64), 0, stream, p);
}

}  // namespace

// Quantise K of a bf16 request into k8 (same token axis, (heads, tokens, D) bytes per batch entry) and fill
// the scale table.  amax: B*M*Nkv uint32 scratch (no initialisation needed).
void br_launch_quantize_fp8(const void* k, const int* plan, void* k8, unsigned* amax, float* scales, const long long* sk,
                            long long k8_b, long long k8_h, int B, int Nkv, int M, int H, int D, hipStream_t stream) {
    BrQuantParams p;
    p.k = static_cast<const __bf16*>(k); p.plan = plan;
    p.k8 = static_cast<unsigned char*>(k8); p.amax = amax; p.scales = scales;
    p.sk_b = sk[0]; p.sk_h = sk[1]; p.sk_t = sk[2];
    p.k8_b = k8_b; p.k8_h = k8_h;
    p.B = B; p.Nkv = Nkv; p.M = M; p.H = H; p.D = D;
    hipLaunchKernelGGL(br_quant_pass_kernel<false>, dim3(B * M, Nkv), dim3(256), 0, stream, p);
    hipLaunchKernelGGL(br_quant_pass_kernel<true>, dim3(B * M, Nkv), dim3(256), 0, stream, p);
}

// The prefill kernel with fp8 logits (p.k8: the quantised K, p.qk_scales: its scales) followed by
// the split merge (with the score reduction ``rank`` asks for, if any).  Returns 0 on success, -1 if (D, NW) has no
// instantiation (only D = 128 is built), 1 if the score reduction does not fit; nothing is launched then.
int br_launch_prefill_fp8qk(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                            hipEvent_t ev_start, hipEvent_t ev_stop, const BrTileScoreParams* rank) {
    const int per_cu = NW <= 4 ? 2 : 1;
    const int grid = n_cu * per_cu;
    if (D != 128 || NW < 4 || NW > 8) return -1;
    if (rank && (size_t)(rank->M - 2) * sizeof(float) > 60 * 1024) return 1;
    if (ev_start) (void)hipEventRecord(ev_start, stream);
    switch (NW) {
        case 4: launch8<128, 4>(p, grid, stream); break;
        case 5: launch8<128, 5>(p, grid, stream); break;
        case 6: launch8<128, 6>(p, grid, stream); break;
        case 7: launch8<128, 7>(p, grid, stream); break;
        case 8: launch8<128, 8>(p, grid, stream); break;
        default: return -1;
    }
    if (ev_stop) (void)hipEventRecord(ev_stop, stream);
    return br_launch_finish<128>(p, NW, combine_grid, rank, stream);
}
