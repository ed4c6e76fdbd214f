// Block-sparse prefill attention with Q K^T in fp8 e4m3 (per-head absmax scales) and P V in bf16:
// quantisation kernels and the fp8 instances of the prefill kernel (templates in
// br_prefill_mfma_impl.h).  Inputs stay bf16; Q and K are quantised into caller-provided scratch.
//
//   br_absmax_kernel   max |x| over the real tokens of every (sequence, head) of Q and of K
//   br_quant_kernel    x * 448 / absmax -> e4m3 (448 is the largest e4m3 value), written on the same
//                      token axis as the input; the dequantisation scale absmax / 448 per
//                      (sequence, head) goes to the scale table the attention kernel reads
// The attention kernel multiplies the two scales of its (sequence, query head, kv head) into the
// softmax scale, so the fp8 products need no further correction.
#include "br_prefill_mfma_impl.h"

namespace {

struct BrQuantParams {
    const __bf16* q;
    const __bf16* k;
    const int* plan;
    unsigned char* q8;
    unsigned char* k8;
    unsigned* amax;      // [B][Nq + Nkv]: bit patterns of non-negative floats (ordered like unsigned ints)
    float* scales;       // [B][Nq] then [B][Nkv]: dequantisation scales
    long long sq_b, sq_h, sq_t, sk_b, sk_h, sk_t;        // input strides (elements)
    long long q8_b, q8_h, k8_b, k8_h;                    // output strides (bytes); token stride is D
    int B, Nq, Nkv, M, H, D;
};

__global__ void br_zero_u32_kernel(unsigned* p, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// One workgroup per (block of a sequence, head): the block table tells where its real tokens are.
template <bool WRITE>
__global__ __launch_bounds__(256) void br_quant_pass_kernel(BrQuantParams p) {
    const int bm = blockIdx.x, hh = blockIdx.y;
    const int b = bm / p.M;
    const int* len = p.plan + br_plan_off_len(p.B, p.M);
    const int* tok = p.plan + br_plan_off_tok(p.B, p.M);
    const int L = len[bm], t0 = tok[bm];
    const bool is_q = hh < p.Nq;
    const int h = is_q ? hh : hh - p.Nq;
    const __bf16* src = is_q ? p.q + (long long)b * p.sq_b + (long long)h * p.sq_h : p.k + (long long)b * p.sk_b + (long long)h * p.sk_h;
    const long long st = is_q ? p.sq_t : p.sk_t;
    const int c8 = p.D / 8;                               // 16-byte pieces per row
    float inv = 0.f;
    unsigned char* dst = nullptr;
    if (WRITE) {
        const float a = __uint_as_float(p.amax[b * (p.Nq + p.Nkv) + hh]);
        inv = a > 0.f ? 448.f / a : 0.f;
        dst = is_q ? p.q8 + (long long)b * p.q8_b + (long long)h * p.q8_h : p.k8 + (long long)b * p.k8_b + (long long)h * p.k8_h;
        if (bm % p.M == 0 && threadIdx.x == 0)
            p.scales[is_q ? (long long)b * p.Nq + h : (long long)p.B * p.Nq + (long long)b * p.Nkv + h] = a / 448.f;
    }
    float mx = 0.f;
    for (int i = threadIdx.x; i < L * c8; i += blockDim.x) {
        const int r = i / c8, c = i - r * c8;
        const uint4 u = *reinterpret_cast<const uint4*>(src + (long long)(t0 + r) * st + c * 8);
        const unsigned w[4] = {u.x, u.y, u.z, u.w};
        float x[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            x[2 * j] = __uint_as_float(w[j] << 16);
            x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
        if (WRITE) {
            int lo = 0, hi = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) x[j] = fminf(fmaxf(x[j] * inv, -448.f), 448.f);
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
    if (!WRITE) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        // NaN never wins fmaxf; a non-finite maximum would make every scale useless, so keep it finite
        if ((threadIdx.x & 63) == 0 && mx > 0.f) atomicMax(&p.amax[b * (p.Nq + p.Nkv) + hh], __float_as_uint(fminf(mx, 3.0e38f)));
    }
}

template <int D, int NW>
void launch8(const BrPrefillParams& p, int grid, hipStream_t stream) {
    hipLaunchKernelGGL((br_prefill_mfma_kernel<D, NW, true>), dim3(grid), dim3(NW * 64), 0, stream, p);
}

}  // namespace

// Quantise Q and K of a bf16 request into q8/k8 (same token axis, (heads, tokens, D) bytes per batch
// entry) and fill the scale table.  amax: B*(Nq+Nkv) uint32 scratch.
void br_launch_quantize_fp8(const void* q, const void* k, const int* plan, void* q8, void* k8, unsigned* amax, float* scales,
                            const long long* sq, const long long* sk, long long q8_b, long long q8_h, long long k8_b, long long k8_h,
                            int B, int Nq, int Nkv, int M, int H, int D, hipStream_t stream) {
    BrQuantParams p;
    p.q = static_cast<const __bf16*>(q); p.k = static_cast<const __bf16*>(k); p.plan = plan;
    p.q8 = static_cast<unsigned char*>(q8); p.k8 = static_cast<unsigned char*>(k8); p.amax = amax; p.scales = scales;
    p.sq_b = sq[0]; p.sq_h = sq[1]; p.sq_t = sq[2]; p.sk_b = sk[0]; p.sk_h = sk[1]; p.sk_t = sk[2];
    p.q8_b = q8_b; p.q8_h = q8_h; p.k8_b = k8_b; p.k8_h = k8_h;
    p.B = B; p.Nq = Nq; p.Nkv = Nkv; p.M = M; p.H = H; p.D = D;
    const int n = B * (Nq + Nkv);
    hipLaunchKernelGGL(br_zero_u32_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, amax, n);
    hipLaunchKernelGGL(br_quant_pass_kernel<false>, dim3(B * M, Nq + Nkv), dim3(256), 0, stream, p);
    hipLaunchKernelGGL(br_quant_pass_kernel<true>, dim3(B * M, Nq + Nkv), dim3(256), 0, stream, p);
}

// The prefill kernel on fp8 Q/K (p.q, p.k point at the quantised tensors, strides in bytes) followed by
// the split merge.  Returns 0 on success, -1 if (D, NW) has no instantiation (only D = 128 is built).
int br_launch_prefill_fp8qk(const BrPrefillParams& p, int D, int NW, int n_cu, int combine_grid, hipStream_t stream,
                            hipEvent_t ev_start, hipEvent_t ev_stop) {
    const int per_cu = NW <= 4 ? 2 : 1;
    const int grid = n_cu * per_cu;
    if (D != 128) return -1;
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
    hipLaunchKernelGGL((br_finish_kernel<128>), dim3(combine_grid), dim3(256), 0, stream, p, NW);
    return 0;
}
