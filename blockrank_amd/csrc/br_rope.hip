// Rotary position embedding of Q and K in one pass: the step in front of the attention kernel.
// out = x * cos + rotate_half(x) * sin with rotate_half(x) = (-x[D/2:], x[:D/2]) - the Hugging Face
// convention (transformers models/mistral/modeling_mistral.py: rotate_half, apply_rotary_pos_emb), which
// the models BlockRank ranks with apply to the projected Q and K before every attention call.  There it
// is four multiplications, a negation, a concatenation and two additions per tensor, each a pass over
// memory; here Q and K are read once and written once, straight into the (batch, token, head, dim)
// layout the attention kernels address through strides.  Arithmetic in fp32, one rounding at the end.
#include "br_common.h"

namespace {

struct BrRopeParams {
    const void* q;
    const void* k;
    const void* cos;
    const void* sin;
    void* q_out;
    void* k_out;
    long long sq_b, sq_h, sq_t;     // element strides of q (batch, head, token); the last dim is dense
    long long sk_b, sk_h, sk_t;
    long long sc_b, sc_t;           // of cos and sin (batch, token); a batch stride of 0 broadcasts
    int B, Nq, Nkv, S, D;
};

template <typename T> struct Vec16;
template <> struct Vec16<__bf16> { static constexpr int N = 8; };
template <> struct Vec16<_Float16> { static constexpr int N = 8; };
template <> struct Vec16<float> { static constexpr int N = 4; };

template <typename T>
__device__ inline void load16(const T* p, float (&f)[Vec16<T>::N]) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    const T* e = reinterpret_cast<const T*>(&u);
#pragma unroll
    for (int i = 0; i < Vec16<T>::N; ++i) f[i] = (float)e[i];
}
template <typename T>
__device__ inline void store16(T* p, const float (&f)[Vec16<T>::N]) {
    uint4 u;
    T* e = reinterpret_cast<T*>(&u);
#pragma unroll
    for (int i = 0; i < Vec16<T>::N; ++i) e[i] = (T)f[i];
    *reinterpret_cast<uint4*>(p) = u;
}

// One thread: one 16-byte piece of the first half of a head's row and the matching piece of the second half.
template <typename T>
__global__ __launch_bounds__(256) void br_rope_kernel(BrRopeParams p) {
    constexpr int V = Vec16<T>::N;
    const int half = p.D / 2;
    const int ppr = half / V;                        // pieces per half row
    const int NH = p.Nq + p.Nkv;
    const long long total = (long long)p.B * p.S * NH * ppr;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(i % ppr);
        long long r = i / ppr;
        const int h = (int)(r % NH);
        r /= NH;
        const int t = (int)(r % p.S);
        const int b = (int)(r / p.S);
        const bool is_q = h < p.Nq;
        const int hh = is_q ? h : h - p.Nq;
        const T* x = is_q ? reinterpret_cast<const T*>(p.q) + b * p.sq_b + hh * p.sq_h + t * p.sq_t
                          : reinterpret_cast<const T*>(p.k) + b * p.sk_b + hh * p.sk_h + t * p.sk_t;
        T* o = is_q ? reinterpret_cast<T*>(p.q_out) + (((long long)b * p.S + t) * p.Nq + hh) * p.D
                    : reinterpret_cast<T*>(p.k_out) + (((long long)b * p.S + t) * p.Nkv + hh) * p.D;
        const T* cs = reinterpret_cast<const T*>(p.cos) + b * p.sc_b + t * p.sc_t;
        const T* sn = reinterpret_cast<const T*>(p.sin) + b * p.sc_b + t * p.sc_t;
        float x1[V], x2[V], c1[V], c2[V], s1[V], s2[V], o1[V], o2[V];
        load16(x + c * V, x1);
        load16(x + half + c * V, x2);
        load16(cs + c * V, c1);
        load16(cs + half + c * V, c2);
        load16(sn + c * V, s1);
        load16(sn + half + c * V, s2);
#pragma unroll
        for (int e = 0; e < V; ++e) {
            o1[e] = x1[e] * c1[e] - x2[e] * s1[e];
            o2[e] = x2[e] * c2[e] + x1[e] * s2[e];
        }
        store16(o + c * V, o1);
        store16(o + half + c * V, o2);
    }
}

}  // namespace

// dtype: 0 fp32, 1 bf16, 2 fp16 (q, k, cos, sin and the outputs alike).
int br_launch_rope(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int B, int Nq, int Nkv, int S,
                   int D, const long long* sq, const long long* sk, const long long* sc, int dtype, int n_cu, hipStream_t stream) {
    BrRopeParams p;
    p.q = q; p.k = k; p.cos = cos; p.sin = sin; p.q_out = q_out; p.k_out = k_out;
    p.sq_b = sq[0]; p.sq_h = sq[1]; p.sq_t = sq[2];
    p.sk_b = sk[0]; p.sk_h = sk[1]; p.sk_t = sk[2];
    p.sc_b = sc[0]; p.sc_t = sc[1];
    p.B = B; p.Nq = Nq; p.Nkv = Nkv; p.S = S; p.D = D;
    const int V = dtype == 0 ? 4 : 8;
    const long long total = (long long)B * S * (Nq + Nkv) * (D / 2 / V);
    long long blocks = (total + 255) / 256;
    const long long cap = (long long)n_cu * 32;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    if (dtype == 0)
        hipLaunchKernelGGL(br_rope_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    else if (dtype == 1)
        hipLaunchKernelGGL(br_rope_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(br_rope_kernel<_Float16>, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    return 0;
}
