// Two elementwise steps of the decoder layers around the attention, each in one pass over memory:
//   RMSNorm      y = w * (x * rsqrt(mean(x^2) + eps))   (transformers models/mistral/modeling_mistral.py,
//                MistralRMSNorm.forward; the same class in the Llama and Qwen2 model files) - there: a cast
//                to fp32, a power, a mean, an addition, a reciprocal square root, two multiplications and
//                a cast back, each a kernel over the (tokens, hidden) activations;
//   SiLU gate    y = silu(gate) * up                     (MistralMLP.forward: act_fn(gate_proj(x)) * up_proj(x)).
// The ranking forward of scripts/eval_attn.py:139-151 runs both in every decoder layer; at the Mistral-7B
// shape they take 17 % of the GPU time of a forward pass.  Rounding follows the model file's order: for bf16
// tensors the normalised value is rounded to bf16 before it is multiplied by the weight, silu(gate) is
// rounded before it is multiplied by up.
#include "br_common.h"

namespace {

struct BrNormParams {
    const void* x;
    const void* w;
    void* out;
    long long rows, sx, so;     // row strides in elements
    int hidden;
    float eps;
};

template <typename T> struct Vec16;
template <> struct Vec16<__bf16> { static constexpr int N = 8; };
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

// One wave per row; a lane keeps its 16-byte pieces of the row (at most MAXC) in registers between the
// sum of squares and the scaling, so the row is read once.
template <typename T, int MAXC>
__global__ __launch_bounds__(256) void br_rmsnorm_kernel(BrNormParams p) {
    constexpr int V = Vec16<T>::N;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int chunks = p.hidden / V;
    const float inv_h = 1.0f / (float)p.hidden;
    for (long long row = (long long)blockIdx.x * 4 + wave; row < p.rows; row += (long long)gridDim.x * 4) {
        const T* x = reinterpret_cast<const T*>(p.x) + row * p.sx;
        T* o = reinterpret_cast<T*>(p.out) + row * p.so;
        float v[MAXC][V];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int c = lane + 64 * i;
            if (c < chunks) {
                load16(x + c * V, v[i]);
#pragma unroll
                for (int e = 0; e < V; ++e) ss += v[i][e] * v[i][e];
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
        const float r = 1.0f / sqrtf(ss * inv_h + p.eps);
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int c = lane + 64 * i;
            if (c < chunks) {
                float w[V], y[V];
                load16(reinterpret_cast<const T*>(p.w) + c * V, w);
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = w[e] * (float)(T)(v[i][e] * r);
                store16(o + c * V, y);
            }
        }
    }
}

// A thread takes four 16-byte pieces 4 KiB apart per iteration, all eight loads issued before the arithmetic.
template <typename T>
__global__ __launch_bounds__(256) void br_silu_mul_kernel(const T* gate, const T* up, T* out, long long n16) {
    constexpr int V = Vec16<T>::N, U = 4;
    const long long tiles = (n16 + U * 256 - 1) / (U * 256);        // a workgroup takes U * 4 KiB of contiguous memory at a time
    for (long long tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const long long i0 = tile * (U * 256) + threadIdx.x;
        constexpr long long stride = 256;
        float g[U][V], u[U][V];
#pragma unroll
        for (int k = 0; k < U; ++k) {
            const long long i = i0 + k * stride;
            if (i < n16) {
                load16(gate + i * V, g[k]);
                load16(up + i * V, u[k]);
            }
        }
#pragma unroll
        for (int k = 0; k < U; ++k) {
            const long long i = i0 + k * stride;
            if (i < n16) {
                float y[V];
#pragma unroll
                for (int e = 0; e < V; ++e) y[e] = (float)(T)(g[k][e] / (1.0f + __expf(-g[k][e]))) * u[k][e];
                store16(out + i * V, y);
            }
        }
    }
}

template <typename T>
int launch_norm(const BrNormParams& p, int n_cu, hipStream_t stream) {
    const int chunks = p.hidden / Vec16<T>::N;
    long long blocks = (p.rows + 3) / 4;
    const long long cap = (long long)n_cu * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    if (chunks <= 64 * 8) hipLaunchKernelGGL((br_rmsnorm_kernel<T, 8>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
    else if (chunks <= 64 * 16) hipLaunchKernelGGL((br_rmsnorm_kernel<T, 16>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
    else if (chunks <= 64 * 32) hipLaunchKernelGGL((br_rmsnorm_kernel<T, 32>), dim3((unsigned)blocks), dim3(256), 0, stream, p);
    else return -1;
    return 0;
}

}  // namespace

// dtype: 0 fp32, 1 bf16.  Returns -1 if the row is too long for the kernel (more than 2048 16-byte pieces).
int br_launch_rmsnorm(const void* x, const void* w, void* out, long long rows, int hidden, long long sx, long long so, float eps, int dtype,
                      int n_cu, hipStream_t stream) {
    BrNormParams p;
    p.x = x; p.w = w; p.out = out; p.rows = rows; p.sx = sx; p.so = so; p.hidden = hidden; p.eps = eps;
    return dtype == 0 ? launch_norm<float>(p, n_cu, stream) : launch_norm<__bf16>(p, n_cu, stream);
}

void br_launch_silu_mul(const void* gate, const void* up, void* out, long long n, int dtype, int n_cu, hipStream_t stream) {
    const int V = dtype == 0 ? 4 : 8;
    const long long n16 = n / V;
    long long blocks = (n16 + 1023) / 1024;
    const long long cap = (long long)n_cu * 32;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    if (dtype == 0)
        hipLaunchKernelGGL(br_silu_mul_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<const float*>(gate),
                           static_cast<const float*>(up), static_cast<float*>(out), n16);
    else
        hipLaunchKernelGGL(br_silu_mul_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<const __bf16*>(gate),
                           static_cast<const __bf16*>(up), static_cast<__bf16*>(out), n16);
}
