// What joins sub-layers' results before they enter the residual stream:
//
//  * gated_branches_kernel: out = sigmoid(g1 + b1) * (A + a_bias) + sigmoid(g2 + b2) * F, element by element in
//    float: two sub-layers that read the same normed rows (a parallel layer), each multiplied by a gate of its own
//    that is a projection of those rows; [g1 | g2] are the columns of one product, [b1 | b2] its bias.  A and F
//    may come as float partial sums [parts][n][H] of a split product; F (and its gate) may be absent.
//  * bias_sum_kernel: out = sum of the parts + bias, for a consumer that knows nothing of biases.
//  * scaled_branches_kernel: out = sa * wa[c] * (A + a_bias) + sf * wf[c] * (F + f_bias): two results that are added
//    with a number each (two mixers side by side whose sum is weighted) and / or a weight a column each (a layer
//    scale on the results of a parallel layer's two sub-layers); wa, wf, F may be absent.
#include "common.h"

template <typename GT, typename AT, typename FT>
__global__ __launch_bounds__(256) void gated_branches_kernel(const GT* __restrict__ g, long ldg,
                                                             const float* __restrict__ g_bias,
                                                             const AT* __restrict__ a, int a_parts, long a_stride,
                                                             const float* __restrict__ a_bias,
                                                             const FT* __restrict__ f, int f_parts, long f_stride,
                                                             const float* __restrict__ f_bias,
                                                             float* __restrict__ out, long total, int H) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const long t = i / H;
        const int c = (int)(i - t * H);
        float av = a_bias ? a_bias[c] : 0.f;
        for (int p = 0; p < a_parts; ++p) av += to_f32(a[(long)p * a_stride + i]);
        const float g1 = to_f32(g[t * ldg + c]) + (g_bias ? g_bias[c] : 0.f);
        float v = av / (1.0f + expf(-g1));
        if (f) {
            float fv = f_bias ? f_bias[c] : 0.f;
            for (int p = 0; p < f_parts; ++p) fv += to_f32(f[(long)p * f_stride + i]);
            const float g2 = to_f32(g[t * ldg + H + c]) + (g_bias ? g_bias[H + c] : 0.f);
            v += fv / (1.0f + expf(-g2));
        }
        out[i] = v;
    }
}

extern "C" const char* cpmcu_gated_branches(const void* g, long ldg, int g_dtype, const float* g_bias, const void* a,
                                            int a_dtype, int a_parts, long a_stride, const float* a_bias, const void* f,
                                            int f_dtype, int f_parts, long f_stride, const float* f_bias, float* out,
                                            int n, int H, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && a && a_parts >= 1, "gated_branches: empty shape");
    CPMCU_REQUIRE(ldg >= (f ? 2L : 1L) * H, "gated_branches: gate rows of %ld for %d columns", ldg, H);
    const long total = (long)n * H;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    const int fd = f ? f_dtype : a_dtype;
#define LAUNCH(GT, AT, FT)                                                                                         \
    gated_branches_kernel<GT, AT, FT><<<blocks, 256, 0, stream>>>((const GT*)g, ldg, g_bias, (const AT*)a, a_parts,  \
                                                                  a_stride, a_bias, (const FT*)f, f_parts, f_stride, \
                                                                  f_bias, out, total, H)
    if (g_dtype == CPMCU_F32 && a_dtype == CPMCU_F32 && fd == CPMCU_F32) LAUNCH(float, float, float);
    else if (g_dtype == CPMCU_BF16 && a_dtype == CPMCU_F32 && fd == CPMCU_F32) LAUNCH(bf16_t, float, float);
    else if (g_dtype == CPMCU_BF16 && a_dtype == CPMCU_BF16 && fd == CPMCU_F32) LAUNCH(bf16_t, bf16_t, float);
    else if (g_dtype == CPMCU_BF16 && a_dtype == CPMCU_F32 && fd == CPMCU_BF16) LAUNCH(bf16_t, float, bf16_t);
    else if (g_dtype == CPMCU_BF16 && a_dtype == CPMCU_BF16 && fd == CPMCU_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (g_dtype == CPMCU_F32 && a_dtype == CPMCU_BF16 && fd == CPMCU_BF16) LAUNCH(float, bf16_t, bf16_t);
    else if (g_dtype == CPMCU_F32 && a_dtype == CPMCU_F32 && fd == CPMCU_BF16) LAUNCH(float, float, bf16_t);
    else if (g_dtype == CPMCU_F32 && a_dtype == CPMCU_BF16 && fd == CPMCU_F32) LAUNCH(float, bf16_t, float);
    else CPMCU_FAIL("gated_branches: unsupported dtypes gate=%d a=%d f=%d", g_dtype, a_dtype, fd);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("gated_branches");
    return nullptr;
}

template <typename AT>
__global__ __launch_bounds__(256) void bias_sum_kernel(const AT* __restrict__ a, int parts, long stride,
                                                       const float* __restrict__ bias, float* __restrict__ out,
                                                       long total, int H) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        float v = bias[i % H];
        for (int p = 0; p < parts; ++p) v += to_f32(a[(long)p * stride + i]);
        out[i] = v;
    }
}

extern "C" const char* cpmcu_bias_sum(const void* a, int dtype, int parts, long stride, const float* bias, float* out,
                                      int n, int H, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && parts >= 1 && bias, "bias_sum: empty shape");
    const long total = (long)n * H;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    if (dtype == CPMCU_F32) bias_sum_kernel<float><<<blocks, 256, 0, stream>>>((const float*)a, parts, stride, bias, out, total, H);
    else if (dtype == CPMCU_BF16) bias_sum_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)a, parts, stride, bias, out, total, H);
    else CPMCU_FAIL("bias_sum: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("bias_sum");
    return nullptr;
}

// out = a * sigmoid(g), element by element: an attention's heads side by side times a gate that is a projection
// of the mixer's input (g may be columns of a wider projection); the sigmoid in float.
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(const T* __restrict__ a, const T* __restrict__ g, long ldg,
                                                           T* __restrict__ out, long total, int W) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const long t = i / W;
        const int c = (int)(i - t * W);
        out[i] = from_f32<T>(to_f32(a[i]) / (1.0f + expf(-to_f32(g[t * ldg + c]))));
    }
}

extern "C" const char* cpmcu_sigmoid_gate(const void* a, const void* g, long ldg, void* out, int dtype, int n, int W,
                                          hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && W > 0 && a && g && out && ldg >= W, "sigmoid_gate: empty shape or rows too short");
    const long total = (long)n * W;
    const long wgs = (total + 255) / 256;
    const unsigned grid = (unsigned)(wgs < 65535L * 16 ? wgs : 65535L * 16);
    if (dtype == CPMCU_F32)
        sigmoid_gate_kernel<float><<<grid, 256, 0, stream>>>((const float*)a, (const float*)g, ldg, (float*)out, total, W);
    else if (dtype == CPMCU_BF16)
        sigmoid_gate_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)a, (const bf16_t*)g, ldg, (bf16_t*)out, total, W);
    else
        CPMCU_FAIL("sigmoid_gate: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("sigmoid_gate");
    return nullptr;
}

template <typename AT, typename FT>
__global__ __launch_bounds__(256) void scaled_branches_kernel(const AT* __restrict__ a, int a_parts, long a_stride,
                                                              const float* __restrict__ a_bias,
                                                              const float* __restrict__ wa, float sa,
                                                              const FT* __restrict__ f, int f_parts, long f_stride,
                                                              const float* __restrict__ f_bias,
                                                              const float* __restrict__ wf, float sf,
                                                              float* __restrict__ out, long total, int H) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const int c = (int)(i % H);
        float av = a_bias ? a_bias[c] : 0.f;
        for (int p = 0; p < a_parts; ++p) av += to_f32(a[(long)p * a_stride + i]);
        float v = sa * (wa ? wa[c] : 1.0f) * av;
        if (f) {
            float fv = f_bias ? f_bias[c] : 0.f;
            for (int p = 0; p < f_parts; ++p) fv += to_f32(f[(long)p * f_stride + i]);
            v += sf * (wf ? wf[c] : 1.0f) * fv;
        }
        out[i] = v;
    }
}

extern "C" const char* cpmcu_scaled_branches(const void* a, int a_dtype, int a_parts, long a_stride, const float* a_bias,
                                             const float* wa, float sa, const void* f, int f_dtype, int f_parts,
                                             long f_stride, const float* f_bias, const float* wf, float sf, float* out,
                                             int n, int H, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && a && a_parts >= 1 && (!f || f_parts >= 1), "scaled_branches: empty shape");
    const long total = (long)n * H;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    const int fd = f ? f_dtype : a_dtype;
#define LAUNCH(AT, FT)                                                                                             \
    scaled_branches_kernel<AT, FT><<<blocks, 256, 0, stream>>>((const AT*)a, a_parts, a_stride, a_bias, wa, sa,       \
                                                               (const FT*)f, f_parts, f_stride, f_bias, wf, sf, out, \
                                                               total, H)
    if (a_dtype == CPMCU_F32 && fd == CPMCU_F32) LAUNCH(float, float);
    else if (a_dtype == CPMCU_BF16 && fd == CPMCU_F32) LAUNCH(bf16_t, float);
    else if (a_dtype == CPMCU_F32 && fd == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (a_dtype == CPMCU_BF16 && fd == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else CPMCU_FAIL("scaled_branches: unsupported dtypes a=%d f=%d", a_dtype, fd);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("scaled_branches");
    return nullptr;
}
