// A residual of several streams (hyper-connections) and the norm that reads it, in one pass over a token's row.
//
// The residual holds S >= 1 rows X_1..X_S a token (float [S][n][H]).  A sub-layer reads u = sum_s read[s] X_s,
// and its result y joins all rows at once: X_t <- sum_s mix[s][t] X_s + out[t] y.  As everywhere in this
// library a sub-layer's result is added by the norm that follows it, so one kernel does, for a token:
//     y    = scale * (sum of the branch's partial sums) + bias                      (if a branch is pending)
//     X_t  = sum_s mix[s][t] X_s + out[t] y      (mix absent: X_t + out[t] y; out absent: 1)
//     u    = sum_t read[t] X_t                   (read absent: the plain sum)
//     h    = (u - mean(u)) / sqrt(mean((u - mean)^2) + eps) * w       (layer norm without bias), or
//            u / sqrt(mean(u^2) + eps) * w                            (RMS norm)
// With S = 1 and no mix this is the ordinary residual add and norm.  With `rows` only those tokens are read and
// normed and X stays as it was (the model's last norm before the head).  Statistics in float; the row u waits
// in LDS between the passes (mean, then squared deviations, then the output).
//
// pair_norm_mean: out = ((a / rms(a)) * wa + (b / rms(b)) * wb) / 2 row by row, a and b branches of two mixers
// side by side (each [n, H] or float partial sums [P, n, H]).
#include "common.h"

#define STREAMS_MAX 8

template <typename BT, typename OT>
__global__ __launch_bounds__(256) void streams_norm_kernel(float* __restrict__ X, long stream_stride, int S,
                                                           const BT* __restrict__ branch, int nparts, long part_stride,
                                                           const float* __restrict__ bias, float scale,
                                                           const float* __restrict__ mix, const float* __restrict__ outw,
                                                           const float* __restrict__ read, int rms,
                                                           const float* __restrict__ weight, float eps,
                                                           OT* __restrict__ out, const int* __restrict__ rows, int H) {
    extern __shared__ float u_s[];                 // [H]
    __shared__ float red[17];
    __shared__ float mix_s[STREAMS_MAX * STREAMS_MAX], out_s[STREAMS_MAX], read_s[STREAMS_MAX];
    const long r = rows ? rows[blockIdx.x] : blockIdx.x;
    if (threadIdx.x < S * S) mix_s[threadIdx.x] = mix ? mix[threadIdx.x] : ((threadIdx.x / S == threadIdx.x % S) ? 1.f : 0.f);
    if (threadIdx.x < S) {
        out_s[threadIdx.x] = outw ? outw[threadIdx.x] : 1.f;
        read_s[threadIdx.x] = read ? read[threadIdx.x] : 1.f;
    }
    __syncthreads();
    float sum = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float xs[STREAMS_MAX];
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s) xs[s] = s < S ? X[s * stream_stride + r * H + c] : 0.f;
        float u = 0.f;
        if (branch) {
            float y = 0.f;
            for (int p = 0; p < nparts; ++p) y += to_f32(branch[p * part_stride + r * H + c]);
            y = y * scale + (bias ? bias[c] : 0.f);
#pragma unroll
            for (int t = 0; t < STREAMS_MAX; ++t) {
                if (t < S) {
                    float v = out_s[t] * y;
#pragma unroll
                    for (int s = 0; s < STREAMS_MAX; ++s)
                        if (s < S) v += mix_s[s * S + t] * xs[s];
                    if (!rows) X[t * stream_stride + r * H + c] = v;
                    u += read_s[t] * v;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < STREAMS_MAX; ++t)
                if (t < S) u += read_s[t] * xs[t];
        }
        u_s[c] = u;
        sum += u;
    }
    float mean = 0.f;
    if (!rms) mean = block_sum(sum, red) / (float)H;
    float sq = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        const float d = u_s[c] - mean;
        sq += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)H + eps);
    OT* o = out + (long)blockIdx.x * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) o[c] = from_f32<OT>((u_s[c] - mean) * inv * weight[c]);
}

extern "C" const char* cpmcu_streams_norm(float* X, long stream_stride, int S, const void* branch, int branch_dtype,
                                          int nparts, long part_stride, const float* bias, float scale,
                                          const float* mix, const float* outw, const float* read, int rms,
                                          const float* weight, float eps, void* out, int out_dtype, const int* rows,
                                          int n_out, int H, hipStream_t stream) {
    CPMCU_REQUIRE(n_out > 0 && H > 0 && S >= 1, "streams_norm: empty shape rows=%d width=%d streams=%d", n_out, H, S);
    CPMCU_REQUIRE(S <= STREAMS_MAX, "streams_norm: %d residual streams (up to %d are taken)", S, STREAMS_MAX);
    CPMCU_REQUIRE((long)H * 4 <= 60 * 1024, "streams_norm: a width of %d does not fit the kernel's LDS", H);
    CPMCU_REQUIRE(X && weight && out, "streams_norm: null pointer");
    CPMCU_REQUIRE(branch || (!mix && !outw), "streams_norm: mixing numbers without a branch to add");
    const long lds = (long)H * 4;
#define LAUNCH(BT, OT)                                                                                               \
    streams_norm_kernel<BT, OT><<<n_out, 256, lds, stream>>>(X, stream_stride, S, (const BT*)branch, nparts,        \
                                                             part_stride, bias, scale, mix, outw, read, rms, weight, \
                                                             eps, (OT*)out, rows, H)
    const int bd = branch ? branch_dtype : CPMCU_F32;
    if (bd == CPMCU_F32 && out_dtype == CPMCU_F32) LAUNCH(float, float);
    else if (bd == CPMCU_F32 && out_dtype == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (bd == CPMCU_BF16 && out_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else if (bd == CPMCU_BF16 && out_dtype == CPMCU_F32) LAUNCH(bf16_t, float);
    else CPMCU_FAIL("streams_norm: unknown dtypes branch=%d out=%d", branch_dtype, out_dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("streams_norm");
    return nullptr;
}

// copies [n, H] -> [S, n, H]: every stream starts as the embedding's output
__global__ void streams_fill_kernel(const float* __restrict__ x, float* __restrict__ X, long count, int S) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (long)gridDim.x * blockDim.x) {
        const float v = x[i];
        for (int s = 0; s < S; ++s) X[s * count + i] = v;
    }
}

extern "C" const char* cpmcu_streams_fill(const float* x, float* X, long count, int S, hipStream_t stream) {
    CPMCU_REQUIRE(count > 0 && S >= 1 && x && X, "streams_fill: empty shape");
    const long wgs = (count + 255) / 256;
    streams_fill_kernel<<<(unsigned)(wgs < 65535L * 16 ? wgs : 65535L * 16), 256, 0, stream>>>(x, X, count, S);
    CPMCU_LAUNCH_CHECK("streams_fill");
    return nullptr;
}

template <typename AT, typename BT>
__global__ __launch_bounds__(256) void pair_norm_mean_kernel(const AT* __restrict__ a, int a_parts, long a_stride,
                                                             const float* __restrict__ a_bias,
                                                             const BT* __restrict__ b, int b_parts, long b_stride,
                                                             const float* __restrict__ b_bias,
                                                             const float* __restrict__ wa, const float* __restrict__ wb,
                                                             float eps, float* __restrict__ out, int H) {
    extern __shared__ float ab_s[];                // [2][H]
    __shared__ float red[17];
    const long r = blockIdx.x;
    float sa = 0.f, sb = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float va = a_bias ? a_bias[c] : 0.f, vb = b_bias ? b_bias[c] : 0.f;
        for (int p = 0; p < a_parts; ++p) va += to_f32(a[p * a_stride + r * H + c]);
        for (int p = 0; p < b_parts; ++p) vb += to_f32(b[p * b_stride + r * H + c]);
        ab_s[c] = va;
        ab_s[H + c] = vb;
        sa += va * va;
        sb += vb * vb;
    }
    const float ra = 0.5f / sqrtf(block_sum(sa, red) / (float)H + eps);
    const float rb = 0.5f / sqrtf(block_sum(sb, red) / (float)H + eps);
    for (int c = threadIdx.x; c < H; c += blockDim.x)
        out[r * H + c] = ab_s[c] * ra * wa[c] + ab_s[H + c] * rb * wb[c];
}

extern "C" const char* cpmcu_pair_norm_mean(const void* a, int a_dtype, int a_parts, long a_stride, const float* a_bias,
                                            const void* b, int b_dtype, int b_parts, long b_stride, const float* b_bias,
                                            const float* wa, const float* wb, float eps, float* out, int n, int H,
                                            hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && a && b && wa && wb && out, "pair_norm_mean: empty shape or null pointer");
    CPMCU_REQUIRE((long)H * 8 <= 60 * 1024, "pair_norm_mean: a width of %d does not fit the kernel's LDS", H);
    const long lds = (long)H * 8;
#define LAUNCH(AT, BT)                                                                                             \
    pair_norm_mean_kernel<AT, BT><<<n, 256, lds, stream>>>((const AT*)a, a_parts, a_stride, a_bias, (const BT*)b, \
                                                           b_parts, b_stride, b_bias, wa, wb, eps, out, H)
    if (a_dtype == CPMCU_F32 && b_dtype == CPMCU_F32) LAUNCH(float, float);
    else if (a_dtype == CPMCU_BF16 && b_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else if (a_dtype == CPMCU_F32 && b_dtype == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (a_dtype == CPMCU_BF16 && b_dtype == CPMCU_F32) LAUNCH(bf16_t, float);
    else CPMCU_FAIL("pair_norm_mean: unknown dtypes %d %d", a_dtype, b_dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("pair_norm_mean");
    return nullptr;
}
