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
#include "vec4.h"

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


// The same with 4 columns a thread and 16-byte accesses (H a multiple of 4, up to 4 vectors a thread): the row u
// stays in registers between the passes.  Steps of few rows spread a row over up to 1024 threads and ask for the
// streams and all of a branch's partial sums together; one workgroup a row of 256 threads with single loads would
// wait for memory once a part and column.
template <typename BT, typename OT, int SM>
__global__ __launch_bounds__(1024) void streams_norm_vec4_kernel(float* __restrict__ X, long stream_stride, int S,
                                                                 const BT* __restrict__ branch, int nparts, long part_stride,
                                                                 const float* __restrict__ bias, float scale,
                                                                 const float* __restrict__ mix, const float* __restrict__ outw,
                                                                 const float* __restrict__ read, int rms,
                                                                 const float* __restrict__ weight, float eps,
                                                                 OT* __restrict__ out, const int* __restrict__ rows, int H) {
    __shared__ float red[17];
    const long r = rows ? rows[blockIdx.x] : blockIdx.x;
    // the streams' numbers are the same for every thread: read where they are used, they come through the scalar
    // unit beside the row's loads (staged through LDS, a barrier would stand between their arrival and the first
    // load of the row)
    auto mix_at = [&](int s_, int t_) { return mix ? mix[s_ * S + t_] : (s_ == t_ ? 1.f : 0.f); };
    auto out_at = [&](int t_) { return outw ? outw[t_] : 1.f; };
    auto read_at = [&](int t_) { return read ? read[t_] : 1.f; };
    const int H4 = H / 4;
    float4 u[4];
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = threadIdx.x + k * blockDim.x;
        u[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c >= H4) continue;
        float* xc = X + r * H + 4 * c;
        float4 xs[SM];
#pragma unroll
        for (int s = 0; s < SM; ++s) xs[s] = *(const float4*)(xc + (long)min(s, S - 1) * stream_stride);
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
        if (branch) {
            float4 y = sum_parts4(branch + r * H + 4 * c, nparts, part_stride);
            const float4 b = bias ? *(const float4*)(bias + 4 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
            y.x = y.x * scale + b.x; y.y = y.y * scale + b.y; y.z = y.z * scale + b.z; y.w = y.w * scale + b.w;
#pragma unroll
            for (int t = 0; t < SM; ++t) {
                if (t < S) {
                    const float o = out_at(t);
                    float4 v = make_float4(o * y.x, o * y.y, o * y.z, o * y.w);
#pragma unroll
                    for (int s = 0; s < SM; ++s)
                        if (s < S) {
                            const float m = mix_at(s, t);
                            v.x += m * xs[s].x; v.y += m * xs[s].y; v.z += m * xs[s].z; v.w += m * xs[s].w;
                        }
                    if (!rows) *(float4*)(xc + (long)t * stream_stride) = v;
                    const float rd = read_at(t);
                    a.x += rd * v.x; a.y += rd * v.y; a.z += rd * v.z; a.w += rd * v.w;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < SM; ++t)
                if (t < S) {
                    const float rd = read_at(t);
                    a.x += rd * xs[t].x; a.y += rd * xs[t].y; a.z += rd * xs[t].z; a.w += rd * xs[t].w;
                }
        }
        u[k] = a;
        sum += (a.x + a.y) + (a.z + a.w);
    }
    float mean = 0.f;
    if (!rms) mean = block_sum(sum, red) / (float)H;
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        if ((int)(threadIdx.x + k * blockDim.x) >= H4) continue;
        const float dx = u[k].x - mean, dy = u[k].y - mean, dz = u[k].z - mean, dw = u[k].w - mean;
        sq += (dx * dx + dy * dy) + (dz * dz + dw * dw);
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)H + eps);
    OT* o = out + (long)blockIdx.x * H;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = threadIdx.x + k * blockDim.x;
        if (c >= H4) continue;
        const float4 w = *(const float4*)(weight + 4 * c);
        store4(o + 4 * c, (u[k].x - mean) * inv * w.x, (u[k].y - mean) * inv * w.y, (u[k].z - mean) * inv * w.z,
               (u[k].w - mean) * inv * w.w);
    }
}

// threads of a row's workgroup for the 4-column kernels: many rows keep more rows in flight on a CU with smaller
// workgroups, few rows spread a row over many threads; 0 if a row needs more than 4 vectors a thread
static int vec4_block(int n_rows, int H) {
    const int h4 = H / 4, cap = n_rows >= 512 ? 256 : 1024;
    int block = 64;
    while (block < cap && block < h4) block *= 2;
    return 4 * block >= h4 ? block : 0;
}
static bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

extern "C" const char* cpmcu_streams_norm(float* X, long stream_stride, int S, const void* branch, int branch_dtype,
                                          int nparts, long part_stride, const float* bias, float scale,
                                          const float* mix, const float* outw, const float* read, int rms,
                                          const float* weight, float eps, void* out, int out_dtype, const int* rows,
                                          int n_out, int H, hipStream_t stream) {
    CPMCU_REQUIRE(n_out > 0 && H > 0 && S >= 1, "streams_norm: empty shape rows=%d width=%d streams=%d", n_out, H, S);
    CPMCU_REQUIRE(S <= STREAMS_MAX, "streams_norm: %d residual streams (up to %d are taken)", S, STREAMS_MAX);
    CPMCU_REQUIRE(X && weight && out, "streams_norm: null pointer");
    CPMCU_REQUIRE(branch || (!mix && !outw), "streams_norm: mixing numbers without a branch to add");
    const int bd = branch ? branch_dtype : CPMCU_F32;
    const int vblock = H % 4 == 0 ? vec4_block(n_out, H) : 0;
    if (vblock && aligned16(X) && stream_stride % 4 == 0 && (!branch || (aligned16(branch) && part_stride % 4 == 0)) &&
        (!bias || aligned16(bias)) && aligned16(weight) && aligned16(out) && (bd == CPMCU_F32 || bd == CPMCU_BF16) &&
        (out_dtype == CPMCU_F32 || out_dtype == CPMCU_BF16)) {
#define VLAUNCH(BT, OT, SMv)                                                                                          \
        streams_norm_vec4_kernel<BT, OT, SMv><<<n_out, vblock, 0, stream>>>(X, stream_stride, S, (const BT*)branch,   \
                                                                            nparts, part_stride, bias, scale, mix,   \
                                                                            outw, read, rms, weight, eps, (OT*)out,  \
                                                                            rows, H)
#define VTYPES(SMv)                                                                 \
        if (bd == CPMCU_F32 && out_dtype == CPMCU_F32) VLAUNCH(float, float, SMv);  \
        else if (bd == CPMCU_F32) VLAUNCH(float, bf16_t, SMv);                      \
        else if (out_dtype == CPMCU_F32) VLAUNCH(bf16_t, float, SMv);               \
        else VLAUNCH(bf16_t, bf16_t, SMv)
        if (S == 1) { VTYPES(1); }
        else if (S <= 4) { VTYPES(4); }
        else { VTYPES(STREAMS_MAX); }
#undef VTYPES
#undef VLAUNCH
        CPMCU_LAUNCH_CHECK("streams_norm");
        return nullptr;
    }
    CPMCU_REQUIRE((long)H * 4 <= 60 * 1024, "streams_norm: a width of %d does not fit the kernel's LDS", H);
    const long lds = (long)H * 4;
#define LAUNCH(BT, OT)                                                                                               \
    streams_norm_kernel<BT, OT><<<n_out, 256, lds, stream>>>(X, stream_stride, S, (const BT*)branch, nparts,        \
                                                             part_stride, bias, scale, mix, outw, read, rms, weight, \
                                                             eps, (OT*)out, rows, H)
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


// The same with 4 columns a thread (see streams_norm_vec4_kernel): both rows stay in registers.
template <typename AT, typename BT>
__global__ __launch_bounds__(1024) void pair_norm_mean_vec4_kernel(const AT* __restrict__ a, int a_parts, long a_stride,
                                                                   const float* __restrict__ a_bias,
                                                                   const BT* __restrict__ b, int b_parts, long b_stride,
                                                                   const float* __restrict__ b_bias,
                                                                   const float* __restrict__ wa, const float* __restrict__ wb,
                                                                   float eps, float* __restrict__ out, int H) {
    __shared__ float red[17];
    const long r = blockIdx.x;
    const int H4 = H / 4;
    float4 va[4], vb[4];
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = threadIdx.x + k * blockDim.x;
        va[k] = vb[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c >= H4) continue;
        float4 x = sum_parts4(a + r * H + 4 * c, a_parts, a_stride);
        float4 y = sum_parts4(b + r * H + 4 * c, b_parts, b_stride);
        if (a_bias) {
            const float4 t = *(const float4*)(a_bias + 4 * c);
            x.x += t.x; x.y += t.y; x.z += t.z; x.w += t.w;
        }
        if (b_bias) {
            const float4 t = *(const float4*)(b_bias + 4 * c);
            y.x += t.x; y.y += t.y; y.z += t.z; y.w += t.w;
        }
        va[k] = x;
        vb[k] = y;
        sa += (x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w);
        sb += (y.x * y.x + y.y * y.y) + (y.z * y.z + y.w * y.w);
    }
    const float ra = 0.5f / sqrtf(block_sum(sa, red) / (float)H + eps);
    const float rb = 0.5f / sqrtf(block_sum(sb, red) / (float)H + eps);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = threadIdx.x + k * blockDim.x;
        if (c >= H4) continue;
        const float4 p = *(const float4*)(wa + 4 * c), q = *(const float4*)(wb + 4 * c);
        store4(out + r * H + 4 * c, va[k].x * ra * p.x + vb[k].x * rb * q.x, va[k].y * ra * p.y + vb[k].y * rb * q.y,
               va[k].z * ra * p.z + vb[k].z * rb * q.z, va[k].w * ra * p.w + vb[k].w * rb * q.w);
    }
}

extern "C" const char* cpmcu_pair_norm_mean(const void* a, int a_dtype, int a_parts, long a_stride, const float* a_bias,
                                            const void* b, int b_dtype, int b_parts, long b_stride, const float* b_bias,
                                            const float* wa, const float* wb, float eps, float* out, int n, int H,
                                            hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && a && b && wa && wb && out, "pair_norm_mean: empty shape or null pointer");
    const int vblock = H % 4 == 0 ? vec4_block(n, H) : 0;
    const bool types_ok = (a_dtype == CPMCU_F32 || a_dtype == CPMCU_BF16) && (b_dtype == CPMCU_F32 || b_dtype == CPMCU_BF16);
    if (vblock && types_ok && aligned16(a) && aligned16(b) && a_stride % 4 == 0 && b_stride % 4 == 0 &&
        (!a_bias || aligned16(a_bias)) && (!b_bias || aligned16(b_bias)) && aligned16(wa) && aligned16(wb) && aligned16(out)) {
#define VLAUNCH(AT, BT)                                                                                            \
        pair_norm_mean_vec4_kernel<AT, BT><<<n, vblock, 0, stream>>>((const AT*)a, a_parts, a_stride, a_bias,      \
                                                                     (const BT*)b, b_parts, b_stride, b_bias, wa,  \
                                                                     wb, eps, out, H)
        if (a_dtype == CPMCU_F32 && b_dtype == CPMCU_F32) VLAUNCH(float, float);
        else if (a_dtype == CPMCU_BF16 && b_dtype == CPMCU_BF16) VLAUNCH(bf16_t, bf16_t);
        else if (a_dtype == CPMCU_F32) VLAUNCH(float, bf16_t);
        else VLAUNCH(bf16_t, float);
#undef VLAUNCH
        CPMCU_LAUNCH_CHECK("pair_norm_mean");
        return nullptr;
    }
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
