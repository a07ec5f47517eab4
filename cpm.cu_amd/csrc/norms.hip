// Norms beyond the residual RMSNorm of elementwise.hip, all with float statistics:
//
//  * rms_norm_groups_kernel: RMS norm of a row cut into equal groups, each by its own root mean square,
//    optionally after a SiLU gate (y <- y * silu(z), the gate before the norm) or followed by a sigmoid gate
//    (out <- norm(y) * w * sigmoid(z), the gate after the norm).  Rows may be slices of wider
//    rows (leading dimensions), so the first columns of a projection are normed where they lie.
//  * branch_norm_add_norm_kernel: a branch that has a norm of its own before it joins the residual
//    (x += rmsnorm(b) * wb), then the norm of the next sub-layer on the sum (out = rmsnorm(x) * w): the
//    arrangement "norm before and after every sub-layer" in one pass over the row.
//  * poly_norm_kernel: the PolyNorm activation a N(z) + b N(z^2) + c N(z^3) + e, N = division by the root mean
//    square of the row's values (powers element by element).
//
// RMS norm here always means x / sqrt(mean(x^2) + eps), eps inside the root.
#include "common.h"

template <typename T>
__device__ inline float sum_slices(const T* p, int nparts, long stride) {
    float v = 0.f;
    for (int i = 0; i < nparts; ++i) v += to_f32(p[(long)i * stride]);
    return v;
}

__device__ inline float silu_f(float z) { return z / (1.0f + expf(-z)); }

// grid (rows, groups); out[r, g*W + c] = v * rsqrt(mean_g(v^2) + eps) * weight[g*W + c], v = x * silu(z) if z and
// gate_after == 0; with gate_after the statistics are those of x alone and the result is multiplied by sigmoid(z)
// (gate_after == 1) or by silu(z) (gate_after == 2)
template <typename XT, typename ZT, typename OT>
__global__ __launch_bounds__(1024) void rms_norm_groups_kernel(const XT* __restrict__ x, long ldx,
                                                              const ZT* __restrict__ z, long ldz,
                                                              const float* __restrict__ weight, OT* __restrict__ out,
                                                              long ldo, int W, float eps, int gate_after,
                                                              const float* __restrict__ divisor) {
    __shared__ float red[17];
    const long r = blockIdx.x;
    const int g = blockIdx.y;
    const XT* xr = x + r * ldx + (long)g * W;
    const ZT* zr = z ? z + r * ldz + (long)g * W : nullptr;
    const bool before = zr && !gate_after;
    // divisor: one number a (row, group) by which the group's values are divided first
    const float pre = divisor ? 1.0f / divisor[r * gridDim.y + g] : 1.0f;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float v = to_f32(xr[c]) * pre;
        if (before) v *= silu_f(to_f32(zr[c]));
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)W + eps);
    OT* orow = out + r * ldo + (long)g * W;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float v = to_f32(xr[c]) * pre;
        if (before) v *= silu_f(to_f32(zr[c]));
        v *= rs;
        if (weight) v *= weight[(long)g * W + c];
        if (zr && gate_after) v *= gate_after == 2 ? silu_f(to_f32(zr[c])) : 1.0f / (1.0f + expf(-to_f32(zr[c])));
        orow[c] = from_f32<OT>(v);
    }
}

extern "C" const char* cpmcu_rms_norm_groups(const void* x, long ldx, int x_dtype, const void* z, long ldz, int z_dtype,
                                             const float* weight, void* out, long ldo, int out_dtype, int n, int groups,
                                             int W, float eps, int gate_after, const float* divisor,
                                             hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && groups > 0 && W > 0, "rms_norm_groups: empty shape rows=%d groups=%d width=%d", n, groups, W);
    CPMCU_REQUIRE(groups <= 65535, "rms_norm_groups: %d groups exceed the launch grid", groups);
    CPMCU_REQUIRE(ldx >= (long)groups * W && ldo >= (long)groups * W && (!z || ldz >= (long)groups * W),
                  "rms_norm_groups: leading dimensions too small for %d groups of %d", groups, W);
    dim3 grid(n, groups);
    // a group as wide as a model (one norm over all heads) on few rows is a handful of workgroups, each a chain of
    // dependent passes over its row: 1,024 threads shorten the chain
    const int block = (W >= 2048 && (long)n * groups < 1024) ? 1024 : (W >= 256 ? 256 : 64);
#define LAUNCH(XT, ZT, OT)                                                                                     \
    rms_norm_groups_kernel<XT, ZT, OT><<<grid, block, 0, stream>>>((const XT*)x, ldx, (const ZT*)z, ldz, weight, \
                                                                   (OT*)out, ldo, W, eps, gate_after, divisor)
    const int zd = z ? z_dtype : x_dtype;
    if (x_dtype == CPMCU_F32 && zd == CPMCU_F32 && out_dtype == CPMCU_F32) LAUNCH(float, float, float);
    else if (x_dtype == CPMCU_F32 && zd == CPMCU_F32 && out_dtype == CPMCU_BF16) LAUNCH(float, float, bf16_t);
    else if (x_dtype == CPMCU_F32 && zd == CPMCU_BF16 && out_dtype == CPMCU_BF16) LAUNCH(float, bf16_t, bf16_t);
    else if (x_dtype == CPMCU_BF16 && zd == CPMCU_BF16 && out_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (x_dtype == CPMCU_BF16 && zd == CPMCU_BF16 && out_dtype == CPMCU_F32) LAUNCH(bf16_t, bf16_t, float);
    else CPMCU_FAIL("rms_norm_groups: unsupported dtypes x=%d z=%d out=%d", x_dtype, zd, out_dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("rms_norm_groups");
    return nullptr;
}

// One workgroup a row.  b may come as float partial sums [nparts][n][H].  With `rows` only those rows are
// computed, into out[R, H], and x stays as it was (the final norm on the wanted rows).
template <typename BT, typename OT>
__global__ __launch_bounds__(256) void branch_norm_add_norm_kernel(float* __restrict__ x, const BT* __restrict__ b,
                                                                   int nparts, long part_stride,
                                                                   const float* __restrict__ wb, float eps_b,
                                                                   const float* __restrict__ w, float eps,
                                                                   OT* __restrict__ out, const int* __restrict__ rows,
                                                                   int H) {
    __shared__ float red[17];
    const long r = rows ? rows[blockIdx.x] : blockIdx.x;
    float* xr = x + r * H;
    const BT* br = b + r * H;
    float sb = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        const float v = sum_slices(br + c, nparts, part_stride);
        sb += v * v;
    }
    sb = block_sum(sb, red);
    const float rb = 1.0f / sqrtf(sb / (float)H + eps_b);
    float sx = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        const float v = xr[c] + sum_slices(br + c, nparts, part_stride) * rb * wb[c];
        if (!rows) xr[c] = v;
        sx += v * v;
    }
    if (!out) return;
    sx = block_sum(sx, red);
    const float rx = 1.0f / sqrtf(sx / (float)H + eps);
    OT* orow = out + (long)blockIdx.x * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        const float v = rows ? xr[c] + sum_slices(br + c, nparts, part_stride) * rb * wb[c] : xr[c];
        orow[c] = from_f32<OT>(v * rx * w[c]);
    }
}

// The same with the row held in registers (H <= 1024 * VPT): one trip to memory for the branch's slices and the
// residual, all loads of a thread in flight together (a loop of dependent passes over the row costs a step of
// few rows ten times as much).
template <typename BT, typename OT, int VPT>
__global__ __launch_bounds__(1024) void branch_norm_add_norm_reg_kernel(float* __restrict__ x, const BT* __restrict__ b,
                                                                        int nparts, long part_stride,
                                                                        const float* __restrict__ wb, float eps_b,
                                                                        const float* __restrict__ w, float eps,
                                                                        OT* __restrict__ out,
                                                                        const int* __restrict__ rows, int H) {
    __shared__ float red[17];
    const long r = rows ? rows[blockIdx.x] : blockIdx.x;
    float* xr = x + r * H;
    const BT* br = b + r * H;
    float bv[VPT], xv[VPT], wbv[VPT], wv[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * 1024;
        bv[i] = 0.f;
        xv[i] = c < H ? xr[c] : 0.f;
        wbv[i] = c < H ? wb[c] : 0.f;
        wv[i] = (c < H && out) ? w[c] : 0.f;
    }
    // four slices' loads are issued before any of them is added
    int p = 0;
    for (; p + 4 <= nparts; p += 4) {
        float t4[4][VPT];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < VPT; ++i) {
                const int c = min((int)threadIdx.x + i * 1024, H - 1);  // clamped: no load in a branch
                t4[u][i] = to_f32(br[(long)(p + u) * part_stride + c]);
            }
#pragma unroll
        for (int i = 0; i < VPT; ++i) bv[i] += (t4[0][i] + t4[1][i]) + (t4[2][i] + t4[3][i]);
    }
    for (; p < nparts; ++p) {
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = min((int)threadIdx.x + i * 1024, H - 1);
            bv[i] += to_f32(br[(long)p * part_stride + c]);
        }
    }
    float sb = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i)
        if ((int)threadIdx.x + i * 1024 >= H) bv[i] = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) sb += bv[i] * bv[i];
    sb = block_sum(sb, red);
    const float rb = 1.0f / sqrtf(sb / (float)H + eps_b);
    float sx = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * 1024;
        xv[i] += bv[i] * rb * wbv[i];
        if (!rows && c < H) xr[c] = xv[i];
        sx += xv[i] * xv[i];
    }
    if (!out) return;
    sx = block_sum(sx, red);
    const float rx = 1.0f / sqrtf(sx / (float)H + eps);
    OT* orow = out + (long)blockIdx.x * H;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * 1024;
        if (c < H) orow[c] = from_f32<OT>(xv[i] * rx * wv[i]);
    }
}

extern "C" const char* cpmcu_branch_norm_add_norm(float* x, const void* b, int b_dtype, int nparts, long part_stride,
                                                  const float* wb, float eps_b, const float* w, float eps, void* out,
                                                  int out_dtype, const int* rows, int n_out, int H,
                                                  hipStream_t stream) {
    CPMCU_REQUIRE(n_out > 0 && H > 0 && nparts >= 1, "branch_norm_add_norm: empty shape rows=%d width=%d", n_out, H);
    CPMCU_REQUIRE(x && b && wb && (!out || w), "branch_norm_add_norm: a pointer is missing");
    CPMCU_REQUIRE(!rows || out, "branch_norm_add_norm: a list of rows needs an output");
#define LAUNCH(BT, OT)                                                                                              \
    do {                                                                                                            \
        if (H <= 2048)                                                                                              \
            branch_norm_add_norm_reg_kernel<BT, OT, 2><<<n_out, 1024, 0, stream>>>(                                 \
                x, (const BT*)b, nparts, part_stride, wb, eps_b, w, eps, (OT*)out, rows, H);                        \
        else if (H <= 4096)                                                                                         \
            branch_norm_add_norm_reg_kernel<BT, OT, 4><<<n_out, 1024, 0, stream>>>(                                 \
                x, (const BT*)b, nparts, part_stride, wb, eps_b, w, eps, (OT*)out, rows, H);                        \
        else if (H <= 8192)                                                                                         \
            branch_norm_add_norm_reg_kernel<BT, OT, 8><<<n_out, 1024, 0, stream>>>(                                 \
                x, (const BT*)b, nparts, part_stride, wb, eps_b, w, eps, (OT*)out, rows, H);                        \
        else                                                                                                        \
            branch_norm_add_norm_kernel<BT, OT><<<n_out, 256, 0, stream>>>(x, (const BT*)b, nparts, part_stride, wb, \
                                                                           eps_b, w, eps, (OT*)out, rows, H);       \
    } while (0)
    if (b_dtype == CPMCU_F32 && out_dtype == CPMCU_F32) LAUNCH(float, float);
    else if (b_dtype == CPMCU_F32 && out_dtype == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (b_dtype == CPMCU_BF16 && out_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else if (b_dtype == CPMCU_BF16 && out_dtype == CPMCU_F32) LAUNCH(bf16_t, float);
    else CPMCU_FAIL("branch_norm_add_norm: unsupported dtypes branch=%d out=%d", b_dtype, out_dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("branch_norm_add_norm");
    return nullptr;
}

// out = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e;  coef = (a, b, c, e) on the device.
// z may come as float partial sums [nparts][n][F].
template <typename ZT, typename OT>
__global__ __launch_bounds__(256) void poly_norm_kernel(const ZT* __restrict__ z, int nparts, long part_stride,
                                                        const float* __restrict__ coef, OT* __restrict__ out, int F,
                                                        float eps) {
    __shared__ float red[17];
    const long r = blockIdx.x;
    const ZT* zr = z + r * F;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
    for (int c = threadIdx.x; c < F; c += blockDim.x) {
        const float v = sum_slices(zr + c, nparts, part_stride);
        const float v2 = v * v;
        s2 += v2;
        s4 += v2 * v2;
        s6 += v2 * v2 * v2;
    }
    s2 = block_sum(s2, red);
    s4 = block_sum(s4, red);
    s6 = block_sum(s6, red);
    const float inv = 1.0f / (float)F;
    const float a = coef[0] / sqrtf(s2 * inv + eps), b = coef[1] / sqrtf(s4 * inv + eps),
                cc = coef[2] / sqrtf(s6 * inv + eps), e = coef[3];
    OT* orow = out + r * F;
    for (int c = threadIdx.x; c < F; c += blockDim.x) {
        const float v = sum_slices(zr + c, nparts, part_stride);
        orow[c] = from_f32<OT>(((cc * v + b) * v + a) * v + e);
    }
}

// The same with the row held in registers (F <= 1024 * VPT).
template <typename ZT, typename OT, int VPT>
__global__ __launch_bounds__(1024) void poly_norm_reg_kernel(const ZT* __restrict__ z, int nparts, long part_stride,
                                                             const float* __restrict__ coef, OT* __restrict__ out,
                                                             int F, float eps) {
    __shared__ float red[17];
    const long r = blockIdx.x;
    const ZT* zr = z + r * F;
    float zv[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) zv[i] = 0.f;
    for (int p = 0; p < nparts; ++p) {
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int c = threadIdx.x + i * 1024;
            if (c < F) zv[i] += to_f32(zr[(long)p * part_stride + c]);
        }
    }
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const float v2 = zv[i] * zv[i];
        s2 += v2;
        s4 += v2 * v2;
        s6 += v2 * v2 * v2;
    }
    s2 = block_sum(s2, red);
    s4 = block_sum(s4, red);
    s6 = block_sum(s6, red);
    const float inv = 1.0f / (float)F;
    const float a = coef[0] / sqrtf(s2 * inv + eps), b = coef[1] / sqrtf(s4 * inv + eps),
                cc = coef[2] / sqrtf(s6 * inv + eps), e = coef[3];
    OT* orow = out + r * F;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * 1024;
        if (c < F) orow[c] = from_f32<OT>(((cc * zv[i] + b) * zv[i] + a) * zv[i] + e);
    }
}

extern "C" const char* cpmcu_poly_norm(const void* z, int z_dtype, int nparts, long part_stride, const float* coef,
                                       void* out, int out_dtype, int n, int F, float eps, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && F > 0 && nparts >= 1, "poly_norm: empty shape rows=%d width=%d", n, F);
#define LAUNCH(ZT, OT)                                                                                          \
    do {                                                                                                        \
        if (F <= 4096)                                                                                          \
            poly_norm_reg_kernel<ZT, OT, 4><<<n, 1024, 0, stream>>>((const ZT*)z, nparts, part_stride, coef,    \
                                                                    (OT*)out, F, eps);                          \
        else if (F <= 16384)                                                                                    \
            poly_norm_reg_kernel<ZT, OT, 16><<<n, 1024, 0, stream>>>((const ZT*)z, nparts, part_stride, coef,   \
                                                                     (OT*)out, F, eps);                         \
        else                                                                                                    \
            poly_norm_kernel<ZT, OT><<<n, 256, 0, stream>>>((const ZT*)z, nparts, part_stride, coef, (OT*)out,  \
                                                            F, eps);                                            \
    } while (0)
    if (z_dtype == CPMCU_F32 && out_dtype == CPMCU_F32) LAUNCH(float, float);
    else if (z_dtype == CPMCU_F32 && out_dtype == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (z_dtype == CPMCU_BF16 && out_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else CPMCU_FAIL("poly_norm: unsupported dtypes in=%d out=%d", z_dtype, out_dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("poly_norm");
    return nullptr;
}
