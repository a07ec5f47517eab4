// State-space (Mamba-2 style) sequence mixing over a packed batch, with per-slot state:
//
//  * conv_silu_kernel: causal convolution per channel over a sequence's tokens (taps weights a channel, the last
//    column is the current token's; inputs before the sequence's start are zero) followed by SiLU, or by nothing.
//    The sequence's last taps-1 inputs live in the slot's state, so a step continues where the last one ended.
//    With in_bias the convolution's inputs are u + in_bias (a projection's bias that is still to be added); the
//    state holds them with it, and the inputs before the start stay zero.  conv_silu_vec4_kernel is the same
//    for 2 to 5 taps and channel counts that are multiples of 4: 4 channels a thread, the last inputs in registers.
//  * conv_state_kernel: moves the step's last inputs into that state (after the convolution has read it); for
//    steps of at most 16 tokens a sequence the convolution's kernel does that itself.
//  * ssm_scan_kernel: the recurrence, per head h (group g = h / (heads / groups)):
//        dt_t = softplus(raw_t + dt_bias_h)             (no clamp)
//        S_t  = exp(-exp(A_log_h) * dt_t) * S_(t-1) + dt_t * B_t x_t^T        S: [state N, head size P]
//        y_t  = S_t^T C_t + D_h x_t
//    all in float, the state in float in the slot, carried from step to step.
//
// The scan walks a sequence's tokens in order; a workgroup owns one (sequence, head, 32 columns of P), a
// column's N state values are spread over 8 neighbouring lanes, and the tokens' B, C, x and dt pass through
// LDS in tiles of 16 or 32 tokens, the next tile asked for while the current one is worked on.
#include "common.h"
#include "vec4.h"

__device__ inline float silu_f(float z) { return z / (1.0f + expf(-z)); }

// grid (sequences, token tiles of 16, channel blocks of 256 threads)
template <typename UT>
__global__ __launch_bounds__(256) void conv_silu_kernel(const UT* __restrict__ u, long ldu,
                                                        const float* __restrict__ weight,
                                                        const float* __restrict__ bias,
                                                        const float* state, float* __restrict__ out,
                                                        const int* __restrict__ cu_q, const int* __restrict__ seq_slot,
                                                        int C, int taps, float* state_out,
                                                        const float* __restrict__ in_bias, int plain) {
    const int b = blockIdx.x;
    const int start = cu_q[b], q = cu_q[b + 1] - start;
    const int slot = seq_slot[b];
    const int c = blockIdx.z * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int i0 = blockIdx.y * 16, i1 = min(i0 + 16, q);
    const float* st = state + (long)slot * (taps - 1) * C + c;        // [slot][taps-1][C]
    const float bs = bias ? bias[c] : 0.f;
    const float ib = in_bias ? in_bias[c] : 0.f;
    for (int i = i0; i < i1; ++i) {
        float acc = bs;
        for (int k = 0; k < taps; ++k) {
            const int j = i - (taps - 1 - k);                          // local index of the input this tap reads
            const float in = j >= 0 ? to_f32(u[(long)(start + j) * ldu + c]) + ib : st[(long)(taps - 1 + j) * C];
            acc += weight[(long)c * taps + k] * in;
        }
        out[(long)(start + i) * C + c] = plain ? acc : silu_f(acc);
    }
    // steps of at most 16 tokens a sequence (decode steps): this thread alone has read its channel's state, so
    // it moves the step's last inputs into it itself and the second kernel is not launched
    if (state_out) {
        float* so = state_out + (long)slot * (taps - 1) * C + c;
        for (int j = 0; j < taps - 1; ++j) {
            const int i = q - (taps - 1) + j;
            so[(long)j * C] = i >= 0 ? to_f32(u[(long)(start + i) * ldu + c]) + ib : so[(long)(j + q) * C];
        }
    }
}

// The same for channel counts and row strides that are multiples of 4: a thread owns 4 neighbouring channels
// (8- or 16-byte loads, 16-byte stores) and walks its tile's tokens with the last TAPS-1 inputs in registers, so
// every input is loaded once a tile instead of once a tap.  grid (sequences, token tiles, blocks of 1,024 channels).
template <typename UT, int TAPS>
__global__ __launch_bounds__(256) void conv_silu_vec4_kernel(const UT* __restrict__ u, long ldu,
                                                             const float* __restrict__ weight,
                                                             const float* __restrict__ bias,
                                                             const float* state, float* __restrict__ out,
                                                             const int* __restrict__ cu_q, const int* __restrict__ seq_slot,
                                                             int C, int tile, float* state_out,
                                                             const float* __restrict__ in_bias, int plain) {
    const int b = blockIdx.x;
    const int start = cu_q[b], q = cu_q[b + 1] - start;
    const int slot = seq_slot[b];
    const int c = (blockIdx.z * 256 + threadIdx.x) * 4;
    if (c >= C) return;
    const int i0 = blockIdx.y * tile, i1 = min(i0 + tile, q);
    float w[4][TAPS];
    {
        float flat[4 * TAPS];
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
            const float4 t = load4(weight + (long)c * TAPS + 4 * j);
            flat[4 * j] = t.x; flat[4 * j + 1] = t.y; flat[4 * j + 2] = t.z; flat[4 * j + 3] = t.w;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int k = 0; k < TAPS; ++k) w[r][k] = flat[r * TAPS + k];
    }
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    const float4 bs = bias ? load4(bias + c) : zero;
    const float4 ib = in_bias ? load4(in_bias + c) : zero;
    const float* st = state + (long)slot * (TAPS - 1) * C + c;        // [slot][TAPS-1][C]
    auto input = [&](int j) {                                          // the input at local index j >= 0
        float4 t = load4(u + (long)(start + j) * ldu + c);
        t.x += ib.x; t.y += ib.y; t.z += ib.z; t.w += ib.w;
        return t;
    };
    float4 win[TAPS > 1 ? TAPS - 1 : 1];
    if (i0 < i1) {
#pragma unroll
        for (int k = 0; k < TAPS - 1; ++k) {
            const int j = i0 - (TAPS - 1) + k;
            win[k] = j >= 0 ? input(j) : load4(st + (long)(TAPS - 1 + j) * C);
        }
    }
    for (int i = i0; i < i1; i += 4) {
        float4 cur[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) cur[e] = input(min(i + e, i1 - 1));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (i + e < i1) {
                float4 acc = bs;
#pragma unroll
                for (int k = 0; k < TAPS - 1; ++k) {
                    acc.x += w[0][k] * win[k].x; acc.y += w[1][k] * win[k].y;
                    acc.z += w[2][k] * win[k].z; acc.w += w[3][k] * win[k].w;
                }
                acc.x += w[0][TAPS - 1] * cur[e].x; acc.y += w[1][TAPS - 1] * cur[e].y;
                acc.z += w[2][TAPS - 1] * cur[e].z; acc.w += w[3][TAPS - 1] * cur[e].w;
                if (!plain) { acc.x = silu_f(acc.x); acc.y = silu_f(acc.y); acc.z = silu_f(acc.z); acc.w = silu_f(acc.w); }
                store4(out + (long)(start + i + e) * C + c, acc.x, acc.y, acc.z, acc.w);
#pragma unroll
                for (int k = 0; k + 1 < TAPS - 1; ++k) win[k] = win[k + 1];
                if (TAPS > 1) win[TAPS - 2] = cur[e];
            }
        }
    }
    // a step of one tile a sequence: this thread alone has read its channels' state and moves it on itself
    if (state_out) {
        float* so = state_out + (long)slot * (TAPS - 1) * C + c;
#pragma unroll
        for (int j = 0; j < TAPS - 1; ++j) {
            const int i = q - (TAPS - 1) + j;
            const float4 t = i >= 0 ? input(i) : load4(so + (long)(j + q) * C);
            store4(so + (long)j * C, t.x, t.y, t.z, t.w);
        }
    }
}

// grid (sequences, channel blocks): state[j] <- the input at local index q - (taps-1) + j, which is one of the
// step's tokens or, for a short step, an older entry of the state (read before it is overwritten: a thread
// walks j upwards and reads index j + q > j).
template <typename UT>
__global__ __launch_bounds__(256) void conv_state_kernel(const UT* __restrict__ u, long ldu, float* __restrict__ state,
                                                         const int* __restrict__ cu_q, const int* __restrict__ seq_slot,
                                                         int C, int taps, const float* __restrict__ in_bias) {
    const int b = blockIdx.x;
    const int start = cu_q[b], q = cu_q[b + 1] - start;
    const int slot = seq_slot[b];
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    float* st = state + (long)slot * (taps - 1) * C + c;
    const float ib = in_bias ? in_bias[c] : 0.f;
    for (int j = 0; j < taps - 1; ++j) {
        const int i = q - (taps - 1) + j;
        st[(long)j * C] = i >= 0 ? to_f32(u[(long)(start + i) * ldu + c]) + ib : st[(long)(j + q) * C];
    }
}

extern "C" const char* cpmcu_conv_silu(const void* u, long ldu, int u_dtype, const float* weight, const float* bias,
                                       float* state, float* out, const int* cu_q, const int* seq_slot, int n_seqs,
                                       int max_q, int C, int taps, int update_state, const float* in_bias, int plain,
                                       hipStream_t stream) {
    CPMCU_REQUIRE(n_seqs > 0 && max_q > 0 && C > 0 && taps >= 1, "conv_silu: empty shape sequences=%d tokens=%d channels=%d taps=%d",
                  n_seqs, max_q, C, taps);
    CPMCU_REQUIRE(ldu >= C, "conv_silu: rows of %ld elements cannot hold %d channels", ldu, C);
    CPMCU_REQUIRE(taps == 1 || state, "conv_silu: the state of the last inputs is missing");
    const int cb = (C + 255) / 256, tb = (max_q + 15) / 16;
    CPMCU_REQUIRE(tb <= 65535 && cb <= 65535, "conv_silu: shape exceeds the launch grid (a step brings at most 1,048,560 "
                  "tokens a sequence)");
    dim3 grid(n_seqs, tb, cb), grid2(n_seqs, cb);
    const bool moves = update_state && taps > 1;
    float* fused = (moves && tb == 1) ? state : nullptr;
    const size_t esize = u_dtype == CPMCU_F32 ? 4 : 2;
    const bool vec4 = taps >= 2 && taps <= 5 && C % 4 == 0 && ldu % 4 == 0 && (uintptr_t)u % (4 * esize) == 0 &&
                      (uintptr_t)out % 16 == 0 && (uintptr_t)state % 16 == 0 && (uintptr_t)weight % 16 == 0 &&
                      (!bias || (uintptr_t)bias % 16 == 0) && (!in_bias || (uintptr_t)in_bias % 16 == 0) &&
                      (u_dtype == CPMCU_F32 || u_dtype == CPMCU_BF16);
    if (vec4) {
        // tiles of 16 tokens, of 64 where that still leaves the chip several workgroups a compute unit
        const int cb4 = (C + 1023) / 1024;
        const int tile = (tb > 1 && (long)n_seqs * ((max_q + 63) / 64) * cb4 >= 1024) ? 64 : 16;
        dim3 grid4(n_seqs, (max_q + tile - 1) / tile, cb4);
#define CONV4(UTv, TAPSv)                                                                                               \
    conv_silu_vec4_kernel<UTv, TAPSv><<<grid4, 256, 0, stream>>>((const UTv*)u, ldu, weight, bias, state, out, cu_q,    \
                                                                 seq_slot, C, tile, fused, in_bias, plain)
#define CONV4_TAPS(UTv)                    \
    do {                                   \
        if (taps == 2) CONV4(UTv, 2);      \
        else if (taps == 3) CONV4(UTv, 3); \
        else if (taps == 4) CONV4(UTv, 4); \
        else CONV4(UTv, 5);                \
    } while (0)
        if (u_dtype == CPMCU_F32) {
            CONV4_TAPS(float);
            if (moves && !fused)
                conv_state_kernel<float><<<grid2, 256, 0, stream>>>((const float*)u, ldu, state, cu_q, seq_slot, C, taps, in_bias);
        } else {
            CONV4_TAPS(bf16_t);
            if (moves && !fused)
                conv_state_kernel<bf16_t><<<grid2, 256, 0, stream>>>((const bf16_t*)u, ldu, state, cu_q, seq_slot, C, taps, in_bias);
        }
#undef CONV4_TAPS
#undef CONV4
    } else if (u_dtype == CPMCU_F32) {
        conv_silu_kernel<float><<<grid, 256, 0, stream>>>((const float*)u, ldu, weight, bias, state, out, cu_q, seq_slot, C, taps, fused, in_bias, plain);
        if (moves && !fused)
            conv_state_kernel<float><<<grid2, 256, 0, stream>>>((const float*)u, ldu, state, cu_q, seq_slot, C, taps, in_bias);
    } else if (u_dtype == CPMCU_BF16) {
        conv_silu_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)u, ldu, weight, bias, state, out, cu_q, seq_slot, C, taps, fused, in_bias, plain);
        if (moves && !fused)
            conv_state_kernel<bf16_t><<<grid2, 256, 0, stream>>>((const bf16_t*)u, ldu, state, cu_q, seq_slot, C, taps, in_bias);
    } else {
        CPMCU_FAIL("conv_silu: unknown dtype %d", u_dtype);
    }
    CPMCU_LAUNCH_CHECK("conv_silu");
    return nullptr;
}

#define SCAN_PB 32       // columns of P a workgroup
#define SCAN_L 8         // lanes a column: state index n = l + 8 i

__device__ inline float softplus_f(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// xbc: float [n, ldx] = [x: heads*P | B: groups*N | C: groups*N]; dt: raw step sizes [n, lddt] (first `heads`
// columns at the given pointer); state: float [slots][heads][P][N]; y: float [n, heads*P].
// Tiles of TT tokens pass through LDS; while a tile is worked on, the next one's values are already asked for
// (held in registers until the tile is done), so that the walk over a long prompt waits for memory once.
template <int NR, int TT, typename DT>
__global__ __launch_bounds__(256) void ssm_scan_kernel(const float* __restrict__ xbc, long ldx,
                                                       const DT* __restrict__ dt, long lddt,
                                                       const float* __restrict__ dt_bias,
                                                       const float* __restrict__ A_log, const float* __restrict__ Dskip,
                                                       float* __restrict__ state, float* __restrict__ y,
                                                       const int* __restrict__ cu_q, const int* __restrict__ seq_slot,
                                                       int heads, int P, int N, int groups, int write_state) {
    constexpr int NS = NR * SCAN_L;                 // state values a column, padded
    constexpr int BC = TT * NS / 256;               // B (and C) values a thread brings a tile
    constexpr int XV = (TT * SCAN_PB + 255) / 256;  // x values a thread brings a tile
    static_assert(TT * NS % 256 == 0 && TT <= 64, "tile shape");
    __shared__ float Bs[TT][NS];
    __shared__ float Cs[TT][NS];
    __shared__ float xs[TT][SCAN_PB];
    __shared__ float dts[TT], das[TT];
    const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * SCAN_PB;
    const int start = cu_q[b], q = cu_q[b + 1] - start;
    const int slot = seq_slot[b];
    const int g = h / (heads / groups);
    const int inner = heads * P;
    const int pl = threadIdx.x / SCAN_L, l = threadIdx.x % SCAN_L;
    const int p = p0 + pl;
    const bool p_ok = p < P;
    float S[NR];
    float* sp = state + (((long)slot * heads + h) * P + (p_ok ? p : 0)) * N;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const int n = l + SCAN_L * i;
        S[i] = (p_ok && n < N) ? sp[n] : 0.f;
    }
    const float A = expf(A_log[h]), bias = dt_bias[h], Dh = Dskip[h];
    float rb[BC], rc[BC], rx[XV], rdt = 0.f;
    auto fetch = [&](int t0) {
        const int tn = min(TT, q - t0);
#pragma unroll
        for (int k = 0; k < BC; ++k) {
            const int e = threadIdx.x + k * 256;
            const int tt = e / NS, n = e % NS;
            const bool ok = tt < tn && n < N;
            const float* row = xbc + (long)(start + t0 + min(tt, tn - 1)) * ldx + inner + (long)g * N + min(n, N - 1);
            rb[k] = ok ? row[0] : 0.f;
            rc[k] = ok ? row[(long)groups * N] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < XV; ++k) {
            const int e = threadIdx.x + k * 256;
            const int tt = e / SCAN_PB, pp = e % SCAN_PB;
            rx[k] = (tt < tn && p0 + pp < P) ? xbc[(long)(start + t0 + tt) * ldx + (long)h * P + p0 + pp] : 0.f;
        }
        if ((int)threadIdx.x < tn) rdt = to_f32(dt[(long)(start + t0 + threadIdx.x) * lddt + h]);
    };
    fetch(0);
    for (int t0 = 0; t0 < q; t0 += TT) {
        const int tn = min(TT, q - t0);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BC; ++k) {
            const int e = threadIdx.x + k * 256;
            Bs[e / NS][e % NS] = rb[k];
            Cs[e / NS][e % NS] = rc[k];
        }
#pragma unroll
        for (int k = 0; k < XV; ++k) {
            const int e = threadIdx.x + k * 256;
            if (e < TT * SCAN_PB) xs[e / SCAN_PB][e % SCAN_PB] = rx[k];
        }
        if ((int)threadIdx.x < tn) {
            const float d = softplus_f(rdt + bias);
            dts[threadIdx.x] = d;
            das[threadIdx.x] = expf(-A * d);
        }
        __syncthreads();
        if (t0 + TT < q) fetch(t0 + TT);
        for (int tt = 0; tt < tn; ++tt) {
            const float d = dts[tt], da = das[tt], xv = xs[tt][pl];
            const float dx = d * xv;
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int n = l + SCAN_L * i;
                S[i] = da * S[i] + dx * Bs[tt][n];
                acc += S[i] * Cs[tt][n];
            }
            // the column's 8 lanes are neighbours: sum inside the vector unit
            acc += CPMCU_DPP(acc, 0xB1);
            acc += CPMCU_DPP(acc, 0x4E);
            acc += CPMCU_DPP(acc, 0x141);
            if (l == 0 && p_ok) y[(long)(start + t0 + tt) * inner + (long)h * P + p] = acc + Dh * xv;
        }
    }
    if (write_state && p_ok) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int n = l + SCAN_L * i;
            if (n < N) sp[n] = S[i];
        }
    }
}

extern "C" const char* cpmcu_ssm_scan(const float* xbc, long ldx, const void* dt, long lddt, int dt_dtype,
                                      const float* dt_bias, const float* A_log, const float* Dskip, float* state,
                                      float* y, const int* cu_q, const int* seq_slot, int n_seqs, int heads, int P,
                                      int N, int groups, int write_state, hipStream_t stream) {
    CPMCU_REQUIRE(n_seqs > 0 && heads > 0 && P > 0 && N > 0 && groups > 0, "ssm_scan: empty shape");
    CPMCU_REQUIRE(heads % groups == 0, "ssm_scan: %d heads are not a multiple of %d groups", heads, groups);
    CPMCU_REQUIRE(N <= 256, "ssm_scan: a state of %d values a column is not supported (at most 256)", N);
    CPMCU_REQUIRE(ldx >= (long)heads * P + 2L * groups * N && lddt >= heads, "ssm_scan: rows too short");
    const int pb = (P + SCAN_PB - 1) / SCAN_PB;
    CPMCU_REQUIRE(heads <= 65535 && pb <= 65535, "ssm_scan: shape exceeds the launch grid");
    dim3 grid(n_seqs, heads, pb);
    const int need = (N + SCAN_L - 1) / SCAN_L;
#define LAUNCH(NRv, TTv, DTv)                                                                                    \
    ssm_scan_kernel<NRv, TTv, DTv><<<grid, 256, 0, stream>>>(xbc, ldx, (const DTv*)dt, lddt, dt_bias, A_log, Dskip, \
                                                             state, y, cu_q, seq_slot, heads, P, N, groups, write_state)
#define BY_NR(DTv)                                \
    do {                                          \
        if (need <= 2) LAUNCH(2, 32, DTv);        \
        else if (need <= 4) LAUNCH(4, 32, DTv);   \
        else if (need <= 8) LAUNCH(8, 32, DTv);   \
        else if (need <= 16) LAUNCH(16, 32, DTv); \
        else LAUNCH(32, 16, DTv);                 \
    } while (0)
    if (dt_dtype == CPMCU_F32) BY_NR(float);
    else if (dt_dtype == CPMCU_BF16) BY_NR(bf16_t);
    else CPMCU_FAIL("ssm_scan: unknown dtype %d", dt_dtype);
#undef BY_NR
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("ssm_scan");
    return nullptr;
}
