// Gated delta rule over a packed batch, with per-slot state: a linear recurrence whose state is a matrix a head
// that forgets by a decay and corrects what it holds under the current key before it writes the new value.
//
// Per head h (its q and k come from head h / (heads / kv_heads)), everything in float:
//     qn = q / sqrt(sum q^2 + 1e-6) * q_scale,  kn = k / sqrt(sum k^2 + 1e-6)
//     beta = sigmoid(b_raw),  g = exp(-exp(A_log[h]) * softplus(a_raw + dt_bias[h]))
//     S <- g S;  u = beta (v - S^T kn);  S <- S + kn u^T;  o = S^T qn            S: [dk, dv], zero at the start
// Since S^T qn after the write is g (S_old^T qn) + (kn . qn) u, both products with the old state are formed in
// one pass over it (a column's two sums meet in one reduction) and the state is read and written once a token.
//
// A workgroup owns one (sequence, head, 32 or 16 columns of dv) and walks the sequence's tokens in order; a
// column's dk state values are spread over 8 or 16 neighbouring lanes (state index i = l + L r), the tokens' q,
// k, v and gates pass through LDS in tiles of 16 or 32 tokens, where the unit norms and k . q are formed once a
// token, and the next tile's values are asked for while the current one is walked.  A token's cost is one
// dependent chain of multiply-adds over a lane's share of the column and a reduction over the column's lanes:
// where the batch has too few (sequence, head, column) triples to fill the chip (a single prompt, a step of one
// sequence), 16 lanes a column halve that chain and double the number of workgroups.
#include "common.h"

__device__ inline float delta_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// qkv: float [n, ld] = [q: kv_heads*dk | k: kv_heads*dk | v: heads*dv] (after convolution and activation);
// gates: raw projections [n, ldg], the decay's at column a_off + h, beta's at b_off + h;
// state: float [slots][heads][dv][dk]; y: float [n, heads*dv].
template <int NR, int TT, int DELTA_L, typename GT>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* __restrict__ qkv, long ld,
                                                         const GT* __restrict__ gates, long ldg, long a_off, long b_off,
                                                         const float* __restrict__ dt_bias,
                                                         const float* __restrict__ A_log, float* __restrict__ state,
                                                         float* __restrict__ y, const int* __restrict__ cu_q,
                                                         const int* __restrict__ seq_slot, int heads, int kv_heads,
                                                         int dk, int dv, float q_scale, int write_state) {
    constexpr int DELTA_PB = 256 / DELTA_L;         // columns of dv a workgroup
    constexpr int NS = NR * DELTA_L;                // state values a column, padded
    constexpr int QK = TT * NS / 256;               // q (and k) values a thread brings a tile
    constexpr int VV = (TT * DELTA_PB + 255) / 256; // v values a thread brings a tile
    constexpr int TPT = 256 / TT;                   // threads that share a token's norms
    static_assert(TT * NS % 256 == 0 && (TT == 16 || TT == 32), "tile shape");
    __shared__ float qs[TT][NS];
    __shared__ float ks[TT][NS];
    __shared__ float vs[TT][DELTA_PB];
    __shared__ float betas[TT], gs[TT], kqs[TT];
    const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * DELTA_PB;
    const int start = cu_q[b], n_q = cu_q[b + 1] - start;
    const int slot = seq_slot[b];
    const int kvh = h / (heads / kv_heads);
    const long k_col = (long)kv_heads * dk, v_col = 2L * kv_heads * dk;
    const int pl = threadIdx.x / DELTA_L, l = threadIdx.x % DELTA_L;
    const int p = p0 + pl;
    const bool p_ok = p < dv;
    float S[NR];
    float* sp = state + (((long)slot * heads + h) * dv + (p_ok ? p : 0)) * dk;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const int n = l + DELTA_L * i;
        S[i] = (p_ok && n < dk) ? sp[n] : 0.f;
    }
    const float A = expf(A_log[h]), bias = dt_bias[h];
    float rq[QK], rk[QK], rv[VV], ra = 0.f, rb = 0.f;
    auto fetch = [&](int t0) {
        const int tn = min(TT, n_q - t0);
#pragma unroll
        for (int k = 0; k < QK; ++k) {
            const int e = threadIdx.x + k * 256;
            const int tt = e / NS, n = e % NS;
            const bool ok = tt < tn && n < dk;
            const float* row = qkv + (long)(start + t0 + min(tt, tn - 1)) * ld + (long)kvh * dk + min(n, dk - 1);
            rq[k] = ok ? row[0] : 0.f;
            rk[k] = ok ? row[k_col] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < VV; ++k) {
            const int e = threadIdx.x + k * 256;
            const int tt = e / DELTA_PB, pp = e % DELTA_PB;
            rv[k] = (tt < tn && p0 + pp < dv) ? qkv[(long)(start + t0 + tt) * ld + v_col + (long)h * dv + p0 + pp] : 0.f;
        }
        if ((int)threadIdx.x < tn) {
            const GT* gr = gates + (long)(start + t0 + threadIdx.x) * ldg;
            ra = to_f32(gr[a_off + h]);
            rb = to_f32(gr[b_off + h]);
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < n_q; t0 += TT) {
        const int tn = min(TT, n_q - t0);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < QK; ++k) {
            const int e = threadIdx.x + k * 256;
            qs[e / NS][e % NS] = rq[k];
            ks[e / NS][e % NS] = rk[k];
        }
#pragma unroll
        for (int k = 0; k < VV; ++k) {
            const int e = threadIdx.x + k * 256;
            if (e < TT * DELTA_PB) vs[e / DELTA_PB][e % DELTA_PB] = rv[k];
        }
        if ((int)threadIdx.x < tn) {
            betas[threadIdx.x] = 1.0f / (1.0f + expf(-rb));
            gs[threadIdx.x] = expf(-A * delta_softplus(ra + bias));
        }
        __syncthreads();
        {
            // unit vectors and k . q, once a token: TPT neighbouring threads share a token's NS values
            const int tt = threadIdx.x / TPT, part = threadIdx.x % TPT;
            float sq = 0.f, sk = 0.f, dot = 0.f;
            for (int n = part; n < NS; n += TPT) {
                const float a = qs[tt][n], c = ks[tt][n];
                sq += a * a;
                sk += c * c;
                dot += a * c;
            }
            sq = lanes_sum<TPT>(sq);
            sk = lanes_sum<TPT>(sk);
            dot = lanes_sum<TPT>(dot);
            const float fq = q_scale / sqrtf(sq + 1e-6f), fk = 1.0f / sqrtf(sk + 1e-6f);
            for (int n = part; n < NS; n += TPT) {
                qs[tt][n] *= fq;
                ks[tt][n] *= fk;
            }
            if (part == 0) kqs[tt] = dot * fq * fk;
        }
        __syncthreads();
        if (t0 + TT < n_q) fetch(t0 + TT);
        for (int tt = 0; tt < tn; ++tt) {
            const float g = gs[tt], beta = betas[tt], vv = vs[tt][pl], kq = kqs[tt];
            float kr[NR];
            float r = 0.f, o = 0.f;
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const int n = l + DELTA_L * i;
                kr[i] = ks[tt][n];
                r += S[i] * kr[i];
                o += S[i] * qs[tt][n];
            }
            // the column's lanes are neighbours: both sums meet inside the vector unit, every lane gets them
            r += CPMCU_DPP(r, 0xB1);
            o += CPMCU_DPP(o, 0xB1);
            r += CPMCU_DPP(r, 0x4E);
            o += CPMCU_DPP(o, 0x4E);
            r += CPMCU_DPP(r, 0x141);
            o += CPMCU_DPP(o, 0x141);
            if (DELTA_L == 16) {
                r += CPMCU_DPP(r, 0x140);
                o += CPMCU_DPP(o, 0x140);
            }
            const float u = beta * (vv - g * r);
#pragma unroll
            for (int i = 0; i < NR; ++i) S[i] = g * S[i] + kr[i] * u;
            if (l == 0 && p_ok) y[(long)(start + t0 + tt) * heads * dv + (long)h * dv + p] = g * o + kq * u;
        }
    }
    if (write_state && p_ok) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const int n = l + DELTA_L * i;
            if (n < dk) sp[n] = S[i];
        }
    }
}

extern "C" const char* cpmcu_delta_scan(const float* qkv, long ld, const void* gates, long ldg, int gate_dtype,
                                        long a_off, long b_off, const float* dt_bias, const float* A_log, float* state,
                                        float* y, const int* cu_q, const int* seq_slot, int n_seqs, int heads,
                                        int kv_heads, int dk, int dv, float q_scale, int write_state, int lanes,
                                        hipStream_t stream) {
    CPMCU_REQUIRE(n_seqs > 0 && heads > 0 && kv_heads > 0 && dk > 0 && dv > 0, "delta_scan: empty shape");
    CPMCU_REQUIRE(heads % kv_heads == 0, "delta_scan: %d heads are not a multiple of %d key heads", heads, kv_heads);
    CPMCU_REQUIRE(dk <= 256, "delta_scan: a key size of %d is not supported (at most 256)", dk);
    CPMCU_REQUIRE(ld >= 2L * kv_heads * dk + (long)heads * dv, "delta_scan: rows of %ld too short", ld);
    CPMCU_REQUIRE(a_off >= 0 && b_off >= 0 && ldg >= a_off + heads && ldg >= b_off + heads, "delta_scan: gate rows too short");
    CPMCU_REQUIRE(lanes == 0 || lanes == 8 || lanes == 16, "delta_scan: %d lanes a column (0: chosen here, 8 or 16)", lanes);
    // 16 lanes a column where 8 would leave fewer than two workgroups a compute unit and a column is long enough
    if (lanes == 0) lanes = ((long)n_seqs * heads * ((dv + 31) / 32) < 512 && dk > 16 && dv > 16) ? 16 : 8;
    const int cols = 256 / lanes;
    const int pb = (dv + cols - 1) / cols;
    CPMCU_REQUIRE(heads <= 65535 && pb <= 65535, "delta_scan: shape exceeds the launch grid");
    dim3 grid(n_seqs, heads, pb);
    const int need = (dk + lanes - 1) / lanes;
#define LAUNCH(NRv, TTv, Lv, GTv)                                                                                   \
    delta_scan_kernel<NRv, TTv, Lv, GTv><<<grid, 256, 0, stream>>>(qkv, ld, (const GTv*)gates, ldg, a_off, b_off,     \
                                                                   dt_bias, A_log, state, y, cu_q, seq_slot, heads,  \
                                                                   kv_heads, dk, dv, q_scale, write_state)
#define BY_NR(GTv)                                        \
    do {                                                  \
        if (lanes == 16) {                                \
            if (need <= 2) LAUNCH(2, 32, 16, GTv);        \
            else if (need <= 4) LAUNCH(4, 32, 16, GTv);   \
            else if (need <= 8) LAUNCH(8, 32, 16, GTv);   \
            else LAUNCH(16, 16, 16, GTv);                 \
        } else {                                          \
            if (need <= 2) LAUNCH(2, 32, 8, GTv);         \
            else if (need <= 4) LAUNCH(4, 32, 8, GTv);    \
            else if (need <= 8) LAUNCH(8, 32, 8, GTv);    \
            else if (need <= 16) LAUNCH(16, 32, 8, GTv);  \
            else LAUNCH(32, 16, 8, GTv);                  \
        }                                                 \
    } while (0)
    if (gate_dtype == CPMCU_F32) BY_NR(float);
    else if (gate_dtype == CPMCU_BF16) BY_NR(bf16_t);
    else CPMCU_FAIL("delta_scan: unknown dtype %d", gate_dtype);
#undef BY_NR
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("delta_scan");
    return nullptr;
}
