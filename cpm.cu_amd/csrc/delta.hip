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
//
// The same walk serves two relatives of the rule (RULE):
//   * RULE_CHANNEL: the decay is a number a head and key channel, g[i] = exp(-exp(A_log[h]) * softplus(a_raw[h, i] +
//     dt_bias[h, i])), acting on the rows of S: S <- diag(g) S, then as above.  With t_i = g_i S_i the two sums are
//     sum t_i kn_i and sum t_i qn_i, the write is S_i = t_i + kn_i u and the read-out sum t_i qn_i + (kn . qn) u.
//   * RULE_DECAY: linear attention with a fixed decay a head and nothing learned in the recurrence:
//     S <- d_h S + k v^T;  o = S^T q = d_h (S_old^T q) + (k . q) v, with q and k taken as they come (no unit
//     norm, no beta, no gates); `A_log` then holds the decays d_h themselves.
#include "common.h"

enum { RULE_DELTA = 0, RULE_CHANNEL = 1, RULE_DECAY = 2 };

__device__ inline float delta_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }

// qkv: float [n, ld] = [q: kv_heads*dk | k: kv_heads*dk | v: heads*dv] (after convolution and activation);
// gates: raw projections [n, ldg], the decay's at column a_off + h, beta's at b_off + h;
// state: float [slots][heads][dv][dk]; y: float [n, heads*dv].
// chan_a (RULE_CHANNEL): float [n, ld_a], the raw decay projection of head h and key channel i at column h*dk + i;
// dt_bias then has heads*dk numbers.
template <int NR, int TT, int DELTA_L, typename GT, int RULE>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* __restrict__ qkv, long ld,
                                                         const GT* __restrict__ gates, long ldg, long a_off, long b_off,
                                                         const float* __restrict__ chan_a, long ld_a,
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
    __shared__ float gcs[RULE == RULE_CHANNEL ? TT : 1][RULE == RULE_CHANNEL ? NS : 1];   // a decay a channel
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
    // RULE_DECAY: A_log holds the head's fixed decay itself
    const float A = RULE == RULE_DECAY ? A_log[h] : expf(A_log[h]);
    const float bias = RULE == RULE_DELTA ? dt_bias[h] : 0.f;
    float rq[QK], rk[QK], rv[VV], ra = 0.f, rb = 0.f;
    float rg[RULE == RULE_CHANNEL ? QK : 1];
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
            if (RULE == RULE_CHANNEL) {
                const float a = chan_a[(long)(start + t0 + min(tt, tn - 1)) * ld_a + (long)h * dk + min(n, dk - 1)];
                rg[k] = ok ? a + dt_bias[(long)h * dk + min(n, dk - 1)] : 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < VV; ++k) {
            const int e = threadIdx.x + k * 256;
            const int tt = e / DELTA_PB, pp = e % DELTA_PB;
            rv[k] = (tt < tn && p0 + pp < dv) ? qkv[(long)(start + t0 + tt) * ld + v_col + (long)h * dv + p0 + pp] : 0.f;
        }
        if (RULE != RULE_DECAY && (int)threadIdx.x < tn) {
            const GT* gr = gates + (long)(start + t0 + threadIdx.x) * ldg;
            if (RULE == RULE_DELTA) ra = to_f32(gr[a_off + h]);
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
            // (rows of the tile that this step does not bring are never walked: no exponentials for them)
            if (RULE == RULE_CHANNEL && e / NS < tn) gcs[e / NS][e % NS] = expf(-A * delta_softplus(rg[k]));
        }
#pragma unroll
        for (int k = 0; k < VV; ++k) {
            const int e = threadIdx.x + k * 256;
            if (e < TT * DELTA_PB) vs[e / DELTA_PB][e % DELTA_PB] = rv[k];
        }
        if ((int)threadIdx.x < tn) {
            betas[threadIdx.x] = RULE == RULE_DECAY ? 1.0f : 1.0f / (1.0f + expf(-rb));
            gs[threadIdx.x] = RULE == RULE_DELTA ? expf(-A * delta_softplus(ra + bias)) : A;
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
            if (RULE == RULE_DECAY) {
                if (part == 0) kqs[tt] = dot;
            } else {
                const float fq = q_scale / sqrtf(sq + 1e-6f), fk = 1.0f / sqrtf(sk + 1e-6f);
                for (int n = part; n < NS; n += TPT) {
                    qs[tt][n] *= fq;
                    ks[tt][n] *= fk;
                }
                if (part == 0) kqs[tt] = dot * fq * fk;
            }
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
                if (RULE == RULE_CHANNEL) S[i] *= gcs[tt][n];      // the channel's decay first: the sums see g_i S_i
                if (RULE != RULE_DECAY) r += S[i] * kr[i];
                o += S[i] * qs[tt][n];
            }
            // the column's lanes are neighbours: both sums meet inside the vector unit, every lane gets them
            if (RULE != RULE_DECAY) r += CPMCU_DPP(r, 0xB1);
            o += CPMCU_DPP(o, 0xB1);
            if (RULE != RULE_DECAY) r += CPMCU_DPP(r, 0x4E);
            o += CPMCU_DPP(o, 0x4E);
            if (RULE != RULE_DECAY) r += CPMCU_DPP(r, 0x141);
            o += CPMCU_DPP(o, 0x141);
            if (DELTA_L == 16) {
                if (RULE != RULE_DECAY) r += CPMCU_DPP(r, 0x140);
                o += CPMCU_DPP(o, 0x140);
            }
            // the decay that the sums still lack: the head's (RULE_CHANNEL applied its own above)
            const float gg = RULE == RULE_CHANNEL ? 1.0f : g;
            const float u = RULE == RULE_DECAY ? vv : beta * (vv - gg * r);
#pragma unroll
            for (int i = 0; i < NR; ++i) S[i] = gg * S[i] + kr[i] * u;
            if (l == 0 && p_ok) y[(long)(start + t0 + tt) * heads * dv + (long)h * dv + p] = gg * o + kq * u;
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
                                        long a_off, long b_off, const float* chan_a, long ld_a, const float* dt_bias,
                                        const float* A_log, float* state, float* y, const int* cu_q,
                                        const int* seq_slot, int n_seqs, int heads, int kv_heads, int dk, int dv,
                                        float q_scale, int write_state, int lanes, int rule, hipStream_t stream) {
    CPMCU_REQUIRE(rule == RULE_DELTA || rule == RULE_CHANNEL || rule == RULE_DECAY, "delta_scan: unknown rule %d", rule);
    CPMCU_REQUIRE(n_seqs > 0 && heads > 0 && kv_heads > 0 && dk > 0 && dv > 0, "delta_scan: empty shape");
    CPMCU_REQUIRE(heads % kv_heads == 0, "delta_scan: %d heads are not a multiple of %d key heads", heads, kv_heads);
    CPMCU_REQUIRE(dk <= 256, "delta_scan: a key size of %d is not supported (at most 256)", dk);
    CPMCU_REQUIRE(ld >= 2L * kv_heads * dk + (long)heads * dv, "delta_scan: rows of %ld too short", ld);
    CPMCU_REQUIRE(rule == RULE_DECAY || (gates && b_off >= 0 && ldg >= b_off + heads), "delta_scan: gate rows too short");
    CPMCU_REQUIRE(rule != RULE_DELTA || (a_off >= 0 && ldg >= a_off + heads), "delta_scan: gate rows too short");
    CPMCU_REQUIRE(rule != RULE_CHANNEL || (chan_a && ld_a >= (long)heads * dk), "delta_scan: channel decay rows too short");
    CPMCU_REQUIRE(A_log && (rule == RULE_DECAY || dt_bias), "delta_scan: decay constants missing");
    CPMCU_REQUIRE(lanes == 0 || lanes == 8 || lanes == 16, "delta_scan: %d lanes a column (0: chosen here, 8 or 16)", lanes);
    // 16 lanes a column where 8 would leave fewer than two workgroups a compute unit and a column is long enough
    if (lanes == 0) lanes = ((long)n_seqs * heads * ((dv + 31) / 32) < 512 && dk > 16 && dv > 16) ? 16 : 8;
    const int cols = 256 / lanes;
    const int pb = (dv + cols - 1) / cols;
    CPMCU_REQUIRE(heads <= 65535 && pb <= 65535, "delta_scan: shape exceeds the launch grid");
    dim3 grid(n_seqs, heads, pb);
    const int need = (dk + lanes - 1) / lanes;
#define LAUNCH(NRv, TTv, Lv, GTv, Rv)                                                                                \
    delta_scan_kernel<NRv, TTv, Lv, GTv, Rv><<<grid, 256, 0, stream>>>(qkv, ld, (const GTv*)gates, ldg, a_off, b_off, \
                                                                       chan_a, ld_a, dt_bias, A_log, state, y, cu_q,  \
                                                                       seq_slot, heads, kv_heads, dk, dv, q_scale,    \
                                                                       write_state)
#define BY_NR(GTv, Rv)                                        \
    do {                                                      \
        if (lanes == 16) {                                    \
            if (need <= 2) LAUNCH(2, 32, 16, GTv, Rv);        \
            else if (need <= 4) LAUNCH(4, 32, 16, GTv, Rv);   \
            else if (need <= 8) LAUNCH(8, 32, 16, GTv, Rv);   \
            else LAUNCH(16, 16, 16, GTv, Rv);                 \
        } else {                                              \
            if (need <= 2) LAUNCH(2, 32, 8, GTv, Rv);         \
            else if (need <= 4) LAUNCH(4, 32, 8, GTv, Rv);    \
            else if (need <= 8) LAUNCH(8, 32, 8, GTv, Rv);    \
            else if (need <= 16) LAUNCH(16, 32, 8, GTv, Rv);  \
            else LAUNCH(32, 16, 8, GTv, Rv);                  \
        }                                                     \
    } while (0)
    if (rule == RULE_DECAY) BY_NR(float, RULE_DECAY);
    else if (gate_dtype == CPMCU_F32 && rule == RULE_DELTA) BY_NR(float, RULE_DELTA);
    else if (gate_dtype == CPMCU_BF16 && rule == RULE_DELTA) BY_NR(bf16_t, RULE_DELTA);
    else if (gate_dtype == CPMCU_F32) BY_NR(float, RULE_CHANNEL);
    else if (gate_dtype == CPMCU_BF16) BY_NR(bf16_t, RULE_CHANNEL);
    else CPMCU_FAIL("delta_scan: unknown dtype %d", gate_dtype);
#undef BY_NR
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("delta_scan");
    return nullptr;
}

// What linear attention puts between its input projection and the recurrence, in float: from a projection's rows
// (q heads at column q_off, k heads at k_off, heads x dk each; v heads at v_off, heads x dv) to rows [q | k | v] of
// float.  With silu, all three pass z sigmoid(z); the first rot_dims features of q and k heads are rotated by
// position * inv_freq[i] (pairs (i, i + rot_dims/2), or (2i, 2i + 1) when interleaved); k is multiplied by k_scale
// afterwards.  grid (tokens, heads), 64 threads.
template <typename T>
__global__ __launch_bounds__(64) void linear_attention_prepare_kernel(const T* __restrict__ proj, long ld, long q_off,
                                                                      long k_off, long v_off, float* __restrict__ out,
                                                                      int heads, int dk, int dv, int silu, int rot_dims,
                                                                      int interleaved, const float* __restrict__ inv_freq,
                                                                      const int* __restrict__ positions, float k_scale) {
    const long t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const T* row = proj + t * ld;
    const long ow = 2L * heads * dk + (long)heads * dv;
    float* o = out + t * ow;
    auto act = [&](float z) { return silu ? z / (1.0f + expf(-z)) : z; };
    const float pos = rot_dims ? (float)positions[t] : 0.f;
    const int half = rot_dims / 2;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const T* src = row + (which ? k_off : q_off) + (long)h * dk;
        float* dst = o + (which ? (long)heads * dk : 0) + (long)h * dk;
        const float mul = which ? k_scale : 1.0f;
        for (int i = lane; i < half; i += 64) {
            const float ang = pos * inv_freq[i];
            const float cs = cosf(ang), sn = sinf(ang);
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            const float u = act(to_f32(src[ia])), v = act(to_f32(src[ib]));
            dst[ia] = (u * cs - v * sn) * mul;
            dst[ib] = (v * cs + u * sn) * mul;
        }
        for (int i = rot_dims + lane; i < dk; i += 64) dst[i] = act(to_f32(src[i])) * mul;
    }
    const T* vsrc = row + v_off + (long)h * dv;
    float* vdst = o + 2L * heads * dk + (long)h * dv;
    for (int i = lane; i < dv; i += 64) vdst[i] = act(to_f32(vsrc[i]));
}

extern "C" const char* cpmcu_linear_attention_prepare(const void* proj, int dtype, long ld, long q_off, long k_off,
                                                      long v_off, float* out, int n, int heads, int dk, int dv, int silu,
                                                      int rot_dims, int interleaved, const float* inv_freq,
                                                      const int* positions, float k_scale, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && heads > 0 && dk > 0 && dv > 0, "linear_attention_prepare: empty shape");
    CPMCU_REQUIRE(heads <= 65535, "linear_attention_prepare: %d heads exceed the launch grid", heads);
    CPMCU_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk && (rot_dims == 0 || (inv_freq && positions)),
                  "linear_attention_prepare: %d rotated features of %d", rot_dims, dk);
    CPMCU_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && ld >= q_off + (long)heads * dk && ld >= k_off + (long)heads * dk &&
                  ld >= v_off + (long)heads * dv, "linear_attention_prepare: rows of %ld too short", ld);
    dim3 grid(n, heads);
    if (dtype == CPMCU_F32)
        linear_attention_prepare_kernel<float><<<grid, 64, 0, stream>>>((const float*)proj, ld, q_off, k_off, v_off, out, heads,
                                                                        dk, dv, silu, rot_dims, interleaved, inv_freq,
                                                                        positions, k_scale);
    else if (dtype == CPMCU_BF16)
        linear_attention_prepare_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)proj, ld, q_off, k_off, v_off, out,
                                                                         heads, dk, dv, silu, rot_dims, interleaved, inv_freq,
                                                                         positions, k_scale);
    else
        CPMCU_FAIL("linear_attention_prepare: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("linear_attention_prepare");
    return nullptr;
}
