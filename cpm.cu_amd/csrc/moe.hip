// A feed-forward of routed experts, for steps of any number of tokens and both element types:
//
//  * moe_logits_kernel, moe_select_kernel: router logits z = Wr h in float (Wr float [E, H]), a wavefront a row,
//    into scratch; then, a wavefront a token: s = softmax(z) over the experts, or sigmoid(z) of each (score_fn);
//    choice scores c = s + correction; the experts form `n_groups` equal groups of neighbours, a group's score is
//    its largest c, or the sum of its two largest (group_fn), and only experts of the `keep_groups` best groups may be
//    chosen (n_groups = 1: any; the others' c count as -inf); the `top` largest c are chosen (ties: the lower index),
//    their weights are s / (sum of the chosen s + 1e-20) * weight_scale.  With w_sg (float [H]) it also
//    gives sigmoid(w_sg . h), the gate of an expert that every token uses.
//  * moe_gated_kernel: act[t, k, :] = act(Wg_e h_t) * (Wu_e h_t) for the k-th chosen expert e of token t (the
//    nonlinearities of common.h: SiLU, or the clamped swish with its limit); the experts' gate and up rows are
//    stacked: wgu [E, 2F, H], gate rows first.
//  * moe_down_kernel: out[t] = sum_k w[t, k] Wd_e act[t, k] (+ sg[t] * shared[t]); wd [E, H, F]; float out.
//
// A wavefront owns output rows and its lanes stride over the input features (16-byte loads when the rows are
// aligned), so an expert's weights stream once for every token that chose it: the form for steps of few tokens.
#include "common.h"

#define MOE_MAX_EXPERTS 1024
enum { MOE_SCORE_SOFTMAX = 0, MOE_SCORE_SIGMOID = 1 };
enum { MOE_GROUP_MAX = 0, MOE_GROUP_TOP2_SUM = 1 };

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> { typedef uint4 type; };
template <> struct Vec8<float> { struct type { float4 a, b; }; };

template <typename T>
__device__ inline void load8(const T* p, float* v);
template <>
__device__ inline void load8<bf16_t>(const bf16_t* p, float* v) {
    const uint4 u = *(const uint4*)p;
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
template <>
__device__ inline void load8<float>(const float* p, float* v) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// the lane's share of dot(a[0:K], b[0:K]); `vec`: both rows are 16-byte aligned (32 for float) and K % 8 == 0
template <typename TA, typename TB>
__device__ inline float lane_dot(const TA* __restrict__ a, const TB* __restrict__ b, int K, int lane, bool vec) {
    float s = 0.f;
    if (vec) {
        for (int c = lane * 8; c < K; c += 64 * 8) {
            float x[8], y[8];
            load8<TA>(a + c, x);
            load8<TB>(b + c, y);
#pragma unroll
            for (int i = 0; i < 8; ++i) s += x[i] * y[i];
        }
    } else {
        for (int c = lane; c < K; c += 64) s += to_f32(a[c]) * to_f32(b[c]);
    }
    return s;
}

__device__ inline float wave_min_f(float v) { return -wave_max(-v); }

// grid (tokens, ceil((E + 1) / 4)), 256 threads: a wavefront a row of the router (row E: the shared expert's gate);
// logits float [n, E + 1]
template <typename T>
__global__ __launch_bounds__(256) void moe_logits_kernel(const T* __restrict__ h, long ldh, const float* __restrict__ wr,
                                                         const float* __restrict__ w_sg, int H, int E,
                                                         float* __restrict__ logits) {
    const long t = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int e = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (e > E || (e == E && !w_sg)) return;
    const T* hr = h + t * ldh;
    const float* row = e < E ? wr + (long)e * H : w_sg;
    const bool vec = (H % 8 == 0) && (ldh % 8 == 0) && ((uintptr_t)h % 32 == 0) && ((uintptr_t)row % 32 == 0);
    const float s = wave_sum(lane_dot<T, float>(hr, row, H, lane, vec));
    if (lane == 0) logits[t * (E + 1) + e] = s;
}

// grid (tokens), 64 threads: softmax, groups, the top choices and their weights from a row of logits
__global__ __launch_bounds__(64) void moe_select_kernel(const float* __restrict__ logits,
                                                        const float* __restrict__ correction, int has_sg, int E,
                                                        int n_groups, int keep_groups, int top, int* __restrict__ idx_out,
                                                        float* __restrict__ w_out, float* __restrict__ sg_out,
                                                        int score_fn, int group_fn, float weight_scale) {
    __shared__ float z[MOE_MAX_EXPERTS];      // logits, then softmax scores
    __shared__ float c[MOE_MAX_EXPERTS];      // choice scores; -inf once an expert is chosen or shut out
    __shared__ float gs[MOE_MAX_EXPERTS];     // group scores
    const long t = blockIdx.x;
    const int lane = threadIdx.x;
    const float* zr = logits + t * (E + 1);
    if (has_sg && lane == 0) sg_out[t] = 1.0f / (1.0f + expf(-zr[E]));
    if (score_fn == MOE_SCORE_SIGMOID) {
        for (int e = lane; e < E; e += 64) {
            z[e] = 1.0f / (1.0f + expf(-zr[e]));
            c[e] = z[e] + (correction ? correction[e] : 0.f);
        }
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) {
            z[e] = zr[e];
            mx = fmaxf(mx, z[e]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += 64) {
            const float p = expf(z[e] - mx);
            z[e] = p;
            sum += p;
        }
        sum = wave_sum(sum);
        const float inv = 1.0f / sum;
        for (int e = lane; e < E; e += 64) {
            z[e] *= inv;
            c[e] = z[e] + (correction ? correction[e] : 0.f);
        }
    }
    __builtin_amdgcn_wave_barrier();
    if (n_groups > 1) {
        const int per = E / n_groups;
        for (int g = lane; g < n_groups; g += 64) {
            // the largest and the second largest choice score of the group
            float b = -INFINITY, b2 = -INFINITY;
            for (int i = 0; i < per; ++i) {
                const float v = c[g * per + i];
                if (v > b) {
                    b2 = b;
                    b = v;
                } else if (v > b2) {
                    b2 = v;
                }
            }
            gs[g] = (group_fn == MOE_GROUP_TOP2_SUM && per > 1) ? b + b2 : b;
        }
        __builtin_amdgcn_wave_barrier();
        // the best groups, one a turn, are marked with +inf; afterwards every other group's experts are shut out
        for (int r = 0; r < keep_groups; ++r) {
            float b = -INFINITY;
            for (int g = lane; g < n_groups; g += 64)
                if (gs[g] != INFINITY) b = fmaxf(b, gs[g]);
            b = wave_max(b);
            float first = 3.0e38f;
            for (int g = lane; g < n_groups; g += 64)
                if (gs[g] != INFINITY && gs[g] == b) first = fminf(first, (float)g);
            const int win = (int)wave_min_f(first);
            if (lane == 0) gs[win] = INFINITY;
            __builtin_amdgcn_wave_barrier();
        }
        for (int e = lane; e < E; e += 64)
            if (gs[e / per] != INFINITY) c[e] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
    }
    float chosen_sum = 0.f;
    for (int r = 0; r < top; ++r) {
        float b = -INFINITY;
        for (int e = lane; e < E; e += 64) b = fmaxf(b, c[e]);
        b = wave_max(b);
        float first = 3.0e38f;
        for (int e = lane; e < E; e += 64)
            if (c[e] == b) first = fminf(first, (float)e);
        const int win = (int)wave_min_f(first);
        chosen_sum += z[win];
        if (lane == 0) {
            idx_out[t * top + r] = win;
            w_out[t * top + r] = z[win];
            c[win] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
    }
    const float norm = weight_scale / (chosen_sum + 1e-20f);
    for (int r = lane; r < top; r += 64) w_out[t * top + r] *= norm;
}

extern "C" const char* cpmcu_moe_route(const void* h, long ldh, int dtype, const float* wr, const float* correction,
                                       const float* w_sg, int n, int H, int E, int n_groups, int keep_groups, int top,
                                       float* logits, int* idx_out, float* w_out, float* sg_out, int score_fn,
                                       int group_fn, float weight_scale, hipStream_t stream) {
    CPMCU_REQUIRE((score_fn == MOE_SCORE_SOFTMAX || score_fn == MOE_SCORE_SIGMOID) &&
                  (group_fn == MOE_GROUP_MAX || group_fn == MOE_GROUP_TOP2_SUM),
                  "moe_route: unknown score function %d or group score %d", score_fn, group_fn);
    CPMCU_REQUIRE(n > 0 && H > 0 && E > 0 && logits, "moe_route: empty shape");
    CPMCU_REQUIRE(E <= MOE_MAX_EXPERTS, "moe_route: %d experts (up to %d are taken)", E, MOE_MAX_EXPERTS);
    CPMCU_REQUIRE(n_groups >= 1 && E % n_groups == 0 && keep_groups >= 1 && keep_groups <= n_groups,
                  "moe_route: %d experts in %d groups of which %d may be chosen from", E, n_groups, keep_groups);
    CPMCU_REQUIRE(top >= 1 && top <= keep_groups * (E / n_groups), "moe_route: %d experts a token of %d that may be chosen",
                  top, keep_groups * (E / n_groups));
    CPMCU_REQUIRE(!w_sg || sg_out, "moe_route: a place for the shared gate is missing");
    dim3 grid(n, (E + 1 + 3) / 4);
    if (dtype == CPMCU_F32)
        moe_logits_kernel<float><<<grid, 256, 0, stream>>>((const float*)h, ldh, wr, w_sg, H, E, logits);
    else if (dtype == CPMCU_BF16)
        moe_logits_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)h, ldh, wr, w_sg, H, E, logits);
    else
        CPMCU_FAIL("moe_route: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("moe_logits");
    moe_select_kernel<<<n, 64, 0, stream>>>(logits, correction, w_sg ? 1 : 0, E, n_groups, keep_groups, top, idx_out, w_out,
                                            sg_out, score_fn, group_fn, weight_scale);
    CPMCU_LAUNCH_CHECK("moe_select");
    return nullptr;
}

#define MOE_ROWS 4       // output rows a wavefront

// grid (tokens * top, ceil(F / 16)), 256 threads: wavefront w takes rows [16 y + 4 w, +4) of the expert's F
template <typename T>
__global__ __launch_bounds__(256) void moe_gated_kernel(const T* __restrict__ h, long ldh, const T* __restrict__ wgu,
                                                        const int* __restrict__ idx, T* __restrict__ act, int H, int F,
                                                        int top, int act_fn, float act_limit) {
    const long pair = blockIdx.x;
    const long t = pair / top;
    const int e = idx[pair];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const T* hr = h + t * ldh;
    const T* wg = wgu + (long)e * 2 * F * H;
    const bool vec = (H % 8 == 0) && (ldh % 8 == 0) && ((uintptr_t)h % 32 == 0) && ((uintptr_t)wgu % 32 == 0);
    const int j0 = blockIdx.y * 4 * MOE_ROWS + wave * MOE_ROWS;
#pragma unroll
    for (int r = 0; r < MOE_ROWS; ++r) {
        const int j = j0 + r;
        if (j >= F) break;
        float g = wave_sum(lane_dot<T, T>(wg + (long)j * H, hr, H, lane, vec));
        float u = wave_sum(lane_dot<T, T>(wg + (long)(F + j) * H, hr, H, lane, vec));
        gate_prepare(g, u, act_fn, act_limit);
        if (lane == 0) act[pair * F + j] = from_f32<T>(gate_act(g, act_fn) * u);
    }
}

extern "C" const char* cpmcu_moe_gated(const void* h, long ldh, int dtype, const void* wgu, const int* idx, void* act,
                                       int n, int H, int F, int top, int act_fn, float act_limit, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && F > 0 && top > 0, "moe_gated: empty shape");
    CPMCU_REQUIRE(CPMCU_ACT_KNOWN(act_fn), "moe_gated: unknown nonlinearity %d", act_fn);
    const int fy = (F + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS);
    CPMCU_REQUIRE(fy <= 65535, "moe_gated: %d rows an expert exceed the launch grid", F);
    dim3 grid((unsigned)((long)n * top), fy);
    if (dtype == CPMCU_F32)
        moe_gated_kernel<float><<<grid, 256, 0, stream>>>((const float*)h, ldh, (const float*)wgu, idx, (float*)act, H, F, top, act_fn, act_limit);
    else if (dtype == CPMCU_BF16)
        moe_gated_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)h, ldh, (const bf16_t*)wgu, idx, (bf16_t*)act, H, F, top, act_fn, act_limit);
    else
        CPMCU_FAIL("moe_gated: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("moe_gated");
    return nullptr;
}

// grid (tokens, ceil(H / 16)), 256 threads.  shared: the every-token expert's output [n, H] (or float partial
// sums [parts][n][H]), multiplied by sg[t]; may be absent.
template <typename T, typename ST>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const T* __restrict__ wd,
                                                       const int* __restrict__ idx, const float* __restrict__ w,
                                                       const ST* __restrict__ shared, int shared_parts,
                                                       long shared_stride, const float* __restrict__ sg,
                                                       float* __restrict__ out, int H, int F, int top) {
    const long t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const bool vec = (F % 8 == 0) && ((uintptr_t)act % 32 == 0) && ((uintptr_t)wd % 32 == 0);
    const int c0 = blockIdx.y * 4 * MOE_ROWS + wave * MOE_ROWS;
#pragma unroll
    for (int r = 0; r < MOE_ROWS; ++r) {
        const int c = c0 + r;
        if (c >= H) break;
        float s = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = idx[t * top + k];
            s += w[t * top + k] * lane_dot<T, T>(wd + ((long)e * H + c) * F, act + (t * top + k) * F, F, lane, vec);
        }
        s = wave_sum(s);
        if (lane == 0) {
            if (shared) {
                float v = 0.f;
                for (int p = 0; p < shared_parts; ++p) v += to_f32(shared[(long)p * shared_stride + t * H + c]);
                s += (sg ? sg[t] : 1.0f) * v;
            }
            out[t * H + c] = s;
        }
    }
}

extern "C" const char* cpmcu_moe_down(const void* act, int dtype, const void* wd, const int* idx, const float* w,
                                      const void* shared, int shared_dtype, int shared_parts, long shared_stride,
                                      const float* sg, float* out, int n, int H, int F, int top, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && F > 0 && top > 0, "moe_down: empty shape");
    const int hy = (H + 4 * MOE_ROWS - 1) / (4 * MOE_ROWS);
    CPMCU_REQUIRE(hy <= 65535, "moe_down: a width of %d exceeds the launch grid", H);
    dim3 grid(n, hy);
#define LAUNCH(Tv, STv)                                                                                            \
    moe_down_kernel<Tv, STv><<<grid, 256, 0, stream>>>((const Tv*)act, (const Tv*)wd, idx, w, (const STv*)shared,   \
                                                       shared_parts, shared_stride, sg, out, H, F, top)
    const int sd = shared ? shared_dtype : CPMCU_F32;
    if (dtype == CPMCU_F32 && sd == CPMCU_F32) LAUNCH(float, float);
    else if (dtype == CPMCU_BF16 && sd == CPMCU_F32) LAUNCH(bf16_t, float);
    else if (dtype == CPMCU_BF16 && sd == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else CPMCU_FAIL("moe_down: unsupported dtypes act=%d shared=%d", dtype, sd);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("moe_down");
    return nullptr;
}

// ===========================================================================
// The same experts for steps of many tokens, bf16 on the matrix cores (v_mfma_f32_16x16x32_bf16): the (token,
// chosen expert) pairs are grouped by expert into tiles of 64 rows, and every tile is a product with its
// expert's weights.
//
//  * moe_group_kernel (one workgroup): counts the pairs of every expert, gives every expert whole tiles of 64 rows
//    (rows[tile * 64 + i] = pair, -1 in a tile's unused rows), tile_expert[tile] and the number of tiles.  Which row
//    of its expert's tiles a pair gets depends on timing; its result does not (a row's sums are its own).
//  * moe_gated_mfma_kernel: act[pair] = silu(Wg_e h_t) * (Wu_e h_t); a wavefront owns the 64 rows of a tile and 32
//    features (two tiles of gate rows, two of up rows): 16 matrix instructions for 8 operand loads, operands
//    straight from memory (the 4 wavefronts of a workgroup read the same rows of h, which meet in the CU's cache).
//  * moe_down_mfma_kernel: y[pair] = Wd_e act[pair] (bf16); a wavefront owns the 64 rows and 64 columns.
//  * moe_combine_kernel: out[t] = sum_k w[t, k] y[t, k] (+ sg[t] * shared[t]) in float, k in order.
// ===========================================================================
typedef __bf16 mbf16x8_t __attribute__((ext_vector_type(8)));
typedef float mfloatx4_t __attribute__((ext_vector_type(4)));

#define MOE_TILE 64

__global__ __launch_bounds__(1024) void moe_group_kernel(const int* __restrict__ idx, int n_pairs, int E,
                                                         int* __restrict__ rows, int* __restrict__ tile_expert,
                                                         int* __restrict__ n_tiles_out, int max_tiles) {
    __shared__ int counts[MOE_MAX_EXPERTS];
    __shared__ int offs[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < E; e += 1024) counts[e] = 0;
    for (int i = threadIdx.x; i < max_tiles * MOE_TILE; i += 1024) rows[i] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += 1024) atomicAdd(&counts[idx[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int e = 0; e < E; ++e) {
            offs[e] = t * MOE_TILE;
            const int nt = (counts[e] + MOE_TILE - 1) / MOE_TILE;
            for (int i = 0; i < nt; ++i) tile_expert[t + i] = e;
            t += nt;
        }
        *n_tiles_out = t;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 1024) counts[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += 1024) {
        const int e = idx[p];
        rows[offs[e] + atomicAdd(&counts[e], 1)] = p;
    }
}

// grid (ceil(F / 128), max_tiles), 256 threads: a wavefront takes all 64 rows of the tile and 32 features
__global__ __launch_bounds__(256) void moe_gated_mfma_kernel(const bf16_t* __restrict__ h, long ldh,
                                                             const bf16_t* __restrict__ wgu, const int* __restrict__ rows,
                                                             const int* __restrict__ tile_expert,
                                                             const int* __restrict__ n_tiles, bf16_t* __restrict__ act,
                                                             int H, int F, int top, int act_fn, float act_limit) {
    const int tile = blockIdx.y;
    if (tile >= *n_tiles) return;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int e = tile_expert[tile];
    const int f0 = blockIdx.x * 128 + wave * 32;
    if (f0 >= F) return;
    const bf16_t* xp[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const int pair = rows[tile * MOE_TILE + rt * 16 + r];
        xp[rt] = h + (long)(pair >= 0 ? pair / top : 0) * ldh + g * 8;
    }
    const bf16_t* wp = wgu + (long)e * 2 * F * H + g * 8;
    mfloatx4_t acc[4][4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[rt][j] = mfloatx4_t{0.f, 0.f, 0.f, 0.f};
    long wrow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {                 // j = 0, 1: gate rows f0 + 16 j + r; j = 2, 3: their up rows
        const int f = min(f0 + 16 * (j & 1) + r, F - 1);
        wrow[j] = (long)((j >> 1) * F + f) * H;
    }
    for (int k0 = 0; k0 < H; k0 += 32) {
        const bool k_ok = k0 + g * 8 < H;
        const int kk = k_ok ? k0 : k0 - g * 8;       // a lane beyond the row's end reads the step's first columns (in range) and is zeroed
        mbf16x8_t a[4], b[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) a[rt] = *(const mbf16x8_t*)(xp[rt] + kk);
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = *(const mbf16x8_t*)(wp + wrow[j] + kk);
        if (!k_ok) {
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = b[j] = mbf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[rt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], b[j], acc[rt][j], 0, 0, 0);
    }
    // lane (feature column r, g): acc[rt][j][i] belongs to the tile's row rt * 16 + 4 g + i
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p = rows[tile * MOE_TILE + rt * 16 + 4 * g + i];
            if (p < 0) continue;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int f = f0 + 16 * j + r;
                if (f < F) {
                    float gt = acc[rt][j][i], up = acc[rt][2 + j][i];
                    gate_prepare(gt, up, act_fn, act_limit);
                    act[(long)p * F + f] = f32_to_bf16(gate_act(gt, act_fn) * up);
                }
            }
        }
}

// grid (ceil(H / 256), max_tiles), 256 threads: a wavefront takes all 64 rows of the tile and 64 columns
__global__ __launch_bounds__(256) void moe_down_mfma_kernel(const bf16_t* __restrict__ act, const bf16_t* __restrict__ wd,
                                                            const int* __restrict__ rows,
                                                            const int* __restrict__ tile_expert,
                                                            const int* __restrict__ n_tiles, bf16_t* __restrict__ y,
                                                            int H, int F) {
    const int tile = blockIdx.y;
    if (tile >= *n_tiles) return;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int e = tile_expert[tile];
    const int c0 = blockIdx.x * 256 + wave * 64;
    if (c0 >= H) return;
    const bf16_t* xp[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const int pair = rows[tile * MOE_TILE + rt * 16 + r];
        xp[rt] = act + (long)(pair >= 0 ? pair : 0) * F + g * 8;
    }
    const bf16_t* wp = wd + (long)e * H * F + g * 8;
    mfloatx4_t acc[4][4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[rt][j] = mfloatx4_t{0.f, 0.f, 0.f, 0.f};
    long wrow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) wrow[j] = (long)min(c0 + 16 * j + r, H - 1) * F;
    for (int k0 = 0; k0 < F; k0 += 32) {
        const bool k_ok = k0 + g * 8 < F;
        const int kk = k_ok ? k0 : k0 - g * 8;
        mbf16x8_t a[4], b[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) a[rt] = *(const mbf16x8_t*)(xp[rt] + kk);
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = *(const mbf16x8_t*)(wp + wrow[j] + kk);
        if (!k_ok) {
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = b[j] = mbf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[rt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[rt], b[j], acc[rt][j], 0, 0, 0);
    }
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int p = rows[tile * MOE_TILE + rt * 16 + 4 * g + i];
            if (p < 0) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = c0 + 16 * j + r;
                if (c < H) y[(long)p * H + c] = f32_to_bf16(acc[rt][j][i]);
            }
        }
}

template <typename ST>
__global__ __launch_bounds__(256) void moe_combine_kernel(const bf16_t* __restrict__ y, const float* __restrict__ w,
                                                          const ST* __restrict__ shared, int shared_parts,
                                                          long shared_stride, const float* __restrict__ sg,
                                                          float* __restrict__ out, long total, int H, int top) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const long t = i / H;
        const int c = (int)(i - t * H);
        float s = 0.f;
        for (int k = 0; k < top; ++k) s += w[t * top + k] * to_f32(y[(t * top + k) * H + c]);
        if (shared) {
            float v = 0.f;
            for (int p = 0; p < shared_parts; ++p) v += to_f32(shared[(long)p * shared_stride + i]);
            s += (sg ? sg[t] : 1.0f) * v;
        }
        out[i] = s;
    }
}

// scratch: rows int [max_tiles * 64], tile_expert int [max_tiles], n_tiles int [1], y bf16 [n * top, H];
// max_tiles = ceil(n * top / 64) + E
extern "C" const char* cpmcu_moe_experts_mfma(const void* h, long ldh, const void* wgu, const void* wd, const int* idx,
                                              const float* w, const void* shared, int shared_dtype, int shared_parts,
                                              long shared_stride, const float* sg, void* act, void* y, int* rows,
                                              int* tile_expert, int* n_tiles, int max_tiles, float* out, int n, int H,
                                              int F, int E, int top, int act_fn, float act_limit, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && F > 0 && E > 0 && top > 0, "moe_experts_mfma: empty shape");
    CPMCU_REQUIRE(CPMCU_ACT_KNOWN(act_fn), "moe_experts_mfma: unknown nonlinearity %d", act_fn);
    CPMCU_REQUIRE(E <= MOE_MAX_EXPERTS, "moe_experts_mfma: %d experts (up to %d are taken)", E, MOE_MAX_EXPERTS);
    CPMCU_REQUIRE(H % 8 == 0 && F % 8 == 0 && ldh % 8 == 0 && (uintptr_t)h % 16 == 0 && (uintptr_t)wgu % 16 == 0 &&
                  (uintptr_t)wd % 16 == 0 && (uintptr_t)act % 16 == 0,
                  "moe_experts_mfma: widths must be multiples of 8 and operands start on 16-byte borders (H=%d, F=%d)", H, F);
    const long pairs = (long)n * top;
    CPMCU_REQUIRE(max_tiles >= (pairs + MOE_TILE - 1) / MOE_TILE + E && max_tiles <= 65535,
                  "moe_experts_mfma: %d tiles of scratch for %ld pairs of %d experts (at most 65535)", max_tiles, pairs, E);
    moe_group_kernel<<<1, 1024, 0, stream>>>(idx, (int)pairs, E, rows, tile_expert, n_tiles, max_tiles);
    CPMCU_LAUNCH_CHECK("moe_group");
    moe_gated_mfma_kernel<<<dim3((F + 127) / 128, max_tiles), 256, 0, stream>>>((const bf16_t*)h, ldh, (const bf16_t*)wgu, rows,
                                                                            tile_expert, n_tiles, (bf16_t*)act, H, F, top, act_fn, act_limit);
    CPMCU_LAUNCH_CHECK("moe_gated_mfma");
    moe_down_mfma_kernel<<<dim3((H + 255) / 256, max_tiles), 256, 0, stream>>>((const bf16_t*)act, (const bf16_t*)wd, rows,
                                                                           tile_expert, n_tiles, (bf16_t*)y, H, F);
    CPMCU_LAUNCH_CHECK("moe_down_mfma");
    const long total = (long)n * H;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    if (!shared || shared_dtype == CPMCU_F32)
        moe_combine_kernel<float><<<blocks, 256, 0, stream>>>((const bf16_t*)y, w, (const float*)shared, shared_parts,
                                                              shared_stride, sg, out, total, H, top);
    else
        moe_combine_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)y, w, (const bf16_t*)shared, shared_parts,
                                                               shared_stride, sg, out, total, H, top);
    CPMCU_LAUNCH_CHECK("moe_combine");
    return nullptr;
}
