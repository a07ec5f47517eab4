// Attention pieces for mixers whose keys and values differ in size, whose rotation covers part of a head,
// or whose mask is cut into chunks:
//
//  * rotate_copy_kernel: copies a run of features of every (token, head) from rows of a projection to plain
//    rows or into the paged cache (key or value layout, at a feature offset inside the cached head), rotating
//    the first `rot_dims` of them: feature i pairs with i + rot_dims/2, (u, v) -> (u cos a - v sin a,
//    v cos a + u sin a), a = position * inv_freq[i] in float, cos and sin times `mag`; features beyond
//    rot_dims pass unchanged.
//  * attention_general_kernel: the plain attention over the paged cache with key size hdk and value size hdv
//    of their own (the cache may hold them padded to pool_hdk, pool_hdv), grouped heads, and an optional chunked mask: the query at position p sees keys j <= p with
//    floor(j / chunk) == floor(p / chunk), chunks counted from position 0 of the sequence; or a sliding window
//    with kept first tokens: key j <= p is seen if p - j < window or j < keep_first.  With `sink` (a float a head)
//    the softmax's denominator holds exp(sink[head]) as one more term that has no key and no value.  Float scores
//    and softmax, both element types; one wavefront a (token, head).
//
// Keys and values lie in their pages as common.h says (key_index, value_index), each with its own head size.
#include "common.h"

enum { DST_ROWS = 0, DST_KEYS = 1, DST_VALUES = 2 };

// grid (tokens, heads), 64 threads.  src: [n, ld_src], head h's run starts at src_off + h * src_head_stride.
// dst rows: dst[t * ld_dst + dst_off + h * dst_head_stride + i]; dst pages: head h of `pool_heads` cached heads
// of `pool_hd` features, feature dst_off + i.
template <typename IT, typename OT, int MODE>
__global__ __launch_bounds__(64) void rotate_copy_kernel(const IT* __restrict__ src, long ld_src, long src_head_stride,
                                                         long src_off, OT* __restrict__ dst, long ld_dst,
                                                         long dst_head_stride, long dst_off, int width, int rot_dims,
                                                         const int* __restrict__ positions,
                                                         const int* __restrict__ tok_slot,
                                                         const float* __restrict__ inv_freq, float mag, PagedView pv,
                                                         int pool_heads, int pool_hd) {
    const long t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const IT* s = src + t * ld_src + src_off + (long)h * src_head_stride;
    OT* d;
    if (MODE == DST_ROWS) {
        d = dst + t * ld_dst + dst_off + (long)h * dst_head_stride;
    } else {
        const long row = paged_row(pv, tok_slot[t], pos);
        d = dst + (MODE == DST_KEYS ? key_index(row, h, pool_heads, pool_hd) : value_index(row, h, pool_heads, pool_hd));
    }
    auto at = [&](int i) -> long {
        if (MODE == DST_ROWS) return i;
        const int f = (int)dst_off + i;
        return MODE == DST_KEYS ? key_d_offset(f) : value_d_offset(f);
    };
    const int half = rot_dims / 2;
    for (int i = lane; i < half; i += 64) {
        const float ang = (float)pos * inv_freq[i];
        const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
        const float u = to_f32(s[i]), v = to_f32(s[i + half]);
        d[at(i)] = from_f32<OT>(u * cs - v * sn);
        d[at(i + half)] = from_f32<OT>(v * cs + u * sn);
    }
    for (int i = rot_dims + lane; i < width; i += 64) d[at(i)] = from_f32<OT>(to_f32(s[i]));
}

extern "C" const char* cpmcu_rotate_copy(const void* src, int src_dtype, long ld_src, long src_head_stride, long src_off,
                                         void* dst, int dst_dtype, int mode, long ld_dst, long dst_head_stride,
                                         long dst_off, int n, int heads, int width, int rot_dims, const int* positions,
                                         const int* tok_slot, const float* inv_freq, float mag, const int* page_table,
                                         int table_width, int page_size, int pool_heads, int pool_hd,
                                         hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && heads > 0 && width > 0, "rotate_copy: empty shape n=%d heads=%d width=%d", n, heads, width);
    CPMCU_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= width,
                  "rotate_copy: %d rotated features of %d (an even number, at most the run)", rot_dims, width);
    CPMCU_REQUIRE(rot_dims == 0 || inv_freq, "rotate_copy: frequencies missing");
    CPMCU_REQUIRE(heads <= 65535, "rotate_copy: %d heads exceed the launch grid", heads);
    CPMCU_REQUIRE(mode == DST_ROWS || (page_table && tok_slot && page_size % 32 == 0 && pool_hd % 16 == 0 &&
                                       heads <= pool_heads && dst_off + width <= pool_hd),
                  "rotate_copy: the cache takes pages of a multiple of 32 tokens and head sizes in steps of 16 "
                  "(page %d, head size %d, features %ld..%ld)", page_size, pool_hd, dst_off, dst_off + width);
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, heads);
#define LAUNCH(IT, OT, M)                                                                                         \
    rotate_copy_kernel<IT, OT, M><<<grid, 64, 0, stream>>>((const IT*)src, ld_src, src_head_stride, src_off, (OT*)dst, \
                                                           ld_dst, dst_head_stride, dst_off, width, rot_dims,     \
                                                           positions, tok_slot, inv_freq, mag, pv, pool_heads, pool_hd)
#define BY_MODE(IT, OT)                           \
    do {                                          \
        if (mode == DST_ROWS) LAUNCH(IT, OT, 0);  \
        else if (mode == DST_KEYS) LAUNCH(IT, OT, 1); \
        else if (mode == DST_VALUES) LAUNCH(IT, OT, 2); \
        else CPMCU_FAIL("rotate_copy: unknown destination %d", mode); \
    } while (0)
    if (src_dtype == CPMCU_F32 && dst_dtype == CPMCU_F32) BY_MODE(float, float);
    else if (src_dtype == CPMCU_F32 && dst_dtype == CPMCU_BF16) BY_MODE(float, bf16_t);
    else if (src_dtype == CPMCU_BF16 && dst_dtype == CPMCU_BF16) BY_MODE(bf16_t, bf16_t);
    else CPMCU_FAIL("rotate_copy: unsupported dtypes in=%d out=%d", src_dtype, dst_dtype);
#undef BY_MODE
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("rotate_copy");
    return nullptr;
}

#define AG_MAX_HD 1024

// v_share (both attention kernels): runs of v_share neighbouring key heads read one value head (the value pages
// hold nkv / v_share heads): several score maps over the same values.  1: every key head has its value head.

template <typename T>
__global__ __launch_bounds__(64) void attention_general_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ kpool, const T* __restrict__ vpool,
    PagedView pv, const int* __restrict__ positions, const int* __restrict__ tok_slot, int nh, int nkv, int hdk,
    int hdv, int pool_hdk, int pool_hdv, float scale, int chunk, int window, int keep_first,
    const float* __restrict__ sink, int v_share, float softcap) {
    __shared__ float qs[AG_MAX_HD];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (nh / nkv);
    const int pos = positions[t], slot = tok_slot[t];
    const T* qrow = q + ((long)t * nh + h) * hdk;
    for (int d = lane; d < hdk; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();
    const int nd = (hdv + 63) / 64;
    float acc[AG_MAX_HD / 64];
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / 64; ++i) acc[i] = 0.f;
    float m = -INFINITY, l = 0.f;
    const int s0 = chunk > 0 ? pos - pos % chunk : (window > 0 ? max(pos - window + 1, 0) : 0), s1 = pos + 1;
    // the visible keys in one list: the kept first tokens that lie before the window, then the window
    const int kept = min(keep_first, s0), total = kept + s1 - s0;
    for (int i0 = 0; i0 < total; i0 += 64) {
        const int i = i0 + lane;
        const bool valid = i < total;
        const int j = i < kept ? i : s0 + (i - kept);
        int row = 0;
        float s = -INFINITY;
        if (valid) {
            row = (int)paged_row(pv, slot, j);
            const T* kr = kpool + key_index(row, g, nkv, pool_hdk);
            float dot = 0.f;
            for (int d = 0; d < hdk; ++d) dot += qs[d] * to_f32(kr[key_d_offset(d)]);
            s = dot * scale;
            if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);
        l = l * corr + wave_sum(p);
        m = m_new;
        const int cnt = min(64, total - i0);
#pragma unroll
        for (int i = 0; i < AG_MAX_HD / 64; ++i) acc[i] *= corr;
        for (int jj = 0; jj < cnt; ++jj) {
            const float pj = __shfl(p, jj, 64);
            const int rj = __shfl(row, jj, 64);
            const T* vr = vpool + value_index(rj, g / v_share, nkv / v_share, pool_hdv);
#pragma unroll
            for (int i = 0; i < AG_MAX_HD / 64; ++i) {
                const int d = lane + 64 * i;
                if (i < nd && d < hdv) acc[i] += pj * to_f32(vr[value_d_offset(d)]);
            }
        }
    }
    T* orow = out + ((long)t * nh + h) * hdv;
    if (sink) l += expf(sink[h] - m);
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / 64; ++i) {
        const int d = lane + 64 * i;
        if (i < nd && d < hdv) orow[d] = from_f32<T>(acc[i] * inv);
    }
}

extern "C" const char* cpmcu_attention_general(const void* q, void* out, int dtype, int n, int nh, int nkv, int hdk,
                                               int hdv, int pool_hdk, int pool_hdv, float scale, int chunk, int window,
                                               int keep_first, const float* sink, const void* kpool,
                                               const void* vpool,
                                               const int* page_table, int table_width, int page_size,
                                               const int* positions, const int* tok_slot, int v_share,
                                               float softcap, hipStream_t stream) {
    CPMCU_REQUIRE(v_share >= 1 && nkv % v_share == 0, "attention_general: %d key heads do not share values in runs of %d", nkv, v_share);
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && hdk > 0 && hdv > 0,
                  "attention_general: empty shape n=%d heads=%d kv_heads=%d key size=%d value size=%d", n, nh, nkv, hdk, hdv);
    CPMCU_REQUIRE(nh % nkv == 0, "attention_general: %d heads are not a multiple of %d kv heads", nh, nkv);
    CPMCU_REQUIRE(hdk <= AG_MAX_HD && hdv <= AG_MAX_HD, "attention_general: key size %d / value size %d (up to %d are taken)",
                  hdk, hdv, AG_MAX_HD);
    CPMCU_REQUIRE(pool_hdk >= hdk && pool_hdv >= hdv && pool_hdk % 16 == 0 && pool_hdv % 16 == 0 && page_size % 32 == 0,
                  "attention_general: the cache holds heads in steps of 16 features and pages of a multiple of 32 tokens "
                  "(cached key size %d, value size %d, page %d)", pool_hdk, pool_hdv, page_size);
    CPMCU_REQUIRE(nh <= 65535, "attention_general: %d heads exceed the launch grid", nh);
    CPMCU_REQUIRE(chunk >= 0 && window >= 0 && keep_first >= 0 && (chunk == 0 || window == 0) && (window > 0 || keep_first == 0),
                  "attention_general: mask chunk %d, window %d, kept first tokens %d (a chunk or a window, not both; "
                  "kept tokens only with a window)", chunk, window, keep_first);
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, nh);
    if (dtype == CPMCU_F32)
        attention_general_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, (float*)out, (const float*)kpool,
                                                                 (const float*)vpool, pv, positions, tok_slot, nh, nkv,
                                                                 hdk, hdv, pool_hdk, pool_hdv, scale, chunk, window,
                                                                 keep_first, sink, v_share, softcap);
    else if (dtype == CPMCU_BF16)
        attention_general_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kpool,
                                                                  (const bf16_t*)vpool, pv, positions, tok_slot, nh,
                                                                  nkv, hdk, hdv, pool_hdk, pool_hdv, scale, chunk, window,
                                                                  keep_first, sink, v_share, softcap);
    else
        CPMCU_FAIL("attention_general: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("attention_general");
    return nullptr;
}

// ===========================================================================
// The same attention in bf16 on the matrix cores (v_mfma_f32_16x16x32_bf16), for prompts and single tokens.
//
// One wavefront owns one query token, one kv head and up to 16 of its query heads, and a share of the
// token's visible keys (split over blockIdx.z for steps of few tokens, and over the 4 wavefronts of a workgroup
// when NW = 4).  Keys are visited in chunks of 32, as they lie in their pages:
//   S^T = K . Q^T     A = 16 keys x 32 features straight from the page, B = Q^T read from LDS (written there
//                     once per token: a head of several hundred features does not fit registers beside the
//                     output), looped over the key size at run time
//   P^T = exp2(S^T c - m) in float per head, running maximum and sum
//   O^T += V^T . P^T  A = V^T, 16 features x 32 keys a tile; the output of up to DTM tiles stays in registers
// The mask is causal, and with chunk > 0 the keys before the start of the query's chunk are skipped (whole
// 32-key chunks) or masked; with window > 0 the keys more than window - 1 positions back are, except the first
// keep_first keys of the sequence, whose 32-key chunks are visited before the window's.  With `sink` the
// denominator gains exp(sink[head]) at the end (here, or in the merge kernel when the keys are split).  Output: out (bf16) when n_splits == 1, else unnormalised shares part_o
// [token][head][split][hdv] and part_ml [token][head][split] = (max, sum) for the merge kernel below.
// ===========================================================================
typedef __bf16 gbf16x8_t __attribute__((ext_vector_type(8)));
typedef float gfloatx4_t __attribute__((ext_vector_type(4)));

// VS (features split): the 4 wavefronts of a workgroup all visit all of the workgroup's keys; each computes the
// scores' share of a quarter of the key features (the shares are summed through LDS) and owns a quarter of the
// value features (DTM tiles of 16 from tile wave * DTM on): for keys and values too wide to keep a whole
// output row in one wavefront's registers.  Every key and value is loaded once, and nothing is merged at the end.
template <int DTM, int NW, int TW, bool VS>
__global__ __launch_bounds__(NW * TW * 64) void attention_general_mfma_kernel(
    const bf16_t* __restrict__ q, void* __restrict__ out, int out_f32, float* __restrict__ part_o,
    float2* __restrict__ part_ml, const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vtpool, PagedView pv,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, int nh, int nkv, int hdk, int hdv,
    int pool_hdk, int pool_hdv, float scale_log2e, int chunk, int window, int keep_first, const float* __restrict__ sink,
    int n_splits, int n_tokens, const int* __restrict__ tiles, int n_tiles, int tpt, int rpt, int v_share,
    const bf16_t* __restrict__ gate, long ld_gate, float cap_in, float cap_out) {
    extern __shared__ __align__(16) unsigned char smem[];
    static_assert(NW == 1 || TW == 1, "either the wavefronts of a workgroup share a token or each has its own");
    const int ksteps = (pool_hdk + 31) >> 5, dtn = pool_hdv >> 4;
    const int kvh = blockIdx.y % nkv, ht = blockIdx.y / nkv, split = blockIdx.z;
    const int wave_id = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wave = TW > 1 ? 0 : wave_id;
    // A wavefront's tile of 16 columns holds one token's heads, or (tiles given, groups smaller than 16) the
    // heads of up to tpt consecutive tokens of one sequence, rpt columns each: column n is token n / rpt of
    // the tile, head n % rpt of the group.
    const int unit = blockIdx.x * TW + (TW > 1 ? wave_id : 0);
    const int n_units = tiles ? n_tiles : n_tokens;
    const bool live = unit < n_units;
    const int un = live ? unit : n_units - 1;
    const int t0 = tiles ? tiles[2 * un] : un, n_tok = tiles ? tiles[2 * un + 1] : 1;
    const int lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int G = nh / nkv;
    const int tk = n / rpt, hh = ht * 16 + n % rpt;
    const bool head_ok = tk < n_tok && tk < tpt && hh < G;
    const int t = t0 + (tk < n_tok ? tk : 0);
    const int head = kvh * G + (hh < G ? hh : 0);
    const int pos = positions[t], slot = tok_slot[t0];
    const int pos_min = positions[t0], pos_max = pos_min + n_tok - 1;     // a tile's tokens are consecutive

    // Q^T fragments of this wavefront's token: [ksteps][lane] of 8 features
    gbf16x8_t* qs = (gbf16x8_t*)smem + (long)(TW > 1 ? wave_id : 0) * ksteps * 64;
    for (int ks = wave; ks < ksteps; ks += NW) {
        gbf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        const int d = ks * 32 + g * 8;
        if (head_ok && d < hdk) v = *(const gbf16x8_t*)(q + ((long)t * nh + head) * hdk + d);
        qs[ks * 64 + lane] = v;
    }
    __syncthreads();

    const int first_key = chunk > 0 ? pos - pos % chunk : (window > 0 ? max(pos - window + 1, 0) : 0);
    const int first_min = chunk > 0 ? pos_min - pos_min % chunk : (window > 0 ? max(pos_min - window + 1, 0) : 0);
    const int first_max = chunk > 0 ? pos_max - pos_max % chunk : (window > 0 ? max(pos_max - window + 1, 0) : 0);
    const int cfirst = first_min >> 5;
    // 32-key chunks of the kept first tokens that lie before the window's first chunk come first in the list
    const int ckeep = min((keep_first + 31) >> 5, cfirst);
    const int total_chunks = ckeep + (pos_max >> 5) + 1 - cfirst;
    const int per_split = (total_chunks + n_splits - 1) / n_splits;
    const int c0 = split * per_split, c1 = min(c0 + per_split, total_chunks);

    gfloatx4_t acc[DTM];
#pragma unroll
    for (int dt = 0; dt < DTM; ++dt) acc[dt] = gfloatx4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const int lane_off = (g * 16 + n) * 8;
    const long kchunk = 32L * pool_hdk, vchunk = 32L * pool_hdv;
    const int tile1 = (pool_hdk >> 3) * 128;                      // the second tile of 16 key slots

    const int dt0 = VS ? wave * DTM : 0;
    const int kq = VS ? (ksteps + NW - 1) / NW : ksteps;
    const int ks_a = VS ? wave * kq : 0, ks_b = VS ? min(ks_a + kq, ksteps) : ksteps;
    float* sc_s = (float*)(smem + (long)ksteps * 64 * 16);        // VS: partial scores, behind the Q fragments
    int parity = 0;
    for (int c = VS ? c0 : c0 + wave; c < c1; c += VS ? 1 : NW) {
        const int key0 = (c < ckeep ? c : cfirst + (c - ckeep)) << 5;
        const long pchunk = paged_row(pv, slot, key0) >> 5;
        const bf16_t* kp = kpool + (pchunk * nkv + kvh) * kchunk + lane_off;
        const bf16_t* vp = vtpool + (pchunk * (nkv / v_share) + kvh / v_share) * vchunk + lane_off;
        // the values are asked for first: they arrive behind the scores' work.  No load stands in a branch
        // (lanes beyond the head's features read its first ones and are zeroed by a select), so that the
        // compiler keeps several steps' loads in flight.
        gbf16x8_t vf[DTM];
#pragma unroll
        for (int dt = 0; dt < DTM; ++dt) vf[dt] = *(const gbf16x8_t*)(vp + min(dt0 + dt, dtn - 1) * 512);
        gfloatx4_t st0 = {0.f, 0.f, 0.f, 0.f}, st1 = {0.f, 0.f, 0.f, 0.f};
        const gbf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 6
        for (int ks = ks_a; ks < ks_b; ++ks) {
            const bool ok = ks * 32 + g * 8 < pool_hdk;
            const int off = ok ? ks * 512 : -g * 128;
            gbf16x8_t k0 = *(const gbf16x8_t*)(kp + off);
            gbf16x8_t k1 = *(const gbf16x8_t*)(kp + tile1 + off);
            k0 = ok ? k0 : zero8;
            k1 = ok ? k1 : zero8;
            const gbf16x8_t qv = qs[ks * 64 + lane];
            st0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qv, st0, 0, 0, 0);
            st1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qv, st1, 0, 0, 0);
        }
        if (VS) {
            // every wavefront took a quarter of the key features: the four partial scores meet in LDS (two
            // buffers in turn, so that one barrier a chunk is enough)
            float* sc = sc_s + (parity ? NW * 8 * 64 : 0);
            parity ^= 1;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                sc[(wave * 8 + e) * 64 + lane] = st0[e];
                sc[(wave * 8 + 4 + e) * 64 + lane] = st1[e];
            }
            __syncthreads();
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float a0 = 0.f, a1 = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    a0 += sc[(w * 8 + e) * 64 + lane];
                    a1 += sc[(w * 8 + 4 + e) * 64 + lane];
                }
                st0[e] = a0;
                st1[e] = a1;
            }
        }
        // lane (head n, g): st0[e] is key key0 + 8g + e, st1[e] is key key0 + 8g + 4 + e
        if (cap_out > 0.f) {
            // capped scores c tanh(s scale / c), here already times log2(e): cap_in = scale / c, cap_out = c log2(e),
            // and scale_log2e is 1 for the softmax below
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                st0[e] = cap_out * tanhf(st0[e] * cap_in);
                st1[e] = cap_out * tanhf(st1[e] * cap_in);
            }
        }
        if (key0 + 31 > pos_min || (key0 < first_max && key0 + 31 >= keep_first)) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int ka = key0 + 8 * g + e, kb = ka + 4;
                if (ka > pos || (ka < first_key && ka >= keep_first)) st0[e] = -INFINITY;
                if (kb > pos || (kb < first_key && kb >= keep_first)) st1[e] = -INFINITY;
            }
        }
        float mx = fmaxf(fmaxf(fmaxf(st0[0], st0[1]), fmaxf(st0[2], st0[3])),
                         fmaxf(fmaxf(st1[0], st1[1]), fmaxf(st1[2], st1[3])));
        mx = rows_max(mx);
        const float m_new = fmaxf(m, mx * scale_log2e);
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;
        const float corr = exp2f(m - m_ref);
        float rs = 0.f;
        gbf16x8_t pb;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float p0 = exp2f(__builtin_fmaf(st0[e], scale_log2e, -m_ref));
            const float p1 = exp2f(__builtin_fmaf(st1[e], scale_log2e, -m_ref));
            rs += p0 + p1;
            pb[e] = (__bf16)p0;
            pb[4 + e] = (__bf16)p1;
        }
        rs = rows_sum(rs);
        l = l * corr + rs;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < DTM; ++dt) {
            if (dt0 + dt < dtn) {
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[dt][e] *= corr;
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pb, acc[dt], 0, 0, 0);
            }
        }
    }

    if (NW > 1 && !VS) {
        // merge the wavefronts' running results through LDS (behind the Q fragments)
        float* ml_s = (float*)(smem + (long)ksteps * 64 * 16);
        float* acc_s = ml_s + NW * 16 * 2;
        __syncthreads();
        if (g == 0) {
            ml_s[(wave * 16 + n) * 2] = m;
            ml_s[(wave * 16 + n) * 2 + 1] = l;
        }
#pragma unroll
        for (int dt = 0; dt < DTM; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_s[((wave * DTM + dt) * 4 + i) * 64 + lane] = acc[dt][i];
        __syncthreads();
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w)
            if (ml_s[(w * 16 + n) * 2 + 1] > 0.f) m_all = fmaxf(m_all, ml_s[(w * 16 + n) * 2]);
        float l_all = 0.f;
        float sw[NW];
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            sw[w] = ml_s[(w * 16 + n) * 2 + 1] > 0.f ? exp2f(ml_s[(w * 16 + n) * 2] - m_all) : 0.f;
            l_all += sw[w] * ml_s[(w * 16 + n) * 2 + 1];
        }
        m = m_all;
        l = l_all;
#pragma unroll
        for (int dt = 0; dt < DTM; ++dt) {
            if (dt % NW != wave) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float a = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) a += sw[w] * acc_s[((w * DTM + dt) * 4 + i) * 64 + lane];
                acc[dt][i] = a;
            }
        }
    }
    if (!head_ok || !live) return;
    // lane (head n, g): acc[dt][i] is O[head][dt*16 + 4g + i]
    if (n_splits == 1) {
        if (sink) l += exp2f(sink[head] * 1.4426950408889634f - m);
        const float inv = 1.0f / l;
        // the output as bf16, or as float for a consumer that goes on in float (a difference of two maps)
        const long o0 = ((long)t * nh + head) * hdv;
#pragma unroll
        for (int dt = 0; dt < DTM; ++dt) {
            if (dt0 + dt >= dtn || (NW > 1 && !VS && dt % NW != wave)) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = (dt0 + dt) * 16 + 4 * g + i;
                if (d < hdv) {
                    float v = acc[dt][i] * inv;
                    // an output gate: times sigmoid of the token's gate row (heads side by side)
                    if (gate) v /= 1.0f + expf(-to_f32(gate[(long)t * ld_gate + (long)head * hdv + d]));
                    if (out_f32) ((float*)out)[o0 + d] = v;
                    else ((bf16_t*)out)[o0 + d] = f32_to_bf16(v);
                }
            }
        }
    } else {
        const long idx = ((long)t * nh + head) * n_splits + split;
        float* o = part_o + idx * hdv;
#pragma unroll
        for (int dt = 0; dt < DTM; ++dt) {
            if (dt0 + dt >= dtn || (NW > 1 && !VS && dt % NW != wave)) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if ((dt0 + dt) * 16 + 4 * g + i < hdv) o[(dt0 + dt) * 16 + 4 * g + i] = acc[dt][i];
        }
        if (g == 0 && wave == 0) part_ml[idx] = make_float2(m, l);
    }
}

// out[token][head][:] = sum_s 2^(m_s - m) o_s / sum_s 2^(m_s - m) l_s over up to 64 shares (a share without keys
// has l = 0): lane s holds share s's (max, sum), the common maximum and the denominator are wave reductions.
__global__ void attention_general_merge_kernel(const float* __restrict__ part_o, const float2* __restrict__ part_ml,
                                               void* __restrict__ out, int out_f32, int hdv, int n_splits,
                                               const float* __restrict__ sink, int nh,
                                               const bf16_t* __restrict__ gate, long ld_gate) {
    const long row = blockIdx.x;
    const float2* ml = part_ml + row * n_splits;
    const float* po = part_o + row * n_splits * hdv;
    const int lane = threadIdx.x & 63;
    float2 v = make_float2(-INFINITY, 0.f);
    if (lane < n_splits) v = ml[lane];
    const bool has = v.y > 0.f;
    const float m = wave_max(has ? v.x : -INFINITY);
    const float wv = has ? exp2f(v.x - m) : 0.f;
    // rows are (token, head): the sink of the row's head joins the denominator once
    const float extra = sink ? exp2f(sink[row % nh] * 1.4426950408889634f - m) : 0.f;
    const float inv = 1.0f / (wave_sum(wv * v.y) + extra);
    for (int d = threadIdx.x; d < hdv; d += blockDim.x) {
        float a = 0.f;
        int s = 0;
        for (; s + 8 <= n_splits; s += 8) {          // eight shares' loads in flight
            float v8[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v8[u] = po[(long)(s + u) * hdv + d];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                a += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv), s + u)) * v8[u];
        }
        for (; s < n_splits; ++s)
            a += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv), s)) * po[(long)s * hdv + d];
        float r = a * inv;
        if (gate) r /= 1.0f + expf(-to_f32(gate[(row / nh) * ld_gate + (row % nh) * hdv + d]));
        if (out_f32) ((float*)out)[row * hdv + d] = r;
        else ((bf16_t*)out)[row * hdv + d] = f32_to_bf16(r);
    }
}

extern "C" const char* cpmcu_attention_general_mfma(const void* q, void* out, int out_f32, float* part_o, float* part_ml, int n,
                                                    int nh, int nkv, int hdk, int hdv, int pool_hdk, int pool_hdv,
                                                    float scale, int chunk, int window, int keep_first,
                                                    const float* sink, const void* kpool, const void* vtpool,
                                                    const int* page_table, int table_width, int page_size,
                                                    const int* positions, const int* tok_slot, int n_splits,
                                                    const int* tiles, int n_tiles, int tokens_per_tile, int v_share,
                                                    const void* gate, long ld_gate, float softcap, hipStream_t stream) {
    CPMCU_REQUIRE(v_share >= 1 && nkv % v_share == 0, "attention_general_mfma: %d key heads do not share values in runs of %d", nkv, v_share);
    CPMCU_REQUIRE(!gate || ld_gate >= (long)nh * hdv, "attention_general_mfma: gate rows of %ld elements for %d heads of %d", ld_gate, nh, hdv);
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_general_mfma: bad shape n=%d heads=%d kv_heads=%d", n, nh, nkv);
    CPMCU_REQUIRE(hdk > 0 && hdk % 8 == 0 && hdk <= 1024 && hdv > 0 && hdv <= 512,
                  "attention_general_mfma: key size %d (a multiple of 8 up to 1024) / value size %d (up to 512) have no "
                  "matrix-core kernel; the plain kernel takes the rest", hdk, hdv);
    CPMCU_REQUIRE(pool_hdk >= hdk && pool_hdv >= hdv && pool_hdk % 16 == 0 && pool_hdv % 16 == 0 && page_size % 32 == 0,
                  "attention_general_mfma: the cache holds heads in steps of 16 features and pages of a multiple of 32 tokens");
    CPMCU_REQUIRE(n_splits >= 1 && n_splits <= 64 && (n_splits == 1 || (part_o && part_ml)),
                  "attention_general_mfma: %d shares of the keys (1..64 are taken)", n_splits);
    CPMCU_REQUIRE(chunk >= 0 && window >= 0 && keep_first >= 0 && (chunk == 0 || window == 0) && (window > 0 || keep_first == 0),
                  "attention_general_mfma: mask chunk %d, window %d, kept first tokens %d (a chunk or a window, not both; "
                  "kept tokens only with a window)", chunk, window, keep_first);
    const int G = nh / nkv, HT = (G + 15) / 16;
    CPMCU_REQUIRE((long)nkv * HT <= 65535, "attention_general_mfma: too many head tiles");
    PagedView pv{page_table, table_width, page_size};
    const float sl = softcap > 0.f ? 1.0f : scale * 1.4426950408889634f;
    const float cap_in = softcap > 0.f ? scale / softcap : 0.f, cap_out = softcap > 0.f ? softcap * 1.4426950408889634f : 0.f;
    const int ksteps = (pool_hdk + 31) / 32, dtn = pool_hdv / 16;
    const long q_bytes = (long)ksteps * 64 * 16;
    // values up to 128 features: few tokens: 4 wavefronts share a token's keys and merge through LDS; many: a
    // wavefront a token, 4 neighbours a workgroup (while their Q fragments fit LDS).  Wider values: the 4
    // wavefronts of a token's workgroup split the value features.
    const bool vs = dtn > 8;
    const int dtm = vs ? (dtn <= 16 ? 4 : 8) : (dtn <= 4 ? 4 : 8);
    // (four wavefronts that merge through LDS need room there beside the Q fragments)
    const long merge_bytes = (4 * 16 * 2 + 4L * dtm * 4 * 64) * 4;
    const int nw = (vs || (n <= 256 && q_bytes + merge_bytes <= 64 * 1024)) ? 4 : 1;
    // tiles that pack several tokens: only where nothing is merged at the end (a wavefront has a tile to itself, or
    // the four of a workgroup split the features of one tile)
    const int rpt = G < 16 ? G : 16;
    CPMCU_REQUIRE(!tiles || (n_tiles > 0 && (nw == 1 || vs) && n_splits == 1 && tokens_per_tile >= 1 && tokens_per_tile * rpt <= 16),
                  "attention_general_mfma: tiles of %d tokens do not suit this step", tokens_per_tile);
    const int tpt = tiles ? tokens_per_tile : 1;
    const int units = tiles ? n_tiles : n;
    const int tw = (nw == 1 && n_splits == 1 && n >= 64 && 4 * q_bytes <= 48 * 1024) ? 4 : 1;
    const long lds = (tw > 1 ? tw * q_bytes : q_bytes) + ((nw > 1 && !vs) ? (nw * 16 * 2 + (long)nw * dtm * 4 * 64) * 4 : 0) +
                     (vs ? 2L * nw * 8 * 64 * 4 : 0);
    CPMCU_REQUIRE(lds <= 64 * 1024, "attention_general_mfma: %ld bytes of LDS", lds);
    dim3 grid((units + tw - 1) / tw, nkv * HT, n_splits);
#define LAUNCH(DTMv, NWv, TWv, VSv)                                                                              \
    attention_general_mfma_kernel<DTMv, NWv, TWv, VSv><<<grid, NWv * TWv * 64, lds, stream>>>(                   \
        (const bf16_t*)q, out, out_f32, part_o, (float2*)part_ml, (const bf16_t*)kpool, (const bf16_t*)vtpool, pv, \
        positions, tok_slot, nh, nkv, hdk, hdv, pool_hdk, pool_hdv, sl, chunk, window, keep_first, sink, n_splits, n,    \
        tiles, n_tiles, tpt, rpt, v_share, n_splits == 1 ? (const bf16_t*)gate : nullptr, ld_gate, cap_in, cap_out)
    if (vs) {
        if (dtm == 4) LAUNCH(4, 4, 1, true);
        else LAUNCH(8, 4, 1, true);
    } else if (nw == 4) {
        if (dtm == 4) LAUNCH(4, 4, 1, false);
        else LAUNCH(8, 4, 1, false);
    } else if (tw == 4) {
        if (dtm == 4) LAUNCH(4, 1, 4, false);
        else LAUNCH(8, 1, 4, false);
    } else {
        if (dtm == 4) LAUNCH(4, 1, 1, false);
        else LAUNCH(8, 1, 1, false);
    }
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("attention_general_mfma");
    if (n_splits > 1) {
        const unsigned rows = (unsigned)((long)n * nh);
        attention_general_merge_kernel<<<rows, hdv > 128 ? 256 : (hdv > 64 ? 128 : 64), 0, stream>>>(
            part_o, (const float2*)part_ml, out, out_f32, hdv, n_splits, sink, nh, (const bf16_t*)gate, ld_gate);
        CPMCU_LAUNCH_CHECK("attention_general_merge");
    }
    return nullptr;
}

// ===========================================================================
// Fused forms of the steps between a mixer's input projection and its attention.
// ===========================================================================
template <typename IT, typename OT>
__device__ inline void rotate_run(const IT* __restrict__ s, OT* __restrict__ d, int width, int rot_dims, int pos,
                                  const float* __restrict__ inv_freq, float mag, int mode, int f0, int lane, int nl,
                                  int interleaved = 0) {
    auto at = [&](int i) -> long {
        if (mode == DST_ROWS) return i;
        return mode == DST_KEYS ? key_d_offset(f0 + i) : value_d_offset(f0 + i);
    };
    // pair i of the rotation: features (i, i + rot_dims/2), or neighbours (2i, 2i + 1) when interleaved
    const int half = rot_dims / 2;
    for (int i = lane; i < half; i += nl) {
        const float ang = (float)pos * inv_freq[i];
        const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
        const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
        const float u = to_f32(s[ia]), v = to_f32(s[ib]);
        d[at(ia)] = from_f32<OT>(u * cs - v * sn);
        d[at(ib)] = from_f32<OT>(v * cs + u * sn);
    }
    for (int i = rot_dims + lane; i < width; i += nl) d[at(i)] = from_f32<OT>(to_f32(s[i]));
}

// q, k, v of a stacked projection [q: nh*dk | k: nkv*dk | v: nkv*dv] in one launch: q rotated to plain rows,
// k rotated into the key pages, v into the value pages.  grid (tokens, nh + 2 nkv) (nh alone without the cache).
template <typename T>
__global__ __launch_bounds__(64) void qkv_rotate_store_kernel(const T* __restrict__ qkv, long ld, T* __restrict__ q_out,
                                                              int nh, int nkv, int dk, int dv, int rot_dims,
                                                              const int* __restrict__ positions,
                                                              const int* __restrict__ tok_slot,
                                                              const float* __restrict__ inv_freq, float mag,
                                                              T* __restrict__ kpool, T* __restrict__ vpool, PagedView pv,
                                                              int pool_hdk, int pool_hdv, int interleaved) {
    const long t = blockIdx.x;
    const int y = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const T* row = qkv + t * ld;
    if (y < nh) {
        rotate_run(row + (long)y * dk, q_out + (t * nh + y) * dk, dk, rot_dims, pos, inv_freq, mag, DST_ROWS, 0, lane, 64,
                   interleaved);
        return;
    }
    const long prow = paged_row(pv, tok_slot[t], pos);
    if (y < nh + nkv) {
        const int h = y - nh;
        rotate_run(row + (long)(nh + h) * dk, kpool + key_index(prow, h, nkv, pool_hdk), dk, rot_dims, pos, inv_freq, mag,
                   DST_KEYS, 0, lane, 64, interleaved);
    } else {
        const int h = y - nh - nkv;
        rotate_run(row + (long)(nh + nkv) * dk + (long)h * dv, vpool + value_index(prow, h, nkv, pool_hdv), dv, 0, pos,
                   inv_freq, mag, DST_VALUES, 0, lane, 64);
    }
}

extern "C" const char* cpmcu_qkv_rotate_store(const void* qkv, long ld, int dtype, void* q_out, int n, int nh, int nkv,
                                              int dk, int dv, int rot_dims, const int* positions, const int* tok_slot,
                                              const float* inv_freq, float mag, void* kpool, void* vpool,
                                              const int* page_table, int table_width, int page_size, int pool_hdk,
                                              int pool_hdv, int write_kv, int interleaved, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0, "qkv_rotate_store: empty shape");
    CPMCU_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk && (rot_dims == 0 || inv_freq),
                  "qkv_rotate_store: %d rotated features of %d", rot_dims, dk);
    CPMCU_REQUIRE(ld >= (long)nh * dk + (write_kv ? (long)nkv * (dk + dv) : 0), "qkv_rotate_store: rows of %ld too short", ld);
    CPMCU_REQUIRE(!write_kv || (kpool && vpool && page_table && page_size % 32 == 0 && pool_hdk % 16 == 0 &&
                                pool_hdv % 16 == 0 && pool_hdk >= dk && pool_hdv >= dv),
                  "qkv_rotate_store: the cache takes pages of a multiple of 32 tokens and head sizes in steps of 16");
    const int heads = nh + (write_kv ? 2 * nkv : 0);
    CPMCU_REQUIRE(heads <= 65535, "qkv_rotate_store: %d heads exceed the launch grid", heads);
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, heads);
    if (dtype == CPMCU_F32)
        qkv_rotate_store_kernel<float><<<grid, 64, 0, stream>>>((const float*)qkv, ld, (float*)q_out, nh, nkv, dk, dv, rot_dims,
                                                                positions, tok_slot, inv_freq, mag, (float*)kpool,
                                                                (float*)vpool, pv, pool_hdk, pool_hdv, interleaved);
    else if (dtype == CPMCU_BF16)
        qkv_rotate_store_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)qkv, ld, (bf16_t*)q_out, nh, nkv, dk, dv,
                                                                 rot_dims, positions, tok_slot, inv_freq, mag,
                                                                 (bf16_t*)kpool, (bf16_t*)vpool, pv, pool_hdk, pool_hdv,
                                                                 interleaved);
    else
        CPMCU_FAIL("qkv_rotate_store: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("qkv_rotate_store");
    return nullptr;
}

// The same for designs that put more between projection and rotation, in one launch, grid (tokens, nh + nkv or
// nh + 2 nkv), a wavefront a (token, head), everything in float:
//   * `bias` (float, as wide as the projection's row) is added to the projection;
//   * q heads and k heads are divided by their root mean square (eps inside the root) and multiplied by a weight
//     of dk numbers shared by the heads (q_norm_w, k_norm_w; either may be absent), before the rotation;
//   * with values_from_keys the row holds no v: the value pages receive k as projected (with its bias, before norm
//     and rotation), so dv == dk;
//   * with norm_after q and k heads are rotated first and then divided by their root mean square (times the
//     weight, if one is given);
//   * with interleaved the rotation pairs neighbouring features (2i, 2i + 1) instead of (i, i + rot_dims/2).
// The projection's rows may be float where the cache is bfloat16 (rows that a convolution wrote).
template <typename IT, typename T>
__global__ __launch_bounds__(64) void qkv_norm_rotate_store_kernel(
    const IT* __restrict__ qkv, long ld, const float* __restrict__ bias, T* __restrict__ q_out, int nh, int nkv, int dk,
    int dv, int rot_dims, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    int values_from_keys, const int* __restrict__ positions, const int* __restrict__ tok_slot,
    const float* __restrict__ inv_freq, float mag, T* __restrict__ kpool, T* __restrict__ vpool, PagedView pv,
    int pool_hdk, int pool_hdv, int norm_after, int interleaved) {
    __shared__ float hs[AG_MAX_HD];
    const long t = blockIdx.x;
    const int y = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const bool is_q = y < nh, is_k = !is_q && y < nh + nkv;
    const int h = is_q ? y : (is_k ? y - nh : y - nh - nkv);
    const int width = (is_q || is_k) ? dk : dv;
    const long col = is_q ? (long)h * dk : (is_k ? (long)(nh + h) * dk : (long)(nh + nkv) * dk + (long)h * dv);
    const IT* src = qkv + t * ld + col;
    const long prow = is_q ? 0 : paged_row(pv, tok_slot[t], pos);
    if (!is_q && !is_k) {               // a value head of its own: copied as it is
        T* vd = vpool + value_index(prow, h, nkv, pool_hdv);
        for (int i = lane; i < dv; i += 64) vd[value_d_offset(i)] = from_f32<T>(to_f32(src[i]) + (bias ? bias[col + i] : 0.f));
        return;
    }
    float ss = 0.f;
    for (int i = lane; i < width; i += 64) {
        const float v = to_f32(src[i]) + (bias ? bias[col + i] : 0.f);
        hs[i] = v;
        ss += v * v;
    }
    if (is_k && values_from_keys) {
        T* vd = vpool + value_index(prow, h, nkv, pool_hdv);
        for (int i = lane; i < width; i += 64) vd[value_d_offset(i)] = from_f32<T>(hs[i]);
    }
    const float* nw = is_q ? q_norm_w : k_norm_w;
    if (norm_after) {
        // the rotation first (in place, in float), then the division by the rotated head's root mean square
        __syncthreads();
        const int half = rot_dims / 2;
        for (int i = lane; i < half; i += 64) {
            const float ang = (float)pos * inv_freq[i];
            const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            const float u = hs[ia], v = hs[ib];
            hs[ia] = u * cs - v * sn;
            hs[ib] = v * cs + u * sn;
        }
        __syncthreads();
        float s2 = 0.f;
        for (int i = lane; i < width; i += 64) s2 += hs[i] * hs[i];
        const float r = 1.0f / sqrtf(wave_sum(s2) / (float)width + eps);
        for (int i = lane; i < width; i += 64) hs[i] = hs[i] * r * (nw ? nw[i] : 1.0f);
        rot_dims = 0;
    } else if (nw) {
        const float r = 1.0f / sqrtf(wave_sum(ss) / (float)width + eps);
        for (int i = lane; i < width; i += 64) hs[i] = hs[i] * r * nw[i];
    }
    __syncthreads();
    if (is_q) rotate_run(hs, q_out + (t * nh + h) * dk, dk, rot_dims, pos, inv_freq, mag, DST_ROWS, 0, lane, 64, interleaved);
    else rotate_run(hs, kpool + key_index(prow, h, nkv, pool_hdk), dk, rot_dims, pos, inv_freq, mag, DST_KEYS, 0, lane, 64,
                    interleaved);
}

extern "C" const char* cpmcu_qkv_norm_rotate_store(const void* qkv, long ld, int dtype, const float* bias, void* q_out,
                                                   int n, int nh, int nkv, int dk, int dv, int rot_dims,
                                                   const float* q_norm_w, const float* k_norm_w, float eps,
                                                   int values_from_keys, const int* positions, const int* tok_slot,
                                                   const float* inv_freq, float mag, void* kpool, void* vpool,
                                                   const int* page_table, int table_width, int page_size, int pool_hdk,
                                                   int pool_hdv, int write_kv, int norm_after, int interleaved, int in_dtype,
                                                   hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && dk > 0 && dv > 0, "qkv_norm_rotate_store: empty shape");
    CPMCU_REQUIRE(dk <= AG_MAX_HD && dv <= AG_MAX_HD, "qkv_norm_rotate_store: key size %d / value size %d (up to %d are taken)",
                  dk, dv, AG_MAX_HD);
    CPMCU_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dk && (rot_dims == 0 || inv_freq),
                  "qkv_norm_rotate_store: %d rotated features of %d", rot_dims, dk);
    CPMCU_REQUIRE(!values_from_keys || dv == dk, "qkv_norm_rotate_store: values that are the keys have the keys' size (%d, %d)", dv, dk);
    const long row = (long)nh * dk + (write_kv ? (long)nkv * dk + (values_from_keys ? 0 : (long)nkv * dv) : 0);
    CPMCU_REQUIRE(ld >= row, "qkv_norm_rotate_store: rows of %ld too short", ld);
    CPMCU_REQUIRE(!write_kv || (kpool && vpool && page_table && page_size % 32 == 0 && pool_hdk % 16 == 0 &&
                                pool_hdv % 16 == 0 && pool_hdk >= dk && pool_hdv >= dv),
                  "qkv_norm_rotate_store: the cache takes pages of a multiple of 32 tokens and head sizes in steps of 16");
    const int heads = nh + (write_kv ? (values_from_keys ? nkv : 2 * nkv) : 0);
    CPMCU_REQUIRE(heads <= 65535, "qkv_norm_rotate_store: %d heads exceed the launch grid", heads);
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, heads);
#define LAUNCH(ITv, Tv)                                                                                              \
    qkv_norm_rotate_store_kernel<ITv, Tv><<<grid, 64, 0, stream>>>(                                                  \
        (const ITv*)qkv, ld, bias, (Tv*)q_out, nh, nkv, dk, dv, rot_dims, q_norm_w, k_norm_w, eps, values_from_keys, \
        positions, tok_slot, inv_freq, mag, (Tv*)kpool, (Tv*)vpool, pv, pool_hdk, pool_hdv, norm_after, interleaved)
    // dtype: the cache's and q_out's element type; in_dtype: the projection rows' (float rows may feed a bfloat16 cache)
    if (dtype == CPMCU_F32 && in_dtype == CPMCU_F32) LAUNCH(float, float);
    else if (dtype == CPMCU_BF16 && in_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else if (dtype == CPMCU_BF16 && in_dtype == CPMCU_F32) LAUNCH(float, bf16_t);
    else CPMCU_FAIL("qkv_norm_rotate_store: unsupported dtypes in=%d out=%d", in_dtype, dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("qkv_norm_rotate_store");
    return nullptr;
}

// Latent attention: from a row [q heads: nh * (dim + rot) | down: rank + rot | ...] in one launch
//   * y < nh: head y's rotated query part goes, rotated, behind the `rank` latent features of its query row
//     q_out[t, y, rank:rank + rot] (the latent features themselves come from a product over heads);
//   * y == nh (layers that own the cache): the latent c = rmsnorm(down[:rank]) * norm_w in float, into the key
//     pages (features 0..rank) and the value pages, and the shared key part down[rank:], rotated, into the key
//     pages behind it.
template <typename T>
__global__ __launch_bounds__(256) void latent_store_kernel(const T* __restrict__ proj, long ld, T* __restrict__ q_out,
                                                           int nh, int dim, int rot, int rank,
                                                           const float* __restrict__ norm_w, float eps,
                                                           const int* __restrict__ positions,
                                                           const int* __restrict__ tok_slot,
                                                           const float* __restrict__ inv_freq, float mag,
                                                           T* __restrict__ kpool, T* __restrict__ vpool, PagedView pv,
                                                           int pool_hdk, int pool_hdv) {
    __shared__ float red[17];
    const long t = blockIdx.x;
    const int y = blockIdx.y;
    const int pos = positions[t];
    const int qw = dim + rot, dk = rank + rot;
    if (y < nh) {
        rotate_run(proj + t * ld + (long)y * qw + dim, q_out + (t * nh + y) * dk + rank, rot, rot, pos, inv_freq, mag,
                   DST_ROWS, 0, (int)threadIdx.x, (int)blockDim.x);
        return;
    }
    const T* down = proj + t * ld + (long)nh * qw;
    float ss = 0.f;
    for (int c = threadIdx.x; c < rank; c += blockDim.x) {
        const float v = to_f32(down[c]);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)rank + eps);
    const long prow = paged_row(pv, tok_slot[t], pos);
    T* kd = kpool + key_index(prow, 0, 1, pool_hdk);
    T* vd = vpool + value_index(prow, 0, 1, pool_hdv);
    for (int c = threadIdx.x; c < rank; c += blockDim.x) {
        const T v = from_f32<T>(to_f32(down[c]) * rs * norm_w[c]);
        kd[key_d_offset(c)] = v;
        vd[value_d_offset(c)] = v;
    }
    rotate_run(down + rank, kd, rot, rot, pos, inv_freq, mag, DST_KEYS, rank, (int)threadIdx.x, (int)blockDim.x);
}

extern "C" const char* cpmcu_latent_store(const void* proj, long ld, int dtype, void* q_out, int n, int nh, int dim,
                                          int rot, int rank, const float* norm_w, float eps, const int* positions,
                                          const int* tok_slot, const float* inv_freq, float mag, void* kpool,
                                          void* vpool, const int* page_table, int table_width, int page_size,
                                          int pool_hdk, int pool_hdv, int write_cache, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && dim > 0 && rank > 0 && rot >= 0 && rot % 2 == 0, "latent_store: bad shape");
    CPMCU_REQUIRE(rot == 0 || inv_freq, "latent_store: frequencies missing");
    CPMCU_REQUIRE(ld >= (long)nh * (dim + rot) + (write_cache ? rank + rot : 0), "latent_store: rows of %ld too short", ld);
    CPMCU_REQUIRE(!write_cache || (norm_w && kpool && vpool && page_table && page_size % 32 == 0 && pool_hdk % 16 == 0 &&
                                   pool_hdv % 16 == 0 && pool_hdk >= rank + rot && pool_hdv >= rank),
                  "latent_store: the cache takes pages of a multiple of 32 tokens and head sizes in steps of 16");
    CPMCU_REQUIRE(nh < 65535, "latent_store: %d heads exceed the launch grid", nh);
    if (!write_cache && rot == 0) return nullptr;
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, nh + (write_cache ? 1 : 0));
    const int block = rank >= 256 ? 256 : 64;
    if (dtype == CPMCU_F32)
        latent_store_kernel<float><<<grid, block, 0, stream>>>((const float*)proj, ld, (float*)q_out, nh, dim, rot, rank,
                                                               norm_w, eps, positions, tok_slot, inv_freq, mag,
                                                               (float*)kpool, (float*)vpool, pv, pool_hdk, pool_hdv);
    else if (dtype == CPMCU_BF16)
        latent_store_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)proj, ld, (bf16_t*)q_out, nh, dim, rot, rank,
                                                                norm_w, eps, positions, tok_slot, inv_freq, mag,
                                                                (bf16_t*)kpool, (bf16_t*)vpool, pv, pool_hdk, pool_hdv);
    else
        CPMCU_FAIL("latent_store: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("latent_store");
    return nullptr;
}
