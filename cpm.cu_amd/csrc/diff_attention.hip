// Differential attention: every head holds two score maps over the same values, and its output is the
// difference of the two attentions, o = a1 - lambda a2, divided by its root mean square and multiplied by a
// constant.  The attention itself is the library's general kernel run over 2 H query heads and 2 G key heads, with
// every two neighbouring key heads reading one value head (v_share = 2).  The two kernels here stand before and
// after it:
//
//  * diff_qkv_store_kernel: a row [q: H*2*dk | k: G*2*dk | v: G*dv] (float or the engine's type; after a
//    convolution, if the design has one), q and k laid out head by head as [map 1 | map 2].  q is multiplied by the
//    position's temperature 1 + coef ln(floor((p + 1) / every) + 1) and written as 2 H heads in the order
//    (kv head, map, head of the group), so that query head (g, m, j) reads key head 2 g + m by the ordinary
//    grouping; k goes into the key pages as 2 G heads, v into the value pages as G heads.
//  * diff_combine_kernel: from the attention's output in that order, per (token, head):
//    o = a1 - lambda a2; o / sqrt(mean(o^2) + eps) * post, written head by head in the design's order.
#include "common.h"

template <typename IT, typename T>
__global__ __launch_bounds__(64) void diff_qkv_store_kernel(const IT* __restrict__ src, long ld, T* __restrict__ q_out,
                                                            int H, int G, int dk, int dv, float temp_coef,
                                                            int temp_every, const int* __restrict__ positions,
                                                            const int* __restrict__ tok_slot, T* __restrict__ kpool,
                                                            T* __restrict__ vpool, PagedView pv, int pool_hdk,
                                                            int pool_hdv) {
    const long t = blockIdx.x;
    const int y = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const IT* row = src + t * ld;
    if (y < 2 * H) {
        const int h = y >> 1, m = y & 1, rep = H / G;
        const int dst_head = ((h / rep) * 2 + m) * rep + h % rep;
        const float temp = temp_every > 0 ? 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f) : 1.0f;
        const IT* s = row + (long)y * dk;
        T* d = q_out + (t * 2 * H + dst_head) * dk;
        for (int i = lane; i < dk; i += 64) d[i] = from_f32<T>(to_f32(s[i]) * temp);
        return;
    }
    const long prow = paged_row(pv, tok_slot[t], pos);
    if (y < 2 * H + 2 * G) {
        const int kh = y - 2 * H;
        const IT* s = row + (long)(2 * H + kh) * dk;
        T* d = kpool + key_index(prow, kh, 2 * G, pool_hdk);
        for (int i = lane; i < dk; i += 64) d[key_d_offset(i)] = from_f32<T>(to_f32(s[i]));
    } else {
        const int vh = y - 2 * H - 2 * G;
        const IT* s = row + (long)(2 * H + 2 * G) * dk + (long)vh * dv;
        T* d = vpool + value_index(prow, vh, G, pool_hdv);
        for (int i = lane; i < dv; i += 64) d[value_d_offset(i)] = from_f32<T>(to_f32(s[i]));
    }
}

extern "C" const char* cpmcu_diff_qkv_store(const void* src, long ld, int src_dtype, void* q_out, int dtype, int n,
                                            int H, int G, int dk, int dv, float temp_coef, int temp_every,
                                            const int* positions, const int* tok_slot, void* kpool, void* vpool,
                                            const int* page_table, int table_width, int page_size, int pool_hdk,
                                            int pool_hdv, int write_kv, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && G > 0 && dk > 0 && dv > 0 && H % G == 0, "diff_qkv_store: bad shape heads=%d kv_heads=%d", H, G);
    CPMCU_REQUIRE(ld >= 2L * H * dk + (write_kv ? 2L * G * dk + (long)G * dv : 0), "diff_qkv_store: rows of %ld too short", ld);
    CPMCU_REQUIRE(!write_kv || (kpool && vpool && page_table && page_size % 32 == 0 && pool_hdk % 16 == 0 &&
                                pool_hdv % 16 == 0 && pool_hdk >= dk && pool_hdv >= dv),
                  "diff_qkv_store: the cache takes pages of a multiple of 32 tokens and head sizes in steps of 16");
    CPMCU_REQUIRE(temp_every >= 0, "diff_qkv_store: a temperature step of %d positions", temp_every);
    const int heads = 2 * H + (write_kv ? 3 * G : 0);
    CPMCU_REQUIRE(heads <= 65535, "diff_qkv_store: %d heads exceed the launch grid", heads);
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, heads);
#define LAUNCH(IT, T)                                                                                              \
    diff_qkv_store_kernel<IT, T><<<grid, 64, 0, stream>>>((const IT*)src, ld, (T*)q_out, H, G, dk, dv, temp_coef, \
                                                          temp_every, positions, tok_slot, (T*)kpool, (T*)vpool,  \
                                                          pv, pool_hdk, pool_hdv)
    if (src_dtype == CPMCU_F32 && dtype == CPMCU_F32) LAUNCH(float, float);
    else if (src_dtype == CPMCU_F32 && dtype == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (src_dtype == CPMCU_BF16 && dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else CPMCU_FAIL("diff_qkv_store: unsupported dtypes in=%d out=%d", src_dtype, dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("diff_qkv_store");
    return nullptr;
}

// grid (tokens, H), a wavefront a (token, head); a [n, 2H, dv] in the order (kv head, map, head of the group)
template <typename AT, typename T>
__global__ __launch_bounds__(64) void diff_combine_kernel(const AT* __restrict__ a, T* __restrict__ out, int H, int G,
                                                          int dv, float lambda, float eps, float post) {
    const long t = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const int rep = H / G, g = h / rep, j = h % rep;
    const AT* a1 = a + (t * 2 * H + (long)(2 * g) * rep + j) * dv;
    const AT* a2 = a1 + (long)rep * dv;
    float ss = 0.f;
    for (int i = lane; i < dv; i += 64) {
        const float o = to_f32(a1[i]) - lambda * to_f32(a2[i]);
        ss += o * o;
    }
    const float r = post / sqrtf(wave_sum(ss) / (float)dv + eps);
    T* d = out + (t * H + h) * dv;
    for (int i = lane; i < dv; i += 64) d[i] = from_f32<T>((to_f32(a1[i]) - lambda * to_f32(a2[i])) * r);
}

extern "C" const char* cpmcu_diff_combine(const void* a, int a_dtype, void* out, int dtype, int n, int H, int G, int dv,
                                          float lambda, float eps, float post, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && G > 0 && dv > 0 && H % G == 0 && H <= 65535, "diff_combine: bad shape heads=%d kv_heads=%d", H, G);
    dim3 grid(n, H);
    if (a_dtype == CPMCU_F32 && dtype == CPMCU_F32)
        diff_combine_kernel<float, float><<<grid, 64, 0, stream>>>((const float*)a, (float*)out, H, G, dv, lambda, eps, post);
    else if (a_dtype == CPMCU_F32 && dtype == CPMCU_BF16)
        diff_combine_kernel<float, bf16_t><<<grid, 64, 0, stream>>>((const float*)a, (bf16_t*)out, H, G, dv, lambda, eps, post);
    else if (a_dtype == CPMCU_BF16 && dtype == CPMCU_BF16)
        diff_combine_kernel<bf16_t, bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)a, (bf16_t*)out, H, G, dv, lambda, eps, post);
    else
        CPMCU_FAIL("diff_combine: unsupported dtypes maps=%d out=%d", a_dtype, dtype);
    CPMCU_LAUNCH_CHECK("diff_combine");
    return nullptr;
}
