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
//    floor(j / chunk) == floor(p / chunk), chunks counted from position 0 of the sequence.  Float scores and
//    softmax, both element types; one wavefront a (token, head).
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

template <typename T>
__global__ __launch_bounds__(64) void attention_general_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ kpool, const T* __restrict__ vpool,
    PagedView pv, const int* __restrict__ positions, const int* __restrict__ tok_slot, int nh, int nkv, int hdk,
    int hdv, int pool_hdk, int pool_hdv, float scale, int chunk) {
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
    const int s0 = chunk > 0 ? pos - pos % chunk : 0, s1 = pos + 1;
    for (int j0 = s0; j0 < s1; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = j < s1;
        int row = 0;
        float s = -INFINITY;
        if (valid) {
            row = (int)paged_row(pv, slot, j);
            const T* kr = kpool + key_index(row, g, nkv, pool_hdk);
            float dot = 0.f;
            for (int d = 0; d < hdk; ++d) dot += qs[d] * to_f32(kr[key_d_offset(d)]);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);
        l = l * corr + wave_sum(p);
        m = m_new;
        const int cnt = min(64, s1 - j0);
#pragma unroll
        for (int i = 0; i < AG_MAX_HD / 64; ++i) acc[i] *= corr;
        for (int jj = 0; jj < cnt; ++jj) {
            const float pj = __shfl(p, jj, 64);
            const int rj = __shfl(row, jj, 64);
            const T* vr = vpool + value_index(rj, g, nkv, pool_hdv);
#pragma unroll
            for (int i = 0; i < AG_MAX_HD / 64; ++i) {
                const int d = lane + 64 * i;
                if (i < nd && d < hdv) acc[i] += pj * to_f32(vr[value_d_offset(d)]);
            }
        }
    }
    T* orow = out + ((long)t * nh + h) * hdv;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < AG_MAX_HD / 64; ++i) {
        const int d = lane + 64 * i;
        if (i < nd && d < hdv) orow[d] = from_f32<T>(acc[i] * inv);
    }
}

extern "C" const char* cpmcu_attention_general(const void* q, void* out, int dtype, int n, int nh, int nkv, int hdk,
                                               int hdv, int pool_hdk, int pool_hdv, float scale, int chunk, const void* kpool,
                                               const void* vpool,
                                               const int* page_table, int table_width, int page_size,
                                               const int* positions, const int* tok_slot, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && hdk > 0 && hdv > 0,
                  "attention_general: empty shape n=%d heads=%d kv_heads=%d key size=%d value size=%d", n, nh, nkv, hdk, hdv);
    CPMCU_REQUIRE(nh % nkv == 0, "attention_general: %d heads are not a multiple of %d kv heads", nh, nkv);
    CPMCU_REQUIRE(hdk <= AG_MAX_HD && hdv <= AG_MAX_HD, "attention_general: key size %d / value size %d (up to %d are taken)",
                  hdk, hdv, AG_MAX_HD);
    CPMCU_REQUIRE(pool_hdk >= hdk && pool_hdv >= hdv && pool_hdk % 16 == 0 && pool_hdv % 16 == 0 && page_size % 32 == 0,
                  "attention_general: the cache holds heads in steps of 16 features and pages of a multiple of 32 tokens "
                  "(cached key size %d, value size %d, page %d)", pool_hdk, pool_hdv, page_size);
    CPMCU_REQUIRE(nh <= 65535, "attention_general: %d heads exceed the launch grid", nh);
    CPMCU_REQUIRE(chunk >= 0, "attention_general: mask chunk %d", chunk);
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, nh);
    if (dtype == CPMCU_F32)
        attention_general_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, (float*)out, (const float*)kpool,
                                                                 (const float*)vpool, pv, positions, tok_slot, nh, nkv,
                                                                 hdk, hdv, pool_hdk, pool_hdv, scale, chunk);
    else if (dtype == CPMCU_BF16)
        attention_general_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kpool,
                                                                  (const bf16_t*)vpool, pv, positions, tok_slot, nh,
                                                                  nkv, hdk, hdv, pool_hdk, pool_hdv, scale, chunk);
    else
        CPMCU_FAIL("attention_general: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("attention_general");
    return nullptr;
}
