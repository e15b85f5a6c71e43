// Rotation first, unit norm second, cache write, and values blended with another layer's: one wave per
// (token, head) over the packed rows [q | k | v] of a step.
//   q heads   the first `rot_dim` channels are rotated by the row's position, then the whole head is divided
//             by its root mean square (x / sqrt(mean(x^2) + eps), with `unit_norm`; times `q_weight` / `k_weight`
//             where given); written back in place
//   k heads   the same, written to the key page   K[page][kv_head][slot][D]
//   v heads   Dv channels; with `mix_rows`: v <- (1 - m) v + m mix_rows[token][head], m = *mix_weight (a number
//             on the device); written to the value page (transposed)   V[page][kv_head][Dv][slot]
// Rotation pairs: (p, p + rot_dim / 2), or (2p, 2p + 1) with `interleaved`; table[pos] = [cos | sin], rot_dim
// floats. Rows of padding (token_seq < 0) and pages that were given back (< 0) are skipped. Any sizes up to 512.
#include "dispatch.h"

#define QR_MAX_D 512

template <typename T>
__global__ void __launch_bounds__(256)
qkv_rotate_norm_store_kernel(T* __restrict__ qkv, long row_stride, int q_off, int k_off, int v_off,
                             const int* __restrict__ positions, const int* __restrict__ token_seq,
                             const int* __restrict__ block_table, int bt_width, int page_size, T* __restrict__ k_pages,
                             T* __restrict__ v_pages, int H, int Hkv, int D, int Dv, WeightPtr qw, WeightPtr kw, int has_weight,
                             int unit_norm, float eps, const float* __restrict__ table, int rot_dim, int interleaved,
                             const T* __restrict__ mix_rows, long mix_stride, WeightPtr mix_weight) {
    __shared__ float sh[4][QR_MAX_D];
    const int tok = blockIdx.x;
    const int wave = threadIdx.x / MV_WAVE, lane = threadIdx.x % MV_WAVE;
    const int head = blockIdx.y * 4 + wave;
    if (head >= H + 2 * Hkv) return;
    const int seq = token_seq[tok];
    if (seq < 0) return;
    const int pos = positions[tok];
    T* row = qkv + (size_t)tok * row_stride;
    float* x = sh[wave];
    if (head >= H + Hkv) {                       // a value head
        const int hh = head - H - Hkv;
        const int page = block_table[(size_t)seq * bt_width + pos / page_size];
        if (page < 0) return;
        const T* src = row + v_off + (size_t)hh * Dv;
        T* dst = v_pages + ((size_t)page * Hkv + hh) * Dv * page_size + pos % page_size;
        float m = 0.f;
        const T* other = nullptr;
        if (mix_rows != nullptr) {
            m = mix_weight.at(0);
            other = mix_rows + (size_t)tok * mix_stride + (size_t)hh * Dv;
        }
        for (int d = lane; d < Dv; d += MV_WAVE) {
            float v = to_f(src[d]);
            if (other != nullptr) v = (1.f - m) * v + m * to_f(other[d]);
            dst[(size_t)d * page_size] = from_f<T>(v);
        }
        return;
    }
    const bool is_k = head >= H;
    const int hh = is_k ? head - H : head;
    T* src = row + (is_k ? k_off : q_off) + (size_t)hh * D;
    for (int d = lane; d < D; d += MV_WAVE) x[d] = to_f(src[d]);
    // (a wave's own LDS writes are visible to it in order: no barrier between the phases)
    __builtin_amdgcn_wave_barrier();
    float ss = 0.f;
    if (table != nullptr) {
        const int half = rot_dim / 2;
        const float* cs = table + (size_t)pos * rot_dim;
        for (int p = lane; p < half; p += MV_WAVE) {
            const int i1 = interleaved ? 2 * p : p;
            const int i2 = interleaved ? 2 * p + 1 : p + half;
            const float c = cs[p], s = cs[half + p];
            const float a = x[i1], b = x[i2];
            x[i1] = a * c - b * s;
            x[i2] = b * c + a * s;
        }
        __builtin_amdgcn_wave_barrier();
    }
    for (int d = lane; d < D; d += MV_WAVE) ss = fmaf(x[d], x[d], ss);
    ss = wave_sum(ss);
    const float inv = unit_norm ? 1.f / sqrtf(ss / (float)D + eps) : 1.f;
    const WeightPtr& w = is_k ? kw : qw;
    if (!is_k) {
        for (int d = lane; d < D; d += MV_WAVE) src[d] = from_f<T>(x[d] * inv * (has_weight ? w.at(d) : 1.f));
        return;
    }
    const int page = block_table[(size_t)seq * bt_width + pos / page_size];
    if (page < 0) return;
    T* dst = k_pages + (((size_t)page * Hkv + hh) * page_size + pos % page_size) * D;
    for (int d = lane; d < D; d += MV_WAVE) dst[d] = from_f<T>(x[d] * inv * (has_weight ? w.at(d) : 1.f));
}

// The same for heads of 64, 128 or 256 channels that are rotated over all of them in half-split pairs (or not at all),
// with values as large as keys and everything 16-byte aligned: a head is spread over L = D / 8 neighbouring lanes,
// eight channels each, read and written 16 bytes at a time; rotation partners and the sum of squares travel by lane
// shuffles. `store_v` 0: the blended values are written back into the rows and a tiled launch takes them to their
// pages (steps of many tokens, where a store per token and head would scatter two bytes at a time); 1: they go to
// their page from here.
template <typename T, int L>
__global__ void __launch_bounds__(256)
qkv_rotate_norm_store_vec_kernel(T* __restrict__ qkv, long row_stride, int q_off, int k_off, int v_off,
                                 const int* __restrict__ positions, const int* __restrict__ token_seq,
                                 const int* __restrict__ block_table, int bt_width, int page_size, T* __restrict__ k_pages,
                                 T* __restrict__ v_pages, int n, int H, int Hkv, WeightPtr qw, WeightPtr kw, int has_weight,
                                 int unit_norm, float eps, const float* __restrict__ table, const T* __restrict__ mix_rows,
                                 long mix_stride, WeightPtr mix_weight, int store_v) {
    constexpr int D = 8 * L;
    const int heads = H + 2 * Hkv;
    const long gid = (long)blockIdx.x * 256 + threadIdx.x;
    const long hidx = gid / L;
    const int j = (int)(gid % L);
    const int tok = (int)(hidx / heads), head = (int)(hidx % heads);
    const int seq = tok < n ? token_seq[tok] : -1;
    const bool active = tok < n && seq >= 0;          // (inactive lanes still take part in the shuffles)
    const int pos = active ? positions[tok] : 0;
    const int kind = head >= H + Hkv ? 2 : (head >= H ? 1 : 0);
    const int hh = kind == 2 ? head - H - Hkv : (kind == 1 ? head - H : head);
    T* src = qkv + (size_t)(active ? tok : 0) * row_stride + (kind == 0 ? q_off : (kind == 1 ? k_off : v_off)) + (size_t)hh * D + 8 * j;
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (active) Vec8<T>::load(src, x);
    if (kind == 2) {
        if (!active) return;
        if (mix_rows != nullptr) {
            const float m = mix_weight.at(0);
            float o[8];
            Vec8<T>::load(mix_rows + (size_t)tok * mix_stride + (size_t)hh * D + 8 * j, o);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (1.f - m) * x[e] + m * o[e];
            if (!store_v) Vec8<T>::store(src, x);
        }
        if (!store_v) return;
        const int page = block_table[(size_t)seq * bt_width + pos / page_size];
        if (page < 0) return;
        T* dst = v_pages + (((size_t)page * Hkv + hh) * D + 8 * j) * page_size + pos % page_size;
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[(size_t)e * page_size] = from_f<T>(x[e]);
        return;
    }
    if (table != nullptr) {
        const float* cs = table + (size_t)pos * D + 8 * (j % (L / 2));
        float c[8], sn[8];
        Vec8<float>::load(cs, c);
        Vec8<float>::load(cs + D / 2, sn);
        const bool low = j < L / 2;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float other = __shfl_xor(x[e], L / 2, MV_WAVE);
            x[e] = low ? x[e] * c[e] - other * sn[e] : x[e] * c[e] + other * sn[e];
        }
    }
    float inv = 1.f;
    if (unit_norm) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss = fmaf(x[e], x[e], ss);
#pragma unroll
        for (int o = L / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, MV_WAVE);
        inv = 1.f / sqrtf(ss / (float)D + eps);
    }
    if (!active) return;
    if (has_weight) {
        float w[8];
        (kind == 0 ? qw : kw).at8(8 * j, w);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] *= w[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] *= inv;
    if (kind == 0) {
        Vec8<T>::store(src, x);
        return;
    }
    const int page = block_table[(size_t)seq * bt_width + pos / page_size];
    if (page < 0) return;
    Vec8<T>::store(k_pages + (((size_t)page * Hkv + hh) * page_size + pos % page_size) * D + 8 * j, x);
}

extern "C" int mv_store_v_pages(const void* qkv, long row_stride, int v_off, const int* positions, const int* token_seq,
                                const int* block_table, int bt_width, int page_size, void* v_pages, int n, int Hkv, int D,
                                int dtype, hipStream_t stream);

// steps of at least this many tokens write their values tile by tile in a launch of their own
#define QR_TILED_V_TOKENS 64

extern "C" int mv_qkv_rotate_norm_store(void* qkv, long row_stride, int q_off, int k_off, int v_off, const int* positions,
                                        const int* token_seq, const int* block_table, int bt_width, int page_size,
                                        void* k_pages, void* v_pages, int n, int H, int Hkv, int D, int Dv,
                                        const void* q_weight, const void* k_weight, int weight_dtype, int unit_norm, float eps,
                                        const float* table, int rot_dim, int interleaved, const void* mix_rows,
                                        long mix_stride, const void* mix_weight, int mix_weight_dtype, int dtype,
                                        hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && Hkv > 0 && D > 0 && Dv > 0 && D <= QR_MAX_D && Dv <= QR_MAX_D,
               "qkv_rotate_norm_store: bad sizes n=%d H=%d Hkv=%d D=%d Dv=%d (heads of at most %d)", n, H, Hkv, D, Dv, QR_MAX_D);
    MV_REQUIRE(table == nullptr || (rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= D),
               "qkv_rotate_norm_store: rotary dim %d must be even and at most head_dim %d", rot_dim, D);
    MV_REQUIRE(qkv && positions && token_seq && block_table && k_pages && v_pages && page_size > 0 && bt_width > 0,
               "qkv_rotate_norm_store: missing operand");
    MV_REQUIRE((q_weight == nullptr) == (k_weight == nullptr) && mv_valid_dtype(weight_dtype) && (!unit_norm || eps > 0.f),
               "qkv_rotate_norm_store: norm weights come in pairs, and eps must be positive");
    MV_REQUIRE(!mix_rows || (mix_weight && mix_stride >= (long)Hkv * Dv && mv_valid_dtype(mix_weight_dtype)),
               "qkv_rotate_norm_store: blending the values needs the other rows and the weight");
    MV_REQUIRE(H + 2 * Hkv <= 4 * 65535, "qkv_rotate_norm_store: too many heads");
    if (n == 0) return 0;
    WeightPtr qw{q_weight, weight_dtype}, kw{k_weight, weight_dtype}, mw{mix_weight, mix_weight_dtype};
    const size_t esz = mv_dtype_size(dtype);
    const bool aligned = ((uintptr_t)qkv % 16) == 0 && (row_stride * esz) % 16 == 0 && (q_off * esz) % 16 == 0 &&
                         (k_off * esz) % 16 == 0 && (v_off * esz) % 16 == 0 && ((uintptr_t)k_pages % 16) == 0 &&
                         ((uintptr_t)q_weight % 16) == 0 && ((uintptr_t)k_weight % 16) == 0 && ((uintptr_t)table % 16) == 0 &&
                         ((uintptr_t)mix_rows % 16) == 0 && (mix_stride * esz) % 16 == 0;
    if (aligned && D == Dv && (D == 64 || D == 128 || D == 256) && (table == nullptr || (rot_dim == D && !interleaved)) &&
        (long)n * (H + 2 * Hkv) * (D / 8) < (1L << 31)) {
        const int store_v = n < QR_TILED_V_TOKENS;
        const long lanes = (long)n * (H + 2 * Hkv) * (D / 8);
        const dim3 vgrid((unsigned)((lanes + 255) / 256));
#define QR_VEC(LL)                                                                                                          \
    MV_DISPATCH_T(dtype, "qkv_rotate_norm_store",                                                                           \
                  hipLaunchKernelGGL((qkv_rotate_norm_store_vec_kernel<T, LL>), vgrid, dim3(256), 0, stream, (T*)qkv,       \
                                     row_stride, q_off, k_off, v_off, positions, token_seq, block_table, bt_width, page_size, \
                                     (T*)k_pages, (T*)v_pages, n, H, Hkv, qw, kw, q_weight != nullptr, unit_norm, eps, table, \
                                     (const T*)mix_rows, mix_stride, mw, store_v))
        if (D == 64) { QR_VEC(8); } else if (D == 128) { QR_VEC(16); } else { QR_VEC(32); }
#undef QR_VEC
        if (int rc = mv_check_launch("qkv_rotate_norm_store")) return rc;
        if (!store_v)
            return mv_store_v_pages(qkv, row_stride, v_off, positions, token_seq, block_table, bt_width, page_size, v_pages, n,
                                    Hkv, Dv, dtype, stream);
        return 0;
    }
    dim3 grid(n, (H + 2 * Hkv + 3) / 4);
    MV_DISPATCH_T(dtype, "qkv_rotate_norm_store",
                  hipLaunchKernelGGL(qkv_rotate_norm_store_kernel<T>, grid, dim3(256), 0, stream, (T*)qkv, row_stride, q_off,
                                     k_off, v_off, positions, token_seq, block_table, bt_width, page_size, (T*)k_pages,
                                     (T*)v_pages, H, Hkv, D, Dv, qw, kw, q_weight != nullptr, unit_norm, eps, table, rot_dim,
                                     interleaved, (const T*)mix_rows, mix_stride, mw));
    return mv_check_launch("qkv_rotate_norm_store");
}
