// RMS normalisation in groups: a row of h columns is cut into `groups` equal runs of neighbouring
// columns, each run is divided by sqrt(mean of its squares + eps), and the whole row is multiplied by
// a weight of h numbers. groups == 1 is the plain RMS norm.
//
//   group_norm_rows      v = (resid[r] | x[r]) (+ delta[r]);  out[i] = gnorm(v) * w
//                        (with a float residual, a delta and no row list the sum goes back to resid)
//   group_norm_add_norm  v = resid[r] + gnorm(y[r]) * wa;  resid[r] = v;  out[r] = gnorm(v) * wb
//                        (the norm behind a sublayer, the residual add and the norm in front of the
//                        next one; the sum stays float from the first norm to the second)
//
// One workgroup per row; the row lives in LDS as float between the passes, so memory is read once.
// Sums of squares are taken by whole waves over fixed slices of a group and added in a fixed order:
// a row's result never depends on the other rows of the launch. All arithmetic is float.
#include "dispatch.h"

#define GN_THREADS 256
#define GN_WAVES (GN_THREADS / MV_WAVE)
#define GN_MAX_GROUPS 256
#define GN_MAX_UNITS (GN_MAX_GROUPS * GN_WAVES)
#define GN_MAX_ROW_BYTES (56 * 1024)      // the row in LDS beside the sums: 64 KB a workgroup without asking for more

// 1 / sqrt(mean square + eps) of every group of the row `v` (LDS, h floats) into rinv[groups].
// A group is cut into `parts` slices (as many as there are waves to a group, at least one); a wave
// sums a slice, thread g adds its group's slices in order.
__device__ __forceinline__ void gn_group_scales(const float* v, int h, int groups, float eps, float* part_sum, float* rinv) {
    const int wave = threadIdx.x / MV_WAVE, lane = threadIdx.x % MV_WAVE;
    const int gw = h / groups;
    const int parts = groups >= GN_WAVES ? 1 : GN_WAVES / groups;
    const int units = groups * parts;
    const int slice = (gw + parts - 1) / parts;
    for (int u = wave; u < units; u += GN_WAVES) {
        const int g = u / parts, p = u % parts;
        const int c0 = g * gw + p * slice;
        int c1 = c0 + slice;
        if (c1 > (g + 1) * gw) c1 = (g + 1) * gw;
        float s = 0.f;
        for (int c = c0 + lane; c < c1; c += MV_WAVE) s = fmaf(v[c], v[c], s);
        s = wave_sum(s);
        if (lane == 0) part_sum[u] = s;
    }
    __syncthreads();
    for (int g = threadIdx.x; g < groups; g += GN_THREADS) {
        float s = 0.f;
        for (int p = 0; p < parts; ++p) s += part_sum[g * parts + p];
        rinv[g] = 1.f / sqrtf(s / (float)gw + eps);
    }
    __syncthreads();
}

template <typename T>
__global__ void __launch_bounds__(GN_THREADS)
group_norm_rows_kernel(float* __restrict__ resid, const T* __restrict__ x, long ldx, const T* __restrict__ delta, WeightPtr w,
                       float eps, int groups, T* __restrict__ out, long ldo, const int* __restrict__ rows, int h) {
    extern __shared__ float gn_row[];
    __shared__ float part_sum[GN_MAX_UNITS];
    __shared__ float rinv[GN_MAX_GROUPS];
    const int i = blockIdx.x;
    const int r = rows ? rows[i] : i;
    T* o = out + (size_t)i * ldo;
    if (r < 0) {
        for (int c = threadIdx.x; c < h; c += GN_THREADS) o[c] = from_f<T>(0.f);
        return;
    }
    for (int c = threadIdx.x; c < h; c += GN_THREADS) {
        float v = resid ? resid[(size_t)r * h + c] : to_f(x[(size_t)r * ldx + c]);
        if (delta) {
            v += to_f(delta[(size_t)r * h + c]);
            if (resid && !rows) resid[(size_t)r * h + c] = v;
        }
        gn_row[c] = v;
    }
    __syncthreads();
    gn_group_scales(gn_row, h, groups, eps, part_sum, rinv);
    const int gw = h / groups;
    for (int c = threadIdx.x; c < h; c += GN_THREADS) o[c] = from_f<T>(gn_row[c] * rinv[c / gw] * w.at(c));
}

// out == null: the add alone happens in the caller's kernels; here an output is always written.
extern "C" int mv_group_norm_rows(float* resid, const void* x, long ldx, const void* delta, const void* weight, int weight_dtype,
                                  float eps, int groups, void* out, long ldo, const int* rows, int n_out, int h, int dtype,
                                  hipStream_t stream) {
    MV_REQUIRE(n_out >= 0 && h > 0 && groups >= 1 && groups <= GN_MAX_GROUPS && h % groups == 0,
               "group_norm: rows of %d columns do not form %d equal groups (at most %d)", h, groups, GN_MAX_GROUPS);
    MV_REQUIRE((resid != nullptr) != (x != nullptr), "group_norm: either a float residual or activation rows are normalised");
    MV_REQUIRE(weight && out && mv_valid_dtype(weight_dtype) && eps > 0.f && ldo >= h && (x == nullptr || ldx >= h),
               "group_norm: missing operand or short rows");
    MV_REQUIRE((size_t)h * sizeof(float) <= GN_MAX_ROW_BYTES, "group_norm: rows of %d columns exceed the %d that fit LDS", h, (int)(GN_MAX_ROW_BYTES / 4));
    if (n_out == 0) return 0;
    WeightPtr w{weight, weight_dtype};
    MV_DISPATCH_T(dtype, "group_norm",
                  hipLaunchKernelGGL(group_norm_rows_kernel<T>, dim3(n_out), dim3(GN_THREADS), (size_t)h * sizeof(float), stream,
                                     resid, (const T*)x, ldx, (const T*)delta, w, eps, groups, (T*)out, ldo, rows, h));
    return mv_check_launch("group_norm");
}

// With `conv_taps` > 0 (steps in which every request brings one token): what goes to `out` is
// g + sum_j conv_w[c][j] * g_(t - taps + 1 + j), g being the row after the second norm as it is stored
// (rounded to T) and the rows in front of it the request's `conv_state` [slot][taps - 1][h], which then
// moves on by one row. Row r belongs to request token_seq[r]; a padding row gives zeros and touches nothing.
template <typename T>
__global__ void __launch_bounds__(GN_THREADS)
group_norm_add_norm_kernel(const T* __restrict__ y, long ldy, WeightPtr wa, float eps_a, float* __restrict__ resid, WeightPtr wb,
                           float eps_b, int groups, T* __restrict__ out, int h, int conv_taps, WeightPtr conv_w,
                           T* __restrict__ conv_state, const int* __restrict__ token_seq, const int* __restrict__ state_slots) {
    extern __shared__ float gn_row[];
    __shared__ float part_sum[GN_MAX_UNITS];
    __shared__ float rinv[GN_MAX_GROUPS];
    const int r = blockIdx.x;
    const int gw = h / groups;
    for (int c = threadIdx.x; c < h; c += GN_THREADS) gn_row[c] = to_f(y[(size_t)r * ldy + c]);
    __syncthreads();
    gn_group_scales(gn_row, h, groups, eps_a, part_sum, rinv);
    float* res = resid + (size_t)r * h;
    for (int c = threadIdx.x; c < h; c += GN_THREADS) {
        const float v = res[c] + gn_row[c] * rinv[c / gw] * wa.at(c);
        res[c] = v;
        gn_row[c] = v;
    }
    if (out == nullptr) return;
    __syncthreads();
    gn_group_scales(gn_row, h, groups, eps_b, part_sum, rinv);
    T* o = out + (size_t)r * h;
    if (conv_taps <= 0) {
        for (int c = threadIdx.x; c < h; c += GN_THREADS) o[c] = from_f<T>(gn_row[c] * rinv[c / gw] * wb.at(c));
        return;
    }
    const int seq = token_seq[r];
    if (seq < 0) {
        for (int c = threadIdx.x; c < h; c += GN_THREADS) o[c] = from_f<T>(0.f);
        return;
    }
    T* hist = conv_state + (size_t)state_slots[seq] * (conv_taps - 1) * h;
    for (int c = threadIdx.x; c < h; c += GN_THREADS) {
        const T g = from_f<T>(gn_row[c] * rinv[c / gw] * wb.at(c));
        float acc = to_f(g);
        for (int j = 0; j + 1 < conv_taps; ++j) {
            const T old = hist[(size_t)j * h + c];
            acc = fmaf(conv_w.at((size_t)c * conv_taps + j), to_f(old), acc);
            if (j > 0) hist[(size_t)(j - 1) * h + c] = old;
        }
        acc = fmaf(conv_w.at((size_t)c * conv_taps + conv_taps - 1), to_f(g), acc);
        if (conv_taps > 1) hist[(size_t)(conv_taps - 2) * h + c] = g;
        o[c] = from_f<T>(acc);
    }
}

// The same for rows of a multiple of 8 columns whose groups are multiples of 8 too, at most 2048 NC columns,
// everything 16-byte aligned: a thread keeps NC chunks of eight neighbouring columns in registers from the
// first load to the last store, and everything it needs from memory (with CONV also the request's kept rows
// and the taps, at most GN_VEC_TAPS of them, given tap by tap: conv_wt[taps][h]) is asked for before the first
// sum, so the kernel waits for memory once. A chunk's sum of squares goes to LDS; wave w adds the chunks of
// groups w, w + 4, ... in a fixed order.
#define GN_VEC_TAPS 4
template <typename T, int NC, bool CONV>
__global__ void __launch_bounds__(GN_THREADS)
group_norm_add_norm_vec_kernel(const T* __restrict__ y, long ldy, WeightPtr wa, float eps_a, float* __restrict__ resid, WeightPtr wb,
                               float eps_b, int groups, T* __restrict__ out, int h, int conv_taps, WeightPtr conv_wt,
                               T* __restrict__ conv_state, const int* __restrict__ token_seq, const int* __restrict__ state_slots) {
    __shared__ float csum[GN_THREADS * NC];
    __shared__ float rinv[GN_MAX_GROUPS];
    const int r = blockIdx.x;
    const int lane = threadIdx.x % MV_WAVE, wave = threadIdx.x / MV_WAVE;
    const int nchunks = h / 8, gc = nchunks / groups;          // chunks of a row, of a group
    const T* yr = y + (size_t)r * ldy;
    float* res = resid + (size_t)r * h;
    const WeightPtr wbl = out != nullptr ? wb : wa;
    float v[NC][8], xr[NC][8], fa[NC][8], fb[NC][8];
    float kept[CONV ? NC : 1][GN_VEC_TAPS - 1][8], wt[CONV ? NC : 1][GN_VEC_TAPS][8];
    int group_of[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int q = threadIdx.x + GN_THREADS * c;
        const bool ok = q < nchunks;
        const int d = ok ? 8 * q : 0;                           // beyond the row's end: the first chunk again, dropped
        group_of[c] = ok ? q / gc : 0;
        Vec8<T>::load(yr + d, v[c]);
        Vec8<float>::load(res + d, xr[c]);
        wa.at8(d, fa[c]);
        wbl.at8(d, fb[c]);
        if constexpr (CONV) {
            // (every load is issued whatever the number of taps, a tap beyond the last reads the last again and is
            // dropped: a load under a condition is a branch with a wait of its own)
#pragma unroll
            for (int j = 0; j < GN_VEC_TAPS; ++j) conv_wt.at8((size_t)(j < conv_taps ? j : conv_taps - 1) * h + d, wt[c][j]);
        }
    }
    // the request's kept rows hang on two loads in a row (the row's request, its slot): asked for behind everything
    // that does not, so that those loads are on their way meanwhile
    const int seq = CONV ? token_seq[r] : 0;
    T* hist = nullptr;
    if (CONV && seq >= 0 && conv_taps > 1) hist = conv_state + (size_t)state_slots[seq] * (conv_taps - 1) * h;
    const T* kept_rows = hist != nullptr ? hist : yr;          // (no kept rows: some row that is there, dropped)
    const int last_kept = hist != nullptr ? conv_taps - 2 : 0;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int q = threadIdx.x + GN_THREADS * c;
        if constexpr (CONV) {
            const int d = q < nchunks ? 8 * q : 0;
#pragma unroll
            for (int j = 0; j < GN_VEC_TAPS - 1; ++j)
                Vec8<T>::load(kept_rows + (size_t)(j < last_kept ? j : last_kept) * h + d, kept[c][j]);
        }
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s = fmaf(v[c][e], v[c][e], s);
        csum[q] = s;
    }
    auto group_scales = [&](float eps) {
        __syncthreads();
        for (int g = wave; g < groups; g += GN_WAVES) {
            float s = 0.f;
            for (int k = lane; k < gc; k += MV_WAVE) s += csum[g * gc + k];
            s = wave_sum(s);
            if (lane == 0) rinv[g] = 1.f / sqrtf(s / (float)(8 * gc) + eps);
        }
        __syncthreads();
    };
    group_scales(eps_a);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int q = threadIdx.x + GN_THREADS * c;
        const float ra = rinv[group_of[c]];
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[c][e] = xr[c][e] + v[c][e] * ra * fa[c][e];
            s = fmaf(v[c][e], v[c][e], s);
        }
        if (q < nchunks) Vec8<float>::store(res + 8 * q, v[c]);
        csum[q] = s;
    }
    if (out == nullptr) return;
    group_scales(eps_b);
    T* o = out + (size_t)r * h;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int q = threadIdx.x + GN_THREADS * c;
        if (q >= nchunks) continue;
        const float rb = rinv[group_of[c]];
        float g8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) g8[e] = v[c][e] * rb * fb[c][e];
        if constexpr (!CONV) {
            Vec8<T>::store(o + 8 * q, g8);
        } else {
            float acc[8];
            if (seq < 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] = 0.f;
                Vec8<T>::store(o + 8 * q, acc);
                continue;
            }
            // the row as it is stored (rounded to T) is what the taps see and what the request keeps
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                g8[e] = to_f(from_f<T>(g8[e]));
                acc[e] = g8[e];
            }
#pragma unroll
            for (int j = 0; j < GN_VEC_TAPS - 1; ++j) {
                if (j < conv_taps - 1) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[e] = fmaf(wt[c][j][e], kept[c][j][e], acc[e]);
                    if (j > 0) Vec8<T>::store(hist + (size_t)(j - 1) * h + 8 * q, kept[c][j]);
                }
            }
#pragma unroll
            for (int j = 0; j < GN_VEC_TAPS; ++j) {
                if (j == conv_taps - 1) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[e] = fmaf(wt[c][j][e], g8[e], acc[e]);
                }
            }
            if (conv_taps > 1) Vec8<T>::store(hist + (size_t)(conv_taps - 2) * h + 8 * q, g8);
            Vec8<T>::store(o + 8 * q, acc);
        }
    }
}

template <typename T, bool CONV>
static void launch_add_norm_vec(int nc, int n, hipStream_t stream, const void* y, long ldy, WeightPtr a, float eps_a, float* resid,
                                WeightPtr b, float eps_b, int groups, void* out, int h, int conv_taps, WeightPtr cwt,
                                void* conv_state, const int* token_seq, const int* state_slots) {
#define GN_LAUNCH(NC)                                                                                                       \
    hipLaunchKernelGGL((group_norm_add_norm_vec_kernel<T, NC, CONV>), dim3(n), dim3(GN_THREADS), 0, stream, (const T*)y, ldy, a, \
                       eps_a, resid, b, eps_b, groups, (T*)out, h, conv_taps, cwt, (T*)conv_state, token_seq, state_slots)
    if (nc == 1) GN_LAUNCH(1);
    else if (nc == 2) GN_LAUNCH(2);
    else GN_LAUNCH(4);
#undef GN_LAUNCH
}

static bool gn_aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

// conv_w [h][taps]; conv_wt the same taps given tap by tap, [taps][h], or null (the vector kernel needs it)
extern "C" int mv_group_norm_add_norm(const void* y, long ldy, const void* wa, int wa_dtype, float eps_a, float* resid,
                                      const void* wb, int wb_dtype, float eps_b, int groups, void* out, int n, int h,
                                      int conv_taps, const void* conv_w, const void* conv_wt, int conv_w_dtype, void* conv_state,
                                      const int* token_seq, const int* state_slots, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && h > 0 && groups >= 1 && groups <= GN_MAX_GROUPS && h % groups == 0 && ldy >= h,
               "group_norm_add_norm: rows of %d columns do not form %d equal groups (at most %d)", h, groups, GN_MAX_GROUPS);
    MV_REQUIRE(y && wa && resid && mv_valid_dtype(wa_dtype) && eps_a > 0.f, "group_norm_add_norm: missing operand");
    MV_REQUIRE(out == nullptr || (wb && mv_valid_dtype(wb_dtype) && eps_b > 0.f), "group_norm_add_norm: an output needs the second norm");
    MV_REQUIRE(conv_taps == 0 || (conv_taps >= 1 && out && conv_w && mv_valid_dtype(conv_w_dtype) && token_seq && state_slots
                                  && (conv_state || conv_taps == 1)),
               "group_norm_add_norm: a convolution needs its taps, the state and the step's request of every row");
    MV_REQUIRE((size_t)h * sizeof(float) <= GN_MAX_ROW_BYTES, "group_norm_add_norm: rows of %d columns exceed the %d that fit LDS", h, (int)(GN_MAX_ROW_BYTES / 4));
    if (n == 0) return 0;
    WeightPtr a{wa, wa_dtype}, b{wb, wb_dtype}, cw{conv_w, conv_w_dtype};
    const size_t item = dtype == MV_F32 ? 4 : 2;
    if (h % 8 == 0 && (h / groups) % 8 == 0 && h <= 2048 * 4 && (ldy * item) % 16 == 0 && gn_aligned16(y) && gn_aligned16(resid)
        && gn_aligned16(wa) && (out == nullptr || (gn_aligned16(out) && gn_aligned16(wb)))
        && (conv_taps == 0 || (conv_taps <= GN_VEC_TAPS && conv_wt != nullptr && gn_aligned16(conv_wt) && gn_aligned16(conv_state)))) {
        const int nc = h <= 2048 ? 1 : h <= 4096 ? 2 : 4;
        const WeightPtr cwt{conv_wt, conv_w_dtype};
        if (conv_taps > 0) {
            MV_DISPATCH_T(dtype, "group_norm_add_norm",
                          (launch_add_norm_vec<T, true>(nc, n, stream, y, ldy, a, eps_a, resid, b, eps_b, groups, out, h, conv_taps,
                                                        cwt, conv_state, token_seq, state_slots)));
        } else {
            MV_DISPATCH_T(dtype, "group_norm_add_norm",
                          (launch_add_norm_vec<T, false>(nc, n, stream, y, ldy, a, eps_a, resid, b, eps_b, groups, out, h, 0, cwt,
                                                         nullptr, nullptr, nullptr)));
        }
        return mv_check_launch("group_norm_add_norm");
    }
    MV_DISPATCH_T(dtype, "group_norm_add_norm",
                  hipLaunchKernelGGL(group_norm_add_norm_kernel<T>, dim3(n), dim3(GN_THREADS), (size_t)h * sizeof(float), stream,
                                     (const T*)y, ldy, a, eps_a, resid, b, eps_b, groups, (T*)out, h, conv_taps, cw,
                                     (T*)conv_state, token_seq, state_slots));
    return mv_check_launch("group_norm_add_norm");
}
