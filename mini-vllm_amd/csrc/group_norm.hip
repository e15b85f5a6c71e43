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

extern "C" int mv_group_norm_add_norm(const void* y, long ldy, const void* wa, int wa_dtype, float eps_a, float* resid,
                                      const void* wb, int wb_dtype, float eps_b, int groups, void* out, int n, int h,
                                      int conv_taps, const void* conv_w, int conv_w_dtype, void* conv_state,
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
    MV_DISPATCH_T(dtype, "group_norm_add_norm",
                  hipLaunchKernelGGL(group_norm_add_norm_kernel<T>, dim3(n), dim3(GN_THREADS), (size_t)h * sizeof(float), stream,
                                     (const T*)y, ldy, a, eps_a, resid, b, eps_b, groups, (T*)out, h, conv_taps, cw,
                                     (T*)conv_state, token_seq, state_slots));
    return mv_check_launch("group_norm_add_norm");
}
