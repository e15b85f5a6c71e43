// Several residual streams (hyper-connections). A token's residual is S rows x_1 .. x_S of the
// model's width, kept in float as lanes[S][n][W]. A sublayer reads one mixture of them,
//     u = sum_s w_in[s] x_s,            h = u / sqrt(mean(u^2) + eps) * w_norm
// and its output y is written back into all of them at once, from the old ones:
//     x_t <- sum_s w_mix[s][t] x_s + w_out[t] y.
// One launch does the write of the sublayer that has just run and the read (with its norm) of the
// sublayer that runs next, so the lanes are read and written once between two sublayers:
//   expand   the lanes do not exist yet: every old x_s is the row of `first` (the embedding's output)
//   y        the write (absent in front of the model's first sublayer)
//   w_in     the read; h goes out in the activation type
//   total    behind the model's last sublayer: the sum of the new lanes, the plain residual again
// Everything is float but y and h. A row's sums depend on nothing but the row: columns are summed in
// a fixed order (thread by thread, then wave by wave).
#include "dispatch.h"

#define HY_MAX_S 8
#define HY_THREADS 256

struct HyperWeights {
    float mix[HY_MAX_S][HY_MAX_S];
    float out[HY_MAX_S];
    float in[HY_MAX_S];
};

template <typename T>
__global__ void __launch_bounds__(HY_THREADS)
hyper_step_kernel(float* __restrict__ lanes, long plane, const float* __restrict__ first, int S, int W,
                  const T* __restrict__ y, long ldy, const float* __restrict__ w_mix, const float* __restrict__ w_out,
                  const float* __restrict__ w_in, WeightPtr w_norm, float eps, T* __restrict__ h, long ldh,
                  float* __restrict__ total) {
    extern __shared__ float u_row[];              // W floats: the mixture that is normalised
    __shared__ float scratch[17];
    __shared__ HyperWeights hw;
    const int row = blockIdx.x, tid = threadIdx.x;
    if (tid < S * S) hw.mix[tid / S][tid % S] = w_mix ? w_mix[tid] : (tid / S == tid % S ? 1.f : 0.f);
    if (tid < S) {
        hw.out[tid] = w_out ? w_out[tid] : 0.f;
        hw.in[tid] = w_in ? w_in[tid] : 0.f;
    }
    __syncthreads();
    const size_t base = (size_t)row * W;
    float ss = 0.f;
    for (int c = tid; c < W; c += HY_THREADS) {
        float x[HY_MAX_S];
        if (first != nullptr) {
            const float e = first[base + c];
#pragma unroll
            for (int s = 0; s < HY_MAX_S; ++s) x[s] = e;
        } else {
#pragma unroll
            for (int s = 0; s < HY_MAX_S; ++s) x[s] = s < S ? lanes[(size_t)s * plane + base + c] : 0.f;
        }
        if (y != nullptr) {
            const float yv = to_f(y[(size_t)row * ldy + c]);
            float nx[HY_MAX_S];
#pragma unroll
            for (int t = 0; t < HY_MAX_S; ++t) {
                float a = 0.f;
                if (t < S) {
#pragma unroll
                    for (int s = 0; s < HY_MAX_S; ++s)
                        if (s < S) a = fmaf(hw.mix[s][t], x[s], a);
                    a = fmaf(hw.out[t], yv, a);
                }
                nx[t] = a;
            }
#pragma unroll
            for (int t = 0; t < HY_MAX_S; ++t) x[t] = nx[t];
        }
        if (total != nullptr) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < HY_MAX_S; ++s)
                if (s < S) a += x[s];
            total[base + c] = a;
        }
        if (total == nullptr || w_in != nullptr) {
            if (y != nullptr || first != nullptr) {
#pragma unroll
                for (int s = 0; s < HY_MAX_S; ++s)
                    if (s < S) lanes[(size_t)s * plane + base + c] = x[s];
            }
        }
        if (w_in != nullptr) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < HY_MAX_S; ++s)
                if (s < S) a = fmaf(hw.in[s], x[s], a);
            u_row[c] = a;
            ss = fmaf(a, a, ss);
        }
    }
    if (w_in == nullptr) return;
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)W + eps);
    for (int c = tid; c < W; c += HY_THREADS) h[(size_t)row * ldh + c] = from_f<T>(u_row[c] * inv * w_norm.at(c));
}

// lanes float [S][n][W] (plane = elements between two lanes); first float [n][W] or null; y [n][>= W] of the
// activation type or null (then w_mix and w_out are not read); w_mix float [S][S] indexed [from][to], w_out and
// w_in float [S]; w_in null: no read (h is not written); total float [n][W] or null.
extern "C" int mv_hyper_step(float* lanes, long plane, const float* first, int S, int n, int W, const void* y, long ldy,
                             const float* w_mix, const float* w_out, const float* w_in, const void* w_norm, int norm_dtype,
                             float eps, void* h, long ldh, float* total, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && S >= 1 && S <= HY_MAX_S && W > 0 && W <= 16384, "hyper_step: bad sizes n=%d streams=%d (at most %d) width=%d",
               n, S, HY_MAX_S, W);
    MV_REQUIRE(lanes && plane >= (long)n * W, "hyper_step: the lanes are missing or their planes too small");
    MV_REQUIRE(!y || (w_mix && w_out && ldy >= W), "hyper_step: a write needs its weights and rows of the width");
    MV_REQUIRE(!w_in || (w_norm && h && ldh >= W && eps > 0.f && mv_valid_dtype(norm_dtype)), "hyper_step: a read needs the norm's weight and an output");
    MV_REQUIRE(y || first || w_in || total, "hyper_step: nothing to do");
    if (n == 0) return 0;
    WeightPtr wn{w_norm, norm_dtype};
    const size_t lds = w_in ? (size_t)W * sizeof(float) : 0;
    MV_DISPATCH_T(dtype, "hyper_step",
                  hipLaunchKernelGGL(hyper_step_kernel<T>, dim3(n), dim3(HY_THREADS), lds, stream, lanes, plane, first, S, W,
                                     (const T*)y, ldy, w_mix, w_out, w_in, wn, eps, (T*)h, ldh, total));
    return mv_check_launch("hyper_step");
}
