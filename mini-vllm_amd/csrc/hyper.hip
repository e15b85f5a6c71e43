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

// The same with a thread keeping NC chunks of four columns in registers from the first load to the last store
// (rows of a multiple of four columns, up to 1024 * NC; everything 16-byte aligned): the lanes go in and out 16
// bytes at a time, and the mixture that is normalised never leaves the registers.
template <typename T> struct Quad;
template <> struct Quad<float> {
    static __device__ __forceinline__ void load(const float* p, float (&x)[4]) {
        const float4 a = *reinterpret_cast<const float4*>(p);
        x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&x)[4]) {
        *reinterpret_cast<float4*>(p) = float4{x[0], x[1], x[2], x[3]};
    }
};
template <> struct Quad<bf16> {
    static __device__ __forceinline__ void load(const bf16* p, float (&x)[4]) {
        const uint2 u = *reinterpret_cast<const uint2*>(p);
        x[0] = __uint_as_float(u.x << 16); x[1] = __uint_as_float(u.x & 0xffff0000u);
        x[2] = __uint_as_float(u.y << 16); x[3] = __uint_as_float(u.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(bf16* p, const float (&x)[4]) {
        *reinterpret_cast<uint2*>(p) = uint2{f32x2_to_bf16x2_bits(x[0], x[1]), f32x2_to_bf16x2_bits(x[2], x[3])};
    }
};

template <typename T, int S, int NC>
__global__ void __launch_bounds__(HY_THREADS)
hyper_step_vec_kernel(float* __restrict__ lanes, long plane, const float* __restrict__ first, int W,
                      const T* __restrict__ y, long ldy, const float* __restrict__ w_mix, const float* __restrict__ w_out,
                      const float* __restrict__ w_in, WeightPtr w_norm, float eps, T* __restrict__ h, long ldh,
                      float* __restrict__ total) {
    __shared__ float scratch[17];
    const int row = blockIdx.x, tid = threadIdx.x;
    const size_t base = (size_t)row * W;
    // the stream weights are the same for every thread: scalar loads
    float mix[S][S], wo[S], wi[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int t = 0; t < S; ++t) mix[s][t] = y != nullptr ? w_mix[s * S + t] : 0.f;
        wo[s] = y != nullptr ? w_out[s] : 0.f;
        wi[s] = w_in != nullptr ? w_in[s] : 0.f;
    }
    float u[NC][4];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NC; ++k) {
        const int c = 4 * (tid + k * HY_THREADS);
        if (c >= W) break;
        float x[S][4];
        if (first != nullptr) {
            float e[4];
            Quad<float>::load(first + base + c, e);
#pragma unroll
            for (int s = 0; s < S; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) x[s][i] = e[i];
        } else {
#pragma unroll
            for (int s = 0; s < S; ++s) Quad<float>::load(lanes + (size_t)s * plane + base + c, x[s]);
        }
        if (y != nullptr) {
            float yv[4];
            Quad<T>::load(y + (size_t)row * ldy + c, yv);
            float nx[S][4];
#pragma unroll
            for (int t = 0; t < S; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float a = 0.f;
#pragma unroll
                    for (int s = 0; s < S; ++s) a = fmaf(mix[s][t], x[s][i], a);
                    nx[t][i] = fmaf(wo[t], yv[i], a);
                }
#pragma unroll
            for (int t = 0; t < S; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) x[t][i] = nx[t][i];
        }
        if (total != nullptr) {
            float a[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[i] = 0.f;
#pragma unroll
                for (int s = 0; s < S; ++s) a[i] += x[s][i];
            }
            Quad<float>::store(total + base + c, a);
        }
        if ((total == nullptr || w_in != nullptr) && (y != nullptr || first != nullptr)) {
#pragma unroll
            for (int s = 0; s < S; ++s) Quad<float>::store(lanes + (size_t)s * plane + base + c, x[s]);
        }
        if (w_in != nullptr) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float a = 0.f;
#pragma unroll
                for (int s = 0; s < S; ++s) a = fmaf(wi[s], x[s][i], a);
                u[k][i] = a;
                ss = fmaf(a, a, ss);
            }
        }
    }
    if (w_in == nullptr) return;
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
    for (int k = 0; k < NC; ++k) {
        const int c = 4 * (tid + k * HY_THREADS);
        if (c >= W) break;
        float wn[4], o[4];
        w_norm.at_few<4>(c, wn);
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = u[k][i] * inv * wn[i];
        Quad<T>::store(h + (size_t)row * ldh + c, o);
    }
}

template <typename T, int S>
static bool hyper_vec_launch(int n, int W, hipStream_t stream, float* lanes, long plane, const float* first, const T* y, long ldy,
                             const float* w_mix, const float* w_out, const float* w_in, WeightPtr wn, float eps, T* h, long ldh,
                             float* total) {
    const int chunks = (W / 4 + HY_THREADS - 1) / HY_THREADS;
#define HY_VEC(NC)                                                                                                       \
    hipLaunchKernelGGL((hyper_step_vec_kernel<T, S, NC>), dim3(n), dim3(HY_THREADS), 0, stream, lanes, plane, first, W, y, ldy, \
                       w_mix, w_out, w_in, wn, eps, h, ldh, total)
    if (chunks <= 1) HY_VEC(1);
    else if (chunks <= 2) HY_VEC(2);
    else if (chunks <= 4) HY_VEC(4);
    else if (chunks <= 8) HY_VEC(8);
    else return false;
#undef HY_VEC
    return true;
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
    // four columns at a time: rows of floats 16 bytes, rows of the activation type at least 8 bytes aligned
    const bool aligned = W % 4 == 0 && plane % 4 == 0 && ((uintptr_t)lanes % 16) == 0 && ((uintptr_t)first % 16) == 0 &&
                         ((uintptr_t)total % 16) == 0 && ((uintptr_t)y % 16) == 0 && ldy % 4 == 0 &&
                         ((uintptr_t)h % 16) == 0 && ldh % 4 == 0 && ((uintptr_t)w_norm % 16) == 0;
    if (aligned && S <= 4 && W <= 4 * HY_THREADS * 8) {
        bool took = false;
#define HY_S(SS)                                                                                                                \
    MV_DISPATCH_T(dtype, "hyper_step",                                                                                          \
                  took = hyper_vec_launch<T, SS>(n, W, stream, lanes, plane, first, (const T*)y, ldy, w_mix, w_out, w_in, wn, eps, \
                                                 (T*)h, ldh, total))
        if (S == 1) { HY_S(1); } else if (S == 2) { HY_S(2); } else if (S == 3) { HY_S(3); } else { HY_S(4); }
#undef HY_S
        if (took) return mv_check_launch("hyper_step");
    }
    const size_t lds = w_in ? (size_t)W * sizeof(float) : 0;
    MV_DISPATCH_T(dtype, "hyper_step",
                  hipLaunchKernelGGL(hyper_step_kernel<T>, dim3(n), dim3(HY_THREADS), lds, stream, lanes, plane, first, S, W,
                                     (const T*)y, ldy, w_mix, w_out, w_in, wn, eps, (T*)h, ldh, total));
    return mv_check_launch("hyper_step");
}
