// Attention over a cached latent: every token caches one row [latent (R) | rotated key part (DR)]
// that all query heads share. A head's key is a linear map of the latent (W_uk) beside the shared
// rotated part, its value another linear map (W_uv); neither is ever materialised. With
// qa = W_uk^T q_plain (the query carried into the latent's space) the score of a key is
//     (qa . latent + q_rot . k_rot) * scale
// and the head's output is W_uv applied to the softmax-weighted sum of the latents. So the kernels are
//     latent_prepare     norms of the two down-projections, rotation of the key part, cache write
//     head_linear        per head y = W_h x (queries into latent space, rotating their rotated part on
//                        the way; weighted latents into values, times the output gate)
//     attention_latent   softmax attention with one shared key row of R + DR numbers whose first R
//                        are also the value
// Page layout: rows[page][slot][R + DR] in the activation type, and the latents once more with a page's slots side
// by side, [page][R][slot], which is how the MFMA kernel's second product wants them. Scores, weights and sums are float.
#include "dispatch.h"

// ---------------------------------------------------------------------------------------
// Prepare. Packed rows: [dq (QR) | dkv (R + DR) | ...]. One workgroup per row:
//   cq[t]           = dq / rms(dq) * wq                      (the query's latent, activation type)
//   page row of t   = [dkv[:R] / rms(dkv[:R]) * wkv | rot(dkv[R:], position)]
// rot pairs channel i with i + DR/2; table[p] = [cos (DR/2) | sin (DR/2)] of position p.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const T* __restrict__ packed, long ld, int QR, int R, int DR, WeightPtr wq, WeightPtr wkv, float eps,
                      const float* __restrict__ table, const int* __restrict__ positions, const int* __restrict__ token_seq,
                      const int* __restrict__ block_table, int bt_width, int page_size, T* __restrict__ cq, long ldq,
                      T* __restrict__ pages, T* __restrict__ pages_t) {
    __shared__ float scratch[17];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int seq = token_seq[t];
    T* qo = cq + (size_t)t * ldq;
    if (seq < 0) {
        for (int c = tid; c < QR; c += 256) qo[c] = from_f<T>(0.f);
        return;
    }
    const T* p = packed + (size_t)t * ld;
    float ss = 0.f;
    for (int c = tid; c < QR; c += 256) {
        const float x = to_f(p[c]);
        ss = fmaf(x, x, ss);
    }
    ss = block_sum(ss, scratch);
    float inv = 1.f / sqrtf(ss / (float)QR + eps);
    for (int c = tid; c < QR; c += 256) qo[c] = from_f<T>(to_f(p[c]) * inv * wq.at(c));
    const T* kv = p + QR;
    ss = 0.f;
    for (int c = tid; c < R; c += 256) {
        const float x = to_f(kv[c]);
        ss = fmaf(x, x, ss);
    }
    ss = block_sum(ss, scratch);
    inv = 1.f / sqrtf(ss / (float)R + eps);
    const int pos = positions[t];
    const int page = block_table[(size_t)seq * bt_width + pos / page_size];
    T* row = pages + ((size_t)page * page_size + pos % page_size) * (size_t)(R + DR);
    // (pages_t, when given, holds the latent once more with the slots of a page side by side: [page][R][slot])
    T* col = pages_t ? pages_t + (size_t)page * R * page_size + pos % page_size : nullptr;
    for (int c = tid; c < R; c += 256) {
        const T v = from_f<T>(to_f(kv[c]) * inv * wkv.at(c));
        row[c] = v;
        if (col) col[(size_t)c * page_size] = v;
    }
    const int half = DR / 2;
    const float* cs = table + (size_t)pos * DR;
    for (int i = tid; i < half; i += 256) {
        const float a = to_f(kv[R + i]), b = to_f(kv[R + half + i]);
        const float c = cs[i], s = cs[half + i];
        row[R + i] = from_f<T>(a * c - b * s);
        row[R + half + i] = from_f<T>(b * c + a * s);
    }
}

extern "C" int mv_latent_prepare(const void* packed, long ld, int n, int QR, int R, int DR, const void* wq, const void* wkv,
                                 int weight_dtype, float eps, const float* table, int table_rows, const int* positions,
                                 const int* token_seq, const int* block_table, int bt_width, int page_size, void* cq,
                                 long ldq, void* pages, void* pages_t, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && QR > 0 && R > 0 && DR >= 0 && DR % 2 == 0, "latent_prepare: bad sizes n=%d QR=%d R=%d DR=%d", n, QR, R, DR);
    MV_REQUIRE(ld >= (long)QR + R + DR && ldq >= QR && page_size > 0 && bt_width > 0, "latent_prepare: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && packed && wq && wkv && (table || DR == 0) && table_rows >= 0 && positions && token_seq
               && block_table && cq && pages && eps > 0.f, "latent_prepare: missing operand");
    if (n == 0) return 0;
    WeightPtr a{wq, weight_dtype}, b{wkv, weight_dtype};
    MV_DISPATCH_T(dtype, "latent_prepare",
                  hipLaunchKernelGGL(latent_prepare_kernel<T>, dim3(n), dim3(256), 0, stream, (const T*)packed, ld, QR, R, DR, a,
                                     b, eps, table, positions, token_seq, block_table, bt_width, page_size, (T*)cq, ldq,
                                     (T*)pages, (T*)pages_t));
    return mv_check_launch("latent_prepare");
}

// ---------------------------------------------------------------------------------------
// Per-head linear map. x rows [n][H][ldx_head] (IN inputs used), w [H][IN][OUT] (the inputs of an
// output column are a stride of OUT apart, so neighbouring threads read neighbouring words),
// y rows [n][H][ldy_head]:  y[t][h][j] = sum_i x[t][h][i] w[h][i][j], the sum in the order of i.
//   tail > 0   x[t][h][IN .. IN+tail) is copied behind the OUT outputs, rotated by the row's position
//              (pairs i, i + tail/2; table[p] = [cos | sin])
//   gate       y is multiplied by sigmoid(gate[t][h * OUT + j]), or by sigmoid(gate[t][h]) with `gate_per_head`
// ---------------------------------------------------------------------------------------
#define HL_TOKENS 8
#define HL_MAX_IN 1024

// A workgroup takes HL_TOKENS rows, one head and HL_COLS output columns; its 256 threads are HL_COLS columns
// times HL_SLICES slices of the inputs (slice s sums inputs s, s + HL_SLICES, ...), the slices are added in
// order through LDS. (64 columns x 4 slices for steps of many rows; 16 x 16 for steps of few rows, whose few
// workgroups a head would otherwise walk long runs of inputs one load after the other.) The order of additions
// depends on IN and the variant.
template <typename TIN, typename TOUT, typename TG, int HL_COLS, int HL_SLICES>
__global__ void __launch_bounds__(256)
head_linear_kernel(const TIN* __restrict__ x, long ldx, int ldx_head, WeightPtr w, int IN, int OUT, TOUT* __restrict__ y, long ldy,
                   int ldy_head, int tail, const float* __restrict__ table, const int* __restrict__ positions,
                   const TG* __restrict__ gate, long ldg, int gate_per_head, const int* __restrict__ token_seq, int n) {
    __shared__ float xs[HL_TOKENS][HL_MAX_IN];
    __shared__ float part[HL_SLICES][HL_TOKENS][HL_COLS];
    const int t0 = blockIdx.x * HL_TOKENS, head = blockIdx.y, tid = threadIdx.x;
    const int nt = min(HL_TOKENS, n - t0);
    for (int e = tid; e < HL_TOKENS * IN; e += 256) {
        const int tt = e / IN, i = e % IN;
        xs[tt][i] = tt < nt ? to_f(x[(size_t)(t0 + tt) * ldx + (size_t)head * ldx_head + i]) : 0.f;
    }
    __syncthreads();
    const int col = tid % HL_COLS, slice = tid / HL_COLS;
    const int j = blockIdx.z * HL_COLS + col;
    float acc[HL_TOKENS];
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = 0.f;
    if (j < OUT) {
        const size_t w0 = (size_t)head * IN * OUT + j;
        int i = slice;
        for (; i + 3 * HL_SLICES < IN; i += 4 * HL_SLICES) {          // four loads in flight
            float wv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) wv[u] = w.at(w0 + (size_t)(i + u * HL_SLICES) * OUT);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(xs[tt][i + u * HL_SLICES], wv[u], acc[tt]);
        }
        for (; i < IN; i += HL_SLICES) {
            const float wv = w.at(w0 + (size_t)i * OUT);
#pragma unroll
            for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(xs[tt][i], wv, acc[tt]);
        }
    }
#pragma unroll
    for (int tt = 0; tt < HL_TOKENS; ++tt) part[slice][tt][col] = acc[tt];
    __syncthreads();
    for (int e = tid; e < nt * HL_COLS; e += 256) {
        const int tt = e / HL_COLS, c = e % HL_COLS;
        const int jj = blockIdx.z * HL_COLS + c;
        if (jj >= OUT) continue;
        float v = 0.f;
#pragma unroll
        for (int sl = 0; sl < HL_SLICES; ++sl) v += part[sl][tt][c];
        if (token_seq[t0 + tt] < 0) v = 0.f;
        else if (gate) v *= 1.f / (1.f + expf(-to_f(gate[(size_t)(t0 + tt) * ldg + (gate_per_head ? (size_t)head : (size_t)head * OUT + jj)])));
        y[(size_t)(t0 + tt) * ldy + (size_t)head * ldy_head + jj] = from_f<TOUT>(v);
    }
    if (blockIdx.z != 0) return;
    const int half = tail / 2;
    for (int e = tid; e < nt * half; e += 256) {
        const int tt = e / half, i = e % half;
        const int t = t0 + tt;
        const TIN* src = x + (size_t)t * ldx + (size_t)head * ldx_head + IN;
        TOUT* dst = y + (size_t)t * ldy + (size_t)head * ldy_head + OUT;
        if (token_seq[t] < 0) {
            dst[i] = from_f<TOUT>(0.f);
            dst[half + i] = from_f<TOUT>(0.f);
            continue;
        }
        const float* cs = table + (size_t)positions[t] * tail;
        const float a = to_f(src[i]), b = to_f(src[half + i]);
        dst[i] = from_f<TOUT>(a * cs[i] - b * cs[half + i]);
        dst[half + i] = from_f<TOUT>(b * cs[i] + a * cs[half + i]);
    }
}

// mode 0: x activation type -> y float (with an optional rotated tail); mode 1: x float -> y activation
// type (with an optional gate of the activation type)
extern "C" int mv_head_linear(const void* x, long ldx, int ldx_head, const void* w, int weight_dtype, int n, int H, int IN,
                              int OUT, void* y, long ldy, int ldy_head, int tail, const float* table, const int* positions,
                              const void* gate, long ldg, int gate_per_head, const int* token_seq, int mode, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && IN > 0 && OUT > 0 && tail >= 0 && tail % 2 == 0, "head_linear: bad sizes n=%d H=%d IN=%d OUT=%d", n, H, IN, OUT);
    MV_REQUIRE(IN <= HL_MAX_IN, "head_linear: %d inputs a head, at most %d are served", IN, HL_MAX_IN);
    MV_REQUIRE(ldx_head >= IN + tail && ldy_head >= OUT + tail && ldx >= (long)(H - 1) * ldx_head + IN + tail
               && ldy >= (long)(H - 1) * ldy_head + OUT + tail, "head_linear: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && x && w && y && token_seq && (tail == 0 || (table && positions)) && H <= 65535
               && (!gate || ldg >= (gate_per_head ? (long)H : (long)H * OUT)), "head_linear: missing operand");
    MV_REQUIRE((mode == 0 && !gate) || (mode == 1 && tail == 0), "head_linear: mode %d does not take these options", mode);
    if (n == 0) return 0;
    WeightPtr wp{w, weight_dtype};
    const bool few = n <= 64;
    const int cols = few ? 16 : 64;
    dim3 grid((n + HL_TOKENS - 1) / HL_TOKENS, H, (OUT + cols - 1) / cols);
#define HL_LAUNCH(C, S)                                                                                                     \
    if (mode == 0) {                                                                                                        \
        MV_DISPATCH_T(dtype, "head_linear",                                                                                 \
                      hipLaunchKernelGGL((head_linear_kernel<T, float, T, C, S>), grid, dim3(256), 0, stream, (const T*)x, ldx, \
                                         ldx_head, wp, IN, OUT, (float*)y, ldy, ldy_head, tail, table, positions,           \
                                         (const T*)nullptr, 0L, 0, token_seq, n));                                             \
    } else {                                                                                                                \
        MV_DISPATCH_T(dtype, "head_linear",                                                                                 \
                      hipLaunchKernelGGL((head_linear_kernel<float, T, T, C, S>), grid, dim3(256), 0, stream, (const float*)x,  \
                                         ldx, ldx_head, wp, IN, OUT, (T*)y, ldy, ldy_head, 0, table, positions,             \
                                         (const T*)gate, ldg, gate_per_head, token_seq, n));                                               \
    }
    if (few) {
        HL_LAUNCH(16, 16)
    } else {
        HL_LAUNCH(64, 4)
    }
#undef HL_LAUNCH
    return mv_check_launch("head_linear");
}

// ---------------------------------------------------------------------------------------
// Attention. One workgroup per (row, group of AL_HEADS heads): the query heads of a row read the same
// key rows, so a key row that a thread has fetched serves all heads of the group. Keys are visited in
// tiles of AL_THREADS from position 0 (causal: a query at position p sees 0..p), so the order of
// additions depends on the position alone. q float [n][H][R + DR]; out float [n][H][R]: the
// weighted sum of the visible latents.
// ---------------------------------------------------------------------------------------
#define AL_THREADS 128
#define AL_HEADS 4
#define AL_MAX_KEY 640
#define AL_MAX_R 512

template <typename T>
__global__ void __launch_bounds__(AL_THREADS)
attention_latent_kernel(const float* __restrict__ q, long ldq, float* __restrict__ out, long ldo, const T* __restrict__ pages,
                        const int* __restrict__ block_table, int bt_width, int page_size, const int* __restrict__ positions,
                        const int* __restrict__ token_seq, int H, int R, int DR, float scale) {
    __shared__ float qs[AL_HEADS][AL_MAX_KEY];
    __shared__ float ps[AL_HEADS][AL_THREADS];
    __shared__ long roff[AL_THREADS];
    __shared__ float scratch[17];
    const int tok = blockIdx.x, h0 = blockIdx.y * AL_HEADS, tid = threadIdx.x;
    const int nh = min(AL_HEADS, H - h0);
    const int DK = R + DR;
    const int seq = token_seq[tok];
    if (seq < 0) {
        for (int e = tid; e < nh * R; e += AL_THREADS) out[(size_t)tok * ldo + (size_t)(h0 + e / R) * R + e % R] = 0.f;
        return;
    }
    const int hi = positions[tok];
    const int* bt = block_table + (size_t)seq * bt_width;
    for (int e = tid; e < AL_HEADS * DK; e += AL_THREADS) {
        const int hh = e / DK, d = e % DK;
        qs[hh][d] = hh < nh ? q[(size_t)tok * ldq + (size_t)(h0 + hh) * DK + d] : 0.f;
    }
    __syncthreads();
    float m[AL_HEADS], l[AL_HEADS];
    float acc[AL_HEADS][AL_MAX_R / AL_THREADS];
#pragma unroll
    for (int hh = 0; hh < AL_HEADS; ++hh) {
        m[hh] = -INFINITY;
        l[hh] = 0.f;
#pragma unroll
        for (int i = 0; i < AL_MAX_R / AL_THREADS; ++i) acc[hh][i] = 0.f;
    }
    for (int base = 0; base <= hi; base += AL_THREADS) {
        const int j = base + tid;
        const bool valid = j <= hi;
        float s[AL_HEADS];
#pragma unroll
        for (int hh = 0; hh < AL_HEADS; ++hh) s[hh] = -INFINITY;
        long ro = 0;
        if (valid) {
            ro = ((long)bt[j / page_size] * page_size + j % page_size) * DK;
            const T* row = pages + ro;
            float dot[AL_HEADS];
#pragma unroll
            for (int hh = 0; hh < AL_HEADS; ++hh) dot[hh] = 0.f;
            for (int d = 0; d < DK; ++d) {
                const float kd = to_f(row[d]);
#pragma unroll
                for (int hh = 0; hh < AL_HEADS; ++hh) dot[hh] = fmaf(qs[hh][d], kd, dot[hh]);
            }
#pragma unroll
            for (int hh = 0; hh < AL_HEADS; ++hh) s[hh] = dot[hh] * scale;
        }
        roff[tid] = ro;
        float corr[AL_HEADS];
#pragma unroll
        for (int hh = 0; hh < AL_HEADS; ++hh) {
            const float tmax = block_max(s[hh], scratch);
            const float m_new = fmaxf(m[hh], tmax);
            const float p = valid ? expf(s[hh] - m_new) : 0.f;
            ps[hh][tid] = p;
            const float tsum = block_sum(p, scratch);      // its barriers also publish ps and roff
            corr[hh] = expf(m[hh] - m_new);                // first tile: exp(-inf) = 0
            l[hh] = l[hh] * corr[hh] + tsum;
            m[hh] = m_new;
        }
        const int cnt = min(AL_THREADS, hi - base + 1);
#pragma unroll
        for (int i = 0; i < AL_MAX_R / AL_THREADS; ++i) {
            const int d = tid + i * AL_THREADS;
            if (d < R) {
                float a[AL_HEADS];
#pragma unroll
                for (int hh = 0; hh < AL_HEADS; ++hh) a[hh] = acc[hh][i] * corr[hh];
                for (int jj = 0; jj < cnt; ++jj) {
                    const float v = to_f(pages[roff[jj] + d]);
#pragma unroll
                    for (int hh = 0; hh < AL_HEADS; ++hh) a[hh] = fmaf(ps[hh][jj], v, a[hh]);
                }
#pragma unroll
                for (int hh = 0; hh < AL_HEADS; ++hh) acc[hh][i] = a[hh];
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int hh = 0; hh < AL_HEADS; ++hh) {
        if (hh < nh) {
            const float inv = 1.f / l[hh];
#pragma unroll
            for (int i = 0; i < AL_MAX_R / AL_THREADS; ++i) {
                const int d = tid + i * AL_THREADS;
                if (d < R) out[(size_t)tok * ldo + (size_t)(h0 + hh) * R + d] = acc[hh][i] * inv;
            }
        }
    }
}

extern "C" int mv_attention_latent(const float* q, long ldq, float* out, long ldo, const void* pages, const int* block_table,
                                   int bt_width, int page_size, const int* positions, const int* token_seq, int n, int H,
                                   int R, int DR, float scale, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && R > 0 && DR >= 0, "attention_latent: bad sizes n=%d H=%d R=%d DR=%d", n, H, R, DR);
    MV_REQUIRE(R <= AL_MAX_R && R + DR <= AL_MAX_KEY, "attention_latent: a latent of %d and a rotated part of %d exceed %d / %d",
               R, DR, AL_MAX_R, AL_MAX_KEY);
    MV_REQUIRE(page_size > 0 && bt_width > 0 && ldq >= (long)H * (R + DR) && ldo >= (long)H * R, "attention_latent: pitches too small");
    MV_REQUIRE(q && out && pages && block_table && positions && token_seq && (H + AL_HEADS - 1) / AL_HEADS <= 65535,
               "attention_latent: missing operand");
    if (n == 0) return 0;
    MV_DISPATCH_T(dtype, "attention_latent",
                  hipLaunchKernelGGL(attention_latent_kernel<T>, dim3(n, (H + AL_HEADS - 1) / AL_HEADS), dim3(AL_THREADS), 0,
                                     stream, q, ldq, out, ldo, (const T*)pages, block_table, bt_width, page_size, positions,
                                     token_seq, H, R, DR, scale));
    return mv_check_launch("attention_latent");
}

// ---------------------------------------------------------------------------------------
// Attention for steps of few rows (single decoded tokens): a row's keys are dealt out to workgroups in
// runs of `run` positions (run s holds positions s * run ..., so the cutting depends on the position and
// the launch's run length alone), a workgroup serves up to ALS_HEADS heads of the row at once and brings each tile of
// ALS_TILE key rows into LDS with 16-byte loads, where all its heads read them. It leaves per run the
// running maximum, the sum of weights and the weighted sum of latents; a second kernel joins the runs
// in their order. Requires (R + DR) * sizeof(T) to be a multiple of 16.
// ---------------------------------------------------------------------------------------
#define ALS_MAX_VEC 8          // 16-byte pieces of a tile a thread brings in: key rows of up to 1,024 bytes
#define ALS_TILE 32
#define ALS_HEADS 16
#define ALS_THREADS 256

template <typename T> struct AlsWord;
template <> struct AlsWord<float> { static constexpr int per = 1; };
template <> struct AlsWord<bf16> { static constexpr int per = 2; };

template <typename T>
__device__ __forceinline__ void als_unpack(uint32_t w, float (&out)[AlsWord<T>::per]) {
    if constexpr (AlsWord<T>::per == 1) {
        out[0] = __uint_as_float(w);
    } else {
        out[0] = __uint_as_float(w << 16);
        out[1] = __uint_as_float(w & 0xffff0000u);
    }
}

template <typename T>
__global__ void __launch_bounds__(ALS_THREADS)
attention_latent_split_kernel(const float* __restrict__ q, long ldq, const T* __restrict__ pages, const int* __restrict__ block_table,
                              int bt_width, int page_size, const int* __restrict__ positions, const int* __restrict__ token_seq,
                              int H, int R, int DR, float scale, int row_words, int run, int max_splits,
                              float* __restrict__ part_o, float* __restrict__ part_ml) {
    extern __shared__ __attribute__((aligned(16))) unsigned char als_lds[];
    constexpr int PER = AlsWord<T>::per;
    const int DK = R + DR;
    const int words = DK / PER;                             // words of a key row; row_words (odd) is its pitch in LDS
    float* qs = reinterpret_cast<float*>(als_lds);          // [ALS_HEADS][DK]
    uint32_t* tile = reinterpret_cast<uint32_t*>(qs + ALS_HEADS * DK);      // [ALS_TILE][row_words]
    float* ps = reinterpret_cast<float*>(tile + ALS_TILE * row_words);      // [ALS_TILE][ALS_HEADS]
    float* cs = ps + ALS_TILE * ALS_HEADS;                  // [ALS_HEADS]
    const int tok = blockIdx.x, h0 = blockIdx.y * ALS_HEADS, split = blockIdx.z, tid = threadIdx.x;
    const int seq = token_seq[tok];
    if (seq < 0) return;
    const int pos = positions[tok];
    const int lo = split * run;
    if (lo > pos) return;
    const int hi = min(pos, lo + run - 1);
    const int nh = min(ALS_HEADS, H - h0);
    const int* bt = block_table + (size_t)seq * bt_width;
    for (int e = tid; e < ALS_HEADS * DK; e += ALS_THREADS) {
        const int hh = e / DK, d = e % DK;
        qs[e] = hh < nh ? q[(size_t)tok * ldq + (size_t)(h0 + hh) * DK + d] * scale : 0.f;
    }
    // scores: thread (key j of the tile, head pair hp) -> heads 2 hp, 2 hp + 1; sums: thread -> latent channels tid, tid + 256
    const int j = tid % ALS_TILE, hp = tid / ALS_TILE;
    float m0 = -INFINITY, m1 = -INFINITY, l0 = 0.f, l1 = 0.f;
    float acc[2][ALS_HEADS];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int hh = 0; hh < ALS_HEADS; ++hh) acc[c][hh] = 0.f;
    const int vec_per_row = words / 4;                      // 16-byte pieces of a key row
    // a tile comes from memory into registers while the tile before it is computed, and from there into LDS
    uint4 held[ALS_MAX_VEC];
    auto fetch = [&](int base) {
        const int cnt = min(ALS_TILE, hi - base + 1);
#pragma unroll
        for (int x = 0; x < ALS_MAX_VEC; ++x) {
            const int e = tid + x * ALS_THREADS;
            if (e < cnt * vec_per_row) {
                const int jj = e / vec_per_row, v = e % vec_per_row;
                const int p = base + jj;
                const T* row = pages + ((size_t)bt[p / page_size] * page_size + p % page_size) * DK;
                held[x] = reinterpret_cast<const uint4*>(row)[v];
            }
        }
    };
    fetch(lo);
    for (int base = lo; base <= hi; base += ALS_TILE) {
        const int cnt = min(ALS_TILE, hi - base + 1);
        __syncthreads();                                    // the tile before has been read (and qs is written)
#pragma unroll
        for (int x = 0; x < ALS_MAX_VEC; ++x) {
            const int e = tid + x * ALS_THREADS;
            if (e < cnt * vec_per_row) {
                uint32_t* dst = tile + (e / vec_per_row) * row_words + 4 * (e % vec_per_row);
                dst[0] = held[x].x; dst[1] = held[x].y; dst[2] = held[x].z; dst[3] = held[x].w;
            }
        }
        if (base + ALS_TILE <= hi) fetch(base + ALS_TILE);
        __syncthreads();
        float s0 = 0.f, s1 = 0.f;
        if (j < cnt) {
            const uint32_t* krow = tile + j * row_words;
            const float* qa = qs + (2 * hp) * DK;
            const float* qb = qa + DK;
            for (int w = 0; w < words; ++w) {
                float k[PER];
                als_unpack<T>(krow[w], k);
#pragma unroll
                for (int u = 0; u < PER; ++u) {
                    s0 = fmaf(qa[w * PER + u], k[u], s0);
                    s1 = fmaf(qb[w * PER + u], k[u], s1);
                }
            }
        } else {
            s0 = s1 = -INFINITY;
        }
        // maximum and sum over the tile's keys: the 32 lanes that share a head pair are half a wave
        float t0 = s0, t1 = s1;
#pragma unroll
        for (int o = ALS_TILE / 2; o > 0; o >>= 1) {
            t0 = fmaxf(t0, __shfl_xor(t0, o, 64));
            t1 = fmaxf(t1, __shfl_xor(t1, o, 64));
        }
        const float n0 = fmaxf(m0, t0), n1 = fmaxf(m1, t1);
        const float p0 = j < cnt ? expf(s0 - n0) : 0.f, p1 = j < cnt ? expf(s1 - n1) : 0.f;
        float u0 = p0, u1 = p1;
#pragma unroll
        for (int o = ALS_TILE / 2; o > 0; o >>= 1) {
            u0 += __shfl_xor(u0, o, 64);
            u1 += __shfl_xor(u1, o, 64);
        }
        const float c0 = expf(m0 - n0), c1 = expf(m1 - n1);           // first tile: exp(-inf) = 0
        l0 = l0 * c0 + u0; l1 = l1 * c1 + u1;
        m0 = n0; m1 = n1;
        ps[j * ALS_HEADS + 2 * hp] = p0;
        ps[j * ALS_HEADS + 2 * hp + 1] = p1;
        if (j == 0) {
            cs[2 * hp] = c0;
            cs[2 * hp + 1] = c1;
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int d = tid + c * ALS_THREADS;
            if (d < R) {
#pragma unroll
                for (int hh = 0; hh < ALS_HEADS; ++hh) acc[c][hh] *= cs[hh];
                for (int jj = 0; jj < cnt; ++jj) {
                    const uint32_t word = tile[jj * row_words + d / PER];
                    const float v = PER == 1 ? __uint_as_float(word) : __uint_as_float((d & 1) ? (word & 0xffff0000u) : (word << 16));
                    const float4* pr = reinterpret_cast<const float4*>(ps + jj * ALS_HEADS);
#pragma unroll
                    for (int g = 0; g < ALS_HEADS / 4; ++g) {
                        const float4 pp = pr[g];
                        acc[c][4 * g] = fmaf(pp.x, v, acc[c][4 * g]);
                        acc[c][4 * g + 1] = fmaf(pp.y, v, acc[c][4 * g + 1]);
                        acc[c][4 * g + 2] = fmaf(pp.z, v, acc[c][4 * g + 2]);
                        acc[c][4 * g + 3] = fmaf(pp.w, v, acc[c][4 * g + 3]);
                    }
                }
            }
        }
    }
    // the run's results: [row][head][run][R] and [row][head][run][2]
    if (j == 0) {
        for (int u = 0; u < 2; ++u) {
            const int hh = 2 * hp + u;
            if (hh < nh) {
                float* ml = part_ml + (((size_t)tok * H + h0 + hh) * max_splits + split) * 2;
                ml[0] = u ? m1 : m0;
                ml[1] = u ? l1 : l0;
            }
        }
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int d = tid + c * ALS_THREADS;
        if (d < R) {
#pragma unroll
            for (int hh = 0; hh < ALS_HEADS; ++hh)
                if (hh < nh) part_o[(((size_t)tok * H + h0 + hh) * max_splits + split) * R + d] = acc[c][hh];
        }
    }
}

__global__ void __launch_bounds__(256)
attention_latent_join_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ positions,
                             const int* __restrict__ token_seq, int H, int R, int run, int max_splits, float* __restrict__ out,
                             long ldo) {
    const int tok = blockIdx.x, head = blockIdx.y;
    float* o = out + (size_t)tok * ldo + (size_t)head * R;
    if (token_seq[tok] < 0) {
        for (int d = threadIdx.x; d < R; d += 256) o[d] = 0.f;
        return;
    }
    const int runs = positions[tok] / run + 1;
    const float* ml = part_ml + ((size_t)tok * H + head) * max_splits * 2;
    float m = -INFINITY;
    for (int s = 0; s < runs; ++s) m = fmaxf(m, ml[2 * s]);
    float l = 0.f;
    for (int s = 0; s < runs; ++s) l += expf(ml[2 * s] - m) * ml[2 * s + 1];
    const float inv = 1.f / l;
    const float* po = part_o + ((size_t)tok * H + head) * max_splits * R;
    for (int d = threadIdx.x; d < R; d += 256) {
        float a = 0.f;
        for (int s = 0; s < runs; ++s) a = fmaf(expf(ml[2 * s] - m), po[(size_t)s * R + d], a);
        o[d] = a * inv;
    }
}

// bytes of LDS the split kernel needs for these sizes, and the pitch of a key row in it (32-bit words, odd)
static void als_layout(int R, int DR, int elem, int& row_words, size_t& lds) {
    const int words = (R + DR) * elem / 4;
    row_words = words | 1;
    lds = (size_t)ALS_HEADS * (R + DR) * 4 + (size_t)ALS_TILE * row_words * 4 + (size_t)ALS_TILE * ALS_HEADS * 4 + ALS_HEADS * 4;
}

// positions of a run: short runs while that keeps their number small (a workgroup's tiles follow one another,
// so few tiles a workgroup and many workgroups is what a step of few rows wants)
static int als_run(int max_context) { return max_context <= 8192 ? 64 : (max_context <= 32768 ? 256 : 1024); }

// floats of scratch for n rows whose contexts reach max_context positions: (weighted sums, maxima and sums)
extern "C" long mv_attention_latent_split_workspace(int n, int H, int R, int max_context) {
    const int run = als_run(max_context);
    const long runs = (max_context + run - 1) / run;
    return (long)n * H * runs * (R + 2);
}

// returns 2 (nothing done) when the sizes are not served: the caller takes the general kernel
extern "C" int mv_attention_latent_split(const float* q, long ldq, float* out, long ldo, const void* pages, const int* block_table,
                                         int bt_width, int page_size, const int* positions, const int* token_seq, int n, int H,
                                         int R, int DR, float scale, int max_context, float* work, long work_floats, int dtype,
                                         hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && R > 0 && DR >= 0 && max_context > 0, "attention_latent_split: bad sizes n=%d H=%d R=%d DR=%d", n, H, R, DR);
    const int elem = (int)mv_dtype_size(dtype);
    int row_words = 0;
    size_t lds = 0;
    als_layout(R, DR, elem, row_words, lds);
    if (((R + DR) * elem) % 16 != 0 || ((uintptr_t)pages % 16) != 0 || R > 2 * ALS_THREADS || lds > 64 * 1024
        || ALS_TILE * ((R + DR) * elem / 16) > ALS_MAX_VEC * ALS_THREADS) return 2;
    MV_REQUIRE(page_size > 0 && bt_width > 0 && ldq >= (long)H * (R + DR) && ldo >= (long)H * R, "attention_latent_split: pitches too small");
    MV_REQUIRE(q && out && pages && block_table && positions && token_seq && work, "attention_latent_split: missing operand");
    const int run = als_run(max_context);
    const int runs = (max_context + run - 1) / run;
    MV_REQUIRE(work_floats >= mv_attention_latent_split_workspace(n, H, R, max_context) && runs <= 65535,
               "attention_latent_split: scratch of %ld floats is too small", work_floats);
    if (n == 0) return 0;
    float* part_o = work;
    float* part_ml = work + (size_t)n * H * runs * R;
    dim3 grid(n, (H + ALS_HEADS - 1) / ALS_HEADS, runs);
    MV_DISPATCH_T(dtype, "attention_latent_split",
                  hipLaunchKernelGGL(attention_latent_split_kernel<T>, grid, dim3(ALS_THREADS), lds, stream, q, ldq, (const T*)pages,
                                     block_table, bt_width, page_size, positions, token_seq, H, R, DR, scale, row_words, run, runs,
                                     part_o, part_ml));
    if (mv_check_launch("attention_latent_split")) return 1;
    hipLaunchKernelGGL(attention_latent_join_kernel, dim3(n, H), dim3(256), 0, stream, part_o, part_ml, positions, token_seq, H, R,
                       run, runs, out, ldo);
    return mv_check_launch("attention_latent_join");
}


#ifdef MV_WITH_BF16
// ---------------------------------------------------------------------------------------
// Attention for steps with prompt portions (bfloat16, MFMA). One wave per (row, group of 16 heads): the heads of a row
// are the 16 rows of the first operand, since they all read the same key rows. Keys are walked 32 at a time from
// position 0:   S = Q K^T (NQ products of 16 x 16 x 32 for each half of the block, key rows straight from the pages),
// a running maximum and sum per head in float, P rounded to bfloat16 and turned from "a lane holds a key's column" to
// "a lane holds a head's row" through the wave's own 1 KB of LDS,   O += P V with V from the pages that hold the
// latents slot-contiguous (a lane's eight keys are eight neighbouring slots of one page: page_size % 8 == 0).
// Keys behind the row's position are masked in S and zeroed in V (their slots may hold anything).
// v_mfma_f32_16x16x32_bf16: lane l holds row l % 16 of the first operand (k = 8 (l / 16) .. + 7), column l % 16 of the
// second, and column l % 16 of rows 4 (l / 16) .. + 3 of the result.
// ---------------------------------------------------------------------------------------
typedef __bf16 alm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float alm_f4 __attribute__((ext_vector_type(4)));
union AlmFrag {
    uint4 u;
    alm_bf16x8 v;
    uint16_t h[8];
};

__device__ __forceinline__ float alm_row16_max(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float alm_row16_sum(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

template <int NQ, int NR>
__global__ void __launch_bounds__(256)
attention_latent_mfma_kernel(const float* __restrict__ q, long ldq, float* __restrict__ out, long ldo, const bf16* __restrict__ pages,
                             const bf16* __restrict__ pages_t, const int* __restrict__ block_table, int bt_width, int page_size,
                             const int* __restrict__ positions, const int* __restrict__ token_seq, int n, int H, float scale) {
    constexpr int DK = NQ * 32, R = NR * 16;
    __shared__ __attribute__((aligned(16))) uint16_t pl[4][16][40];          // a wave's P: [head][key], rows 80 bytes apart
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int tok = blockIdx.x * 4 + wave, h0 = blockIdx.y * 16;
    if (tok >= n) return;
    const int r = lane % 16, kq = lane / 16;
    const int nh = min(16, H - h0);
    const int seq = token_seq[tok];
    if (seq < 0) {
        for (int e = lane; e < nh * R; e += 64) out[(size_t)tok * ldo + (size_t)(h0 + e / R) * R + e % R] = 0.f;
        return;
    }
    const int pos = positions[tok];
    const int* bt = block_table + (size_t)seq * bt_width;
    AlmFrag qf[NQ];
#pragma unroll
    for (int c = 0; c < NQ; ++c) {
        if (r < nh) {
            const float* src = q + (size_t)tok * ldq + (size_t)(h0 + r) * DK + 32 * c + 8 * kq;
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[c].h[e] = f32_to_bf16_bits(src[e] * scale);
        } else {
            qf[c].u = uint4{0u, 0u, 0u, 0u};
        }
    }
    float m[4], l[4];
    alm_f4 acc[NR];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        m[i] = -INFINITY;
        l[i] = 0.f;
    }
#pragma unroll
    for (int t = 0; t < NR; ++t) acc[t] = alm_f4{0.f, 0.f, 0.f, 0.f};
    for (int kb = 0; kb <= pos; kb += 32) {
        alm_f4 s[2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            s[sub] = alm_f4{0.f, 0.f, 0.f, 0.f};
            const int key = kb + 16 * sub + r;
            const int kc = key <= pos ? key : pos;           // keys behind the row: some valid row, masked below
            const bf16* krow = pages + ((size_t)bt[kc / page_size] * page_size + kc % page_size) * DK + 8 * kq;
#pragma unroll
            for (int c = 0; c < NQ; ++c) {
                AlmFrag kf;
                kf.u = *reinterpret_cast<const uint4*>(krow + 32 * c);
                s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[c].v, kf.v, s[sub], 0, 0, 0);
            }
        }
        const bool ok0 = kb + r <= pos, ok1 = kb + 16 + r <= pos;
        float corr[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float a = ok0 ? s[0][i] : -INFINITY, b = ok1 ? s[1][i] : -INFINITY;
            const float m_new = fmaxf(m[i], alm_row16_max(fmaxf(a, b)));
            const float p0 = ok0 ? expf(a - m_new) : 0.f, p1 = ok1 ? expf(b - m_new) : 0.f;
            corr[i] = expf(m[i] - m_new);                    // first block: exp(-inf) = 0
            l[i] = l[i] * corr[i] + alm_row16_sum(p0 + p1);
            m[i] = m_new;
            pl[wave][4 * kq + i][r] = f32_to_bf16_bits(p0);
            pl[wave][4 * kq + i][16 + r] = f32_to_bf16_bits(p1);
        }
#pragma unroll
        for (int t = 0; t < NR; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][i] *= corr[i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        AlmFrag pf;
        pf.u = *reinterpret_cast<const uint4*>(&pl[wave][r][8 * kq]);
        const int key0 = kb + 8 * kq;                        // this lane's eight keys: one page's neighbouring slots
        const int live = min(8, pos - key0 + 1);             // how many of them the row sees (<= 0: none)
        // (every lane loads and multiplies, whatever it sees: a matrix instruction is the whole wave's. A lane that
        // sees none of its keys reads the row's own page instead and zeroes all eight.)
        const int keyc = live > 0 ? key0 : (pos / 8) * 8;
        const bf16* vbase = pages_t + ((size_t)bt[keyc / page_size] * R + r) * page_size + keyc % page_size;
#pragma unroll
        for (int t = 0; t < NR; ++t) {
            AlmFrag vf;
            vf.u = *reinterpret_cast<const uint4*>(vbase + (size_t)16 * t * page_size);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (e >= live) vf.h[e] = 0;
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf.v, vf.v, acc[t], 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int head = 4 * kq + i;
        if (head < nh) {
            const float inv = 1.f / l[i];
#pragma unroll
            for (int t = 0; t < NR; ++t) out[(size_t)tok * ldo + (size_t)(h0 + head) * R + 16 * t + r] = acc[t][i] * inv;
        }
    }
}

// returns 2 (nothing done) for sizes it does not serve: (R, DR) in (64, 32), (128, 32), (128, 64), (256, 64), pages
// whose size is a multiple of 8
extern "C" int mv_attention_latent_mfma(const float* q, long ldq, float* out, long ldo, const void* pages, const void* pages_t,
                                        const int* block_table, int bt_width, int page_size, const int* positions,
                                        const int* token_seq, int n, int H, int R, int DR, float scale, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && R > 0 && DR >= 0, "attention_latent_mfma: bad sizes n=%d H=%d R=%d DR=%d", n, H, R, DR);
    const bool served = (R == 64 && DR == 32) || (R == 128 && DR == 32) || (R == 128 && DR == 64) || (R == 256 && DR == 64);
    if (!served || page_size % 8 != 0 || !pages_t || ((uintptr_t)pages % 16) || ((uintptr_t)pages_t % 16)) return 2;
    MV_REQUIRE(bt_width > 0 && ldq >= (long)H * (R + DR) && ldo >= (long)H * R, "attention_latent_mfma: pitches too small");
    MV_REQUIRE(q && out && pages && block_table && positions && token_seq, "attention_latent_mfma: missing operand");
    if (n == 0) return 0;
    dim3 grid((n + 3) / 4, (H + 15) / 16);
#define ALM_LAUNCH(NQ, NR)                                                                                                 \
    hipLaunchKernelGGL((attention_latent_mfma_kernel<NQ, NR>), grid, dim3(256), 0, stream, q, ldq, out, ldo, (const bf16*)pages, \
                       (const bf16*)pages_t, block_table, bt_width, page_size, positions, token_seq, n, H, scale)
    if (R == 64) ALM_LAUNCH(3, 4);
    else if (R == 128 && DR == 32) ALM_LAUNCH(5, 8);
    else if (R == 128) ALM_LAUNCH(6, 8);
    else ALM_LAUNCH(10, 16);
#undef ALM_LAUNCH
    return mv_check_launch("attention_latent_mfma");
}
#endif

#ifdef MV_WITH_BF16
// ---------------------------------------------------------------------------------------
// The per-head maps for steps of many rows (bfloat16, MFMA): y[t][h] = W_h x[t][h] with w [H][OUT][IN], the inputs of an
// output row side by side (the other layout than head_linear's). A workgroup takes 64 rows, one head and 128 output
// columns; each of its four waves 16 rows x 128 columns (v_mfma_f32_16x16x32_bf16, operands straight from memory; lane
// l holds row l % 16 of x, column l % 16 of the weight, 8 inputs from 8 (l / 16)). IN must be a multiple of 32.
//   mode 0   x bfloat16 [n][H][IN + tail] -> y float [n][H][OUT + tail], the tail rotated by the row's position
//   mode 1   x float [n][H][IN] (rounded to bfloat16 as it is read) -> y bfloat16 [n][H * OUT], times sigmoid(gate)
// ---------------------------------------------------------------------------------------
template <int MODE>
__global__ void __launch_bounds__(256)
head_linear_mfma_kernel(const void* __restrict__ xv, long ldx, int ldx_head, const bf16* __restrict__ w, int IN, int OUT,
                        void* __restrict__ yv, long ldy, int ldy_head, int tail, const float* __restrict__ table,
                        const int* __restrict__ positions, const bf16* __restrict__ gate, long ldg, int gate_per_head,
                        const int* __restrict__ token_seq, int n) {
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int t0 = blockIdx.x * 64 + 16 * wave, head = blockIdx.y, n0 = blockIdx.z * 128;
    if (t0 >= n) return;                                     // (the whole wave: its 16 rows are past the end)
    const int r = lane % 16, kq = lane / 16;
    const int trow = min(t0 + r, n - 1);                     // rows past the end: the last row; never stored
    const bf16* wrow[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int col = min(n0 + 16 * s + r, OUT - 1);       // columns past the end: the last column; never stored
        wrow[s] = w + ((size_t)head * OUT + col) * IN + 8 * kq;
    }
    alm_f4 acc[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) acc[s] = alm_f4{0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < IN; k0 += 32) {
        AlmFrag fa;
        if (MODE == 0) {
            const bf16* x = (const bf16*)xv + (size_t)trow * ldx + (size_t)head * ldx_head + k0 + 8 * kq;
            if ((((uintptr_t)x) & 15) == 0) {
                fa.u = *reinterpret_cast<const uint4*>(x);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) fa.h[e] = x[e].bits;
            }
        } else {
            const float* x = (const float*)xv + (size_t)trow * ldx + (size_t)head * ldx_head + k0 + 8 * kq;
#pragma unroll
            for (int e = 0; e < 8; ++e) fa.h[e] = f32_to_bf16_bits(x[e]);
        }
        AlmFrag fb[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) fb[s].u = *reinterpret_cast<const uint4*>(wrow[s] + k0);
#pragma unroll
        for (int s = 0; s < 8; ++s) acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa.v, fb[s].v, acc[s], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int t = t0 + 4 * kq + i;
        if (t >= n) continue;
        const bool pad = token_seq[t] < 0;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int col = n0 + 16 * s + r;
            if (col >= OUT) continue;
            float v = pad ? 0.f : acc[s][i];
            if (MODE == 0) {
                ((float*)yv)[(size_t)t * ldy + (size_t)head * ldy_head + col] = v;
            } else {
                if (gate && !pad) v *= 1.f / (1.f + expf(-to_f(gate[(size_t)t * ldg + (gate_per_head ? (size_t)head : (size_t)head * OUT + col)])));
                ((bf16*)yv)[(size_t)t * ldy + (size_t)head * ldy_head + col] = from_f<bf16>(v);
            }
        }
    }
    if (MODE == 0 && blockIdx.z == 0 && tail > 0) {
        const int half = tail / 2;
        const int rows = min(16, n - t0);
        for (int e = lane; e < rows * half; e += 64) {
            const int t = t0 + e / half, i = e % half;
            const bf16* src = (const bf16*)xv + (size_t)t * ldx + (size_t)head * ldx_head + IN;
            float* dst = (float*)yv + (size_t)t * ldy + (size_t)head * ldy_head + OUT;
            if (token_seq[t] < 0) {
                dst[i] = 0.f;
                dst[half + i] = 0.f;
                continue;
            }
            const float* cs = table + (size_t)positions[t] * tail;
            const float a = to_f(src[i]), b = to_f(src[half + i]);
            dst[i] = a * cs[i] - b * cs[half + i];
            dst[half + i] = b * cs[i] + a * cs[half + i];
        }
    }
}

// returns 2 (nothing done) for sizes it does not serve
extern "C" int mv_head_linear_mfma(const void* x, long ldx, int ldx_head, const void* w, int n, int H, int IN, int OUT, void* y,
                                   long ldy, int ldy_head, int tail, const float* table, const int* positions, const void* gate,
                                   long ldg, int gate_per_head, const int* token_seq, int mode, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && IN > 0 && OUT > 0 && tail >= 0 && tail % 2 == 0, "head_linear_mfma: bad sizes");
    if (IN % 32 != 0 || ((uintptr_t)w % 16) != 0 || (mode == 1 && (ldx % 4 || ldx_head % 4))) return 2;
    MV_REQUIRE(ldx_head >= IN + tail && ldy_head >= OUT + (mode == 0 ? tail : 0) && x && w && y && token_seq && H <= 65535
               && (tail == 0 || (table && positions)) && (mode == 0 ? !gate : tail == 0), "head_linear_mfma: operands do not fit");
    if (n == 0) return 0;
    dim3 grid((n + 63) / 64, H, (OUT + 127) / 128);
    if (mode == 0)
        hipLaunchKernelGGL(head_linear_mfma_kernel<0>, grid, dim3(256), 0, stream, x, ldx, ldx_head, (const bf16*)w, IN, OUT, y, ldy,
                           ldy_head, tail, table, positions, (const bf16*)nullptr, 0L, 0, token_seq, n);
    else
        hipLaunchKernelGGL(head_linear_mfma_kernel<1>, grid, dim3(256), 0, stream, x, ldx, ldx_head, (const bf16*)w, IN, OUT, y, ldy,
                           ldy_head, 0, table, positions, (const bf16*)gate, ldg, gate_per_head, token_seq, n);
    return mv_check_launch("head_linear_mfma");
}
#endif
