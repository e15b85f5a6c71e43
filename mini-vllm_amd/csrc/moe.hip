// Mixture of experts: the router's choice and the kernels around the experts' products.
//
//   moe_route          from float logits [n][E] (E = real experts + identity experts): scores = softmax
//                      over all E; choice = scores + correction; the experts form `groups` equal runs of
//                      neighbours, a group's worth is its largest choice, only experts of the `keep`
//                      worthiest groups can be chosen; the `top` largest choices are chosen; the weight of
//                      a chosen expert is its score divided by the chosen scores' sum (+ sum_eps).
//                      Leaves the weights dense, [n][E] with zeros for the others, and as lists
//                      (ids [n][top], weights [n][top], in the order chosen).
//                      Options (`flags`): MR_SIGMOID scores = sigmoid(logit) instead of the softmax;
//                      MR_WORTH_TOP2 a group's worth is the sum of its two largest choices (of its one
//                      choice when it has one); MR_RAW_WEIGHTS the weights are the chosen scores as they
//                      are, not divided by their sum.
//   moe_swiglu_scale   act[t][e][c] = weight[t][e] * silu(gate[t][e][c]) * up[t][e][c]: the gated pair of
//                      every expert with the router's weight applied before the one rounding, so that
//                      one product with all experts' down matrices side by side sums the chosen experts.
//                      With a `limit` > 0 the pair is the clamped one: g = min(gate, limit),
//                      u = clamp(up, -limit, limit), act = weight * g * sigmoid(slope * g) * (u + 1).
//   moe_identity_add   y[t] += (sum of the weights of the identity experts of t) * h[t]
#include "dispatch.h"

#define MR_MAX_E 1024
#define MR_SIGMOID 1
#define MR_WORTH_TOP2 2
#define MR_RAW_WEIGHTS 4

// the largest value over the wave and the smallest index that holds it (index INT_MAX: nothing left)
__device__ __forceinline__ void wave_argmax(float& best, int& at) {
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oa = __shfl_xor(at, o, 64);
        if (ob > best || (ob == best && oa < at)) {
            best = ob;
            at = oa;
        }
    }
}

__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ logits, long ld, int E, WeightPtr correction, int has_correction, int groups, int keep,
                 int top, float sum_eps, int flags, float* __restrict__ dense, int* __restrict__ ids, float* __restrict__ weights) {
    __shared__ float score[MR_MAX_E];
    __shared__ float choice[MR_MAX_E];
    __shared__ float worth[MR_MAX_E];          // of the groups
    __shared__ int open_group[MR_MAX_E];       // 1: its experts may be chosen
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * ld;
    float inv = 1.f;
    if (flags & MR_SIGMOID) {
        for (int e = lane; e < E; e += 64) score[e] = 1.f / (1.f + expf(-z[e]));
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += 64) {
            const float p = expf(z[e] - mx);
            score[e] = p;
            sum += p;
        }
        sum = wave_sum(sum);
        inv = 1.f / sum;
    }
    for (int e = lane; e < E; e += 64) {
        const float s = score[e] * inv;
        score[e] = s;
        choice[e] = s + (has_correction ? correction.at(e) : 0.f);
        dense[(size_t)t * E + e] = 0.f;
    }
    __syncthreads();
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
        float w = -INFINITY, second = -INFINITY;
        for (int i = 0; i < per; ++i) {
            const float c = choice[g * per + i];
            if (c > w) {
                second = w;
                w = c;
            } else if (c > second) {
                second = c;
            }
        }
        worth[g] = ((flags & MR_WORTH_TOP2) && per > 1) ? w + second : w;
        open_group[g] = keep >= groups ? 1 : 0;
    }
    __syncthreads();
    if (keep < groups) {
        for (int round = 0; round < keep; ++round) {          // the best group left, the first among equals
            float best = -INFINITY;
            int at = 0x7fffffff;
            for (int g = lane; g < groups; g += 64)
                if (!open_group[g] && (at == 0x7fffffff || worth[g] > best)) {
                    best = worth[g];
                    at = g;
                }
            wave_argmax(best, at);
            __syncthreads();
            if (lane == 0 && at != 0x7fffffff) open_group[at] = 1;
            __syncthreads();
        }
    }
    float picked_sum = 0.f;
    float my_w = 0.f;                                          // lane r holds the r-th chosen score (top <= 64)
    int my_id = -1;
    for (int round = 0; round < top; ++round) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < E; e += 64)
            if (open_group[e / per] && choice[e] != -INFINITY && (at == 0x7fffffff || choice[e] > best)) {
                best = choice[e];
                at = e;
            }
        wave_argmax(best, at);
        __syncthreads();
        if (at != 0x7fffffff) {
            const float s = score[at];
            picked_sum += s;
            if (lane == round) {
                my_w = s;
                my_id = at;
            }
            if (lane == 0) choice[at] = -INFINITY;            // taken
        }
        __syncthreads();
    }
    if (lane < top) {
        const float w = my_id >= 0 ? ((flags & MR_RAW_WEIGHTS) ? my_w : my_w / (picked_sum + sum_eps)) : 0.f;
        ids[(size_t)t * top + lane] = my_id;
        weights[(size_t)t * top + lane] = w;
        if (my_id >= 0) dense[(size_t)t * E + my_id] = w;
    }
}

extern "C" int mv_moe_route(const float* logits, long ld, int n, int E, const void* correction, int weight_dtype, int groups,
                            int keep, int top, float sum_eps, int flags, float* dense, int* ids, float* weights, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && E > 0 && E <= MR_MAX_E && ld >= E, "moe_route: bad sizes n=%d E=%d (at most %d)", n, E, MR_MAX_E);
    MV_REQUIRE(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups, "moe_route: %d groups of which %d stay do not fit %d experts",
               groups, keep, E);
    MV_REQUIRE(top >= 1 && top <= 64 && top <= (E / groups) * keep, "moe_route: top %d does not fit", top);
    MV_REQUIRE(logits && dense && ids && weights && (!correction || mv_valid_dtype(weight_dtype)), "moe_route: missing operand");
    if (n == 0) return 0;
    WeightPtr c{correction, weight_dtype};
    hipLaunchKernelGGL(moe_route_kernel, dim3(n), dim3(64), 0, stream, logits, ld, E, c, correction ? 1 : 0, groups, keep, top,
                       sum_eps, flags, dense, ids, weights);
    return mv_check_launch("moe_route");
}

// gate_up rows: [gate of expert 0 (F) | ... | gate of expert E-1 | up of expert 0 | ... | up of expert E-1 | gate of the
// shared expert (FS) | its up (FS)]; act rows [E][F] and behind them the shared expert's FS, whose weight is one.
// The weight of (row, expert) comes from `dense`, or, with a table, from the row's token id: 1 / top when
// table[token][0 .. top) names the expert, else zero (a token id outside the table chooses nothing).
struct MoeWeights {
    const float* dense;
    int ld_dense;
    const int* tokens;
    const int* table;
    int table_rows, top;
    __device__ __forceinline__ float of(long t, int e) const {
        if (table == nullptr) return dense[t * ld_dense + e];
        const int tok = tokens[t];
        if (tok < 0 || tok >= table_rows) return 0.f;
        float w = 0.f;
        for (int k = 0; k < top; ++k)
            if (table[(size_t)tok * top + k] == e) w += 1.f / (float)top;
        return w;
    }
};

__device__ __forceinline__ float moe_pair(float w, float g, float u, float limit, float slope) {
    if (limit > 0.f) {
        const float gc = fminf(g, limit), uc = fminf(fmaxf(u, -limit), limit);
        return w * (gc / (1.f + expf(-slope * gc))) * (uc + 1.f);
    }
    return w * (g / (1.f + expf(-g))) * u;
}

template <typename T>
__global__ void __launch_bounds__(256)
moe_swiglu_scale_kernel(const T* __restrict__ gate_up, long ld, MoeWeights mw, int E, int F, int FS,
                        T* __restrict__ act, long total, float limit, float slope) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long EF = (long)E * F;
    const long t = i / (EF + FS), c = i % (EF + FS);
    const bool shared = c >= EF;
    const float w = shared ? 1.f : mw.of(t, (int)(c / F));
    float v = 0.f;
    if (w != 0.f) {
        const long gi = shared ? 2 * EF + (c - EF) : c, ui = shared ? 2 * EF + FS + (c - EF) : EF + c;
        v = moe_pair(w, to_f(gate_up[t * ld + gi]), to_f(gate_up[t * ld + ui]), limit, slope);
    }
    act[t * (EF + FS) + c] = from_f<T>(v);
}

// The same, eight columns a thread (F and FS multiples of eight, rows 16-byte aligned): a thread's columns belong to
// one expert, so its weight is looked up once, and the pair of an expert that was not chosen is never loaded.
template <typename T>
__global__ void __launch_bounds__(256)
moe_swiglu_scale_vec_kernel(const T* __restrict__ gate_up, long ld, MoeWeights mw, int E, int F, int FS,
                            T* __restrict__ act, long total8, float limit, float slope) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total8) return;
    const long EF = (long)E * F;
    const long row8 = (EF + FS) / 8;
    const long t = i / row8, c = (i % row8) * 8;
    const bool shared = c >= EF;
    const float w = shared ? 1.f : mw.of(t, (int)(c / F));
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (w != 0.f) {
        const long gi = shared ? 2 * EF + (c - EF) : c, ui = shared ? 2 * EF + FS + (c - EF) : EF + c;
        float g[8], u[8];
        Vec8<T>::load(gate_up + t * ld + gi, g);
        Vec8<T>::load(gate_up + t * ld + ui, u);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = moe_pair(w, g[e], u[e], limit, slope);
    }
    Vec8<T>::store(act + t * (EF + FS) + c, v);
}

extern "C" int mv_moe_swiglu_scale(const void* gate_up, long ld, const float* dense, int ld_dense, int n, int E, int F, int FS,
                                   void* act, float limit, float slope, const int* tokens, const int* table, int table_rows,
                                   int top, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && E > 0 && F > 0 && FS >= 0 && ld >= 2L * E * F + 2L * FS, "moe_swiglu_scale: bad sizes n=%d E=%d F=%d shared=%d",
               n, E, F, FS);
    MV_REQUIRE(gate_up && act && (table ? (tokens && table_rows > 0 && top > 0) : (dense && ld_dense >= E)),
               "moe_swiglu_scale: missing operand");
    const long total = (long)n * ((long)E * F + FS);
    if (total == 0) return 0;
    MoeWeights mw{dense, ld_dense, tokens, table, table_rows, top};
    const size_t esz = mv_dtype_size(dtype);
    if (F % 8 == 0 && FS % 8 == 0 && (ld * esz) % 16 == 0 && ((uintptr_t)gate_up % 16) == 0 && ((uintptr_t)act % 16) == 0) {
        const long total8 = total / 8;
        MV_DISPATCH_T(dtype, "moe_swiglu_scale",
                      hipLaunchKernelGGL(moe_swiglu_scale_vec_kernel<T>, dim3((unsigned)((total8 + 255) / 256)), dim3(256), 0, stream,
                                         (const T*)gate_up, ld, mw, E, F, FS, (T*)act, total8, limit, slope));
        return mv_check_launch("moe_swiglu_scale");
    }
    MV_DISPATCH_T(dtype, "moe_swiglu_scale",
                  hipLaunchKernelGGL(moe_swiglu_scale_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                                     (const T*)gate_up, ld, mw, E, F, FS, (T*)act, total, limit, slope));
    return mv_check_launch("moe_swiglu_scale");
}

// Experts named by a table instead of a router: row t uses table[ids[t]][0 .. top), each with the weight 1 / top.
// Leaves what moe_route leaves: dense [n][ld_dense] (the first E columns; zeros for the others), ids and weights
// [n][top] in the table's order. A token id outside the table, and an entry outside the experts, choose nothing.
__global__ void __launch_bounds__(64)
moe_table_route_kernel(const int* __restrict__ tokens, const int* __restrict__ table, int rows, int E, int top,
                       float* __restrict__ dense, int ld_dense, int* __restrict__ ids, float* __restrict__ weights) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const int tok = tokens[t];
    const bool known = tok >= 0 && tok < rows;
    const float w = 1.f / (float)top;
    for (int e = lane; e < E; e += 64) {
        float v = 0.f;
        if (known)
            for (int k = 0; k < top; ++k)
                if (table[(size_t)tok * top + k] == e) v += w;
        dense[(size_t)t * ld_dense + e] = v;
    }
    for (int k = lane; k < top; k += 64) {
        const int e = known ? table[(size_t)tok * top + k] : -1;
        const bool ok = e >= 0 && e < E;
        ids[(size_t)t * top + k] = ok ? e : -1;
        weights[(size_t)t * top + k] = ok ? w : 0.f;
    }
}

extern "C" int mv_moe_table_route(const int* tokens, const int* table, int rows, int n, int E, int top, float* dense,
                                  int ld_dense, int* ids, float* weights, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && rows > 0 && E > 0 && top > 0 && top <= E && ld_dense >= E, "moe_table_route: bad sizes n=%d rows=%d E=%d top=%d",
               n, rows, E, top);
    MV_REQUIRE(tokens && table && dense && ids && weights, "moe_table_route: missing operand");
    if (n == 0) return 0;
    hipLaunchKernelGGL(moe_table_route_kernel, dim3(n), dim3(64), 0, stream, tokens, table, rows, E, top, dense, ld_dense, ids,
                       weights);
    return mv_check_launch("moe_table_route");
}

template <typename T>
__global__ void __launch_bounds__(256)
moe_identity_add_kernel(T* __restrict__ y, long ldy, const T* __restrict__ h, long ldh, const float* __restrict__ dense,
                        int ld_dense, int first, int count, int width, int set) {
    const int t = blockIdx.x;
    float w = 0.f;
    for (int e = 0; e < count; ++e) w += dense[(size_t)t * ld_dense + first + e];
    if (w == 0.f && !set) return;
    for (int c = threadIdx.x; c < width; c += 256) {
        T* p = y + (size_t)t * ldy + c;
        *p = from_f<T>((set ? 0.f : to_f(*p)) + w * to_f(h[(size_t)t * ldh + c]));
    }
}

// y[t] (+)= (dense[t][first .. first+count) summed) * h[t]; `set` writes instead of adding
extern "C" int mv_moe_identity_add(void* y, long ldy, const void* h, long ldh, const float* dense, int ld_dense, int first,
                                   int count, int n, int width, int set, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && width > 0 && ldy >= width && ldh >= width && first >= 0 && count >= 0 && ld_dense >= first + count,
               "moe_identity_add: bad sizes n=%d width=%d", n, width);
    MV_REQUIRE(y && h && dense, "moe_identity_add: missing operand");
    if (n == 0 || (count == 0 && !set)) return 0;
    MV_DISPATCH_T(dtype, "moe_identity_add",
                  hipLaunchKernelGGL(moe_identity_add_kernel<T>, dim3(n), dim3(256), 0, stream, (T*)y, ldy, (const T*)h, ldh, dense,
                                     ld_dense, first, count, width, set));
    return mv_check_launch("moe_identity_add");
}

// rows of the activation type: y <- y + x, added in float
template <typename T>
__global__ void __launch_bounds__(256)
add_rows_kernel(T* __restrict__ y, long ldy, const T* __restrict__ x, long ldx, int cols, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    T* p = y + (i / cols) * ldy + (i % cols);
    *p = from_f<T>(to_f(*p) + to_f(x[(i / cols) * ldx + (i % cols)]));
}

extern "C" int mv_add_rows(void* y, long ldy, const void* x, long ldx, int rows, int cols, int dtype, hipStream_t stream) {
    MV_REQUIRE(rows >= 0 && cols > 0 && ldy >= cols && ldx >= cols && y && x, "add_rows: bad sizes rows=%d cols=%d", rows, cols);
    const long total = (long)rows * cols;
    if (total == 0) return 0;
    MV_DISPATCH_T(dtype, "add_rows",
                  hipLaunchKernelGGL(add_rows_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, (T*)y, ldy,
                                     (const T*)x, ldx, cols, total));
    return mv_check_launch("add_rows");
}

// float rows in place: x <- x * factor
__global__ void scale_f32_kernel(float* __restrict__ x, long ld, int cols, long total, float factor) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    x[(i / cols) * ld + (i % cols)] *= factor;
}

extern "C" int mv_scale_f32(float* x, long ld, int rows, int cols, float factor, hipStream_t stream) {
    MV_REQUIRE(rows >= 0 && cols > 0 && ld >= cols && x, "scale: bad sizes rows=%d cols=%d", rows, cols);
    const long total = (long)rows * cols;
    if (total == 0) return 0;
    hipLaunchKernelGGL(scale_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, x, ld, cols, total, factor);
    return mv_check_launch("scale");
}

#ifdef MV_WITH_BF16
// =======================================================================================
// The experts' products over the chosen (token, expert) pairs only (bfloat16, MFMA).
//
//   moe_sort      counts the pairs of every expert, lays the pairs out expert by expert (`sorted`: pair
//                 indices, a pair is token * top + place) and cuts every expert's run into tiles of 64 rows
//                 (`tile_expert`, `tile_row0`, `tile_rows`; unused entries hold expert -1). Identity experts
//                 and pairs without an expert are left out. Within an expert the order of the pairs is
//                 whatever the counters gave; no result depends on it (a row's products read only its own row).
//   moe_gate_up   per tile and 128 columns: act[pair] = weight[pair] * silu(x W_gate^T) * (x W_up^T), the rows of x
//                 gathered through `sorted`, rounded once (with a `limit` > 0 the clamped pair of moe_swiglu_scale)
//   moe_down      per tile and 128 columns: out[pair] = act[pair] W_down^T as floats
//   moe_combine   y[token] = sum over its places (in order) of out[pair] + (identity weights) * x[token]
//
// A workgroup takes a tile and 128 columns; each of its four waves computes 16 rows x 128 columns (x 2 for gate and
// up) with v_mfma_f32_16x16x32_bf16: lane l holds row l % 16 of the first operand (8 values of k from 8 (l / 16))
// and column l % 16 of the second, and ends with column l % 16 of rows 4 (l / 16) .. + 3. The four waves read the
// same weight rows, which the caches serve; a weight is read once for 64 rows. K must be a multiple of 32 and rows
// 16-byte aligned.
// =======================================================================================
typedef __bf16 mg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mg_f4 __attribute__((ext_vector_type(4)));
union MgFrag {
    uint4 u;
    mg_bf16x8 v;
};
#define MG_ROWS 64             // rows of a tile: four waves of 16 rows each
#define MG_COLS 128            // columns of a workgroup (gate columns, with their up columns, when gated)

__global__ void __launch_bounds__(1024)
moe_sort_kernel(const int* __restrict__ ids, int n_pairs, int n_real, int max_tiles, int* __restrict__ sorted,
                int* __restrict__ tile_expert, int* __restrict__ tile_row0, int* __restrict__ tile_rows) {
    __shared__ int count[MR_MAX_E], offset[MR_MAX_E], cursor[MR_MAX_E];
    const int tid = threadIdx.x;
    for (int e = tid; e < n_real; e += 1024) {
        count[e] = 0;
        cursor[e] = 0;
    }
    __syncthreads();
    for (int p = tid; p < n_pairs; p += 1024) {
        const int e = ids[p];
        if (e >= 0 && e < n_real) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int off = 0, t = 0;
        for (int e = 0; e < n_real; ++e) {
            offset[e] = off;
            const int c = count[e];
            for (int r = 0; r < c && t < max_tiles; r += MG_ROWS, ++t) {
                tile_expert[t] = e;
                tile_row0[t] = off + r;
                tile_rows[t] = min(MG_ROWS, c - r);
            }
            off += c;
        }
        for (; t < max_tiles; ++t) tile_expert[t] = -1;
    }
    __syncthreads();
    for (int p = tid; p < n_pairs; p += 1024) {
        const int e = ids[p];
        if (e >= 0 && e < n_real) sorted[offset[e] + atomicAdd(&cursor[e], 1)] = p;
    }
}

// GATED: W holds [E gate blocks of F rows | E up blocks of F rows], K columns each (ldw = K); the output is the
// weighted activation. Otherwise W is [N rows][ldw] with the expert's K columns from column e * K (all down
// matrices side by side); the output is float.
template <bool GATED>
__global__ void __launch_bounds__(256)
moe_expert_product_kernel(const bf16* __restrict__ a, long lda, int a_by_token, const bf16* __restrict__ w, long ldw, int E, int N,
                          int K, const int* __restrict__ sorted, const int* __restrict__ tile_expert,
                          const int* __restrict__ tile_row0, const int* __restrict__ tile_rows, const float* __restrict__ weights,
                          int top, bf16* __restrict__ act, float* __restrict__ out, float limit, float slope) {
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int row0 = tile_row0[tile] + 16 * wave, nrows = tile_rows[tile] - 16 * wave;     // this wave's 16 rows
    if (nrows <= 0) return;
    const int r = lane % 16, kq = lane / 16;
    const int pair = r < nrows ? sorted[row0 + r] : -1;
    const bf16* arow = pair < 0 ? nullptr : a + (size_t)(a_by_token ? pair / top : pair) * lda;
    const int n0 = blockIdx.y * MG_COLS;
    constexpr int NS = MG_COLS / 16;
    const bf16* b0[NS];
    const bf16* b1[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int col = n0 + 16 * s + r;
        const int c = col < N ? col : N - 1;               // columns past the end: some column; never stored
        if (GATED) {
            b0[s] = w + ((size_t)e * N + c) * ldw;
            b1[s] = w + ((size_t)(E + e) * N + c) * ldw;
        } else {
            b0[s] = w + (size_t)c * ldw + (size_t)e * K;
            b1[s] = b0[s];
        }
    }
    mg_f4 acc0[NS], acc1[GATED ? NS : 1];
#pragma unroll
    for (int s = 0; s < NS; ++s) acc0[s] = mg_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < (GATED ? NS : 1); ++s) acc1[s] = mg_f4{0.f, 0.f, 0.f, 0.f};
    const uint4 zero = uint4{0u, 0u, 0u, 0u};
    for (int k0 = 0; k0 < K; k0 += 32) {
        const int kk = k0 + 8 * kq;
        MgFrag fa, fb[NS], fc[GATED ? NS : 1];
        fa.u = arow ? *reinterpret_cast<const uint4*>(arow + kk) : zero;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            fb[s].u = *reinterpret_cast<const uint4*>(b0[s] + kk);
            if (GATED) fc[s].u = *reinterpret_cast<const uint4*>(b1[s] + kk);
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            acc0[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa.v, fb[s].v, acc0[s], 0, 0, 0);
            if (GATED) acc1[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa.v, fc[s].v, acc1[s], 0, 0, 0);
        }
    }
#pragma unroll
    for (int idx = 0; idx < 4; ++idx) {
        const int i = 4 * kq + idx;
        if (i >= nrows) continue;
        const int p = sorted[row0 + i];
        const float wt = GATED ? weights[p] : 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int col = n0 + 16 * s + r;
            if (col >= N) continue;
            if (GATED) {
                const float g = acc0[s][idx], u = acc1[s][idx];
                float v;
                if (limit > 0.f) {          // the clamped pair, as in moe_swiglu_scale
                    const float gc = fminf(g, limit), uc = fminf(fmaxf(u, -limit), limit);
                    v = wt * (gc / (1.f + expf(-slope * gc))) * (uc + 1.f);
                } else {
                    v = wt * (g / (1.f + expf(-g))) * u;
                }
                act[(size_t)p * N + col] = from_f<bf16>(v);
            } else {
                out[(size_t)p * N + col] = acc0[s][idx];
            }
        }
    }
}

__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ out, const int* __restrict__ ids, int top, int n_real, const bf16* __restrict__ x,
                   long ldx, const float* __restrict__ dense, int ld_dense, int identity, bf16* __restrict__ y, long ldy, int width) {
    const int t = blockIdx.x;
    float idw = 0.f;
    for (int e = 0; e < identity; ++e) idw += dense[(size_t)t * ld_dense + n_real + e];
    for (int c = threadIdx.x; c < width; c += 256) {
        float v = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = ids[(size_t)t * top + k];
            if (e >= 0 && e < n_real) v += out[((size_t)t * top + k) * width + c];
        }
        if (idw != 0.f) v = fmaf(idw, to_f(x[(size_t)t * ldx + c]), v);
        y[(size_t)t * ldy + c] = from_f<bf16>(v);
    }
}

// ints of scratch: sorted pairs and the three tile tables; floats: the down products of every pair
extern "C" long mv_moe_grouped_ints(int n, int top, int n_real) { return (long)n * top + 3L * ((long)n * top / MG_ROWS + n_real + 1); }

// returns 2 (nothing done) for sizes it does not serve
extern "C" int mv_moe_grouped(const void* x, long ldx, int n, int hidden, const void* w_gate_up, const void* w_down, int n_real,
                              int identity, int F, const int* ids, const float* weights, int top, const float* dense,
                              int ld_dense, int* ints, void* act, float* out, void* y, long ldy, float limit, float slope,
                              hipStream_t stream) {
    MV_REQUIRE(n >= 0 && hidden > 0 && n_real > 0 && F > 0 && top > 0 && identity >= 0 && limit >= 0.f, "moe_grouped: bad sizes");
    if (hidden % 32 || F % 32 || ldx % 8 || ((uintptr_t)x % 16) || ((uintptr_t)w_gate_up % 16) || ((uintptr_t)w_down % 16)
        || ((uintptr_t)act % 16) || n_real > MR_MAX_E)
        return 2;
    MV_REQUIRE(x && w_gate_up && w_down && ids && weights && dense && ints && act && out && y && ld_dense >= n_real + identity
               && ldy >= hidden, "moe_grouped: missing operand");
    if (n == 0) return 0;
    const int n_pairs = n * top;
    const int max_tiles = n_pairs / MG_ROWS + n_real + 1;
    int* sorted = ints;
    int* tile_expert = ints + n_pairs;
    int* tile_row0 = tile_expert + max_tiles;
    int* tile_rows = tile_row0 + max_tiles;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, n_pairs, n_real, max_tiles, sorted, tile_expert,
                       tile_row0, tile_rows);
    if (mv_check_launch("moe_sort")) return 1;
    hipLaunchKernelGGL(moe_expert_product_kernel<true>, dim3(max_tiles, (F + MG_COLS - 1) / MG_COLS), dim3(256), 0, stream, (const bf16*)x, ldx,
                       1, (const bf16*)w_gate_up, (long)hidden, n_real, F, hidden, sorted, tile_expert, tile_row0, tile_rows,
                       weights, top, (bf16*)act, (float*)nullptr, limit, slope);
    if (mv_check_launch("moe_gate_up")) return 1;
    hipLaunchKernelGGL(moe_expert_product_kernel<false>, dim3(max_tiles, (hidden + MG_COLS - 1) / MG_COLS), dim3(256), 0, stream,
                       (const bf16*)act, (long)F, 0, (const bf16*)w_down, (long)n_real * F, n_real, hidden, F, sorted, tile_expert,
                       tile_row0, tile_rows, weights, top, (bf16*)nullptr, out, 0.f, 0.f);
    if (mv_check_launch("moe_down")) return 1;
    hipLaunchKernelGGL(moe_combine_kernel, dim3(n), dim3(256), 0, stream, out, ids, top, n_real, (const bf16*)x, ldx, dense,
                       ld_dense, identity, (bf16*)y, ldy, hidden);
    return mv_check_launch("moe_combine");
}
#endif
