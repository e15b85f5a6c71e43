// Kernels of mixers that carry a fixed-size state per request from token to token.
//
//   token shift      out[t] = h[t] + (h[t-1] - h[t]) * mix, the row in front of a request's first token
//                    of the step taken from the request's state, which then takes the step's last row
//   delta rule       S <- diag(w) S - (a*u)(u^T S) + k v^T,  o = S^T r,  one matrix S per head
//                    (prepare: w, a*u, u in float from the packed projection; scan: the recurrence
//                    over each request's tokens of the step; finish: per-head RMS, weight, gate)
//
// A step is any mix of requests: token_seq[t] names the request of row t (-1: a padding row),
// cu_seqlens[s] .. cu_seqlens[s+1] are the rows of request s, state_slots[s] its row of the state
// tensors. States are float (the shift's row has the activation type, it is a copy); decays,
// rates, unit keys and the recurrence are float whatever the activation type T is.
#include "dispatch.h"

// ---------------------------------------------------------------------------------------
// Token shift. One workgroup per row. The thread that serves column c of a request's first row
// is the only one that touches state[slot][c]: it reads the old value and then stores the
// request's last row of this step there.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(const T* __restrict__ h, long ldh, T* __restrict__ out, long ldo, WeightPtr mix,
                   T* __restrict__ state, const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                   const int* __restrict__ state_slots, int width) {
    const int t = blockIdx.x;
    const int seq = token_seq[t];
    T* o = out + (size_t)t * ldo;
    if (seq < 0) {
        for (int c = threadIdx.x; c < width; c += blockDim.x) o[c] = from_f<T>(0.f);
        return;
    }
    const int first = cu_seqlens[seq];
    const int last = cu_seqlens[seq + 1] - 1;
    const T* cur = h + (size_t)t * ldh;
    if (t > first) {
        const T* prev = cur - ldh;
        for (int c = threadIdx.x; c < width; c += blockDim.x) {
            const float x = to_f(cur[c]);
            o[c] = from_f<T>(fmaf(to_f(prev[c]) - x, mix.at(c), x));
        }
        return;
    }
    T* st = state + (size_t)state_slots[seq] * width;
    const T* tail = h + (size_t)last * ldh;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float x = to_f(cur[c]);
        const float p = to_f(st[c]);
        st[c] = tail[c];
        o[c] = from_f<T>(fmaf(p - x, mix.at(c), x));
    }
}

extern "C" int mv_token_shift(const void* h, long ldh, void* out, long ldo, const void* mix, int mix_dtype, void* state,
                              const int* token_seq, const int* cu_seqlens, const int* state_slots, int n, int width,
                              int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && width > 0 && ldh >= width && ldo >= width, "token_shift: bad sizes n=%d width=%d", n, width);
    MV_REQUIRE(h != out, "token_shift: a row reads the row in front of it, the output must be another buffer");
    MV_REQUIRE(mv_valid_dtype(mix_dtype) && mix && state && token_seq && cu_seqlens && state_slots,
               "token_shift: missing operand");
    if (n == 0) return 0;
    WeightPtr m{mix, mix_dtype};
    MV_DISPATCH_T(dtype, "token_shift",
                  hipLaunchKernelGGL(token_shift_kernel<T>, dim3(n), dim3(256), 0, stream, (const T*)h, ldh, (T*)out, ldo,
                                     m, (T*)state, token_seq, cu_seqlens, state_slots, width));
    return mv_check_launch("token_shift");
}

// ---------------------------------------------------------------------------------------
// Delta rule, prepare. The packed rows hold [r | k | v | g | a | w1] (H*D columns each, `rank` for
// w1) from column 0 on. For DP_TOKENS rows and 256 channels a workgroup, with c = (head, d):
//   coef[t][head][0][d] = w  = exp(-decay_rate * sigmoid(w0[c] + sum_j W2t[j][c] tanh(w1[t][j])))
//   coef[t][head][2][d] = u  = k[t][c] / sqrt(sum over the head of k^2 + key_eps)
//   coef[t][head][1][d] = a u, a = sigmoid(a[t][c] + a_bias[c])
//   coef[t][head][3][d] = k[t][c],  coef[t][head][4][d] = r[t][c]                (as floats)
// W2 comes transposed, [rank][H*D], so that neighbouring channels read neighbouring words; a row of
// it is read once for the workgroup's rows. The five vectors of a (token, head) lie side by side:
// the scan stages them with straight copies.
// ---------------------------------------------------------------------------------------
#define DP_TOKENS 8
#define DP_MAX_RANK 512
#define DP_MAX_HEADS 260      // heads that 256 channels can touch, for head sizes >= 1

__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

// NT sums over j in [j0, j1) of w2t[j][c] * th[t][j] (th rows `pitch` floats apart), the weight's element
// type known at compile time and eight loads in flight at a time; the additions run in the order of j
template <typename W, int NT>
__device__ __forceinline__ void decay_dots(const W* __restrict__ w2t_c, size_t inner, const float* th, int pitch, int j0,
                                           int j1, float (&acc)[NT]) {
    int j = j0;
    for (; j + 8 <= j1; j += 8) {
        float w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = to_f(w2t_c[(size_t)(j + e) * inner]);
#pragma unroll
        for (int e = 0; e < 8; ++e)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = fmaf(w[e], th[t * pitch + j + e], acc[t]);
    }
    for (; j < j1; ++j) {
        const float w = to_f(w2t_c[(size_t)j * inner]);
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = fmaf(w, th[t * pitch + j], acc[t]);
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const T* __restrict__ packed, long ld, int H, int D, int rank, WeightPtr w2t, WeightPtr w0,
                     WeightPtr a_bias, float decay_rate, float key_eps, float* __restrict__ coef, int n) {
    __shared__ float th[DP_TOKENS][DP_MAX_RANK];
    __shared__ float inv_len[DP_TOKENS][DP_MAX_HEADS];
    const int inner = H * D;
    const int t0 = blockIdx.x * DP_TOKENS;
    const int c0 = blockIdx.y * 256;
    const int nt = min(DP_TOKENS, n - t0);
    const int tid = threadIdx.x;
    const int lane = tid % MV_WAVE, wave = tid / MV_WAVE;
    for (int i = tid; i < nt * rank; i += 256) {
        const int tt = i / rank, j = i % rank;
        th[tt][j] = tanhf(to_f(packed[(size_t)(t0 + tt) * ld + 5 * (size_t)inner + j]));
    }
    // lengths of the keys of the heads these channels belong to, a wave per (row, head)
    const int h_lo = c0 / D;
    const int h_hi = min(H - 1, (c0 + 255) / D);
    const int nh = h_hi - h_lo + 1;
    for (int p = wave; p < nt * nh; p += 4) {
        const int tt = p / nh, hh = p % nh;
        const T* k = packed + (size_t)(t0 + tt) * ld + inner + (size_t)(h_lo + hh) * D;
        float ss = 0.f;
        for (int d = lane; d < D; d += MV_WAVE) {
            const float v = to_f(k[d]);
            ss = fmaf(v, v, ss);
        }
        ss = wave_sum(ss);
        if (lane == 0) inv_len[tt][hh] = 1.f / sqrtf(ss + key_eps);
    }
    __syncthreads();
    const int c = c0 + tid;
    if (c >= inner) return;
    float acc[DP_TOKENS];
#pragma unroll
    for (int tt = 0; tt < DP_TOKENS; ++tt) acc[tt] = 0.f;
    if (w2t.dtype == MV_F32)
        decay_dots<float, DP_TOKENS>((const float*)w2t.p + c, inner, &th[0][0], DP_MAX_RANK, 0, rank, acc);
    else
        decay_dots<bf16, DP_TOKENS>((const bf16*)w2t.p + c, inner, &th[0][0], DP_MAX_RANK, 0, rank, acc);
    const float b0 = w0.at(c), ab = a_bias.at(c);
    const int head = c / D, d = c % D;
    const int hh = head - h_lo;
    // (the rows' loads first, all of them, from clamped rows: under a condition each would wait on its own)
    float lk[DP_TOKENS], la[DP_TOKENS], lr[DP_TOKENS];
#pragma unroll
    for (int tt = 0; tt < DP_TOKENS; ++tt) {
        const T* p = packed + (size_t)(t0 + (tt < nt ? tt : 0)) * ld;
        lk[tt] = to_f(p[inner + c]);
        la[tt] = to_f(p[4 * (size_t)inner + c]);
        lr[tt] = to_f(p[c]);
    }
#pragma unroll
    for (int tt = 0; tt < DP_TOKENS; ++tt) {
        if (tt < nt) {
            const size_t row = (size_t)(t0 + tt);
            const float k = lk[tt];
            const float u = k * inv_len[tt][hh];
            const float rate = sigmoid_f(la[tt] + ab);
            float* o = coef + ((row * H + head) * 5) * (size_t)D + d;
            o[0] = expf(-decay_rate * sigmoid_f(acc[tt] + b0));
            o[D] = rate * u;
            o[2 * D] = u;
            o[3 * D] = k;
            o[4 * D] = lr[tt];
        }
    }
}

extern "C" int mv_delta_prepare(const void* packed, long ld, int n, int H, int D, int rank, const void* w2t, const void* w0,
                                const void* a_bias, int weight_dtype, float decay_rate, float key_eps, float* coef,
                                int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && D > 0 && rank > 0, "delta_prepare: bad sizes n=%d H=%d D=%d rank=%d", n, H, D, rank);
    MV_REQUIRE(rank <= DP_MAX_RANK, "delta_prepare: rank %d exceeds the supported maximum %d", rank, DP_MAX_RANK);
    MV_REQUIRE(ld >= 5L * H * D + rank, "delta_prepare: rows of %ld columns do not hold 5 x %d + %d", ld, H * D, rank);
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && w2t && w0 && a_bias && coef, "delta_prepare: missing operand");
    MV_REQUIRE(key_eps > 0.f, "delta_prepare: key_eps must be positive");
    if (n == 0) return 0;
    WeightPtr pw2{w2t, weight_dtype}, pw0{w0, weight_dtype}, pab{a_bias, weight_dtype};
    dim3 grid((n + DP_TOKENS - 1) / DP_TOKENS, (H * D + 255) / 256);
    MV_REQUIRE(grid.y <= 65535, "delta_prepare: too many channels");
    MV_DISPATCH_T(dtype, "delta_prepare",
                  hipLaunchKernelGGL(delta_prepare_kernel<T>, grid, dim3(256), 0, stream, (const T*)packed, ld, H, D,
                                     rank, pw2, pw0, pab, decay_rate, key_eps, coef, n));
    return mv_check_launch("delta_prepare");
}

// ---------------------------------------------------------------------------------------
// Delta rule, scan. A workgroup of 256 threads owns 256 / L value columns of one head of one
// request: L neighbouring lanes share a column j, each keeps R rows of S[:, j] in registers (rows
// sub*R .. sub*R+R-1, so D <= L*R; rows beyond D stay zero). Per token
//     read = sum_i u_i S_ij            (R multiply-adds a lane, then a sum over the L lanes)
//     S_ij = w_i S_ij - (a u)_i read + k_i v_j ;   o_j = sum_i r_i S_ij
// The per-token vectors w, a*u, u, k, r (the same for every column) and v are staged in LDS, a run of
// tokens at a time, in two buffers: the next run's loads from memory are in flight while this run
// is computed, and a token's vectors come from LDS into registers while the token before it is
// computed. The request's state is read at the start and written at the end.
// ---------------------------------------------------------------------------------------

// the sum of a value over the L lanes that share a column (L = 4, 8 or 16 neighbouring lanes of a row
// of 16): exchanges inside the row by data-parallel moves; every lane ends with the sum
template <int L>
__device__ __forceinline__ float lanes_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad [2,3,0,1]
    if constexpr (L >= 8)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // mirror of 8
    if constexpr (L >= 16)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // mirror of 16
    return v;
}

template <int R>
struct DeltaTokenRegs {
    float w[R], au[R], u[R], k[R], r[R], v;
};

template <int R, int DPAD>
__device__ __forceinline__ void delta_read_token(DeltaTokenRegs<R>& t, const float* vec, const float* vals, int sub, int col) {
    // vec: [5][DPAD] of one token; vals: the token's value columns of this workgroup
    const float* p = vec + sub * R;
#pragma unroll
    for (int e = 0; e < R; ++e) {
        t.w[e] = p[e];
        t.au[e] = p[DPAD + e];
        t.u[e] = p[2 * DPAD + e];
        t.k[e] = p[3 * DPAD + e];
        t.r[e] = p[4 * DPAD + e];
    }
    t.v = vals[col];
}

template <int R, int L>
__device__ __forceinline__ float delta_update(float (&s)[R], const DeltaTokenRegs<R>& t) {
    float read = 0.f;
#pragma unroll
    for (int e = 0; e < R; ++e) read = fmaf(t.u[e], s[e], read);
    read = lanes_sum<L>(read);
    float o = 0.f;
#pragma unroll
    for (int e = 0; e < R; ++e) {
        const float x = fmaf(t.w[e], s[e], fmaf(t.k[e], t.v, -t.au[e] * read));
        s[e] = x;
        o = fmaf(t.r[e], x, o);
    }
    return lanes_sum<L>(o);
}

// a lane's R rows of its column, between registers and the column's D floats in memory (rows
// sub*R .. sub*R+R-1; rows beyond D are zero and are not stored)
template <int R, bool STORE>
__device__ __forceinline__ void delta_state_io(float (&s)[R], float* column, int sub, int D, bool live) {
    const int i0 = sub * R;
    if ((D & 3) == 0) {
#pragma unroll
        for (int e = 0; e < R; e += 4) {
            const bool ok = live && i0 + e < D;
            float4* p = reinterpret_cast<float4*>(column + (i0 + e < D ? i0 + e : 0));
            if constexpr (STORE) {
                if (ok) *p = float4{s[e], s[e + 1], s[e + 2], s[e + 3]};
            } else {
                const float4 v = *p;                  // always issued (a valid address either way), dropped where it does not count
                s[e] = ok ? v.x : 0.f; s[e + 1] = ok ? v.y : 0.f; s[e + 2] = ok ? v.z : 0.f; s[e + 3] = ok ? v.w : 0.f;
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < R; ++e) {
            const bool ok = live && i0 + e < D;
            if constexpr (STORE) {
                if (ok) column[i0 + e] = s[e];
            } else {
                const float v = column[i0 + e < D ? i0 + e : 0];
                s[e] = ok ? v : 0.f;
            }
        }
    }
}

// V4: the head size is a multiple of four, so the staged vectors come in 16 bytes a lane: a run of tokens
// is 5 loads a thread instead of 20, and it is the number of load instructions, not their bytes, that a
// workgroup waits for here (measured on one prompt of 2,048 tokens, 16 heads of 64: 1,034 us with 4-byte
// loads, 442 us with 16-byte loads, 353 us with no loads at all).
template <typename T, int R, int L, bool V4>
__global__ void __launch_bounds__(256)
delta_scan_kernel(const T* __restrict__ packed, long ld, const float* __restrict__ coef, float* __restrict__ state,
                  const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots, int H, int D,
                  float* __restrict__ out, int n) {
    constexpr int DPAD = L * R;                     // padded key size
    constexpr int COLS = 256 / L;                   // value columns of a workgroup
    constexpr int TT = DPAD > 128 ? 4 : (DPAD > 64 ? 8 : 16);          // tokens staged at a time
    constexpr int NVEC = (TT * 5 * DPAD + 255) / 256;                   // staged words a thread brings in
    constexpr int NVAL = (TT * COLS + 255) / 256;
    __shared__ __attribute__((aligned(16))) float sv[2][TT][5][DPAD];
    __shared__ float svv[2][TT][COLS];
    const int seq = blockIdx.x, head = blockIdx.y, j0 = blockIdx.z * COLS;
    const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
    if (end <= begin) return;
    const int tid = threadIdx.x;
    const int sub = tid % L;
    const int col = tid / L;
    const int j = j0 + col;
    const bool live = j < D;
    const int inner = H * D;
    // the state of a head is stored column by column, S[j][i]: a lane's rows are neighbours in memory
    float* S = state + ((size_t)state_slots[seq] * H + head) * (size_t)D * D + (size_t)(live ? j : 0) * D;
    float s[R];
    delta_state_io<R, false>(s, S, sub, D, live);
    // a run of tokens from memory into registers, and from there into an LDS buffer
    constexpr int NV4 = (TT * 5 * DPAD / 4 + 255) / 256;
    float gv[V4 ? 1 : NVEC], gx[NVAL];
    float4 g4[V4 ? NV4 : 1];
    int fetched = 0;                                 // tokens of the run in flight
    auto fetch = [&](int base) {
        const int nt = min(TT, end - base);
        fetched = nt;
        if constexpr (V4) {
#pragma unroll
            for (int q = 0; q < NV4; ++q) {
                const int x = (tid + q * 256) * 4;
                const int tt = x / (5 * DPAD), rem = x % (5 * DPAD), a = rem / DPAD, i = rem % DPAD;
                // (always issued, from a clamped address; what does not count is dropped in `stash`)
                g4[q] = *reinterpret_cast<const float4*>(
                    coef + (((size_t)(base + (tt < nt ? tt : 0)) * H + head) * 5 + a) * D + (i < D ? i : 0));
            }
        } else
#pragma unroll
        for (int q = 0; q < NVEC; ++q) {
            const int x = tid + q * 256;
            const int tt = x / (5 * DPAD), rem = x % (5 * DPAD), a = rem / DPAD, i = rem % DPAD;
            // (the load is issued whatever the index, from a clamped address, and its value dropped where
            // it does not count: loads under a condition would each wait for memory on their own)
            const bool ok = tt < nt && i < D;
            const float l = coef[(((size_t)(base + (tt < nt ? tt : 0)) * H + head) * 5 + a) * D + (i < D ? i : 0)];
            gv[q] = ok ? l : 0.f;
        }
#pragma unroll
        for (int q = 0; q < NVAL; ++q) {
            const int x = tid + q * 256;
            const int tt = x / COLS, jj = x % COLS;
            const bool ok = tt < nt && j0 + jj < D;
            const float l = to_f(packed[(size_t)(base + (tt < nt ? tt : 0)) * ld + 2 * (size_t)inner + (size_t)head * D
                                        + (j0 + jj < D ? j0 + jj : 0)]);
            gx[q] = ok ? l : 0.f;
        }
    };
    auto stash = [&](int buf) {
        float* dst = &sv[buf][0][0][0];
        if constexpr (V4) {
#pragma unroll
            for (int q = 0; q < NV4; ++q) {
                const int x4 = tid + q * 256, x = x4 * 4;
                const int tt = x / (5 * DPAD), i = (x % (5 * DPAD)) % DPAD;
                if (x < TT * 5 * DPAD)
                    reinterpret_cast<float4*>(dst)[x4] = (tt < fetched && i < D) ? g4[q] : float4{0.f, 0.f, 0.f, 0.f};
            }
        } else
#pragma unroll
        for (int q = 0; q < NVEC; ++q) {
            const int x = tid + q * 256;
            if (x < TT * 5 * DPAD) dst[x] = gv[q];
        }
        float* dv = &svv[buf][0][0];
#pragma unroll
        for (int q = 0; q < NVAL; ++q) {
            const int x = tid + q * 256;
            if (x < TT * COLS) dv[x] = gx[q];
        }
    };
    fetch(begin);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int base = begin; base < end; base += TT, buf ^= 1) {
        const int nt = min(TT, end - base);
        const bool more = base + TT < end;
        if (more) fetch(base + TT);                  // in flight while this run is computed
        DeltaTokenRegs<R> ta, tb;
        delta_read_token<R, DPAD>(ta, &sv[buf][0][0][0], &svv[buf][0][0], sub, col);
        for (int tt = 0; tt < nt; tt += 2) {
            if (tt + 1 < nt) delta_read_token<R, DPAD>(tb, &sv[buf][tt + 1][0][0], &svv[buf][tt + 1][0], sub, col);
            const float o0 = delta_update<R, L>(s, ta);
            if (live && sub == 0) out[(size_t)(base + tt) * inner + (size_t)head * D + j] = o0;
            if (tt + 1 < nt) {
                if (tt + 2 < nt) delta_read_token<R, DPAD>(ta, &sv[buf][tt + 2][0][0], &svv[buf][tt + 2][0], sub, col);
                const float o1 = delta_update<R, L>(s, tb);
                if (live && sub == 0) out[(size_t)(base + tt + 1) * inner + (size_t)head * D + j] = o1;
            }
        }
        if (more) stash(buf ^ 1);                    // nobody reads that buffer: its run was computed before the last barrier
        __syncthreads();
    }
    delta_state_io<R, true>(s, S, sub, D, live);
}

// how a head of size D is dealt out: (rows a lane keeps, lanes a column); 0 when D is not served
static void delta_scan_shape(int D, int& R, int& L) {
    // few rows a lane and many lanes a column: a token costs the fewest instructions of the one wave a
    // SIMD runs, and a head is spread over the most workgroups
    if (D <= 16) { R = 4; L = 4; }
    else if (D <= 32) { R = 4; L = 8; }
    else if (D <= 64) { R = 4; L = 16; }
    else if (D <= 128) { R = 8; L = 16; }
    else { R = 16; L = 16; }
}

extern "C" int mv_delta_scan(const void* packed, long ld, const float* coef, float* state, const int* cu_seqlens,
                             const int* state_slots, int n_seqs, int n, int H, int D, float* out, int dtype,
                             hipStream_t stream) {
    MV_REQUIRE(n >= 0 && n_seqs >= 0 && H > 0 && D > 0, "delta_scan: bad sizes n=%d seqs=%d H=%d D=%d", n, n_seqs, H, D);
    MV_REQUIRE(D <= 256, "delta_scan: head size %d exceeds the supported maximum 256", D);
    MV_REQUIRE(ld >= 3L * H * D, "delta_scan: rows of %ld columns do not hold r, k and v of %d", ld, H * D);
    MV_REQUIRE(packed && coef && state && cu_seqlens && state_slots && out, "delta_scan: missing operand");
    int R = 0, L = 0;
    delta_scan_shape(D, R, L);
    const int cols = 256 / L;
    MV_REQUIRE(H <= 65535 && (D + cols - 1) / cols <= 65535, "delta_scan: too many heads");
    if (n == 0 || n_seqs == 0) return 0;
    dim3 grid(n_seqs, H, (D + cols - 1) / cols);
    const bool v4 = D % 4 == 0 && ((uintptr_t)coef % 16) == 0;
#define DS_LAUNCH(RR, LL)                                                                                                \
    if (v4) {                                                                                                            \
        MV_DISPATCH_T(dtype, "delta_scan",                                                                               \
                      hipLaunchKernelGGL((delta_scan_kernel<T, RR, LL, true>), grid, dim3(256), 0, stream, (const T*)packed, \
                                         ld, coef, state, cu_seqlens, state_slots, H, D, out, n))                        \
    } else {                                                                                                             \
        MV_DISPATCH_T(dtype, "delta_scan",                                                                               \
                      hipLaunchKernelGGL((delta_scan_kernel<T, RR, LL, false>), grid, dim3(256), 0, stream, (const T*)packed, \
                                         ld, coef, state, cu_seqlens, state_slots, H, D, out, n))                        \
    }
    if (R == 4 && L == 4) {
        DS_LAUNCH(4, 4);
    } else if (R == 4 && L == 8) {
        DS_LAUNCH(4, 8);
    } else if (R == 4 && L == 16) {
        DS_LAUNCH(4, 16);
    } else if (R == 8 && L == 16) {
        DS_LAUNCH(8, 16);
    } else {
        DS_LAUNCH(16, 16);
    }
#undef DS_LAUNCH
    return mv_check_launch("delta_scan");
}

// ---------------------------------------------------------------------------------------
// Delta rule, a step of single tokens: prepare, the recurrence and finish for one (row, head) in one
// workgroup. Row t is the one new token of request token_seq[t] (a padding row, < 0, gives zeros and
// touches no state). The head's columns are taken 256 / L at a time with the lanes laid out as in the
// scan; the additions are the scan's and the other kernels', in the same order, so a token computed here
// has the bits it would have as a prompt's last token.
// ---------------------------------------------------------------------------------------
template <typename T, int R, int L>
__global__ void __launch_bounds__(256)
delta_step_kernel(const T* __restrict__ packed, long ld, int H, int D, int rank, WeightPtr w2t, WeightPtr w0,
                  WeightPtr a_bias, float decay_rate, float key_eps, float* __restrict__ state,
                  const int* __restrict__ token_seq, const int* __restrict__ state_slots, WeightPtr norm_w, float eps,
                  T* __restrict__ out, long ldo) {
    constexpr int DPAD = L * R;
    constexpr int COLS = 256 / L;
    __shared__ float th[DP_MAX_RANK];
    __shared__ __attribute__((aligned(16))) float vec[5][DPAD];
    __shared__ float vals[DPAD];
    __shared__ float outs[DPAD];
    __shared__ float partial[256];               // [parts][D], parts * D <= 256
    __shared__ float red[8];
    const int t = blockIdx.x, head = blockIdx.y;
    const int tid = threadIdx.x;
    const int lane = tid % MV_WAVE, wave = tid / MV_WAVE;
    const int inner = H * D;
    const int seq = token_seq[t];
    T* y = out + (size_t)t * ldo + (size_t)head * D;
    if (seq < 0) {
        for (int d = tid; d < D; d += 256) y[d] = from_f<T>(0.f);
        return;
    }
    const T* p = packed + (size_t)t * ld;
    for (int j = tid; j < rank; j += 256) th[j] = tanhf(to_f(p[5 * (size_t)inner + j]));
    // the head's key and its length (the sum runs as the prepare kernel's: a wave over the head, lane by lane)
    if (wave == 0) {
        float ss = 0.f;
        for (int d = lane; d < D; d += MV_WAVE) {
            const float v = to_f(p[inner + head * D + d]);
            ss = fmaf(v, v, ss);
        }
        ss = wave_sum(ss);
        if (lane == 0) red[0] = 1.f / sqrtf(ss + key_eps);
    }
    __syncthreads();
    // the decay's small product, dealt out over all threads: thread (part, d) sums a run of j for channel d
    // (one part when D >= 256), the parts are added in order
    {
        const int parts = D >= 256 ? 1 : 256 / D;
        const int per = (rank + parts - 1) / parts;
        for (int x = tid; x < parts * D; x += 256) {
            const int part = x / D, d = x % D;
            const int cc = head * D + d;
            const int j0 = min(rank, part * per), j1 = min(rank, j0 + per);
            float acc[1] = {0.f};
            if (w2t.dtype == MV_F32)
                decay_dots<float, 1>((const float*)w2t.p + cc, inner, th, 0, j0, j1, acc);
            else
                decay_dots<bf16, 1>((const bf16*)w2t.p + cc, inner, th, 0, j0, j1, acc);
            partial[part * D + d] = acc[0];
        }
    }
    __syncthreads();
    for (int d = tid; d < DPAD; d += 256) {
        float w = 0.f, au = 0.f, u = 0.f, k = 0.f, r = 0.f, v = 0.f;
        if (d < D) {
            const int cc = head * D + d;
            const int parts = D >= 256 ? 1 : 256 / D;
            float acc = 0.f;
            for (int part = 0; part < parts; ++part) acc += partial[part * D + d];
            k = to_f(p[inner + cc]);
            u = k * red[0];
            au = sigmoid_f(to_f(p[4 * (size_t)inner + cc]) + a_bias.at(cc)) * u;
            w = expf(-decay_rate * sigmoid_f(acc + w0.at(cc)));
            r = to_f(p[cc]);
            v = to_f(p[2 * (size_t)inner + cc]);
        }
        vec[0][d] = w; vec[1][d] = au; vec[2][d] = u; vec[3][d] = k; vec[4][d] = r;
        vals[d] = v;
    }
    __syncthreads();
    const int sub = tid % L, col = tid / L;
    float* S0 = state + ((size_t)state_slots[seq] * H + head) * (size_t)D * D;
    // the next columns' state is asked for before this run of columns is stored: a load behind a store
    // would wait for the store to be acknowledged
    float s[R], s_next[R];
    delta_state_io<R, false>(s, S0 + (size_t)(col < D ? col : 0) * D, sub, D, col < D);
    for (int j0 = 0; j0 < D; j0 += COLS) {
        const int j = j0 + col;
        const bool live = j < D;
        float* S = S0 + (size_t)(live ? j : 0) * D;
        const int jn = j + COLS;
        if (j0 + COLS < D) delta_state_io<R, false>(s_next, S0 + (size_t)(jn < D ? jn : 0) * D, sub, D, jn < D);
        DeltaTokenRegs<R> tk;
        delta_read_token<R, DPAD>(tk, &vec[0][0], vals, sub, live ? j : 0);
        const float o = delta_update<R, L>(s, tk);
        delta_state_io<R, true>(s, S, sub, D, live);
        if (live && sub == 0) outs[j] = o;
#pragma unroll
        for (int e = 0; e < R; ++e) s[e] = s_next[e];
    }
    __syncthreads();
    // the head's root mean square (a wave over the head, lane by lane, as the finish kernel sums), weight, gate
    if (wave == 0) {
        float ss = 0.f;
        for (int d = lane; d < D; d += MV_WAVE) ss = fmaf(outs[d], outs[d], ss);
        ss = wave_sum(ss);
        if (lane == 0) red[1] = 1.f / sqrtf(ss / (float)D + eps);
    }
    __syncthreads();
    for (int d = tid; d < D; d += 256) {
        const int cc = head * D + d;
        y[d] = from_f<T>(outs[d] * red[1] * norm_w.at(cc) * sigmoid_f(to_f(p[3 * (size_t)inner + cc])));
    }
}

extern "C" int mv_delta_step(const void* packed, long ld, int n, int H, int D, int rank, const void* w2t, const void* w0,
                             const void* a_bias, const void* norm_w, int weight_dtype, float decay_rate, float key_eps,
                             float eps, float* state, const int* token_seq, const int* state_slots, void* out, long ldo,
                             int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && D > 0 && rank > 0, "delta_step: bad sizes n=%d H=%d D=%d rank=%d", n, H, D, rank);
    MV_REQUIRE(rank <= DP_MAX_RANK && D <= 256, "delta_step: rank %d or head size %d exceed what is served", rank, D);
    MV_REQUIRE(ld >= 5L * H * D + rank && ldo >= (long)H * D, "delta_step: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && packed && w2t && w0 && a_bias && norm_w && state && token_seq && state_slots && out,
               "delta_step: missing operand");
    MV_REQUIRE(key_eps > 0.f && eps > 0.f && H <= 65535, "delta_step: bad constants");
    if (n == 0) return 0;
    int R = 0, L = 0;
    delta_scan_shape(D, R, L);
    WeightPtr pw2{w2t, weight_dtype}, pw0{w0, weight_dtype}, pab{a_bias, weight_dtype}, pn{norm_w, weight_dtype};
    dim3 grid(n, H);
#define DT_LAUNCH(RR, LL)                                                                                                   \
    MV_DISPATCH_T(dtype, "delta_step",                                                                                      \
                  hipLaunchKernelGGL((delta_step_kernel<T, RR, LL>), grid, dim3(256), 0, stream, (const T*)packed, ld, H, D,  \
                                     rank, pw2, pw0, pab, decay_rate, key_eps, state, token_seq, state_slots, pn, eps,      \
                                     (T*)out, ldo))
    if (R == 4 && L == 4) {
        DT_LAUNCH(4, 4);
    } else if (R == 4 && L == 8) {
        DT_LAUNCH(4, 8);
    } else if (R == 4 && L == 16) {
        DT_LAUNCH(4, 16);
    } else if (R == 8 && L == 16) {
        DT_LAUNCH(8, 16);
    } else {
        DT_LAUNCH(16, 16);
    }
#undef DT_LAUNCH
    return mv_check_launch("delta_step");
}

// ---------------------------------------------------------------------------------------
// Delta rule, finish. One wave per (row, head):
//   y[t][c] = o[t][c] / sqrt(mean over the head of o^2 + eps) * weight[c] * sigmoid(g[t][c])
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
delta_finish_kernel(const float* __restrict__ raw, const T* __restrict__ packed, long ld, WeightPtr weight, int H, int D,
                    float eps, T* __restrict__ out, long ldo, int n) {
    const int lane = threadIdx.x % MV_WAVE;
    const long unit = (long)blockIdx.x * 4 + threadIdx.x / MV_WAVE;
    if (unit >= (long)n * H) return;
    const int t = (int)(unit / H), head = (int)(unit % H);
    const int inner = H * D;
    const float* o = raw + (size_t)t * inner + (size_t)head * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += MV_WAVE) ss = fmaf(o[d], o[d], ss);
    ss = wave_sum(ss);
    const float rinv = 1.f / sqrtf(ss / (float)D + eps);
    const T* g = packed + (size_t)t * ld + 3 * (size_t)inner + (size_t)head * D;
    T* y = out + (size_t)t * ldo + (size_t)head * D;
    for (int d = lane; d < D; d += MV_WAVE)
        y[d] = from_f<T>(o[d] * rinv * weight.at((size_t)head * D + d) * sigmoid_f(to_f(g[d])));
}

extern "C" int mv_delta_finish(const float* raw, const void* packed, long ld, const void* weight, int weight_dtype, int n,
                               int H, int D, float eps, void* out, long ldo, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && D > 0 && eps > 0.f, "delta_finish: bad sizes n=%d H=%d D=%d", n, H, D);
    MV_REQUIRE(ld >= 4L * H * D && ldo >= (long)H * D, "delta_finish: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && raw && packed && weight && out, "delta_finish: missing operand");
    if (n == 0) return 0;
    const long units = (long)n * H;
    WeightPtr w{weight, weight_dtype};
    MV_DISPATCH_T(dtype, "delta_finish",
                  hipLaunchKernelGGL(delta_finish_kernel<T>, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, raw,
                                     (const T*)packed, ld, w, H, D, eps, (T*)out, ldo, n));
    return mv_check_launch("delta_finish");
}

// =======================================================================================
// Mixers with a decayed matrix state per head and scalar gates: S is [key size DK][columns DV],
//     S <- a S;  u = b (v - [READ] S^T k);  S <- S + k u^T;  o = S^T q
// READ = true is the gated delta rule (a the decay, b the writing strength); READ = false, with a
// column of ones appended to the values, is the matrix memory of the mLSTM (a, b its stabilised
// forget and input gates, the extra column its normaliser). The per-token vectors come as floats:
//     qk    [n][G][2][DK]   query and key of each of the G key groups (head h reads group h / (H / G))
//     vals  [n][H][DV]      value columns
//     gates [n][H][4]       a, b, and two numbers the finishing kernel may use
// and the state as [slots][H][DV][DK], a head's matrix column by column. Prepare kernels make them
// from the packed projection rows, the scan runs the recurrence request by request, the finish
// kernel divides each head's output by its root mean square, applies weight and gate.
// =======================================================================================
#define MS_MAX_TAPS 16

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }
// log(sigmoid(z)) without overflow
__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One input of the causal convolution: row r of the step when the request's rows reach back that far,
// else the request's kept inputs (hist[slot][taps-1][C], the last one the newest).
template <typename T>
__device__ __forceinline__ float conv_input(const T* __restrict__ rows, long ld, const T* __restrict__ hist, int C, int taps,
                                            int first, int r, int c) {
    if (r >= first) return to_f(rows[(size_t)r * ld + c]);
    return to_f(hist[(size_t)(taps - 1 + (r - first)) * C + c]);
}

// ---------------------------------------------------------------------------------------
// Gated delta rule, prepare. Packed rows: [q (G*DK) | k (G*DK) | v (H*DV) | g (H*DV) | b (H) | a (H)].
// q, k and v pass a causal convolution over time per channel (taps[c][j], the last tap the current
// token's) and SiLU; q and k become unit vectors per group (q also times DK^-1/2);
// b = sigmoid(b), a = exp(-exp(A_log[h]) * softplus(a + dt_bias[h])). Workgroup (row, unit): units
// 0..G-1 make a group's q and k, units G..G+H-1 a head's values and gates.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(128)
gdelta_prepare_kernel(const T* __restrict__ packed, long ld, int H, int G, int DK, int DV, int taps, WeightPtr conv_w,
                      const T* __restrict__ conv_state, WeightPtr a_log, WeightPtr dt_bias, float unit_eps,
                      const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                      const int* __restrict__ state_slots, float* __restrict__ qk, float* __restrict__ vals,
                      float* __restrict__ gates) {
    __shared__ float scratch[17];
    const int t = blockIdx.x, unit = blockIdx.y, tid = threadIdx.x;
    const int seq = token_seq[t];
    if (seq < 0) return;                                   // a padding row: nobody reads its vectors
    const int C = 2 * G * DK + H * DV;
    const int first = cu_seqlens[seq];
    const T* hist = conv_state + (size_t)state_slots[seq] * (taps - 1) * C;
    auto conv = [&](int c) {
        float acc = 0.f;
        for (int j = 0; j < taps; ++j)
            acc = fmaf(conv_w.at((size_t)c * taps + j), conv_input(packed, ld, hist, C, taps, first, t - (taps - 1) + j, c), acc);
        return silu_f(acc);
    };
    if (unit < G) {
        for (int which = 0; which < 2; ++which) {
            const int c0 = which * G * DK + unit * DK;
            float* o = qk + (((size_t)t * G + unit) * 2 + which) * DK;
            float ss = 0.f;
            for (int d = tid; d < DK; d += 128) {
                const float x = conv(c0 + d);
                o[d] = x;                                  // (the thread that wrote it scales it below)
                ss = fmaf(x, x, ss);
            }
            ss = block_sum(ss, scratch);
            const float inv = (which == 0 ? 1.f / sqrtf((float)DK) : 1.f) / sqrtf(ss + unit_eps);
            for (int d = tid; d < DK; d += 128) o[d] *= inv;
        }
        return;
    }
    const int head = unit - G;
    const int c0 = 2 * G * DK + head * DV;
    float* o = vals + ((size_t)t * H + head) * DV;
    for (int d = tid; d < DV; d += 128) o[d] = conv(c0 + d);
    if (tid == 0) {
        const T* p = packed + (size_t)t * ld + 2 * (size_t)G * DK + 2 * (size_t)H * DV;
        float* g = gates + ((size_t)t * H + head) * 4;
        g[0] = expf(-expf(a_log.at(head)) * softplus_f(to_f(p[H + head]) + dt_bias.at(head)));
        g[1] = sigmoid_f(to_f(p[head]));
        g[2] = 0.f;
        g[3] = 0.f;
    }
}

// The convolution's kept inputs after the step: the last taps-1 inputs of each request, from the step's
// rows and, where the step brought fewer, from what was kept before. Thread (request, channel) reads all
// it needs before it writes, and no other thread touches its channel.
template <typename T>
__global__ void __launch_bounds__(256)
conv_state_kernel(const T* __restrict__ packed, long ld, int C, int taps, T* __restrict__ conv_state,
                  const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots) {
    const int seq = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    const int first = cu_seqlens[seq], end = cu_seqlens[seq + 1];
    if (end <= first || c >= C) return;
    T* hist = conv_state + (size_t)state_slots[seq] * (taps - 1) * C;
    T keep[MS_MAX_TAPS];
    for (int i = 0; i < taps - 1; ++i) {
        const int r = end - (taps - 1) + i;
        keep[i] = r >= first ? packed[(size_t)r * ld + c] : hist[(size_t)(taps - 1 + (r - first)) * C + c];
    }
    for (int i = 0; i < taps - 1; ++i) hist[(size_t)i * C + c] = keep[i];
}

// A causal convolution over time added to its own input, channel by channel:
//   out[t][c] = h[t][c] + sum_j w[c][j] * h[t - taps + 1 + j][c]      (the last tap multiplies h[t] itself)
// Rows in front of a request's first row of the step come from its kept inputs conv_state[slot][taps-1][C]
// (zeros at a request's start); conv_state_kernel moves them on afterwards. The sum starts from h[t] and takes
// the taps in order, so a row's value does not depend on where the step cut the request.
template <typename T>
__global__ void __launch_bounds__(256)
input_conv_kernel(const T* __restrict__ h, long ldh, T* __restrict__ out, long ldo, WeightPtr w, int taps,
                  const T* __restrict__ conv_state, const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                  const int* __restrict__ state_slots, int C) {
    const int t = blockIdx.x;
    const int seq = token_seq[t];
    T* o = out + (size_t)t * ldo;
    if (seq < 0) {
        for (int c = threadIdx.x; c < C; c += blockDim.x) o[c] = from_f<T>(0.f);
        return;
    }
    const int first = cu_seqlens[seq];
    const T* hist = taps > 1 ? conv_state + (size_t)state_slots[seq] * (taps - 1) * C : nullptr;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        float acc = to_f(h[(size_t)t * ldh + c]);
        for (int j = 0; j < taps; ++j) {
            const int r = t - (taps - 1) + j;
            const float x = r >= first ? to_f(h[(size_t)r * ldh + c]) : to_f(hist[(size_t)(taps - 1 + (r - first)) * C + c]);
            acc = fmaf(w.at((size_t)c * taps + j), x, acc);
        }
        o[c] = from_f<T>(acc);
    }
}

// The same for channels in chunks of eight (C a multiple of 8, rows 16-byte aligned), with the taps given tap by
// tap, wt[taps][C]: a thread takes eight neighbouring channels of one row, 16 bytes a load. The same sum in the
// same order as above.
template <typename T>
__global__ void __launch_bounds__(256)
input_conv_vec_kernel(const T* __restrict__ h, long ldh, T* __restrict__ out, long ldo, WeightPtr wt, int taps,
                      const T* __restrict__ conv_state, const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                      const int* __restrict__ state_slots, int C, int n) {
    const int per_row = C / 8;
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long)n * per_row) return;
    const int t = (int)(idx / per_row), c = (int)(idx % per_row) * 8;
    const int seq = token_seq[t];
    T* o = out + (size_t)t * ldo + c;
    float acc[8];
    if (seq < 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
        Vec8<T>::store(o, acc);
        return;
    }
    const int first = cu_seqlens[seq];
    const T* hist = taps > 1 ? conv_state + (size_t)state_slots[seq] * (taps - 1) * C : nullptr;
    Vec8<T>::load(h + (size_t)t * ldh + c, acc);
    for (int j = 0; j < taps; ++j) {
        const int r = t - (taps - 1) + j;
        float x[8], w[8];
        Vec8<T>::load(r >= first ? h + (size_t)r * ldh + c : hist + (size_t)(taps - 1 + (r - first)) * C + c, x);
        wt.at8((size_t)j * C + c, w);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = fmaf(w[e], x[e], acc[e]);
    }
    Vec8<T>::store(o, acc);
}

// h, ldh, out, ldo: [n][C] rows; w [C][taps] (wt: the same tap by tap, [taps][C], or null); conv_state [slots][taps-1][C] in
// the activation type (may be null with one tap)
extern "C" int mv_input_conv(const void* h, long ldh, void* out, long ldo, const void* w, const void* wt, int weight_dtype, int taps,
                             void* conv_state, const int* token_seq, const int* cu_seqlens, const int* state_slots, int n,
                             int n_seqs, int C, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && n_seqs >= 0 && C > 0 && ldh >= C && ldo >= C, "input_conv: bad sizes n=%d C=%d", n, C);
    MV_REQUIRE(taps >= 1 && taps <= MS_MAX_TAPS, "input_conv: %d taps, 1 to %d are served", taps, MS_MAX_TAPS);
    MV_REQUIRE(h != out, "input_conv: a row reads the rows in front of it, the output must be another buffer");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && h && out && w && (conv_state || taps == 1) && token_seq && cu_seqlens && state_slots,
               "input_conv: missing operand");
    MV_REQUIRE((C + 255) / 256 <= 65535, "input_conv: too many channels");
    if (n == 0) return 0;
    WeightPtr wp{w, weight_dtype};
    const size_t item = dtype == MV_F32 ? 4 : 2;
    const auto aligned = [](const void* p) { return ((uintptr_t)p % 16) == 0; };
    if (wt != nullptr && C % 8 == 0 && (ldh * item) % 16 == 0 && (ldo * item) % 16 == 0 && aligned(h) && aligned(out) && aligned(wt)
        && aligned(conv_state) && (long)n * (C / 8) / 256 + 1 < 0x7fffffffL) {
        const WeightPtr wtp{wt, weight_dtype};
        const unsigned blocks = (unsigned)(((long)n * (C / 8) + 255) / 256);
        MV_DISPATCH_T(dtype, "input_conv",
                      hipLaunchKernelGGL(input_conv_vec_kernel<T>, dim3(blocks), dim3(256), 0, stream, (const T*)h, ldh, (T*)out, ldo,
                                         wtp, taps, (const T*)conv_state, token_seq, cu_seqlens, state_slots, C, n));
    } else {
        MV_DISPATCH_T(dtype, "input_conv",
                      hipLaunchKernelGGL(input_conv_kernel<T>, dim3(n), dim3(256), 0, stream, (const T*)h, ldh, (T*)out, ldo, wp, taps,
                                         (const T*)conv_state, token_seq, cu_seqlens, state_slots, C));
    }
    if (mv_check_launch("input_conv")) return 1;
    if (taps > 1 && n_seqs > 0) {
        MV_DISPATCH_T(dtype, "conv_state",
                      hipLaunchKernelGGL(conv_state_kernel<T>, dim3(n_seqs, (unsigned)((C + 255) / 256)), dim3(256), 0, stream,
                                         (const T*)h, ldh, C, taps, (T*)conv_state, cu_seqlens, state_slots));
        return mv_check_launch("conv_state");
    }
    return 0;
}

extern "C" int mv_gdelta_prepare(const void* packed, long ld, int n, int n_seqs, int H, int G, int DK, int DV, int taps,
                                 const void* conv_w, const void* a_log, const void* dt_bias, int weight_dtype,
                                 void* conv_state, float unit_eps, const int* token_seq, const int* cu_seqlens,
                                 const int* state_slots, float* qk, float* vals, float* gates, int dtype,
                                 hipStream_t stream) {
    MV_REQUIRE(n >= 0 && n_seqs >= 0 && H > 0 && G > 0 && H % G == 0 && DK > 0 && DV > 0,
               "gdelta_prepare: bad sizes n=%d H=%d G=%d DK=%d DV=%d", n, H, G, DK, DV);
    MV_REQUIRE(taps >= 1 && taps <= MS_MAX_TAPS, "gdelta_prepare: %d taps, 1 to %d are served", taps, MS_MAX_TAPS);
    const long C = 2L * G * DK + (long)H * DV;
    MV_REQUIRE(ld >= C + (long)H * DV + 2L * H, "gdelta_prepare: rows of %ld columns are too short", ld);
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && packed && conv_w && a_log && dt_bias && (conv_state || taps == 1) && token_seq
               && cu_seqlens && state_slots && qk && vals && gates, "gdelta_prepare: missing operand");
    MV_REQUIRE(unit_eps > 0.f && G + H <= 65535 && (C + 255) / 256 <= 65535, "gdelta_prepare: bad constants");
    if (n == 0) return 0;
    WeightPtr cw{conv_w, weight_dtype}, al{a_log, weight_dtype}, db{dt_bias, weight_dtype};
    MV_DISPATCH_T(dtype, "gdelta_prepare",
                  hipLaunchKernelGGL(gdelta_prepare_kernel<T>, dim3(n, G + H), dim3(128), 0, stream, (const T*)packed, ld, H,
                                     G, DK, DV, taps, cw, (const T*)conv_state, al, db, unit_eps, token_seq, cu_seqlens,
                                     state_slots, qk, vals, gates));
    if (mv_check_launch("gdelta_prepare")) return 1;
    if (taps > 1 && n_seqs > 0) {
        MV_DISPATCH_T(dtype, "conv_state",
                      hipLaunchKernelGGL(conv_state_kernel<T>, dim3(n_seqs, (unsigned)((C + 255) / 256)), dim3(256), 0, stream,
                                         (const T*)packed, ld, (int)C, taps, (T*)conv_state, cu_seqlens, state_slots));
        return mv_check_launch("conv_state");
    }
    return 0;
}

// ---------------------------------------------------------------------------------------
// mLSTM, gates. Packed rows: [q (H*DK) | k (H*DK) | v (H*DV) | g (H*DV) | i (H) | f (H)]. With the log
// input gate i = cap tanh((i + i_bias) / cap), the log forget gate f = logsigmoid(cap tanh((f + f_bias) / cap))
// and the running maximum m (kept per request and head, 0 at the start):
//     m' = max(f + m, i);   a = exp(f + m - m');   b = exp(i - m');   gates = (a, b, exp(-m'), 0)
// One wave per (request, head) walks the request's rows 64 at a time: the gates' functions are computed
// a row a lane, the maximum itself in the order of the rows.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(64)
mlstm_gates_kernel(const T* __restrict__ packed, long ld, int H, long gate_off, WeightPtr i_bias, WeightPtr f_bias, float cap,
                   float* __restrict__ max_state, const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots,
                   float* __restrict__ gates) {
    const int seq = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int first = cu_seqlens[seq], end = cu_seqlens[seq + 1];
    if (end <= first) return;
    float* ms = max_state + (size_t)state_slots[seq] * H + head;
    float m = *ms;
    const float bi = i_bias.at(head), bf = f_bias.at(head);
    for (int base = first; base < end; base += 64) {
        const int t = base + lane;
        const bool live = t < end;
        const T* p = packed + (size_t)(live ? t : first) * ld + gate_off;
        const float gi = __fmul_rn(cap, tanhf((to_f(p[head]) + bi) / cap));      // (rounded here: never fused into a later sum)
        const float gf = logsigmoid_f(cap * tanhf((to_f(p[H + head]) + bf) / cap));
        // the maximum runs token by token, in the same order however the request was cut into steps: every lane
        // walks the 64 rows (their gates come by lane broadcasts), lane j keeps the values of row j
        float m_prev = m, m_new = m;
        const int nt = min(64, end - base);
        for (int j = 0; j < nt; ++j) {
            const float fj = __shfl(gf, j, 64), ij = __shfl(gi, j, 64);
            const float next = fmaxf(fj + m, ij);
            if (lane == j) {
                m_prev = m;
                m_new = next;
            }
            m = next;
        }
        if (live) {
            float* g = gates + ((size_t)t * H + head) * 4;
            g[0] = expf(gf + m_prev - m_new);
            g[1] = expf(gi - m_new);
            g[2] = expf(-m_new);
            g[3] = 0.f;
        }
    }
    if (lane == 0) *ms = m;
}

// mLSTM, the vectors of the scan: q * DK^-1/2 and k as floats, the values with a one behind them.
template <typename T>
__global__ void __launch_bounds__(128)
mlstm_prepare_kernel(const T* __restrict__ packed, long ld, int H, int DK, int DV, const int* __restrict__ token_seq,
                     float* __restrict__ qk, float* __restrict__ vals) {
    const int t = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    if (token_seq[t] < 0) return;
    const T* p = packed + (size_t)t * ld;
    float* o = qk + ((size_t)t * H + head) * 2 * DK;
    const float qs = 1.f / sqrtf((float)DK);
    for (int d = tid; d < DK; d += 128) {
        o[d] = to_f(p[(size_t)head * DK + d]) * qs;
        o[DK + d] = to_f(p[(size_t)(H + head) * DK + d]);
    }
    float* v = vals + ((size_t)t * H + head) * (DV + 1);
    for (int d = tid; d < DV; d += 128) v[d] = to_f(p[2 * (size_t)H * DK + (size_t)head * DV + d]);
    if (tid == 0) v[DV] = 1.f;
}

extern "C" int mv_mlstm_prepare(const void* packed, long ld, int n, int n_seqs, int H, int DK, int DV, const void* i_bias,
                                const void* f_bias, int weight_dtype, float cap, float* max_state, const int* token_seq,
                                const int* cu_seqlens, const int* state_slots, float* qk, float* vals, float* gates,
                                int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && n_seqs >= 0 && H > 0 && DK > 0 && DV > 0, "mlstm_prepare: bad sizes n=%d H=%d DK=%d DV=%d", n, H, DK, DV);
    const long gate_off = 2L * H * DK + 2L * H * DV;
    MV_REQUIRE(ld >= gate_off + 2L * H, "mlstm_prepare: rows of %ld columns are too short", ld);
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && packed && i_bias && f_bias && max_state && token_seq && cu_seqlens && state_slots
               && qk && vals && gates, "mlstm_prepare: missing operand");
    MV_REQUIRE(cap > 0.f && H <= 65535, "mlstm_prepare: bad constants");
    if (n == 0 || n_seqs == 0) return 0;
    WeightPtr ib{i_bias, weight_dtype}, fb{f_bias, weight_dtype};
    MV_DISPATCH_T(dtype, "mlstm_gates",
                  hipLaunchKernelGGL(mlstm_gates_kernel<T>, dim3(n_seqs, H), dim3(64), 0, stream, (const T*)packed, ld, H,
                                     gate_off, ib, fb, cap, max_state, cu_seqlens, state_slots, gates));
    if (mv_check_launch("mlstm_gates")) return 1;
    MV_DISPATCH_T(dtype, "mlstm_prepare",
                  hipLaunchKernelGGL(mlstm_prepare_kernel<T>, dim3(n, H), dim3(128), 0, stream, (const T*)packed, ld, H, DK, DV,
                                     token_seq, qk, vals));
    return mv_check_launch("mlstm_prepare");
}

// ---------------------------------------------------------------------------------------
// The scan. A workgroup of 256 threads owns 256 / L columns of one head of one request, L
// neighbouring lanes share a column and keep R of its DK rows each (as in the delta rule's scan
// above). The vectors of a run of tokens are staged in LDS; the additions of a token depend on
// nothing but the sizes, so a token computed alone has the bits it has inside a prompt.
// ---------------------------------------------------------------------------------------
// one token of one column: the lane's R rows of the column in s, its R channels of q and k; returns the column's output
template <int R, int L, bool READ>
__device__ __forceinline__ float state_update(float (&s)[R], const float (&q)[R], const float (&k)[R], float a, float b, float v) {
    float u = v;
    if constexpr (READ) {
        float read = 0.f;
#pragma unroll
        for (int e = 0; e < R; ++e) read = fmaf(k[e], s[e], read);
        u = v - a * lanes_sum<L>(read);
    }
    u *= b;
    float o = 0.f;
#pragma unroll
    for (int e = 0; e < R; ++e) {
        s[e] = fmaf(a, s[e], k[e] * u);
        o = fmaf(q[e], s[e], o);
    }
    return lanes_sum<L>(o);
}

template <int R, int L, bool READ>
__global__ void __launch_bounds__(256)
state_scan_kernel(const float* __restrict__ qk, const float* __restrict__ vals, const float* __restrict__ gates,
                  float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots, int H,
                  int G, int DK, int DV, float* __restrict__ out) {
    constexpr int DPAD = L * R;
    constexpr int COLS = 256 / L;
    constexpr int TT = DPAD > 128 ? 4 : (DPAD > 64 ? 8 : 16);
    __shared__ __attribute__((aligned(16))) float sv[TT][2][DPAD];
    __shared__ float sx[TT][COLS];
    __shared__ float sg[TT][2];
    const int seq = blockIdx.x, head = blockIdx.y, j0 = blockIdx.z * COLS;
    const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
    if (end <= begin) return;
    const int tid = threadIdx.x, sub = tid % L, col = tid / L;
    const int j = j0 + col;
    const bool live = j < DV;
    const int group = head / (H / G);
    float* S = state + (((size_t)state_slots[seq] * H + head) * DV + (live ? j : 0)) * (size_t)DK;
    float s[R];
    delta_state_io<R, false>(s, S, sub, DK, live);
    // a run of tokens comes from memory into registers while the run before it is computed, and from there into LDS
    // (loads are issued whatever the index, from clamped addresses, and dropped where they do not count)
    constexpr int NQ = (TT * 2 * DPAD + 255) / 256;
    constexpr int NV = (TT * COLS + 255) / 256;
    float gq[NQ], gx[NV], gg = 0.f;
    auto fetch = [&](int base) {
        const int nt = min(TT, end - base);
#pragma unroll
        for (int x = 0; x < NQ; ++x) {
            const int e = tid + x * 256;
            const int tt = e / (2 * DPAD), rem = e % (2 * DPAD), a = rem / DPAD, i = rem % DPAD;
            const bool ok = tt < nt && i < DK;
            const float l = qk[(((size_t)(base + (tt < nt ? tt : 0)) * G + group) * 2 + a) * DK + (i < DK ? i : 0)];
            gq[x] = ok ? l : 0.f;
        }
#pragma unroll
        for (int x = 0; x < NV; ++x) {
            const int e = tid + x * 256;
            const int tt = e / COLS, jj = e % COLS;
            const bool ok = tt < nt && j0 + jj < DV;
            const float l = vals[((size_t)(base + (tt < nt ? tt : 0)) * H + head) * DV + (j0 + jj < DV ? j0 + jj : 0)];
            gx[x] = ok ? l : 0.f;
        }
        if (tid < TT * 2) {
            const int tt = tid / 2;
            gg = gates[((size_t)(base + (tt < nt ? tt : 0)) * H + head) * 4 + tid % 2];
        }
    };
    fetch(begin);
    for (int base = begin; base < end; base += TT) {
        const int nt = min(TT, end - base);
        __syncthreads();                                   // the run before has been read
#pragma unroll
        for (int x = 0; x < NQ; ++x) {
            const int e = tid + x * 256;
            if (e < TT * 2 * DPAD) (&sv[0][0][0])[e] = gq[x];
        }
#pragma unroll
        for (int x = 0; x < NV; ++x) {
            const int e = tid + x * 256;
            if (e < TT * COLS) (&sx[0][0])[e] = gx[x];
        }
        if (tid < TT * 2) sg[tid / 2][tid % 2] = gg;
        if (base + TT < end) fetch(base + TT);             // in flight while this run is computed
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float a = sg[tt][0], b = sg[tt][1], v = sx[tt][col];
            float q[R], k[R];
#pragma unroll
            for (int e = 0; e < R; ++e) {
                q[e] = sv[tt][0][sub * R + e];
                k[e] = sv[tt][1][sub * R + e];
            }
            const float o = state_update<R, L, READ>(s, q, k, a, b, v);
            if (live && sub == 0) out[((size_t)(base + tt) * H + head) * DV + j] = o;
        }
    }
    delta_state_io<R, true>(s, S, sub, DK, live);
}

extern "C" int mv_state_scan(const float* qk, const float* vals, const float* gates, float* state, const int* cu_seqlens,
                             const int* state_slots, int n_seqs, int n, int H, int G, int DK, int DV, int read,
                             float* out, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && n_seqs >= 0 && H > 0 && G > 0 && H % G == 0 && DK > 0 && DV > 0,
               "state_scan: bad sizes n=%d seqs=%d H=%d G=%d DK=%d DV=%d", n, n_seqs, H, G, DK, DV);
    MV_REQUIRE(DK <= 256, "state_scan: key size %d exceeds the supported maximum 256", DK);
    MV_REQUIRE(qk && vals && gates && state && cu_seqlens && state_slots && out, "state_scan: missing operand");
    int R = 0, L = 0;
    delta_scan_shape(DK, R, L);
    const int cols = 256 / L;
    MV_REQUIRE(H <= 65535 && (DV + cols - 1) / cols <= 65535, "state_scan: too many heads or columns");
    if (n == 0 || n_seqs == 0) return 0;
    dim3 grid(n_seqs, H, (DV + cols - 1) / cols);
#define MS_LAUNCH(RR, LL)                                                                                                  \
    if (read)                                                                                                              \
        hipLaunchKernelGGL((state_scan_kernel<RR, LL, true>), grid, dim3(256), 0, stream, qk, vals, gates, state, cu_seqlens, \
                           state_slots, H, G, DK, DV, out);                                                                \
    else                                                                                                                   \
        hipLaunchKernelGGL((state_scan_kernel<RR, LL, false>), grid, dim3(256), 0, stream, qk, vals, gates, state,         \
                           cu_seqlens, state_slots, H, G, DK, DV, out);
    if (R == 4 && L == 4) {
        MS_LAUNCH(4, 4)
    } else if (R == 4 && L == 8) {
        MS_LAUNCH(4, 8)
    } else if (R == 4 && L == 16) {
        MS_LAUNCH(4, 16)
    } else if (R == 8 && L == 16) {
        MS_LAUNCH(8, 16)
    } else {
        MS_LAUNCH(16, 16)
    }
#undef MS_LAUNCH
    return mv_check_launch("state_scan");
}

// ---------------------------------------------------------------------------------------
// Finish. One wave per (row, head): the head's DV outputs (of DVS columns the scan wrote), with
// `normaliser` divided by max(|column DV|, gates[2]) + denom_eps first; then
//     y[d] = o[d] / sqrt(mean(o^2) + eps) * weight[shared ? d : head * DV + d] * act(g[head * DV + d])
// act = SiLU (silu_gate) or the logistic function; g at column g_off of the packed rows.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
state_finish_kernel(const float* __restrict__ raw, const float* __restrict__ gates, const T* __restrict__ packed, long ld,
                    long g_off, WeightPtr weight, int shared_weight, int silu_gate, int normaliser, float denom_eps, int H,
                    int DV, int DVS, float eps, const int* __restrict__ token_seq, T* __restrict__ out, long ldo, int n) {
    const int lane = threadIdx.x % MV_WAVE;
    const long unit = (long)blockIdx.x * 4 + threadIdx.x / MV_WAVE;
    if (unit >= (long)n * H) return;
    const int t = (int)(unit / H), head = (int)(unit % H);
    T* y = out + (size_t)t * ldo + (size_t)head * DV;
    if (token_seq[t] < 0) {
        for (int d = lane; d < DV; d += MV_WAVE) y[d] = from_f<T>(0.f);
        return;
    }
    const float* o = raw + ((size_t)t * H + head) * DVS;
    float scale = 1.f;
    if (normaliser) scale = 1.f / (fmaxf(fabsf(o[DV]), gates[((size_t)t * H + head) * 4 + 2]) + denom_eps);
    float ss = 0.f;
    for (int d = lane; d < DV; d += MV_WAVE) {
        const float x = o[d] * scale;
        ss = fmaf(x, x, ss);
    }
    ss = wave_sum(ss);
    const float rinv = scale / sqrtf(ss / (float)DV + eps);
    const T* g = packed + (size_t)t * ld + g_off + (size_t)head * DV;
    for (int d = lane; d < DV; d += MV_WAVE) {
        const float z = to_f(g[d]);
        const float act = silu_gate ? silu_f(z) : sigmoid_f(z);
        y[d] = from_f<T>(o[d] * rinv * weight.at(shared_weight ? d : (size_t)head * DV + d) * act);
    }
}

extern "C" int mv_state_finish(const float* raw, const float* gates, const void* packed, long ld, long g_off,
                               const void* weight, int weight_dtype, int shared_weight, int silu_gate, int normaliser,
                               float denom_eps, int n, int H, int DV, float eps, const int* token_seq, void* out, long ldo,
                               int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && DV > 0 && eps > 0.f, "state_finish: bad sizes n=%d H=%d DV=%d", n, H, DV);
    MV_REQUIRE(g_off >= 0 && ld >= g_off + (long)H * DV && ldo >= (long)H * DV, "state_finish: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && raw && gates && packed && weight && token_seq && out, "state_finish: missing operand");
    if (n == 0) return 0;
    const long units = (long)n * H;
    WeightPtr w{weight, weight_dtype};
    MV_DISPATCH_T(dtype, "state_finish",
                  hipLaunchKernelGGL(state_finish_kernel<T>, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, raw, gates,
                                     (const T*)packed, ld, g_off, w, shared_weight, silu_gate, normaliser, denom_eps, H, DV,
                                     DV + (normaliser ? 1 : 0), eps, token_seq, (T*)out, ldo, n));
    return mv_check_launch("state_finish");
}

// ---------------------------------------------------------------------------------------
// A step of single tokens: prepare, the recurrence and finish of one (row, head) in one workgroup, for both
// mixers (READ: the gated delta rule, whose convolution reads the request's kept inputs; they are advanced by
// conv_state_kernel afterwards, since the heads of a group share them. Otherwise the mLSTM, whose running
// maximum belongs to the head and is advanced here). Sums run in the order of the kernels above, so a token
// computed here has the bits it has as a prompt's last token.
// ---------------------------------------------------------------------------------------
struct StepArgs {
    const void* packed; long ld;
    int H, G, DK, DV, taps;
    WeightPtr conv_w, a_log, dt_bias, i_bias, f_bias, norm_w;
    const void* conv_state; float* max_state; float* state;
    float unit_eps, cap, denom_eps, eps;
    const int* token_seq; const int* state_slots;
    void* out; long ldo;
};

template <typename T, int R, int L, bool READ>
__global__ void __launch_bounds__(256)
state_step_kernel(StepArgs A) {
    constexpr int DPAD = L * R;
    constexpr int COLS = 256 / L;
    __shared__ float vq[DPAD], vk[DPAD];
    __shared__ float vals[260], outs[260];
    __shared__ float red[8];
    const int H = A.H, G = A.G, DK = A.DK, DV = A.DV;
    const int DVS = READ ? DV : DV + 1;                     // columns of the state
    const int t = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int lane = tid % MV_WAVE, wave = tid / MV_WAVE;
    const int seq = A.token_seq[t];
    T* y = (T*)A.out + (size_t)t * A.ldo + (size_t)head * DV;
    if (seq < 0) {
        for (int d = tid; d < DV; d += 256) y[d] = from_f<T>(0.f);
        return;
    }
    const int slot = A.state_slots[seq];
    const T* packed = (const T*)A.packed;
    const T* p = packed + (size_t)t * A.ld;
    long g_off;
    if constexpr (READ) {
        const int C = 2 * G * DK + H * DV, taps = A.taps;
        const int group = head / (H / G);
        const T* hist = (const T*)A.conv_state + (size_t)slot * (taps - 1) * C;
        // the row is its request's only one in the step: every earlier input comes from the kept ones
        auto conv = [&](int c) {
            float acc = 0.f;
            for (int j = 0; j < taps - 1; ++j) acc = fmaf(A.conv_w.at((size_t)c * taps + j), to_f(hist[(size_t)j * C + c]), acc);
            acc = fmaf(A.conv_w.at((size_t)c * taps + taps - 1), to_f(p[c]), acc);
            return silu_f(acc);
        };
        // as the prepare kernel sums: 128 threads over the channels, a wave's sum, the waves in order
        float sq = 0.f, sk = 0.f, xq[2] = {0.f, 0.f}, xk[2] = {0.f, 0.f};
        if (tid < 128) {
            int u = 0;
            for (int d = tid; d < DK; d += 128, ++u) {
                xq[u] = conv(group * DK + d);
                xk[u] = conv(G * DK + group * DK + d);
                sq = fmaf(xq[u], xq[u], sq);
                sk = fmaf(xk[u], xk[u], sk);
            }
            sq = wave_sum(sq);
            sk = wave_sum(sk);
            if (lane == 0) {
                red[wave] = sq;
                red[2 + wave] = sk;
            }
        }
        for (int d = tid; d < DV; d += 256) vals[d] = conv(2 * G * DK + head * DV + d);
        __syncthreads();
        if (tid < 128) {
            const float iq = (1.f / sqrtf((float)DK)) / sqrtf((0.f + red[0]) + red[1] + A.unit_eps);
            const float ik = 1.f / sqrtf((0.f + red[2]) + red[3] + A.unit_eps);
            int u = 0;
            for (int d = tid; d < DPAD; d += 128, ++u) {
                vq[d] = d < DK ? xq[u] * iq : 0.f;
                vk[d] = d < DK ? xk[u] * ik : 0.f;
            }
        }
        if (tid == 0) {
            const T* gp = p + C + (size_t)H * DV;
            red[4] = expf(-expf(A.a_log.at(head)) * softplus_f(to_f(gp[H + head]) + A.dt_bias.at(head)));
            red[5] = sigmoid_f(to_f(gp[head]));
            red[6] = 0.f;
        }
        g_off = C;
    } else {
        const float qs = 1.f / sqrtf((float)DK);
        for (int d = tid; d < DPAD; d += 256) {
            vq[d] = d < DK ? to_f(p[(size_t)head * DK + d]) * qs : 0.f;
            vk[d] = d < DK ? to_f(p[(size_t)(H + head) * DK + d]) : 0.f;
        }
        for (int d = tid; d < DV; d += 256) vals[d] = to_f(p[2 * (size_t)H * DK + (size_t)head * DV + d]);
        g_off = 2L * H * DK + (long)H * DV;
        if (tid == 0) {
            vals[DV] = 1.f;
            const T* gp = p + g_off + (size_t)H * DV;
            const float gi = __fmul_rn(A.cap, tanhf((to_f(gp[head]) + A.i_bias.at(head)) / A.cap));
            const float gf = logsigmoid_f(A.cap * tanhf((to_f(gp[H + head]) + A.f_bias.at(head)) / A.cap));
            float* ms = A.max_state + (size_t)slot * H + head;
            const float m = *ms;
            const float m_new = fmaxf(gf + m, gi);
            red[4] = expf(gf + m - m_new);
            red[5] = expf(gi - m_new);
            red[6] = expf(-m_new);
            *ms = m_new;
        }
    }
    __syncthreads();
    const float a = red[4], b = red[5];
    const int sub = tid % L, col = tid / L;
    float q[R], k[R];
#pragma unroll
    for (int e = 0; e < R; ++e) {
        q[e] = vq[sub * R + e];
        k[e] = vk[sub * R + e];
    }
    float* S0 = A.state + ((size_t)slot * H + head) * (size_t)DVS * DK;
    float s[R], s_next[R];
    delta_state_io<R, false>(s, S0 + (size_t)(col < DVS ? col : 0) * DK, sub, DK, col < DVS);
    for (int j0 = 0; j0 < DVS; j0 += COLS) {
        const int j = j0 + col;
        const bool live = j < DVS;
        const int jn = j + COLS;
        if (j0 + COLS < DVS) delta_state_io<R, false>(s_next, S0 + (size_t)(jn < DVS ? jn : 0) * DK, sub, DK, jn < DVS);
        const float o = state_update<R, L, READ>(s, q, k, a, b, vals[live ? j : 0]);
        delta_state_io<R, true>(s, S0 + (size_t)(live ? j : 0) * DK, sub, DK, live);
        if (live && sub == 0) outs[j] = o;
#pragma unroll
        for (int e = 0; e < R; ++e) s[e] = s_next[e];
    }
    __syncthreads();
    if (wave == 0) {
        float scale = 1.f;
        if constexpr (!READ) scale = 1.f / (fmaxf(fabsf(outs[DV]), red[6]) + A.denom_eps);
        float ss = 0.f;
        for (int d = lane; d < DV; d += MV_WAVE) {
            const float x = outs[d] * scale;
            ss = fmaf(x, x, ss);
        }
        ss = wave_sum(ss);
        if (lane == 0) red[7] = scale / sqrtf(ss / (float)DV + A.eps);
    }
    __syncthreads();
    const float rinv = red[7];
    const T* g = p + g_off + (size_t)head * DV;
    for (int d = tid; d < DV; d += 256) {
        const float z = to_f(g[d]);
        const float act = READ ? silu_f(z) : sigmoid_f(z);
        y[d] = from_f<T>(outs[d] * rinv * A.norm_w.at(READ ? d : (size_t)head * DV + d) * act);
    }
}

// mode 1: gated delta rule (conv_state, conv_w, a_log, dt_bias); mode 0: mLSTM (max_state, i_bias, f_bias, cap).
// Returns 2 (nothing done) for sizes it does not serve.
extern "C" int mv_state_step(int mode, const void* packed, long ld, int n, int n_seqs, int H, int G, int DK, int DV, int taps,
                             const void* conv_w, const void* a_log, const void* dt_bias, const void* i_bias,
                             const void* f_bias, const void* norm_w, int weight_dtype, void* conv_state, float* max_state,
                             float* state, float unit_eps, float cap, float denom_eps, float eps, const int* token_seq,
                             const int* cu_seqlens, const int* state_slots, void* out, long ldo, int dtype,
                             hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0 && DK > 0 && DV > 0, "state_step: bad sizes n=%d H=%d G=%d DK=%d DV=%d", n, H, G, DK, DV);
    if (DK > 256 || DV + 1 > 260 || (mode == 1 && (taps < 1 || taps > MS_MAX_TAPS))) return 2;
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && packed && norm_w && state && token_seq && cu_seqlens && state_slots && out,
               "state_step: missing operand");
    MV_REQUIRE(mode == 1 ? (conv_w && a_log && dt_bias && (conv_state || taps == 1) && unit_eps > 0.f)
                         : (i_bias && f_bias && max_state && cap > 0.f), "state_step: missing operand of the mode");
    MV_REQUIRE(eps > 0.f && H <= 65535 && ldo >= (long)H * DV, "state_step: bad constants");
    if (n == 0) return 0;
    StepArgs A;
    A.packed = packed; A.ld = ld; A.H = H; A.G = G; A.DK = DK; A.DV = DV; A.taps = taps;
    A.conv_w = WeightPtr{conv_w, weight_dtype}; A.a_log = WeightPtr{a_log, weight_dtype}; A.dt_bias = WeightPtr{dt_bias, weight_dtype};
    A.i_bias = WeightPtr{i_bias, weight_dtype}; A.f_bias = WeightPtr{f_bias, weight_dtype}; A.norm_w = WeightPtr{norm_w, weight_dtype};
    A.conv_state = conv_state; A.max_state = max_state; A.state = state;
    A.unit_eps = unit_eps; A.cap = cap; A.denom_eps = denom_eps; A.eps = eps;
    A.token_seq = token_seq; A.state_slots = state_slots; A.out = out; A.ldo = ldo;
    int R = 0, L = 0;
    delta_scan_shape(DK, R, L);
    dim3 grid(n, H);
#define SS_LAUNCH(RR, LL)                                                                                              \
    if (mode == 1) {                                                                                                   \
        MV_DISPATCH_T(dtype, "state_step", hipLaunchKernelGGL((state_step_kernel<T, RR, LL, true>), grid, dim3(256), 0, stream, A)) \
    } else {                                                                                                           \
        MV_DISPATCH_T(dtype, "state_step", hipLaunchKernelGGL((state_step_kernel<T, RR, LL, false>), grid, dim3(256), 0, stream, A)) \
    }
    if (R == 4 && L == 4) {
        SS_LAUNCH(4, 4)
    } else if (R == 4 && L == 8) {
        SS_LAUNCH(4, 8)
    } else if (R == 4 && L == 16) {
        SS_LAUNCH(4, 16)
    } else if (R == 8 && L == 16) {
        SS_LAUNCH(8, 16)
    } else {
        SS_LAUNCH(16, 16)
    }
#undef SS_LAUNCH
    if (mv_check_launch("state_step")) return 1;
    if (mode == 1 && taps > 1 && n_seqs > 0) {
        const long C = 2L * G * DK + (long)H * DV;
        MV_DISPATCH_T(dtype, "conv_state",
                      hipLaunchKernelGGL(conv_state_kernel<T>, dim3(n_seqs, (unsigned)((C + 255) / 256)), dim3(256), 0, stream,
                                         (const T*)packed, ld, (int)C, taps, (T*)conv_state, cu_seqlens, state_slots));
        return mv_check_launch("conv_state");
    }
    return 0;
}
