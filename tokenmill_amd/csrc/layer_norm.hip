// Layer norm with weight and bias behind a gated, scaled residual add; a short causal convolution over time with
// per-request state; and the PolyNorm activation. Everything is computed in 32-bit and rounded once where stored.
//
//   tm_layer_norm      v = resid[r] + mult * y[r] * sigmoid(gate[r])    (gate null: no gate; y null: v = resid[r])
//                      resid[r] = v                                     (only with y, and only when every row is run)
//                      out[r] = (v - mean(v)) / sqrt(mean((v - mean(v))^2) + eps) * w + b      (out null: the add alone)
//                      rows != null: row rows[r] of resid, y and gate is read, nothing is written back, out row r.
//   tm_short_conv      out[t] = h[t] + sum_j w[:, j] * h[t - taps + 1 + j], the rows before a request's first row of the
//                      step taken from its state [taps - 1, width] (zeros at a sequence's start);
//   tm_short_conv_state  then the state becomes the last taps - 1 rows the request has seen.
//   tm_short_conv_walk   both in one launch, for steps whose requests bring few rows each; the same bits.
//   tm_poly_norm       out = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over a row, powers by element.
#include "common.h"
#include "api.h"

#define LN_THREADS 256

template <typename T>
__global__ __launch_bounds__(LN_THREADS) void layer_norm_kernel(float* __restrict__ resid, const T* __restrict__ y,
                                                                const T* __restrict__ gate, float mult,
                                                                const int* __restrict__ rows, const float* __restrict__ w,
                                                                const float* __restrict__ b, T* __restrict__ out, int hidden,
                                                                float eps) {
    extern __shared__ float row_s[];
    __shared__ float red[LN_THREADS / TM_WAVE];
    const int r = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[r] : r) * hidden;
    float sum = 0.f;
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS) {
        float v = resid[src + c];
        if (y) {
            float d = Elem<T>::load(y + src + c);
            if (gate) d *= 1.0f / (1.0f + __expf(-Elem<T>::load(gate + src + c)));
            v += mult * d;
            if (!rows) resid[src + c] = v;
        }
        row_s[c] = v;
        sum += v;
    }
    if (!out) return;
    const float mean = block_sum<LN_THREADS>(sum, red) / (float)hidden;
    float ss = 0.f;
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS) {
        const float d = row_s[c] - mean;
        ss += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum<LN_THREADS>(ss, red) / (float)hidden + eps);
    T* o = out + (size_t)r * hidden;
    for (int c = threadIdx.x; c < hidden; c += LN_THREADS)
        Elem<T>::store(o + c, (row_s[c] - mean) * inv * w[c] + b[c]);
}

extern "C" int tm_layer_norm(float* resid, const void* y, const void* gate, float mult, const int* rows, const float* w,
                             const float* b, void* out, int dtype, int R, int hidden, float eps, hipStream_t stream) {
    if (!resid || R < 0 || hidden <= 0 || hidden > 16384 || (gate && !y) || (out && (!w || !b)) || !(eps > 0.f)) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (R == 0 || (!y && !out)) return TM_OK;
    const size_t lds = (size_t)hidden * sizeof(float);
    if (dtype == TM_F32)
        layer_norm_kernel<float><<<R, LN_THREADS, lds, stream>>>(resid, (const float*)y, (const float*)gate, mult, rows, w, b,
                                                                 (float*)out, hidden, eps);
    else
        layer_norm_kernel<bf16_t><<<R, LN_THREADS, lds, stream>>>(resid, (const bf16_t*)y, (const bf16_t*)gate, mult, rows, w, b,
                                                                  (bf16_t*)out, hidden, eps);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ short convolution

#define SC_THREADS 256
#define SC_MAX_TAPS 16

// sum_j w[j] * x[j], j ascending, every product and sum rounded on its own: the two kernels below give the same bits
// (MAXT: the most taps the instantiation takes; the sum is the same sequence of operations at every MAXT)
template <int MAXT>
__device__ __forceinline__ float tap_sum(const float (&wv)[MAXT], const float (&xv)[MAXT], int taps) {
#pragma clang fp contract(off)
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < MAXT; ++j)
        if (j < taps) acc += wv[j] * xv[j];
    return acc;
}

template <typename T, int MAXT>
__global__ __launch_bounds__(SC_THREADS) void short_conv_kernel(const T* __restrict__ h, T* __restrict__ out,
                                                                const T* __restrict__ w, const T* __restrict__ state,
                                                                const int* __restrict__ cu, const int* __restrict__ slots,
                                                                const int* __restrict__ seq_of_token, int width, int taps) {
    const int t = blockIdx.x;
    const int s = seq_of_token[t];
    const int first = cu[s];
    const int i = t - first;                                 // the token's place among its request's rows of this step
    const T* st = state + (size_t)slots[s] * (taps - 1) * width;
    for (int c = blockIdx.y * SC_THREADS + threadIdx.x; c < width; c += gridDim.y * SC_THREADS) {
        float wv[MAXT], xv[MAXT];
#pragma unroll
        for (int j = 0; j < MAXT; ++j) {
            wv[j] = xv[j] = 0.f;
            if (j < taps) {
                const int at = i - (taps - 1) + j;           // < 0: before this step's rows, in the state
                xv[j] = at >= 0 ? Elem<T>::load(h + (size_t)(first + at) * width + c)
                                : Elem<T>::load(st + (size_t)(taps - 1 + at) * width + c);
                wv[j] = Elem<T>::load(w + (size_t)c * taps + j);
            }
        }
        Elem<T>::store(out + (size_t)t * width + c, Elem<T>::load(h + (size_t)t * width + c) + tap_sum<MAXT>(wv, xv, taps));
    }
}

// The same for steps whose requests bring few rows each (single tokens): a thread takes a channel of a request, walks the
// request's rows with the window of the last taps rows in registers, and leaves the new state behind: one launch.
template <typename T, int MAXT>
__global__ __launch_bounds__(SC_THREADS) void short_conv_walk_kernel(const T* __restrict__ h, T* __restrict__ out,
                                                                     const T* __restrict__ w, T* __restrict__ state,
                                                                     const int* __restrict__ cu, const int* __restrict__ slots,
                                                                     int width, int taps) {
    const int s = blockIdx.x;
    const int first = cu[s], n = cu[s + 1] - first;
    if (n <= 0) return;
    T* st = state + (size_t)slots[s] * (taps - 1) * width;
    for (int c = blockIdx.y * SC_THREADS + threadIdx.x; c < width; c += gridDim.y * SC_THREADS) {
        float wv[MAXT], xv[MAXT];
#pragma unroll
        for (int j = 0; j < MAXT; ++j) {
            wv[j] = j < taps ? Elem<T>::load(w + (size_t)c * taps + j) : 0.f;
            xv[j] = j < taps - 1 ? Elem<T>::load(st + (size_t)j * width + c) : 0.f;
        }
        for (int i = 0; i < n; ++i) {
            const float cur = Elem<T>::load(h + (size_t)(first + i) * width + c);
#pragma unroll
            for (int j = 0; j < MAXT; ++j)
                if (j == taps - 1) xv[j] = cur;
            Elem<T>::store(out + (size_t)(first + i) * width + c, cur + tap_sum<MAXT>(wv, xv, taps));
#pragma unroll
            for (int j = 0; j + 1 < MAXT; ++j)
                if (j < taps - 1) xv[j] = xv[j + 1];
        }
#pragma unroll
        for (int j = 0; j < MAXT; ++j)
            if (j < taps - 1) Elem<T>::store(st + (size_t)j * width + c, xv[j]);
    }
}

template <typename T>
__global__ __launch_bounds__(SC_THREADS) void short_conv_state_kernel(const T* __restrict__ h, T* __restrict__ state,
                                                                      const int* __restrict__ cu, const int* __restrict__ slots,
                                                                      int width, int taps) {
    const int s = blockIdx.x;
    const int first = cu[s], n = cu[s + 1] - first;
    if (n <= 0) return;
    T* st = state + (size_t)slots[s] * (taps - 1) * width;
    const int keep = taps - 1;
    for (int c = blockIdx.y * SC_THREADS + threadIdx.x; c < width; c += gridDim.y * SC_THREADS) {
        T next[SC_MAX_TAPS - 1];
        for (int k = 0; k < keep; ++k) {
            const int at = n - keep + k;                     // the row that becomes state row k
            next[k] = at >= 0 ? h[(size_t)(first + at) * width + c] : st[(size_t)(keep + at) * width + c];
        }
        for (int k = 0; k < keep; ++k) st[(size_t)k * width + c] = next[k];
    }
}

extern "C" int tm_short_conv(const void* h, void* out, const void* w, const void* state, const int* cu_q_lens,
                             const int* state_slots, const int* seq_of_token, int T, int width, int taps, int dtype,
                             hipStream_t stream) {
    if (!h || !out || !w || T < 0 || width <= 0 || taps < 1 || taps > SC_MAX_TAPS || (taps > 1 && !state)) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    dim3 grid(T, (width + SC_THREADS - 1) / SC_THREADS > 8 ? 8 : (width + SC_THREADS - 1) / SC_THREADS);
#define SC_GO(T_, MAXT_)                                                                                                  \
    short_conv_kernel<T_, MAXT_><<<grid, SC_THREADS, 0, stream>>>((const T_*)h, (T_*)out, (const T_*)w, (const T_*)state, cu_q_lens, \
                                                                  state_slots, seq_of_token, width, taps)
    if (dtype == TM_F32) {
        if (taps <= 4) SC_GO(float, 4); else if (taps <= 8) SC_GO(float, 8); else SC_GO(float, SC_MAX_TAPS);
    } else {
        if (taps <= 4) SC_GO(bf16_t, 4); else if (taps <= 8) SC_GO(bf16_t, 8); else SC_GO(bf16_t, SC_MAX_TAPS);
    }
#undef SC_GO
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// tm_short_conv and tm_short_conv_state in one launch, for steps whose requests bring few rows each: the same bits.
extern "C" int tm_short_conv_walk(const void* h, void* out, const void* w, void* state, const int* cu_q_lens, const int* state_slots,
                                  int S, int width, int taps, int dtype, hipStream_t stream) {
    if (!h || !out || !w || S < 0 || width <= 0 || taps < 2 || taps > SC_MAX_TAPS || !state) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (S == 0) return TM_OK;
    dim3 grid(S, (width + SC_THREADS - 1) / SC_THREADS > 8 ? 8 : (width + SC_THREADS - 1) / SC_THREADS);
#define SC_GO(T_, MAXT_)                                                                                                       \
    short_conv_walk_kernel<T_, MAXT_><<<grid, SC_THREADS, 0, stream>>>((const T_*)h, (T_*)out, (const T_*)w, (T_*)state, cu_q_lens,     \
                                                                       state_slots, width, taps)
    if (dtype == TM_F32) {
        if (taps <= 4) SC_GO(float, 4); else if (taps <= 8) SC_GO(float, 8); else SC_GO(float, SC_MAX_TAPS);
    } else {
        if (taps <= 4) SC_GO(bf16_t, 4); else if (taps <= 8) SC_GO(bf16_t, 8); else SC_GO(bf16_t, SC_MAX_TAPS);
    }
#undef SC_GO
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_short_conv_state(const void* h, void* state, const int* cu_q_lens, const int* state_slots, int S, int width,
                                   int taps, int dtype, hipStream_t stream) {
    if (!h || S < 0 || width <= 0 || taps < 1 || taps > SC_MAX_TAPS || (taps > 1 && !state)) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (S == 0 || taps == 1) return TM_OK;
    dim3 grid(S, (width + SC_THREADS - 1) / SC_THREADS > 8 ? 8 : (width + SC_THREADS - 1) / SC_THREADS);
    if (dtype == TM_F32)
        short_conv_state_kernel<float><<<grid, SC_THREADS, 0, stream>>>((const float*)h, (float*)state, cu_q_lens, state_slots, width, taps);
    else
        short_conv_state_kernel<bf16_t><<<grid, SC_THREADS, 0, stream>>>((const bf16_t*)h, (bf16_t*)state, cu_q_lens, state_slots, width, taps);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------ PolyNorm

template <typename T>
__global__ __launch_bounds__(LN_THREADS) void poly_norm_kernel(const float* __restrict__ z, const float* __restrict__ coef,
                                                               T* __restrict__ out, int F, float eps) {
    __shared__ float red[LN_THREADS / TM_WAVE];
    const float* zr = z + (size_t)blockIdx.x * F;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
    for (int c = threadIdx.x; c < F; c += LN_THREADS) {
        const float v = zr[c], v2 = v * v, v3 = v2 * v;
        s2 += v2;
        s4 += v2 * v2;
        s6 += v3 * v3;
    }
    const float r1 = 1.0f / sqrtf(block_sum<LN_THREADS>(s2, red) / (float)F + eps);
    const float r2 = 1.0f / sqrtf(block_sum<LN_THREADS>(s4, red) / (float)F + eps);
    const float r3 = 1.0f / sqrtf(block_sum<LN_THREADS>(s6, red) / (float)F + eps);
    const float a = coef[0], b = coef[1], c3 = coef[2], e = coef[3];
    T* o = out + (size_t)blockIdx.x * F;
    for (int c = threadIdx.x; c < F; c += LN_THREADS) {
        const float v = zr[c], v2 = v * v;
        Elem<T>::store(o + c, a * (v * r1) + b * (v2 * r2) + c3 * (v2 * v * r3) + e);
    }
}

extern "C" int tm_poly_norm(const float* z, const float* coef, void* out, int dtype, int T, int F, float eps,
                            hipStream_t stream) {
    if (!z || !coef || !out || T < 0 || F <= 0 || !(eps > 0.f)) return TM_ERR_ARG;
    if (dtype != TM_F32 && dtype != TM_BF16) return TM_ERR_ARG;
    if (T == 0) return TM_OK;
    if (dtype == TM_F32)
        poly_norm_kernel<float><<<T, LN_THREADS, 0, stream>>>(z, coef, (float*)out, F, eps);
    else
        poly_norm_kernel<bf16_t><<<T, LN_THREADS, 0, stream>>>(z, coef, (bf16_t*)out, F, eps);
    TM_CHECK_LAUNCH();
    return TM_OK;
}
