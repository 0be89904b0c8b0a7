// RMS norm in groups, around a sublayer: the result y of a mixer or feed-forward is normed, added to the 32-bit
// residual stream, and the sum is normed again for the sublayer that follows, in one kernel.
//
//   norm_g(v)[c] = w[c] * v[c] / sqrt(mean(v[group of c]^2) + eps)     the row cut into `groups` equal consecutive parts
//
//   resid[r] += norm_g(y[r]; post_w)     (post_w == nullptr: y is added as it is; y == nullptr: nothing is added)
//   out[r]    = norm_g(resid[r]; pre_w)  (out == nullptr: no second norm)
//
// rows == nullptr: every row, the residual updated in place. rows != nullptr: row rows[r] is read, nothing is written
// back, out row r (the rows whose logits are wanted).
//
// Everything is 32-bit; a bfloat16 result is rounded once, where it is stored. The sums of squares have one order
// per (width, groups): a group (or, with fewer than four groups, each of its 4 / groups equal pieces) is summed by
// one wavefront, lanes striding over it, and a group's pieces are added in their order.
#include "common.h"
#include "api.h"

#define GN_THREADS 256
#define GN_WAVES (GN_THREADS / TM_WAVE)

// sums of squares of the units of a row held in `v` (LDS or global), into part[units]
template <typename Load>
__device__ __forceinline__ void unit_sums(Load at, float* part, int glen, int split, int units) {
    const int wave = threadIdx.x / TM_WAVE, lane = threadIdx.x % TM_WAVE;
    const int plen = (glen + split - 1) / split;
    for (int u = wave; u < units; u += GN_WAVES) {
        const int g = u / split, i = u - g * split;
        const int lo = g * glen + i * plen;
        const int hi = min(lo + plen, (g + 1) * glen);
        float ss = 0.f;
#pragma unroll 8
        for (int c = lo + lane; c < hi; c += TM_WAVE) {
            const float x = at(c);
            ss += x * x;
        }
        ss = wave_sum(ss);
        if (lane == 0) part[u] = ss;
    }
}

// The groups' 1 / sqrt(mean + eps) from their units' sums, once per group (a root and two divisions per element
// were most of a small step's time), into scale[groups]. Ends with a barrier.
__device__ __forceinline__ void group_scales(const float* part, float* scale, int groups, int split, int glen, float eps) {
    for (int g = threadIdx.x; g < groups; g += GN_THREADS) {
        float ss = part[g * split];
        for (int i = 1; i < split; ++i) ss += part[g * split + i];
        scale[g] = 1.0f / sqrtf(ss / (float)glen + eps);
    }
    __syncthreads();
}

// STAGE: the row of y and both weight vectors are copied into LDS beside the residual row by the first loop, so that
// everything the block needs from memory is asked for at once (one trip instead of four dependent ones: a step of a
// few rows is nothing but those trips); without it (rows too wide for that much LDS) they are read where they are used.
template <typename T, typename WT, bool STAGE>
__global__ __launch_bounds__(GN_THREADS) void group_norm_kernel(float* __restrict__ resid, const T* __restrict__ y,
                                                                const WT* __restrict__ post_w,
                                                                const int* __restrict__ rows,
                                                                const WT* __restrict__ pre_w, T* __restrict__ out,
                                                                int hidden, int groups, int split, float eps) {
    extern __shared__ float lds[];
    float* xs = lds;                                        // the row, [hidden]
    float* ys = lds + hidden;                               // STAGE: y, post_w, pre_w, [hidden] each
    float* pw = lds + 2 * hidden;
    float* qw = lds + 3 * hidden;
    float* part = lds + (STAGE ? 4 : 1) * hidden;           // [groups * split]
    float* scale = part + groups * split;                   // [groups]
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* x = resid + src * hidden;
    const T* yr = y ? y + src * hidden : nullptr;
    const int glen = hidden / groups, units = groups * split;
    // unrolled: the loads of eight rounds are in flight together (left as a loop, every round waits for its own)
#pragma unroll 8
    for (int c = threadIdx.x; c < hidden; c += GN_THREADS) {
        xs[c] = x[c];
        if (STAGE) {
            if (yr) ys[c] = Elem<T>::load(yr + c);
            if (post_w) pw[c] = Elem<WT>::load(post_w + c);
            if (pre_w) qw[c] = Elem<WT>::load(pre_w + c);
        }
    }
    if (STAGE) __syncthreads();
    if (yr) {
        if (post_w) {
            if (STAGE) unit_sums([&](int c) { return ys[c]; }, part, glen, split, units);
            else unit_sums([&](int c) { return Elem<T>::load(yr + c); }, part, glen, split, units);
            __syncthreads();
            group_scales(part, scale, groups, split, glen, eps);
        }
#pragma unroll 8
        for (int c = threadIdx.x; c < hidden; c += GN_THREADS) {
            float d = STAGE ? ys[c] : Elem<T>::load(yr + c);
            if (post_w) d = (STAGE ? pw[c] : Elem<WT>::load(post_w + c)) * (d * scale[c / glen]);
            const float v = xs[c] + d;
            xs[c] = v;
            if (!rows) x[c] = v;
        }
    }
    if (!out) return;
    __syncthreads();
    unit_sums([&](int c) { return xs[c]; }, part, glen, split, units);
    __syncthreads();
    group_scales(part, scale, groups, split, glen, eps);
    T* o = out + (size_t)r * hidden;
#pragma unroll 8
    for (int c = threadIdx.x; c < hidden; c += GN_THREADS)
        Elem<T>::store(o + c, (STAGE ? qw[c] : Elem<WT>::load(pre_w + c)) * (xs[c] * scale[c / glen]));
}

template <typename T, typename WT>
static void launch_group_norm(float* resid, const void* y, const void* post_w, const int* rows, const void* pre_w, void* out, int R,
                              int hidden, int groups, int split, float eps, hipStream_t stream) {
    const size_t units = (size_t)groups * split + groups;       // the units' sums and the groups' scales
    const size_t staged = (4 * (size_t)hidden + units) * sizeof(float), plain = ((size_t)hidden + units) * sizeof(float);
    if (staged <= 64 * 1024)
        group_norm_kernel<T, WT, true><<<R, GN_THREADS, staged, stream>>>(resid, (const T*)y, (const WT*)post_w, rows, (const WT*)pre_w,
                                                                         (T*)out, hidden, groups, split, eps);
    else
        group_norm_kernel<T, WT, false><<<R, GN_THREADS, plain, stream>>>(resid, (const T*)y, (const WT*)post_w, rows, (const WT*)pre_w,
                                                                         (T*)out, hidden, groups, split, eps);
}

extern "C" int tm_group_norm(float* resid, const void* y, const void* post_w, const int* rows, const void* pre_w,
                             int w_dtype, void* out, int dtype, int R, int hidden, int groups, float eps,
                             hipStream_t stream) {
    if (R <= 0) return TM_OK;
    if (hidden <= 0 || groups <= 0 || hidden % groups || !(eps > 0.f) || !resid) return TM_ERR_ARG;
    if ((out == nullptr) != (pre_w == nullptr)) return TM_ERR_ARG;
    if (!y && post_w) return TM_ERR_ARG;
    const int split = groups >= GN_WAVES ? 1 : GN_WAVES / groups;
    const size_t lds = ((size_t)hidden + (size_t)groups * split + groups) * sizeof(float);
    if (lds > 64 * 1024) return TM_ERR_ARG;
    if (dtype == TM_F32 && w_dtype == TM_F32)
        launch_group_norm<float, float>(resid, y, post_w, rows, pre_w, out, R, hidden, groups, split, eps, stream);
    else if (dtype == TM_BF16 && w_dtype == TM_BF16)
        launch_group_norm<bf16_t, bf16_t>(resid, y, post_w, rows, pre_w, out, R, hidden, groups, split, eps, stream);
    else if (dtype == TM_BF16 && w_dtype == TM_F32)
        launch_group_norm<bf16_t, float>(resid, y, post_w, rows, pre_w, out, R, hidden, groups, split, eps, stream);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
