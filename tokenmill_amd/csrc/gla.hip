// Gated linear attention: a recurrent mixer whose state per request and head is a matrix S [D, Dv] of 32-bit floats,
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T          a_t [D]: a decay per key channel, in (0, 1)
//   o_t = S_t^T q_t                              [Dv]
//
// advanced token by token in the order of the positions, within a step's portion and from one step to the next
// (the state lives in the request's state slot between steps). Three kernels:
//   gla_decay     a = sigmoid(z)^(1/tau) from the gate projection z, as exp(logsigmoid(z) / tau), 32-bit
//   gla_scan      the recurrence; reads q, k, v from the rows of the stacked projection, writes o in 32-bit
//   gla_out_gate  y = w * o / rms(o) (per head, over Dv) * silu(g), rounded once to the model's type
// Everything that enters the recurrence is 32-bit. The columns of S are independent of each other, so the scan is
// dealt over (request, head, 16 columns) wavefronts; a lane keeps a quarter of a column's D rows in registers, and a
// column's four partial dot products are added in a fixed order. A token's result depends on its request's state
// and tokens only, never on the step's other rows or on how the prompt was cut.
#include "common.h"
#include "api.h"

__global__ void gla_decay_kernel(const float* __restrict__ z, float* __restrict__ a, float inv_tau, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float x = z[i];
        const float ls = fminf(x, 0.f) - log1pf(expf(-fabsf(x)));        // log sigmoid(x)
        a[i] = expf(ls * inv_tau);
    }
}

extern "C" int tm_gla_decay(const float* z, float* a, float tau, long long n, hipStream_t stream) {
    if (n <= 0) return TM_OK;
    if (!z || !a || !(tau > 0.f)) return TM_ERR_ARG;
    const size_t want = ((size_t)n + 255) / 256;
    gla_decay_kernel<<<(int)(want < 16384 ? want : 16384), 256, 0, stream>>>(z, a, 1.0f / tau, (size_t)n);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

#define GLA_PARTS 4                         // lanes that share a column's rows
#define GLA_COLS (TM_WAVE / GLA_PARTS)      // columns of a wavefront

// grid (ceil(Dv / GLA_COLS), H, S); a block is one wavefront. lane = column * GLA_PARTS + part; part p keeps rows
// p * R .. p * R + R - 1 of its column, R = ceil(D / GLA_PARTS) <= RMAX.
template <typename T, int RMAX>
__global__ __launch_bounds__(TM_WAVE) void gla_scan_kernel(const T* __restrict__ proj, int ld, int q_off, int k_off, int v_off,
                                                          const float* __restrict__ decay, float* __restrict__ o,
                                                          float* __restrict__ state, const int* __restrict__ cu_q_lens,
                                                          const int* __restrict__ state_slots, int H, int D, int Dv,
                                                          float q_scale) {
    const int lane = threadIdx.x, part = lane % GLA_PARTS;
    const int e = blockIdx.x * GLA_COLS + lane / GLA_PARTS;
    const int h = blockIdx.y, s = blockIdx.z;
    const int R = (D + GLA_PARTS - 1) / GLA_PARTS;
    const int d0 = part * R;
    const bool col = e < Dv;
    const int t0 = cu_q_lens[s], t1 = cu_q_lens[s + 1];
    if (t1 <= t0) return;
    float* st = state + (((size_t)state_slots[s] * H + h) * D) * Dv + (col ? e : 0);
    float S[RMAX];
#pragma unroll
    for (int i = 0; i < RMAX; ++i) S[i] = (col && i < R && d0 + i < D) ? st[(size_t)(d0 + i) * Dv] : 0.f;
    for (int t = t0; t < t1; ++t) {
        const T* row = proj + (size_t)t * ld;
        const T* qr = row + q_off + h * D + d0;
        const T* kr = row + k_off + h * D + d0;
        const float* ar = decay + ((size_t)t * H + h) * D + d0;
        const float v = col ? Elem<T>::load(row + v_off + h * Dv + e) : 0.f;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < RMAX; ++i) {
            if (i < R && d0 + i < D) {
                const float kv = Elem<T>::load(kr + i) * v;
                S[i] = ar[i] * S[i] + kv;
                acc += S[i] * (Elem<T>::load(qr + i) * q_scale);
            }
        }
        acc += __shfl_xor(acc, 1, TM_WAVE);
        acc += __shfl_xor(acc, 2, TM_WAVE);
        if (col && part == 0) o[((size_t)t * H + h) * Dv + e] = acc;
    }
#pragma unroll
    for (int i = 0; i < RMAX; ++i)
        if (col && i < R && d0 + i < D) st[(size_t)(d0 + i) * Dv] = S[i];
}

template <typename T>
static int launch_gla_scan(const void* proj, int ld, int q_off, int k_off, int v_off, const float* decay, float* o, float* state,
                           const int* cu, const int* slots, int S, int H, int D, int Dv, float q_scale, hipStream_t stream) {
    const dim3 grid((Dv + GLA_COLS - 1) / GLA_COLS, H, S);
    const int R = (D + GLA_PARTS - 1) / GLA_PARTS;
    if (R <= 16)
        gla_scan_kernel<T, 16><<<grid, TM_WAVE, 0, stream>>>((const T*)proj, ld, q_off, k_off, v_off, decay, o, state, cu, slots, H,
                                                            D, Dv, q_scale);
    else if (R <= 32)
        gla_scan_kernel<T, 32><<<grid, TM_WAVE, 0, stream>>>((const T*)proj, ld, q_off, k_off, v_off, decay, o, state, cu, slots, H,
                                                            D, Dv, q_scale);
    else
        gla_scan_kernel<T, 64><<<grid, TM_WAVE, 0, stream>>>((const T*)proj, ld, q_off, k_off, v_off, decay, o, state, cu, slots, H,
                                                            D, Dv, q_scale);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

// proj rows hold q [H, D] at q_off, k [H, D] at k_off, v [H, Dv] at v_off (element offsets into a row of ld elements);
// decay float32 [T, H, D]; o float32 [T, H, Dv]; state float32 [slots, H, D, Dv]; request s of the step owns rows
// cu_q_lens[s] .. cu_q_lens[s + 1] - 1 and the state row state_slots[s].
extern "C" int tm_gla_scan(const void* proj, int ld, int q_off, int k_off, int v_off, int dtype, const float* decay, float* o,
                           float* state, const int* cu_q_lens, const int* state_slots, int S, int H, int D, int Dv,
                           float q_scale, hipStream_t stream) {
    if (S <= 0) return TM_OK;
    if (H <= 0 || D <= 0 || D > 256 || Dv <= 0 || H > 65535 || S > 65535 || !proj || !decay || !o || !state || !cu_q_lens ||
        !state_slots || q_off < 0 || k_off < 0 || v_off < 0 || ld < q_off + H * D || ld < k_off + H * D || ld < v_off + H * Dv)
        return TM_ERR_ARG;
    if (dtype == TM_F32) return launch_gla_scan<float>(proj, ld, q_off, k_off, v_off, decay, o, state, cu_q_lens, state_slots, S, H, D, Dv, q_scale, stream);
    if (dtype == TM_BF16) return launch_gla_scan<bf16_t>(proj, ld, q_off, k_off, v_off, decay, o, state, cu_q_lens, state_slots, S, H, D, Dv, q_scale, stream);
    return TM_ERR_ARG;
}

// y[t, h, e] = w[e] * o[t, h, e] / sqrt(mean_e(o[t, h]^2) + eps) * silu(g[t, h, e]); grid (T, H), one wavefront each.
template <typename T>
__global__ __launch_bounds__(TM_WAVE) void gla_out_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate, int ldg,
                                                              const float* __restrict__ w, T* __restrict__ y, int H, int Dv,
                                                              float eps) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + ((size_t)t * H + h) * Dv;
    const T* grow = gate + (size_t)t * ldg + (size_t)h * Dv;
    T* yrow = y + ((size_t)t * H + h) * Dv;
    float ss = 0.f;
    for (int e = lane; e < Dv; e += TM_WAVE) ss += orow[e] * orow[e];
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
    for (int e = lane; e < Dv; e += TM_WAVE) {
        const float g = Elem<T>::load(grow + e);
        Elem<T>::store(yrow + e, (w[e] * (orow[e] * r)) * (g / (1.f + expf(-g))));
    }
}

extern "C" int tm_gla_out_gate(const float* o, const void* gate, int ldg, int dtype, const float* w, void* y, int T, int H, int Dv,
                               float eps, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (H <= 0 || H > 65535 || Dv <= 0 || ldg < H * Dv || !o || !gate || !w || !y || !(eps > 0.f)) return TM_ERR_ARG;
    const dim3 grid(T, H);
    if (dtype == TM_F32)
        gla_out_gate_kernel<float><<<grid, TM_WAVE, 0, stream>>>(o, (const float*)gate, ldg, w, (float*)y, H, Dv, eps);
    else if (dtype == TM_BF16)
        gla_out_gate_kernel<bf16_t><<<grid, TM_WAVE, 0, stream>>>(o, (const bf16_t*)gate, ldg, w, (bf16_t*)y, H, Dv, eps);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
