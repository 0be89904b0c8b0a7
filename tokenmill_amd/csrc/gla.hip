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

// The same scan for sizes whose rows come in whole 16-byte pieces (D a multiple of 4 * 16 / sizeof(T), aligned rows): a
// lane's R values of q, k and the decays are a few 16-byte loads instead of R small ones, and the next token's are
// asked for before the current token is worked on. Same products and sums in the same order as the kernel above.
// PARTS lanes share a column's rows (4 or 8: with 8, a lane holds half as much and twice as many wavefronts hide each
// other's loads); OUT = false leaves q and the results out (the scan that only builds the segments' local states).
template <typename T, int RMAX, int PARTS, bool OUT>
__global__ __launch_bounds__(TM_WAVE) void gla_scan_vec_kernel(const T* __restrict__ proj, int ld, int q_off, int k_off, int v_off,
                                                              const float* __restrict__ decay, float* __restrict__ o,
                                                              float* __restrict__ state, const int* __restrict__ cu_q_lens,
                                                              const int* __restrict__ state_slots, int H, int D, int Dv,
                                                              float q_scale) {
    constexpr int EV = Piece<T>::N, NQ = RMAX / EV, NA = RMAX / 4;
    const int lane = threadIdx.x, part = lane % PARTS;
    const int e = blockIdx.x * (TM_WAVE / PARTS) + lane / PARTS;
    const int h = blockIdx.y, s = blockIdx.z;
    const int R = D / PARTS;                          // a multiple of EV (and of 4): the host checks
    const int nq = R / EV, na = R / 4;
    const int d0 = part * R;
    const bool col = e < Dv;
    const int t0 = cu_q_lens[s], t1 = cu_q_lens[s + 1];
    if (t1 <= t0) return;
    float* st = state + (((size_t)state_slots[s] * H + h) * D) * Dv + (col ? e : 0);
    float S[RMAX];
#pragma unroll
    for (int i = 0; i < RMAX; ++i) S[i] = (col && i < R) ? st[(size_t)(d0 + i) * Dv] : 0.f;
    uint4 cq[NQ], ck[NQ], nq_[NQ], nk_[NQ];
    float4 ca[NA], na_[NA];
    float cv, nv;
    const size_t head_q = (size_t)q_off + h * D + d0, head_k = (size_t)k_off + h * D + d0;
    {
        const T* row = proj + (size_t)t0 * ld;
        const float* ar = decay + ((size_t)t0 * H + h) * D + d0;
#pragma unroll
        for (int i = 0; i < NQ; ++i)
            if (i < nq) {
                if (OUT) cq[i] = *(const uint4*)(row + head_q + i * EV);
                ck[i] = *(const uint4*)(row + head_k + i * EV);
            }
#pragma unroll
        for (int i = 0; i < NA; ++i)
            if (i < na) ca[i] = *(const float4*)(ar + 4 * i);
        cv = col ? Elem<T>::load(row + v_off + h * Dv + e) : 0.f;
    }
    for (int t = t0; t < t1; ++t) {
        const int tn = t + 1 < t1 ? t + 1 : t;            // the last token asks for itself again
        {
            const T* row = proj + (size_t)tn * ld;
            const float* ar = decay + ((size_t)tn * H + h) * D + d0;
#pragma unroll
            for (int i = 0; i < NQ; ++i)
                if (i < nq) {
                    if (OUT) nq_[i] = *(const uint4*)(row + head_q + i * EV);
                    nk_[i] = *(const uint4*)(row + head_k + i * EV);
                }
#pragma unroll
            for (int i = 0; i < NA; ++i)
                if (i < na) na_[i] = *(const float4*)(ar + 4 * i);
            nv = col ? Elem<T>::load(row + v_off + h * Dv + e) : 0.f;
        }
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            if (i < nq) {
                float qf[EV], kf[EV];
                if (OUT) Piece<T>::unpack(cq[i], qf);
                Piece<T>::unpack(ck[i], kf);
#pragma unroll
                for (int j = 0; j < EV; ++j) {
                    const int r = i * EV + j;
                    const float4 a4 = ca[r / 4];
                    const float a = (r % 4 == 0) ? a4.x : (r % 4 == 1) ? a4.y : (r % 4 == 2) ? a4.z : a4.w;
                    const float kv = kf[j] * cv;
                    S[r] = a * S[r] + kv;
                    if (OUT) acc += S[r] * (qf[j] * q_scale);
                }
            }
        }
        if (OUT) {
            acc += __shfl_xor(acc, 1, TM_WAVE);
            acc += __shfl_xor(acc, 2, TM_WAVE);
            if (PARTS == 8) acc += __shfl_xor(acc, 4, TM_WAVE);
            if (col && part == 0) o[((size_t)t * H + h) * Dv + e] = acc;
        }
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            if (OUT) cq[i] = nq_[i];
            ck[i] = nk_[i];
        }
#pragma unroll
        for (int i = 0; i < NA; ++i) ca[i] = na_[i];
        cv = nv;
    }
#pragma unroll
    for (int i = 0; i < RMAX; ++i)
        if (col && i < R) st[(size_t)(d0 + i) * Dv] = S[i];
}

template <typename T>
static bool gla_scan_in_pieces(const void* proj, int ld, int q_off, int k_off, const float* decay, int D, int parts) {
    constexpr int EV = Piece<T>::N;
    return D % (parts * EV) == 0 && ld % EV == 0 && q_off % EV == 0 && k_off % EV == 0 && ((uintptr_t)proj % 16) == 0 &&
           ((uintptr_t)decay % 16) == 0;
}

template <typename T>
static int launch_gla_scan(const void* proj, int ld, int q_off, int k_off, int v_off, const float* decay, float* o, float* state,
                           const int* cu, const int* slots, int S, int H, int D, int Dv, float q_scale, hipStream_t stream) {
    const dim3 grid((Dv + GLA_COLS - 1) / GLA_COLS, H, S);
    const int R = (D + GLA_PARTS - 1) / GLA_PARTS;
    // o == nullptr: only the states are wanted (the first scan of a portion in segments)
#define GLA_VEC(RM, P, OUT_)                                                                                                     \
    gla_scan_vec_kernel<T, RM, P, OUT_><<<dim3((Dv + TM_WAVE / P - 1) / (TM_WAVE / P), H, S), TM_WAVE, 0, stream>>>(              \
        (const T*)proj, ld, q_off, k_off, v_off, decay, o, state, cu, slots, H, D, Dv, q_scale)
    if (D / 8 <= 32 && gla_scan_in_pieces<T>(proj, ld, q_off, k_off, decay, D, 8)) {           // eight lanes a column
        if (D / 8 <= 16) { if (o) GLA_VEC(16, 8, true); else GLA_VEC(16, 8, false); }
        else { if (o) GLA_VEC(32, 8, true); else GLA_VEC(32, 8, false); }
        TM_CHECK_LAUNCH();
        return TM_OK;
    }
    if (R <= 32 && gla_scan_in_pieces<T>(proj, ld, q_off, k_off, decay, D, GLA_PARTS)) {       // beyond 32 rows a lane the registers do not hold two tokens
        if (R <= 16) { if (o) GLA_VEC(16, 4, true); else GLA_VEC(16, 4, false); }
        else { if (o) GLA_VEC(32, 4, true); else GLA_VEC(32, 4, false); }
        TM_CHECK_LAUNCH();
        return TM_OK;
    }
#undef GLA_VEC
    if (!o) return TM_ERR_ARG;                                  // the scan without results exists for rows in 16-byte pieces only
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

// Does the scan of these operands run in 16-byte pieces (and so also without results, o == nullptr)?
template <typename T>
static bool gla_scan_pieces_any(const void* proj, int ld, int q_off, int k_off, const float* decay, int D) {
    return (D / 8 <= 32 && gla_scan_in_pieces<T>(proj, ld, q_off, k_off, decay, D, 8)) ||
           ((D + GLA_PARTS - 1) / GLA_PARTS <= 32 && gla_scan_in_pieces<T>(proj, ld, q_off, k_off, decay, D, GLA_PARTS));
}

extern "C" int tm_gla_scan_in_pieces(int dtype, const void* proj, int ld, int q_off, int k_off, const float* decay, int D) {
    if (D <= 0) return 0;
    if (dtype == TM_F32) return gla_scan_pieces_any<float>(proj, ld, q_off, k_off, decay, D) ? 1 : 0;
    if (dtype == TM_BF16) return gla_scan_pieces_any<bf16_t>(proj, ld, q_off, k_off, decay, D) ? 1 : 0;
    return 0;
}

// proj rows hold q [H, D] at q_off, k [H, D] at k_off, v [H, Dv] at v_off (element offsets into a row of ld elements);
// decay float32 [T, H, D]; o float32 [T, H, Dv]; state float32 [slots, H, D, Dv]; request s of the step owns rows
// cu_q_lens[s] .. cu_q_lens[s + 1] - 1 and the state row state_slots[s].
extern "C" int tm_gla_scan(const void* proj, int ld, int q_off, int k_off, int v_off, int dtype, const float* decay, float* o,
                           float* state, const int* cu_q_lens, const int* state_slots, int S, int H, int D, int Dv,
                           float q_scale, hipStream_t stream) {
    if (S <= 0) return TM_OK;
    if (H <= 0 || D <= 0 || D > 256 || Dv <= 0 || H > 65535 || S > 65535 || !proj || !decay || !state || !cu_q_lens ||
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

// ------------------------------------------------------------------------------------------------------------------
// The decays straight from the narrow projection: a[t, n] = sigmoid(z)^(1/tau), z = sum_k x[t, k] W[n, k] + b[n], with
// the sum and everything behind it in 32-bit. K is the gate's width (a handful of channels), so a thread per output
// walks it in ascending k; the row of x is the same for all threads of a block.
// ------------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gla_gate_decay_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ W,
                                                            const T* __restrict__ bias, float* __restrict__ a, int N, int K,
                                                            float inv_tau) {
    const int n = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;
    if (n >= N) return;
    const T* xr = x + (size_t)t * ldx;
    const T* wr = W + (size_t)n * K;
    float z = bias ? Elem<T>::load(bias + n) : 0.f;
#pragma unroll 16
    for (int k = 0; k < K; ++k) z += Elem<T>::load(xr + k) * Elem<T>::load(wr + k);
    const float ls = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
    a[(size_t)t * N + n] = expf(ls * inv_tau);
}

extern "C" int tm_gla_gate_decay(const void* x, int ldx, const void* W, const void* bias, int dtype, float* a, int T, int N,
                                 int K, float tau, hipStream_t stream) {
    if (T <= 0 || N <= 0) return TM_OK;
    if (!x || !W || !a || K <= 0 || ldx < K || !(tau > 0.f) || T > 65535 * 32) return TM_ERR_ARG;
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int rows = T - t0 < 65535 ? T - t0 : 65535;
        const dim3 grid((N + 255) / 256, rows);
        if (dtype == TM_F32)
            gla_gate_decay_kernel<float><<<grid, 256, 0, stream>>>((const float*)x + (size_t)t0 * ldx, ldx, (const float*)W,
                                                                  (const float*)bias, a + (size_t)t0 * N, N, K, 1.0f / tau);
        else if (dtype == TM_BF16)
            gla_gate_decay_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x + (size_t)t0 * ldx, ldx, (const bf16_t*)W,
                                                                   (const bf16_t*)bias, a + (size_t)t0 * N, N, K, 1.0f / tau);
        else
            return TM_ERR_ARG;
        TM_CHECK_LAUNCH();
    }
    return TM_OK;
}

// ------------------------------------------------------------------------------------------------------------------
// A long portion in segments. The recurrence is linear in the state, so a segment's rows can be worked on before the
// state at its start is known: with the rows of a request cut into segments c = 0, 1, ...
//   L_c = the state the segment's own rows build from zero          (tm_gla_scan over the segments, from zero states)
//   P_c = the product of the segment's decays, per key channel      (gla_segment_decay)
//   B_0 = the request's state, B_(c+1) = diag(P_c) B_c + L_c        (gla_combine; the last one is the request's new state)
// and then every segment is scanned again from its true start B_c, all segments at once (tm_gla_scan once more).
// The chain over tokens becomes a chain over segments plus two scans that fill the chip.
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gla_segment_decay_kernel(const float* __restrict__ decay, const int* __restrict__ cu_seg,
                                                               float* __restrict__ P, int HD) {
    const int j = blockIdx.x * 256 + threadIdx.x, c = blockIdx.y;
    if (j >= HD) return;
    float p = 1.f;
    for (int t = cu_seg[c]; t < cu_seg[c + 1]; ++t) p *= decay[(size_t)t * HD + j];
    P[(size_t)c * HD + j] = p;
}

// grid (ceil(H * D * Dv / 256), S): element (h, d, e) of request s walks the request's segments first_seg[s] ..
// first_seg[s + 1] - 1 in order. local [n_seg, H, D, Dv] holds L_c; start receives B_c.
__global__ __launch_bounds__(256) void gla_combine_kernel(float* __restrict__ state, const int* __restrict__ state_slots,
                                                         const int* __restrict__ first_seg, const float* __restrict__ P,
                                                         const float* __restrict__ local, float* __restrict__ start, int HD,
                                                         int Dv) {
    const size_t per = (size_t)HD * Dv;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= per) return;
    const int s = blockIdx.y;
    const size_t hd = idx / Dv;
    float* st = state + (size_t)state_slots[s] * per + idx;
    float S = *st;
    for (int c = first_seg[s]; c < first_seg[s + 1]; ++c) {
        start[(size_t)c * per + idx] = S;
        S = P[(size_t)c * HD + hd] * S + local[(size_t)c * per + idx];
    }
    *st = S;
}

extern "C" int tm_gla_segment_decay(const float* decay, const int* cu_seg, float* P, int n_seg, int HD, hipStream_t stream) {
    if (n_seg <= 0) return TM_OK;
    if (!decay || !cu_seg || !P || HD <= 0 || n_seg > 65535) return TM_ERR_ARG;
    gla_segment_decay_kernel<<<dim3((HD + 255) / 256, n_seg), 256, 0, stream>>>(decay, cu_seg, P, HD);
    TM_CHECK_LAUNCH();
    return TM_OK;
}

extern "C" int tm_gla_combine(float* state, const int* state_slots, const int* first_seg, const float* P, const float* local,
                              float* start, int S, int HD, int Dv, hipStream_t stream) {
    if (S <= 0) return TM_OK;
    if (!state || !state_slots || !first_seg || !P || !local || !start || HD <= 0 || Dv <= 0 || S > 65535) return TM_ERR_ARG;
    const size_t per = (size_t)HD * Dv;
    gla_combine_kernel<<<dim3((unsigned)((per + 255) / 256), S), 256, 0, stream>>>(state, state_slots, first_seg, P, local, start, HD, Dv);
    TM_CHECK_LAUNCH();
    return TM_OK;
}
