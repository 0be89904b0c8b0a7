// Attention whose weights are not normalized over the keys: a visible key j weighs sigmoid(scale * q.k_j + b_h)
// for query head h, and the output is the plain sum of the weighted values. Keys and values may have different
// sizes (D and Dv). What is visible: keys up to the query's own position, not before the start of the query's
// chunk (chunks of `chunk` positions counted from position 0 of the sequence; 0 = one chunk) and not further back
// than `window` positions (0 = any).
//
// Two kernels, for both storage types and any head sizes up to 256:
//   qk_norm_rope_store   per head RMS norm of q and k (weight shared by the heads), rotation of the first `rot`
//                        channels by the token's position, k and v to the token's cache slot
//   attn_sigmoid_paged   one wavefront per (token, head) over the paged cache; prompt portions and single tokens alike
//
// Everything between the loads and the stores is 32-bit. A token's result depends on its own request's cache and
// position only: keys are met in rounds of 64 from the first visible one, each lane sums its key's products in
// ascending d, and an output channel adds its keys in ascending order.
#include "common.h"
#include "api.h"

// qkv row = [H heads of q | G heads of k, D wide each | G heads of v, Dv wide]. K pool [pages, page, G, D]; V pool
// [pages, G, Dv, page]. grid (T, H + G + 1): a block per head of q and k, the last one stores v.
template <typename T>
__global__ __launch_bounds__(TM_WAVE) void qk_norm_rope_store_kernel(
    T* __restrict__ qkv, int ld, int H, int G, int D, int Dv, int rot, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ k_pool, T* __restrict__ v_pool,
    int page, int write_kv) {
    extern __shared__ float hs[];       // one head, [D]
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    T* row = qkv + (size_t)t * ld;
    const int slot = slots ? slots[t] : -1;
    const bool store = write_kv && slot >= 0;
    if (hh == H + G) {
        if (!store) return;
        const int pg = slot / page, in_page = slot % page;
        const T* v = row + (size_t)(H + G) * D;
        for (int idx = lane; idx < G * Dv; idx += TM_WAVE)
            v_pool[((size_t)pg * G * Dv + idx) * page + in_page] = v[idx];
        return;
    }
    T* x = row + (size_t)hh * D;
    const float* w = hh < H ? q_w : k_w;
    float ss = 0.f;
    for (int d = lane; d < D; d += TM_WAVE) {
        const float v = Elem<T>::load(x + d);
        hs[d] = v;
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = w ? 1.0f / sqrtf(ss / (float)D + eps) : 1.f;
    __syncthreads();
    for (int d = lane; d < D; d += TM_WAVE) hs[d] = w ? w[d] * (hs[d] * r) : hs[d];
    __syncthreads();
    T* kd = (store && hh >= H) ? k_pool + ((size_t)slot * G + (hh - H)) * D : nullptr;
    const int half = cos_t ? rot / 2 : 0;
    if (half) {
        const float* c = cos_t + (size_t)positions[t] * half;
        const float* s = sin_t + (size_t)positions[t] * half;
        for (int j = lane; j < half; j += TM_WAVE) {
            float y1, y2;
            rotate_pair(hs[j], hs[j + half], c[j], s[j], y1, y2);
            Elem<T>::store(x + j, y1);
            Elem<T>::store(x + j + half, y2);
            if (kd) {
                Elem<T>::store(kd + j, y1);
                Elem<T>::store(kd + j + half, y2);
            }
        }
    }
    for (int d = 2 * half + lane; d < D; d += TM_WAVE) {
        Elem<T>::store(x + d, hs[d]);
        if (kd) Elem<T>::store(kd + d, hs[d]);
    }
}

extern "C" int tm_qk_norm_rope_store(void* qkv, int ld, int dtype, int T, int H, int G, int D, int Dv, int rot,
                                     const float* q_w, const float* k_w, float eps, const float* cos_t,
                                     const float* sin_t, const int* positions, const int* slots, void* k_pool,
                                     void* v_pool, int page, int write_kv, hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (H <= 0 || G <= 0 || D <= 0 || Dv <= 0 || rot < 0 || rot > D || (rot & 1) || ld < (H + G) * D + G * Dv) return TM_ERR_ARG;
    if ((q_w == nullptr) != (k_w == nullptr) || (q_w && !(eps > 0.f))) return TM_ERR_ARG;
    if (cos_t && rot && (!sin_t || !positions)) return TM_ERR_ARG;
    if (write_kv && (!slots || !k_pool || !v_pool || page <= 0)) return TM_ERR_ARG;
    if (H + G + 1 > 65535) return TM_ERR_ARG;
    const dim3 grid(T, H + G + 1);
    const size_t lds = (size_t)D * sizeof(float);
    if (dtype == TM_F32)
        qk_norm_rope_store_kernel<float><<<grid, TM_WAVE, lds, stream>>>((float*)qkv, ld, H, G, D, Dv, rot, q_w, k_w, eps, cos_t,
                                                                        sin_t, positions, slots, (float*)k_pool,
                                                                        (float*)v_pool, page, write_kv);
    else if (dtype == TM_BF16)
        qk_norm_rope_store_kernel<bf16_t><<<grid, TM_WAVE, lds, stream>>>((bf16_t*)qkv, ld, H, G, D, Dv, rot, q_w, k_w, eps,
                                                                         cos_t, sin_t, positions, slots, (bf16_t*)k_pool,
                                                                         (bf16_t*)v_pool, page, write_kv);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}

#define SG_MAX_DV 256

__device__ __forceinline__ float sigmoid_f32(float s) { return 1.0f / (1.0f + expf(-s)); }

template <typename T>
__global__ __launch_bounds__(TM_WAVE) void attn_sigmoid_paged_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, const float* __restrict__ head_bias, int H,
    int G, int D, int Dv, int page, float scale, int chunk, int window, int split_keys, float* __restrict__ parts,
    size_t part_stride) {
    extern __shared__ float lds[];
    float* qs = lds;                            // [D]
    float* wl = lds + D;                        // [64] weights of a round's keys
    int* pl = (int*)(lds + D + TM_WAVE);        // [64] their pages
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (H / G);
    const int pos = positions[t];
    const int* tab = block_tables + (size_t)seq_of_token[t] * table_width;
    int lo = chunk > 0 ? (pos / chunk) * chunk : 0;
    if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
    // With `parts` the visible keys are dealt to blockIdx.z in runs of split_keys, counted from the first visible key, and
    // the runs' sums go to parts[z] in 32-bit for the caller to add up in the order of z (a run without keys gives zeros).
    int hi = pos;
    if (parts) {
        lo += (int)blockIdx.z * split_keys;
        if (lo + split_keys - 1 < hi) hi = lo + split_keys - 1;
    }
    const T* qr = q + (size_t)t * q_stride + (size_t)h * D;
    for (int d = lane; d < D; d += TM_WAVE) qs[d] = Elem<T>::load(qr + d);
    const float bias = head_bias ? head_bias[h] : 0.f;
    float acc[SG_MAX_DV / TM_WAVE] = {0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    for (int j0 = lo; j0 <= hi; j0 += TM_WAVE) {
        const int j = j0 + lane;
        const bool valid = j <= hi;
        const int pid = valid ? tab[j / page] : 0;
        float w = 0.f;
        if (valid) {
            const T* kr = k_pool + (((size_t)pid * page + j % page) * G + g) * D;
            float s = 0.f;
#pragma unroll 16
            for (int d = 0; d < D; ++d) s += qs[d] * Elem<T>::load(kr + d);       // sixteen loads in flight, added in ascending d
            w = sigmoid_f32(s * scale + bias);
        }
        wl[lane] = w;
        pl[lane] = pid;
        __syncthreads();
        const int n = min(TM_WAVE, hi - j0 + 1);
#pragma unroll
        for (int i = 0; i < SG_MAX_DV / TM_WAVE; ++i) {
            const int e = lane + TM_WAVE * i;
            if (e < Dv) {
                float a = acc[i];
#pragma unroll 16
                for (int jj = 0; jj < n; ++jj)
                    a += wl[jj] * Elem<T>::load(v_pool + (((size_t)pl[jj] * G + g) * Dv + e) * page + (j0 + jj) % page);
                acc[i] = a;
            }
        }
        __syncthreads();
    }
    if (parts) {
        float* po = parts + (size_t)blockIdx.z * part_stride + ((size_t)t * H + h) * Dv;
#pragma unroll
        for (int i = 0; i < SG_MAX_DV / TM_WAVE; ++i) {
            const int e = lane + TM_WAVE * i;
            if (e < Dv) po[e] = acc[i];
        }
        return;
    }
    T* o = out + (size_t)t * out_stride + (size_t)h * Dv;
#pragma unroll
    for (int i = 0; i < SG_MAX_DV / TM_WAVE; ++i) {
        const int e = lane + TM_WAVE * i;
        if (e < Dv) Elem<T>::store(o + e, acc[i]);
    }
}

// The same kernel for sizes whose key rows and pages come in whole 16-byte pieces (D and the page size multiples of
// 16 / sizeof(T)): a key's row is read by eight lanes in 16-byte pieces (eight keys a step, all of a round's loads
// in flight at once) and a value channel reads its keys 16 bytes at a time, so a round is a few trips to memory instead
// of a hundred small dependent ones. The scores' sums are ordered otherwise than in the kernel above (a lane's pieces in
// ascending order, then the eight lanes by a fixed tree); which of the two kernels runs follows from the model's sizes.
template <typename T>
__global__ __launch_bounds__(TM_WAVE) void attn_sigmoid_paged_vec_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int* __restrict__ block_tables, int table_width,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, const float* __restrict__ head_bias, int H,
    int G, int D, int Dv, int page, float scale, int chunk, int window, int split_keys, float* __restrict__ parts,
    size_t part_stride) {
    constexpr int EV = Piece<T>::N;
    extern __shared__ float lds[];
    float* qs = lds;                            // [D]
    float* wl = lds + D;                        // [64] weights of a round's keys
    int* pl = (int*)(lds + D + TM_WAVE);        // [64] their pages
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (H / G);
    const int pos = positions[t];
    const int* tab = block_tables + (size_t)seq_of_token[t] * table_width;
    int lo = chunk > 0 ? (pos / chunk) * chunk : 0;
    if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
    int hi = pos;
    if (parts) {
        lo += (int)blockIdx.z * split_keys;
        if (lo + split_keys - 1 < hi) hi = lo + split_keys - 1;
    }
    const T* qr = q + (size_t)t * q_stride + (size_t)h * D;
    for (int d = lane; d < D; d += TM_WAVE) qs[d] = Elem<T>::load(qr + d);
    const float bias = head_bias ? head_bias[h] : 0.f;
    float acc[SG_MAX_DV / TM_WAVE] = {0.f, 0.f, 0.f, 0.f};
    const int kk = lane / 8, piece = lane % 8;  // eight lanes a key, eight keys a step
    const int np = D / EV;
    __syncthreads();
    for (int j0 = lo; j0 <= hi; j0 += TM_WAVE) {
#pragma unroll
        for (int ss = 0; ss < 8; ++ss) {
            const int jj = ss * 8 + kk, j = j0 + jj;
            const bool valid = j <= hi;
            const int pid = valid ? tab[j / page] : 0;
            float part = 0.f;
            if (valid) {
                const T* kr = k_pool + (((size_t)pid * page + j % page) * G + g) * D;
                for (int p = piece; p < np; p += 8) {
                    float kf[EV];
                    Piece<T>::unpack(*(const uint4*)(kr + p * EV), kf);
#pragma unroll
                    for (int i = 0; i < EV; ++i) part += qs[p * EV + i] * kf[i];
                }
            }
            part += __shfl_xor(part, 1, TM_WAVE);
            part += __shfl_xor(part, 2, TM_WAVE);
            part += __shfl_xor(part, 4, TM_WAVE);
            if (piece == 0) {
                wl[jj] = valid ? sigmoid_f32(part * scale + bias) : 0.f;
                pl[jj] = pid;
            }
        }
        __syncthreads();
        const int n = min(TM_WAVE, hi - j0 + 1);
        const int head = min(n, (EV - j0 % EV) % EV);       // keys before the first that starts a 16-byte piece
        const int pieces = (n - head) / EV;
#pragma unroll
        for (int i = 0; i < SG_MAX_DV / TM_WAVE; ++i) {
            const int e = lane + TM_WAVE * i;
            if (e < Dv) {
                float a = acc[i];
                int jj = 0;
                for (; jj < head; ++jj)
                    a += wl[jj] * Elem<T>::load(v_pool + (((size_t)pl[jj] * G + g) * Dv + e) * page + (j0 + jj) % page);
#pragma unroll 4
                for (int pc = 0; pc < pieces; ++pc, jj += EV) {
                    float vf[EV];
                    Piece<T>::unpack(*(const uint4*)(v_pool + (((size_t)pl[jj] * G + g) * Dv + e) * page + (j0 + jj) % page), vf);
#pragma unroll
                    for (int k = 0; k < EV; ++k) a += wl[jj + k] * vf[k];
                }
                for (; jj < n; ++jj)
                    a += wl[jj] * Elem<T>::load(v_pool + (((size_t)pl[jj] * G + g) * Dv + e) * page + (j0 + jj) % page);
                acc[i] = a;
            }
        }
        __syncthreads();
    }
    if (parts) {
        float* po = parts + (size_t)blockIdx.z * part_stride + ((size_t)t * H + h) * Dv;
#pragma unroll
        for (int i = 0; i < SG_MAX_DV / TM_WAVE; ++i) {
            const int e = lane + TM_WAVE * i;
            if (e < Dv) po[e] = acc[i];
        }
        return;
    }
    T* o = out + (size_t)t * out_stride + (size_t)h * Dv;
#pragma unroll
    for (int i = 0; i < SG_MAX_DV / TM_WAVE; ++i) {
        const int e = lane + TM_WAVE * i;
        if (e < Dv) Elem<T>::store(o + e, acc[i]);
    }
}

template <typename T>
static bool sigmoid_in_pieces(const void* k_pool, const void* v_pool, int D, int page) {
    constexpr int EV = Piece<T>::N;
    return D % EV == 0 && page % EV == 0 && ((uintptr_t)k_pool % 16) == 0 && ((uintptr_t)v_pool % 16) == 0;
}

// n_splits > 0: the keys of every token in runs of split_keys over grid.z, 32-bit sums to parts [n_splits][T][H * Dv]
// (`out` is not written; tm_sum_parts adds them up).
extern "C" int tm_attn_sigmoid_paged(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                     const void* v_pool, const int* block_tables, int table_width, const int* seq_of_token,
                                     const int* positions, const float* head_bias, int T, int H, int G, int D, int Dv, int page,
                                     float scale, int chunk, int window, int dtype, int split_keys, int n_splits, float* parts,
                                     hipStream_t stream) {
    if (T <= 0) return TM_OK;
    if (H <= 0 || G <= 0 || H % G || D <= 0 || D > 256 || Dv <= 0 || Dv > SG_MAX_DV || page <= 0 || chunk < 0 || window < 0 ||
        table_width <= 0 || q_stride < H * D || out_stride < H * Dv || H > 65535)
        return TM_ERR_ARG;
    if (n_splits < 0 || n_splits > 65535 || (n_splits > 0 && (split_keys <= 0 || !parts))) return TM_ERR_ARG;
    const dim3 grid(T, H, n_splits > 0 ? n_splits : 1);
    float* pp = n_splits > 0 ? parts : nullptr;
    const size_t part_stride = (size_t)T * H * Dv;
    const size_t lds = ((size_t)D + 2 * TM_WAVE) * sizeof(float);
    if (dtype == TM_F32 && sigmoid_in_pieces<float>(k_pool, v_pool, D, page))
        attn_sigmoid_paged_vec_kernel<float><<<grid, TM_WAVE, lds, stream>>>(
            (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_pool, (const float*)v_pool, block_tables,
            table_width, seq_of_token, positions, head_bias, H, G, D, Dv, page, scale, chunk, window, split_keys, pp, part_stride);
    else if (dtype == TM_BF16 && sigmoid_in_pieces<bf16_t>(k_pool, v_pool, D, page))
        attn_sigmoid_paged_vec_kernel<bf16_t><<<grid, TM_WAVE, lds, stream>>>(
            (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_tables,
            table_width, seq_of_token, positions, head_bias, H, G, D, Dv, page, scale, chunk, window, split_keys, pp, part_stride);
    else if (dtype == TM_F32)
        attn_sigmoid_paged_kernel<float><<<grid, TM_WAVE, lds, stream>>>(
            (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_pool, (const float*)v_pool, block_tables,
            table_width, seq_of_token, positions, head_bias, H, G, D, Dv, page, scale, chunk, window, split_keys, pp, part_stride);
    else if (dtype == TM_BF16)
        attn_sigmoid_paged_kernel<bf16_t><<<grid, TM_WAVE, lds, stream>>>(
            (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_tables,
            table_width, seq_of_token, positions, head_bias, H, G, D, Dv, page, scale, chunk, window, split_keys, pp, part_stride);
    else
        return TM_ERR_ARG;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
