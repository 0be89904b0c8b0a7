// The attention over a shared latent (latent.hip) on MFMA, bfloat16, for the prompt portions and the single tokens of a step.
//
// Every head reads the same cached rows, so a block stages a run of 32 rows in LDS once, as they lie (for the scores) and
// transposed (latent channels x rows, for the results), and works on up to HB tiles of 16 (token, head) pairs with them:
//   a prompt tile  : 16 consecutive tokens of one portion, HB heads one after the other;
//   a single token : its heads, 16 a tile.
// Per run of rows and tile:
//   S^T = K Q^T      A = rows  [16 rows x 32 d] from LDS, B = Q^T [32 d x 16 pairs] in registers; the d chunks are dealt to
//                    the block's four wavefronts, whose partial sums meet in LDS and are added in wavefront order
//   P   = 2^(S * scale * log2 e - m), zero where the row is not visible to the pair, running maximum m and sum l per pair
//   O^T = alpha O^T + C^T P^T   A = latent^T [16 channels x 32 rows] from LDS, B = P^T straight from the S^T accumulators;
//                    the latent's channels are dealt to the wavefronts in four equal ranges
// Runs are aligned to absolute positions and visited in ascending order, so a pair's result depends on its request's cache
// and its position only, in a prompt tile and alone alike.
#include "common.h"
#include "api.h"
#include "attention_prefill_common.h"

#define LM_WAVES 4
#define LM_KEYS 32
#define LM_PAD 8
#define LM_VT_STRIDE (LM_KEYS + LM_PAD)

template <int HB, int NDTW, int NCW>
__global__ __launch_bounds__(64 * LM_WAVES) void attn_latent_mfma_kernel(
    const bf16_t* __restrict__ qa, int q_stride, bf16_t* __restrict__ out, int out_stride, const bf16_t* __restrict__ pool,
    const int* __restrict__ block_tables, int table_width, const int* __restrict__ tiles, int prompt_blocks, int head_groups,
    const int* __restrict__ seq_of_token, const int* __restrict__ positions, int first_single, int H, int Lk, int Dk, int page,
    float scale_log2, int window) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int DKP = (Dk + 31) / 32 * 32, NDC = DKP / 32;
    const int ks_stride = DKP + LM_PAD;
    bf16_t* Ks = (bf16_t*)lds_raw;                                       // [32][DKP + 8]
    bf16_t* Vt = Ks + LM_KEYS * ks_stride;                               // [4 * NDTW * 16][40]
    float* Sp = (float*)(Vt + 4 * NDTW * 16 * LM_VT_STRIDE);             // [HB][4][32][16]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE);
    const int lane = threadIdx.x % TM_WAVE, r = lane % 16, g = lane / 16;

    // what this block works on
    int s, row0, valid, pos0, h0, single;
    if ((int)blockIdx.x < prompt_blocks) {
        const int* tl = tiles + (size_t)(blockIdx.x / head_groups) * 4;
        s = tl[0], row0 = tl[1], valid = tl[2], pos0 = tl[3];
        h0 = (blockIdx.x % head_groups) * HB;
        single = 0;
    } else {
        const int d = blockIdx.x - prompt_blocks;
        row0 = first_single + d / head_groups;
        s = seq_of_token[row0];
        pos0 = positions[row0];
        h0 = (d % head_groups) * HB * 16;
        valid = 1;
        single = 1;
    }
    const int* table = block_tables + (size_t)s * table_width;
    const int last_key = pos0 + valid - 1;
    const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    // pair (j, r): a prompt tile's token row0 + r with head h0 + j; a single token's head h0 + 16 j + r
    const int my_pos = single ? pos0 : (pos0 + r < last_key ? pos0 + r : last_key);
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;

    PFrag qf[HB][NCW];
    bool pair_ok[HB];
#pragma unroll
    for (int j = 0; j < HB; ++j) {
        const int head = single ? h0 + 16 * j + r : h0 + j;
        const int token = single ? row0 : row0 + r;
        pair_ok[j] = head < H && (single || r < valid);
#pragma unroll
        for (int cc = 0; cc < NCW; ++cc) {
            const int ch = 32 * (wave + LM_WAVES * cc) + 8 * g;
            if (pair_ok[j] && ch < Dk)
                qf[j][cc].u = *(const u32x4_t*)(qa + (size_t)token * q_stride + (size_t)head * Dk + ch);
            else
                qf[j][cc].u = u32x4_t{0, 0, 0, 0};
        }
    }
    float m[HB], l[HB];
    f32x4_t o[HB][NDTW];
#pragma unroll
    for (int j = 0; j < HB; ++j) {
        m[j] = -INFINITY;
        l[j] = 0.f;
#pragma unroll
        for (int d = 0; d < NDTW; ++d) o[j][d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    // tiles of this block that hold a pair at all (block-uniform)
    int n_tiles_here = 0;
#pragma unroll
    for (int j = 0; j < HB; ++j)
        if ((single ? h0 + 16 * j : h0 + j) < H) n_tiles_here = j + 1;

    const int pieces = DKP / 8;                                           // 16-byte pieces of a staged row
    for (int kb = first_key / LM_KEYS; kb <= last_key / LM_KEYS; ++kb) {
        __syncthreads();                                                  // the run before is done with
        for (int idx = threadIdx.x; idx < LM_KEYS * pieces; idx += 64 * LM_WAVES) {
            const int key = idx / pieces, c8 = idx % pieces;
            const int kj = kb * LM_KEYS + key;
            u32x4_t v = {0, 0, 0, 0};
            if (kj >= first_key && kj <= last_key && 8 * c8 < Dk) {
                const size_t slot = (size_t)table[kj / page] * page + kj % page;
                v = *(const u32x4_t*)(pool + slot * Dk + 8 * c8);
            }
            *(u32x4_t*)(Ks + key * ks_stride + 8 * c8) = v;
            if (8 * c8 < Lk) {                                            // Lk % 8 == 0: a piece lies wholly inside the latent or not
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    Vt[(8 * c8 + 2 * e) * LM_VT_STRIDE + key] = (bf16_t)(v[e] & 0xffffu);
                    Vt[(8 * c8 + 2 * e + 1) * LM_VT_STRIDE + key] = (bf16_t)(v[e] >> 16);
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < HB; ++j) {
            if (j >= n_tiles_here) continue;
            f32x4_t sc[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int cc = 0; cc < NCW; ++cc) {
                const int c = wave + LM_WAVES * cc;
                if (c >= NDC) continue;                                   // wave-uniform
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    PFrag kf;
                    kf.u = *(const u32x4_t*)(Ks + (16 * t + r) * ks_stride + 32 * c + 8 * g);
                    sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.b, qf[j][cc].b, sc[t], 0, 0, 0);
                }
            }
            float* sp = Sp + ((size_t)(j * LM_WAVES + wave) * LM_KEYS) * 16;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) sp[(16 * t + 4 * g + i) * 16 + r] = sc[t][i];
        }
        __syncthreads();
        const int key0 = kb * LM_KEYS;
#pragma unroll
        for (int j = 0; j < HB; ++j) {
            if (j >= n_tiles_here) continue;
            float sv[2][4];
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int k = 16 * t + 4 * g + i;
                    const float* sp = Sp + ((size_t)(j * LM_WAVES) * LM_KEYS + k) * 16 + r;
                    float v = sp[0];
#pragma unroll
                    for (int w = 1; w < LM_WAVES; ++w) v += sp[(size_t)w * LM_KEYS * 16];
                    v *= scale_log2;
                    const int kj = key0 + k;
                    if (kj > my_pos || kj < my_lo) v = -INFINITY;
                    sv[t][i] = v;
                    mx = fmaxf(mx, v);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, TM_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, TM_WAVE));
            const float m_new = fmaxf(m[j], mx);
            const float ref = m_new == -INFINITY ? 0.f : m_new;           // no row seen yet: every weight is zero
            const float alpha = __builtin_amdgcn_exp2f(m[j] - ref);
            m[j] = m_new;
            float pr[2][4], sum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pr[t][i] = __builtin_amdgcn_exp2f(sv[t][i] - ref);
                    sum += pr[t][i];
                }
            l[j] = l[j] * alpha + sum;
            PFrag pt;
            pt.u = u32x4_t{pk_bf16(pr[0][0], pr[0][1]), pk_bf16(pr[0][2], pr[0][3]), pk_bf16(pr[1][0], pr[1][1]),
                           pk_bf16(pr[1][2], pr[1][3])};
#pragma unroll
            for (int d = 0; d < NDTW; ++d) {
                const int dt = wave * NDTW + d;
                if (16 * dt >= Lk) continue;                              // wave-uniform
                o[j][d] *= alpha;
                const bf16_t* vrow = Vt + (16 * dt + r) * LM_VT_STRIDE + 4 * g;
                const u32x2_t v0 = *(const u32x2_t*)vrow, v1 = *(const u32x2_t*)(vrow + 16);
                PFrag vf;
                vf.u = u32x4_t{v0[0], v0[1], v1[0], v1[1]};
                o[j][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, o[j][d], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < HB; ++j) {
        if (j >= n_tiles_here) continue;
        float total = l[j];
        total += __shfl_xor(total, 16, TM_WAVE);
        total += __shfl_xor(total, 32, TM_WAVE);
        if (!pair_ok[j]) continue;
        const float inv = 1.0f / total;
        const int head = single ? h0 + 16 * j + r : h0 + j;
        const int token = single ? row0 : row0 + r;
        bf16_t* dst = out + (size_t)token * out_stride + (size_t)head * Lk;
#pragma unroll
        for (int d = 0; d < NDTW; ++d) {
            const int ch = 16 * (wave * NDTW + d) + 4 * g;
            if (ch >= Lk) continue;
            *(u32x2_t*)(dst + ch) = u32x2_t{pk_bf16(o[j][d][0] * inv, o[j][d][1] * inv), pk_bf16(o[j][d][2] * inv, o[j][d][3] * inv)};
        }
    }
}

static size_t lm_lds_bytes(int HB, int NDTW, int Dk) {
    const int DKP = (Dk + 31) / 32 * 32;
    return (size_t)LM_KEYS * (DKP + LM_PAD) * 2 + (size_t)4 * NDTW * 16 * LM_VT_STRIDE * 2 + (size_t)HB * LM_WAVES * LM_KEYS * 16 * 4;
}

// bfloat16; Dk and Lk multiples of 8 (16-byte pieces of a row lie inside the latent or outside it), rows of up to 704
// channels with up to 512 of latent.
extern "C" int tm_attn_latent_mfma_takes(int Lk, int Dk, int q_stride, int out_stride) {
    return Lk > 0 && Lk <= 512 && Dk >= Lk && Dk <= 704 && Lk % 8 == 0 && Dk % 8 == 0 && q_stride % 8 == 0 && out_stride % 4 == 0;
}

template <int HB, int NDTW, int NCW>
static int lm_launch(int blocks, size_t lds, hipStream_t stream, const bf16_t* qa, int q_stride, bf16_t* out, int out_stride,
                     const bf16_t* pool, const int* block_tables, int table_width, const int* tiles, int prompt_blocks,
                     int head_groups, const int* seq_of_token, const int* positions, int first_single, int H, int Lk, int Dk,
                     int page, float scale_log2, int window) {
    auto kernel = attn_latent_mfma_kernel<HB, NDTW, NCW>;
    static size_t allowed = 64 * 1024;                                   // per instantiation: the most LDS asked for so far
    if (lds > allowed) {
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return TM_ERR_LAUNCH;
        allowed = lds;
    }
    kernel<<<blocks, 64 * LM_WAVES, lds, stream>>>(qa, q_stride, out, out_stride, pool, block_tables, table_width, tiles,
                                                   prompt_blocks, head_groups, seq_of_token, positions, first_single, H, Lk, Dk,
                                                   page, scale_log2, window);
    return TM_OK;
}

// The prompt tiles of a step (tiles [n_tiles][4] as for tm_attn_prefill_mfma; n_tiles 0: none) or its single tokens (rows
// first_single .. first_single + n_single - 1 of the step; n_single 0: none); one of the two per call.
extern "C" int tm_attn_latent_mfma(const void* qa, int q_stride, void* out, int out_stride, const void* pool,
                                   const int* block_tables, int table_width, const int* tiles, int n_tiles,
                                   const int* seq_of_token, const int* positions, int first_single, int n_single, int H, int Lk,
                                   int Dk, int page, float scale, int window, hipStream_t stream) {
    if ((n_tiles > 0) == (n_single > 0)) return (n_tiles == 0 && n_single == 0) ? TM_OK : TM_ERR_ARG;
    if (!qa || !out || !pool || !block_tables || H <= 0 || page <= 0 || window < 0 || table_width <= 0 ||
        !tm_attn_latent_mfma_takes(Lk, Dk, q_stride, out_stride) || ((uintptr_t)qa % 16) || ((uintptr_t)out % 8) ||
        ((uintptr_t)pool % 16) || (long long)q_stride < (long long)H * Dk || (long long)out_stride < (long long)H * Lk ||
        (n_tiles > 0 && !tiles) || (n_single > 0 && (!seq_of_token || !positions)))
        return TM_ERR_ARG;
    const bool prompt = n_tiles > 0;
    const int per_block = prompt ? 1 : 16;                               // heads a tile of a block takes
    const int tiles_of_heads = (H + per_block - 1) / per_block;
    const int hb = tiles_of_heads >= 4 ? 4 : 1;
    const int head_groups = (tiles_of_heads + hb - 1) / hb;
    const long long blocks = (long long)(prompt ? n_tiles : n_single) * head_groups;
    if (blocks > 0x7fffffffLL) return TM_ERR_ARG;
    const int prompt_blocks = prompt ? (int)blocks : 0;
    const int ndtw = Lk <= 128 ? 2 : 8;
    const int ndc = (Dk + 31) / 32;
    const int ncw = ndc <= 8 ? 2 : 6;
    const size_t lds = lm_lds_bytes(hb, ndtw, Dk);
    const float scale_log2 = scale * 1.4426950408889634f;
    int rc;
#define LM_GO(HB_, NDTW_, NCW_)                                                                                                  \
    rc = lm_launch<HB_, NDTW_, NCW_>((int)blocks, lds, stream, (const bf16_t*)qa, q_stride, (bf16_t*)out, out_stride,          \
                                     (const bf16_t*)pool, block_tables, table_width, tiles, prompt_blocks, head_groups,        \
                                     seq_of_token, positions, first_single, H, Lk, Dk, page, scale_log2, window)
    if (hb == 4) {
        if (ndtw == 2) { if (ncw == 2) LM_GO(4, 2, 2); else LM_GO(4, 2, 6); }
        else { if (ncw == 2) LM_GO(4, 8, 2); else LM_GO(4, 8, 6); }
    } else {
        if (ndtw == 2) { if (ncw == 2) LM_GO(1, 2, 2); else LM_GO(1, 2, 6); }
        else { if (ncw == 2) LM_GO(1, 8, 2); else LM_GO(1, 8, 6); }
    }
#undef LM_GO
    if (rc != TM_OK) return rc;
    TM_CHECK_LAUNCH();
    return TM_OK;
}
