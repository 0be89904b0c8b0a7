// The sigmoid-weight attention (attention_sigmoid.hip) for portions of prompts on MFMA, bfloat16.
//
// There is no softmax, so nothing is carried from one block of keys to the next but the sum itself: a block of 32
// keys is two products with the weights computed on the vector unit between them,
//
//   S^T = K Q^T      A = keys  [16 keys x 32 d]   from K[page][slot][g][d]
//                    B = Q^T   [32 d x 16 tokens]
//   P   = sigmoid(scale * S + b_h), zero where the key is not visible, rounded to bfloat16
//   O^T += V^T P^T   A = V^T   [16 dv x 32 keys]  from V[page][g][dv][slot]
//                    B = P^T   [32 keys x 16 tokens] straight from the S^T accumulators
//
// with the tile of 16 query tokens, the pairing of heads that share a kv head in one wavefront, the key blocks
// aligned to absolute positions and dealt to the block's wavefronts by (block index mod wavefronts), and the paged
// loads of the softmax prefill kernel (attention_prefill.hip). A token's result depends on its request's cache and
// its position only: its visible keys always fall into the same blocks, the same wavefronts, and the wavefronts'
// sums are added in their order.
//
// Head sizes: D a multiple of 8 up to 128 (padded with zeros to a multiple of 32 in registers), Dv a multiple of 4 up
// to 128 (rows beyond Dv repeat the last one and are not stored).
#include "common.h"
#include "api.h"
#include "attention_prefill_common.h"

#define SP_HPW 2            // query heads of one kv head a wavefront takes
#define SP_KS 4             // wavefronts of a block, sharing the key blocks of a tile

template <int DP, int DVP>
struct SgBlock {
    PFrag k[2][DP / 32];        // [16-key tile][d chunk]
    u32x2_t v[DVP / 16][2];     // [dv tile][16-key tile]: 4 keys each
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t sg_uniform_buffer(const void* base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}

// page and place in the page of 16-key tile `tile`, clamped to the tiles some query of the wavefront can see
__device__ __forceinline__ void sg_tile_place(int tile, int first_tile, int last_tile, const int* __restrict__ table,
                                              int page_shift, int& pg, int& in_page) {
    tile = tile < first_tile ? first_tile : (tile > last_tile ? last_tile : tile);
    const int t0 = 16 * tile;
    pg = table[t0 >> page_shift];
    in_page = t0 & ((1 << page_shift) - 1);
}

template <int DP, int DVP>
__device__ __forceinline__ void sg_load_block(SgBlock<DP, DVP>& blk, int kb, int first_tile, int last_tile,
                                              const int* __restrict__ table, const bf16_t* __restrict__ k_pool,
                                              const bf16_t* __restrict__ v_pool, int g_kv, int G, int D, int DV,
                                              int page_shift, int r, int g) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        // A tile no query of the wavefront can see (wholly before the first visible key, or beyond the newest) is not
        // loaded: its place in the table may name no page, and what another tile's slots hold beyond the newest key
        // can be anything. Its keys and values are zeros; its weights are masked by position like any other's.
        if (2 * kb + t < first_tile || 2 * kb + t > last_tile) {
#pragma unroll
            for (int c = 0; c < DP / 32; ++c) blk.k[t][c].u = u32x4_t{0, 0, 0, 0};
#pragma unroll
            for (int dt = 0; dt < DVP / 16; ++dt) blk.v[dt][t] = u32x2_t{0, 0};
            continue;
        }
        int pg, in_page;
        sg_tile_place(2 * kb + t, first_tile, last_tile, table, page_shift, pg, in_page);
        pg = __builtin_amdgcn_readfirstlane(pg);
        in_page = __builtin_amdgcn_readfirstlane(in_page);
        const __amdgpu_buffer_rsrc_t kbuf = sg_uniform_buffer(k_pool + ((((size_t)pg << page_shift) + in_page) * G + g_kv) * D);
        const __amdgpu_buffer_rsrc_t vbuf = sg_uniform_buffer(v_pool + ((((size_t)pg * G + g_kv) * DV) << page_shift) + in_page);
        const uint32_t koff = (uint32_t)(((size_t)r * G * D + 8 * g) * sizeof(bf16_t));
#pragma unroll
        for (int c = 0; c < DP / 32; ++c) {
            // a lane's 8 channels lie wholly inside the head or wholly in the padding (D % 8 == 0)
            if (32 * c + 8 * g < D)
                blk.k[t][c].u = __builtin_amdgcn_raw_buffer_load_b128(kbuf, koff, 64 * c, 0);
            else
                blk.k[t][c].u = u32x4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int dt = 0; dt < DVP / 16; ++dt) {
            const int row = min(16 * dt + r, DV - 1);
            const uint32_t voff = (uint32_t)((((size_t)row << page_shift) + 4 * g) * sizeof(bf16_t));
            blk.v[dt][t] = __builtin_amdgcn_raw_buffer_load_b64(vbuf, voff, 0, 0);
        }
    }
}

struct SgTile {
    int pos0, last_key, last_lo, my_pos, my_lo;
};

template <int DP, int DVP>
__device__ __forceinline__ void sg_attend_block(SgBlock<DP, DVP>& blk, f32x4_t (&o)[SP_HPW][DVP / 16],
                                                const PFrag (&qf)[SP_HPW][DP / 32], int key0, int nh, const SgTile& tv, int g,
                                                float scale_log2, const float (&bias_log2)[SP_HPW]) {
    constexpr int NDC = DP / 32, NDT = DVP / 16;
    // values of keys nobody may see yet (beyond the newest key) can hold anything: clear them
    if (key0 + 31 > tv.last_key) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int k0 = key0 + 16 * t + 4 * g;
            const uint32_t keep0 = ((k0 <= tv.last_key) ? 0x0000ffffu : 0u) | ((k0 + 1 <= tv.last_key) ? 0xffff0000u : 0u);
            const uint32_t keep1 = ((k0 + 2 <= tv.last_key) ? 0x0000ffffu : 0u) | ((k0 + 3 <= tv.last_key) ? 0xffff0000u : 0u);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                blk.v[dt][t][0] &= keep0;
                blk.v[dt][t][1] &= keep1;
            }
        }
    }
    const bool edge = (key0 + 31 > tv.pos0) || (key0 < tv.last_lo);
    f32x4_t sc[SP_HPW][2];
#pragma unroll
    for (int hh = 0; hh < SP_HPW; ++hh) {
        if (hh >= nh) continue;                                  // wave-uniform
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NDC; ++c)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[t][c].b, qf[hh][c].b, acc, 0, 0, 0);
            sc[hh][t] = acc;
        }
    }
#pragma unroll
    for (int hh = 0; hh < SP_HPW; ++hh) {
        if (hh >= nh) continue;
        float pr[2][4];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // sigmoid(x) = 1 / (1 + 2^(-x log2 e)), x = scale * s + b
                const float e = __builtin_amdgcn_exp2f(-fmaf(sc[hh][t][i], scale_log2, bias_log2[hh]));
                float p = __builtin_amdgcn_rcpf(1.0f + e);
                if (edge) {
                    const int kj = key0 + 16 * t + 4 * g + i;
                    if (kj > tv.my_pos || kj < tv.my_lo) p = 0.f;
                }
                pr[t][i] = p;
            }
        PFrag pt;
        pt.u = u32x4_t{pk_bf16(pr[0][0], pr[0][1]), pk_bf16(pr[0][2], pr[0][3]), pk_bf16(pr[1][0], pr[1][1]),
                       pk_bf16(pr[1][2], pr[1][3])};
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            PFrag vf;
            vf.u = u32x4_t{blk.v[dt][0][0], blk.v[dt][0][1], blk.v[dt][1][0], blk.v[dt][1][1]};
            o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.b, pt.b, o[hh][dt], 0, 0, 0);
        }
    }
}

// tiles: int32 [n_tiles][4] = (request index in the step, first row of the tile in the flat batch, tokens in the
// tile (1..16), position of its first token). grid (n_tiles, G * ceil(H / G / SP_HPW)), SP_KS wavefronts a block.
template <int DP, int DVP>
__global__ __launch_bounds__(64 * SP_KS) void attn_sigmoid_prefill_kernel(
    const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int* __restrict__ block_tables, int table_width, const int* __restrict__ tiles,
    const float* __restrict__ head_bias, int H, int G, int D, int DV, int page_shift, float scale_log2, int chunk, int window) {
    constexpr int NDC = DP / 32, NDT = DVP / 16;
    __shared__ float s_o[SP_KS][16][DVP + 1];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / TM_WAVE);
    const int lane = threadIdx.x % TM_WAVE, r = lane % 16, g = lane / 16;
    const int rep = H / G;
    const int splits = (rep + SP_HPW - 1) / SP_HPW;
    const int g_kv = blockIdx.y / splits, split = blockIdx.y % splits;
    const int h0 = g_kv * rep + split * SP_HPW;
    const int nh = (rep - split * SP_HPW) < SP_HPW ? (rep - split * SP_HPW) : SP_HPW;
    const int* tl = tiles + (size_t)blockIdx.x * 4;
    const int s = tl[0], row0 = tl[1], valid = tl[2], pos0 = tl[3];
    const int* table = block_tables + (size_t)s * table_width;

    auto lowest = [&](int pos) {
        int lo = chunk > 0 ? (pos / chunk) * chunk : 0;
        if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
        return lo;
    };
    SgTile tv;
    tv.pos0 = pos0;
    tv.last_key = pos0 + valid - 1;
    tv.my_pos = pos0 + r < tv.last_key ? pos0 + r : tv.last_key;
    tv.my_lo = lowest(tv.my_pos);
    tv.last_lo = lowest(tv.last_key);
    const int first_key = lowest(pos0);
    const int kb0 = first_key / 32, kb1 = tv.last_key / 32;
    const int first_tile = first_key / 16, last_tile = tv.last_key / 16;

    PFrag qf[SP_HPW][NDC];
    float bias_log2[SP_HPW];
#pragma unroll
    for (int hh = 0; hh < SP_HPW; ++hh) {
        bias_log2[hh] = (hh < nh && head_bias) ? head_bias[h0 + hh] * 1.4426950408889634f : 0.f;
#pragma unroll
        for (int c = 0; c < NDC; ++c) {
            if (hh < nh && r < valid && 32 * c + 8 * g < D)
                qf[hh][c].u = *(const u32x4_t*)(q + (size_t)(row0 + r) * q_stride + (size_t)(h0 + hh) * D + 32 * c + 8 * g);
            else
                qf[hh][c].u = u32x4_t{0, 0, 0, 0};
        }
    }
    f32x4_t o[SP_HPW][NDT];
#pragma unroll
    for (int hh = 0; hh < SP_HPW; ++hh)
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) o[hh][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // two register sets take turns: one is worked on while the other's loads are in flight
    int kb = kb0 + ((wave - kb0) & (SP_KS - 1));                     // first block >= kb0 of this wavefront
    SgBlock<DP, DVP> ba, bb;
    if (kb <= kb1) sg_load_block<DP, DVP>(ba, kb, first_tile, last_tile, table, k_pool, v_pool, g_kv, G, D, DV, page_shift, r, g);
    while (kb <= kb1) {
        sg_load_block<DP, DVP>(bb, kb + SP_KS, first_tile, last_tile, table, k_pool, v_pool, g_kv, G, D, DV, page_shift, r, g);
        sg_attend_block<DP, DVP>(ba, o, qf, kb * 32, nh, tv, g, scale_log2, bias_log2);
        kb += SP_KS;
        if (kb > kb1) break;
        sg_load_block<DP, DVP>(ba, kb + SP_KS, first_tile, last_tile, table, k_pool, v_pool, g_kv, G, D, DV, page_shift, r, g);
        sg_attend_block<DP, DVP>(bb, o, qf, kb * 32, nh, tv, g, scale_log2, bias_log2);
        kb += SP_KS;
    }

    // add the wavefronts' sums head by head, in wavefront order; lane: dv = 16 dt + 4 g + i of token r
#pragma unroll
    for (int hh = 0; hh < SP_HPW; ++hh) {
        if (hh >= nh) continue;                                      // block-uniform
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s_o[wave][r][16 * dt + 4 * g + i] = o[hh][dt][i];
        __syncthreads();
        for (int idx = threadIdx.x; idx < 16 * (DV / 2); idx += 64 * SP_KS) {
            const int col = idx / (DV / 2), d = 2 * (idx % (DV / 2));
            if (col >= valid) continue;
            float o0 = s_o[0][col][d], o1 = s_o[0][col][d + 1];
#pragma unroll
            for (int w = 1; w < SP_KS; ++w) {
                o0 += s_o[w][col][d];
                o1 += s_o[w][col][d + 1];
            }
            *(uint32_t*)(out + (size_t)(row0 + col) * out_stride + (size_t)(h0 + hh) * DV + d) = pk_bf16(o0, o1);
        }
        __syncthreads();
    }
}

extern "C" int tm_attn_sigmoid_prefill_takes(int D, int DV, int page, int q_stride) {
    return D > 0 && D <= 128 && D % 8 == 0 && DV > 0 && DV <= 128 && DV % 4 == 0 && page >= 16 && !(page & (page - 1)) &&
           q_stride % 8 == 0;
}

extern "C" int tm_attn_sigmoid_prefill(const void* q, int q_stride, void* out, int out_stride, const void* k_pool,
                                       const void* v_pool, const int* block_tables, int table_width, const int* tiles,
                                       int n_tiles, const float* head_bias, int H, int G, int D, int DV, int page, float scale,
                                       int chunk, int window, hipStream_t stream) {
    if (n_tiles <= 0) return TM_OK;
    if (H <= 0 || G <= 0 || H % G || !tm_attn_sigmoid_prefill_takes(D, DV, page, q_stride) || chunk < 0 || window < 0 ||
        table_width <= 0 || ((uintptr_t)q % 16) || (out_stride % 2) || ((uintptr_t)out % 4) || q_stride < H * D ||
        out_stride < H * DV)
        return TM_ERR_ARG;
    int page_shift = 0;
    while ((1 << page_shift) < page) ++page_shift;
    const int splits = (H / G + SP_HPW - 1) / SP_HPW;
    if ((long long)G * splits > 65535) return TM_ERR_ARG;
    const dim3 grid(n_tiles, G * splits);
    const float scale_log2 = scale * 1.4426950408889634f;
    const int dp = (D + 31) / 32 * 32;
    const int dvp = DV <= 32 ? 32 : (DV <= 64 ? 64 : 128);
#define SG_LAUNCH(DP_, DVP_)                                                                                              \
    attn_sigmoid_prefill_kernel<DP_, DVP_><<<grid, 64 * SP_KS, 0, stream>>>(                                               \
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_tables, \
        table_width, tiles, head_bias, H, G, D, DV, page_shift, scale_log2, chunk, window)
#define SG_CASE(DP_)                                   \
    case DP_:                                          \
        if (dvp == 32) SG_LAUNCH(DP_, 32);             \
        else if (dvp == 64) SG_LAUNCH(DP_, 64);        \
        else SG_LAUNCH(DP_, 128);                      \
        break;
    switch (dp) {
        SG_CASE(32)
        SG_CASE(64)
        SG_CASE(96)
        SG_CASE(128)
        default:
            return TM_ERR_ARG;
    }
#undef SG_CASE
#undef SG_LAUNCH
    TM_CHECK_LAUNCH();
    return TM_OK;
}
