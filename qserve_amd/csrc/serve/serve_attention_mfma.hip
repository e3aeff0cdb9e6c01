// serve_attention_mfma.hip -- latent attention on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16), prompts and decoding.
//
// Work unit ("tile", made by the host): up to TPB consecutive tokens of ONE sequence in this step.  A workgroup of four waves
// serves a tile; a wave owns 32 query rows = TQ tokens x HP head slots (HP = heads rounded up to a power of two, at most 32;
// more than 32 heads: blockIdx.y walks head groups of 32).  Keys arrive in tiles of 32 cache rows, staged once per workgroup
// in LDS in two forms: row-major (A operand of S^T = K Q^T, plain 16-byte reads) and transposed (A operand of
// O^T = C^T P^T, 8-byte reads).  With the products swapped like this a lane holds 16 of the 32 scores of ITS query row, so
// the softmax needs one exchange with lane ^ 32 and the probabilities already sit in B-operand order (the k-slot <-> key
// mapping of the second product is chosen to match the accumulator layout of the first).
// A tile with few tokens (decoding: one) does not fill four waves with rows; then the waves split the KEY tiles among them and
// merge their partial softmax results through LDS at the end.
// Scores, running maxima and sums are float; q and the probabilities enter the matrix cores as bfloat16.
#include "serve_common.h"

namespace {
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

constexpr int NWV = 4;
constexpr int BN = 32;          // keys per tile
constexpr int VS = BN + 8;      // row stride (elements) of the transposed tile

__device__ __forceinline__ unsigned pack_bf2(float a, float b) { return (unsigned)f2bf(a) | ((unsigned)f2bf(b) << 16); }

template <int RT, int CT>
__global__ __launch_bounds__(64 * NWV) void latent_attention_mfma_kernel(
    bf16_t* __restrict__ out, const float* __restrict__ qf, const bf16_t* __restrict__ pool,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ pos, const int32_t* __restrict__ tiles,
    int window, int H, int rank, int R, int page, int HP, int TQ) {
    constexpr int RS = 16 * RT + 8;                      // row stride (elements) of the row-major tile
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16_t* Ks = (bf16_t*)smem;                          // [BN][RS]
    bf16_t* Vt = Ks + BN * RS;                           // [32 CT][VS]
    float* scratch = (float*)smem;                       // merge phase (after the key loop)

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int col = lane & 31, half = lane >> 5;
    const int slot = tiles[3 * blockIdx.x], t0 = tiles[3 * blockIdx.x + 1], ntok = tiles[3 * blockIdx.x + 2];
    const int h0 = blockIdx.y * 32;
    const int32_t* bt = block_table + (size_t)slot * table_stride;

    // rows of this wave: group g of TQ tokens, key split sp
    const int G = (ntok + TQ - 1) / TQ;                  // 1 .. 4
    const int S = NWV / G;
    const bool active = w < G * S;
    const int grp = active ? w % G : 0, sp = active ? w / G : 0;
    const int tok_in = grp * TQ + col / HP;              // token of this lane's query row within the tile
    const int head = h0 + col % HP;
    const bool row_ok = active && tok_in < ntok && (col % HP) < HP && head < H && (col / HP) < TQ;
    const int t = t0 + (tok_in < ntok ? tok_in : 0);
    const int p_row = pos[t];
    const int lo_row = window > 0 ? max(0, p_row - window + 1) : 0;

    // block key range (tokens of a tile are consecutive positions; read both ends)
    const int p_first = pos[t0], p_last = pos[t0 + ntok - 1];
    const int kstart = ((window > 0 ? max(0, p_first - window + 1) : 0) / BN) * BN;
    // wave key range: rows of this wave's group
    const int gt_first = min(grp * TQ, ntok - 1), gt_last = min(grp * TQ + TQ - 1, ntok - 1);
    const int wp_last = p_first + gt_last;
    const int wlo = window > 0 ? max(0, p_first + gt_first - window + 1) : 0;

    // Q fragments (B operand of S^T): 8 consecutive elements 16 s + 8 half of this lane's row
    v4u qfrag[RT];
    {
        const float* qrow = qf + ((size_t)t * H + (row_ok ? head : 0)) * (size_t)R;
#pragma unroll
        for (int s = 0; s < RT; ++s) {
            const int e0 = 16 * s + 8 * half;
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (row_ok && e0 + e < R) ? qrow[e0 + e] : 0.f;
            qfrag[s] = v4u{pack_bf2(v[0], v[1]), pack_bf2(v[2], v[3]), pack_bf2(v[4], v[5]), pack_bf2(v[6], v[7])};
        }
    }
    v16f oacc[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[c][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    const int chunks_per_row = R / 8;                    // 16-byte pieces of a cache row (R % 8 == 0)
    int ti = 0;
    for (int k0 = kstart; k0 <= p_last; k0 += BN, ++ti) {
        __syncthreads();                                 // the previous tile has been read
        // ---- stage 32 cache rows: row-major and transposed ----
        for (int q = tid; q < BN * 2 * RT; q += 64 * NWV) {
            const int row = q / (2 * RT), cc = q % (2 * RT);
            const int j = k0 + row;
            v4u d = {0u, 0u, 0u, 0u};
            if (j <= p_last && cc < chunks_per_row) {
                const bf16_t* src = pool + ((size_t)bt[j / page] * page + (size_t)(j % page)) * (size_t)R + cc * 8;
                d = *(const v4u*)src;
            }
            *(v4u*)(Ks + row * RS + cc * 8) = d;
            if (cc * 8 < 32 * CT) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    Vt[(cc * 8 + 2 * e) * VS + row] = (bf16_t)(d[e] & 0xffffu);
                    Vt[(cc * 8 + 2 * e + 1) * VS + row] = (bf16_t)(d[e] >> 16);
                }
            }
        }
        __syncthreads();
        if (!active || (ti % S) != sp || k0 > wp_last || k0 + BN - 1 < wlo) continue;   // (wave-uniform)
        // ---- S^T = K Q^T ----
        v16f sacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
#pragma unroll
        for (int s = 0; s < RT; ++s) {
            const v4u a = *(const v4u*)(Ks + col * RS + 16 * s + 8 * half);
            sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, qfrag[s]), sacc, 0, 0, 0);
        }
        // ---- mask + online softmax (this lane: 16 keys of its own query row) ----
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int key = k0 + 8 * (i >> 2) + 4 * half + (i & 3);
            const bool vis = key <= p_row && key >= lo_row;
            sacc[i] = vis ? sacc[i] : -INFINITY;
            tmax = fmaxf(tmax, sacc[i]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float mnew = fmaxf(m, tmax);
        const float msafe = mnew == -INFINITY ? 0.f : mnew;
        const float alpha = __expf(m - msafe);           // m = -inf: 0
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            sacc[i] = __expf(sacc[i] - msafe);
            psum += sacc[i];
        }
        l = l * alpha + psum;
        m = mnew;
#pragma unroll
        for (int c = 0; c < CT; ++c)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[c][i] *= alpha;
        // probabilities as B operand: k-slot (half, e) <-> key 16 s2 + 8 (e / 4) + 4 half + e % 4 = accumulator index 8 s2 + e
        v4u pb[2];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
            pb[s2] = v4u{pack_bf2(sacc[8 * s2 + 0], sacc[8 * s2 + 1]), pack_bf2(sacc[8 * s2 + 2], sacc[8 * s2 + 3]),
                         pack_bf2(sacc[8 * s2 + 4], sacc[8 * s2 + 5]), pack_bf2(sacc[8 * s2 + 6], sacc[8 * s2 + 7])};
        // ---- O^T += C^T P^T ----
#pragma unroll
        for (int c = 0; c < CT; ++c) {
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                const bf16_t* vrow = Vt + (32 * c + col) * VS + 16 * s2 + 4 * half;
                const v2u a0 = *(const v2u*)vrow, a1 = *(const v2u*)(vrow + 8);
                const v4u a = {a0[0], a0[1], a1[0], a1[1]};
                oacc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, pb[s2]), oacc[c], 0, 0, 0);
            }
        }
    }
    l += __shfl_xor(l, 32, 64);

    // ---- merge the key splits (waves grp + G s, s = 1 .. S - 1, into wave grp) ----
    if (S > 1) {                                         // (block-uniform)
        __syncthreads();                                 // the last tile has been read: LDS becomes scratch
        float* ml = scratch + NWV * 64 * 16;             // [NWV][64][2]
        if (active && sp > 0) {
            ml[(w * 64 + lane) * 2] = m;
            ml[(w * 64 + lane) * 2 + 1] = l;
        }
        __syncthreads();
        float f[NWV];
#pragma unroll
        for (int s = 0; s < NWV; ++s) f[s] = 0.f;
        if (active && sp == 0) {
            float M = m;
            for (int s = 1; s < S; ++s) M = fmaxf(M, ml[((grp + G * s) * 64 + lane) * 2]);
            const float Ms = M == -INFINITY ? 0.f : M;
            f[0] = __expf(m - Ms);
            float L = f[0] * l;
            for (int s = 1; s < S; ++s) {
                f[s] = __expf(ml[((grp + G * s) * 64 + lane) * 2] - Ms);
                L += f[s] * ml[((grp + G * s) * 64 + lane) * 2 + 1];
            }
            l = L;
        }
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            __syncthreads();
            if (active && sp > 0) {
#pragma unroll
                for (int i = 0; i < 16; ++i) scratch[(w * 64 + lane) * 16 + i] = oacc[c][i];
            }
            __syncthreads();
            if (active && sp == 0) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    float a = f[0] * oacc[c][i];
                    for (int s = 1; s < S; ++s) a += f[s] * scratch[((grp + G * s) * 64 + lane) * 16 + i];
                    oacc[c][i] = a;
                }
            }
        }
    }
    if (!row_ok || sp != 0) return;
    const float inv = 1.0f / l;
    bf16_t* o = out + ((size_t)t * H + head) * (size_t)rank;
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int c0 = 32 * c + 8 * b + 4 * half;
            if (c0 < rank) {                             // rank % 8 == 0: the four values are all inside
                const v2u v = {pack_bf2(oacc[c][4 * b] * inv, oacc[c][4 * b + 1] * inv),
                               pack_bf2(oacc[c][4 * b + 2] * inv, oacc[c][4 * b + 3] * inv)};
                *(v2u*)(o + c0) = v;
            }
        }
}

struct Geometry {
    int HP, TQ;
};
Geometry geometry(int H) {
    int hp = 1;
    while (hp < H && hp < 32) hp <<= 1;
    return {hp, 32 / hp};
}
}  // namespace

// Tokens of one sequence a work tile may hold, for `heads` heads (the host cuts a step's portions into tiles of this size).
extern "C" int qsv_latent_attention_tile_tokens(int heads) {
    if (heads <= 0) return 0;
    return NWV * geometry(heads).TQ;
}

// 1 if the matrix-core kernel takes these sizes (bfloat16 storage only), else 0 and the caller uses the wave kernel.
extern "C" int qsv_latent_attention_mfma_ok(int rank, int row_width, int dtype) {
    return dtype == QSV_BF16 && rank % 8 == 0 && row_width % 8 == 0 && row_width <= 576 && rank <= 512 && rank >= 8;
}

// tiles: int32 [n_tiles, 3] = (sequence slot, first flat token index, tokens <= qsv_latent_attention_tile_tokens(heads))
extern "C" int qsv_latent_attention_mfma(void* out, const float* qf, const void* pool, const int32_t* block_table,
                                         int table_stride, const int32_t* pos, const int32_t* tiles, int n_tiles, int window,
                                         int H, int rank, int R, int page, void* stream) {
    QSV_REQUIRE(out && qf && pool && block_table && pos && tiles, "qsv_latent_attention_mfma: null argument");
    QSV_REQUIRE(qsv_latent_attention_mfma_ok(rank, R, QSV_BF16) && R >= rank && H > 0 && page > 0 && window >= 0 && n_tiles >= 0,
                "qsv_latent_attention_mfma: sizes not supported (rank %d, row %d)", rank, R);
    if (n_tiles == 0) return QSV_OK;
    const Geometry g = geometry(H);
    const dim3 grid(n_tiles, (H + 31) / 32), block(64 * NWV);
    const int rt = (R + 15) / 16, ct = (rank + 31) / 32;
#define QSV_MFMA(RT, CT)                                                                                                     \
    do {                                                                                                                     \
        size_t lds = (size_t)(BN * (16 * RT + 8) + 32 * CT * VS) * 2;                                                        \
        const size_t need = (size_t)NWV * 64 * 18 * 4;                                                                       \
        if (lds < need) lds = need;                                                                                          \
        if (lds > 64 * 1024) {   /* above the default limit of dynamic LDS: raise it for this kernel */                        \
            const hipError_t e = hipFuncSetAttribute((const void*)latent_attention_mfma_kernel<RT, CT>,                      \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                  \
            QSV_REQUIRE(e == hipSuccess, "qsv_latent_attention_mfma: %s", hipGetErrorString(e));                             \
        }                                                                                                                    \
        hipLaunchKernelGGL((latent_attention_mfma_kernel<RT, CT>), grid, block, lds, (hipStream_t)stream, (bf16_t*)out, qf,  \
                           (const bf16_t*)pool, block_table, table_stride, pos, tiles, window, H, rank, R, page, g.HP, g.TQ); \
    } while (0)
    if (rt <= 8 && ct <= 4) QSV_MFMA(8, 4);
    else if (rt <= 12 && ct <= 6) QSV_MFMA(12, 6);
    else if (rt <= 20 && ct <= 8) QSV_MFMA(20, 8);
    else QSV_MFMA(36, 16);
#undef QSV_MFMA
    return qsv_launch_status("qsv_latent_attention_mfma");
}
