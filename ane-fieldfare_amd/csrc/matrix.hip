// Resident INT4 matrix: a [M][N] weight in the reference's row-major layout is re-tiled once into
// two-stream tiles and then serves 1..16 input rows per call at streaming speed, with an optional
// greedy choice (argmax) over the outputs.
//
// Replaces the LM head of LMHeadChainInt4.encodeGreedyDecode / encodeGreedyRows
// (Kernels/Fusions/LMHeadChainInt4.swift:94-139,225-284; Metal/Sampling/logit.metal:614-720,952-1005) and the
// static-weight uses of DequantInt4GEMV.encodeRows (Kernels/Quant/DequantInt4GEMV.swift:72-182).
// A tile holds rows a = 32 p + l % 16 (stream A) and a + 16 (stream B) of one 64-wide group, in the
// same lane order as the expert arena, so the kernels share the expert path's register-ring code.
//
// An 8-bit affine weight (Metal/Quant/dequant_int8.metal:5-12: w = q s + b, q = 0 .. 255) rides the same kernels as two
// 4-bit ones: q = 16 h + l, so w = (16 s) h + b + s l. A tile then holds rows 16 p + l % 16 twice - stream A their
// high nibbles with scale 16 s (exact: a power of two) and bias b, stream B their low nibbles with scale s and bias
// 0 - and an output is the sum of its two streams. Same bytes as the 8-bit matrix, same stream, same speed.
#include "common.hpp"
#include "kernels.hpp"
#include "stream.hpp"

namespace ffmoe {
namespace {

__device__ __forceinline__ uint32_t ref_nibbles8(const uint8_t *row, uint32_t k0) {
    const uint8_t *p = row + (k0 >> 1);
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

// reference order (nibble j = element j) -> arena order (position m = element 2m, m + 4 = element 2m + 1)
__device__ __forceinline__ uint32_t to_arena_order(uint32_t v) {
    uint32_t out = 0;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        out |= ((v >> (8 * m)) & 0xFu) << (4 * m);
        out |= ((v >> (8 * m + 4)) & 0xFu) << (4 * m + 16);
    }
    return out;
}

__device__ __forceinline__ uint16_t load_u16(const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }

// One thread per (tile, lane). Rows past M (M is padded up to a multiple of 32) become zero weights
// with zero scale and bias.
__global__ __launch_bounds__(256) void repack_matrix_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ s,
                                                            const uint8_t *__restrict__ b, uint32_t m, uint32_t n,
                                                            uint8_t *__restrict__ tiles, uint8_t *__restrict__ scales) {
    const uint32_t n_groups = n / kGroup, row_bytes = n / 2;
    const size_t n_tiles = (size_t)((m + 31) / 32) * n_groups;
    const size_t total = n_tiles * kWave;
    for (size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total;
         gid += (size_t)gridDim.x * blockDim.x) {
        const uint32_t lane = gid & 63, i = lane & 15, jq = lane >> 4;
        const size_t tile = gid >> 6;
        const uint32_t rbp = tile / n_groups, grp = tile % n_groups;
        const uint32_t row_a = rbp * 2 * kTileRows + i, row_b = row_a + kTileRows;
        const uint32_t k0 = grp * kGroup + 8 * jq;
        uint4 chunk = {0, 0, 0, 0};
        if (row_a < m) {
            chunk.x = to_arena_order(ref_nibbles8(w + (size_t)row_a * row_bytes, k0));
            chunk.y = to_arena_order(ref_nibbles8(w + (size_t)row_a * row_bytes, k0 + 32));
        }
        if (row_b < m) {
            chunk.z = to_arena_order(ref_nibbles8(w + (size_t)row_b * row_bytes, k0));
            chunk.w = to_arena_order(ref_nibbles8(w + (size_t)row_b * row_bytes, k0 + 32));
        }
        reinterpret_cast<uint4 *>(tiles + tile * kTileBytes)[lane] = chunk;
        if (jq == 0) {
            uint2 sc = {0, 0};
            const size_t ia = ((size_t)row_a * n_groups + grp) * 2, ib = ((size_t)row_b * n_groups + grp) * 2;
            if (row_a < m) sc.x = (uint32_t)load_u16(s + ia) | ((uint32_t)load_u16(b + ia) << 16);
            if (row_b < m) sc.y = (uint32_t)load_u16(s + ib) | ((uint32_t)load_u16(b + ib) << 16);
            reinterpret_cast<uint2 *>(scales + tile * kTileScaleBytes)[i] = sc;
        }
    }
}

// The 8-bit form: w uint8 [m][n]. One thread per (tile, lane); a tile = 16 rows x one group, both nibble planes.
__device__ __forceinline__ void nibble_planes8(const uint8_t *p, uint32_t &high, uint32_t &low) {
    high = low = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        high |= (uint32_t)(p[i] >> 4) << (4 * i);
        low |= (uint32_t)(p[i] & 15u) << (4 * i);
    }
}

__global__ __launch_bounds__(256) void repack_matrix8_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ s,
                                                             const uint8_t *__restrict__ b, uint32_t m, uint32_t n,
                                                             uint8_t *__restrict__ tiles, uint8_t *__restrict__ scales) {
    const uint32_t n_groups = n / kGroup;
    const size_t n_tiles = (size_t)((m + 15) / 16) * n_groups;
    const size_t total = n_tiles * kWave;
    for (size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gid < total;
         gid += (size_t)gridDim.x * blockDim.x) {
        const uint32_t lane = gid & 63, i = lane & 15, jq = lane >> 4;
        const size_t tile = gid >> 6;
        const uint32_t rb = tile / n_groups, grp = tile % n_groups;
        const uint32_t row = rb * kTileRows + i, k0 = grp * kGroup + 8 * jq;
        uint4 chunk = {0, 0, 0, 0};
        if (row < m) {
            uint32_t h0, l0, h1, l1;
            nibble_planes8(w + (size_t)row * n + k0, h0, l0);
            nibble_planes8(w + (size_t)row * n + k0 + 32, h1, l1);
            chunk = uint4{to_arena_order(h0), to_arena_order(h1), to_arena_order(l0), to_arena_order(l1)};
        }
        reinterpret_cast<uint4 *>(tiles + tile * kTileBytes)[lane] = chunk;
        if (jq == 0) {
            uint2 sc = {0, 0};
            if (row < m) {
                const size_t at = ((size_t)row * n_groups + grp) * 2;
                const uint16_t scale = load_u16(s + at), bias = load_u16(b + at);
                sc.x = (uint32_t)f32_to_bf16(bf16_to_f32(scale) * 16.0f) | ((uint32_t)bias << 16);
                sc.y = (uint32_t)scale;
            }
            reinterpret_cast<uint2 *>(scales + tile * kTileScaleBytes)[i] = sc;
        }
    }
}

// Greedy choice per row: the largest finite value wins, ties go to the lowest index, NaN and +-inf never
// win; a row with no candidate yields index 0 (Metal/Sampling/logit.metal:689-720, 916-921). Two stages: the
// GEMV's blocks each leave the winner of the weight rows they walked, then one block per input row picks
// among those. A key orders by value first and by lower index second, so the order of comparisons is free.
__device__ __forceinline__ unsigned long long argmax_key(float v, uint32_t i) {
    if (!(__builtin_fabsf(v) < INFINITY)) return 0ull;       // NaN or +-inf: never chosen
    const uint32_t u = __float_as_uint(v);
    const uint32_t ord = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return ((unsigned long long)ord << 32) | (0xFFFFFFFFu - i);
}

// The winner's probability under the final logit softcap, as argmax_rows_f32 leaves it for a drafter
// (Metal/Sampling/logit.metal:946-1010): softmax over the finite logits, each capped to softcap * tanh(v / softcap)
// when softcap > 0, kept as an online (maximum, sum of exp(c - maximum)) pair that merges associatively.
struct SoftmaxAcc {
    float m, s;      // m = -inf: nothing seen yet
};
__device__ __forceinline__ float capped(float v, float softcap) {
    if (!(softcap > 0.0f)) return v;
    // tanh z = 1 - 2 / (exp(2 z) + 1); exp saturates to inf / 0 cleanly, so large |z| give +-1
    const float z = v / softcap;
    return softcap * (1.0f - 2.0f / (__expf(2.0f * z) + 1.0f));
}
__device__ __forceinline__ void softmax_take(SoftmaxAcc &a, float v, float softcap) {
    if (!(__builtin_fabsf(v) < INFINITY)) return;          // non-finite logits take no part (they never win either)
    const float c = capped(v, softcap);
    if (c > a.m) {
        a.s = a.s * __expf(a.m - c) + 1.0f;                 // exp(-inf) = 0 covers the first value
        a.m = c;
    } else {
        a.s += __expf(c - a.m);
    }
}
__device__ __forceinline__ SoftmaxAcc softmax_merge(const SoftmaxAcc &a, const SoftmaxAcc &b) {
    const float m = fmaxf(a.m, b.m);
    if (m == -INFINITY) return SoftmaxAcc{-INFINITY, 0.0f};
    return SoftmaxAcc{m, a.s * __expf(a.m - m) + b.s * __expf(b.m - m)};
}
__device__ __forceinline__ SoftmaxAcc softmax_shuffle(const SoftmaxAcc &a, int mask) {
    return SoftmaxAcc{__shfl_xor(a.m, mask, 64), __shfl_xor(a.s, mask, 64)};
}

// y[r][m] = sum_g [ s_g * sum_k q_k x_k + b_g * sum_k x_k ] (moe.metal:323-378, logit.metal:614-667) for all
// input rows at once. grid = (blocks): every block walks a range of 32-row tiles; its four waves split K
// (at most kRing groups each), keep their slice of the input rows in registers and refill the weight
// ring across tiles; per tile the partial sums meet in LDS, are added in wave order, and each wave
// stores a quarter of the input rows. GREEDY: nothing is stored per weight row; every lane keeps the best
// (value, index) key of the sums it finishes and the block leaves one key per input row in
// y_[row * gridDim.x + block], so the [rows][m] fp32 logits never travel to memory and back. CONF: the block also
// leaves the softmax pair of the sums it finished in conf_part[row * gridDim.x + block].
// PLANES8: the matrix is an 8-bit one stored as two nibble planes (above): a tile is 16 rows, an output the sum of its
// two streams.
template <bool Y_F32, bool F16, bool GREEDY = false, bool CONF = false, bool PLANES8 = false, int GLU = 0>
__global__ __launch_bounds__(256, 2) void matrix_gemv_kernel(const uint8_t *__restrict__ tiles,
                                                             const uint8_t *__restrict__ scales, uint32_t m,
                                                             uint32_t n_groups, const uint16_t *__restrict__ x,
                                                             uint32_t x_stride, uint32_t rows, void *__restrict__ y_,
                                                             uint32_t y_stride, float2 *__restrict__ conf_part = nullptr,
                                                             float softcap = 0.0f) {
    __shared__ float s_red[2][kKSplit][8][64];
    static_assert(!(PLANES8 && GREEDY), "the greedy choice is built for the 4-bit head only");
    static_assert((GLU == 1) ? PLANES8 : true, "tile pairs are the 8-bit planes' gated form");
    static_assert((GLU == 2) ? !PLANES8 && !GREEDY : true, "gate and up as a tile's two streams is the 4-bit gated form");
    // GLU == 2: a 4-bit tile's stream A holds 16 rows of a gate projection and its stream B the same rows of the up
    // projection - the expert arena's gate/up tiles - and `m` counts the outputs gelu_tanh(gate . x) * (up . x), both sums
    // fp32 in front of the activation as in the expert kernels (moe.metal:496).
    // GLU == 1: tiles 2 p and 2 p + 1 hold rows 16 p ... 16 p + 15 of a gate and of an up projection; a block takes whole
    // pairs, and `m` counts the outputs gelu_tanh(gate . x) * (up . x)
    const uint32_t n_tiles = GLU == 1 ? 2 * ((m + 15) / 16) : (PLANES8 || GLU == 2) ? (m + 15) / 16 : (m + 31) / 32;
    uint32_t rb0, rb1;
    split_range(GLU == 1 ? n_tiles / 2 : n_tiles, gridDim.x, blockIdx.x, rb0, rb1);
    if (GLU == 1) {
        rb0 *= 2;
        rb1 *= 2;
    }
    if (rb0 >= rb1) {
        if (GREEDY && threadIdx.x < rows) reinterpret_cast<unsigned long long *>(y_)[(size_t)threadIdx.x * gridDim.x + blockIdx.x] = 0ull;
        if (CONF && threadIdx.x < rows) conf_part[(size_t)threadIdx.x * gridDim.x + blockIdx.x] = make_float2(-INFINITY, 0.0f);
        return;
    }
    const uint32_t lane = threadIdx.x & 63, ks = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t j = lane & 15, jq = lane >> 4;
    const uint32_t per = (n_groups + kKSplit - 1) / kKSplit;
    const uint32_t g0 = min(ks * per, n_groups), g1 = min(n_groups, g0 + per), ng = g1 - g0;
    const uint32_t g_last = g1 > g0 ? g1 - 1 : n_groups - 1;
    const TileSource src = make_tile_source(tiles, (size_t)n_tiles * n_groups * kTileBytes, scales,
                                            (size_t)n_tiles * n_groups * kTileScaleBytes);
    // more than 16 input rows (the plain forms only): grid row y takes rows 16 y ... 16 y + 15 - the same pass over the
    // weights again, which then come from the caches
    if (!GREEDY && blockIdx.y != 0) {
        x += (size_t)blockIdx.y * FFMOE_MAX_VERIFY_ROWS * x_stride;
        y_ = Y_F32 ? static_cast<void *>(reinterpret_cast<float *>(y_) + (size_t)blockIdx.y * FFMOE_MAX_VERIFY_ROWS * y_stride)
                   : static_cast<void *>(reinterpret_cast<uint16_t *>(y_) + (size_t)blockIdx.y * FFMOE_MAX_VERIFY_ROWS * y_stride);
    }
    if (!GREEDY) rows = min((uint32_t)FFMOE_MAX_VERIFY_ROWS, rows - blockIdx.y * FFMOE_MAX_VERIFY_ROWS);

    WeightRing ring;
#pragma unroll
    for (int u = 0; u < kRing; ++u) ring_fill(ring, u, src, rb0 * n_groups + min(g0 + u, g_last), lane);
    // the input rows of this wave's K-slice: requested as 64-byte pieces (four lanes per row), then turned into the
    // operand layout - with 16 rows the operand layout itself would make every lane of every load a request of its own
    uint4 x0[kRing], x1[kRing];
    load_token_rows(x, x_stride, rows, lane, KSlice{g0, ng, g_last}, x0, x1);
    turn_token_rows(lane, x0, x1);
    // per group: the sum of its inputs per token column, once for all the tile rows this wave walks
    f32x4 sx[kRing];
#pragma unroll
    for (int u = 0; u < kRing; ++u) sx[u] = group_input_sum<F16>(x0[u], x1[u]);
    const uint32_t my_row = 4 * jq + ks;        // the input row this lane finishes
    float *y32 = reinterpret_cast<float *>(y_);
    uint16_t *y16 = reinterpret_cast<uint16_t *>(y_);
    unsigned long long best = 0ull;
    SoftmaxAcc soft{-INFINITY, 0.0f};
    float gate_kept = 0.0f;

    for (uint32_t rb = rb0; rb < rb1; ++rb) {
        const uint32_t next_row = min(rb + 1, rb1 - 1) * n_groups;
        TwoStreamAcc tot;
        tot.a = f32x4{0.f, 0.f, 0.f, 0.f};
        tot.b = tot.a;
#pragma unroll
        for (int u = 0; u < kRing; ++u)
            ring_step<F16>(ring, u, (uint32_t)u < ng, x0[u], x1[u], sx[u], tot, src, next_row + min(g0 + u, g_last), lane);
        const int buf = (rb - rb0) & 1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s_red[buf][ks][r][lane] = tot.a[r];
            s_red[buf][ks][4 + r][lane] = tot.b[r];
        }
        lds_barrier();
        float va = s_red[buf][0][ks][lane], vb = s_red[buf][0][4 + ks][lane];
#pragma unroll
        for (int o = 1; o < kKSplit; ++o) {
            va += s_red[buf][o][ks][lane];
            vb += s_red[buf][o][4 + ks][lane];
        }
        if (GLU == 2) {
            const uint32_t col = rb * kTileRows + j;
            if (my_row < rows && col < m) {
                const float act = gelu_tanh_fast(va) * vb;
                if (Y_F32) y32[(size_t)my_row * y_stride + col] = act;
                else y16[(size_t)my_row * y_stride + col] = Act<F16>::round(act);
            }
        } else if (GLU == 1) {
            // both projections are rounded to 16 bits in front of the activation, as shared_int8_gate_up_act_simd does
            // (Metal/Quant/dequant_int8.metal:131-136) and as two separate calls with the activation between them would
            const float v = Act<F16>::widen(Act<F16>::round(va + vb));
            const uint32_t col = (rb >> 1) * kTileRows + j;
            if (!(rb & 1u)) {
                gate_kept = v;
            } else if (my_row < rows && col < m) {
                const float act = gelu_tanh_fast(gate_kept) * v;
                if (Y_F32) y32[(size_t)my_row * y_stride + col] = act;
                else y16[(size_t)my_row * y_stride + col] = Act<F16>::round(act);
            }
        } else if (PLANES8) {
            const uint32_t row = rb * kTileRows + j;
            if (my_row < rows && row < m) {
                const float v = va + vb;
                if (Y_F32) y32[(size_t)my_row * y_stride + row] = v;
                else y16[(size_t)my_row * y_stride + row] = Act<F16>::round(v);
            }
        } else if (my_row < rows) {
            const uint32_t row_a = rb * 2 * kTileRows + j, row_b = row_a + kTileRows;
            const size_t base = (size_t)my_row * y_stride;
            if (GREEDY) {
                const unsigned long long ka = row_a < m ? argmax_key(va, row_a) : 0ull;
                const unsigned long long kb = row_b < m ? argmax_key(vb, row_b) : 0ull;
                best = max(best, max(ka, kb));
                if (CONF) {
                    if (row_a < m) softmax_take(soft, va, softcap);
                    if (row_b < m) softmax_take(soft, vb, softcap);
                }
            } else if (Y_F32) {
                if (row_a < m) y32[base + row_a] = va;
                if (row_b < m) y32[base + row_b] = vb;
            } else {
                if (row_a < m) y16[base + row_a] = Act<F16>::round(va);
                if (row_b < m) y16[base + row_b] = Act<F16>::round(vb);
            }
        }
    }
    if (GREEDY) {
        // the 16 lanes that share lane / 16 finished the same input row
#pragma unroll
        for (int mk = 8; mk >= 1; mk >>= 1) best = max(best, (unsigned long long)__shfl_xor(best, mk, 64));
        if (j == 0 && my_row < rows)
            reinterpret_cast<unsigned long long *>(y_)[(size_t)my_row * gridDim.x + blockIdx.x] = best;
        if (CONF) {
#pragma unroll
            for (int mk = 8; mk >= 1; mk >>= 1) soft = softmax_merge(soft, softmax_shuffle(soft, mk));
            if (j == 0 && my_row < rows) conf_part[(size_t)my_row * gridDim.x + blockIdx.x] = make_float2(soft.m, soft.s);
        }
    }
}

__device__ __forceinline__ unsigned long long block_max_key(unsigned long long k, unsigned long long *s_k) {
#pragma unroll
    for (int mk = 32; mk >= 1; mk >>= 1) {
        const unsigned long long o = __shfl_xor(k, mk, 64);
        k = o > k ? o : k;
    }
    if ((threadIdx.x & 63) == 0) s_k[threadIdx.x >> 6] = k;
    __syncthreads();
    k = s_k[0];
    for (uint32_t v = 1; v < blockDim.x / 64; ++v) k = s_k[v] > k ? s_k[v] : k;
    return k;
}

// The block's softmax pair, the same in every thread.
__device__ __forceinline__ SoftmaxAcc block_softmax(SoftmaxAcc a, float2 *s_p) {
#pragma unroll
    for (int mk = 32; mk >= 1; mk >>= 1) a = softmax_merge(a, softmax_shuffle(a, mk));
    if ((threadIdx.x & 63) == 0) s_p[threadIdx.x >> 6] = make_float2(a.m, a.s);
    __syncthreads();
    a = SoftmaxAcc{s_p[0].x, s_p[0].y};
    for (uint32_t v = 1; v < blockDim.x / 64; ++v) a = softmax_merge(a, SoftmaxAcc{s_p[v].x, s_p[v].y});
    return a;
}

// The winner's value from its key (argmax_key is a bijection on the finite values).
__device__ __forceinline__ float key_value(unsigned long long k) {
    const uint32_t ord = (uint32_t)(k >> 32);
    return __uint_as_float((ord & 0x80000000u) ? (ord & 0x7FFFFFFFu) : ~ord);
}

__device__ __forceinline__ float winner_confidence(unsigned long long best, const SoftmaxAcc &all, float softcap) {
    if (best == 0ull || !(all.s > 0.0f)) return 0.0f;
    return __expf(capped(key_value(best), softcap) - all.m) / all.s;
}

__global__ __launch_bounds__(256) void argmax_final_kernel(const unsigned long long *__restrict__ part, uint32_t n_seg,
                                                           uint32_t *__restrict__ out, const float2 *__restrict__ conf_part,
                                                           float softcap, float *__restrict__ out_conf) {
    __shared__ unsigned long long s_k[4];
    __shared__ float2 s_p[4];
    const uint32_t row = blockIdx.x;
    unsigned long long best = 0ull;
    SoftmaxAcc soft{-INFINITY, 0.0f};
    for (uint32_t i = threadIdx.x; i < n_seg; i += 256) {
        const unsigned long long k = part[(size_t)row * n_seg + i];
        best = k > best ? k : best;
        if (out_conf) {
            const float2 q = conf_part[(size_t)row * n_seg + i];
            soft = softmax_merge(soft, SoftmaxAcc{q.x, q.y});
        }
    }
    best = block_max_key(best, s_k);
    if (threadIdx.x == 0) out[row] = best ? 0xFFFFFFFFu - (uint32_t)best : 0u;
    if (out_conf) {
        soft = block_softmax(soft, s_p);
        if (threadIdx.x == 0) out_conf[row] = winner_confidence(best, soft, softcap);
    }
}

// argmax_rows_f32 (Metal/Sampling/logit.metal:946-1010): the greedy choice over rows of fp32 logits that are in
// memory already (the listed GEMV's output: a drafter's hot vocabulary), one block per row: the largest finite value,
// ties to the lowest position, 0xFFFFFFFF and confidence 0 when no value is finite; and the winner's probability
// under the softcap.
__global__ __launch_bounds__(256) void argmax_rows_kernel(const float *__restrict__ logits, uint32_t stride, uint32_t count,
                                                          float softcap, uint32_t *__restrict__ out, float *__restrict__ out_conf) {
    __shared__ unsigned long long s_k[4];
    __shared__ float2 s_p[4];
    const float *row = logits + (size_t)blockIdx.x * stride;
    unsigned long long best = 0ull;
    SoftmaxAcc soft{-INFINITY, 0.0f};
    for (uint32_t i = threadIdx.x; i < count; i += 256) {
        const float v = row[i];
        const unsigned long long k = argmax_key(v, i);
        best = k > best ? k : best;
        if (out_conf) softmax_take(soft, v, softcap);
    }
    best = block_max_key(best, s_k);
    if (threadIdx.x == 0) out[blockIdx.x] = best ? 0xFFFFFFFFu - (uint32_t)best : 0xFFFFFFFFu;
    if (out_conf) {
        soft = block_softmax(soft, s_p);
        if (threadIdx.x == 0) out_conf[blockIdx.x] = winner_confidence(best, soft, softcap);
    }
}

}  // namespace

size_t matrix_tiles_bytes(uint32_t m, uint32_t n, bool planes8) {
    return (size_t)(planes8 ? (m + 15) / 16 : (m + 31) / 32) * (n / kGroup) * kTileBytes;
}
size_t matrix_scales_bytes(uint32_t m, uint32_t n, bool planes8) {
    return (size_t)(planes8 ? (m + 15) / 16 : (m + 31) / 32) * (n / kGroup) * kTileScaleBytes;
}
bool matrix_shape_ok(uint32_t n) { return n % kGroup == 0 && (n / kGroup + kKSplit - 1) / kKSplit <= (uint32_t)kRing; }

hipError_t launch_matrix_repack(hipStream_t s, const uint8_t *w, const uint16_t *scales, const uint16_t *biases,
                                uint32_t m, uint32_t n, uint8_t *tiles_out, uint8_t *scales_out, bool planes8) {
    const size_t total = matrix_tiles_bytes(m, n, planes8) / kTileBytes * kWave;
    const uint32_t blocks = (uint32_t)min((size_t)65535 * 16, (total + 255) / 256);
    if (planes8)
        hipLaunchKernelGGL(repack_matrix8_kernel, dim3(blocks), dim3(256), 0, s, w, reinterpret_cast<const uint8_t *>(scales),
                           reinterpret_cast<const uint8_t *>(biases), m, n, tiles_out, scales_out);
    else
        hipLaunchKernelGGL(repack_matrix_kernel, dim3(blocks), dim3(256), 0, s, w, reinterpret_cast<const uint8_t *>(scales),
                           reinterpret_cast<const uint8_t *>(biases), m, n, tiles_out, scales_out);
    return hipGetLastError();
}

hipError_t launch_matrix_gemv(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n,
                              const uint16_t *x, uint32_t x_stride, uint32_t rows, void *y, uint32_t y_stride,
                              bool y_f32, uint32_t n_cus, bool f16, bool planes8, int glu) {
    // glu: 0 plain, 1 the 8-bit planes' tile pairs, 2 a 4-bit tile's two streams as gate and up (m = the gated outputs)
    if (glu == 2 && (planes8 || y_f32)) return hipErrorInvalidValue;
    const uint32_t n_tiles = (planes8 || glu == 2) ? (m + 15) / 16 : (m + 31) / 32;      // glu == 1: pairs of tiles
    if (rows == 0 || (rows + FFMOE_MAX_VERIFY_ROWS - 1) / FFMOE_MAX_VERIFY_ROWS > 65535u) return hipErrorInvalidValue;
    dim3 grid(min(2 * n_cus, n_tiles), (rows + FFMOE_MAX_VERIFY_ROWS - 1) / FFMOE_MAX_VERIFY_ROWS);
    // several grid rows: a multiple of 8 blocks per row keeps a tile on one XCD (blocks go to the XCDs round robin), whose L2
    // then serves every pass after the first; the blocks past the tile count leave at once
    if (grid.y > 1) grid.x = (grid.x + 7) / 8 * 8;
#define FFMOE_MGEMV(Y, H, P, G)                                                                                             \
    hipLaunchKernelGGL((matrix_gemv_kernel<Y, H, false, false, P, G>), grid, dim3(256), 0, s, tiles, scales, m, n / kGroup, x, x_stride, \
                       rows, y, y_stride)
    if (glu == 2) {
        if (f16) FFMOE_MGEMV(false, true, false, 2); else FFMOE_MGEMV(false, false, false, 2);
    } else if (glu == 1) {
        if (f16) { if (y_f32) FFMOE_MGEMV(true, true, true, 1); else FFMOE_MGEMV(false, true, true, 1); }
        else { if (y_f32) FFMOE_MGEMV(true, false, true, 1); else FFMOE_MGEMV(false, false, true, 1); }
    } else if (planes8) {
        if (f16) { if (y_f32) FFMOE_MGEMV(true, true, true, 0); else FFMOE_MGEMV(false, true, true, 0); }
        else { if (y_f32) FFMOE_MGEMV(true, false, true, 0); else FFMOE_MGEMV(false, false, true, 0); }
    } else {
        if (f16) { if (y_f32) FFMOE_MGEMV(true, true, false, 0); else FFMOE_MGEMV(false, true, false, 0); }
        else { if (y_f32) FFMOE_MGEMV(true, false, false, 0); else FFMOE_MGEMV(false, false, false, 0); }
    }
#undef FFMOE_MGEMV
    return hipGetLastError();
}

// out = round16(gelu_tanh(gate) * up) per element of `rows` rows of `count` values: gelu_mul_fp16
// (Metal/Primitives/utility.metal:4-17), the step between the projections of the 8-bit shared expert
// (shared_int8_gate_up_act_simd rounds gate and up to 16 bits in front of it: Metal/Quant/dequant_int8.metal:131-136).
template <bool F16>
__global__ __launch_bounds__(256) void gelu_mul_kernel(const uint16_t *gate, uint32_t gate_stride, const uint16_t *up,
                                                       uint32_t up_stride, uint16_t *out, uint32_t out_stride, uint32_t count) {
    // no __restrict__: `out` may be `gate` or `up` itself (each element is read before it is written, by the same lane)
    const uint32_t row = blockIdx.y;
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < count; i += gridDim.x * 256) {
        const float g = Act<F16>::widen(gate[(size_t)row * gate_stride + i]), u = Act<F16>::widen(up[(size_t)row * up_stride + i]);
        out[(size_t)row * out_stride + i] = Act<F16>::round(gelu_tanh_fast(g) * u);
    }
}

hipError_t launch_gelu_mul(hipStream_t s, const uint16_t *gate, uint32_t gate_stride, const uint16_t *up, uint32_t up_stride,
                           uint16_t *out, uint32_t out_stride, uint32_t rows, uint32_t count, bool f16) {
    const dim3 grid(min(64u, (count + 255) / 256), rows);
    if (f16) hipLaunchKernelGGL(gelu_mul_kernel<true>, grid, dim3(256), 0, s, gate, gate_stride, up, up_stride, out, out_stride, count);
    else hipLaunchKernelGGL(gelu_mul_kernel<false>, grid, dim3(256), 0, s, gate, gate_stride, up, up_stride, out, out_stride, count);
    return hipGetLastError();
}

// Rows of the resident 4-bit matrix dequantised: out[i][k] = round16((q s + b) * out_scale) for weight row ids[i] (or
// the one row `token_id` when ids is null) - embed_lookup_int4 (Metal/Quant/dequant_int4.metal:53-73) on the re-tiled
// copy, so that tied embeddings need no second table. One thread per 8 consecutive elements: one 32-bit word of a tile
// (lane 16 (k / 8 % 4) + row % 16, word 2 (row / 16 % 2) + (k / 32 % 2)) and the row's scale pair. An id past the
// table gives a row of zeros.
template <bool F16>
__global__ __launch_bounds__(256) void matrix_rows_kernel(const uint8_t *__restrict__ tiles, const uint8_t *__restrict__ scales,
                                                          uint32_t m, uint32_t n_groups, const uint32_t *__restrict__ ids,
                                                          uint32_t token_id, float out_scale, uint16_t *__restrict__ out,
                                                          uint32_t out_stride) {
    const uint32_t r = ids ? ids[blockIdx.y] : token_id;
    for (uint32_t w = blockIdx.x * 256 + threadIdx.x; w < n_groups * 8; w += gridDim.x * 256) {
        const uint32_t grp = w >> 3, piece = w & 7;
        uint32_t packed[4] = {0, 0, 0, 0};
        if (r < m) {
            const size_t tile = (size_t)(r >> 5) * n_groups + grp;
            const uint32_t i = r & 15, half = (r >> 4) & 1, jq = piece & 3, hi = piece >> 2;
            const uint32_t word = reinterpret_cast<const uint32_t *>(tiles + tile * kTileBytes)[(jq * 16 + i) * 4 + half * 2 + hi];
            const uint32_t sb = reinterpret_cast<const uint32_t *>(scales + tile * kTileScaleBytes)[i * 2 + half];
            const float sc = bf16_to_f32((uint16_t)(sb & 0xFFFFu)), bi = bf16_to_f32((uint16_t)(sb >> 16));
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int pos = (t & 1) ? 4 + (t >> 1) : (t >> 1);          // arena order: position p = element 2p, p + 4 = element 2p + 1
                const float q = (float)((word >> (4 * pos)) & 0xFu);
                const float v = (q * sc + bi) * out_scale;                  // q * sc is exact in fp32: the reference's expression
                packed[t >> 1] |= (uint32_t)Act<F16>::round(v) << (16 * (t & 1));
            }
        }
        *reinterpret_cast<uint4 *>(out + (size_t)blockIdx.y * out_stride + grp * kGroup + 8 * piece) =
            uint4{packed[0], packed[1], packed[2], packed[3]};
    }
}

hipError_t launch_matrix_rows(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n, const uint32_t *ids,
                              uint32_t token_id, uint32_t count, float out_scale, uint16_t *out, uint32_t out_stride, bool f16) {
    if (count == 0 || count > 65535u) return hipErrorInvalidValue;
    const dim3 grid(min(64u, (n / 8 + 255) / 256), count);
    if (f16)
        hipLaunchKernelGGL(matrix_rows_kernel<true>, grid, dim3(256), 0, s, tiles, scales, m, n / kGroup, ids, token_id, out_scale, out, out_stride);
    else
        hipLaunchKernelGGL(matrix_rows_kernel<false>, grid, dim3(256), 0, s, tiles, scales, m, n / kGroup, ids, token_id, out_scale, out, out_stride);
    return hipGetLastError();
}

// An 8-bit matrix for the library's dense GEMM, used beyond the row counts the streaming passes are good for: a 16-bit
// matrix element cannot hold w = q s + b of an 8-bit q, so w is written as two - hi = round16(w) and lo = round16(w - hi),
// together 16 (bf16) or 22 (FP16) significant bits of w - and the GEMM multiplies by both: out[r] = hi rows, out[rows + r]
// = lo rows ([2 m][n], row-major; the gated matrix: gate hi, gate lo, up hi, up lo, [4 f][n]). Read back from the nibble
// planes, so it can be made again when the activation type changes. One thread per 8 consecutive elements.
template <bool F16>
__global__ __launch_bounds__(256) void expand_planes8_kernel(const uint8_t *__restrict__ tiles, const uint8_t *__restrict__ scales,
                                                             uint32_t m, uint32_t n_groups, bool glu, uint16_t *__restrict__ out) {
    const uint32_t n = n_groups * kGroup, tile_rows = (glu ? 2u : 1u) * ((m + 15) / 16);
    const size_t total = (size_t)tile_rows * 16 * n_groups * 8;
    for (size_t gid = (size_t)blockIdx.x * 256 + threadIdx.x; gid < total; gid += (size_t)gridDim.x * 256) {
        const uint32_t w = (uint32_t)(gid % (n_groups * 8)), stored_row = (uint32_t)(gid / (n_groups * 8));
        const uint32_t grp = w >> 3, piece = w & 7, tr = stored_row >> 4, i = stored_row & 15;
        // the weight row this stored row is, and where its hi / lo rows go
        const uint32_t row = glu ? (tr >> 1) * 16 + i : stored_row;
        if (row >= m) continue;
        const size_t hi_row = glu ? ((tr & 1u) ? 2 * (size_t)m + row : row) : row, lo_row = hi_row + m;
        const size_t tile = (size_t)tr * n_groups + grp;
        const uint32_t jq = piece & 3, second = piece >> 2;
        const uint32_t *lane_words = reinterpret_cast<const uint32_t *>(tiles + tile * kTileBytes) + (jq * 16 + i) * 4;
        const uint32_t high = lane_words[second], low = lane_words[2 + second];
        const uint2 sb = reinterpret_cast<const uint2 *>(scales + tile * kTileScaleBytes)[i];
        const float sc = bf16_to_f32((uint16_t)(sb.y & 0xFFFFu)), bi = bf16_to_f32((uint16_t)(sb.x >> 16));
        uint32_t hi_w[4] = {0, 0, 0, 0}, lo_w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int pos = (t & 1) ? 4 + (t >> 1) : (t >> 1);
            const float q = (float)(16u * ((high >> (4 * pos)) & 0xFu) + ((low >> (4 * pos)) & 0xFu));
            const float v = q * sc + bi;                       // q * sc is exact in fp32 (8 + 8 bits): the reference's q s + b
            const uint16_t h = Act<F16>::round(v);
            hi_w[t >> 1] |= (uint32_t)h << (16 * (t & 1));
            lo_w[t >> 1] |= (uint32_t)Act<F16>::round(v - Act<F16>::widen(h)) << (16 * (t & 1));
        }
        *reinterpret_cast<uint4 *>(out + hi_row * n + grp * kGroup + 8 * piece) = uint4{hi_w[0], hi_w[1], hi_w[2], hi_w[3]};
        *reinterpret_cast<uint4 *>(out + lo_row * n + grp * kGroup + 8 * piece) = uint4{lo_w[0], lo_w[1], lo_w[2], lo_w[3]};
    }
}

hipError_t launch_expand_planes8(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n, bool glu,
                                 uint16_t *out, bool f16) {
    const size_t total = (size_t)(glu ? 2 : 1) * ((m + 15) / 16) * 16 * (n / 8);
    const dim3 grid((uint32_t)min((size_t)65535 * 16, (total + 255) / 256));
    if (f16) hipLaunchKernelGGL(expand_planes8_kernel<true>, grid, dim3(256), 0, s, tiles, scales, m, n / kGroup, glu, out);
    else hipLaunchKernelGGL(expand_planes8_kernel<false>, grid, dim3(256), 0, s, tiles, scales, m, n / kGroup, glu, out);
    return hipGetLastError();
}

// Behind the GEMMs on the hi / lo rows: a weight row's result is the sum of its two columns.
// gated: sums [rows][4 f] (gate hi, gate lo, up hi, up lo) -> act[r][j] = round16(gelu_tanh(round16(gate)) * round16(up)),
// the same roundings as the streaming form's epilogue. plain: sums [rows][2 d] -> y[r][i] = round16(hi + lo).
template <bool F16, bool GATED>
__global__ __launch_bounds__(256) void hilo_epilogue_kernel(const float *__restrict__ sums, uint32_t width, uint16_t *__restrict__ out,
                                                            uint32_t out_stride) {
    const float *row = sums + (size_t)blockIdx.y * width * (GATED ? 4 : 2);
    for (uint32_t j = blockIdx.x * 256 + threadIdx.x; j < width; j += gridDim.x * 256) {
        float v = row[j] + row[width + j];
        if (GATED) {
            const float g = Act<F16>::widen(Act<F16>::round(v));
            const float u = Act<F16>::widen(Act<F16>::round(row[2 * width + j] + row[3 * width + j]));
            v = gelu_tanh_fast(g) * u;
        }
        out[(size_t)blockIdx.y * out_stride + j] = Act<F16>::round(v);
    }
}

hipError_t launch_hilo_epilogue(hipStream_t s, const float *sums, uint32_t rows, uint32_t width, bool gated, uint16_t *out,
                                uint32_t out_stride, bool f16) {
    if (rows == 0 || rows > 65535u) return hipErrorInvalidValue;
    const dim3 grid(min(16u, (width + 255) / 256), rows);
#define FFMOE_HILO(H, G) hipLaunchKernelGGL((hilo_epilogue_kernel<H, G>), grid, dim3(256), 0, s, sums, width, out, out_stride)
    if (f16) { if (gated) FFMOE_HILO(true, true); else FFMOE_HILO(true, false); }
    else { if (gated) FFMOE_HILO(false, true); else FFMOE_HILO(false, false); }
#undef FFMOE_HILO
    return hipGetLastError();
}

// keys per input row that launch_matrix_greedy leaves between its two kernels
uint32_t greedy_segments(uint32_t m, uint32_t n_cus) { return min(2 * n_cus, (m + 31) / 32); }

// `partials`: [16][segments] keys, then (when out_conf is wanted) [16][segments] softmax pairs
hipError_t launch_matrix_greedy(hipStream_t s, const uint8_t *tiles, const uint8_t *scales, uint32_t m, uint32_t n,
                                const uint16_t *x, uint32_t x_stride, uint32_t rows, unsigned long long *partials,
                                uint32_t *out, uint32_t n_cus, bool f16, KernelTimer *timer, float softcap, float *out_conf) {
    const dim3 grid(greedy_segments(m, n_cus));
    float2 *conf_part = reinterpret_cast<float2 *>(partials + (size_t)FFMOE_MAX_VERIFY_ROWS * grid.x);
#define FFMOE_GREEDY(H, C)                                                                                                  \
    hipLaunchKernelGGL((matrix_gemv_kernel<true, H, true, C>), grid, dim3(256), 0, s, tiles, scales, m, n / kGroup, x, x_stride, \
                       rows, partials, 0u, conf_part, softcap)
    if (f16) { if (out_conf) FFMOE_GREEDY(true, true); else FFMOE_GREEDY(true, false); }
    else { if (out_conf) FFMOE_GREEDY(false, true); else FFMOE_GREEDY(false, false); }
#undef FFMOE_GREEDY
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    timer->mark(s, FFMOE_K_GEMV);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(rows), dim3(256), 0, s, partials, grid.x, out, conf_part, softcap, out_conf);
    timer->mark(s, FFMOE_K_ARGMAX);
    return hipGetLastError();
}

hipError_t launch_argmax_rows(hipStream_t s, const float *logits, uint32_t stride, uint32_t rows, uint32_t count, float softcap,
                              uint32_t *out, float *out_conf) {
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(256), 0, s, logits, stride, count, softcap, out, out_conf);
    return hipGetLastError();
}

}  // namespace ffmoe
