// The sampled choice over rows of fp32 logits (sample_rows_f32, Metal/Sampling/logit.metal:1010-1259; dispatched by
// LMHeadChainInt4.encodeChoice, Kernels/Fusions/LMHeadChainInt4.swift:192-223): per row one draw from the tempered
// softmax of the soft-capped logits by the Gumbel-max rule,
//     token = argmax_i  capped(logit_i) / T + G(seed, key, token_i),
// over the entries the truncation keeps. The noise is a counter-based hash of (seed, position key, token id), so every
// producer that draws a position draws the same noise. Truncation in the sampler's order: the top_k largest capped
// logits (ties to the lower index), of those the shortest prefix whose T = 1 probability mass reaches top_p, then
// the draw at temperature T over the survivors.
//
// One block of 1,024 threads per row (a row is up to 262,144 logits: 1 MiB, which stays in the XCD's L2 across the
// sweeps). Without truncation: two sweeps (the largest capped logit; the draw and the normaliser). With it the k-th
// largest is found EXACTLY by a radix select over the order-preserving integer image of the capped logits - three
// sweeps with LDS histograms of 11, 11 and 10 bits - instead of a histogram over the value range whose edge bin has to
// fit a candidate buffer; a fourth sweep gathers the values above the threshold (any order: they are ranked
// afterwards) and, of the values equal to it, the lowest indices (in index order, wave by wave). The <= 256
// candidates are ranked by counting, thread 0 walks the top_p prefix, and the survivors draw.
#include <hip/hip_runtime.h>

#include "common.hpp"
#include "kernels.hpp"

namespace ffmoe {
namespace {

constexpr int kSampleThreads = 1024, kSampleWaves = kSampleThreads / 64;
constexpr int kSampleMaxK = 256;

struct SampleRule {
    float temperature, top_p;
    uint32_t top_k, key_base;
    float softcap;
    uint32_t seed_lo, seed_hi;
};

// logits are capped to (-cap, cap); a non-finite logit never takes part (logit.metal:1055-1057)
__device__ __forceinline__ float sample_capped(float v, float cap) {
    return (v - v == 0.0f) ? cap * tanhf(v / cap) : -INFINITY;
}

// Standard Gumbel noise from the hash of (seed, key, token): one SplitMix64 step of the mixed state, its top 24 bits
// as a uniform in (0, 1) (logit.metal:1042-1051).
__device__ __forceinline__ float sample_gumbel(unsigned long long seed, uint32_t key, uint32_t token) {
    unsigned long long z = seed ^ ((unsigned long long)key * 0x9E3779B97F4A7C15ull) ^ ((unsigned long long)token * 0xD1B54A32D192ED03ull);
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const float u = ((float)(uint32_t)(z >> 40) + 0.5f) * (1.0f / 16777216.0f);
    return -logf(-logf(u));
}

// float -> unsigned, order preserving (-inf lowest of the values that occur here)
__device__ __forceinline__ uint32_t sample_key(float v) {
    const uint32_t b = __float_as_uint(v);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

struct SampleShared {
    uint32_t hist[2048];
    float red_f[kSampleWaves];
    unsigned long long red_k[kSampleWaves];
    uint32_t wave_eq[kSampleWaves][kSampleMaxK];     // per wave: the first indices (in index order) whose value equals the threshold
    uint32_t wave_eq_n[kSampleWaves];
    float cand_v[kSampleMaxK], sorted_v[kSampleMaxK];
    uint32_t cand_i[kSampleMaxK], sorted_i[kSampleMaxK];
    uint32_t n_above, bin, above, keep;
    float f0;
    unsigned long long k0;
};

__device__ __forceinline__ float block_max_f(float v, SampleShared &sh) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh.red_f[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = sh.red_f[0];
    for (int w = 1; w < kSampleWaves; ++w) r = fmaxf(r, sh.red_f[w]);
    return r;
}

// sum in a fixed order: lanes by xor-butterfly, then the waves one after the other
__device__ __forceinline__ float block_sum_f(float v, SampleShared &sh) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh.red_f[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = 0.0f;
    for (int w = 0; w < kSampleWaves; ++w) r += sh.red_f[w];
    return r;
}

__device__ __forceinline__ unsigned long long block_max_k(unsigned long long v, SampleShared &sh) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = ((unsigned long long)(uint32_t)__shfl_xor((int)(v >> 32), o, 64) << 32) |
                                         (uint32_t)__shfl_xor((int)(uint32_t)v, o, 64);
        v = other > v ? other : v;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh.red_k[threadIdx.x >> 6] = v;
    __syncthreads();
    unsigned long long r = sh.red_k[0];
    for (int w = 1; w < kSampleWaves; ++w) r = sh.red_k[w] > r ? sh.red_k[w] : r;
    return r;
}

// Of `bins` histogram counts (a multiple of 64, <= 2048) find, from the top, the bin that holds the want-th largest
// entry (1-based): sh.bin = that bin, sh.above = entries in the bins above it. Run by the whole block (wave 0 works).
__device__ __forceinline__ void find_bin(SampleShared &sh, uint32_t bins, uint32_t want) {
    __syncthreads();
    if (threadIdx.x < 64) {
        const uint32_t lane = threadIdx.x, per = bins / 64;
        // lane l owns the bins [bins - per (l + 1), bins - per l): lane 0 the highest
        const uint32_t hi = bins - per * lane;
        uint32_t mine = 0;
        for (uint32_t b = 0; b < per; ++b) mine += sh.hist[hi - 1 - b];
        uint32_t incl = mine;                      // entries in this lane's bins and all higher lanes'
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = (uint32_t)__shfl_up((int)incl, o, 64);
            if (lane >= (uint32_t)o) incl += up;
        }
        const uint32_t before = incl - mine;
        if (before < want && want <= incl) {
            uint32_t acc = before;
            for (uint32_t b = 0; b < per; ++b) {
                const uint32_t c = sh.hist[hi - 1 - b];
                if (acc + c >= want) {
                    sh.bin = hi - 1 - b;
                    sh.above = acc;
                    break;
                }
                acc += c;
            }
        }
    }
    __syncthreads();
}

__global__ __launch_bounds__(kSampleThreads) void sample_rows_kernel(const float *__restrict__ logits, uint32_t stride, uint32_t count,
                                                                     const uint32_t *__restrict__ ids, SampleRule p,
                                                                     const uint32_t *__restrict__ key_offset,
                                                                     uint32_t *__restrict__ out_tokens, float *__restrict__ out_prob) {
    __shared__ SampleShared sh;
    const uint32_t r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *row = logits + (size_t)r * stride;
    const float cap = p.softcap, invT = 1.0f / p.temperature;
    const uint32_t key = p.key_base + (key_offset ? key_offset[0] : 0u) + r;
    const unsigned long long seed = ((unsigned long long)p.seed_hi << 32) | p.seed_lo;
    const bool truncated = p.top_k > 0u && p.top_k < count;
    auto token_of = [&](uint32_t i) { return ids ? ids[i] : i; };

    if (!truncated) {
        float m = -INFINITY;
        for (uint32_t i = tid; i < count; i += kSampleThreads) m = fmaxf(m, sample_capped(row[i], cap));
        m = block_max_f(m, sh);
        unsigned long long best = 0ull;
        float sum = 0.0f;
        for (uint32_t i = tid; i < count; i += kSampleThreads) {
            const float c = sample_capped(row[i], cap);
            if (c == -INFINITY) continue;
            sum += expf((c - m) * invT);
            const float g = c * invT + sample_gumbel(seed, key, token_of(i));
            const unsigned long long k = ((unsigned long long)sample_key(g) << 32) | (0xFFFFFFFFu - i);
            best = k > best ? k : best;
        }
        best = block_max_k(best, sh);
        const float total = block_sum_f(sum, sh);
        if (tid == 0) {
            const uint32_t j = best ? 0xFFFFFFFFu - (uint32_t)best : 0xFFFFFFFFu;
            out_tokens[r] = j;
            out_prob[r] = (j == 0xFFFFFFFFu || !(total > 0.0f)) ? 0.0f : expf((sample_capped(row[j], cap) - m) * invT) / total;
        }
        return;
    }

    // ---- exact top_k: radix select on the keys of the capped logits, 11 + 11 + 10 bits -------------------------
    const uint32_t k = p.top_k;
    float s1 = 0.0f;
    for (uint32_t b = tid; b < 2048; b += kSampleThreads) sh.hist[b] = 0;
    if (tid < kSampleWaves) sh.wave_eq_n[tid] = 0;
    if (tid == 0) sh.n_above = 0;
    __syncthreads();
    uint32_t n_finite = 0;
    for (uint32_t i = tid; i < count; i += kSampleThreads) {
        const float c = sample_capped(row[i], cap);
        if (c == -INFINITY) continue;
        s1 += expf(c - cap);                                   // the T = 1 normaliser, offset by the cap
        ++n_finite;
        atomicAdd(&sh.hist[sample_key(c) >> 21], 1u);
    }
    const float total1 = block_sum_f(s1, sh);
    const uint32_t finite = (uint32_t)block_sum_f((float)n_finite, sh);      // counts up to 2^18 per row: exact in fp32
    if (finite == 0) {
        if (tid == 0) {
            out_tokens[r] = 0xFFFFFFFFu;
            out_prob[r] = 0.0f;
        }
        return;
    }
    const uint32_t want = min(k, finite);                      // fewer finite entries than top_k: all of them
    find_bin(sh, 2048, want);
    const uint32_t b1 = sh.bin, above1 = sh.above;
    __syncthreads();
    for (uint32_t b = tid; b < 2048; b += kSampleThreads) sh.hist[b] = 0;
    __syncthreads();
    for (uint32_t i = tid; i < count; i += kSampleThreads) {
        const float c = sample_capped(row[i], cap);
        if (c == -INFINITY) continue;
        const uint32_t q = sample_key(c);
        if ((q >> 21) == b1) atomicAdd(&sh.hist[(q >> 10) & 2047u], 1u);
    }
    find_bin(sh, 2048, want - above1);
    const uint32_t b2 = sh.bin, above2 = above1 + sh.above;
    __syncthreads();
    for (uint32_t b = tid; b < 1024; b += kSampleThreads) sh.hist[b] = 0;
    __syncthreads();
    const uint32_t top22 = (b1 << 11) | b2;
    for (uint32_t i = tid; i < count; i += kSampleThreads) {
        const float c = sample_capped(row[i], cap);
        if (c == -INFINITY) continue;
        const uint32_t q = sample_key(c);
        if ((q >> 10) == top22) atomicAdd(&sh.hist[q & 1023u], 1u);
    }
    find_bin(sh, 1024, want - above2);
    const uint32_t threshold = (top22 << 10) | sh.bin;         // the key of the want-th largest capped logit
    const uint32_t above = above2 + sh.above, need = want - above;     // `need` of the entries equal to it, lowest indices first
    __syncthreads();

    // ---- gather: everything above the threshold, and per wave the first `need` indices equal to it -----------
    // wave w walks the contiguous piece [w * piece, (w + 1) * piece) of the row 64 entries at a time, so a ballot's
    // bit order is index order
    const uint32_t piece = ((count + kSampleWaves - 1) / kSampleWaves + 63) / 64 * 64;
    uint32_t eq_seen = 0;
    for (uint32_t base = wave * piece; base < min(count, (wave + 1) * piece); base += 64) {
        const uint32_t i = base + lane;
        float c = -INFINITY;
        if (i < count) c = sample_capped(row[i], cap);
        const uint32_t q = c == -INFINITY ? 0u : sample_key(c);
        if (q > threshold) {
            const uint32_t slot = atomicAdd(&sh.n_above, 1u);
            sh.cand_v[slot] = c;                                // fewer than want <= 256 of them
            sh.cand_i[slot] = i;
        }
        const bool eq = c != -INFINITY && q == threshold;
        const unsigned long long mask = __ballot(eq);
        if (eq) {
            const uint32_t rank = eq_seen + __popcll(mask & ((1ull << lane) - 1ull));
            if (rank < need) sh.wave_eq[wave][rank] = i;
        }
        eq_seen += __popcll(mask);
    }
    if (lane == 0) sh.wave_eq_n[wave] = min(eq_seen, need);
    __syncthreads();
    // the equal entries in index order: wave 0's first, then wave 1's, ... until `need` are placed
    if (tid < need) {
        uint32_t skip = tid, w = 0;
        while (w < (uint32_t)kSampleWaves && skip >= sh.wave_eq_n[w]) skip -= sh.wave_eq_n[w++];
        const uint32_t i = sh.wave_eq[w][skip];                // exists: the waves hold at least `need` together
        sh.cand_v[above + tid] = sample_capped(row[i], cap);
        sh.cand_i[above + tid] = i;
    }
    __syncthreads();
    const uint32_t n = want;
    // ---- rank the candidates: larger value first, then lower index (sample_before, logit.metal:1059-1062) -----
    if (tid < n) {
        const float v = sh.cand_v[tid];
        const uint32_t i = sh.cand_i[tid];
        uint32_t rank = 0;
        for (uint32_t u = 0; u < n; ++u) {
            const float vu = sh.cand_v[u];
            const uint32_t iu = sh.cand_i[u];
            rank += (vu > v || (vu == v && iu < i)) ? 1u : 0u;
        }
        sh.sorted_v[rank] = v;
        sh.sorted_i[rank] = i;
    }
    __syncthreads();
    // ---- top_p over the T = 1 distribution within the top k (logit.metal:1213-1224) ---------------------------
    if (tid == 0) {
        float cum = 0.0f;
        uint32_t keep = 0;
        while (keep < n) {
            cum += expf(sh.sorted_v[keep] - cap) / total1;
            keep += 1;
            if (cum >= p.top_p) break;
        }
        sh.keep = max(keep, 1u);
    }
    __syncthreads();
    const uint32_t keep = sh.keep;
    // ---- the draw over the survivors --------------------------------------------------------------------------
    unsigned long long best = 0ull;
    float e = 0.0f;
    if (tid < keep) {
        const float v = sh.sorted_v[tid];
        const float g = v * invT + sample_gumbel(seed, key, token_of(sh.sorted_i[tid]));
        e = expf((v - sh.sorted_v[0]) * invT);
        best = ((unsigned long long)sample_key(g) << 32) | (0xFFFFFFFFu - tid);
    }
    best = block_max_k(best, sh);
    const float esum = block_sum_f(e, sh);
    if (tid == 0) {
        const uint32_t bj = 0xFFFFFFFFu - (uint32_t)best;
        out_tokens[r] = sh.sorted_i[bj];
        out_prob[r] = expf((sh.sorted_v[bj] - sh.sorted_v[0]) * invT) / esum;
    }
}

}  // namespace

hipError_t launch_sample_rows(hipStream_t s, const float *logits, uint32_t stride, uint32_t rows, uint32_t count,
                              const uint32_t *ids, float temperature, float top_p, uint32_t top_k, uint32_t key_base,
                              float softcap, unsigned long long seed, const uint32_t *key_offset, uint32_t *out_tokens,
                              float *out_prob) {
    const SampleRule rule{temperature, top_p, top_k, key_base, softcap, (uint32_t)seed, (uint32_t)(seed >> 32)};
    hipLaunchKernelGGL(sample_rows_kernel, dim3(rows), dim3(kSampleThreads), 0, s, logits, stride, count, ids, rule, key_offset,
                       out_tokens, out_prob);
    return hipGetLastError();
}

}  // namespace ffmoe
