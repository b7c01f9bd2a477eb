// Decode-step attention for the BitNet decoder: rotary embedding of q and k,
// KV-cache write and grouped-query attention of one new token per sequence,
// in one kernel.  It is the caller-side glue between the wqkv and wo BitLinear
// calls (gpu/model.py:128-157 of the reference, which uses xformers'
// rope_padded and flash attention there); a floating-point kernel, checked
// against a torch fp32 restatement within a stated tolerance.
//
// One workgroup per (kv head, sequence): the g = n_heads / n_kv_heads query
// heads that share the kv head are processed together so every cached K / V
// row is read once.  Phases: (1) rope + cache write, rotated q kept in LDS as
// bf16; (2) scores with bf16 MFMA, 16 cached positions per wave and step; (3) softmax per head; (4) P.V with the positions split
// over the waves and combined through LDS.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bitnet_decoder_ops.h"

namespace {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kHeadDim = 128;
constexpr int kMaxGroup = 8;
constexpr int kAttnThreads = 1024;
constexpr int kAttnWaves = kAttnThreads / 64;

__device__ __forceinline__ float bf16f(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ uint16_t to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float wave_max_f32(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}
__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

template <int G>  // query heads per kv head
__global__ __launch_bounds__(kAttnThreads) void attn_decode_kernel(
    const uint16_t* __restrict__ qkv, uint16_t* __restrict__ cache_k, uint16_t* __restrict__ cache_v,
    const int64_t* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    uint16_t* __restrict__ out, int S, int n_heads, int n_kv_heads) {
    extern __shared__ float sc[];  // [g][S] scores, then probabilities; then part[kAttnWaves][g][kHeadDim]
    __shared__ __attribute__((aligned(16))) uint16_t qb[G][kHeadDim];  // rotated q as bf16
    __shared__ float inv_sum[G];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int kvh = blockIdx.x;
    const int b = blockIdx.y;
    constexpr int g = G;
    const int p = (int)positions[b];
    const int row_elems = (n_heads + 2 * n_kv_heads) * kHeadDim;
    const uint16_t* row = qkv + (size_t)b * row_elems;
    const size_t cache_row = (size_t)n_kv_heads * kHeadDim;  // elements between positions
    uint16_t* ck = cache_k + ((size_t)b * S * n_kv_heads + kvh) * kHeadDim;
    uint16_t* cv = cache_v + ((size_t)b * S * n_kv_heads + kvh) * kHeadDim;
    float* part = sc + (size_t)g * S;

    // (1) rope on adjacent pairs, in fp32, results rounded to bf16; k and v of the new
    // token go to the cache, from where phases 2 and 4 read them like any other row
    // (same workgroup, after a barrier)
    for (int it = tid; it < (g + 2) * (kHeadDim / 2); it += kAttnThreads) {
        const int hh = it / (kHeadDim / 2);
        const int i = it - hh * (kHeadDim / 2);
        if (hh < g + 1) {
            const int src = hh < g ? (kvh * g + hh) * kHeadDim : (n_heads + kvh) * kHeadDim;
            const uint32_t pr = *(const uint32_t*)(row + src + 2 * i);
            const float a = bf16f(pr & 0xffffu), c = bf16f(pr >> 16);
            const float cs = cos_t[(size_t)p * (kHeadDim / 2) + i], sn = sin_t[(size_t)p * (kHeadDim / 2) + i];
            const uint16_t r0 = to_bf16(a * cs - c * sn), r1 = to_bf16(a * sn + c * cs);
            if (hh < g) {
                *(uint32_t*)(&qb[hh][2 * i]) = (uint32_t)r0 | ((uint32_t)r1 << 16);
            } else {
                *(uint32_t*)(ck + (size_t)p * cache_row + 2 * i) = (uint32_t)r0 | ((uint32_t)r1 << 16);
            }
        } else {
            const uint32_t pr = *(const uint32_t*)(row + (n_heads + n_kv_heads + kvh) * kHeadDim + 2 * i);
            *(uint32_t*)(cv + (size_t)p * cache_row + 2 * i) = pr;
        }
    }
    __syncthreads();

    // (2) scores with bf16 MFMA 16x16x32 (products of bf16 values are exact in fp32, sums are
    // fp32): A = the rotated q rows (heads, zero rows beyond G), B = 16 cached positions; a lane
    // supplies 8 consecutive dims (lane / 16 picks which 8 of a 32-dim step) of row / position
    // lane % 16, i.e. one 16-byte piece of a K row.  Four steps cover the 128 dims.
    const float scale = 0.08838834764831845f;  // 128^-0.5
    {
        const int c = lane & 15, g4 = lane >> 4;
        v8bf qa[4];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            uint4 t = make_uint4(0, 0, 0, 0);
            if (c < G) t = *(const uint4*)(&qb[c][kk * 32 + g4 * 8]);
            qa[kk] = __builtin_bit_cast(v8bf, t);
        }
        // R blocks of 16 positions per wave and round, all their K pieces requested before the first MFMA
        constexpr int R = 3;
        for (int s0 = wave * 16; s0 <= p; s0 += kAttnWaves * 16 * R) {
            uint4 kb[R][4];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int s = s0 + r * kAttnWaves * 16 + c;
                const uint16_t* kr = ck + (size_t)(s <= p ? s : p) * cache_row + g4 * 8;
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) kb[r][kk] = *(const uint4*)(kr + kk * 32);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int s = s0 + r * kAttnWaves * 16 + c;
                v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int kk = 0; kk < 4; ++kk)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[kk], __builtin_bit_cast(v8bf, kb[r][kk]), acc, 0, 0, 0);
                // result lane: position c, heads 4 * g4 + j in register j
                if (s <= p) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (4 * g4 + j < G) sc[(size_t)(4 * g4 + j) * S + s] = acc[j] * scale;
                }
            }
        }
    }
    __syncthreads();

    // (3) softmax over positions 0..p, one head per wave at a time
    for (int hh = wave; hh < g; hh += kAttnWaves) {
        float* srow = sc + (size_t)hh * S;
        float mx = -INFINITY;
        for (int s = lane; s <= p; s += 64) mx = fmaxf(mx, srow[s]);
        mx = wave_max_f32(mx);
        float sum = 0.0f;
        for (int s = lane; s <= p; s += 64) {
            const float e = __expf(srow[s] - mx);
            srow[s] = e;
            sum += e;
        }
        sum = wave_sum_f32(sum);
        if (lane == 0) inv_sum[hh] = 1.0f / sum;
    }
    __syncthreads();

    // (4) out[hh][d] = sum_s prob[hh][s] * v[s][d]: every wave takes positions wave, wave + 16, ...
    // for all g heads at once (a V row is read once), a lane owns dims 2*lane, 2*lane+1;
    // 32 rows are requested per round so their latencies overlap
    float a0[G], a1[G];
#pragma unroll
    for (int hh = 0; hh < G; ++hh) a0[hh] = a1[hh] = 0.0f;
    constexpr int U = 32;
    for (int s0 = wave; s0 <= p; s0 += kAttnWaves * U) {
        uint32_t pr[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int s = s0 + j * kAttnWaves;
            pr[j] = *(const uint32_t*)(cv + (size_t)(s <= p ? s : p) * cache_row + 2 * lane);
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int s = s0 + j * kAttnWaves;
            if (s <= p) {
                const float v0 = bf16f(pr[j] & 0xffffu), v1 = bf16f(pr[j] >> 16);
#pragma unroll
                for (int hh = 0; hh < G; ++hh) {
                    const float pw = sc[(size_t)hh * S + s];
                    a0[hh] += pw * v0;
                    a1[hh] += pw * v1;
                }
            }
        }
    }
#pragma unroll
    for (int hh = 0; hh < G; ++hh) {
        part[((size_t)wave * g + hh) * kHeadDim + 2 * lane] = a0[hh];
        part[((size_t)wave * g + hh) * kHeadDim + 2 * lane + 1] = a1[hh];
    }
    __syncthreads();
    for (int hh = wave; hh < g; hh += kAttnWaves) {
        float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
        for (int k = 0; k < kAttnWaves; ++k) {
            o0 += part[((size_t)k * g + hh) * kHeadDim + 2 * lane];
            o1 += part[((size_t)k * g + hh) * kHeadDim + 2 * lane + 1];
        }
        const float is = inv_sum[hh];
        const uint32_t pk = (uint32_t)to_bf16(o0 * is) | ((uint32_t)to_bf16(o1 * is) << 16);
        *(uint32_t*)(out + (size_t)b * n_heads * kHeadDim + (size_t)(kvh * g + hh) * kHeadDim + 2 * lane) = pk;
    }
}

}  // namespace

extern "C" int bitnet_attn_decode(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v, const int64_t* positions,
                                  const float* cos_table, const float* sin_table, uint16_t* out, int B, int S,
                                  int n_heads, int n_kv_heads, int head_dim, void* stream) {
    if (B < 1 || S < 1 || n_heads < 1 || n_kv_heads < 1 || head_dim != kHeadDim) return 1;
    if (n_heads % n_kv_heads) return 1;
    const int g = n_heads / n_kv_heads;
    if (g != 1 && g != 2 && g != 4 && g != 8) return 1;
    if (!qkv || !cache_k || !cache_v || !positions || !cos_table || !sin_table || !out) return 2;
    const size_t lds = ((size_t)g * S + (size_t)kAttnWaves * g * kHeadDim) * sizeof(float);
    if (lds > 96u * 1024u) return 1;
    const dim3 grid(n_kv_heads, B, 1), block(kAttnThreads, 1, 1);
#define BITNET_ATTN_LAUNCH(GG)                                                                                        \
    {                                                                                                                 \
        static bool raised = false; /* more than 64 KiB of dynamic LDS has to be asked for, once per process */     \
        if (!raised) {                                                                                                \
            (void)hipFuncSetAttribute((const void*)attn_decode_kernel<GG>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                      96 * 1024);                                                                     \
            raised = true;                                                                                            \
        }                                                                                                             \
        hipLaunchKernelGGL(attn_decode_kernel<GG>, grid, block, lds, (hipStream_t)stream, qkv, cache_k, cache_v,      \
                           positions, cos_table, sin_table, out, S, n_heads, n_kv_heads);                            \
    }
    switch (g) {
        case 1: BITNET_ATTN_LAUNCH(1) break;
        case 2: BITNET_ATTN_LAUNCH(2) break;
        case 4: BITNET_ATTN_LAUNCH(4) break;
        case 8: BITNET_ATTN_LAUNCH(8) break;
        default: return 1;
    }
#undef BITNET_ATTN_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : 3;
}
