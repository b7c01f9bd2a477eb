// Host entry points of the decode-step attention (rotary embedding of q and k, KV-cache write and
// grouped-query attention of one new token per sequence, in one kernel: the caller-side glue between
// the wqkv and wo BitLinear calls, gpu/model.py:128-157 of the reference, which uses xformers'
// rope_padded and flash attention there; the kernel itself lives in attn_prefill.hip), and the final
// RMSNorm + bf16 LM head + greedy token.  Floating-point kernels, checked against torch fp32
// restatements within stated tolerances.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "bitnet_decoder_ops.h"
#include "host_util.h"

namespace {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kHeadDim = 128;
constexpr int kMaxGroup = 8;
constexpr int kAttnMinThreads = 256;
constexpr int kAttnMaxThreads = 512;

__device__ __forceinline__ float bf16f(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ uint16_t to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Wave-wide reductions with DPP lane permutes (no LDS traffic, no waiting): two quad permutes and
// two mirrors leave every lane of a 16-lane row with the row's result; the four row results are
// combined through scalar registers.  All lanes must be active.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_f32(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_f32<0x4E>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_f32<0x141>(v));  // row_half_mirror
    v = fmaxf(v, dpp_f32<0x140>(v));  // row_mirror
    return fmaxf(fmaxf(lane_f32(v, 0), lane_f32(v, 16)), fmaxf(lane_f32(v, 32), lane_f32(v, 48)));
}
__device__ __forceinline__ float wave_sum_f32(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    return (lane_f32(v, 0) + lane_f32(v, 16)) + (lane_f32(v, 32) + lane_f32(v, 48));
}

// Workspace record of one (sequence, kv head, split): G heads x (128 unnormalised outputs,
// running maximum, sum of exponentials)
constexpr int kRecFloats = kHeadDim + 2;
constexpr int kMaxSplits = 16;

// ---------------------------------------------------------------------------
// Final RMSNorm + bf16 LM head + greedy token (gpu/model.py:280-281 followed by
// the argmax of gpu/generate.py:264-288)
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2));
}

// y = bf16((h * rstd) * g), rstd = 1 / sqrt(mean(h^2) + eps): the sum of squares in fp64 (exact
// for bf16 data, so independent of the order), rounded to fp32 and divided by K in fp32.
// One workgroup per row.
constexpr int kNormThreads = 256;
__global__ __launch_bounds__(kNormThreads) void rmsnorm_rows_kernel(const uint16_t* __restrict__ h,
                                                                    const uint16_t* __restrict__ g, float eps,
                                                                    uint16_t* __restrict__ y, int K) {
    __shared__ double wsum[kNormThreads / 64];
    const int row = blockIdx.x, tid = threadIdx.x;
    const int nvec = K >> 3;
    const uint4* hr = (const uint4*)(h + (size_t)row * K);
    double sq = 0.0;
    for (int i = tid; i < nvec; i += kNormThreads) {
        const uint4 v = hr[i];
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float lo = bf16f(d[j] & 0xffffu), hi = bf16f(d[j] >> 16);
            sq += (double)(lo * lo) + (double)(hi * hi);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off);
    if ((tid & 63) == 0) wsum[tid >> 6] = sq;
    __syncthreads();
    double total = 0.0;
#pragma unroll
    for (int i = 0; i < kNormThreads / 64; ++i) total += wsum[i];
    const float mean = (float)total / (float)K;
    const float rstd = 1.0f / __builtin_sqrtf(mean + eps);
    uint4* yr = (uint4*)(y + (size_t)row * K);
    for (int i = tid; i < nvec; i += kNormThreads) {
        const uint4 v = hr[i], w = ((const uint4*)g)[i];
        const uint32_t d[4] = {v.x, v.y, v.z, v.w}, e[4] = {w.x, w.y, w.z, w.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            o[j] = pack_bf16x2(bf16f(d[j] & 0xffffu) * rstd * bf16f(e[j] & 0xffffu), bf16f(d[j] >> 16) * rstd * bf16f(e[j] >> 16));
        yr[i] = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// logits[b, v] = bf16(sum_k y[b, k] * emb[v, k]) (fp32 accumulation), token[b] = the first v with
// the largest logit.  A wave owns 16 vocabulary rows over all of K: the embedding streams through
// registers as the row operand of bf16 MFMA 16x16x32 (a lane holds 16 consecutive k of one row
// per 64-k step, two MFMAs), kLmDepth steps in flight; the normalised rows sit in LDS and are
// the column operand (columns = tokens).  Each workgroup leaves its best (value, row) per token
// in a workspace; lm_head_final_kernel reduces them.
constexpr int kLmThreads = 256;
constexpr int kLmDepth = 4;
constexpr int kLmMaxTokens = 16;
constexpr int kLmRowPad = 32;  // bytes between token rows in LDS beyond 2 * K

__device__ __forceinline__ bool lm_better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

__global__ __launch_bounds__(kLmThreads) void lm_head_kernel(const uint16_t* __restrict__ y,
                                                             const uint16_t* __restrict__ emb, float* __restrict__ logits,
                                                             float* __restrict__ part_val, int* __restrict__ part_idx,
                                                             int B, int V, int K) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_y[];  // [B][2 * K + pad]
    __shared__ float wv[kLmThreads / 64][kLmMaxTokens];
    __shared__ int wi[kLmThreads / 64][kLmMaxTokens];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int steps = K >> 6;
    const int row_stride = 2 * K + kLmRowPad;
    const int rb = blockIdx.x * (kLmThreads / 64) + wave;
    int row = rb * 16 + r16;
    row = row < V ? row : V - 1;
    const v4u* wrow = (const v4u*)(emb + (size_t)row * K + g * 16);

    v4u w[kLmDepth][2];
#pragma unroll
    for (int j = 0; j < kLmDepth; ++j) {
        const int st = j < steps ? j : steps - 1;
        w[j][0] = __builtin_nontemporal_load(wrow + st * 8);
        w[j][1] = __builtin_nontemporal_load(wrow + st * 8 + 1);
    }
    // the normalised rows -> LDS while the first embedding pieces are in flight
    {
        const int vec_per_row = K >> 3;
        for (int i = tid; i < B * vec_per_row; i += kLmThreads) {
            const int b = i / vec_per_row, c = i - b * vec_per_row;
            *(uint4*)(lds_y + (size_t)b * row_stride + c * 16) = *(const uint4*)(y + (size_t)b * K + c * 8);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

    const int tok = r16 < B ? r16 : B - 1;  // columns of tokens >= B are never read
    const uint8_t* yb = lds_y + (size_t)tok * row_stride + g * 32;
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int s0 = 0; s0 < steps; s0 += kLmDepth) {
#pragma unroll
        for (int j = 0; j < kLmDepth; ++j) {
            const int st = s0 + j;
            if (st < steps) {  // uniform
                const uint4 b0 = *(const uint4*)(yb + st * 128), b1 = *(const uint4*)(yb + st * 128 + 16);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, w[j][0]), __builtin_bit_cast(v8bf, b0), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, w[j][1]), __builtin_bit_cast(v8bf, b1), acc, 0, 0, 0);
            }
            const int nx = (st + kLmDepth) < steps ? (st + kLmDepth) : (steps - 1);
            w[j][0] = __builtin_nontemporal_load(wrow + nx * 8);
            w[j][1] = __builtin_nontemporal_load(wrow + nx * 8 + 1);
        }
    }

    // result lane (g, token r16): rows rb*16 + 4g + r in register r
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int vr = rb * 16 + 4 * g + r;
        const float val = bf16f(pack_bf16x2(acc[r], 0.0f) & 0xffffu);
        if (vr < V && r16 < B) {
            if (logits) logits[(size_t)r16 * V + vr] = val;
            if (lm_better(val, vr, bv, bi)) {
                bv = val;
                bi = vr;
            }
        }
    }
#pragma unroll
    for (int off = 16; off < 64; off <<= 1) {
        const float ov = __shfl_xor(bv, off);
        const int oi = __shfl_xor(bi, off);
        if (lm_better(ov, oi, bv, bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if (g == 0) {
        wv[wave][r16] = bv;
        wi[wave][r16] = bi;
    }
    __syncthreads();
    if (tid < kLmMaxTokens) {
        float v = wv[0][tid];
        int i = wi[0][tid];
#pragma unroll
        for (int k = 1; k < kLmThreads / 64; ++k)
            if (lm_better(wv[k][tid], wi[k][tid], v, i)) {
                v = wv[k][tid];
                i = wi[k][tid];
            }
        part_val[(size_t)blockIdx.x * kLmMaxTokens + tid] = v;
        part_idx[(size_t)blockIdx.x * kLmMaxTokens + tid] = i;
    }
}


// The same result for up to 8 tokens without the matrix pipe: a wave owns 8 consecutive
// vocabulary rows (40 KB of the embedding at K = 2560, contiguous), every load instruction takes
// 1 KB of ONE row (64 lanes x 8 consecutive k), and a lane multiplies its 8 values with the
// matching 8 of each token (bf16 dot2 with fp32 accumulation).  Long contiguous requests are
// what the memory system serves best; the per-lane partial sums of the 8 x TB (row, token)
// pairs are combined at the end by a halving butterfly over the lanes.
constexpr int kLsRows = 8;
// a + w.lo * x.lo + w.hi * x.hi on packed bf16 pairs, products and sums in fp32
__device__ __forceinline__ float bf16_dot2(uint32_t w, uint32_t x, float a) {
    a = __builtin_fmaf(__uint_as_float(w << 16), __uint_as_float(x << 16), a);
    return __builtin_fmaf(__uint_as_float(w & 0xffff0000u), __uint_as_float(x & 0xffff0000u), a);
}

template <int TB>  // tokens (columns) computed: 1, 2, 4 or 8 >= B
__global__ __launch_bounds__(kLmThreads) void lm_head_stream_kernel(const uint16_t* __restrict__ y,
                                                                    const uint16_t* __restrict__ emb,
                                                                    float* __restrict__ logits,
                                                                    float* __restrict__ part_val,
                                                                    int* __restrict__ part_idx, int B, int V, int K) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_y[];  // [B][2 * K]
    __shared__ float cv[kLmThreads / 64][kLmMaxTokens][kLsRows];
    __shared__ int ci[kLmThreads / 64][kLmMaxTokens][kLsRows];
    constexpr int NV = kLsRows * TB;  // (row, token) pairs per wave and row group
    constexpr int kShift = NV == 64 ? 0 : (NV == 32 ? 1 : (NV == 16 ? 2 : 3));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int steps = K >> 9;  // 512 k per step
    const int groups = (V + kLsRows - 1) / kLsRows;
    const int nwaves = gridDim.x * (kLmThreads / 64);
    int grp = blockIdx.x * (kLmThreads / 64) + wave;  // persistent: groups grp, grp + nwaves, ...

    // first 1 KB of each of the first group's rows (a wave without a group re-reads the last row)
    const v4u* wp[kLsRows];
    v4u w[kLsRows];
    auto group_rows = [&](int gidx) {
#pragma unroll
        for (int r = 0; r < kLsRows; ++r) {
            int row = gidx * kLsRows + r;
            row = row < V ? row : V - 1;
            wp[r] = (const v4u*)(emb + (size_t)row * K) + lane;
        }
    };
    group_rows(grp < groups ? grp : groups - 1);
#pragma unroll
    for (int r = 0; r < kLsRows; ++r) w[r] = __builtin_nontemporal_load(wp[r]);
    {
        const int nvec = (B * K) >> 3;
        for (int i = tid; i < nvec; i += kLmThreads) *(uint4*)(lds_y + (size_t)i * 16) = *(const uint4*)(y + (size_t)i * 8);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

    // the lane that ends up with pair (row pr of a group, token pt) keeps the best over its groups
    const int pair = lane >> kShift;
    const int pr = pair / TB, pt = pair % TB;
    const bool owner = (lane & ((1 << kShift) - 1)) == 0 && pt < B;
    float bv = -INFINITY;
    int bi = 0x7fffffff;

    for (; grp < groups; grp += nwaves) {
        float acc[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[i] = 0.0f;
        for (int s = 0; s < steps; ++s) {
            v4u xs[TB];
#pragma unroll
            for (int t = 0; t < TB; ++t) {
                const int tok = t < B ? t : B - 1;
                xs[t] = *(const v4u*)(lds_y + (size_t)tok * 2 * K + (size_t)s * 1024 + lane * 16);
            }
            // what to request next: this group's next 1 KB per row, or the first 1 KB of the wave's next group
            int off = (s + 1) * 64;
            if (s + 1 == steps) {  // uniform
                const int nxt = grp + nwaves;
                group_rows(nxt < groups ? nxt : grp);
                off = 0;
            }
#pragma unroll
            for (int r = 0; r < kLsRows; ++r) {
                const v4u wr = w[r];
                w[r] = __builtin_nontemporal_load(wp[r] + off);
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    float a = acc[r * TB + t];
#pragma unroll
                    for (int j = 0; j < 4; ++j) a = bf16_dot2(wr[j], xs[t][j], a);
                    acc[r * TB + t] = a;
                }
            }
        }
        // halving butterfly: after the stage with lane-xor mask m a lane keeps the half of its values
        // chosen by its bit m; after log2(NV) stages lane l holds pair l >> log2(64 / NV), still as a
        // partial over the lanes that differ in the low bits, which a plain xor reduction finishes
        int m = 32;
#pragma unroll
        for (int n = NV; n > 1; n >>= 1) {
            const bool up = (lane & m) != 0;
#pragma unroll
            for (int i = 0; i < n / 2; ++i) {
                const float keep = up ? acc[i + n / 2] : acc[i];
                const float send = up ? acc[i] : acc[i + n / 2];
                acc[i] = keep + __shfl_xor(send, m);
            }
            m >>= 1;
        }
        float total = acc[0];
        for (; m > 0; m >>= 1) total += __shfl_xor(total, m);
        const int vr = grp * kLsRows + pr;
        const float val = bf16f(pack_bf16x2(total, 0.0f) & 0xffffu);
        if (owner && vr < V) {
            if (logits) logits[(size_t)pt * V + vr] = val;
            if (lm_better(val, vr, bv, bi)) {
                bv = val;
                bi = vr;
            }
        }
    }
    if (owner) {
        cv[wave][pt][pr] = bv;
        ci[wave][pt][pr] = bi;
    }
    __syncthreads();
    if (tid < kLmMaxTokens) {
        float v = -INFINITY;
        int i = 0x7fffffff;
        if (tid < B) {
#pragma unroll
            for (int k = 0; k < kLmThreads / 64; ++k)
#pragma unroll
                for (int r = 0; r < kLsRows; ++r)
                    if (lm_better(cv[k][tid][r], ci[k][tid][r], v, i)) {
                        v = cv[k][tid][r];
                        i = ci[k][tid][r];
                    }
        }
        part_val[(size_t)blockIdx.x * kLmMaxTokens + tid] = v;
        part_idx[(size_t)blockIdx.x * kLmMaxTokens + tid] = i;
    }
}

// Best (value, row) per token over the workgroups' partial results: one workgroup, all loads of a
// thread independent and in flight together (a dependent chain of single loads would cost a
// memory round trip each).  A kernel of its own: the kernel boundary orders the partial results for
// free, where a device-wide arrival counter would serialise thousands of atomics on one address.
constexpr int kLmFinalThreads = kLmMaxTokens * 64;
// Optional bookkeeping of a greedy decode step, done by the same kernel instead of four small
// launches behind it: the token becomes the next step's input, goes into the history row of the
// current step, and the positions and the step counter advance.  Null pointers: not done.
struct LmStepBook {
    int64_t* next_input;  // [B]
    int64_t* positions;   // [B], each += 1
    int64_t* history;     // [steps][B], row step_idx[0] written
    int64_t* step_idx;    // [1], += 1
};

__global__ __launch_bounds__(kLmFinalThreads) void lm_head_final_kernel(const float* __restrict__ part_val,
                                                                        const int* __restrict__ part_idx,
                                                                        int64_t* __restrict__ token_out, int nparts, int B,
                                                                        LmStepBook book) {
    // The candidates are [nparts][16 token slots]; a thread reads whole 16-byte pieces (four token
    // slots of one workgroup's candidates), consecutive threads consecutive pieces.  One workgroup's
    // loads all go through one CU's address path, which handles one 64-byte segment per cycle: with
    // a lane per candidate and a wave per token every load instruction touched 64 segments and the
    // kernel took 16 us; now a load instruction touches 16.
    __shared__ float sv[kLmFinalThreads / 64][kLmMaxTokens];
    __shared__ int si[kLmFinalThreads / 64][kLmMaxTokens];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = tid & 3;  // this thread's token slots are 4 q .. 4 q + 3
    float v[4];
    int i[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        v[e] = -INFINITY;
        i[e] = 0x7fffffff;
    }
    const int nvec = nparts * 4;
    constexpr int U = 4;
    for (int base = tid; base < nvec; base += kLmFinalThreads * U) {
        v4f ov[U];
        v4i oi[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = base + kLmFinalThreads * u;
            const int at = k < nvec ? k : nvec - 4 + q;  // a piece of the same token slots
            ov[u] = ((const v4f*)part_val)[at];
            oi[u] = ((const v4i*)part_idx)[at];
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (base + kLmFinalThreads * u < nvec) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (lm_better(ov[u][e], oi[u][e], v[e], i[e])) {
                        v[e] = ov[u][e];
                        i[e] = oi[u][e];
                    }
            }
    }
    // the 16 lanes of a wave that hold the same token slots
#pragma unroll
    for (int off = 4; off < 64; off <<= 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float ov = __shfl_xor(v[e], off);
            const int oi = __shfl_xor(i[e], off);
            if (lm_better(ov, oi, v[e], i[e])) {
                v[e] = ov;
                i[e] = oi;
            }
        }
    }
    if (lane < 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            sv[wave][4 * lane + e] = v[e];
            si[wave][4 * lane + e] = i[e];
        }
    }
    __syncthreads();
    if (tid < kLmMaxTokens) {
        const int t = tid;
        float bv = sv[0][t];
        int bi = si[0][t];
#pragma unroll
        for (int w = 1; w < kLmFinalThreads / 64; ++w)
            if (lm_better(sv[w][t], si[w][t], bv, bi)) {
                bv = sv[w][t];
                bi = si[w][t];
            }
        if (t < B) {
            token_out[t] = (int64_t)bi;
            if (book.next_input) book.next_input[t] = (int64_t)bi;
            if (book.positions) book.positions[t] += 1;
            if (book.history && book.step_idx) book.history[book.step_idx[0] * B + t] = (int64_t)bi;
        }
    }
    if (book.step_idx) {
        __syncthreads();  // every token's history row index has been read
        if (tid == 0) book.step_idx[0] += 1;
    }
}


}  // namespace

static std::atomic<int> g_attn_threads{0};

// in attn_prefill.hip
int bitnet_attn_decode_flash_launch(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v, const int64_t* positions,
                                    const float* cos_table, const float* sin_table, const float* rope_rows, uint16_t* out,
                                    float* workspace, int* counters, int n_splits, int threads, int B, int S,
                                    int n_heads, int n_kv_heads, int spin_limit, hipStream_t stream);

static std::atomic<int> g_attn_spin_limit{-1};  // polls of the merging workgroup; < 0 = the kernel's own limit

/* test hook: the bound of the merging workgroup's poll (< 0 restores the built-in bound; 0 makes every
   merge of more than one split give up at once, which is how the failure path is tested) */
extern "C" int bitnet_attn_decode_set_spin_limit(int polls) {
    g_attn_spin_limit = polls < 0 ? -1 : polls;
    return 0;
}

/* tuning override: threads per workgroup of the attention kernel (0 = built-in choice) */
extern "C" int bitnet_attn_decode_set_threads(int threads) {
    if (threads != 0 && threads != 256 && threads != 512) return 1;
    g_attn_threads = threads;
    return 0;
}

// records of 8-byte units (value, tag) per (sequence, kv head, split, head), then one epoch per
// (sequence, kv head), then the error word and a word of padding
static long long attn_ws_error_index(int B, int n_heads, int n_kv_heads, int n_splits) {
    return (long long)B * n_kv_heads * n_splits * (n_heads / n_kv_heads) * kRecFloats * 2 + (long long)B * n_kv_heads;
}

extern "C" int bitnet_attn_decode_workspace_floats(int B, int n_heads, int n_kv_heads, int n_splits) {
    if (B < 1 || n_heads < 1 || n_kv_heads < 1 || n_splits < 1 || n_heads % n_kv_heads) return -1;
    const long long n = attn_ws_error_index(B, n_heads, n_kv_heads, n_splits) + 2;
    return n < (1ll << 31) ? (int)n : -1;
}

extern "C" int bitnet_attn_decode_error_index(int B, int n_heads, int n_kv_heads, int n_splits) {
    if (B < 1 || n_heads < 1 || n_kv_heads < 1 || n_splits < 1 || n_heads % n_kv_heads) return -1;
    const long long n = attn_ws_error_index(B, n_heads, n_kv_heads, n_splits);
    return n + 2 < (1ll << 31) ? (int)n : -1;
}

static int attn_decode_impl(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v, const int64_t* positions,
                            const float* cos_table, const float* sin_table, const float* rope_rows, uint16_t* out,
                            float* workspace, int* counters, int n_splits, int B, int S, int n_heads, int n_kv_heads,
                            int head_dim, void* stream) {
    if (B < 1 || S < 1 || n_heads < 1 || n_kv_heads < 1 || head_dim != kHeadDim) return 1;
    if (n_heads % n_kv_heads) return 1;
    const int g = n_heads / n_kv_heads;
    if (g != 1 && g != 2 && g != 4 && g != 8) return 1;
    if (n_splits < 1 || n_splits > kMaxSplits) return 1;
    if (!qkv || !cache_k || !cache_v || !positions || !cos_table || !sin_table || !out) return 2;
    if (n_splits > 1 && (!workspace || !counters)) return 2;
    if (((uintptr_t)workspace) & 7u) return 1;
    // the kernel's 32-bit byte offsets into one sequence's cache (the first blocks requested may lie up to 4096 rows in)
    if ((size_t)((S > 4096 ? S : 4096) + 512) * n_kv_heads * kHeadDim * 2 >= ((size_t)1 << 31)) return 1;
    const int span = ((S + n_splits - 1) / n_splits + 15) & ~15;  // a split's share of the cache capacity
    // The kernel deals blocks of 32 rows to splits and waves: four waves cover a split's share of up to 128
    // rows of the capacity in one round (measured at 96 rows: 6.85 us with four waves, 7.12 with eight; at 272
    // rows 8.77 / 8.46).  Eight waves while every workgroup has a CU of its own (up to 256 of them); beyond
    // that two 512-thread workgroups share a CU badly and 256 threads are the better choice.
    int threads = (span > 128 && (long long)n_kv_heads * B * n_splits <= 256) ? 512 : 256;
    if (const int forced = g_attn_threads.load()) threads = forced;
    return bitnet_attn_decode_flash_launch(qkv, cache_k, cache_v, positions, cos_table, sin_table, rope_rows, out, workspace,
                                           counters, n_splits, threads, B, S, n_heads, n_kv_heads, g_attn_spin_limit.load(),
                                           (hipStream_t)stream);
}

extern "C" int bitnet_attn_decode(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v, const int64_t* positions,
                                  const float* cos_table, const float* sin_table, uint16_t* out, float* workspace,
                                  int* counters, int n_splits, int B, int S, int n_heads, int n_kv_heads, int head_dim,
                                  void* stream) {
    return attn_decode_impl(qkv, cache_k, cache_v, positions, cos_table, sin_table, nullptr, out, workspace, counters, n_splits,
                            B, S, n_heads, n_kv_heads, head_dim, stream);
}

extern "C" int bitnet_attn_decode_rows(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v, const int64_t* positions,
                                       const float* cos_table, const float* sin_table, const float* rope_rows, uint16_t* out,
                                       float* workspace, int* counters, int n_splits, int B, int S, int n_heads,
                                       int n_kv_heads, int head_dim, void* stream) {
    if (!rope_rows) return 2;
    return attn_decode_impl(qkv, cache_k, cache_v, positions, cos_table, sin_table, rope_rows, out, workspace, counters,
                            n_splits, B, S, n_heads, n_kv_heads, head_dim, stream);
}

static std::atomic<int> g_lm_kernel{0};  // 0 = built-in choice, 1 = matrix-pipe kernel, 2 = streaming kernel where it applies

/* tuning override for tests and measurements; results differ only in the order of fp32 additions */
extern "C" int bitnet_lm_head_set_kernel(int which) {
    if (which < 0 || which > 2) return 1;
    g_lm_kernel = which;
    return 0;
}

extern "C" int bitnet_lm_head_workgroups(int V) {
    if (V < 1) return -1;
    const int rows_per_wg = kLsRows * (kLmThreads / 64);  // the kernel with the fewest rows per workgroup
    return (V + rows_per_wg - 1) / rows_per_wg;
}

static int lm_head_greedy_impl(const uint16_t* h, const uint16_t* norm_weight, float eps, const uint16_t* emb,
                               uint16_t* y_ws, float* logits, int64_t* token_out, float* part_val, int* part_idx,
                               const LmStepBook& book, int B, int V, int K, void* stream) {
    if (B < 1 || B > kLmMaxTokens || V < 1 || K < 64 || (K % 64) != 0) return 1;
    if (!h || !norm_weight || !emb || !y_ws || !token_out || !part_val || !part_idx) return 2;
    if ((((uintptr_t)h) | ((uintptr_t)norm_weight) | ((uintptr_t)emb) | ((uintptr_t)y_ws) | ((uintptr_t)part_val) |
         ((uintptr_t)part_idx)) & 15u)
        return 1;
    const size_t lds = (size_t)B * (2 * (size_t)K + kLmRowPad);
    if (lds > 96u * 1024u) return 1;
    static bitnet_host::OncePerDevice raised;  // more than 64 KiB of dynamic LDS has to be asked for
    if (raised.run([] {
            return hipFuncSetAttribute((const void*)lm_head_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
        }) != hipSuccess)
        return 3;
    hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3(B), dim3(kNormThreads), 0, (hipStream_t)stream, h, norm_weight, eps, y_ws, K);
    int nparts = 0;
    const bool stream_ok = B <= 8 && (K % 512) == 0 && (size_t)B * 2 * K <= 60u * 1024u;
    if (stream_ok && g_lm_kernel != 1) {
        // persistent waves: at most 4 workgroups per CU of a 256-CU part, each wave walking row groups
        const int full = (V + kLsRows * (kLmThreads / 64) - 1) / (kLsRows * (kLmThreads / 64));
        const dim3 grid(full < 1024 ? full : 1024);
        nparts = (int)grid.x;
        const size_t lds_s = (size_t)B * 2 * K;
#define BITNET_LM_STREAM(TB)                                                                                          \
    hipLaunchKernelGGL(lm_head_stream_kernel<TB>, grid, dim3(kLmThreads), lds_s, (hipStream_t)stream, y_ws, emb, logits, \
                       part_val, part_idx, B, V, K)
        if (B == 1) BITNET_LM_STREAM(1);
        else if (B == 2) BITNET_LM_STREAM(2);
        else if (B <= 4) BITNET_LM_STREAM(4);
        else BITNET_LM_STREAM(8);
#undef BITNET_LM_STREAM
    } else {
        const int rows_per_wg = 16 * (kLmThreads / 64);
        nparts = (V + rows_per_wg - 1) / rows_per_wg;
        hipLaunchKernelGGL(lm_head_kernel, dim3(nparts), dim3(kLmThreads), lds, (hipStream_t)stream, y_ws, emb, logits, part_val,
                           part_idx, B, V, K);
    }
    hipLaunchKernelGGL(lm_head_final_kernel, dim3(1), dim3(kLmFinalThreads), 0, (hipStream_t)stream, part_val, part_idx, token_out, nparts, B, book);
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

extern "C" int bitnet_lm_head_greedy(const uint16_t* h, const uint16_t* norm_weight, float eps, const uint16_t* emb,
                                     uint16_t* y_ws, float* logits, int64_t* token_out, float* part_val,
                                     int* part_idx, int B, int V, int K, void* stream) {
    return lm_head_greedy_impl(h, norm_weight, eps, emb, y_ws, logits, token_out, part_val, part_idx,
                               LmStepBook{nullptr, nullptr, nullptr, nullptr}, B, V, K, stream);
}

extern "C" int bitnet_lm_head_greedy_step(const uint16_t* h, const uint16_t* norm_weight, float eps, const uint16_t* emb,
                                          uint16_t* y_ws, float* logits, int64_t* token_out, float* part_val,
                                          int* part_idx, int64_t* next_input, int64_t* positions, int64_t* history,
                                          int64_t* step_idx, int B, int V, int K, void* stream) {
    if ((history != nullptr) != (step_idx != nullptr)) return 2;
    return lm_head_greedy_impl(h, norm_weight, eps, emb, y_ws, logits, token_out, part_val, part_idx,
                               LmStepBook{next_input, positions, history, step_idx}, B, V, K, stream);
}
