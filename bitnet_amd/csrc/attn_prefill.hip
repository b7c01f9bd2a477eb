// Prompt-side glue of the BitNet decoder's attention block (Attention.forward,
// gpu/model.py:128-157, where the reference calls xformers' rope_padded and
// flash attention): rotary embedding + KV-cache write for a block of new
// tokens, and their causal attention over the cache.  Floating-point kernels,
// checked against torch fp32 restatements within stated tolerances.
//
// This file is compiled with -mllvm -amdgpu-mfma-vgpr-form=1: the attention
// kernel rescales its output accumulators with vector instructions between
// matrix instructions, and with the accumulators in the other register file the
// compiler moves all of them across and back in every step.

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "bitnet_decoder_ops.h"

namespace {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr int kHeadDim = 128;

__device__ __forceinline__ float bf16f(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
// fp32 -> bf16, round to nearest even, NaN kept: the same expression as the decode-step kernel's
__device__ __forceinline__ uint16_t to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {  // round to nearest even, one instruction on gfx950
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Rotary embedding and cache write for a block of new tokens (a prompt): one workgroup per
// token.  Items are (head, pair) of the token's q | k | v row; q heads are rotated into q_out,
// k heads rotated into the cache row of the token's position, v heads copied there.  The same
// expressions as phase 1 of attn_decode_kernel, so a prompt processed here and a token
// processed there leave identical cache rows.
constexpr int kRopeThreads = 256;
__global__ __launch_bounds__(kRopeThreads) void rope_cache_tokens_kernel(
    const uint16_t* __restrict__ qkv, uint16_t* __restrict__ cache_k, uint16_t* __restrict__ cache_v,
    const int64_t* __restrict__ positions, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    uint16_t* __restrict__ q_out, int T, int S, int n_heads, int n_kv_heads) {
    const int tok = blockIdx.x;  // b * T + t
    const int b = tok / T;
    const int row_elems = (n_heads + 2 * n_kv_heads) * kHeadDim;
    const uint16_t* row = qkv + (size_t)tok * row_elems;
    const int64_t p_raw = positions[tok];
    const int p = p_raw < 0 ? 0 : (p_raw >= (int64_t)S ? S - 1 : (int)p_raw);  // clamped: nothing outside the buffers is touched
    const size_t cache_off = ((size_t)b * S + p) * n_kv_heads * kHeadDim;
    const int items = (n_heads + 2 * n_kv_heads) * (kHeadDim / 2);
    for (int it = threadIdx.x; it < items; it += kRopeThreads) {
        const int hh = it / (kHeadDim / 2);
        const int i = it - hh * (kHeadDim / 2);
        const uint32_t raw = *(const uint32_t*)(row + (size_t)hh * kHeadDim + 2 * i);
        if (hh < n_heads + n_kv_heads) {
            const float a = bf16f(raw & 0xffffu), cc = bf16f(raw >> 16);
            const float cs = cos_t[(size_t)p * (kHeadDim / 2) + i], sn = sin_t[(size_t)p * (kHeadDim / 2) + i];
            const uint32_t rot = (uint32_t)to_bf16(a * cs - cc * sn) | ((uint32_t)to_bf16(a * sn + cc * cs) << 16);
            if (hh < n_heads)
                *(uint32_t*)(q_out + ((size_t)tok * n_heads + hh) * kHeadDim + 2 * i) = rot;
            else
                *(uint32_t*)(cache_k + cache_off + (size_t)(hh - n_heads) * kHeadDim + 2 * i) = rot;
        } else {
            *(uint32_t*)(cache_v + cache_off + (size_t)(hh - n_heads - n_kv_heads) * kHeadDim + 2 * i) = raw;
        }
    }
}


// Causal attention of a block of T new tokens per sequence (a prompt) over the cache rows
// written for them: flash-attention style, scores and output on the bf16 matrix pipe (16x16x32).
// One wave = 16 consecutive tokens of one query head; the G waves of a workgroup are the G heads
// that share a kv head, so they walk the same cache rows together: the workgroup brings every
// block of 32 K and V rows into LDS once (double buffered, requested two steps ahead, one
// LDS-only barrier per step) and each wave takes its operands from there.
//   S^T block = K rows (A operand: 16 positions x 32 dims per step) x q^T (B operand: 16 tokens),
//   so a result lane (c, g4) holds, for token c, positions 4 g4 + j of the block (j = 0..3).  Two
//   blocks make the 8 positions that this lane contributes, as its k-slots, to the B operand of
//   O^T += V^T P^T: the probabilities go from the accumulators straight into the next MFMA.
//   The matching A operand is V transposed: lane (d, g4) loads, for each of those 8 positions, the
//   16-byte piece d of the V row (dims 8 d .. 8 d + 7); output tile t takes element t of every
//   piece (one byte-permute per pair of positions), i.e. tile t's row d is dim 8 d + t.  A result
//   lane (c, g4) then holds, for token c, dims 32 g4 + 8 j + t: eight contiguous dims per j.
// Online softmax per 32 positions: the running maximum of a token is agreed between its four lanes
// (c, c + 16, c + 32, c + 48) with two lane permutes; the sums stay per lane until the end.
// Workgroup barrier that orders LDS traffic only (__syncthreads() would also wait for the global
// loads in flight).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
constexpr int kApRowBytes = kHeadDim * 2 + 16;  // padded LDS row: the 16 rows of a K operand read spread over all banks
__device__ __forceinline__ float xor_lane_f32(float v, int lane, int mask) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, __float_as_int(v)));
}

template <int G>
__global__ __launch_bounds__(64 * G) void attn_prefill_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache_k, const uint16_t* __restrict__ cache_v,
    uint16_t* __restrict__ out, int T, int S, int start, int n_heads, int n_kv_heads) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, g4 = lane >> 4;
    const int qb = gridDim.x - 1 - blockIdx.x;  // the blocks with the most positions start first
    const int kvh = blockIdx.y, b = blockIdx.z;
    const int head = kvh * G + wave;
    const int t0 = qb * 16;
    const int tq = (t0 + c) < T ? (t0 + c) : (T - 1);
    const int pq = start + t0 + c;  // position of this lane's token: cache rows 0..pq are visible to it
    const int n_pos = start + ((t0 + 16) < T ? (t0 + 16) : T);  // rows [0, n_pos) matter to this block
    const int steps = (n_pos + 31) >> 5;

    // q^T as the B operand of the four 32-dim steps
    v8bf qa[4];
    {
        const uint16_t* qrow = q + (((size_t)b * T + tq) * n_heads + head) * kHeadDim;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) qa[kk] = __builtin_bit_cast(v8bf, *(const uint4*)(qrow + kk * 32 + g4 * 8));
    }
    // cache rows through descriptors that end behind row n_pos - 1: requests beyond read as zero
    // at no cost, so neither the last step nor the prefetch past it needs a clamped index, and no
    // stale row behind the prompt can put a NaN into the products
    const int row_bytes = n_kv_heads * kHeadDim * 2;
    const int span_bytes = (n_pos - 1) * row_bytes + kHeadDim * 2;
    const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(cache_k + ((size_t)b * S * n_kv_heads + kvh) * kHeadDim), 0, span_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(cache_v + ((size_t)b * S * n_kv_heads + kvh) * kHeadDim), 0, span_bytes, 0x00020000);
    // staging map: piece p = tid + i * NT is the 16-byte piece p % 16 of row p / 16 of a 32-row block
    constexpr int NT = 64 * G;
    constexpr int PPT = 512 / NT;
    __shared__ __attribute__((aligned(16))) uint8_t lds_kv[2][2][32 * kApRowBytes];  // [buffer][K | V]
    const int tid = threadIdx.x;
    int g_off[PPT], l_off[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
        const int pce = tid + i * NT;
        g_off[i] = (pce >> 4) * row_bytes + (pce & 15) * 16;
        l_off[i] = (pce >> 4) * kApRowBytes + (pce & 15) * 16;
    }
    v4u kst[PPT], vst[PPT];
    // the whole offset goes into the per-lane operand: that is the one the range check looks at
    auto request = [&](int st) {
        const int base = st * 32 * row_bytes;
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
            kst[i] = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, base + g_off[i], 0, 0);
            vst[i] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, base + g_off[i], 0, 0);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PPT; ++i) {
            *(v4u*)(&lds_kv[buf][0][l_off[i]]) = kst[i];
            *(v4u*)(&lds_kv[buf][1][l_off[i]]) = vst[i];
        }
    };
    const int k_lds_off = c * kApRowBytes + g4 * 16;        // K operand: row c of a 16-row block, piece g4 of a 64-byte step
    const int v_lds_off = 4 * g4 * kApRowBytes + c * 16;    // V: rows 4 g4 + jj (and 16 + 4 g4 + jj), piece c

    v4f o_acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) o_acc[t] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    // softmax in base 2: exp(x * scale - m) = exp2(x * c2 - m2) with c2 = scale * log2(e); the running
    // maximum m_run is kept in raw score units (the scale is positive, so maxima commute with it)
    float m_run = -INFINITY, l_run = 0.0f;
    const float c2 = 0.08838834764831845f * 1.4426950408889634f;  // 128^-0.5 * log2(e)

    auto step = [&](int st) {
        const uint8_t* kl = &lds_kv[st & 1][0][k_lds_off];
        const uint8_t* vl = &lds_kv[st & 1][1][v_lds_off];
        v4u kb[2][4], vb[8];
#pragma unroll
        for (int bi = 0; bi < 2; ++bi)
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) kb[bi][kk] = *(const v4u*)(kl + bi * 16 * kApRowBytes + kk * 64);
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) vb[jj] = *(const v4u*)(vl + ((jj & 3) + (jj >> 2) * 16) * kApRowBytes);
        float sc[8];
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
            v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, kb[bi][kk]), qa[kk], acc, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) sc[bi * 4 + j] = acc[j];
        }
        // only the steps that reach beyond the block's first token need the causal mask (uniform test)
        if (st * 32 + 31 > start + t0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int pos = st * 32 + (i >> 2) * 16 + 4 * g4 + (i & 3);
                sc[i] = pos <= pq ? sc[i] : -INFINITY;
            }
        }
        float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
        mx = fmaxf(mx, xor_lane_f32(mx, lane, 16));
        mx = fmaxf(mx, xor_lane_f32(mx, lane, 32));
        const float m_new = fmaxf(m_run, mx);  // finite from the first step on: position 0 is visible to every token
        const float m2 = m_new * c2;
        float p[8], psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], c2, -m2));
            psum += p[i];
        }
        // the accumulated outputs are rescaled only when some token's maximum has moved (uniform test):
        // after the first few steps it rarely does
        if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
            const float alpha = __builtin_amdgcn_exp2f(__builtin_fmaf(m_run, c2, -m2));
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < 8; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j) o_acc[t][j] *= alpha;
            m_run = m_new;
        }
        l_run += psum;
        v4u pw;
        pw.x = pack_bf16x2(p[0], p[1]);
        pw.y = pack_bf16x2(p[2], p[3]);
        pw.z = pack_bf16x2(p[4], p[5]);
        pw.w = pack_bf16x2(p[6], p[7]);
        const v8bf pb = __builtin_bit_cast(v8bf, pw);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;  // both high halves / both low halves
            v4u va;
            va.x = __builtin_amdgcn_perm(vb[1][t >> 1], vb[0][t >> 1], sel);
            va.y = __builtin_amdgcn_perm(vb[3][t >> 1], vb[2][t >> 1], sel);
            va.z = __builtin_amdgcn_perm(vb[5][t >> 1], vb[4][t >> 1], sel);
            va.w = __builtin_amdgcn_perm(vb[7][t >> 1], vb[6][t >> 1], sel);
            o_acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, va), pb, o_acc[t], 0, 0, 0);
        }
    };

    request(0);
    stage(0);
    request(1);
    lds_barrier();
    for (int st = 0; st < steps; ++st) {
        step(st);
        stage((st + 1) & 1);  // rows of step st + 1, requested a step ago, into the buffer that step st - 1 used
        request(st + 2);
        lds_barrier();
    }

    float l_tot = l_run + xor_lane_f32(l_run, lane, 16);
    l_tot += xor_lane_f32(l_tot, lane, 32);
    const float inv = 1.0f / l_tot;
    if (t0 + c < T) {
        uint16_t* orow = out + ((size_t)b * T + t0 + c) * n_heads * kHeadDim + (size_t)head * kHeadDim + 32 * g4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v4u w;
            w.x = pack_bf16x2(o_acc[0][j] * inv, o_acc[1][j] * inv);
            w.y = pack_bf16x2(o_acc[2][j] * inv, o_acc[3][j] * inv);
            w.z = pack_bf16x2(o_acc[4][j] * inv, o_acc[5][j] * inv);
            w.w = pack_bf16x2(o_acc[6][j] * inv, o_acc[7][j] * inv);
            *(v4u*)(orow + 8 * j) = w;
        }
    }
}


// ---------------------------------------------------------------------------
// Decode step (one new token per sequence) with the same matrix-pipe scheme
// ---------------------------------------------------------------------------
// One workgroup per (kv head, sequence, split of the cached positions), as attn_decode_kernel; the
// difference is what happens between the rope and the records: every wave takes 32 positions of
// the slice at a time and does scores, softmax and P.V for the G query heads (columns c < G of the
// 16-column tiles) entirely in registers; the waves' (maximum, sum, outputs) are combined through
// LDS once.  No score buffer, no barrier between scores, softmax and P.V.
constexpr int kDfRecUnits = kHeadDim + 2;  // record of one (sequence, kv head, split, head): 128 outputs, maximum, sum,
                                            // each an 8-byte unit (value, tag of the call that wrote it)
constexpr int kDfSpinLimit = 1 << 16;       // polls of the merging workgroup before it gives up (see the merge below)
constexpr int kDfMaxSplits = 16;
constexpr int kDfMaxWaves = 8;

// ROWS: the rotation's cos / sin values of every sequence's position come as a ready row
// (rope_rows[b] = cos[64] | sin[64], written once per step by decode_step_begin_kernel) instead of
// from the tables at an index that has to be loaded first: one memory round trip less in front of
// the rope.
template <int G, bool ROWS>
__global__ __launch_bounds__(kDfMaxWaves * 64) void attn_decode_flash_kernel(
    // parameter order: what the loads at the kernel's entry need comes first, in the leading dwords
    // that arrive in registers at wave start (kernel-argument preload).  `epochs` is the epoch array
    // inside the workspace (any readable address with one split); `shape` = n_heads | n_kv_heads << 8 |
    // splits << 16 | waves << 24 repeats the launch geometry, which is not among those dwords
    const uint16_t* __restrict__ qkv, uint16_t* __restrict__ cache_k, uint16_t* __restrict__ cache_v,
    const int64_t* __restrict__ positions, const float* __restrict__ rope_rows, int* epochs, int S, int shape,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, uint16_t* __restrict__ out, float* workspace,
    int* err_word, int spin_limit) {
    const int n_heads = shape & 0xff, n_kv_heads = (shape >> 8) & 0xff;
    __shared__ __attribute__((aligned(16))) uint16_t qb[G][kHeadDim];  // rotated q as bf16
    __shared__ __attribute__((aligned(16))) uint16_t knew[kHeadDim];   // rotated k of the new token
    __shared__ __attribute__((aligned(16))) uint16_t vnew[kHeadDim];
    __shared__ __attribute__((aligned(16))) float part_o[kDfMaxWaves][G][kHeadDim];
    __shared__ float part_m[kDfMaxWaves][G], part_l[kDfMaxWaves][G];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = (shape >> 24) & 0xff;
    const int nthreads = nwaves * 64;
    const int kvh = blockIdx.x, b = blockIdx.y, sp = blockIdx.z;
    const int nsplit = (shape >> 16) & 0xff;
    // two scalar requests from preloaded pointers, under way before anything else: the position, and
    // the tag of this call's records -- one more than the epoch the last merge of this (sequence, kv
    // head) left behind (with one split the value is unused)
    const int64_t p_raw = positions[b];
    const int epoch = epochs[nsplit > 1 ? b * n_kv_heads + kvh : 0];
    const int c = lane & 15, g4 = lane >> 4;
    const int row_elems = (n_heads + 2 * n_kv_heads) * kHeadDim;
    const uint16_t* row = qkv + (size_t)b * row_elems;
    const size_t cache_row = (size_t)n_kv_heads * kHeadDim;
    uint16_t* ck = cache_k + ((size_t)b * S * n_kv_heads + kvh) * kHeadDim;
    uint16_t* cv = cache_v + ((size_t)b * S * n_kv_heads + kvh) * kHeadDim;
    const int row_bytes = n_kv_heads * kHeadDim * 2;
    const int cache_bytes = (S - 1) * row_bytes + kHeadDim * 2;
    const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)ck, 0, cache_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)cv, 0, cache_bytes, 0x00020000);
    // The cache rows are dealt to the splits in blocks of 32: split sp owns blocks sp, sp + nsplit,
    // sp + 2 nsplit, ... and within the split wave w takes the blocks sp + nsplit * (w + nwaves * round).
    // Whatever the current position is, the visible rows are then spread evenly over all splits
    // (contiguous slices of the cache capacity leave most splits idle while the position is far
    // below the capacity), and the blocks of the first round can still be requested before the
    // position is known.
    const int blk0 = sp + nsplit * wave;
    const int blk_stride = nsplit * nwaves;

    // Everything that depends on nothing is requested first: the token's q / k / v, the position,
    // and the wave's first block of K and V rows (a block beyond the end of the cache lies beyond
    // the descriptor: its requests cost no memory access and read as zero).
    constexpr int kItems = (G + 2) * (kHeadDim / 2);
    constexpr int kIters = (kItems + 255) / 256;
    uint32_t praw[kIters];
    float rcs[kIters], rsn[kIters];
#pragma unroll
    for (int u = 0; u < kIters; ++u) {
        const int it = tid + u * nthreads;
        const int hh = it / (kHeadDim / 2);
        const int i = it - hh * (kHeadDim / 2);
        const int src = hh < G ? (kvh * G + hh) * kHeadDim : (hh == G ? (n_heads + kvh) : (n_heads + n_kv_heads + kvh)) * kHeadDim;
        praw[u] = *(const uint32_t*)(row + (it < kItems ? src + 2 * i : 0));
        if (ROWS) {
            rcs[u] = rope_rows[(size_t)b * kHeadDim + i];
            rsn[u] = rope_rows[(size_t)b * kHeadDim + kHeadDim / 2 + i];
        }
    }
    v4u kb[2][4], vb[8];
    auto load_rows = [&](int blk) {  // cache rows 32 blk .. 32 blk + 31
        const int base = blk * 32 * row_bytes;
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
            const int off = base + (bi * 16 + c) * row_bytes + g4 * 16;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) kb[bi][kk] = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, off + kk * 64, 0, 0);
        }
#pragma unroll
        for (int jj = 0; jj < 8; ++jj)
            vb[jj] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, base + ((jj & 3) + (jj >> 2) * 16 + 4 * g4) * row_bytes + c * 16, 0, 0);
    };
    load_rows(blk0);
    const int p = __builtin_amdgcn_readfirstlane(p_raw < 0 ? 0 : (p_raw >= (int64_t)S ? S - 1 : (int)p_raw));  // clamped into the cache
    const int pblk = p >> 5;                        // the block of the new token's row
    const bool owns_new = pblk % nsplit == sp;
    const int nact = pblk + 1 < nsplit ? pblk + 1 : nsplit;  // splits that own a block with visible rows
    const bool active = sp < nact;
    // The workgroup of the last active split merges the splits' records: workgroups start in the
    // order of their index, so when it runs every other active split of this (sequence, kv head)
    // has started and will deliver its record; and having a slice of its own to work through, it
    // begins to poll about when the others finish (the last split of the grid, idle while the
    // position is below its slice, polled from the start and its traffic slowed the others down).
    const bool merger = nact > 1 && sp == nact - 1;

    // rope on adjacent pairs, fp32, rounded to bf16: q into LDS; the split that holds position p also
    // rotates k, keeps k and v of the new token in LDS and writes them to the cache
#pragma unroll
    for (int u = 0; u < kIters; ++u) {
        const int it = tid + u * nthreads;
        const int hh = it / (kHeadDim / 2);
        const int i = it - hh * (kHeadDim / 2);
        if (it < kItems && active) {
            if (hh <= G) {
                if (hh < G || owns_new) {
                    const float a = bf16f(praw[u] & 0xffffu), cc = bf16f(praw[u] >> 16);
                    const float cs = ROWS ? rcs[u] : cos_t[(size_t)p * (kHeadDim / 2) + i];
                    const float sn = ROWS ? rsn[u] : sin_t[(size_t)p * (kHeadDim / 2) + i];
                    const uint32_t rot = (uint32_t)to_bf16(a * cs - cc * sn) | ((uint32_t)to_bf16(a * sn + cc * cs) << 16);
                    if (hh < G) {
                        *(uint32_t*)(&qb[hh][2 * i]) = rot;
                    } else {
                        *(uint32_t*)(&knew[2 * i]) = rot;
                        *(uint32_t*)(ck + (size_t)p * cache_row + 2 * i) = rot;
                    }
                }
            } else if (owns_new) {
                *(uint32_t*)(&vnew[2 * i]) = praw[u];
                *(uint32_t*)(cv + (size_t)p * cache_row + 2 * i) = praw[u];
            }
        }
    }
    __syncthreads();
    if (!active) return;  // after the barrier: a branch on the position in front of the loads above would delay them

    // q^T as the B operand: column c = head c (zero beyond G)
    v8bf qa[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        uint4 t = make_uint4(0, 0, 0, 0);
        if (c < G) t = *(const uint4*)(&qb[c][kk * 32 + g4 * 8]);
        qa[kk] = __builtin_bit_cast(v8bf, t);
    }
    v4f o_acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) o_acc[t] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY, l_run = 0.0f;
    const float scale = 0.08838834764831845f;           // 128^-0.5
    const float c2 = scale * 1.4426950408889634f;        // * log2(e): the softmax runs in base 2
    for (int blk = blk0; blk <= pblk; blk += blk_stride) {
        if (blk != blk0) load_rows(blk);
        // the new token's own row is not in the cache yet for this kernel's loads: it comes from LDS
        if (blk == pblk) {
#pragma unroll
            for (int bi = 0; bi < 2; ++bi)
                if (blk * 32 + bi * 16 + c == p) {
#pragma unroll
                    for (int kk = 0; kk < 4; ++kk) kb[bi][kk] = *(const v4u*)(&knew[kk * 32 + g4 * 8]);
                }
            // V rows behind the position are cleared: their probability is zero, but whatever the
            // cache holds there (it may never have been written) must not reach the product as 0 x NaN
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                const int r = blk * 32 + (jj & 3) + (jj >> 2) * 16 + 4 * g4;
                if (r == p) vb[jj] = *(const v4u*)(&vnew[c * 8]);
                if (r > p) vb[jj] = v4u{0u, 0u, 0u, 0u};
            }
        }
        float sc[8];
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
            v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, kb[bi][kk]), qa[kk], acc, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int pos = blk * 32 + bi * 16 + 4 * g4 + j;
                sc[bi * 4 + j] = pos <= p ? acc[j] : -INFINITY;
            }
        }
        float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
        mx = fmaxf(mx, xor_lane_f32(mx, lane, 16));
        mx = fmaxf(mx, xor_lane_f32(mx, lane, 32));
        const float m_new = fmaxf(m_run, mx);  // finite: the block's first row is visible (32 blk <= p)
        const float m2 = m_new * c2;
        float pr[8], psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pr[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], c2, -m2));
            psum += pr[i];
        }
        if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
            const float alpha = __builtin_amdgcn_exp2f(__builtin_fmaf(m_run, c2, -m2));
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < 8; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j) o_acc[t][j] *= alpha;
            m_run = m_new;
        }
        l_run += psum;
        v4u pw;
        pw.x = pack_bf16x2(pr[0], pr[1]);
        pw.y = pack_bf16x2(pr[2], pr[3]);
        pw.z = pack_bf16x2(pr[4], pr[5]);
        pw.w = pack_bf16x2(pr[6], pr[7]);
        const v8bf pb = __builtin_bit_cast(v8bf, pw);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
            v4u va;
            va.x = __builtin_amdgcn_perm(vb[1][t >> 1], vb[0][t >> 1], sel);
            va.y = __builtin_amdgcn_perm(vb[3][t >> 1], vb[2][t >> 1], sel);
            va.z = __builtin_amdgcn_perm(vb[5][t >> 1], vb[4][t >> 1], sel);
            va.w = __builtin_amdgcn_perm(vb[7][t >> 1], vb[6][t >> 1], sel);
            o_acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, va), pb, o_acc[t], 0, 0, 0);
        }
    }
    // the wave's result for head c (lanes c < G): maximum, sum over its positions, 32 outputs per lane
    float l_tot = l_run + xor_lane_f32(l_run, lane, 16);
    l_tot += xor_lane_f32(l_tot, lane, 32);
    if (c < G) {
        if (g4 == 0) {
            part_m[wave][c] = m_run;  // -inf, and a sum of 0, for a wave without visible positions
            part_l[wave][c] = l_tot;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < 8; ++t) part_o[wave][c][32 * g4 + 8 * j + t] = o_acc[t][j];
    }
    __syncthreads();

    uint16_t* orow = out + (size_t)b * n_heads * kHeadDim + (size_t)(kvh * G) * kHeadDim;
    // Records are 8-byte units (value, tag) written with single device-coherent (write-through)
    // stores: a reader that finds this call's tag in a unit has that unit's value, so nobody waits
    // for the stores to be acknowledged and no arrival counter is needed -- the merging workgroup
    // polls the units it needs until they carry the tag.  Against "stores, barrier until they are
    // acknowledged, device-scope counter, loads" this saves one of the three trips across the chip.
    unsigned long long* rec = (unsigned long long*)workspace + ((size_t)(b * n_kv_heads + kvh) * nsplit) * G * kDfRecUnits;
    const unsigned long long tag = (unsigned long long)(unsigned)(epoch + 1) << 32;
    for (int hh = wave; hh < G; hh += nwaves) {
        float mx = -INFINITY;
        for (int k = 0; k < nwaves; ++k) mx = fmaxf(mx, part_m[k][hh]);
        float o0 = 0.0f, o1 = 0.0f, l = 0.0f;
        for (int k = 0; k < nwaves; ++k) {
            const float lk = part_l[k][hh];
            if (lk > 0.0f) {
                const float w = __builtin_amdgcn_exp2f((part_m[k][hh] - mx) * c2);
                l += lk * w;
                o0 += w * part_o[k][hh][2 * lane];
                o1 += w * part_o[k][hh][2 * lane + 1];
            }
        }
        if (nact == 1) {
            const float is = 1.0f / l;
            *(uint32_t*)(orow + hh * kHeadDim + 2 * lane) = (uint32_t)to_bf16(o0 * is) | ((uint32_t)to_bf16(o1 * is) << 16);
        } else {
            unsigned long long* r = rec + ((size_t)sp * G + hh) * kDfRecUnits;
            __hip_atomic_store(r + 2 * lane, tag | __float_as_uint(o0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(r + 2 * lane + 1, tag | __float_as_uint(o1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0) {
                __hip_atomic_store(r + kHeadDim, tag | __float_as_uint(mx * scale), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // in units of the scaled scores
                __hip_atomic_store(r + kHeadDim + 1, tag | __float_as_uint(l), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    if (!merger) return;

    // The merge, eight splits at a time: all units of a batch are requested together and requested
    // again while one of them still carries an older tag.  Every split polled was dispatched before
    // this workgroup and writes its record without waiting for anything, so the poll is expected to
    // end after a few rounds; that order of dispatch is observed behaviour, not something the
    // hardware promises, and a workspace that was not zero before its first use breaks the tags.  The
    // poll is therefore bounded, and a poll that runs out is not papered over: the head's output row
    // becomes NaN and the workspace's error word is set (it stays set; the host reads it, see
    // bitnet_attn_decode_error_index).
    constexpr int kBatch = 8;
    for (int hh = wave; hh < G; hh += nwaves) {
        float mx = -INFINITY, l = 0.0f, o0 = 0.0f, o1 = 0.0f;
        bool gave_up = false;
        for (int k0 = 0; k0 < nact; k0 += kBatch) {
            unsigned long long um[kBatch], ul[kBatch], u0[kBatch], u1[kBatch];
#pragma unroll
            for (int k = 0; k < kBatch; ++k) um[k] = ul[k] = u0[k] = u1[k] = 0ull;
            bool complete = false;
            for (int spin = 0; spin < spin_limit; ++spin) {
                bool ok = true;
#pragma unroll
                for (int k = 0; k < kBatch; ++k) {
                    const unsigned long long* r = rec + ((size_t)((k0 + k) < nact ? (k0 + k) : k0) * G + hh) * kDfRecUnits;
                    um[k] = __hip_atomic_load(r + kHeadDim, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ul[k] = __hip_atomic_load(r + kHeadDim + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    u0[k] = __hip_atomic_load(r + 2 * lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    u1[k] = __hip_atomic_load(r + 2 * lane + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int k = 0; k < kBatch; ++k)
                    ok = ok && ((um[k] & ul[k] & u0[k] & u1[k]) >> 32) == (tag >> 32) && ((um[k] | ul[k] | u0[k] | u1[k]) >> 32) == (tag >> 32);
                if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
                    complete = true;
                    break;
                }
            }
            gave_up = gave_up || !complete;
            float bm = mx;
#pragma unroll
            for (int k = 0; k < kBatch; ++k)
                if (k0 + k < nact) bm = fmaxf(bm, __uint_as_float((unsigned)um[k]));
            const float wold = l > 0.0f ? __expf(mx - bm) : 0.0f;
            l *= wold;
            o0 *= wold;
            o1 *= wold;
            mx = bm;
#pragma unroll
            for (int k = 0; k < kBatch; ++k) {
                const float lk = __uint_as_float((unsigned)ul[k]);
                if (k0 + k < nact && lk > 0.0f) {
                    const float w = __expf(__uint_as_float((unsigned)um[k]) - mx);
                    l += lk * w;
                    o0 += w * __uint_as_float((unsigned)u0[k]);
                    o1 += w * __uint_as_float((unsigned)u1[k]);
                }
            }
        }
        const float is = gave_up ? __builtin_nanf("") : 1.0f / l;
        *(uint32_t*)(orow + hh * kHeadDim + 2 * lane) = (uint32_t)to_bf16(o0 * is) | ((uint32_t)to_bf16(o1 * is) << 16);
        if (gave_up && lane == 0) __hip_atomic_store(err_word, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();  // every wave has read its records
    if (tid == 0) epochs[b * n_kv_heads + kvh] = epoch + 1;
}

}  // namespace

// Launcher used by bitnet_attn_decode / bitnet_attn_decode_rows (decoder_ops.hip), which have validated
// the arguments.  rope_rows may be null: the rotation values then come from the tables.
int bitnet_attn_decode_flash_launch(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v, const int64_t* positions,
                                    const float* cos_table, const float* sin_table, const float* rope_rows, uint16_t* out,
                                    float* workspace, int* counters, int n_splits, int threads, int B, int S,
                                    int n_heads, int n_kv_heads, int spin_limit, hipStream_t stream) {
    (void)counters;  // the arrival counters belong to the other kernel
    const int g = n_heads / n_kv_heads;
    if (n_heads > 255 || n_splits > 255 || threads > 64 * 255) return 1;  // packed into one kernel argument
    const dim3 grid(n_kv_heads, B, n_splits), block(threads, 1, 1);
    // the epoch array follows the splits' records in the workspace
    int* epochs = n_splits > 1 ? (int*)(workspace + (size_t)B * n_kv_heads * n_splits * g * kDfRecUnits * 2) : (int*)positions;
    // the error word follows the epochs (with one split nothing is merged and nothing can fail)
    int* err_word = n_splits > 1 ? epochs + (size_t)B * n_kv_heads : nullptr;
    if (spin_limit < 0) spin_limit = kDfSpinLimit;
#define BITNET_DF_LAUNCH(GG, RR)                                                                                           \
    hipLaunchKernelGGL((attn_decode_flash_kernel<GG, RR>), grid, block, 0, stream, qkv, cache_k, cache_v, positions,       \
                       rope_rows, epochs, S, n_heads | (n_kv_heads << 8) | (n_splits << 16) | ((threads / 64) << 24),        \
                       cos_table, sin_table, out, workspace, err_word, spin_limit)
#define BITNET_DF_LAUNCH_G(GG)     \
    if (rope_rows)                 \
        BITNET_DF_LAUNCH(GG, true); \
    else                           \
        BITNET_DF_LAUNCH(GG, false)
    switch (g) {
        case 1: BITNET_DF_LAUNCH_G(1); break;
        case 2: BITNET_DF_LAUNCH_G(2); break;
        case 4: BITNET_DF_LAUNCH_G(4); break;
        default: BITNET_DF_LAUNCH_G(8); break;
    }
#undef BITNET_DF_LAUNCH_G
#undef BITNET_DF_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

namespace {
// Start of a decode step: the embedding row of every sequence's input token (tok_embeddings,
// gpu/model.py:272) and the cos | sin row of its position, so that the layers' attention kernels
// need not look the position up before they can rotate.  One workgroup per sequence.
__global__ __launch_bounds__(256) void decode_step_begin_kernel(
    const int64_t* __restrict__ tokens, const int64_t* __restrict__ positions, const uint16_t* __restrict__ emb,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, uint16_t* __restrict__ h_out,
    float* __restrict__ rope_rows, int V, int dim, int S) {
    const int b = blockIdx.x;
    const int64_t t_raw = tokens[b], p_raw = positions[b];
    const int64_t t = t_raw < 0 ? 0 : (t_raw >= (int64_t)V ? V - 1 : t_raw);       // clamped: nothing outside the buffers is read
    const int p = p_raw < 0 ? 0 : (p_raw >= (int64_t)S ? S - 1 : (int)p_raw);
    const uint4* src = (const uint4*)(emb + (size_t)t * dim);
    uint4* dst = (uint4*)(h_out + (size_t)b * dim);
    for (int i = threadIdx.x; i < dim / 8; i += 256) dst[i] = src[i];
    if (threadIdx.x < kHeadDim) {
        const int i = threadIdx.x & (kHeadDim / 2 - 1);
        rope_rows[(size_t)b * kHeadDim + threadIdx.x] =
            threadIdx.x < kHeadDim / 2 ? cos_t[(size_t)p * (kHeadDim / 2) + i] : sin_t[(size_t)p * (kHeadDim / 2) + i];
    }
}
}  // namespace

extern "C" int bitnet_decode_step_begin(const int64_t* tokens, const int64_t* positions, const uint16_t* emb,
                                        const float* cos_table, const float* sin_table, uint16_t* h_out, float* rope_rows,
                                        int B, int V, int dim, int S, int head_dim, void* stream) {
    if (B < 1 || V < 1 || dim < 8 || dim % 8 || S < 1 || head_dim != kHeadDim) return 1;
    if (!tokens || !positions || !emb || !cos_table || !sin_table || !h_out || !rope_rows) return 2;
    if ((((uintptr_t)emb) | ((uintptr_t)h_out)) & 15u) return 1;
    hipLaunchKernelGGL(decode_step_begin_kernel, dim3(B, 1, 1), dim3(256, 1, 1), 0, (hipStream_t)stream, tokens, positions, emb,
                       cos_table, sin_table, h_out, rope_rows, V, dim, S);
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

extern "C" int bitnet_rope_cache_tokens(const uint16_t* qkv, uint16_t* cache_k, uint16_t* cache_v, const int64_t* positions,
                                        const float* cos_table, const float* sin_table, uint16_t* q_out, int B, int T,
                                        int S, int n_heads, int n_kv_heads, int head_dim, void* stream) {
    if (B < 1 || T < 1 || S < 1 || n_heads < 1 || n_kv_heads < 1 || head_dim != kHeadDim) return 1;
    if ((long long)B * T >= (1ll << 31)) return 1;
    if (!qkv || !cache_k || !cache_v || !positions || !cos_table || !sin_table || !q_out) return 2;
    hipLaunchKernelGGL(rope_cache_tokens_kernel, dim3(B * T, 1, 1), dim3(kRopeThreads, 1, 1), 0, (hipStream_t)stream, qkv,
                       cache_k, cache_v, positions, cos_table, sin_table, q_out, T, S, n_heads, n_kv_heads);
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

extern "C" int bitnet_attn_prefill(const uint16_t* q, const uint16_t* cache_k, const uint16_t* cache_v, uint16_t* out, int B,
                                   int T, int S, int start, int n_heads, int n_kv_heads, int head_dim, void* stream) {
    if (B < 1 || T < 1 || S < 1 || start < 0 || n_heads < 1 || n_kv_heads < 1 || head_dim != kHeadDim) return 1;
    if ((long long)start + T > S || n_heads % n_kv_heads) return 1;
    const int g = n_heads / n_kv_heads;
    if (g != 1 && g != 2 && g != 4 && g != 8) return 1;
    if ((size_t)(S + 64) * n_kv_heads * kHeadDim * 2 >= ((size_t)1 << 31)) return 1;  // 32-bit byte offsets into one sequence's cache
    if (B > 65535 || n_kv_heads > 65535) return 1;
    if (!q || !cache_k || !cache_v || !out) return 2;
    if ((((uintptr_t)q) | ((uintptr_t)cache_k) | ((uintptr_t)cache_v) | ((uintptr_t)out)) & 15u) return 1;
    const dim3 grid((T + 15) / 16, n_kv_heads, B), block(64 * g, 1, 1);
    switch (g) {
        case 1: hipLaunchKernelGGL(attn_prefill_kernel<1>, grid, block, 0, (hipStream_t)stream, q, cache_k, cache_v, out, T, S, start, n_heads, n_kv_heads); break;
        case 2: hipLaunchKernelGGL(attn_prefill_kernel<2>, grid, block, 0, (hipStream_t)stream, q, cache_k, cache_v, out, T, S, start, n_heads, n_kv_heads); break;
        case 4: hipLaunchKernelGGL(attn_prefill_kernel<4>, grid, block, 0, (hipStream_t)stream, q, cache_k, cache_v, out, T, S, start, n_heads, n_kv_heads); break;
        default: hipLaunchKernelGGL(attn_prefill_kernel<8>, grid, block, 0, (hipStream_t)stream, q, cache_k, cache_v, out, T, S, start, n_heads, n_kv_heads); break;
    }
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

