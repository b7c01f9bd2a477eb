// Ternary BitLinear for MI355X (gfx950 / CDNA4): hand-written HIP kernels and
// the C ABI declared in include/bitlinear_hip.h.
//
// Data layout consumed in place (what gpu/pack_weight.py:76-98 of the reference
// writes): 16 weight rows x 32 k form a 128-byte tile of 32 little-endian
// int32 words; tiles of one 16-row block are contiguous over k (K words per
// block).  Word t of a tile holds 16 consecutive k of row (t/16)*8 + t%8,
// k-half (t/8)%2; element e of the word sits at bit (e%4)*8 + (e/4)*2, so
// (word >> 2i) & 0x03030303 is elements 4i..4i+3 as four bytes.  Stored code
// = w + 2.
//
// Decode GEMV (M <= 16 per workgroup): one workgroup owns one 16-row block and
// one group of 16 tokens.  Its waves split K in steps of 64.  For one step a
// lane loads ONE packed word (row lane%16, 16 k chosen by lane/16) -- the 64
// lanes of a wave cover 256 contiguous bytes -- expands it to 16 int8 with 3
// shifts + 4 ands, and that is exactly the A operand of
// v_mfma_i32_16x16x64_i8.  The B operand is 16 int8 of token lane%16 for the
// same 16 k.  The +2 bias of the stored codes is removed exactly by a second
// MFMA whose A operand is the constant -2: sum((q-2)*a) = sum(q*a) + sum(-2*a).
// Partial 16x16 tiles of the waves are summed through LDS and the reference's
// epilogue (gpu/bitnet_kernels/bitnet_kernels.h:79-82) is applied.

#include <hip/hip_runtime.h>
#include <atomic>
#include <mutex>
#include <string>
#include <type_traits>
#include <stdint.h>
#include <stdio.h>

#include "bitlinear_hip.h"
#include "bitlinear_probes.h"
#include "host_util.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// Scratch of bitlinear_forward_bf16_static: the quantized activations and their scales travel from
// the quantizer kernel to the product kernel through this array instead of through workspaces that
// a caller allocates.  Every GPU the library runs on holds its own copy, at its own address, until
// the process ends.  Layout: bf16 scales of up to kStaticMaxTokens tokens, then the int8 rows.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
constexpr int kStaticMaxTokens = 16384;
constexpr size_t kStaticScaleBytes = (size_t)kStaticMaxTokens * 2;
constexpr size_t kStaticMaxElems = kStaticScratchBytes - kStaticScaleBytes;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxSeg = 8;
constexpr int kMaxWaves = 16;

struct ScaleMap {
    int nseg;
    int ends[kMaxSeg];
};

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// fp32 -> bf16, round to nearest even: gfx950 has the conversion in hardware
// (two values per instruction)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) { return (uint16_t)(f32x2_to_bf16x2(f, 0.0f) & 0xffffu); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits
// for every outstanding global load of the wave, which would serialise the
// weight stream behind the barrier; here the weight words stay in flight.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Wave-wide reductions with DPP lane permutes (no LDS): two quad permutes and
// two mirrors leave every lane of a 16-lane row with the row's result; the
// four row results are then combined through scalar registers.
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, (uint32_t)dpp_move<0xB1>((int)v));   // quad_perm [1,0,3,2]
    v = max(v, (uint32_t)dpp_move<0x4E>((int)v));   // quad_perm [2,3,0,1]
    v = max(v, (uint32_t)dpp_move<0x141>((int)v));  // row_half_mirror
    v = max(v, (uint32_t)dpp_move<0x140>((int)v));  // row_mirror
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(a, b), max(c, d));
}
__device__ __forceinline__ int wave_sum_i32(int v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    v += dpp_move<0x140>(v);
    return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
           __builtin_amdgcn_readlane(v, 48);
}

// Scale slot of output row n: ends[] ascend, so it is the number of segment
// boundaries at or below n.
__device__ __forceinline__ int scale_slot(const ScaleMap& smap, int n) {
    int slot = 0;
#pragma unroll
    for (int j = 0; j < kMaxSeg - 1; ++j) slot += (j < smap.nseg - 1 && n >= smap.ends[j]) ? 1 : 0;
    return slot;
}

// The same for a wave-uniform n: a short scalar loop instead of the unrolled select chain.
__device__ __forceinline__ int scale_slot_uniform(const ScaleMap& smap, int n) {
    int slot = 0;
    while (slot < smap.nseg - 1 && n >= smap.ends[slot]) ++slot;
    return slot;
}

// Up to this many tokens a product goes through the kernels that keep the token rows in LDS or registers per
// wave (the staged and the streaming kernel); beyond, through the kernels that split the tokens over MFMA columns
constexpr int kDecodeMaxTokens = 4;

// ---------------------------------------------------------------------------
// Streaming kernel (M <= 4 tokens): waves that own whole 16-row blocks and never meet
// ---------------------------------------------------------------------------
// For matrices (or groups of matrices) large enough to be bandwidth-bound.  A work item is one
// 16-row block of one problem: 4 * K contiguous bytes.  A workgroup of four waves belongs to one
// problem; each of its waves takes a run of consecutive row blocks and walks them with ONE software
// pipeline that does not stop at item boundaries: a ring of D 16-byte weight loads per lane (D KB per
// wave, the lanes of one load covering 1 KB = 16 rows x 256 k), each slot re-requested for the next
// round of k-steps -- or for the first round of the wave's next row block -- right after the MFMAs
// that consumed it.  Operand scheme: a lane loads 16 bytes = four packed words = rows 4q..4q+3 of one
// 16-k chunk (the wave's 64 lanes cover 1 KB contiguous = 16 rows x 256 k).  Word i of every lane is the A
// operand of MFMA i (i = 0..3), which therefore sees row 4q+i at A-row index p = 4*sigma + q with k-chunk
// 4g + sigma (g = lane / 16).  The B operand puts token m's chunk 4g + sigma' at column p' = 4*sigma' + m.
// Entry (p, p') of the 16x16 result is a true partial dot product exactly when sigma == sigma': those
// entries sit in lanes 20*G + m (G = sigma), register q, and the four G parts are added at the end; the
// off-diagonal entries are never read.  The problem's int8
// activation rows are copied into LDS once per workgroup (requested before the weights, so that they
// are not queued behind them: loads return in the order of their requests); after that single barrier
// no wave waits for another, and the only other LDS traffic is each wave's own 1 KB transposition of
// its diagonal results.  What stands between the arrival of the first weight words and their use is
// time in which the wave's ring is not refilled, so the copy is all there is in front of the loop
// (only the 16-byte pieces that exist are requested; measured per launch of 30 problems against a
// prologue that also summed the rows: 3840 x 2560 14.9 -> 14.3 us, 2560 x 2560 11.3 -> 10.8): sum(a)
// per token, which removes the +2 of the stored codes, is taken by every wave from the rows in LDS
// behind the products of its first row block, when the ring is full again.
// Several problems of one shape (a grouped launch) are the grid's second dimension.
constexpr int kStreamMaxProblems = 48;  // the operands of a grouped launch travel as kernel arguments
constexpr int kStreamMaxTokens = 4;
constexpr int kStreamMaxActBytes = 32768;  // M * K: at most 8 16-byte pieces per thread of the staging pass
constexpr int kStreamRowPad = 64;          // bytes between token rows in LDS beyond K: the 4 tokens of a read hit different banks
struct StreamProblem {
    const int8_t* act;     // int8 [M, K]
    const int8_t* packed;  // packed weight [N, K/4]
    uint16_t* out;         // bf16 [M, N] or nullptr
    const uint16_t* s;     // bf16 [M]
    const uint16_t* ws;    // bf16 weight scales
};
struct StreamArgs {
    int M, N, K;
    int blocks16;     // N / 16: items per problem
    int ipw;          // consecutive items per wave
    int rounds;       // rounds of D 256-k steps per item
    int steps;        // ceil(K / 256)
    int pad_;
    int32_t* acc_out;  // int32 [M, N] of problem 0, or nullptr
    ScaleMap smap;     // every boundary a multiple of 16
    StreamProblem p[kStreamMaxProblems];
};

template <int D, bool COMPUTE>
__global__ __launch_bounds__(256) void gemv_i2_stream_kernel(const StreamArgs a, uint32_t* __restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) int8_t lds_act[];  // [M][K + pad] + tail
    __shared__ __attribute__((aligned(16))) int red[4][256];         // per wave: [G][token][row]
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int pid = blockIdx.y;
    int rb = (blockIdx.x * 4 + wave) * a.ipw;
    const int rb_end = (rb + a.ipw) < a.blocks16 ? (rb + a.ipw) : a.blocks16;
    const bool have_items = rb < rb_end;  // uniform over the wave
    const int g = lane >> 4;
    const int sg = (lane >> 2) & 3;
    const int q = lane & 3;
    const int chunk = 4 * g + sg;  // 16-k chunk inside a 256-k step
    // 16-byte group of (row quad q, chunk) inside the step's 1 KB: tile chunk / 2, k-half chunk & 1
    const int w_voff = ((chunk >> 1) * 8 + (q >> 1) * 4 + (chunk & 1) * 2 + (q & 1)) * 16;
    const int tokB = q < a.M ? q : a.M - 1;  // columns of tokens >= M are never read
    const int kp = a.K + kStreamRowPad;
    const int wbytes = a.K * 4;  // one 16-row block
    const StreamProblem prob = a.p[pid];

    // Descriptors span exactly one row block: a k-step past the end of K is out of range and reads as
    // zero weights (which contribute nothing, whatever the B operand holds), and the requests of a
    // wave that has run out of row blocks go to an empty descriptor: no memory access.
    auto w_desc = [&](int rb_, bool valid) {
        return __builtin_amdgcn_make_buffer_rsrc((void*)(prob.packed + (size_t)rb_ * (size_t)wbytes), 0, valid ? wbytes : 0,
                                                 0x00020000);
    };

    // the activation block first (it comes from cache and must not queue behind the weights) ...
    constexpr int kPieces = kStreamMaxActBytes / 16 / 256;  // 16-byte pieces per thread
    v4i piece[kPieces];
    int prow[kPieces], pdst[kPieces];
    uint16_t e_sb = 0, e_wb = 0;
    if (COMPUTE) {
        const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)prob.act, 0, a.M * a.K, 0x00020000);
        const int kp16 = a.K >> 4;
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int pc = tid + i * 256;
            const int row = (pc >= kp16 ? 1 : 0) + (pc >= 2 * kp16 ? 1 : 0) + (pc >= 3 * kp16 ? 1 : 0);
            prow[i] = pc < a.M * kp16 ? row : -1;
            pdst[i] = row * kp + (pc - row * kp16) * 16;
            // a wave whose 64 pieces of this pass all lie past the block requests nothing (wave-uniform)
            if ((wave * 64 + i * 256) < a.M * kp16)
                piece[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, pc * 16, 0, 0));  // past the end: zeros
        }
        // (unconditional: a call without output hands in addresses that exist; a load under a branch would
        // be waited for inside the branch, in front of the weight requests)
        e_sb = prob.s[tokB];
        e_wb = prob.ws[(lane & 7) < a.smap.nseg ? (lane & 7) : 0];
    }
    // ... then the first round of weight words
    v4u w[D];
    __amdgpu_buffer_rsrc_t cw = w_desc(have_items ? rb : 0, have_items);
#pragma unroll
    for (int j = 0; j < D; ++j) {
        w[j] = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(cw, w_voff, j * 1024, 2 /* nt */));
        __builtin_amdgcn_sched_barrier(0);  // requested in the order in which the slots are consumed
    }
    int rowsum2_tok = 0;  // twice the sum of the int8 row of this lane's token (lane & 3)
    float e_sf = 1.0f;    // that token's activation scale
    uint32_t e_wsv = 0;   // lane j < nseg: weight scale of slot j, as fp32 bits
    if (COMPUTE) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i)
            if (prow[i] >= 0) *(v4i*)(lds_act + pdst[i]) = piece[i];
        e_sf = bf16_to_f32(e_sb);
        e_wsv = ((uint32_t)e_wb) << 16;
        lds_barrier();  // LDS only: the weight words stay in flight
    }
    if (!have_items) return;  // behind the only barrier
    bool rowsum_due = COMPUTE;

    const int8_t* bp = lds_act + tokB * kp + chunk * 16;
    uint32_t x_acc = 0;  // load-only variant: something that depends on every byte
    for (; rb < rb_end; ++rb) {
        const bool nvalid = (rb + 1) < rb_end;
        const __amdgpu_buffer_rsrc_t nw = w_desc(nvalid ? rb + 1 : rb, nvalid);
        v4i acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0}, acc2 = {0, 0, 0, 0}, acc3 = {0, 0, 0, 0};
        for (int sub = 0; sub < a.rounds; ++sub) {
            // what the ring requests while this round is multiplied: the row block's next round, or the
            // first round of the wave's next row block
            const bool last = (sub + 1) == a.rounds;
            const __amdgpu_buffer_rsrc_t rw = last ? nw : cw;
            const int so = last ? 0 : (sub + 1) * D;
            const int st0 = sub * D;
            v4i bcur;
            if (COMPUTE) bcur = *(const v4i*)(bp + (st0 < a.steps ? st0 : a.steps - 1) * 256);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < D; ++j) {
                const uint32_t wd[4] = {w[j].x, w[j].y, w[j].z, w[j].w};
                if (COMPUTE) {
                    // the next step's B operand is read while this step is multiplied (a step past the
                    // end re-reads the last one: its weights are zero)
                    const int stn = st0 + j + 1;
                    const v4i bnext = *(const v4i*)(bp + (stn < a.steps ? stn : a.steps - 1) * 256);
                    v4i e[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        e[i].x = (int)(wd[i] & 0x03030303u);
                        e[i].y = (int)((wd[i] >> 2) & 0x03030303u);
                        e[i].z = (int)((wd[i] >> 4) & 0x03030303u);
                        e[i].w = (int)((wd[i] >> 6) & 0x03030303u);
                    }
                    w[j] = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(rw, w_voff, (so + j) * 1024, 2 /* nt */));
                    acc0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(e[0], bcur, acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(e[1], bcur, acc1, 0, 0, 0);
                    acc2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(e[2], bcur, acc2, 0, 0, 0);
                    acc3 = __builtin_amdgcn_mfma_i32_16x16x64_i8(e[3], bcur, acc3, 0, 0, 0);
                    bcur = bnext;
                } else {
                    x_acc ^= wd[0] ^ wd[1] ^ wd[2] ^ wd[3];
                    w[j] = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(rw, w_voff, (so + j) * 1024, 2 /* nt */));
                }
                __builtin_amdgcn_sched_barrier(0);  // the slot's re-request stays where it is written: right behind its use
            }
        }
        if (COMPUTE) {
            if (rowsum_due) {
                // once per wave: the sum of the lane's token's row, from the chunks the lane multiplies (chunk
                // `chunk` of every 256-k step that lies inside K), added up over the 16 lanes of the token
                rowsum_due = false;
                const int ones = 0x01010101;
                int rs = 0;
                for (int st = 0; st < a.steps; ++st) {
                    const v4i v = *(const v4i*)(bp + st * 256);
                    int d = __builtin_amdgcn_sdot4(v.x, ones, 0, false);
                    d = __builtin_amdgcn_sdot4(v.y, ones, d, false);
                    d = __builtin_amdgcn_sdot4(v.z, ones, d, false);
                    d = __builtin_amdgcn_sdot4(v.w, ones, d, false);
                    rs += (st * 256 + chunk * 16) < a.K ? d : 0;
                }
                rs += dpp_move<0x124>(rs);  // row_ror:4 and :8: the four lanes of the 16-lane row with this token
                rs += dpp_move<0x128>(rs);
                rs += __shfl_xor(rs, 16);
                rs += __shfl_xor(rs, 32);
                rowsum2_tok = 2 * rs;
            }
            // result lane 16 G + p' holds A-rows 4 G + r (r = register); the diagonal blocks (sigma' == G) sit in
            // the lanes with g == sg, token q; register r of MFMA i is weight row 4 r + i
            int* my = red[wave];
            if (sg == g) {
                int* dst = my + (g * 4 + q) * 16;
                *(v4i*)(dst + 0) = v4i{acc0.x, acc1.x, acc2.x, acc3.x};
                *(v4i*)(dst + 4) = v4i{acc0.y, acc1.y, acc2.y, acc3.y};
                *(v4i*)(dst + 8) = v4i{acc0.z, acc1.z, acc2.z, acc3.z};
                *(v4i*)(dst + 12) = v4i{acc0.w, acc1.w, acc2.w, acc3.w};
            }
            // the same wave wrote and reads: LDS operations of a wave complete in order
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int row = lane >> 2;  // token = q
            const int sum = my[(0 * 4 + q) * 16 + row] + my[(1 * 4 + q) * 16 + row] + my[(2 * 4 + q) * 16 + row] +
                            my[(3 * 4 + q) * 16 + row] - rowsum2_tok;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int n = rb * 16 + row;
            const int slot = scale_slot_uniform(a.smap, rb * 16);
            const float wsf = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)e_wsv, slot));
            if (q < a.M) {
                const size_t o = (size_t)q * a.N + n;
                if (a.acc_out && pid == 0) a.acc_out[o] = sum;
                if (prob.out) prob.out[o] = f32_to_bf16_rne((float)sum / e_sf * wsf);
            }
        }
        cw = nw;
    }
    if (!COMPUTE && x_acc == 0x9e3779b9u && sink) sink[0] = x_acc;  // keeps the loads alive; practically never taken
}

// ---------------------------------------------------------------------------
// Small-batch kernel (M <= 16 per workgroup), K split across the waves
// ---------------------------------------------------------------------------
template <int UPW>
__global__ __launch_bounds__(kMaxWaves * 64) void gemv_i2_mfma_kernel(
    const int8_t* __restrict__ act, const uint32_t* __restrict__ wq, int M, int N, int K, int nwaves,
    uint16_t* __restrict__ out, int32_t* __restrict__ acc_out, const uint16_t* __restrict__ s,
    const uint16_t* __restrict__ ws, ScaleMap smap, const uint16_t* __restrict__ residual) {
    __shared__ int red[kMaxWaves * 256];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int g = lane >> 4;  // which 16 of the step's 64 k
    const int p = lane & 15;  // weight row (A operand) / token (B operand)
    const int nb = blockIdx.x;
    const int m0 = blockIdx.y * 16;
    const int units = K >> 6;

    // word of (row p, k-chunk g) inside a 64-k step: two tiles of 32 words
    const int lane_word = (g >> 1) * 32 + (p >> 3) * 16 + (g & 1) * 8 + (p & 7);
    const uint32_t* wrow = wq + (size_t)nb * K + lane_word;
    const bool tok_ok = (m0 + p) < M;
    const int8_t* arow = act + (size_t)(tok_ok ? (m0 + p) : 0) * K + g * 16;

    v4i acc_q = {0, 0, 0, 0};
    v4i acc_b = {0, 0, 0, 0};
    const int neg2w = (int)0xFEFEFEFEu;
    const v4i neg2 = {neg2w, neg2w, neg2w, neg2w};

    // Rounds of UPW k-steps, two register sets: the loads of the round after next are issued
    // before a round is multiplied, so 1 to 2 rounds stay in flight.  Loads are unconditional
    // (indices clamped); a step past the end is multiplied by zeros.
    uint32_t w0[UPW], w1[UPW];
    v4i b0[UPW], b1[UPW];
    auto load_round = [&](uint32_t(&w)[UPW], v4i(&b)[UPW], int base) {
#pragma unroll
        for (int j = 0; j < UPW; ++j) {
            const int u = (base + j) < units ? (base + j) : (units - 1);
            w[j] = __builtin_nontemporal_load(wrow + (size_t)u * 64);
            b[j] = *(const v4i*)(arow + (size_t)u * 64);
        }
    };
    auto use_round = [&](const uint32_t(&w)[UPW], const v4i(&b)[UPW], int base) {
#pragma unroll
        for (int j = 0; j < UPW; ++j) {
            const bool live = (base + j) < units && tok_ok;
            const v4i bj = live ? b[j] : v4i{0, 0, 0, 0};
            v4i a;
            a.x = (int)(w[j] & 0x03030303u);
            a.y = (int)((w[j] >> 2) & 0x03030303u);
            a.z = (int)((w[j] >> 4) & 0x03030303u);
            a.w = (int)((w[j] >> 6) & 0x03030303u);
            acc_q = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bj, acc_q, 0, 0, 0);
            acc_b = __builtin_amdgcn_mfma_i32_16x16x64_i8(neg2, bj, acc_b, 0, 0, 0);
        }
    };
    const int stride = nwaves * UPW;
    const int base0 = wave * UPW;
    load_round(w0, b0, base0);
    if (base0 + stride < units) load_round(w1, b1, base0 + stride);

    // The thread that will finish output (row, token) fetches its two scales
    // now -- behind the first weight requests, which need nothing but
    // arguments that arrive in registers, while the scale map and these
    // pointers come through a scalar load -- as raw bits with nothing
    // depending on them until the epilogue, so their latency overlaps the
    // weight stream.  Indices are clamped so every thread may load.
    const int e_lane = threadIdx.x & 63;
    const int e_m = m0 + (e_lane & 15);
    const int e_n = nb * 16 + 4 * (e_lane >> 4) + ((threadIdx.x >> 6) & 3);
    uint16_t e_sb = 0, e_wsb = 0, e_res = 0;
    if (out) {
        e_sb = s[e_m < M ? e_m : M - 1];
        e_wsb = ws[scale_slot(smap, e_n)];
        if (residual) e_res = residual[(size_t)(e_m < M ? e_m : M - 1) * N + e_n];
    }
    for (int base = base0; base < units; base += 2 * stride) {
        use_round(w0, b0, base);
        if (base + 2 * stride < units) load_round(w0, b0, base + 2 * stride);
        if (base + stride < units) {
            use_round(w1, b1, base + stride);
            if (base + 3 * stride < units) load_round(w1, b1, base + 3 * stride);
        }
    }

    // lane holds token p, rows 4g + i in register i
    int* my = red + wave * 256 + lane;
    my[0] = acc_q.x + acc_b.x;
    my[64] = acc_q.y + acc_b.y;
    my[128] = acc_q.z + acc_b.z;
    my[192] = acc_q.w + acc_b.w;
    __syncthreads();

    if (nwaves >= 4) {
        if (threadIdx.x < 256 && e_m < M) {
            int part[kMaxWaves];  // independent LDS reads, one wait
#pragma unroll
            for (int wv = 0; wv < kMaxWaves; ++wv) part[wv] = (wv < nwaves) ? red[wv * 256 + threadIdx.x] : 0;
            int sum = 0;
#pragma unroll
            for (int wv = 0; wv < kMaxWaves; ++wv) sum += part[wv];
            if (acc_out) acc_out[(size_t)e_m * N + e_n] = sum;
            if (out) {
                uint16_t o = f32_to_bf16_rne((float)sum / bf16_to_f32(e_sb) * bf16_to_f32(e_wsb));
                if (residual) o = f32_to_bf16_rne(bf16_to_f32(e_res) + bf16_to_f32(o));
                out[(size_t)e_m * N + e_n] = o;
            }
        }
        return;
    }
    // fewer than four waves: every thread finishes several outputs
    for (int t = threadIdx.x; t < 256; t += nwaves * 64) {
        const int l = t & 63;
        const int m = m0 + (l & 15);
        if (m >= M) continue;
        int sum = 0;
        for (int wv = 0; wv < nwaves; ++wv) sum += red[wv * 256 + t];
        const int n = nb * 16 + 4 * (l >> 4) + (t >> 6);
        if (acc_out) acc_out[(size_t)m * N + n] = sum;
        if (out) {
            const float v = (float)sum / bf16_to_f32(s[m]) * bf16_to_f32(ws[scale_slot(smap, n)]);
            uint16_t o = f32_to_bf16_rne(v);
            if (residual) o = f32_to_bf16_rne(bf16_to_f32(residual[(size_t)m * N + n]) + bf16_to_f32(o));
            out[(size_t)m * N + n] = o;
        }
    }
}

// ---------------------------------------------------------------------------
// Prefill GEMM (M > 16): int8 MFMA 32x32x32, activations tiled through LDS
// ---------------------------------------------------------------------------
// out[m, n] = sum_k a[m, k] * w[n, k].  A workgroup of four waves owns a
// (32*MT) x (128*NT) output tile; the waves sit side by side along n and share
// the activation rows, which are staged through LDS in 256-k chunks (double
// buffered, one LDS-only barrier per chunk).  Weights never touch LDS: one
// packed word is the 16 k of one weight row that a lane needs as its MFMA row
// operand for a 32-k step (row n = lane % 32, k-half = lane / 32), so each wave reads its
// own words straight from global memory -- two full 128-byte tiles per step
// and 32 columns -- expands them once (3 shifts + 4 ands) and reuses the
// result for all MT row tiles.  The +2 bias of the codes is removed in the
// epilogue with sum_k a[m, k], collected while the rows pass through staging.
constexpr int kPfWaves = 4;
constexpr int kPfSteps = 8;                     // 32-k MFMA steps per LDS chunk (256 k)
constexpr int kPfChunk = kPfSteps * 32;
constexpr int kPfRowBytes = kPfChunk + 16;      // padded row: 16-byte reads of 32 rows spread over the banks
constexpr int kPfPieces = kPfChunk / 16;        // 16-byte pieces per row and chunk
typedef int v16i __attribute__((ext_vector_type(16)));

template <int MT, int NT, int KS>
__global__ __launch_bounds__(kPfWaves * 64 * KS)
__attribute__((amdgpu_waves_per_eu(MT == 2 && NT == 2 && KS == 1 ? 3 : (MT * NT == 8 && KS == 1 ? 2 : 1))))
void gemm_i2_prefill_kernel(
    // parameter order: what the first loads need comes first (kernel-argument preload)
    // (band and seg_cols repeat gridDim.x / 8 and gridDim.y: the grid's own size is not among the preloaded dwords)
    const int8_t* __restrict__ act, const uint32_t* __restrict__ wq, int M, int N, int K, int nunits, int cseg_shift,
    int band, int seg_cols, const uint16_t* __restrict__ s, uint16_t* __restrict__ out, int32_t* __restrict__ acc_out,
    const uint16_t* __restrict__ ws, ScaleMap smap, const uint16_t* __restrict__ residual) {
    constexpr int TM = MT * 32;
    constexpr int NTHR = kPfWaves * 64;
    constexpr int PPT = TM * kPfPieces / NTHR;  // pieces of a chunk per thread
    extern __shared__ __attribute__((aligned(16))) int8_t lds_all[];  // [KS][2][TM * kPfRowBytes]
    __shared__ int rowsum[KS][TM];
    __shared__ float sval[TM];
    __shared__ float rinv[TM];

    // KS groups of four waves share the tile and split its 256-k chunks between them (group g
    // takes chunks g, g + KS, ...): with few tiles on the machine a tile's chain of chunks is
    // pure latency, and KS groups walk it in 1/KS of the time.  Each group stages its own chunks
    // in its own LDS buffers; the groups' accumulators are added through LDS at the end.
    const int grp = KS > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x / NTHR) : 0;
    int8_t* lds_a = lds_all + grp * (2 * TM * kPfRowBytes);
    const int tid = threadIdx.x % NTHR;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    // Workgroup -> tile.  Workgroups are handed to the 8 XCDs round-robin by
    // linear id, and each XCD has its own L2.  The tile grid is cut into bands of
    // `band` row tiles; a band belongs to one XCD (band b -> XCD b % 8), which
    // walks it column tile by column tile.  The workgroups running on an XCD at
    // any time therefore share a few row tiles (kept in that L2 for the whole
    // band) and a few column tiles, instead of every tile pulling both of its
    // operands through the memory-side cache on its own.  Unless the number of
    // bands is a multiple of 8, the column tiles are cut into segments too, so
    // that every XCD gets the same number of (band, segment) units.
    // The grid spells the mapping out so that no division stands between the
    // kernel's entry and its first load: x = XCD + 8 * (row tile within the
    // band), y = column tile within the segment, z = round of 8 units (the
    // linear workgroup id, which picks the XCD, is x + 8 * band * (y + ...)).
    const int row_tiles = (M + TM - 1) / TM;
    const int col_tiles = (N + kPfWaves * NT * 32 - 1) / (kPfWaves * NT * 32);
    const int unit = (blockIdx.x & 7) + 8 * blockIdx.z;  // unit = (band, column segment) -> XCD unit % 8
    if (unit >= nunits) return;
    const bool has_out = (cseg_shift >> 8) != 0;  // bit 8 repeats out != nullptr (out itself is not among the preloaded dwords)
    cseg_shift &= 0xff;
    const int col_tile = (unit & ((1 << cseg_shift) - 1)) * seg_cols + blockIdx.y;
    const int row_tile = (unit >> cseg_shift) * band + (blockIdx.x >> 3);
    if (row_tile >= row_tiles || col_tile >= col_tiles) return;  // ragged last band / segment (uniform over the workgroup)
    const int m0 = row_tile * TM;
    const int n0 = (col_tile * kPfWaves + wave) * NT * 32;
    const int nl = lane & 31;
    const int kc = lane >> 5;
    const int ksteps = K >> 5;
    const int nchunks = ((ksteps + kPfSteps - 1) / kPfSteps + KS - 1) / KS;  // per group; chunk c of group g is chunk c * KS + g of the row

    // All loads of the main loop are buffer loads: base (a resource descriptor in
    // scalar registers) + a per-lane byte offset computed once + a scalar offset
    // that advances with k, so the loop spends no vector instructions on
    // addresses.  The activation descriptor covers this workgroup's rows only:
    // rows past M lie beyond it and read as zeros.
    // staging map: piece p = tid + i * NTHR is 16 bytes of row p / kPfPieces at k-offset (p % kPfPieces) * 16
    const int rows_here = (M - m0) < TM ? (M - m0) : TM;
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(act + (size_t)m0 * K), 0, rows_here * K, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)wq, 0, (N >> 2) * K, 0x00020000);
    // (NTHR / kPfPieces = 16 rows per round i: piece i of a thread is its piece 0 moved down 16 * i rows, so one
    // offset per thread and constants / scalar multiples of K do for all of them)
    static_assert(NTHR % kPfPieces == 0, "a thread's pieces share their k offset");
    constexpr int kRowsPerRound = NTHR / kPfPieces;
    const int a_koff = (tid % kPfPieces) * 16;
    const int a_off0 = (tid / kPfPieces) * K + a_koff;
    const int a_dst0 = (tid / kPfPieces) * kPfRowBytes + a_koff;
    const int a_round = kRowsPerRound * K;  // bytes between a thread's consecutive pieces in global memory
    // packed word of (column n, 32-k step, k-half kc), as a byte offset; columns past N re-read column N-1
    int w_off[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int n = n0 + nt * 32 + nl;
        n = n < N ? n : N - 1;
        w_off[nt] = ((n >> 4) * K + ((n & 15) >> 3) * 16 + kc * 8 + (n & 7)) * 4;
    }
    // the tokens' scales: requested here, ahead of everything else, and used (a division) only
    // once the loads of the first chunks are on their way; without output there are no scales
    // (the accumulator-only entry): the request then goes to an address that exists
    const int s_row = (m0 + (tid & (TM - 1))) < M ? (m0 + (tid & (TM - 1))) : (M - 1);
    const uint16_t s_raw = *(has_out ? s + s_row : (const uint16_t*)wq);

    v16i acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0;
    int rs[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) rs[i] = 0;

    // Software pipeline over the 256-k chunks, one register set per operand.
    // While chunk c is multiplied out of LDS, the activation pieces of chunk c+1
    // move from their registers (aP) into the other LDS buffer and the same
    // registers are at once re-requested for chunk c+2; no register is ever
    // copied (a copy would wait for the load it copies).  A weight word is
    // re-requested for chunk c+1 right after the MFMAs that consumed it.  Either
    // load has most of a chunk to land.  (Second sets requested a chunk further
    // ahead measured the same or 1 % slower at every size; without the second
    // set of words the 64 x 256 tile fits three waves per SIMD instead of two:
    // a layer's four GEMMs 1.67 -> 1.81 POP/s at M = 4096, 1.50 -> 1.54 at M = 2048.)
    v4i aP[PPT];
    uint32_t wW[kPfSteps][NT];
    const v4i zero4 = {0, 0, 0, 0};
    const int ones = 0x01010101;
    const int last_step_off = (ksteps - 1) * 128;  // byte offset of the last 32-k step inside a row block
    auto load_piece = [&](int c, int i) -> v4i {
        // a chunk past the end re-reads chunk 0; it is never staged into a buffer that is multiplied.
        // The whole offset is the vector offset, the one the descriptor's range check sees: a piece past the end
        // of K in the workgroup's last row, or in a row past M, lies beyond the descriptor and is not fetched
        // (the scalar offset is outside that check).
        const int k0 = (c * KS + grp) * kPfChunk < K ? (c * KS + grp) * kPfChunk : 0;
        int base = a_off0 + k0;
        asm volatile("" : "+v"(base));  // one add per piece here instead of PPT offsets kept in registers
        return __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, base + i * a_round, 0, 0);
    };
    auto load_word = [&](int c, int ks, int nt) -> uint32_t {
        const int so = ((c * KS + grp) * kPfSteps + ks) * 128;
        return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(w_rsrc, w_off[nt], so < last_step_off ? so : last_step_off, 0);
    };
    auto stage_piece = [&](int c, int i, const v4i& piece, int8_t* buf) {
        const v4i v = ((c * KS + grp) * kPfChunk + a_koff) >= K ? zero4 : piece;  // ragged last chunk, or a chunk past the end
        *(v4i*)(buf + a_dst0 + i * (kRowsPerRound * kPfRowBytes)) = v;
        rs[i] = __builtin_amdgcn_sdot4(v.x, ones, rs[i], false);
        rs[i] = __builtin_amdgcn_sdot4(v.y, ones, rs[i], false);
        rs[i] = __builtin_amdgcn_sdot4(v.z, ones, rs[i], false);
        rs[i] = __builtin_amdgcn_sdot4(v.w, ones, rs[i], false);
    };

#pragma unroll
    for (int i = 0; i < PPT; ++i) aP[i] = load_piece(0, i);
#pragma unroll
    for (int ks = 0; ks < kPfSteps; ++ks)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wW[ks][nt] = load_word(0, ks, nt);
#pragma unroll
    for (int i = 0; i < PPT; ++i) stage_piece(0, i, aP[i], lds_a);
#pragma unroll
    for (int i = 0; i < PPT; ++i) aP[i] = load_piece(1, i);
    if (threadIdx.x < TM) {
        const float sv = has_out ? bf16_to_f32(s_raw) : 1.0f;
        sval[tid] = sv;
        rinv[tid] = 1.0f / sv;
    }
    lds_barrier();

    // Per k-step, besides its MFMAs: one slice of the staging of chunk c+1 (LDS
    // write + row-sum), the reload of that slice's registers for chunk c+2, the
    // reload of this step's weight words for chunk c+1, and the LDS reads of the
    // next step's A operands.  Spread like this the memory work issues in the
    // shadow of the MFMAs instead of stopping all four waves at once.  Nothing is
    // conditional: pieces at k >= K (ragged last chunk, or a whole chunk past the
    // end) are staged as zeros and multiply to nothing; the words of a k-step
    // past the end re-read the last step and meet those zeros.
    // The matrix pipe runs one 32x32x32 for 32 cycles and a wave issues in
    // order, so a run of MFMAs back to back blocks the wave's other instructions
    // behind it.  Every k-step is therefore written as MT*NT slots of
    // "one MFMA + a share of the preparation of the NEXT k-step" (expanding its
    // weight words, reading its A operands from LDS, a slice of the staging,
    // re-requesting the words just consumed), fenced so the order survives
    // scheduling: the preparation issues in the shadow of the MFMA before it.
    auto expand = [&](uint32_t wd) -> v4i {
        v4i r;
        r.x = (int)(wd & 0x03030303u);
        r.y = (int)((wd >> 2) & 0x03030303u);
        r.z = (int)((wd >> 4) & 0x03030303u);
        r.w = (int)((wd >> 6) & 0x03030303u);
        return r;
    };
    auto chunk_body = [&](int c, uint32_t(&wuse)[kPfSteps][NT], v4i(&astage)[PPT]) {
        const int8_t* abuf = lds_a + (c & 1) * (TM * kPfRowBytes) + nl * kPfRowBytes + kc * 16;
        int8_t* sbuf = lds_a + ((c + 1) & 1) * (TM * kPfRowBytes);
        constexpr int SLOTS = MT * NT;
        v4i aop[2][MT], bop[2][NT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) aop[0][mt] = *(const v4i*)(abuf + mt * 32 * kPfRowBytes);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) bop[0][nt] = expand(wuse[0][nt]);
#pragma unroll
        for (int ks = 0; ks < kPfSteps; ++ks) {
            const int cur = ks & 1, nxt = cur ^ 1;
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot) {
                const int mt = slot / NT, nt = slot % NT;
                acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bop[cur][nt], aop[cur][mt], acc[mt][nt], 0, 0, 0);
                // preparation items, dealt round-robin over the slots
                // (the LDS reads first: they have the longest way to go before their first use)
                if (ks + 1 < kPfSteps) {
#pragma unroll
                    for (int j = 0; j < MT; ++j)
                        if (j % SLOTS == slot)
                            aop[nxt][j] = *(const v4i*)(abuf + j * 32 * kPfRowBytes + (ks + 1) * 32);
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        if ((MT + j) % SLOTS == slot) bop[nxt][j] = expand(wuse[ks + 1][j]);
                }
                if ((NT + MT) % SLOTS == slot) {
#pragma unroll
                    for (int i = ks * PPT / kPfSteps; i < (ks + 1) * PPT / kPfSteps; ++i) {
                        stage_piece(c + 1, i, astage[i], sbuf);
                        astage[i] = load_piece(c + 2, i);
                    }
                }
                if (slot == SLOTS - 1) {
                    // the words of this step were expanded during the previous one: re-request them
#pragma unroll
                    for (int j = 0; j < NT; ++j) wuse[ks][j] = load_word(c + 1, ks, j);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        lds_barrier();
    };
    for (int c = 0; c < nchunks; ++c) chunk_body(c, wW, aP);

    // row sums: the kPfPieces (= 16) threads of one DPP row staged the pieces of one activation row
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
        int v = rs[i];
        v += dpp_move<0xB1>(v);
        v += dpp_move<0x4E>(v);
        v += dpp_move<0x141>(v);
        v += dpp_move<0x140>(v);
        if ((tid & 15) == 0) rowsum[grp][(tid + i * NTHR) / kPfPieces] = v;
    }
    if (KS > 1) {
        // groups 1.. leave their accumulators in LDS (the staging buffers are free: every wave is
        // past the barrier of its last chunk) and are done; group 0 adds them up and finishes the tile
        int* red = (int*)lds_all;  // [KS - 1][kPfWaves][MT * NT * 16][64]
        if (grp > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        red[(((grp - 1) * kPfWaves + wave) * (MT * NT * 16) + (mt * NT + nt) * 16 + r) * 64 + lane] = acc[mt][nt][r];
        }
        lds_barrier();
        if (grp > 0) return;
#pragma unroll
        for (int g = 1; g < KS; ++g)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[mt][nt][r] += red[(((g - 1) * kPfWaves + wave) * (MT * NT * 16) + (mt * NT + nt) * 16 + r) * 64 + lane];
    } else {
        lds_barrier();
    }

    // The weights are the MFMA's row operand, so a result lane holds one token
    // (m = lane % 32 of the row tile) and, in register r, output column
    // (r / 4) * 8 + (lane / 32) * 4 + r % 4 of the 32-column tile: four
    // consecutive columns per register quad, stored as one 8-byte (bf16) or
    // 16-byte (int32) piece.  Everything per token (row sum, scale, its
    // reciprocal) is a single value per lane; the weight scales of the lane's
    // 16 * NT columns are fetched once.
    // Division by the token's scale: a correctly rounded reciprocal per token
    // (one IEEE divide) and, per element, q0 = a * rinv refined by
    // e = fma(-q0, s, a), q = fma(e, rinv, q0).
    // Weight scales of the lane's 16 * NT columns.  Nearly always the wave's whole column range
    // lies in one scale slot (a uniform test): one load; otherwise a slot per column.
    float wsf[NT][16];
    if (out) {
        const int n_first = n0 < N ? n0 : N - 1;
        const int n_last = (n0 + NT * 32 - 1) < N ? (n0 + NT * 32 - 1) : N - 1;
        const int slot_first = scale_slot(smap, n_first);
        if (slot_first == scale_slot(smap, n_last)) {
            const float w1 = bf16_to_f32(ws[slot_first]);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 16; ++r) wsf[nt][r] = w1;
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int n = n0 + nt * 32 + (r >> 2) * 8 + kc * 4 + (r & 3);
                    wsf[nt][r] = bf16_to_f32(ws[scale_slot(smap, n < N ? n : N - 1)]);
                }
        }
    }
    if (out && !acc_out) {
        // bf16 output through LDS: a lane holds one token and four consecutive columns per register quad, so
        // storing from the accumulator layout writes 8-byte pieces of 32 different rows per instruction (a row's
        // 128 bytes arrive as 16 separate partial writes).  Each wave instead parks the 32 rows of one row tile
        // in a region of its own (the staging buffers are free: every wave is past the last chunk's barrier,
        // and group 0 past the reduction), padded so that neither the 8-byte writes nor the 16-byte reads
        // pile up on a bank, and stores them as 16-byte pieces, a row's bytes side by side: 4 * NT store
        // instructions per wave and row tile, every one of them whole 64-byte runs.
        constexpr int kRowB = NT * 64 + 16;                       // bytes per parked row
        // (with several k-groups, behind the accumulators the other groups left: another wave of this group may still be adding its share)
        // (where both do not fit, the group's waves meet once more before they park over them: the other groups'
        // waves have ended by then, and a barrier waits for the surviving waves only)
        constexpr int kRedBytes = (KS - 1) * kPfWaves * MT * NT * 16 * 64 * 4;
        constexpr bool kParkOverRed = kRedBytes + kPfWaves * 32 * kRowB > KS * 2 * MT * 32 * kPfRowBytes;
        if (kParkOverRed) lds_barrier();
        int8_t* park = lds_all + (kParkOverRed ? 0 : kRedBytes) + wave * (32 * kRowB);
        static_assert(kPfWaves * 32 * kRowB <= KS * 2 * MT * 32 * kPfRowBytes, "parked rows must fit the staging buffers");
        constexpr int kPiecesPerRow = NT * 4;                     // 16-byte pieces
        constexpr int kRowsPerStore = 64 / kPiecesPerRow;
        const int pr = lane / kPiecesPerRow, pc = lane % kPiecesPerRow;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int ml = mt * 32 + nl;
            int rs2 = 0;
#pragma unroll
            for (int g = 0; g < KS; ++g) rs2 += 2 * rowsum[g][ml];
            const float sv = sval[ml], ri = rinv[ml];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    float h[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float a = (float)(acc[mt][nt][g4 * 4 + j] - rs2);
                        const float q0 = a * ri;
                        const float q = __builtin_fmaf(__builtin_fmaf(-q0, sv, a), ri, q0);
                        h[j] = q * wsf[nt][g4 * 4 + j];
                    }
                    *(uint2*)(park + nl * kRowB + (nt * 32 + g4 * 8 + kc * 4) * 2) =
                        make_uint2(f32x2_to_bf16x2(h[0], h[1]), f32x2_to_bf16x2(h[2], h[3]));
                }
            // the same wave wrote and reads: LDS operations of a wave complete in order
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int r0 = 0; r0 < 32; r0 += kRowsPerStore) {
                const int row = r0 + pr;
                const int m = m0 + mt * 32 + row;
                const int n = n0 + pc * 8;  // N % 16 == 0 and n0 % 32 == 0: the eight columns are in or out together
                uint4 v = *(const uint4*)(park + row * kRowB + pc * 16);
                if (m < M && n < N) {
                    const size_t o = (size_t)m * N + n;
                    if (residual) {  // out = bf16(residual + bf16(result))
                        const uint4 rv = *(const uint4*)(residual + o);
                        const uint32_t a4[4] = {v.x, v.y, v.z, v.w}, r4[4] = {rv.x, rv.y, rv.z, rv.w};
                        uint32_t o4[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            o4[j] = f32x2_to_bf16x2(__uint_as_float(r4[j] << 16) + __uint_as_float(a4[j] << 16),
                                                    __uint_as_float(r4[j] & 0xffff0000u) + __uint_as_float(a4[j] & 0xffff0000u));
                        v = make_uint4(o4[0], o4[1], o4[2], o4[3]);
                    }
                    *(uint4*)(out + o) = v;
                }
            }
            // the next row tile's writes must not overtake these reads
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        return;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int ml = mt * 32 + nl;
        const int m = m0 + ml;
        int rs2 = 0;
#pragma unroll
        for (int g = 0; g < KS; ++g) rs2 += 2 * rowsum[g][ml];
        const float sv = sval[ml], ri = rinv[ml];
        if (m >= M) continue;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int n = n0 + nt * 32 + g4 * 8 + kc * 4;  // N % 16 == 0: the four columns are in or out together
                if (n >= N) continue;
                const size_t o = (size_t)m * N + n;
                int sum[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) sum[j] = acc[mt][nt][g4 * 4 + j] - rs2;
                if (acc_out) *(v4i*)(acc_out + o) = v4i{sum[0], sum[1], sum[2], sum[3]};
                if (out) {
                    float h[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float a = (float)sum[j];
                        const float q0 = a * ri;
                        const float q = __builtin_fmaf(__builtin_fmaf(-q0, sv, a), ri, q0);
                        h[j] = q * wsf[nt][g4 * 4 + j];
                    }
                    uint2 ob = make_uint2(f32x2_to_bf16x2(h[0], h[1]), f32x2_to_bf16x2(h[2], h[3]));
                    if (residual) {  // out = bf16(residual + bf16(result))
                        const uint2 rv = *(const uint2*)(residual + o);
                        ob.x = f32x2_to_bf16x2(__uint_as_float(rv.x << 16) + __uint_as_float(ob.x << 16),
                                               __uint_as_float(rv.x & 0xffff0000u) + __uint_as_float(ob.x & 0xffff0000u));
                        ob.y = f32x2_to_bf16x2(__uint_as_float(rv.y << 16) + __uint_as_float(ob.y << 16),
                                               __uint_as_float(rv.y & 0xffff0000u) + __uint_as_float(ob.y & 0xffff0000u));
                    }
                    *(uint2*)(out + o) = ob;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Prefill GEMM for the 64 x 256 (and 128 x 256) output tile once the machine is full: the same decomposition as
// gemm_i2_prefill_kernel (four waves side by side along n, weights from global straight into the MFMA row
// operand, activations through LDS), rebuilt around what the CU's vector-memory path costs.  Measured with a
// loop of MFMAs and one kind of other instruction between them: vector, scalar and wait instructions are free
// next to v_mfma_i32_32x32x32_i8, two 16-byte LDS reads per four MFMAs as well, but every vector-memory
// instruction occupies the CU's one 64-byte-per-cycle load path for as long as its bytes take, a path all waves
// of the CU share, and a wave stands still while its request is taken.  So:
//  * the activation chunk goes from global memory straight into LDS (buffer_load ... lds, 1 KB per wave and
//    instruction, no registers, no vector instructions; rows XOR-swizzled in 16-byte pieces so that the MFMA
//    operand reads hit every bank once), three stages deep;
//  * a lane fetches the words of its NT column tiles with ONE load per 32-k step: the wave's 32 * NT columns
//    are 2 * NT row blocks of the packed layout, a lane takes NT consecutive words of a tile's run of eight
//    (NT consecutive weight rows, one k-half) and word i feeds column tile i, which therefore holds every
//    NT-th column; half (a quarter) as many weight requests as one word per column tile;
//  * the stored codes c = w + 2 are expanded to bytes that read 64 * w -- xor with 0b10 gives w in two-bit two's
//    complement, and a two-bit field at the top of a byte is that number times 64 -- so the accumulators are
//    64 * sum(w * a) exactly (|.| <= 64 * 127 * K < 2^31 up to K = 262144), the +2 of the codes never enters,
//    no row sums are collected and the epilogue starts with an exact shift;
//  * with the interleaved column tiles a lane's accumulators of one register quad are 4 * NT consecutive output
//    columns: 16-byte (NT = 2) or 32-byte stores per token instead of 8.
// K must be a multiple of CK.
template <int NT>
struct PfxWords;
template <>
struct PfxWords<2> {
    typedef uint32_t type __attribute__((ext_vector_type(2)));
};
template <>
struct PfxWords<4> {
    typedef uint32_t type __attribute__((ext_vector_type(4)));
};
// 16 bytes per lane from a buffer straight into LDS: lane l's piece lands at ldsp + 16 l (ldsp wave-uniform)
__device__ __forceinline__ void load16_to_lds(__amdgpu_buffer_rsrc_t rsrc, int8_t* ldsp, int voff, int soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)ldsp, 16, voff, soff, 0, 0);
}

// One output tile of (32 MT) rows x (WAVES x 32 NT) columns at (row_tile, column n_base) by the WAVES waves of the
// calling workgroup (further waves of the workgroup must not enter).
template <int MT, int NT, int CK, int WAVES>
__device__ __forceinline__ void pfx_tile(
    const int8_t* __restrict__ act, const uint32_t* __restrict__ wq, int M, int N, int K, int row_tile, int n_base, bool has_out,
    const uint16_t* __restrict__ s, uint16_t* __restrict__ out, int32_t* __restrict__ acc_out,
    const uint16_t* __restrict__ ws, const ScaleMap& smap, const uint16_t* __restrict__ residual) {
    constexpr int kPfxWaves = WAVES;
    constexpr int TM = MT * 32;
    constexpr int KSTEPS = CK / 32;
    constexpr int PPR = CK / 16;             // 16-byte pieces per row and chunk
    constexpr int RPI = 64 / PPR;            // rows one load instruction of a wave covers
    constexpr int ROUNDS = TM / (RPI * kPfxWaves);  // load instructions per wave and stage
    constexpr int SB = TM * CK;              // bytes per stage
    constexpr int QR = 8 / NT;               // lanes per run of eight words
    static_assert(NT == 2 || NT == 4, "two or four interleaved column tiles");
    static_assert(TM % (RPI * kPfxWaves) == 0 && (CK == 128 || CK == 256), "stage shape");
    extern __shared__ __attribute__((aligned(1024))) int8_t lds_x[];  // [3][TM][CK], rows swizzled in 16-byte pieces

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = row_tile * TM;
    const int n0 = n_base + wave * NT * 32;
    const int nl = lane & 31;
    const int kc = lane >> 5;
    const int nchunks = K / CK;

    // rows past M lie beyond the activation descriptor: they arrive in LDS as zeros
    const int rows_here = (M - m0) < TM ? (M - m0) : TM;
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(act + (size_t)m0 * K), 0, rows_here * K, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)wq, 0, (N >> 2) * K, 0x00020000);

    // activation requests: instruction (r * 4 + wave) of a stage fills 1 KB of it = RPI rows; the lane at LDS
    // piece p of row i fetches global piece p ^ (i & 7) (the row offset is part of the vector offset: the one
    // the descriptor's range check sees)
    const int arow = wave * RPI + lane / PPR;
    const int akp = (lane % PPR) ^ (arow & 7);
    int a_voff[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) a_voff[r] = (arow + r * kPfxWaves * RPI) * K + akp * 16;
    auto load_stage = [&](int c, int st) {
#pragma unroll
        for (int r = 0; r < ROUNDS; ++r) load16_to_lds(a_rsrc, lds_x + st * SB + (r * kPfxWaves + wave) * 1024, a_voff[r], c * CK);
    };
    // weight requests (row blocks past N repeat the last one; their columns are never stored)
    const int wb = nl / (2 * QR), wp = nl % (2 * QR), whi = wp / QR, wlo = NT * (wp % QR);
    int w_voff;
    {
        int blk = (n0 >> 4) + wb;
        blk = blk < (N >> 4) ? blk : (N >> 4) - 1;
        w_voff = blk * K * 4 + (whi * 16 + kc * 8 + wlo) * 4;
    }
    const int last_step_off = ((K >> 5) - 1) * 128;
    typedef typename PfxWords<NT>::type wvec_t;
    auto load_words = [&](int c, int ks) -> wvec_t {
        int so = (c * KSTEPS + ks) * 128;
        so = so < last_step_off ? so : last_step_off;  // the step behind the last chunk re-reads the last one
        if constexpr (NT == 2)
            return __builtin_bit_cast(wvec_t, __builtin_amdgcn_raw_buffer_load_b64(w_rsrc, w_voff, so, 0));
        else
            return __builtin_bit_cast(wvec_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, w_voff, so, 0));
    };
    // the scales of the lane's MT tokens (without output there are none: the request goes to an address that exists)
    uint16_t s_raw[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + mt * 32 + nl;
        s_raw[mt] = *(has_out ? s + (m < M ? m : M - 1) : (const uint16_t*)wq);
    }

    v16i acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0;

    wvec_t wW[KSTEPS];
    load_stage(0, 0);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) wW[ks] = load_words(0, ks);
    if (nchunks > 1) load_stage(1, 1);

    // LDS read offsets: row nl, piece (2 ks + kc) ^ (nl & 7)
    int a_rd[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) a_rd[ks] = nl * CK + (((ks * 2 + kc) ^ (nl & 7)) * 16);

    auto expand = [&](uint32_t wd) -> v4i {
        const uint32_t x = wd ^ 0xAAAAAAAAu;
        v4i r;
        r.x = (int)((x << 6) & 0xC0C0C0C0u);
        r.y = (int)((x << 4) & 0xC0C0C0C0u);
        r.z = (int)((x << 2) & 0xC0C0C0C0u);
        r.w = (int)(x & 0xC0C0C0C0u);
        return r;
    };

    // the first chunk: every wave waits for its own requests, then all meet
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0); the other counters untouched
    lds_barrier();

    auto chunk_body = [&](int c, auto stc) {
        constexpr int ST = decltype(stc)::value;
        constexpr int SLOTS = MT * NT;
        // stage (ST + 2) % 3 was read in chunk c - 1, which every wave has left (the barrier at its end)
        if (c + 2 < nchunks) load_stage(c + 2, (ST + 2) % 3);
        const int8_t* abuf = lds_x + ST * SB;
        v4i aop[2][MT], bop[2][NT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) aop[0][mt] = *(const v4i*)(abuf + a_rd[0] + mt * 32 * CK);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) bop[0][nt] = expand(wW[0][nt]);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const int cur = ks & 1, nxt = cur ^ 1;
#pragma unroll
            for (int slot = 0; slot < SLOTS; ++slot) {
                const int mt = slot / NT, nt = slot % NT;
                acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bop[cur][nt], aop[cur][mt], acc[mt][nt], 0, 0, 0);
                if (ks + 1 < KSTEPS) {
#pragma unroll
                    for (int j = 0; j < MT; ++j)
                        if (j % SLOTS == slot) aop[nxt][j] = *(const v4i*)(abuf + a_rd[ks + 1] + j * 32 * CK);
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        if ((MT + j) % SLOTS == slot) bop[nxt][j] = expand(wW[ks + 1][j]);
                }
                if (slot == SLOTS - 1) wW[ks] = load_words(c + 1, ks);  // expanded during the step before: re-request
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the next chunk's activations (requested two chunks ago) are older than every request that may stay in
        // flight: this chunk's re-requested words and the stage requested at its start
        constexpr int kYounger = KSTEPS + ROUNDS;
        __builtin_amdgcn_s_waitcnt(0x0f70 | (kYounger & 15) | ((kYounger >> 4) << 14));
        lds_barrier();
    };
    int c = 0;
    for (; c + 3 <= nchunks; c += 3) {
        chunk_body(c, std::integral_constant<int, 0>{});
        chunk_body(c + 1, std::integral_constant<int, 1>{});
        chunk_body(c + 2, std::integral_constant<int, 2>{});
    }
    if (c < nchunks) chunk_body(c, std::integral_constant<int, 0>{});
    if (c + 1 < nchunks) chunk_body(c + 1, std::integral_constant<int, 1>{});

    // Epilogue.  A lane holds token nl of row tile mt; register r of column tile nt is the weight row with
    // operand index (r / 4) * 8 + kc * 4 + r % 4, i.e. column n0 + 16 b + 8 hi + lo + nt with that index split
    // into (b, hi, lo) as in the weight requests: for one register quad the 4 * NT values over (r % 4, nt) are
    // 4 * NT consecutive columns.  Division by the token's scale as in gemm_i2_prefill_kernel (reciprocal and
    // one correction step: the bits of the IEEE divide for these integer numerators).
    const int n_first = n0 < N ? n0 : N - 1;
    const int n_last = (n0 + NT * 32 - 1) < N ? (n0 + NT * 32 - 1) : N - 1;
    const int slot_first = scale_slot(smap, n_first);
    const bool one_slot = slot_first == scale_slot(smap, n_last);
    const float w1 = out ? bf16_to_f32(ws[slot_first]) : 1.0f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + mt * 32 + nl;
        const float sv = has_out ? bf16_to_f32(s_raw[mt]) : 1.0f;
        const float ri = 1.0f / sv;
        if (m >= M) continue;
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const int ridx = g4 * 8 + kc * 4;
            const int n = n0 + 16 * (ridx / (2 * QR)) + 8 * ((ridx % (2 * QR)) / QR) + NT * (ridx % QR);
            if (n >= N) continue;  // N % 16 == 0 and n % (4 * NT) == 0: the columns of a quad are in or out together
            const size_t o = (size_t)m * N + n;
            int sum[4 * NT];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    // column offset of (register j of the quad, column tile nt) from n
                    const int col = NT == 2 ? 2 * j + nt : 8 * (j / 2) + 4 * (j % 2) + nt;
                    sum[col] = acc[mt][nt][g4 * 4 + j] >> 6;  // exact: the accumulator is 64 * sum(w * a)
                }
            if (acc_out) {
#pragma unroll
                for (int v = 0; v < NT; ++v) *(v4i*)(acc_out + o + 4 * v) = v4i{sum[4 * v], sum[4 * v + 1], sum[4 * v + 2], sum[4 * v + 3]};
            }
            if (out) {
                float h[4 * NT];
#pragma unroll
                for (int col = 0; col < 4 * NT; ++col) {
                    const float a = (float)sum[col];
                    const float q0 = a * ri;
                    const float q = __builtin_fmaf(__builtin_fmaf(-q0, sv, a), ri, q0);
                    h[col] = q * (one_slot ? w1 : bf16_to_f32(ws[scale_slot(smap, n + col)]));
                }
#pragma unroll
                for (int v = 0; v < NT / 2; ++v) {
                    uint4 ob = make_uint4(f32x2_to_bf16x2(h[8 * v], h[8 * v + 1]), f32x2_to_bf16x2(h[8 * v + 2], h[8 * v + 3]),
                                          f32x2_to_bf16x2(h[8 * v + 4], h[8 * v + 5]), f32x2_to_bf16x2(h[8 * v + 6], h[8 * v + 7]));
                    if (residual) {  // out = bf16(residual + bf16(result))
                        const uint4 rv = *(const uint4*)(residual + o + 8 * v);
                        const uint32_t a4[4] = {ob.x, ob.y, ob.z, ob.w}, r4[4] = {rv.x, rv.y, rv.z, rv.w};
                        uint32_t o4[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            o4[j] = f32x2_to_bf16x2(__uint_as_float(r4[j] << 16) + __uint_as_float(a4[j] << 16),
                                                    __uint_as_float(r4[j] & 0xffff0000u) + __uint_as_float(a4[j] & 0xffff0000u));
                        ob = make_uint4(o4[0], o4[1], o4[2], o4[3]);
                    }
                    *(uint4*)(out + o + 8 * v) = ob;
                }
            }
        }
    }
}

constexpr int kPfxWaves = 4;
template <int MT, int NT, int CK>
__global__ __launch_bounds__(kPfxWaves * 64) __attribute__((amdgpu_waves_per_eu(MT * NT <= 4 ? 3 : 2)))
void gemm_i2_prefill_dma_kernel(
    const int8_t* __restrict__ act, const uint32_t* __restrict__ wq, int M, int N, int K, int nunits, int cseg_shift,
    int band, int seg_cols, const uint16_t* __restrict__ s, uint16_t* __restrict__ out, int32_t* __restrict__ acc_out,
    const uint16_t* __restrict__ ws, ScaleMap smap, const uint16_t* __restrict__ residual) {
    // workgroup -> tile: as gemm_i2_prefill_kernel (bands of row tiles per XCD, column segments)
    const int row_tiles = (M + MT * 32 - 1) / (MT * 32);
    const int col_tiles = (N + kPfxWaves * NT * 32 - 1) / (kPfxWaves * NT * 32);
    const int unit = (blockIdx.x & 7) + 8 * blockIdx.z;
    if (unit >= nunits) return;
    const bool has_out = (cseg_shift >> 8) != 0;
    cseg_shift &= 0xff;
    const int col_tile = (unit & ((1 << cseg_shift) - 1)) * seg_cols + blockIdx.y;
    const int row_tile = (unit >> cseg_shift) * band + (blockIdx.x >> 3);
    if (row_tile >= row_tiles || col_tile >= col_tiles) return;
    pfx_tile<MT, NT, CK, kPfxWaves>(act, wq, M, N, K, row_tile, col_tile * (kPfxWaves * NT * 32), has_out, s, out, acc_out, ws, smap,
                                    residual);
}

// The same tiles in two sizes from one launch, for output shapes that leave a little more than one 64 x 256 tile per CU
// (2048 x 2560: 320 tiles on 256 CUs -- a quarter of the CUs with two tiles, or three half-height tiles on half of them):
// the first big_cols column tiles of 256 go to workgroups that take a 64 x 256 tile each, the columns behind them to
// workgroups of which two waves take a 32 x 128 tile (a quarter of the work; the other two waves leave at once), so that
// a CU holds one tile of each kind.  Workgroup w of a kind -> XCD w % 8 -> a band of row tiles of its own.
template <int CK>
__global__ __launch_bounds__(kPfxWaves * 64) __attribute__((amdgpu_waves_per_eu(3)))
void gemm_i2_prefill_mix_kernel(
    const int8_t* __restrict__ act, const uint32_t* __restrict__ wq, int M, int N, int K, int nbig, int big_cols, int flags,
    int small_cols, const uint16_t* __restrict__ s, uint16_t* __restrict__ out, int32_t* __restrict__ acc_out,
    const uint16_t* __restrict__ ws, ScaleMap smap, const uint16_t* __restrict__ residual) {
    const bool has_out = (flags & 1) != 0;
    const int w = blockIdx.x;
    if (w < nbig) {
        // 64-row tiles: XCD x takes a band of row tiles x * band .. and walks the columns (nbig = 8 * band * big_cols)
        const int rt = (M + 63) >> 6;
        const int band = (rt + 7) >> 3;
        const int j = w >> 3;
        const int row_tile = (w & 7) * band + j % band;
        const int col_tile = j / band;
        if (row_tile >= rt) return;  // a ragged last band
        pfx_tile<2, 2, CK, 4>(act, wq, M, N, K, row_tile, col_tile * 256, has_out, s, out, acc_out, ws, smap, residual);
    } else {
        if (threadIdx.x >= 128) return;
        const int v = w - nbig;
        const int rt = (M + 31) >> 5;
        const int band = (rt + 7) >> 3;  // 32-row tiles per XCD
        const int j = v >> 3;
        const int row_tile = (v & 7) * band + j % band;
        const int col_tile = j / band;
        if (row_tile >= rt || col_tile >= small_cols) return;
        pfx_tile<1, 2, CK, 2>(act, wq, M, N, K, row_tile, big_cols * 256 + col_tile * 128, has_out, s, out, acc_out, ws, smap, residual);
    }
}

// ---------------------------------------------------------------------------
// Per-token absmax quantizer: one workgroup per token row
// ---------------------------------------------------------------------------
constexpr int kQuantThreads = 256;
constexpr int kQuantMaxThreads = 1024;
constexpr int kQuantRegVecs = 4;  // 16-byte vectors (8 bf16) kept in registers per thread
constexpr int kQuantRowsMin = 2;   // from this many rows on the quantizer runs a wave per row (rows of up to 4096 values)

// max |x| over 8 packed bf16 as a bit pattern (|x| as bf16 bits orders like the values): one
// and + one packed 16-bit max per pair
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t absmax_bits8(const uint4& v, uint32_t cur) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    u16x2_t m = {(unsigned short)0, (unsigned short)0};
#pragma unroll
    for (int i = 0; i < 4; ++i) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2_t, d[i] & 0x7fff7fffu));
    const uint32_t both = __builtin_bit_cast(uint32_t, m);
    return max(cur, max(both & 0xffffu, both >> 16));
}

// One value to its int8 code, left in the low byte of the result: the product
// x * s in fp32 (mode 1: rounded to bf16), clamped to [-128, 127], then
// + 1.5 * 2^23, which rounds to the nearest integer (ties to even, as rint does)
// and leaves that integer's two's complement in the low mantissa bits.
// Clamping before rounding equals rounding before clamping: the bounds are integers.
template <int MODE>
__device__ __forceinline__ uint32_t quant_low_byte(uint32_t x_f32_bits, float s32) {
    float pr = __uint_as_float(x_f32_bits) * s32;
    if (MODE == 1) pr = bf16_to_f32(f32_to_bf16_rne(pr));
    pr = __builtin_amdgcn_fmed3f(pr, -128.0f, 127.0f);
    return __float_as_uint(pr + 12582912.0f);
}

template <int MODE>
__device__ __forceinline__ int quant_one(uint32_t bits16, float s32) {
    return (int)(quant_low_byte<MODE>(bits16 << 16, s32) & 0xffu);
}

template <int MODE>
__device__ __forceinline__ uint2 quant_vec8(const uint4& v, float s32) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    uint32_t p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo = quant_low_byte<MODE>(d[i] << 16, s32);
        const uint32_t hi = quant_low_byte<MODE>(d[i] & 0xffff0000u, s32);
        p[i] = __builtin_amdgcn_perm(hi, lo, 0x0c0c0400u);  // bytes (lo.0, hi.0, 0, 0)
    }
    // (p0.0, p0.1, p1.0, p1.1)
    return make_uint2(__builtin_amdgcn_perm(p[1], p[0], 0x05040100u), __builtin_amdgcn_perm(p[3], p[2], 0x05040100u));
}

// Activation scale from the row's |x| maximum (as bf16 bits).  torch evaluates
// 127 / t as t.reciprocal() * 127: a reciprocal, then a multiply.  The value
// returned is exactly representable in bf16.
template <int MODE>
__device__ __forceinline__ float quant_scale(uint32_t amax_bits) {
    float amax = __uint_as_float(amax_bits << 16);
    if (MODE == 0) {
        const float r = 1.0f / fmaxf(amax, 1e-5f);
        return bf16_to_f32(f32_to_bf16_rne(r * 127.0f));
    }
    amax = fmaxf(amax, bf16_to_f32(f32_to_bf16_rne(1e-5f)));
    const float r = bf16_to_f32(f32_to_bf16_rne(1.0f / amax));
    return bf16_to_f32(f32_to_bf16_rne(r * 127.0f));
}

template <int MODE>
__global__ __launch_bounds__(kQuantMaxThreads) void quant_absmax_kernel(const uint16_t* __restrict__ x,
                                                                     int8_t* __restrict__ q,
                                                                     uint16_t* __restrict__ s, int K,
                                                                     int32_t* __restrict__ rowsum) {
    __shared__ uint32_t wmax[kQuantMaxThreads / 64];
    __shared__ int wsum[kQuantMaxThreads / 64];
    const int nthreads = blockDim.x;  // 256, or up to 1024 for long rows so that a row still fits the registers
    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const int nvec = K >> 3;
    const uint4* xr = (const uint4*)(x + (size_t)row * K);
    uint2* qr = (uint2*)(q + (size_t)row * K);

    uint4 v[kQuantRegVecs];
    uint32_t am = 0;
#pragma unroll
    for (int r = 0; r < kQuantRegVecs; ++r) {
        const int idx = tid + r * nthreads;
        if (idx < nvec) {
            v[r] = xr[idx];
            am = absmax_bits8(v[r], am);
        } else {
            v[r] = make_uint4(0, 0, 0, 0);
        }
    }
    for (int idx = tid + kQuantRegVecs * nthreads; idx < nvec; idx += nthreads)
        am = absmax_bits8(xr[idx], am);

    // |x| as bf16 bit patterns orders like the values, so the max is an integer max
    am = wave_max_u32(am);
    if ((tid & 63) == 0) wmax[tid >> 6] = am;
    __syncthreads();
    am = wmax[0];
    for (int i = 1; i < (nthreads >> 6); ++i) am = max(am, wmax[i]);

    const float s32 = quant_scale<MODE>(am);
    if (tid == 0) s[row] = f32_to_bf16_rne(s32);

    int part = 0;  // sum of this thread's int8 values (only kept when the caller asks for the row sums)
    const int ones = 0x01010101;
#pragma unroll
    for (int r = 0; r < kQuantRegVecs; ++r) {
        const int idx = tid + r * nthreads;
        if (idx < nvec) {
            const uint2 qv = quant_vec8<MODE>(v[r], s32);
            qr[idx] = qv;
            part = __builtin_amdgcn_sdot4((int)qv.x, ones, __builtin_amdgcn_sdot4((int)qv.y, ones, part, false), false);
        }
    }
    for (int idx = tid + kQuantRegVecs * nthreads; idx < nvec; idx += nthreads) {
        const uint2 qv = quant_vec8<MODE>(xr[idx], s32);
        qr[idx] = qv;
        part = __builtin_amdgcn_sdot4((int)qv.x, ones, __builtin_amdgcn_sdot4((int)qv.y, ones, part, false), false);
    }
    if (rowsum) {  // uniform
        const int ws_ = wave_sum_i32(part);
        if ((tid & 63) == 0) wsum[tid >> 6] = ws_;
        __syncthreads();
        if (tid == 0) {
            int tot = 0;
            for (int i = 0; i < (nthreads >> 6); ++i) tot += wsum[i];
            rowsum[row] = tot;
        }
    }
}

// The same quantizer for many rows (a prompt): one WAVE per row, four rows per workgroup.  The row stays in the
// wave's registers (V vectors of 8 values per lane), the maximum and the row sum are wave reductions: no LDS, no
// barrier, all of a row's loads in flight at once, and enough independent rows per CU to keep the memory busy
// (one workgroup per row leaves a 5 KB row to a chain of load -> reduce -> barrier -> quantize -> store).
template <int MODE, int V>
__global__ __launch_bounds__(256) void quant_absmax_rows_kernel(const uint16_t* __restrict__ x, int8_t* __restrict__ q,
                                                                uint16_t* __restrict__ s, int M, int K,
                                                                int32_t* __restrict__ rowsum) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;  // uniform per wave; nothing below synchronises across waves
    const int nvec = K >> 3;
    const uint4* xr = (const uint4*)(x + (size_t)row * K);
    uint2* qr = (uint2*)(q + (size_t)row * K);
    uint4 v[V];
    uint32_t am = 0;
#pragma unroll
    for (int r = 0; r < V; ++r) {
        const int idx = lane + r * 64;
        v[r] = idx < nvec ? xr[idx] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < V; ++r) am = absmax_bits8(v[r], am);
    am = wave_max_u32(am);
    const float s32 = quant_scale<MODE>(am);
    if (lane == 0) s[row] = f32_to_bf16_rne(s32);
    int part = 0;
    const int ones = 0x01010101;
#pragma unroll
    for (int r = 0; r < V; ++r) {
        const int idx = lane + r * 64;
        const uint2 qv = quant_vec8<MODE>(v[r], s32);
        if (idx < nvec) qr[idx] = qv;
        part = __builtin_amdgcn_sdot4((int)qv.x, ones, __builtin_amdgcn_sdot4((int)qv.y, ones, part, false), false);  // zeros past the row
    }
    if (rowsum) {  // uniform
        const int tot = wave_sum_i32(part);
        if (lane == 0) rowsum[row] = tot;
    }
}

// ---------------------------------------------------------------------------
// BitLinearKernel.forward in one kernel: absmax quantizer + product + epilogue
// ---------------------------------------------------------------------------
// Every workgroup quantizes the (small) activation block itself -- it is a few
// KB read from L2 while the weight words are already in flight -- keeps the
// int8 rows in LDS, and feeds the B operand of the MFMAs from there.  The
// +2 bias of the stored codes is removed with sum(q) per token, collected
// while quantizing: sum((c - 2) * q) = sum(c * q) - 2 * sum(q).
// A workgroup owns RB consecutive 16-row blocks; S waves split K for each.
constexpr int kFusedMaxRB = 4;
constexpr int kFusedMaxTokens = 16;
constexpr int kFusedRowPad = 64;  // bytes between token rows in LDS beyond K
constexpr int kFusedTailPad = 1024;  // bytes after the last row: unclamped reads of k-steps past the end land here

// What the caller wants done to x before the quantizer, and to the result
// after the epilogue.  All of it is what sits around a BitLinear in the
// decoder (gpu/model.py:159-160, 195-196, 237-243 of the reference): the
// sub-layer RMSNorms, the squared-ReLU gate, the residual add.
struct FusedExtras {
    const uint16_t* norm_weight;  // bf16 [K]; nullptr = no RMSNorm in front
    const uint16_t* residual;     // bf16 [M, N]; nullptr = none; out = bf16(residual + bf16(result))
    float eps;
    int glu;                      // 1: x is [M, 2K] = (x1 | x3); h = bf16(bf16(relu(x1)^2) * x3) feeds the norm
    const uint16_t* act_scale;    // PRO 3 only: bf16 [M], the scales of the int8 rows handed in as x
    int32_t* acc_out;             // int32 [M, N] or nullptr: the raw accumulators (parity tests)
};

__device__ __forceinline__ double dpp_sum_f64_row(double v) {
    // adds v over each 16-lane row with the same four lane permutes as above, on both halves of the double
#define BITLINEAR_DPP64(CTRL)                                                                      \
    {                                                                                              \
        const long long bits = __double_as_longlong(v);                                            \
        const int lo = dpp_move<CTRL>((int)(bits & 0xffffffffll)), hi = dpp_move<CTRL>((int)(bits >> 32)); \
        v += __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);                        \
    }
    BITLINEAR_DPP64(0xB1)
    BITLINEAR_DPP64(0x4E)
    BITLINEAR_DPP64(0x141)
    BITLINEAR_DPP64(0x140)
#undef BITLINEAR_DPP64
    return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
    v = dpp_sum_f64_row(v);
    double t = 0.0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const long long bits = __double_as_longlong(v);
        const int lo = __builtin_amdgcn_readlane((int)(bits & 0xffffffffll), 16 * r);
        const int hi = __builtin_amdgcn_readlane((int)(bits >> 32), 16 * r);
        t += __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
    }
    return t;
}

// 8 bf16 (as 4 dwords) -> sum of squares; every square of a bf16 is exact in
// fp32 and the fp64 sum of a few thousand of them is exact for any data whose
// magnitudes span less than 2^24, so the result does not depend on the order
// of the additions.
__device__ __forceinline__ double sumsq8(const uint4& v) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(d[i] << 16), hi = __uint_as_float(d[i] & 0xffff0000u);
        acc += (double)(lo * lo) + (double)(hi * hi);
    }
    return acc;
}

// y = bf16(x * rstd * g) on 8 packed bf16
__device__ __forceinline__ uint4 norm8(const uint4& v, const uint4& g, float rstd) {
    const uint32_t d[4] = {v.x, v.y, v.z, v.w};
    const uint32_t w[4] = {g.x, g.y, g.z, g.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(d[i] << 16) * rstd * __uint_as_float(w[i] << 16);
        const float hi = __uint_as_float(d[i] & 0xffff0000u) * rstd * __uint_as_float(w[i] & 0xffff0000u);
        o[i] = f32x2_to_bf16x2(lo, hi);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// h = bf16(bf16(relu(x1)^2) * x3) on 8 packed bf16
__device__ __forceinline__ uint4 glu8(const uint4& a, const uint4& b) {
    const uint32_t d[4] = {a.x, a.y, a.z, a.w};
    const uint32_t e[4] = {b.x, b.y, b.z, b.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float r0 = fmaxf(__uint_as_float(d[i] << 16), 0.0f), r1 = fmaxf(__uint_as_float(d[i] & 0xffff0000u), 0.0f);
        const uint32_t sq = f32x2_to_bf16x2(r0 * r0, r1 * r1);
        const float s0 = __uint_as_float(sq << 16), s1 = __uint_as_float(sq & 0xffff0000u);
        const float lo = s0 * __uint_as_float(e[i] << 16), hi = s1 * __uint_as_float(e[i] & 0xffff0000u);
        o[i] = f32x2_to_bf16x2(lo, hi);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// ---------------------------------------------------------------------------
// Gate / RMSNorm / absmax quantizer as a kernel of its own: one workgroup per
// token row.  Used in front of the product kernels when the activation block
// is too large for every workgroup of the fused kernel to redo this work.
// Same arithmetic, in the same order, as the PRO 1 / 2 prologue below.
// ---------------------------------------------------------------------------
constexpr int kPreThreads = 512;
constexpr int kPreVecs = 8;  // at most this many 16-byte vectors per thread: rows up to 8 * 512 * 8 = 32768 elements

template <int PRO, int VQ>  // VQ: vectors per thread, VQ * 512 * 8 >= K
__global__ __launch_bounds__(kPreThreads) void norm_quant_kernel(const uint16_t* __restrict__ x,
                                                                 const uint16_t* __restrict__ norm_weight, float eps,
                                                                 int8_t* __restrict__ q, uint16_t* __restrict__ s,
                                                                 int K, int mode) {
    __shared__ uint32_t wmax[kPreThreads / 64];
    __shared__ double wsq[kPreThreads / 64];
    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int nvec = K >> 3;
    const int xstride = PRO == 2 ? 2 * K : K;
    const uint16_t* xr = x + (size_t)row * xstride;

    uint4 xv[VQ], gv[VQ], x3v[PRO == 2 ? VQ : 1];
#pragma unroll
    for (int r = 0; r < VQ; ++r) {
        const int idx = (tid + r * kPreThreads) < nvec ? (tid + r * kPreThreads) : (nvec - 1);
        xv[r] = *(const uint4*)(xr + idx * 8);
        if (PRO == 2) x3v[r] = *(const uint4*)(xr + K + idx * 8);
        gv[r] = *(const uint4*)(norm_weight + idx * 8);
    }
    double sq = 0.0;
#pragma unroll
    for (int r = 0; r < VQ; ++r) {
        if (PRO == 2) xv[r] = glu8(xv[r], x3v[r]);
        if (tid + r * kPreThreads < nvec) sq += sumsq8(xv[r]);
    }
    const double wsum = wave_sum_f64(sq);
    if (lane == 0) wsq[wave] = wsum;
    __syncthreads();
    double total = 0.0;
#pragma unroll
    for (int i = 0; i < kPreThreads / 64; ++i) total += wsq[i];
    const float mean = (float)total / (float)K;
    const float rstd = 1.0f / __builtin_sqrtf(mean + eps);
    uint32_t am = 0;
#pragma unroll
    for (int r = 0; r < VQ; ++r) {
        xv[r] = norm8(xv[r], gv[r], rstd);
        if (tid + r * kPreThreads < nvec) am = absmax_bits8(xv[r], am);
    }
    am = wave_max_u32(am);
    if (lane == 0) wmax[wave] = am;
    __syncthreads();
    am = wmax[0];
#pragma unroll
    for (int i = 1; i < kPreThreads / 64; ++i) am = max(am, wmax[i]);
    const float s32 = mode == 0 ? quant_scale<0>(am) : quant_scale<1>(am);
    if (tid == 0) s[row] = f32_to_bf16_rne(s32);
    uint2* qr = (uint2*)(q + (size_t)row * K);
#pragma unroll
    for (int r = 0; r < VQ; ++r) {
        const int idx = tid + r * kPreThreads;
        if (idx < nvec) qr[idx] = mode == 0 ? quant_vec8<0>(xv[r], s32) : quant_vec8<1>(xv[r], s32);
    }
}

// The same for many rows (a prompt): one wave per row, four rows per workgroup, the row in the wave's registers,
// every reduction a wave reduction (no LDS, no barrier).  Same arithmetic, in the same order, as norm_quant_kernel:
// the fp64 sum of squares is exact, so the order of its additions does not matter.
template <int PRO, int V>  // V: vectors of 8 values per lane, V * 64 * 8 >= K
__global__ __launch_bounds__(256) void norm_quant_rows_kernel(const uint16_t* __restrict__ x,
                                                              const uint16_t* __restrict__ norm_weight, float eps,
                                                              int8_t* __restrict__ q, uint16_t* __restrict__ s, int M,
                                                              int K, int mode) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;  // uniform per wave; nothing below synchronises across waves
    const int nvec = K >> 3;
    const int xstride = PRO == 2 ? 2 * K : K;
    const uint16_t* xr = x + (size_t)row * xstride;
    uint4 xv[V], gv[V], x3v[PRO == 2 ? V : 1];
#pragma unroll
    for (int r = 0; r < V; ++r) {
        const int idx = (lane + r * 64) < nvec ? (lane + r * 64) : (nvec - 1);
        xv[r] = *(const uint4*)(xr + idx * 8);
        if (PRO == 2) x3v[r] = *(const uint4*)(xr + K + idx * 8);
        gv[r] = *(const uint4*)(norm_weight + idx * 8);
    }
    double sq = 0.0;
#pragma unroll
    for (int r = 0; r < V; ++r) {
        if (PRO == 2) xv[r] = glu8(xv[r], x3v[r]);
        if (lane + r * 64 < nvec) sq += sumsq8(xv[r]);
    }
    const double total = wave_sum_f64(sq);
    const float mean = (float)total / (float)K;
    const float rstd = 1.0f / __builtin_sqrtf(mean + eps);
    uint32_t am = 0;
#pragma unroll
    for (int r = 0; r < V; ++r) {
        xv[r] = norm8(xv[r], gv[r], rstd);
        if (lane + r * 64 < nvec) am = absmax_bits8(xv[r], am);
    }
    am = wave_max_u32(am);
    const float s32 = mode == 0 ? quant_scale<0>(am) : quant_scale<1>(am);
    if (lane == 0) s[row] = f32_to_bf16_rne(s32);
    uint2* qr = (uint2*)(q + (size_t)row * K);
#pragma unroll
    for (int r = 0; r < V; ++r) {
        const int idx = lane + r * 64;
        if (idx < nvec) qr[idx] = mode == 0 ? quant_vec8<0>(xv[r], s32) : quant_vec8<1>(xv[r], s32);
    }
}

// PRO 0: plain, 1: RMSNorm in front, 2: squared-ReLU gate + RMSNorm in front,
// 3: x already holds the int8 rows [M, K] (16 per vector) and ex.act_scale their scales: no quantizer
// RES: a residual is added in the epilogue (its values are requested at the start; an instance of
// its own, because loads under a runtime branch would make the compiler wait conservatively later)
template <int UPW, int VMAX, int PRO, bool RES>
__global__ __launch_bounds__(kMaxWaves * 64) void bitlinear_fused_kernel(
    // parameter order: what stands between the kernel's entry and its first loads comes first, in
    // the leading dwords that are handed over in registers at wave start (kernel-argument preload)
    // (aux: the second thing the prologue loads -- ex.norm_weight for PRO 1 and 2, ex.act_scale for PRO 3)
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, int M, int N, int K, int RB, int S, int mode,
    float inv_vec_per_row, const uint16_t* __restrict__ aux, uint16_t* __restrict__ out,
    const uint16_t* __restrict__ ws, ScaleMap smap, int8_t* __restrict__ q_out, uint16_t* __restrict__ s_out,
    FusedExtras ex) {
    extern __shared__ __attribute__((aligned(16))) int8_t lds_q[];  // [M][K + pad]
    __shared__ int red[kFusedMaxRB * 256];
    __shared__ uint32_t amax_bits[kFusedMaxTokens];
    __shared__ int qsum[kFusedMaxTokens];
    __shared__ float sval[kFusedMaxTokens];  // activation scale per token (a bf16 value)
    __shared__ float rinv[kFusedMaxTokens];  // its correctly rounded reciprocal
    __shared__ double sumsq[kFusedMaxTokens];

    // A wave's own instruction stream is the critical path of this kernel (a wave issues roughly one
    // instruction per 4 cycles, and a few hundred of them are most of its lifetime), so everything
    // in front of the first load is kept short: wave-uniform values on the scalar unit, no integer
    // division, no 64-bit address arithmetic.
    const int tid = threadIdx.x;
    // = blockDim.x; where the prologue needs it early (more than one vector per thread) it is taken
    // from arguments that arrive in registers instead of from the hidden arguments (a scalar load)
    const int nthreads = VMAX == 1 ? (int)blockDim.x : 64 * RB * S;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rbl = (wave >= S ? 1 : 0) + (wave >= 2 * S ? 1 : 0) + (wave >= 3 * S ? 1 : 0);  // wave / S, RB <= 4
    const int ks = wave - rbl * S;
    const int rb = blockIdx.x * RB + rbl;
    const bool rows_ok = rb < (N >> 4);
    const int g = lane >> 4;
    const int p = lane & 15;
    const int units = K >> 6;
    const int kp = K + kFusedRowPad;

    const int lane_word = (g >> 1) * 32 + (p >> 3) * 16 + (g & 1) * 8 + (p & 7);
    // Weight words through a buffer descriptor that spans exactly this wave's block of 16 rows
    // (K * 4 contiguous bytes; nothing for a row block past the end): a word of a k-step past
    // the end of K is out of the descriptor's range and reads as zero, which is also the A
    // operand that contributes nothing, so the loads need neither clamping nor masking.  The
    // k-step goes into the instruction's immediate offset, the round into the vector offset.
    // The weights are read once: the non-temporal hint keeps them from displacing the
    // activations and scales that every workgroup re-reads.
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)((const char*)wq + (size_t)(rows_ok ? rb : 0) * K * 4), 0, rows_ok ? K * 4 : 0, 0x00020000);
    int w_voff = lane_word * 4 + ks * (UPW * 256);
#define FUSED_WLOAD(j) (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(w_rsrc, w_voff + (j) * 256, 0, 2 /* nt */)

    // Activation block first: 16-byte vectors of 8 bf16, VMAX per thread.  The
    // memory counter retires loads in issue order, so what is needed first
    // (x) is requested first and the weight words stay outstanding behind it.
    // Loads are unconditional (indices clamped into range, surplus results
    // ignored later): a load under a branch would force a full wait for all
    // earlier loads at the first use of x.  Row and column of a vector come
    // from a multiplication with 1 / vec_per_row (exact: (idx + 0.5) / vec_per_row
    // is at least 0.5 / vec_per_row > 1e-4 away from an integer and below 16, far
    // above the fp32 rounding error of the product).
    const int vec_per_row = PRO == 3 ? K >> 4 : K >> 3;
    const int nvec = M * vec_per_row;
    const int xstride = PRO == 2 ? 2 * K : K;  // elements between token rows of x
    uint4 xv[VMAX], x3v[PRO == 2 ? VMAX : 1], gv[(PRO == 1 || PRO == 2) ? VMAX : 1];
    int vrc[VMAX];  // row << 16 | col of the vector of round v; -1: this thread has none
#pragma unroll
    for (int v = 0; v < VMAX; ++v) {
        const int raw = tid + v * nthreads;
        const int idx = raw < nvec ? raw : (nvec - 1);
        const int row = M == 1 ? 0 : (int)(((float)idx + 0.5f) * inv_vec_per_row);
        const int col = idx - row * vec_per_row;
        vrc[v] = raw < nvec ? (row << 16 | col) : -1;
        if (PRO == 3) {
            xv[v] = *(const uint4*)((const int8_t*)x + idx * 16);          // rows are contiguous
        } else if (PRO == 2) {
            xv[v] = *(const uint4*)(x + row * xstride + col * 8);
            x3v[v] = *(const uint4*)(x + row * xstride + K + col * 8);
        } else {
            xv[v] = *(const uint4*)(x + idx * 8);                            // rows are contiguous
        }
        if (PRO == 1 || PRO == 2) gv[v] = *(const uint4*)(aux + col * 8);
    }
    // PRO 3: the scale of token row tid, raw bits; any other variant re-reads a weight scale and ignores it
    const uint16_t* asp = PRO == 3 ? aux : ws;
    const uint16_t e_as = asp[PRO == 3 ? (tid < M ? tid : M - 1) : 0];
    // weight words of the first round
    uint32_t w[UPW];
#pragma unroll
    for (int j = 0; j < UPW; ++j) w[j] = FUSED_WLOAD(j);
    // Epilogue operands, raw bits, nothing depends on them until the end.  Nearly always all
    // rows of a workgroup share one weight-scale slot (found with scalar arithmetic): one load
    // with a uniform address here; a workgroup that straddles a slot boundary fetches per row in
    // the epilogue.
    constexpr bool kHasRes = RES;
    const int n_first = blockIdx.x * RB * 16;
    const int n_last = (n_first + RB * 16 - 1) < N ? (n_first + RB * 16 - 1) : N - 1;
    const int slot_first = scale_slot_uniform(smap, n_first), slot_last = scale_slot_uniform(smap, n_last);
    const uint16_t wsb_first = ws[slot_first];
    uint16_t e_res[kFusedMaxRB];
    if (kHasRes) {
        // loads through a descriptor of the residual: output slots this thread does not own get an
        // offset past its end, which costs no memory access
        const __amdgpu_buffer_rsrc_t r_rsrc =
            __builtin_amdgcn_make_buffer_rsrc((void*)ex.residual, 0, M * N * 2, 0x00020000);
#pragma unroll
        for (int r = 0; r < kFusedMaxRB; ++r) {
            const int t = tid + r * nthreads;  // output slot t of the workgroup: [row block][reg][lane]
            const int n = (blockIdx.x * RB + (t >> 8)) * 16 + 4 * ((t & 63) >> 4) + ((t >> 6) & 3);
            const int m = t & 15;
            const bool live = t < RB * 256 && m < M && n < N;
            e_res[r] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r_rsrc, live ? (m * N + n) * 2 : 0x7fff0000, 0, 0);
        }
    }

    for (int i = tid; i < RB * 256; i += nthreads) red[i] = 0;
    if (tid < kFusedMaxTokens) {
        amax_bits[tid] = 0u;
        qsum[tid] = 0;
        sumsq[tid] = 0.0;
    }
    lds_barrier();

    if (PRO == 1 || PRO == 2) {
        // gate (PRO 2), then sum of squares per token row, then y = bf16(h * rstd * g)
#pragma unroll
        for (int v = 0; v < VMAX; ++v) {
            const int row = vrc[v] >> 16;
            if (PRO == 2) xv[v] = glu8(xv[v], x3v[v]);
            const double sq = row >= 0 ? sumsq8(xv[v]) : 0.0;
            const int row0 = __builtin_amdgcn_readfirstlane(row);
            if (__builtin_amdgcn_ballot_w64(row != row0) == 0) {
                const double wsum = wave_sum_f64(sq);
                if (lane == 0 && row0 >= 0) atomicAdd(&sumsq[row0], wsum);
            } else if (row >= 0) {
                atomicAdd(&sumsq[row], sq);
            }
        }
        lds_barrier();
#pragma unroll
        for (int v = 0; v < VMAX; ++v) {
            if (vrc[v] >= 0) {
                const float mean = (float)sumsq[vrc[v] >> 16] / (float)K;
                const float rstd = 1.0f / __builtin_sqrtf(mean + ex.eps);
                xv[v] = norm8(xv[v], gv[v], rstd);
            }
        }
    }

    // one LDS atomic per wave and token row where the wave's 64 vectors lie in
    // one row (always so when K/8 is a multiple of 64); per lane otherwise
    if (PRO != 3) {
#pragma unroll
        for (int v = 0; v < VMAX; ++v) {
            const int row = vrc[v] >> 16;
            const uint32_t lm = row >= 0 ? absmax_bits8(xv[v], 0u) : 0u;
            const int row0 = __builtin_amdgcn_readfirstlane(row);
            if (__builtin_amdgcn_ballot_w64(row != row0) == 0) {
                const uint32_t wm = wave_max_u32(lm);
                if (lane == 0 && row0 >= 0) atomicMax(&amax_bits[row0], wm);
            } else if (row >= 0) {
                atomicMax(&amax_bits[row], lm);
            }
        }
        lds_barrier();
    } else if (tid < M) {
        sval[tid] = bf16_to_f32(e_as);
        rinv[tid] = 1.0f / bf16_to_f32(e_as);
    }

#pragma unroll
    for (int v = 0; v < VMAX; ++v) {
        const int idx = tid + v * nthreads;
        const int prow = vrc[v] >> 16, pcol = vrc[v] & 0xffff;
        int part = 0;  // sum of this thread's quantized values
        if (PRO == 3) {
            if (prow >= 0) {
                *(uint4*)(lds_q + prow * kp + pcol * 16) = xv[v];
                const int ones = 0x01010101;
                part = __builtin_amdgcn_sdot4((int)xv[v].x, ones, __builtin_amdgcn_sdot4((int)xv[v].y, ones, 0, false), false);
                part = __builtin_amdgcn_sdot4((int)xv[v].z, ones, __builtin_amdgcn_sdot4((int)xv[v].w, ones, part, false), false);
            }
        } else if (prow >= 0) {
            const int row = prow;
            const int col = pcol;
            const float sf = mode == 0 ? quant_scale<0>(amax_bits[row]) : quant_scale<1>(amax_bits[row]);
            const uint2 qv = mode == 0 ? quant_vec8<0>(xv[v], sf) : quant_vec8<1>(xv[v], sf);
            *(uint2*)(lds_q + row * kp + col * 8) = qv;
            const int ones = 0x01010101;
            part = __builtin_amdgcn_sdot4((int)qv.x, ones, __builtin_amdgcn_sdot4((int)qv.y, ones, 0, false), false);
            if (col == 0) {
                sval[row] = sf;
                rinv[row] = 1.0f / sf;
            }
            if (blockIdx.x == 0) {
                if (q_out) *(uint2*)(q_out + (size_t)idx * 8) = qv;
                if (s_out && col == 0) s_out[row] = f32_to_bf16_rne(sf);
            }
        }
        const int row0 = __builtin_amdgcn_readfirstlane(prow);
        if (__builtin_amdgcn_ballot_w64(prow != row0) == 0) {
            const int wsum = wave_sum_i32(part);
            if (lane == 0 && row0 >= 0) atomicAdd(&qsum[row0], wsum);
        } else if (prow >= 0) {
            atomicAdd(&qsum[prow], part);
        }
    }
    lds_barrier();

    const bool tok_ok = p < M;
    const int8_t* brow = lds_q + (tok_ok ? p : 0) * kp + g * 16;
    v4i acc = {0, 0, 0, 0};
    for (int base = ks * UPW; base < units; base += S * UPW) {
        if (base != ks * UPW) {
            w_voff += S * (UPW * 256);
#pragma unroll
            for (int j = 0; j < UPW; ++j) w[j] = FUSED_WLOAD(j);
        }
        // all B operands of the round first (independent LDS reads, one wait);
        // a k-step past the end contributes nothing because its A operand is zero:
        // its B operand is whatever follows in LDS (the next token's row or the
        // tail padding of the allocation), read without clamping
        v4i b[UPW];
#pragma unroll
        for (int j = 0; j < UPW; ++j) b[j] = *(const v4i*)(brow + (base + j) * 64);
#pragma unroll
        for (int j = 0; j < UPW; ++j) {
            const uint32_t wj = w[j];  // zero past the end of K
            v4i a;
            a.x = (int)(wj & 0x03030303u);
            a.y = (int)((wj >> 2) & 0x03030303u);
            a.z = (int)((wj >> 4) & 0x03030303u);
            a.w = (int)((wj >> 6) & 0x03030303u);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[j], acc, 0, 0, 0);
        }
    }

    if (tok_ok) {  // lane holds token p, rows 4g + i in register i
        int* dst = red + rbl * 256 + lane;
        atomicAdd(dst, acc.x);
        atomicAdd(dst + 64, acc.y);
        atomicAdd(dst + 128, acc.z);
        atomicAdd(dst + 192, acc.w);
    }
    lds_barrier();

    // Division by the token's scale as in the GEMM: q0 = a * (1/s) refined by
    // e = fma(-q0, s, a), q = fma(e, 1/s, q0) -- the same bits as the IEEE divide
    // for these integer-valued a, at a third of the instructions.
#pragma unroll
    for (int r = 0; r < kFusedMaxRB; ++r) {
        const int t = tid + r * nthreads;
        if (t >= RB * 256) break;
        const int l = t & 63;
        const int m = l & 15;
        const int n = (blockIdx.x * RB + (t >> 8)) * 16 + 4 * (l >> 4) + ((t >> 6) & 3);
        if (m < M && n < N) {
            uint16_t wsb = wsb_first;
            if (slot_first != slot_last) wsb = ws[scale_slot(smap, n)];  // uniform branch, rare
            const int acc_i = red[t] - 2 * qsum[m];
            if (ex.acc_out) ex.acc_out[(size_t)m * N + n] = acc_i;  // uniform branch: parity tests only
            const float a = (float)acc_i;
            const float sv = sval[m], ri = rinv[m];
            const float q0 = a * ri;
            const float q = __builtin_fmaf(__builtin_fmaf(-q0, sv, a), ri, q0);
            uint16_t o = f32_to_bf16_rne(q * bf16_to_f32(wsb));
            if (kHasRes) o = f32_to_bf16_rne(bf16_to_f32(e_res[r]) + bf16_to_f32(o));
            if (out) out[(size_t)m * N + n] = o;  // uniform: the accumulator-only call has no output
        }
    }
}

// ---------------------------------------------------------------------------
// BitLinearKernel.forward for one to four tokens with waves that prepare their own operands
// ---------------------------------------------------------------------------
// Same decomposition as bitlinear_fused_kernel (a workgroup owns RB 16-row blocks, S waves split K
// for each, one packed word per lane and k-step is the MFMA's row operand) but no wave waits for
// another before its products are done: every wave takes the row maximum of the activation rows
// itself (the whole rows, a few KB that every wave of the machine reads from cache: redundant work,
// but no workgroup-wide reduction, no LDS atomics and no barrier in front of the products),
// quantizes only the slice of k that its own k-steps multiply, and hands it to itself through a
// private LDS region.  The +2 of the stored codes is removed per wave with the sum of its own slice.
// One barrier, behind the products: the waves' partial tiles are added by the threads that finish
// the outputs.  A wave's instruction stream is what a call of this size costs, and this one is
// about half as long as the shared-prologue kernel's.
constexpr int kSoloMaxTokens = 4;
constexpr int kSoloRedSlots = 32;  // partial tiles a workgroup keeps (one token; 16 with more): row blocks x waves per row block
constexpr int kSoloMaxUPW = 8;  // at most 8 k-steps (512 k = 64 vectors of 8 values) per wave: one slice vector per lane

// COOP: the row maximum is taken over the workgroup's slices and exchanged through LDS (one barrier more,
// no redundant reads of the rows): for rows too long for every wave to scan them
// PRO 1: RMSNorm in front of the quantizer (aux = its weights), 2: squared-ReLU gate, then the RMSNorm (x holds
// [M, 2K] = (x1 | x3)); both with the sums of squares exchanged like the maxima (COOP only, one more barrier).
// RES: out = bf16(residual + bf16(result)).  The arithmetic is that of bitlinear_fused_kernel's prologues.
// RPW: 16-row blocks per wave.  A wave multiplies its slice with the words of RPW consecutive row blocks: the
// slice is prepared once for all of them (with many row blocks the preparation, repeated in every wave of the
// machine, is what the vector units spend their time on).
template <int UPW, int VROW, int MT, bool COOP, int PRO, bool RES, int RPW>
__global__ __launch_bounds__(kMaxWaves * 64) void bitlinear_solo_kernel(
    // parameter order: what stands between the kernel's entry and its first loads comes first
    // (the weight scales' slots are at most eight runs of slot_rows output rows each, run j reading entry
    // (slot_map >> 3 j) & 7 of ws: the reference's rule n / (N / ws_num) is the identity map, a fused q/k/v
    // matrix with its true segments of 2560 / 640 / 640 rows is six runs of 640 reading 0 0 0 0 1 2; two
    // integers among the leading arguments instead of a table behind them, the map in the upper bits of rb_map)
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, int M, int N, int K, int rb_map, int S, int slot_rows,
    const uint16_t* __restrict__ aux, const uint16_t* __restrict__ ws, uint16_t* __restrict__ out,
    const uint16_t* __restrict__ residual, float eps, int8_t* __restrict__ q_out, uint16_t* __restrict__ s_out,
    int32_t* __restrict__ acc_out) {
    static_assert(PRO == 0 || COOP, "the norm prologues exchange their partial sums between the waves");
    __shared__ __attribute__((aligned(16))) int8_t lds_q[kMaxWaves][MT][kSoloMaxUPW * 64];  // a wave's quantized slice per token
    __shared__ __attribute__((aligned(16))) int red[MT == 1 ? kSoloRedSlots : kMaxWaves][256];                    // a wave's partial 16 x 16 tiles, [row block * S + k slice]
    __shared__ uint32_t wmax[kMaxWaves][MT];                                                // COOP: a wave's slice maximum per token
    __shared__ double wsq[PRO ? kMaxWaves : 1][MT];                                         // PRO 1, 2: a wave's slice sum of squares per token
    const int RB = rb_map & 0xff;                      // row blocks per workgroup
    const uint32_t slot_map = (uint32_t)rb_map >> 8;   // run j of slot_rows output rows reads ws[(slot_map >> 3 j) & 7]
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rbl = (wave >= S ? 1 : 0) + (wave >= 2 * S ? 1 : 0) + (wave >= 3 * S ? 1 : 0);  // wave / S, RB <= 4
    const int ks = wave - rbl * S;
    const int rb = (blockIdx.x * RB + rbl) * RPW;  // the wave's first row block
    const int g = lane >> 4;
    const int p = lane & 15;

    // requests, all at once: the slice's vectors (needed last, but they are part of the rows and
    // return with them), the whole rows for the maximum, then the weight words
    const int xstride = PRO == 2 ? 2 * K : K;  // elements between token rows of x
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * xstride * 2, 0x00020000);
    const int slice_k0 = ks * (UPW * 64);
    const bool slice_lane = lane < UPW * 8 && slice_k0 + lane * 8 < K;
    uint4 sv[MT];
    uint4 s3[PRO == 2 ? MT : 1];
    uint4 rv[MT][VROW];
    uint4 gvec = make_uint4(0u, 0u, 0u, 0u);
    if (PRO != 0) {
        const __amdgpu_buffer_rsrc_t g_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)aux, 0, K * 2, 0x00020000);
        gvec = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, slice_lane ? (slice_k0 + lane * 8) * 2 : 0x7ffffff0, 0, 0));
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int row_off = (m < M ? m : M - 1) * xstride * 2;
        // a lane without a slice vector, or a vector past the end of the row, asks past the end of the buffer: zeros, no access
        sv[m] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                                              x_rsrc, slice_lane ? row_off + (slice_k0 + lane * 8) * 2 : 0x7ffffff0, 0, 0));
        if (PRO == 2)
            s3[m] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                                                  x_rsrc, slice_lane ? row_off + (K + slice_k0 + lane * 8) * 2 : 0x7ffffff0, 0, 0));
        if (!COOP) {
#pragma unroll
            for (int v = 0; v < VROW; ++v) {
                const int k = (lane + v * 64) * 8;
                rv[m][v] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, k < K ? row_off + k * 2 : 0x7ffffff0, 0, 0));
            }
        }
    }
    const int lane_word = (g >> 1) * 32 + (p >> 3) * 16 + (g & 1) * 8 + (p & 7);
    // one descriptor per row block, spanning exactly its K * 4 bytes: a k-step past the end of K reads as zero
    const int w_voff = lane_word * 4 + ks * (UPW * 256);
    uint32_t w[RPW][UPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const bool rows_ok = rb + i < (N >> 4);
        const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)((const char*)wq + (size_t)(rows_ok ? rb + i : 0) * K * 4), 0, rows_ok ? K * 4 : 0, 0x00020000);
#pragma unroll
        for (int j = 0; j < UPW; ++j) w[i][j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(w_rsrc, w_voff + j * 256, 0, 2 /* nt */);
    }
    // epilogue operand, raw bits: the weight scale of the workgroup's first row (a workgroup that
    // straddles a slot boundary fetches per row in the epilogue); the slot by a few scalar
    // comparisons (at most six slots), so that this request leaves with the others
    const int n_first = blockIdx.x * RB * RPW * 16;
    const int n_last = (n_first + RB * RPW * 16 - 1) < N ? (n_first + RB * RPW * 16 - 1) : N - 1;
    int slot_first = 0, slot_last = 0;
#pragma unroll
    for (int j = 1; j < kMaxSeg; ++j) {
        slot_first += n_first >= j * slot_rows ? 1 : 0;
        slot_last += n_last >= j * slot_rows ? 1 : 0;
    }
    const uint16_t wsb_first = ws[(slot_map >> (3 * slot_first)) & 7u];
    const int nthreads = 64 * RB * S;
    uint16_t e_res[kFusedMaxRB];
    if (RES) {
        // the residual values of the output slots this thread will finish; slots it does not own get an
        // offset past the end of the descriptor, which costs no memory access
        const __amdgpu_buffer_rsrc_t r_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)residual, 0, M * N * 2, 0x00020000);
#pragma unroll
        for (int r = 0; r < kFusedMaxRB; ++r) {
            const int t = tid + r * nthreads;
            const int n = (blockIdx.x * RB * RPW + (t >> 8)) * 16 + 4 * ((t & 63) >> 4) + ((t >> 6) & 3);
            const int m = t & 15;
            const bool live = t < RB * RPW * 256 && m < M && n < N;
            e_res[r] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r_rsrc, live ? (m * N + n) * 2 : 0x7fff0000, 0, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every request above is on its way before anything below is looked at

    if (PRO != 0) {
        // gate (PRO 2), the slices' sums of squares exchanged (fp64: exact, so the order of the additions does
        // not matter), then y = bf16(h * rstd * g) on the wave's own slice
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (PRO == 2) sv[m] = glu8(sv[m], s3[m]);
            const double wsum = wave_sum_f64(sumsq8(sv[m]));  // lanes without a slice vector hold zeros
            if (lane == 0) wsq[wave][m] = wsum;
        }
        lds_barrier();
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            double total = 0.0;
            for (int k = 0; k < S; ++k) total += wsq[rbl * S + k][m];
            const float mean = (float)total / (float)K;
            const float rstd = 1.0f / __builtin_sqrtf(mean + eps);
            sv[m] = norm8(sv[m], gvec, rstd);
        }
    }

    // row maxima -> scales; this wave's slice -> int8 in its LDS region, with the slice's sum
    float sf[MT];
    int qsum2[MT];  // twice the sum of the slice's int8 values
    if (COOP) {
        // the S waves of a row block cover all of K between them: their slice maxima make the row maximum
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t am = wave_max_u32(absmax_bits8(sv[m], 0u));
            if (lane == 0) wmax[wave][m] = am;
        }
        lds_barrier();
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        uint32_t am = 0;
        if (COOP) {
            for (int k = 0; k < S; ++k) am = max(am, wmax[rbl * S + k][m]);
        } else {
#pragma unroll
            for (int v = 0; v < VROW; ++v) am = absmax_bits8(rv[m][v], am);
            am = wave_max_u32(am);
        }
        sf[m] = quant_scale<0>(am);
        const uint2 qv = quant_vec8<0>(sv[m], sf[m]);  // zeros for a lane without a slice vector
        if (lane < UPW * 8) *(uint2*)(&lds_q[wave][m][lane * 8]) = qv;
        const int ones = 0x01010101;
        const int part = __builtin_amdgcn_sdot4((int)qv.x, ones, __builtin_amdgcn_sdot4((int)qv.y, ones, 0, false), false);
        qsum2[m] = 2 * wave_sum_i32(part);
        if (blockIdx.x == 0 && rbl == 0 && m < M) {
            if (q_out && slice_lane) *(uint2*)(q_out + (size_t)m * K + slice_k0 + lane * 8) = qv;
            if (s_out && ks == 0 && lane == 0) s_out[m] = f32_to_bf16_rne(sf[m]);
        }
    }
    // the same wave wrote and reads: LDS operations of a wave complete in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // products: B operand = 16 int8 of token p for the 16 k of chunk g (columns of tokens >= M repeat the last token and are never read)
    const int8_t* brow = &lds_q[wave][p < MT ? (p < M ? p : M - 1) : 0][g * 16];
    v4i b[UPW];
#pragma unroll
    for (int j = 0; j < UPW; ++j) b[j] = *(const v4i*)(brow + j * 64);
    // lane holds token p, rows 4 g + i in register i; the +2 of the codes goes with the slice's sum
    int q2 = qsum2[0];
#pragma unroll
    for (int m = 1; m < MT; ++m) q2 = p == m ? qsum2[m] : q2;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        v4i acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < UPW; ++j) {
            const uint32_t wj = w[i][j];  // zero past the end of K
            v4i e;
            e.x = (int)(wj & 0x03030303u);
            e.y = (int)((wj >> 2) & 0x03030303u);
            e.z = (int)((wj >> 4) & 0x03030303u);
            e.w = (int)((wj >> 6) & 0x03030303u);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(e, b[j], acc, 0, 0, 0);
        }
        int* dst = &red[(rbl * RPW + i) * S + ks][lane];
        dst[0] = acc.x - q2;
        dst[64] = acc.y - q2;
        dst[128] = acc.z - q2;
        dst[192] = acc.w - q2;
    }
    lds_barrier();

    // every thread finishes the output slots t = tid, tid + nthreads, ... of the workgroup: [row block][reg][lane]
#pragma unroll
    for (int r = 0; r < kFusedMaxRB; ++r) {
        const int t = tid + r * nthreads;
        if (t >= RB * RPW * 256) break;
        const int l = t & 63;
        const int m = l & 15;
        const int tb = t >> 8;  // row block of the slot
        const int n = (blockIdx.x * RB * RPW + tb) * 16 + 4 * (l >> 4) + ((t >> 6) & 3);
        if (m < M && n < N) {
            int sum = 0;
            for (int k = 0; k < S; ++k) sum += red[tb * S + k][t & 255];
            if (acc_out) acc_out[(size_t)m * N + n] = sum;  // uniform: parity tests only
            float sv_ = sf[0];
#pragma unroll
            for (int mm = 1; mm < MT; ++mm) sv_ = m == mm ? sf[mm] : sv_;
            uint16_t wsb = wsb_first;
            if (slot_first != slot_last) wsb = ws[(slot_map >> (3 * (n / slot_rows))) & 7u];  // uniform branch, rare
            uint16_t o = f32_to_bf16_rne((float)sum / sv_ * bf16_to_f32(wsb));
            if (RES) o = f32_to_bf16_rne(bf16_to_f32(e_res[r]) + bf16_to_f32(o));
            if (out) out[(size_t)m * N + n] = o;
        }
    }
}

// ---------------------------------------------------------------------------
// The drop-in product (int8 rows in, up to 16 tokens) in the same decomposition: no staging at all
// ---------------------------------------------------------------------------
// A workgroup owns RB x RPW 16-row blocks, S waves split K, every wave multiplies exactly UPW k-steps
// (bitlinear_solo_kernel's launch shapes).  The activation operand of a k-step -- 16 int8 of token p
// for the 16 k of chunk g, p = lane % 16, g = lane / 16 -- is one 16-byte load per lane straight from
// the caller's rows, requested together with the weight words: nothing passes through LDS before the
// products and no wave waits for another.  The +2 of the stored codes leaves with a second product
// per k-step whose row operand is all ones (sum_k a[p, k] in every row of the tile), shared by the
// wave's row blocks.  One barrier, behind the products, as in bitlinear_solo_kernel.
template <int UPW, int RPW, bool RES>
__global__ __launch_bounds__(kMaxWaves * 64) void gemv_i2_solo_kernel(
    const int8_t* __restrict__ act, const uint32_t* __restrict__ wq, int M, int N, int K, int rb_map, int S, int slot_rows,
    const uint16_t* __restrict__ s, const uint16_t* __restrict__ ws, uint16_t* __restrict__ out,
    const uint16_t* __restrict__ residual, int32_t* __restrict__ acc_out) {
    __shared__ __attribute__((aligned(16))) int red[kSoloRedSlots][256];  // partial 16 x 16 tiles, [row block * S + k slice]
    const int RB = rb_map & 0xff;                      // row blocks per workgroup
    const uint32_t slot_map = (uint32_t)rb_map >> 8;   // run j of slot_rows output rows reads ws[(slot_map >> 3 j) & 7]
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rbl = (wave >= S ? 1 : 0) + (wave >= 2 * S ? 1 : 0) + (wave >= 3 * S ? 1 : 0);  // wave / S, RB <= 4
    const int ks = wave - rbl * S;
    const int rb = (blockIdx.x * RB + rbl) * RPW;  // the wave's first row block
    const int g = lane >> 4;
    const int p = lane & 15;

    // requests: the slice's activation operands (a token past M, or a k-step past the end of K, asks past
    // the end of the descriptor: zeros, no access), then the weight words, then what the epilogue needs
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)act, 0, M * K, 0x00020000);
    const int slice_k0 = ks * (UPW * 64);
    v4i b[UPW];
#pragma unroll
    for (int j = 0; j < UPW; ++j) {
        const bool live = p < M && slice_k0 + j * 64 < K;  // K % 64 == 0: a k-step is inside K or outside
        b[j] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, live ? p * K + slice_k0 + j * 64 + g * 16 : 0x7ffffff0, 0, 0);
    }
    const int lane_word = (g >> 1) * 32 + (p >> 3) * 16 + (g & 1) * 8 + (p & 7);
    const int w_voff = lane_word * 4 + ks * (UPW * 256);
    uint32_t w[RPW][UPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        // one descriptor per row block, spanning exactly its K * 4 bytes: a k-step past the end of K reads as zero
        const bool rows_ok = rb + i < (N >> 4);
        const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)((const char*)wq + (size_t)(rows_ok ? rb + i : 0) * K * 4), 0, rows_ok ? K * 4 : 0, 0x00020000);
#pragma unroll
        for (int j = 0; j < UPW; ++j) w[i][j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(w_rsrc, w_voff + j * 256, 0, 2 /* nt */);
    }
    const int n_first = blockIdx.x * RB * RPW * 16;
    const int n_last = (n_first + RB * RPW * 16 - 1) < N ? (n_first + RB * RPW * 16 - 1) : N - 1;
    int slot_first = 0, slot_last = 0;
#pragma unroll
    for (int j = 1; j < kMaxSeg; ++j) {
        slot_first += n_first >= j * slot_rows ? 1 : 0;
        slot_last += n_last >= j * slot_rows ? 1 : 0;
    }
    const uint16_t wsb_first = ws[(slot_map >> (3 * slot_first)) & 7u];
    const uint16_t e_sb = s[(tid & 15) < M ? (tid & 15) : M - 1];  // every output slot of a thread belongs to token tid % 16
    const int nthreads = 64 * RB * S;
    uint16_t e_res[kFusedMaxRB];
    if (RES) {
        const __amdgpu_buffer_rsrc_t r_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)residual, 0, M * N * 2, 0x00020000);
#pragma unroll
        for (int r = 0; r < kFusedMaxRB; ++r) {
            const int t = tid + r * nthreads;
            const int n = (blockIdx.x * RB * RPW + (t >> 8)) * 16 + 4 * ((t & 63) >> 4) + ((t >> 6) & 3);
            const int m = t & 15;
            const bool live = t < RB * RPW * 256 && m < M && n < N;
            e_res[r] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r_rsrc, live ? (m * N + n) * 2 : 0x7fff0000, 0, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every request above is on its way before anything below is looked at

    // sum_k a[p, k] over the slice, in the accumulator layout (every row of the tile holds it)
    const int ones_w = 0x01010101;
    const v4i ones = {ones_w, ones_w, ones_w, ones_w};
    v4i asum = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < UPW; ++j) asum = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, b[j], asum, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        v4i acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < UPW; ++j) {
            const uint32_t wj = w[i][j];  // zero past the end of K
            v4i e;
            e.x = (int)(wj & 0x03030303u);
            e.y = (int)((wj >> 2) & 0x03030303u);
            e.z = (int)((wj >> 4) & 0x03030303u);
            e.w = (int)((wj >> 6) & 0x03030303u);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(e, b[j], acc, 0, 0, 0);
        }
        // lane holds token p, rows 4 g + i in register i
        int* dst = &red[(rbl * RPW + i) * S + ks][lane];
        dst[0] = acc.x - 2 * asum.x;
        dst[64] = acc.y - 2 * asum.y;
        dst[128] = acc.z - 2 * asum.z;
        dst[192] = acc.w - 2 * asum.w;
    }
    lds_barrier();

    // every thread finishes the output slots t = tid, tid + nthreads, ... of the workgroup: [row block][reg][lane]
    const float sf = bf16_to_f32(e_sb);
#pragma unroll
    for (int r = 0; r < kFusedMaxRB; ++r) {
        const int t = tid + r * nthreads;
        if (t >= RB * RPW * 256) break;
        const int l = t & 63;
        const int m = l & 15;
        const int tb = t >> 8;  // row block of the slot
        const int n = (blockIdx.x * RB * RPW + tb) * 16 + 4 * (l >> 4) + ((t >> 6) & 3);
        if (m < M && n < N) {
            int sum = 0;
            for (int k = 0; k < S; ++k) sum += red[tb * S + k][t & 255];
            if (acc_out) acc_out[(size_t)m * N + n] = sum;  // uniform: parity tests only
            uint16_t wsb = wsb_first;
            if (slot_first != slot_last) wsb = ws[(slot_map >> (3 * (n / slot_rows))) & 7u];  // uniform branch, rare
            uint16_t o = f32_to_bf16_rne((float)sum / sf * bf16_to_f32(wsb));
            if (RES) o = f32_to_bf16_rne(bf16_to_f32(e_res[r]) + bf16_to_f32(o));
            if (out) out[(size_t)m * N + n] = o;
        }
    }
}

// ---------------------------------------------------------------------------
// BitLinearKernel.forward for up to eight tokens in one launch: every lane quantizes for its own token
// ---------------------------------------------------------------------------
// gemv_i2_solo_kernel's decomposition (a workgroup owns RPW 16-row blocks, S waves split K, UPW k-steps per
// wave) with the quantizer in front of the products inside the wave.  The activation operand of a k-step is
// 16 int8 of token p = lane % 16 for the 16 k of chunk g = lane / 16, and that is also how the bf16 rows are
// read: lanes p and p + 8 share token p % 8 and load 8 of the 16 values behind that operand each, swapped with
// one rotation inside the 16-lane row per register.  The tokens are quantized side by side, so a call with
// eight tokens runs about the instructions of a call with one, and nothing passes through LDS in front of
// the products but a token's slice maxima, exchanged between the waves behind one barrier.  Arithmetic,
// rounding points and the +2 of the codes as in bitlinear_solo_kernel and gemv_i2_solo_kernel.
// Measured per call against the quantizer kernel + gemv_i2_solo_kernel (HIP graph of dependent launches, distinct
// weights): 3840 x 2560 at 5 / 8 tokens 4.80 -> 4.21 / 5.51 -> 4.59 us, 2560 x 2560 4.49 -> 4.15 / 5.39 -> 4.55,
// 13824 x 2560 5.83 -> 5.56 / 6.61 -> 5.91.  Variants measured and left out: sixteen values per lane for nine to
// sixteen tokens (twice the quantizer instructions per wave: 5.74 -> 5.79 at 12 tokens, 5.90 -> 6.64 at 16), rows
// of 6912 values (16 waves of 7 k-steps: 7.42 -> 8.65 at 8 tokens), and the RMSNorm / gate prologues in front
// (fp64 sums of squares per lane and a second exchange: 5.79 -> 5.72 at 8 tokens, level with the two launches).
constexpr int kTokMaxTokens = 8;

__device__ __forceinline__ uint32_t token_max_u32(uint32_t v) {
    v = max(v, (uint32_t)__shfl_xor((int)v, 16));
    v = max(v, (uint32_t)__shfl_xor((int)v, 32));
    return max(v, (uint32_t)dpp_move<0x128>((int)v));  // row_ror:8: the lane with the token's other half
}

template <int UPW, int RPW>
__global__ __launch_bounds__(kMaxWaves * 64) void bitlinear_solo_tok_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ wq, int M, int N, int K, int rb_map, int S, int slot_rows,
    const uint16_t* __restrict__ ws, uint16_t* __restrict__ out, int8_t* __restrict__ q_out, uint16_t* __restrict__ s_out,
    int32_t* __restrict__ acc_out) {
    __shared__ __attribute__((aligned(16))) int red[kSoloRedSlots][256];  // partial 16 x 16 tiles, [row block * S + k slice]
    __shared__ uint32_t wmax[kMaxWaves][kTokMaxTokens];                   // a wave's slice maximum per token
    const uint32_t slot_map = (uint32_t)rb_map >> 8;  // run j of slot_rows output rows reads ws[(slot_map >> 3 j) & 7]
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int ks = __builtin_amdgcn_readfirstlane(tid >> 6);  // one group of waves per workgroup: the wave is the k slice
    const int rb = blockIdx.x * RPW;                          // the wave's first row block
    const int g = lane >> 4;
    const int p = lane & 15;
    const int tk = p & 7;     // the token this lane prepares
    const int half = p >> 3;  // which 8 of the chunk's 16 values

    // requests, all at once: the lane's vectors of its token's row (a token past M, or a k-step past the end of
    // K, asks past the end of the descriptor: zeros, no access), then the weight words
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00020000);
    const int slice_k0 = ks * (UPW * 64);
    const int lane_k = slice_k0 + g * 16 + half * 8;
    uint4 sv[UPW];
#pragma unroll
    for (int j = 0; j < UPW; ++j) {
        const int k = lane_k + j * 64;
        const bool live = tk < M && k < K;  // K % 64 == 0: a k-step is inside K or outside
        sv[j] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, live ? (tk * K + k) * 2 : 0x7ffffff0, 0, 0));
    }
    const int lane_word = (g >> 1) * 32 + (p >> 3) * 16 + (g & 1) * 8 + (p & 7);
    const int w_voff = lane_word * 4 + ks * (UPW * 256);
    uint32_t w[RPW][UPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        // one descriptor per row block, spanning exactly its K * 4 bytes: a k-step past the end of K reads as zero
        const bool rows_ok = rb + i < (N >> 4);
        const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)((const char*)wq + (size_t)(rows_ok ? rb + i : 0) * K * 4), 0, rows_ok ? K * 4 : 0, 0x00020000);
#pragma unroll
        for (int j = 0; j < UPW; ++j) w[i][j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(w_rsrc, w_voff + j * 256, 0, 2 /* nt */);
    }
    const int n_first = blockIdx.x * RPW * 16;
    const int n_last = (n_first + RPW * 16 - 1) < N ? (n_first + RPW * 16 - 1) : N - 1;
    int slot_first = 0, slot_last = 0;
#pragma unroll
    for (int j = 1; j < kMaxSeg; ++j) {
        slot_first += n_first >= j * slot_rows ? 1 : 0;
        slot_last += n_last >= j * slot_rows ? 1 : 0;
    }
    const uint16_t wsb_first = ws[(slot_map >> (3 * slot_first)) & 7u];
    const int nthreads = 64 * S;
    __builtin_amdgcn_sched_barrier(0);  // every request above is on its way before anything below is looked at

    // row maxima -> scales: the S waves cover all of K between them
    uint32_t am = 0;
#pragma unroll
    for (int j = 0; j < UPW; ++j) am = absmax_bits8(sv[j], am);
    am = token_max_u32(am);
    if (lane < kTokMaxTokens) wmax[ks][lane] = am;
    lds_barrier();
    am = 0;
    for (int k = 0; k < S; ++k) am = max(am, wmax[k][tk]);
    const float sf = quant_scale<0>(am);

    // the lane's values -> int8 -> the MFMA's activation operands, in registers: lanes p < 8 hold values 0..7 of
    // the chunk and fetch 8..15 from lane p + 8; the columns p >= 8 of the product belong to no token and are
    // never read
    v4i b[UPW];
#pragma unroll
    for (int j = 0; j < UPW; ++j) {
        const uint2 qv = quant_vec8<0>(sv[j], sf);
        const int k = lane_k + j * 64;
        if (blockIdx.x == 0 && q_out && tk < M && k < K) *(uint2*)(q_out + (size_t)tk * K + k) = qv;
        b[j] = v4i{(int)qv.x, (int)qv.y, dpp_move<0x128>((int)qv.x), dpp_move<0x128>((int)qv.y)};
    }
    if (blockIdx.x == 0 && s_out && ks == 0 && lane < kTokMaxTokens && tk < M) s_out[tk] = f32_to_bf16_rne(sf);

    // sum_k a[p, k] over the slice, in the accumulator layout (every row of the tile holds it)
    const int ones_w = 0x01010101;
    const v4i ones = {ones_w, ones_w, ones_w, ones_w};
    v4i asum = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < UPW; ++j) asum = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, b[j], asum, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        v4i acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < UPW; ++j) {
            const uint32_t wj = w[i][j];  // zero past the end of K
            v4i e;
            e.x = (int)(wj & 0x03030303u);
            e.y = (int)((wj >> 2) & 0x03030303u);
            e.z = (int)((wj >> 4) & 0x03030303u);
            e.w = (int)((wj >> 6) & 0x03030303u);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(e, b[j], acc, 0, 0, 0);
        }
        // lane holds token p, rows 4 g + i in register i
        int* dst = &red[i * S + ks][lane];
        dst[0] = acc.x - 2 * asum.x;
        dst[64] = acc.y - 2 * asum.y;
        dst[128] = acc.z - 2 * asum.z;
        dst[192] = acc.w - 2 * asum.w;
    }
    lds_barrier();

    // every thread finishes the output slots t = tid, tid + nthreads, ... of the workgroup: [row block][reg][lane];
    // a slot's token is t % 16 = p, and for every token there is (p < 8) that is the token whose scale the lane holds
#pragma unroll
    for (int r = 0; r < kFusedMaxRB; ++r) {
        const int t = tid + r * nthreads;
        if (t >= RPW * 256) break;
        const int l = t & 63;
        const int m = l & 15;
        const int tb = t >> 8;  // row block of the slot
        const int n = (blockIdx.x * RPW + tb) * 16 + 4 * (l >> 4) + ((t >> 6) & 3);
        if (m < M && n < N) {
            int sum = 0;
            for (int k = 0; k < S; ++k) sum += red[tb * S + k][t & 255];
            if (acc_out) acc_out[(size_t)m * N + n] = sum;  // uniform: parity tests only
            uint16_t wsb = wsb_first;
            if (slot_first != slot_last) wsb = ws[(slot_map >> (3 * (n / slot_rows))) & 7u];  // uniform branch, rare
            if (out) out[(size_t)m * N + n] = f32_to_bf16_rne((float)sum / sf * bf16_to_f32(wsb));
        }
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
thread_local int g_status = BITLINEAR_OK;
// name of the product kernel the calling thread's most recent call launched (tests and the smoke
// check report which kernel they exercised)
thread_local const char* g_last_kernel = "none";
// Launch-shape overrides (bitlinear_set_tuning).  The process-wide copy is guarded by a mutex; every
// entry point takes one snapshot of it into the calling thread's own copy before it plans a launch,
// so a call never sees half of another thread's update.
struct Tuning {
    int waves = 0;
    int upw = 0;
    int path = 0;  // 0 = built-in choice, 2 = split-K kernel, 3 = fused shape, 4 = never fuse, 5 = GEMM tile
    int fused[3] = {1, 10, 4};
    int prefill_big = 0;
    int prefill_band = 0;  // row tiles per band of the prefill GEMM's tile order, 0 = built-in choice
    int prefill_ks = 0;    // groups of waves splitting K in the small prefill tiles, 0 = built-in choice
    int staged = 0;        // product through the LDS-staged kernel: 0 = built-in choice, 1 = whenever it fits, 2 = never
    int stream = 0;        // product through the streaming kernel: 0 = built-in choice, 1 = whenever it applies, 2 = never
    int stream_depth = 0;  // its ring depth (0 = built-in choice)
    int stream_waves = 0;  // its waves per CU (0 = built-in choice)
    int solo = 0;          // forward through the kernel whose waves prepare their own operands: 0 = built-in choice, 1..4 = always,
                           // with that many row blocks per workgroup, 5 = never
    int solo_s = 0, solo_upw = 0;  // its waves per row block and k-steps per wave when forced
    int solo_coop = 0;             // row maximum: 0 = built-in choice, 1 = exchanged between the waves, 2 = every wave scans the rows
    int solo_rpw = 0;              // row blocks per wave: 0 = built-in choice, 1, 2, 4
    int prod_solo = 0;             // the drop-in product through gemv_i2_solo_kernel: 0 = built-in choice, 1 = always (prod_s waves of prod_upw k-steps), 2 = never
    int prod_s = 0, prod_upw = 0;
    int tok = 0;  // forward for up to 8 tokens through bitlinear_solo_tok_kernel: 0 = built-in choice (from 5 tokens), 1 = wherever an instance exists, 2 = never
};
std::mutex g_tuning_mutex;
Tuning g_tuning_shared;
thread_local Tuning t_tune;
void refresh_tuning() {
    std::lock_guard<std::mutex> lock(g_tuning_mutex);
    t_tune = g_tuning_shared;
}

using bitnet_host::OncePerDevice;
// ---------------------------------------------------------------------------
// Every crossover of the dispatch code below, in one place.  Each value is where two kernels (or two launch
// shapes of one kernel) measured level on an MI355X, per call from a HIP graph of dependent launches over
// distinct weights; the figures that set it stand beside it.  bitlinear_plan_name() reports what these rules
// choose for a given (entry, M, N, K); tests/test_dispatch_plan.py pins the choice over a grid of shapes, so
// that a changed value shows up as a changed row of that table.
// ---------------------------------------------------------------------------
namespace dispatch {
// --- which kernel -----------------------------------------------------------
// tokens above which the product is the MFMA GEMM instead of a GEMV kernel (the GEMV kernels hold at most 16
// tokens: one MFMA column block)
constexpr int kPrefillMinTokens = 16;
// bitlinear_forward_bf16 from this many tokens up to eight (rows of up to 3200 values) in one launch through
// bitlinear_solo_tok_kernel; below, the kernels for one to four tokens are ahead (3840 x 2560 at 4 tokens 4.14 us
// against 4.24; at 5 tokens 4.80 against 4.21)
constexpr int kTokMinTokens = 5;
// ... and rows of up to this many values (waves of five k-steps, at most ten of them; 2560 x 6912 with 16 waves of
// seven k-steps measured 7.42 us against 8.65 through this kernel at 8 tokens)
constexpr int kTokMaxK = 3200;
// ... and at most one workgroup per CU (3200 x 3200, 200 workgroups, at 8 tokens 6.03 -> 5.46 us; 4800 x 3200, 300
// workgroups, 6.88 -> 7.35; 20480 x 3200, 640 workgroups, 10.04 -> 10.50)
constexpr int kTokMaxWorkgroups = 256;
// 16 < M <= this: GEMM or split-K GEMV by the estimate in launch_gemv (fitted to the 2B shapes; above it the
// GEMM is always ahead)
constexpr int kSplitKMaxTokens = 256;
// row blocks (N / 16) from which ONE product at up to 4 tokens goes through the streaming kernel: 55296 x 5120
// (3456 blocks) 12.7 us against 13.3 with the staged kernel's many small workgroups, at 4 tokens 13.0 against
// 15.4; 20480 x 3200 (1280 blocks) 6.5 against 5.0: with few row blocks per CU the waves that split K finish earlier
constexpr int kStreamMinBlocks = 2048;
// row blocks from which the product without staging (gemv_i2_solo_kernel) is ahead of the staged kernel at up to
// 4 tokens: 13824 x 2560 (864 blocks) 4.46 -> 4.19 us; 3840 x 2560 (240) 2.89 staged against 2.95, 2560 x 6912 (160)
// 3.65 against 4.06.  Above 4 tokens it is ahead at every 2B shape (3840 x 2560 at 8 tokens 3.40 -> 3.34, 2560 x 6912
// 4.90 -> 4.71), and the staged kernel only stays where a workgroup shares the rows between row blocks (same bound)
constexpr int kManyBlocks = 432;
// ... and up to here: from 1024 row blocks on the staged kernel's many small workgroups stay ahead (20480 x 3200:
// 5.0 us against 5.9) until the streaming kernel takes over
constexpr int kSmallWorkgroupBlocks = 1024;
// row blocks from which a wave of the two kernels without a shared prologue takes four row blocks instead of two
// (13824 x 2560: 4.80 -> 4.46 us forward; product at 8 tokens 4.67 -> 4.62, at 16 5.78 -> 5.15)
constexpr int kFourRowBlocksPerWave = 864;
// activation elements (M * K) up to which the forward call is ONE kernel in which every workgroup quantizes the
// block again; above, quantizer kernel + product kernel (8 x 2560 = 20480: 5.9-6.2 us fused against 5.6 as two
// kernels; 16 x 2560: 9.7 against 6.1)
constexpr int kFuseMaxElems = 16384;
// the same with a norm (and gate) in the prologue (K = 2560: 3 tokens 5.2 us fused against 5.5, 4 tokens 6.5
// against 5.7; K = 6912: 2 tokens 7.4 against 6.7)
constexpr int kFuseMaxElemsNorm = 9216;
// bitlinear_solo_kernel (every wave prepares its own slice) instead of the shared-prologue kernel: one token up
// to this K (3840 x 2560 3.40 -> 3.18 us, 2560 x 2560 3.33 -> 3.13, 13824 x 2560 5.03 -> 4.81, 2560 x 6912
// 4.56 -> 4.31) ...
constexpr int kSoloMaxK = 8192;
// ... two to four tokens above this K (2560 x 6912: two tokens 5.61 -> 5.21, four 6.81 -> 6.61; at K = 2560 four
// tokens 4.16 -> 4.59, not taken), two tokens also below kManyBlocks row blocks (3.86 -> 3.69, 3.75 -> 3.62;
// 13824 x 2560 5.14 -> 6.07, not taken); with a norm in front only at one token up to this K (3840 x 2560
// 3.95 -> 3.80, 13824 x 2560 5.44 -> 5.16; 2560 x 6912 with gate and residual 5.87 -> 6.12, not taken)
constexpr int kSoloLongRowK = 4096;
// rows from which the norm + quantizer kernel of a prompt runs a wave per row (norm + product at K = 2560:
// 32.2 -> 30.1 us at 2048 rows, 53.6 -> 48.7 at 4096; below 0.2-0.9 us behind)
constexpr int kNormRowsPerWaveMinRows = 1024;
// --- prefill GEMM: tile and k-split by the number of tiles ------------------
// up to this many 64 x 128 tiles the GEMM uses 32 x 128 tiles (M = 128: 11.4 -> 9.0 us at 3840 x 2560, 21.5 -> 16.4
// at 2560 x 6912); beyond, 64 x 256 (level or ahead from here on: 2560 x 6912 at M = 1536 31.7 -> 29.2)
constexpr int kPrefillFewTiles = 330;
// wide matrices at prompt sizes take the 64 x 256 tile whatever the count
constexpr int kPrefillWideN = 8192, kPrefillWideMinTokens = 512;
// up to this many 32 x 128 tiles two groups of waves split a tile's K (M = 128, K = 2560: 9.0 -> 8.0 us), ...
constexpr int kPrefillSplit2Tiles = 320;
// ... up to this many, and from this K on, four (K = 6912: 16.6 -> 13.1 -> 12.6 us with two and four)
constexpr int kPrefillSplit4Tiles = 200;
constexpr int kPrefillSplit4MinK = 5120;
// about one tile per CU (more than half the CUs, at most all 256): 64 x 128 tiles with two k-groups (2560 x 6912
// at M = 512 19.1 -> 17.3 us) and 64 x 256 tiles with two k-groups (2560 x 6912 at M = 1024 25.9 -> 23.4)
constexpr int kPrefillOnePerCuMin = 128, kPrefillOnePerCuMax = 256;
// a little more than one round of 64 x 256 tiles (three per CU): one round of 128 x 256 tiles (two per CU) instead
// (13824 x 2560 at M = 1024: 864 tiles, 46.5 -> 42.3 us)
constexpr int kPrefillRound64 = 768, kPrefillRound128 = 1024;
// gemm_i2_prefill_mix_kernel: CUs a round of 64 x 256 tiles is sized for, and the most 32 x 128 tiles behind the whole
// rounds for which the launch with two tile sizes is taken (about 1.4 per CU; figures at launch_prefill)
constexpr int kPrefillMixCus = 256;
constexpr int kPrefillMixMaxQuarters = 360;
}  // namespace dispatch
using namespace dispatch;

// Planning calls (bitlinear_plan_name): the entry points' own dispatch code runs, and every launch is recorded --
// the kernel with its template arguments, grid, block and dynamic LDS -- instead of issued.  Nothing touches a device.
struct PlanLog {
    bool active = false;
    std::string text;
};
thread_local PlanLog t_plan;
void plan_note(const char* kernel, dim3 grid, dim3 block, size_t lds) {
    char buf[96];
    snprintf(buf, sizeof(buf), " grid=(%u,%u,%u) block=%u lds=%zu", grid.x, grid.y, grid.z, block.x, lds);
    if (!t_plan.text.empty()) t_plan.text += " + ";
    // the kernel as written at the launch site, without the parentheses that protect its commas
    std::string k(kernel);
    if (k.size() >= 2 && k.front() == '(' && k.back() == ')') k = k.substr(1, k.size() - 2);
    t_plan.text += k + buf;
}
#define BL_LAUNCH(KERNEL, GRID, BLOCK, LDS, STREAM, ...)                           \
    do {                                                                           \
        if (t_plan.active)                                                         \
            plan_note(#KERNEL, GRID, BLOCK, LDS);                                  \
        else                                                                       \
            hipLaunchKernelGGL(KERNEL, GRID, BLOCK, LDS, STREAM, __VA_ARGS__);     \
    } while (0)
int launch_status() { return (t_plan.active || hipGetLastError() == hipSuccess) ? BITLINEAR_OK : BITLINEAR_ERR_LAUNCH; }

int set_status(int st) {
    g_status = st;
    return st;
}

struct ShapeWs {
    int n, k, ws_num;
};

// The weight-scale segments as the kernels with two leading integers take them: at most eight runs of
// slot_rows output rows, run j reading ws[(map >> 3 j) & 7].  Every boundary must be a multiple of the run
// length (their greatest common divisor); a map that needs more than eight runs goes to the kernels that
// take the whole table.
struct SlotRule {
    int slot_rows;
    uint32_t map;
    bool ok;
};
SlotRule slot_rule(const ScaleMap& smap, int N) {
    auto gcd = [](int a, int b) {
        while (b) {
            const int t = a % b;
            a = b;
            b = t;
        }
        return a;
    };
    int g = N;
    for (int j = 0; j + 1 < smap.nseg; ++j) g = gcd(g, smap.ends[j]);
    SlotRule r = {g, 0u, g > 0 && N / g <= 8};
    if (!r.ok) return r;
    for (int run = 0; run < 8; ++run) {
        const int n = run * g < N ? run * g : N - 1;
        int seg = 0;
        while (seg < smap.nseg - 1 && n >= smap.ends[seg]) ++seg;
        r.map |= (uint32_t)seg << (3 * run);
    }
    return r;
}
// (N, K) -> ws_num of the reference's template instances (bitnet_kernels.cu:4-33)
const ShapeWs kShapeTable[] = {
    {3840, 2560, 3},  {2560, 2560, 1},  {13824, 2560, 2}, {2560, 6912, 1},  {4800, 3200, 6},
    {3200, 3200, 1},  {20480, 3200, 2}, {3200, 10240, 1}, {5120, 27648, 1}, {55296, 5120, 1},
};

bool shape_ok(int M, int N, int K) { return M >= 1 && N >= 16 && K >= 64 && (N % 16) == 0 && (K % 64) == 0; }

void pick_launch(int K, int* waves, int* upw) {
    const int units = K / 64;
    int u = 1;
    while (u < 8 && (units + u - 1) / u > kMaxWaves) u *= 2;  // at most 8: two rounds of 8 fit the register file
    if (u < 4 && units >= 4 * 4) u = 4;  // keep a few loads in flight per wave
    int w = (units + u - 1) / u;
    if (w > kMaxWaves) w = kMaxWaves;
    if (t_tune.waves > 0) {
        w = t_tune.waves;
        u = t_tune.upw;
    }
    *waves = w;
    *upw = u;
}

int launch_splitk(const int8_t* act, const int8_t* packed, uint16_t* out, int32_t* acc_out, const uint16_t* s,
                  const uint16_t* ws, const ScaleMap& smap, int M, int N, int K, hipStream_t stream,
                  const uint16_t* residual = nullptr) {
    int waves, upw;
    pick_launch(K, &waves, &upw);
    g_last_kernel = "gemv_i2_mfma_kernel";
    const dim3 grid(N / 16, (M + 15) / 16, 1);
    const dim3 block(waves * 64, 1, 1);
    const uint32_t* wq = (const uint32_t*)packed;
#define BITLINEAR_LAUNCH(U)                                                                                  \
    BL_LAUNCH(gemv_i2_mfma_kernel<U>, grid, block, 0, stream, act, wq, M, N, K, waves, out, acc_out, s, ws, smap, residual)
    switch (upw) {
        case 1: BITLINEAR_LAUNCH(1); break;
        case 2: BITLINEAR_LAUNCH(2); break;
        case 4: BITLINEAR_LAUNCH(4); break;
        default: BITLINEAR_LAUNCH(8); break;
    }
#undef BITLINEAR_LAUNCH
    return launch_status();
}

// Launch shape of the fused kernel: RB 16-row blocks per workgroup, S waves
// splitting K for each, UPW 64-wide k-steps in flight per wave.
struct FusedPlan {
    int rb, s, upw, vmax;
    bool ok;
};

// The activation block a workgroup of the fused kernel may hold in LDS: what a
// kernel gets without asking when it also quantizes the block; the
// pre-quantized variant raises its limit (see raise_fused_lds).
constexpr size_t kFusedLdsPlain = 58u * 1024u;
constexpr size_t kFusedLdsRaised = 144u * 1024u;
// (kFuseMaxElems / kFuseMaxElemsNorm, the activation block up to which a forward call stays one kernel: dispatch table)

FusedPlan plan_fused(int M, int N, int K, int pro = 0) {
    FusedPlan pl = {1, 1, 4, 1, false};
    if (M > kFusedMaxTokens) return pl;
    if ((size_t)N * (size_t)K / 4 >= (size_t)1 << 31) return pl;  // the kernel addresses the weights with 32-bit byte offsets
    if ((size_t)M * (K + kFusedRowPad) > (pro == 3 ? kFusedLdsRaised : kFusedLdsPlain)) return pl;
    const int units = K / 64;
    if (t_tune.path == 3) {
        pl.rb = t_tune.fused[0];
        pl.s = t_tune.fused[1];
        pl.upw = t_tune.fused[2];
    } else if (N / 16 >= kSmallWorkgroupBlocks && M <= kDecodeMaxTokens) {
        // Many row blocks (N >= 16384) and few tokens: the matrix is large enough to be bandwidth-bound, and what
        // measured best there is many small workgroups (four or five waves per row block, several
        // workgroups per CU covering each other's latencies) that walk K in two to four rounds:
        // 55296 x 5120: 13.7 us against 18.8 with one large workgroup per CU; 27648 x 10240: 13.2
        // against 16.4; 20480 x 3200: 5.4 against 7.2.  (With 8 tokens the activation block every
        // workgroup stages is too large for that: 9.0 against 8.2 us at 20480 x 3200.)
        const int blocks16 = N / 16;
        pl.rb = units >= 128 ? 4 : (blocks16 >= 2048 ? 2 : 1);
        const int cand[9][2] = {{4, 10}, {5, 8}, {4, 8}, {5, 10}, {4, 5}, {5, 5}, {4, 16}, {5, 16}, {4, 4}};
        int best = -1, best_cost = 1 << 30;
        for (int i = 0; i < 9; ++i) {
            if (cand[i][0] * pl.rb > kMaxWaves) continue;  // a workgroup has at most 16 waves
            const int per_round = cand[i][0] * cand[i][1];
            const int rounds = (units + per_round - 1) / per_round;
            const int waste = rounds * per_round - units;
            // few idle k-steps first, two to four rounds preferred, then the order of the list
            const int cost = waste * 64 + (rounds > 4 ? 400 * (rounds - 4) : (rounds == 1 ? 34 : 0));
            if (cost < best_cost) {
                best_cost = cost;
                best = i;
            }
        }
        pl.s = cand[best][0];
        pl.upw = cand[best][1];
    } else {
        // enough row blocks per workgroup to keep about 200 workgroups; up to 8
        // (16 for K > 4096) waves splitting K for each, with the fewest k-steps per wave that fit
        const int blocks16 = N / 16;
        pl.rb = blocks16 / 216;
        pl.rb = pl.rb < 1 ? 1 : (pl.rb > kFusedMaxRB ? kFusedMaxRB : pl.rb);
        // long rows: more threads share the prologue (with a norm or gate in it; the plain quantizer is
        // light enough that fewer waves with more words each in flight measure faster: 4.44 vs 4.61 us at K = 6912)
        const int want_s = units > 64 ? (pro == 0 ? 12 : kMaxWaves) : 8;
        const int max_s = (kMaxWaves / pl.rb) < want_s ? (kMaxWaves / pl.rb) : want_s;
        const int sizes[5] = {4, 5, 8, 10, 16};
        pl.upw = 0;
        for (int i = 0; i < 5; ++i)
            if ((units + sizes[i] - 1) / sizes[i] <= max_s) {
                pl.upw = sizes[i];
                break;
            }
        if (pl.upw == 0) pl.upw = 8;  // several rounds per wave: short rounds measured best (K = 27648: 9.3 us with 8, 10.7 with 16)
        pl.s = (units + pl.upw - 1) / pl.upw;
        if (pl.s > max_s) pl.s = max_s;
        // three to six tokens through the plain quantizer: more waves than the k-steps need, because the
        // quantizer's work grows with the tokens and is shared by the workgroup's threads (measured at
        // K = 2560: 4 tokens 4.72 -> 4.15 us with 12 waves, 6 tokens 5.38 -> 5.06 with 16)
        if (pro == 0 && M >= 3 && units <= 64 && pl.rb == 1) {
            pl.s = M <= 4 ? 12 : 16;
            pl.upw = 4;
            while (pl.upw * pl.s < units) pl.upw = pl.upw == 4 ? 5 : (pl.upw == 5 ? 8 : (pl.upw == 8 ? 10 : 16));
        }
    }
    const int nvec = M * (K / (pro == 3 ? 16 : 8));
    int need = (nvec + 64 * pl.rb * pl.s - 1) / (64 * pl.rb * pl.s);
    if (need > 8 && t_tune.path != 3) {
        // a large activation block: as many waves as a workgroup may have, so that every
        // thread quantizes at most 8 vectors
        pl.s = kMaxWaves / pl.rb;
        const int per_wave = (units + pl.s - 1) / pl.s;
        const int sizes[5] = {4, 5, 8, 10, 16};
        pl.upw = 16;
        for (int i = 0; i < 5; ++i)
            if (sizes[i] >= per_wave) {
                pl.upw = sizes[i];
                break;
            }
        need = (nvec + 64 * pl.rb * pl.s - 1) / (64 * pl.rb * pl.s);
    }
    pl.vmax = need <= 1 ? 1 : (need <= 2 ? 2 : (need <= 4 ? 4 : 8));
    pl.ok = need <= 8 && pl.rb * pl.s <= kMaxWaves;
    return pl;
}

// A kernel gets 64 KiB of dynamic LDS without asking; the pre-quantized variant
// may hold up to 16 rows of 6912 and more, so its limit is raised once per
// instance (a host-side attribute, no stream work).
template <int U, int V, bool R>
hipError_t raise_fused_lds() {
    static OncePerDevice once;
    return once.run([] {
        return hipFuncSetAttribute((const void*)bitlinear_fused_kernel<U, V, 3, R>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)(kFusedLdsRaised + kFusedTailPad));
    });
}

int launch_fused(const uint16_t* x, const int8_t* packed, uint16_t* out, const uint16_t* ws, const ScaleMap& smap,
                 int8_t* q_out, uint16_t* s_out, const FusedExtras& ex, int M, int N, int K, int mode,
                 const FusedPlan& pl, hipStream_t stream) {
    const int blocks16 = N / 16;
    const dim3 grid((blocks16 + pl.rb - 1) / pl.rb, 1, 1);
    const dim3 block(64 * pl.rb * pl.s, 1, 1);
    const size_t lds = (size_t)M * (K + kFusedRowPad) + kFusedTailPad;
    const uint32_t* wq = (const uint32_t*)packed;
    const int pro = ex.act_scale ? 3 : (ex.norm_weight ? (ex.glu ? 2 : 1) : 0);
    if (pro == 0 && ex.residual) return BITLINEAR_ERR_ARG;  // the plain forward has no residual epilogue
    static const char* const kFusedNames[4] = {"bitlinear_fused_kernel<quantizer>", "bitlinear_fused_kernel<norm>",
                                               "bitlinear_fused_kernel<gate+norm>", "bitlinear_fused_kernel<staged int8>"};
    g_last_kernel = kFusedNames[pro];
#define BITLINEAR_LAUNCH_UVPR(U, V, P, R)                                                                            \
    BL_LAUNCH((bitlinear_fused_kernel<U, V, P, R>), grid, block, lds, stream, x, wq, M, N, K, pl.rb, pl.s,  \
                       mode, 1.0f / (float)(K / (pro == 3 ? 16 : 8)), pro == 3 ? ex.act_scale : ex.norm_weight, out, ws, \
                       smap, q_out, s_out, ex)
#define BITLINEAR_LAUNCH_UVP(U, V, P)              \
    if (ex.residual)                               \
        BITLINEAR_LAUNCH_UVPR(U, V, P, true);      \
    else                                           \
        BITLINEAR_LAUNCH_UVPR(U, V, P, false)
#define BITLINEAR_LAUNCH_UV(U, V)                                   \
    switch (pro) {                                                  \
        case 0: BITLINEAR_LAUNCH_UVPR(U, V, 0, false); break;       \
        case 1: BITLINEAR_LAUNCH_UVP(U, V, 1); break;               \
        case 2: BITLINEAR_LAUNCH_UVP(U, V, 2); break;               \
        default:                                                    \
            if (lds > 48u * 1024u && !t_plan.active) {              \
                const hipError_t e = ex.residual ? raise_fused_lds<U, V, true>() : raise_fused_lds<U, V, false>(); \
                if (e != hipSuccess) return BITLINEAR_ERR_LAUNCH;   \
            }                                                       \
            BITLINEAR_LAUNCH_UVP(U, V, 3);                          \
            break;                                                  \
    }
#define BITLINEAR_LAUNCH_U(U)                      \
    switch (pl.vmax) {                             \
        case 1: BITLINEAR_LAUNCH_UV(U, 1); break;  \
        case 2: BITLINEAR_LAUNCH_UV(U, 2); break;  \
        case 4: BITLINEAR_LAUNCH_UV(U, 4); break;  \
        default: BITLINEAR_LAUNCH_UV(U, 8); break; \
    }
    switch (pl.upw) {
        case 4: BITLINEAR_LAUNCH_U(4); break;
        case 5: BITLINEAR_LAUNCH_U(5); break;
        case 8: BITLINEAR_LAUNCH_U(8); break;
        case 10: BITLINEAR_LAUNCH_U(10); break;
        default: BITLINEAR_LAUNCH_U(16); break;
    }
#undef BITLINEAR_LAUNCH_U
#undef BITLINEAR_LAUNCH_UV
#undef BITLINEAR_LAUNCH_UVP
#undef BITLINEAR_LAUNCH_UVPR
    return launch_status();
}

// Launch shape of bitlinear_solo_kernel: every wave multiplies exactly UPW (<= 8) k-steps, so S * UPW
// must cover K / 64; instances exist for one token (rows up to 8192 values), two (up to 4096) and
// three or four (up to 2560).
struct SoloPlan {
    int rb, s, upw, vrow, mt, rpw;
    bool coop;
    bool ok;
};

// Where the library takes it by itself.  Measured per call (HIP graph of dependent launches, distinct
// weights; shared-prologue kernel -> this one): one token 3840 x 2560 3.40 -> 3.18 us, 2560 x 2560
// 3.33 -> 3.13, 13824 x 2560 5.03 -> 4.81, 2560 x 6912 4.56 -> 4.31 (row maximum exchanged between the
// waves; 5.24 with every wave scanning the 13.8 KB row); two tokens 3.86 -> 3.69 / 3.75 -> 3.62 / 5.14 -> 6.07
// (not taken) / 5.61 -> 5.21; four tokens 4.16 -> 4.59 (not taken) and 6.81 -> 6.61 at K = 6912.
bool solo_wanted(int M, int N, int K) {
    if (M == 1) return K <= kSoloMaxK;
    if (K > kSoloLongRowK) return true;  // long rows, two to four tokens
    return M == 2 && (N / 16) < kManyBlocks;
}

// The same with an RMSNorm (pro 1) or gate + RMSNorm (pro 2) in front: measured against the shared-prologue kernel
// at one token, see bitlinear_norm_forward_bf16.
bool solo_norm_wanted(int M, int N, int K, int pro) {
    (void)N;
    // measured at one token (shared-prologue kernel -> this one): 3840 x 2560 3.95 -> 3.80 us, 2560 x 2560 with
    // the residual 3.91 -> 3.80, 13824 x 2560 5.44 -> 5.16; 2560 x 6912 with the gate and the residual 5.87 -> 6.12
    // (not taken); two to four tokens 4.7 -> 4.9 and worse (not taken)
    return M == 1 && pro == 1 && K <= kSoloLongRowK;
}

SoloPlan plan_solo(int M, int N, int K, int pro = 0, bool has_res = false) {
    SoloPlan pl = {1, 8, 5, 5, 1, 1, false, false};
    if (M < 1 || M > kSoloMaxTokens) return pl;
    if ((size_t)N * (size_t)K / 4 >= (size_t)1 << 31 || (long long)M * K * 4 >= 0x7ffffff0ll) return pl;
    const int units = K / 64;
    const int need_v = (K + 511) / 512;
    pl.mt = M == 1 ? 1 : (M == 2 ? 2 : 4);
    const int vmax = pl.mt == 1 ? 16 : (pl.mt == 2 ? 8 : 5);
    // every wave scans the whole rows while they are short and there is one token; otherwise the
    // row maximum is exchanged between the waves of the workgroup
    pl.coop = t_tune.solo_coop == 1 || (t_tune.solo_coop == 0 && (need_v > 8 || M > 1));
    if (need_v > vmax || pro != 0) pl.coop = true;
    pl.vrow = pl.coop ? 1 : (need_v <= 5 ? 5 : (need_v <= 8 ? 8 : (need_v <= 14 ? 14 : 16)));
    if (t_tune.solo >= 1 && t_tune.solo <= 4) {
        pl.rb = t_tune.solo;
        pl.s = t_tune.solo_s;
        pl.upw = t_tune.solo_upw;
    } else {
        // one row block per workgroup; with few row blocks (about one workgroup per CU) short waves of five
        // k-steps, with many the fewest waves per row block (13824 x 2560: 4.80 us with 5 waves of 8 k-steps,
        // 5.28 with 8 of 5)
        const int blocks16 = N / 16;
        pl.rb = 1;
        const int order_few[4] = {5, 7, 8, 4}, order_many[4] = {8, 7, 5, 4};
        const int* order = blocks16 >= kManyBlocks ? order_many : order_few;
        pl.upw = 0;
        for (int i = 0; i < 4; ++i)
            if ((units + order[i] - 1) / order[i] <= ((blocks16 >= kManyBlocks || units > 64) ? kMaxWaves : 10)) {
                pl.upw = order[i];
                break;
            }
        if (pl.upw == 0) pl.upw = 8;
        pl.s = (units + pl.upw - 1) / pl.upw;
        // one token and many row blocks: waves of five k-steps that take two or four row blocks each, so that a
        // slice is prepared once for all of them (13824 x 2560: 4.80 -> 4.46 us; with the RMSNorm in front 5.44,
        // the shared-prologue kernel's time, -> 5.16)
        if (M == 1 && pro <= 1 && !has_res && blocks16 >= kManyBlocks && (units + 4) / 5 <= 16 && (pl.coop || pl.vrow == 5)) {
            const int s5 = (units + 4) / 5;
            int rpw = blocks16 >= kFourRowBlocksPerWave ? 4 : 2;
            while (rpw > 1 && (rpw * s5 > kSoloRedSlots || rpw > s5)) --rpw;
            if (rpw > 1) {
                pl.upw = 5;
                pl.s = s5;
                pl.rpw = rpw;
            }
        }
    }
    // several row blocks per wave: instances exist for one token, 5 or 8 k-steps per wave, and the plain or
    // norm prologue without residual
    if (t_tune.solo_rpw >= 1) pl.rpw = t_tune.solo_rpw;
    if (pl.rpw > 1 && !(M == 1 && (pl.upw == 5 || pl.upw == 8) && pro <= 1 && !has_res && (pl.coop || pl.vrow == 5) && pl.s >= pl.rpw &&
                        pl.rb * pl.rpw * pl.s <= kSoloRedSlots && pl.rpw >= 2 && pl.rpw <= 4))
        pl.rpw = 1;
    pl.ok = pl.rb >= 1 && pl.rb <= kFusedMaxRB && pl.s >= 1 && pl.rb * pl.s <= kMaxWaves && pl.s * pl.upw >= units &&
            (pl.upw == 4 || pl.upw == 5 || pl.upw == 7 || pl.upw == 8);
    return pl;
}

int launch_solo(const uint16_t* x, const int8_t* packed, uint16_t* out, int32_t* acc_out, const uint16_t* ws,
                const ScaleMap& smap, int8_t* q_out, uint16_t* s_out, int M, int N, int K, const SoloPlan& pl,
                hipStream_t stream, int pro = 0, const uint16_t* norm_weight = nullptr, float eps = 0.0f,
                const uint16_t* residual = nullptr) {
    const int blocks16 = N / 16;
    const dim3 grid((blocks16 + pl.rb * pl.rpw - 1) / (pl.rb * pl.rpw), 1, 1);
    const dim3 block(64 * pl.rb * pl.s, 1, 1);
    const uint32_t* wq = (const uint32_t*)packed;
    const SlotRule rule = slot_rule(smap, N);
    if (!rule.ok) return BITLINEAR_ERR_ARG;
    const int slot_rows = rule.slot_rows;
    const int rb_map = pl.rb | (int)(rule.map << 8);
    if (pro != 0 && (!pl.coop || !norm_weight)) return BITLINEAR_ERR_ARG;
    g_last_kernel = pro == 0 ? "bitlinear_solo_kernel" : (pro == 1 ? "bitlinear_solo_kernel<norm>" : "bitlinear_solo_kernel<gate+norm>");
#define BITLINEAR_LAUNCH_SOLO_W(U, V, T, C, P, R, W)                                                                      \
    BL_LAUNCH((bitlinear_solo_kernel<U, V, T, C, P, R, W>), grid, block, 0, stream, x, wq, M, N, K, rb_map, pl.s, \
                       slot_rows, norm_weight, ws, out, residual, eps, q_out, s_out, acc_out)
#define BITLINEAR_LAUNCH_SOLO_P(U, V, T, C, P, R) BITLINEAR_LAUNCH_SOLO_W(U, V, T, C, P, R, 1)
#define BITLINEAR_LAUNCH_SOLO(U, V, T, C) BITLINEAR_LAUNCH_SOLO_P(U, V, T, C, 0, false)
    if (pl.rpw > 1) {
        // one token, several row blocks per wave (plan_solo admits only what is instantiated here)
        if (residual || pro > 1 || pl.mt != 1) return BITLINEAR_ERR_ARG;
#define BITLINEAR_LAUNCH_SOLO_RW(U, W)                                        \
    if (pro == 1) BITLINEAR_LAUNCH_SOLO_W(U, 1, 1, true, 1, false, W);        \
    else if (pl.coop) BITLINEAR_LAUNCH_SOLO_W(U, 1, 1, true, 0, false, W);    \
    else BITLINEAR_LAUNCH_SOLO_W(U, 5, 1, false, 0, false, W)
        if (pl.upw == 8) {
            if (pl.rpw == 2) { BITLINEAR_LAUNCH_SOLO_RW(8, 2); } else if (pl.rpw == 3) { BITLINEAR_LAUNCH_SOLO_RW(8, 3); } else { BITLINEAR_LAUNCH_SOLO_RW(8, 4); }
        } else {
            if (pl.rpw == 2) { BITLINEAR_LAUNCH_SOLO_RW(5, 2); } else if (pl.rpw == 3) { BITLINEAR_LAUNCH_SOLO_RW(5, 3); } else { BITLINEAR_LAUNCH_SOLO_RW(5, 4); }
        }
#undef BITLINEAR_LAUNCH_SOLO_RW
        return launch_status();
    }
    // norm / gate prologues: the exchanging variant only, with or without the residual epilogue
#define BITLINEAR_LAUNCH_SOLO_N(U, T)                                        \
    if (pro == 1) {                                                          \
        if (residual) BITLINEAR_LAUNCH_SOLO_P(U, 1, T, true, 1, true);       \
        else BITLINEAR_LAUNCH_SOLO_P(U, 1, T, true, 1, false);               \
    } else {                                                                 \
        if (residual) BITLINEAR_LAUNCH_SOLO_P(U, 1, T, true, 2, true);       \
        else BITLINEAR_LAUNCH_SOLO_P(U, 1, T, true, 2, false);               \
    }
#define BITLINEAR_LAUNCH_SOLO_NU(U)                          \
    if (pl.mt == 1) { BITLINEAR_LAUNCH_SOLO_N(U, 1) }        \
    else if (pl.mt == 2) { BITLINEAR_LAUNCH_SOLO_N(U, 2) }   \
    else { BITLINEAR_LAUNCH_SOLO_N(U, 4) }
    if (pro != 0) {
        switch (pl.upw) {
            case 4: BITLINEAR_LAUNCH_SOLO_NU(4); break;
            case 5: BITLINEAR_LAUNCH_SOLO_NU(5); break;
            case 7: BITLINEAR_LAUNCH_SOLO_NU(7); break;
            default: BITLINEAR_LAUNCH_SOLO_NU(8); break;
        }
        return launch_status();
    }
#define BITLINEAR_LAUNCH_SOLO_U(U)                                      \
    if (pl.coop) {                                                      \
        if (pl.mt == 1) BITLINEAR_LAUNCH_SOLO(U, 1, 1, true);           \
        else if (pl.mt == 2) BITLINEAR_LAUNCH_SOLO(U, 1, 2, true);      \
        else BITLINEAR_LAUNCH_SOLO(U, 1, 4, true);                      \
    } else if (pl.mt == 1) {                                            \
        if (pl.vrow == 5) BITLINEAR_LAUNCH_SOLO(U, 5, 1, false);        \
        else if (pl.vrow == 8) BITLINEAR_LAUNCH_SOLO(U, 8, 1, false);   \
        else if (pl.vrow == 14) BITLINEAR_LAUNCH_SOLO(U, 14, 1, false); \
        else BITLINEAR_LAUNCH_SOLO(U, 16, 1, false);                    \
    } else if (pl.mt == 2) {                                            \
        if (pl.vrow == 5) BITLINEAR_LAUNCH_SOLO(U, 5, 2, false);        \
        else BITLINEAR_LAUNCH_SOLO(U, 8, 2, false);                     \
    } else {                                                            \
        BITLINEAR_LAUNCH_SOLO(U, 5, 4, false);                          \
    }
    switch (pl.upw) {
        case 4: BITLINEAR_LAUNCH_SOLO_U(4); break;
        case 5: BITLINEAR_LAUNCH_SOLO_U(5); break;
        case 7: BITLINEAR_LAUNCH_SOLO_U(7); break;
        default: BITLINEAR_LAUNCH_SOLO_U(8); break;
    }
#undef BITLINEAR_LAUNCH_SOLO_U
#undef BITLINEAR_LAUNCH_SOLO_NU
#undef BITLINEAR_LAUNCH_SOLO_N
#undef BITLINEAR_LAUNCH_SOLO
#undef BITLINEAR_LAUNCH_SOLO_P
#undef BITLINEAR_LAUNCH_SOLO_W
    return launch_status();
}

// Launch shape of gemv_i2_solo_kernel (up to 16 tokens): one row block per group of S waves, UPW k-steps per wave
// as in plan_solo; with many row blocks a wave takes two or four of them.
struct ProdPlan {
    int s, upw, rpw;
    bool ok;
};

ProdPlan plan_prod_solo(int M, int N, int K) {
    ProdPlan pl = {8, 5, 1, false};
    if (M < 1 || M > 16) return pl;
    if ((size_t)N * (size_t)K / 4 >= (size_t)1 << 31) return pl;
    const int units = K / 64;
    const int blocks16 = N / 16;
    if (t_tune.prod_solo == 1) {
        pl.s = t_tune.prod_s;
        pl.upw = t_tune.prod_upw;
    } else {
        const int order[4] = {5, 7, 8, 4};
        pl.upw = 0;
        for (int i = 0; i < 4; ++i)
            if ((units + order[i] - 1) / order[i] <= (units > 64 ? kMaxWaves : 10)) {
                pl.upw = order[i];
                break;
            }
        if (pl.upw == 0) pl.upw = 8;
        pl.s = (units + pl.upw - 1) / pl.upw;
        // measured at 13824 x 2560: up to four tokens two row blocks per wave (4.19 / 4.22 / 4.33 us at one / two /
        // four tokens, 4.39 / 4.41 / 4.49 with four), from eight tokens on four (4.62 against 4.67; 5.15 against 5.78 at 16)
        if (blocks16 >= kManyBlocks) pl.rpw = (blocks16 >= kFourRowBlocksPerWave && M > kDecodeMaxTokens) ? 4 : 2;
    }
    if (t_tune.solo_rpw >= 1) pl.rpw = t_tune.solo_rpw;
    if (pl.rpw == 3) pl.rpw = 2;
    while (pl.rpw > 1 && (pl.rpw * pl.s > kSoloRedSlots || pl.rpw > pl.s)) pl.rpw >>= 1;
    pl.ok = pl.s >= 1 && pl.s <= kMaxWaves && pl.s * pl.upw >= units && (pl.upw == 4 || pl.upw == 5 || pl.upw == 7 || pl.upw == 8);
    return pl;
}

int launch_prod_solo(const int8_t* act, const int8_t* packed, uint16_t* out, int32_t* acc_out, const uint16_t* s,
                     const uint16_t* ws, const ScaleMap& smap, int M, int N, int K, const ProdPlan& pl, hipStream_t stream,
                     const uint16_t* residual) {
    const int blocks16 = N / 16;
    const dim3 grid((blocks16 + pl.rpw - 1) / pl.rpw, 1, 1);
    const dim3 block(64 * pl.s, 1, 1);
    const uint32_t* wq = (const uint32_t*)packed;
    const SlotRule rule = slot_rule(smap, N);
    if (!rule.ok) return BITLINEAR_ERR_ARG;
    const int slot_rows = rule.slot_rows;
    const int rb_map = 1 | (int)(rule.map << 8);
    g_last_kernel = "gemv_i2_solo_kernel";
#define BITLINEAR_LAUNCH_PS(U, W, R)                                                                               \
    BL_LAUNCH((gemv_i2_solo_kernel<U, W, R>), grid, block, 0, stream, act, wq, M, N, K, rb_map, pl.s, slot_rows, \
                       s, ws, out, residual, acc_out)
#define BITLINEAR_LAUNCH_PS_W(U, W)         \
    if (residual) BITLINEAR_LAUNCH_PS(U, W, true); \
    else BITLINEAR_LAUNCH_PS(U, W, false)
#define BITLINEAR_LAUNCH_PS_U(U)                       \
    if (pl.rpw == 1) { BITLINEAR_LAUNCH_PS_W(U, 1); }  \
    else if (pl.rpw == 2) { BITLINEAR_LAUNCH_PS_W(U, 2); } \
    else { BITLINEAR_LAUNCH_PS_W(U, 4); }
    switch (pl.upw) {
        case 4: BITLINEAR_LAUNCH_PS_U(4); break;
        case 5: BITLINEAR_LAUNCH_PS_U(5); break;
        case 7: BITLINEAR_LAUNCH_PS_U(7); break;
        default: BITLINEAR_LAUNCH_PS_U(8); break;
    }
#undef BITLINEAR_LAUNCH_PS_U
#undef BITLINEAR_LAUNCH_PS_W
#undef BITLINEAR_LAUNCH_PS
    return launch_status();
}

// bitlinear_solo_tok_kernel: launch shape as plan_prod_solo (S waves of UPW k-steps, RPW row blocks per wave);
// instances exist for five k-steps per wave, which the plan chooses for rows of up to 3200 values, and one or
// four row blocks per wave (two, the plan's choice from 432 row blocks on, measured behind the other kernels:
// 8192 x 2048 at 5 tokens 4.70 us against 5.12).
bool tok_plan_ok(int M, const ProdPlan& pl) {
    return pl.ok && pl.upw == 5 && (pl.rpw == 1 || pl.rpw == 4) && M >= 1 && M <= kTokMaxTokens;
}

int launch_solo_tok(const uint16_t* x, const int8_t* packed, uint16_t* out, int32_t* acc_out, const uint16_t* ws,
                    const ScaleMap& smap, int8_t* q_out, uint16_t* s_out, int M, int N, int K, const ProdPlan& pl,
                    hipStream_t stream) {
    const int blocks16 = N / 16;
    const dim3 grid((blocks16 + pl.rpw - 1) / pl.rpw, 1, 1);
    const dim3 block(64 * pl.s, 1, 1);
    const uint32_t* wq = (const uint32_t*)packed;
    const SlotRule rule = slot_rule(smap, N);
    if (!rule.ok || !tok_plan_ok(M, pl)) return BITLINEAR_ERR_ARG;
    const int slot_rows = rule.slot_rows;
    const int rb_map = 1 | (int)(rule.map << 8);
    g_last_kernel = "bitlinear_solo_tok_kernel";
#define BITLINEAR_LAUNCH_TOK(W)                                                                                        \
    BL_LAUNCH((bitlinear_solo_tok_kernel<5, W>), grid, block, 0, stream, x, wq, M, N, K, rb_map, pl.s, slot_rows, ws, \
              out, q_out, s_out, acc_out)
    if (pl.rpw == 1) BITLINEAR_LAUNCH_TOK(1);
    else BITLINEAR_LAUNCH_TOK(4);
#undef BITLINEAR_LAUNCH_TOK
    return launch_status();
}

int launch_prefill(const int8_t* act, const int8_t* packed, uint16_t* out, int32_t* acc_out, const uint16_t* s,
                   const uint16_t* ws, const ScaleMap& smap, int M, int N, int K, hipStream_t stream,
                   const uint16_t* residual = nullptr) {
    const uint32_t* wq = (const uint32_t*)packed;
    // the kernel addresses the packed weights through a buffer descriptor with 32-bit offsets
    if ((long long)N * K / 4 >= (1ll << 31)) return BITLINEAR_ERR_SHAPE;
    g_last_kernel = "gemm_i2_prefill_kernel";
    // the large tile double-buffers 2 x 128 rows x 272 bytes = 68 KiB of LDS (so do four groups of the
    // small one): above the 64 KiB a kernel gets without asking (a host-side attribute, set once per process)
    static OncePerDevice lds_limit_raised;
    const hipError_t lds_err = t_plan.active ? hipSuccess : lds_limit_raised.run([] {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_i2_prefill_kernel<4, 2, 1>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 2 * 128 * kPfRowBytes);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)gemm_i2_prefill_kernel<1, 1, 4>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    4 * 2 * 32 * kPfRowBytes);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)gemm_i2_prefill_kernel<2, 1, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    2 * 2 * 64 * kPfRowBytes);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)gemm_i2_prefill_kernel<2, 2, 2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    2 * 2 * 64 * kPfRowBytes);
        return e;
    });
    if (lds_err != hipSuccess) return BITLINEAR_ERR_LAUNCH;
    // tile (rows x columns of the output per workgroup): 0 = 64 x 128, 1 = 128 x 256, 2 = 64 x 256,
    // 3 = 64 x 512, 4 = 32 x 128.  Measured: the wide tile pays once there are many tiles (about four
    // per CU of the narrow kind); with few tiles (up to about 1.3 per CU) half-height tiles put twice as
    // many workgroups on the machine and finish a tile's chain of k-chunks earlier (M = 128: 11.4 -> 9.0
    // us at 3840 x 2560, 21.5 -> 16.4 at 2560 x 6912).
    const long long narrow_tiles = (long long)((N + 127) / 128) * ((M + 63) / 64);
    // (beyond the few-tile range the wide tile: against 64 x 128 it measured level or ahead from 330 tiles on --
    // 2560 x 6912 at M = 1536 31.7 -> 29.2 us, 2560 x 2560 there 14.3 -> 13.6, elsewhere within 2 %)
    const long long wide_tiles = (long long)((N + 255) / 256) * ((M + 63) / 64);
    // (the kernel that brings the activation chunks straight into LDS needs 128-k chunks that divide K and 16-byte
    // aligned output rows)
    const bool dma_fits = K % 128 == 0 && ((((uintptr_t)out) | ((uintptr_t)acc_out) | ((uintptr_t)residual)) & 15u) == 0;
    int tile = ((N >= kPrefillWideN && M >= kPrefillWideMinTokens) || narrow_tiles > kPrefillFewTiles) ? 2 : 4;
    // 64 x 256 tiles run three workgroups per CU (768 at a time), 128 x 256 tiles two (512): with a little more than
    // one full round of the former, one round of the latter finishes earlier (13824 x 2560 at M = 1024: 864 tiles,
    // 46.5 -> 42.3 us; 3840 x 2560 at M = 4096: 960 tiles, 45.1 -> 44.1)
    // (with the direct-to-LDS kernel the 64 x 256 tiles stay: 13824 x 2560 at M = 1024 41.5 -> 39.8 us)
    if (tile == 2 && wide_tiles > kPrefillRound64 && wide_tiles <= kPrefillRound128 && !dma_fits) tile = 1;
    // the 64 x 256 tile goes through the kernel that brings the activations into LDS without registers and the
    // weight words of two column tiles with one request (a layer's four GEMMs at M = 2048: 1.72 -> 1.92 POP/s on
    // uniform random int8; 13824 x 2560 73.3 -> 64.8 us, 2560 x 6912 46.3 -> 42.2, at M = 4096 1.97 -> 2.20),
    // given 128-k chunks that divide K and 16-byte aligned rows
    // one launch with tiles of two sizes (see gemm_i2_prefill_mix_kernel): whole rounds of one 64 x 256 tile per CU over the
    // first columns, the columns behind them as 32 x 128 tiles.  Taken when those quarter tiles are at most about 1.4
    // per CU (measured, 64 x 256 tiles or half-height ones -> this: 2560 x 2560 at M = 2048 19.0 -> 17.3 us, at M = 3584
    // 28.5 -> 25.9, at 5120 39.4 -> 36.1; 2560 x 6912 41.0 -> 36.5 / 62.7 -> 57.3 / 91.4 -> 82.0; 3200 x 3200 at M = 1536
    // 22.4 -> 20.1, 2560 33.0 -> 28.5, 5120 58.0 -> 49.9; with more of them the even tiles are ahead: 2560 x 2560 at
    // M = 2560 21.3 against 26.5, 3840 x 2560 at M = 2048 22.8 against 28.0)
    if (dma_fits && (t_tune.path == 0 || (t_tune.path == 5 && t_tune.prefill_big == 8))) {
        const int rt64 = (M + 63) / 64, rt32 = (M + 31) / 32;
        const int band64 = (rt64 + 7) / 8, band32 = (rt32 + 7) / 8;
        const long long wide = (long long)((N + 255) / 256) * rt64;
        const int rounds = wide / kPrefillMixCus > 1 ? (int)(wide / kPrefillMixCus) : 1;
        int big_cols = (int)((long long)kPrefillMixCus * rounds / rt64);
        if (big_cols > N / 256) big_cols = N / 256;
        const int small_cols = (N - big_cols * 256 + 127) / 128;
        const long long quarters = (long long)rt32 * small_cols;
        const bool wanted = t_tune.path == 5 || (wide > kPrefillMixCus && big_cols >= 1 && quarters > 0 && quarters <= kPrefillMixMaxQuarters);
        const long long groups = 8ll * band64 * big_cols + 8ll * band32 * small_cols;
        if (wanted && rt64 <= 4096 && groups < (1ll << 30)) {
            const int nbig = 8 * band64 * big_cols;
            const dim3 mgrid((unsigned)groups, 1, 1), mblock(256, 1, 1);
            g_last_kernel = "gemm_i2_prefill_mix_kernel";
            if (K % 256 == 0)
                BL_LAUNCH((gemm_i2_prefill_mix_kernel<256>), mgrid, mblock, 3 * 64 * 256, stream, act, wq, M, N, K, nbig, big_cols,
                          out ? 1 : 0, small_cols, s, out, acc_out, ws, smap, residual);
            else
                BL_LAUNCH((gemm_i2_prefill_mix_kernel<128>), mgrid, mblock, 3 * 64 * 128, stream, act, wq, M, N, K, nbig, big_cols,
                          out ? 1 : 0, small_cols, s, out, acc_out, ws, smap, residual);
            return launch_status();
        }
    }
    bool dma = true;
    int dma_mt = 2;  // row tiles of 32 tokens per workgroup of that kernel: 64 x 256, or 32 x 256 / 128 x 256 when forced
    if (t_tune.path == 5) {
        tile = t_tune.prefill_big;
        dma = tile >= 5;
        dma_mt = tile == 6 ? 1 : (tile == 7 ? 4 : 2);
        if (tile >= 5) tile = tile == 7 ? 1 : (tile == 6 ? 8 : 2);  // 8: 32 x 256, a shape only that kernel has
    }
    // groups of waves that split a tile's K between them (small tiles only): while the small tiles
    // leave SIMDs with one or two waves, a tile's chain of chunks runs at the speed of one wave's
    // instruction stream, and more groups shorten it
    const long long small_tiles = (long long)((N + 127) / 128) * ((M + 31) / 32);
    int ks = 1;
    // measured at M = 128: 9.0 -> 8.0 us at K = 2560 with two groups (four: 9.0), 16.6 -> 13.1 -> 12.6 at
    // K = 6912 with two and four; with more than one tile per CU the groups only compete (M = 512, 3840 x 2560:
    // 11.6 -> 13.6 us)
    if (tile == 4 && small_tiles <= kPrefillSplit2Tiles)
        ks = (small_tiles <= kPrefillSplit4Tiles && K >= kPrefillSplit4MinK) ? 4 : 2;
    // between half a tile and about one tile of 64 x 128 per CU: those tiles, with two groups of waves each
    // (2560 x 6912: M = 512 19.1 -> 17.3 us, M = 640 20.5 -> 17.7, M = 768 22.1 -> 20.0; 2560 x 2560: M = 640
    // 10.2 -> 9.5; 3840 x 2560: M = 384 10.0 -> 9.5, M = 512 9.7 -> 9.3)
    if (t_tune.path != 5 && tile == 4 && narrow_tiles > kPrefillOnePerCuMin && narrow_tiles <= kPrefillOnePerCuMax) {
        tile = 0;
        ks = 2;
    }
    // about one 64 x 256 tile per CU: those tiles, two groups of waves each (2560 x 6912: M = 1024 25.9 -> 23.4 us,
    // M = 1536 29.2 -> 27.9; 13824 x 2560 at M = 256 15.8 -> 14.3; 2560 x 2560 at M = 1280 13.6 -> 13.1; with 320
    // tiles 42.6 -> 49.4: not taken; at K = 2560 the 32 x 128 tiles stay ahead up to 330 of the 64 x 128 kind)
    // (with the direct-to-LDS kernel one group does as well or better: 13824 x 2560 at M = 256 17.1 -> 14.8 us,
    // 2560 x 6912 at M = 1024 27.3 -> 27.0)
    if (t_tune.path != 5 && (tile == 2 || (tile == 4 && K >= kPrefillSplit4MinK)) && wide_tiles > kPrefillOnePerCuMin &&
        wide_tiles <= kPrefillOnePerCuMax && narrow_tiles > kPrefillOnePerCuMax) {
        tile = 2;
        ks = (dma_fits && K < kPrefillSplit4MinK) ? 1 : 2;  // (long rows keep the two groups: 2560 x 6912 at M = 1024 level)
    }
    // between one and one and a half 64 x 256 tiles per CU a quarter of the CUs would get two tiles and the rest one:
    // half-height tiles (32 x 256, the direct-to-LDS kernel only) spread evenly, at most three per CU (2560 x 2560 at
    // M = 2048 21.3 -> 20.0 us, 2560 x 6912 43.5 -> 42.5, 3840 x 2560 at M = 1536 21.5 -> 21.1; from two tiles per CU
    // on the full-height tiles are ahead again: 2560 x 2560 at M = 4096 30.7 against 32.1)
    if (t_tune.path != 5 && tile == 2 && ks == 1 && dma_fits && wide_tiles > kPrefillOnePerCuMax &&
        wide_tiles <= kPrefillOnePerCuMax + kPrefillOnePerCuMin)
        tile = 8;
    if (t_tune.path == 5 && t_tune.prefill_ks > 0) ks = (tile == 4 || ((tile == 0 || tile == 2) && t_tune.prefill_ks == 2)) ? t_tune.prefill_ks : 1;
    if (K <= kPfChunk * (ks - 1)) ks = 1;  // fewer chunks than groups
    const dim3 block(kPfWaves * 64 * ks, 1, 1);
    // grid of 8 XCDs x bands per XCD x tiles per band (see the kernel); bands of up to 8 row
    // tiles, fewer when there are not enough row tiles to give every XCD a band
    if (tile == 8 && !dma_fits) tile = 4;
    const int tm = tile == 1 ? 128 : ((tile == 4 || tile == 8) ? 32 : 64);
    const int tn = (tile == 0 || tile == 4) ? 128 : (tile == 3 ? 512 : 256);
    const int row_tiles = (M + tm - 1) / tm, col_tiles = (N + tn - 1) / tn;
    int band = row_tiles / 8;
    band = band < 1 ? 1 : (band > 8 ? 8 : band);
    if (t_tune.path == 5 && t_tune.prefill_band > 0) band = t_tune.prefill_band;
    const int nbands = (row_tiles + band - 1) / band;
    // the columns are cut into segments as well, as many as it takes for the number of (band,
    // segment) units to be a multiple of the 8 XCDs: every XCD then gets the same number of units
    // (3 bands x 3 segments left one XCD with two units and the others with one: M = 96 took longer
    // than M = 128)
    int g8 = nbands & 7;
    g8 = g8 == 0 ? 8 : (g8 & -g8);  // gcd(nbands, 8)
    int cseg_shift = g8 == 8 ? 0 : (g8 == 4 ? 1 : (g8 == 2 ? 2 : 3));  // 8 / g8 segments, a power of two
    while ((1 << cseg_shift) > col_tiles) --cseg_shift;
    const int cseg = 1 << cseg_shift;
    const int seg_cols = (col_tiles + cseg - 1) / cseg;
    const int units = nbands * cseg;
    // x = XCD + 8 * (row tile within the band), y = column tile within the segment, z = round of 8
    // units: the same order of workgroups as a linear grid, without divisions in the kernel
    if (seg_cols > 65535 || (units + 7) / 8 > 65535) return BITLINEAR_ERR_SHAPE;
    const dim3 grid(8 * band, seg_cols, (units + 7) / 8);
#define BITLINEAR_LAUNCH_PF(MT_, NT_, KS_)                                                                          \
    BL_LAUNCH((gemm_i2_prefill_kernel<MT_, NT_, KS_>), grid, block, KS_ * 2 * 32 * MT_ * kPfRowBytes, stream, \
                       act, wq, M, N, K, units, cseg_shift | (out ? 256 : 0), band, seg_cols, s, out, acc_out, ws, smap, residual)
#define BITLINEAR_LAUNCH_PFX(MT_, CK_)                                                                                   \
    BL_LAUNCH((gemm_i2_prefill_dma_kernel<MT_, 2, CK_>), grid, block, 3 * 32 * MT_ * CK_, stream, act, wq, M, N, K, units, \
              cseg_shift | (out ? 256 : 0), band, seg_cols, s, out, acc_out, ws, smap, residual)
    if (dma && dma_fits && ks == 1 && (tile == 8 || (tile == 1 && dma_mt == 4))) {
        g_last_kernel = "gemm_i2_prefill_dma_kernel";
        if (tile == 8) {
            if (K % 256 == 0) BITLINEAR_LAUNCH_PFX(1, 256);
            else BITLINEAR_LAUNCH_PFX(1, 128);
        } else {
            BITLINEAR_LAUNCH_PFX(4, 128);
        }
    } else if (tile == 4) {
        if (ks == 4) {
            BITLINEAR_LAUNCH_PF(1, 1, 4);
        } else if (ks == 2) {
            BITLINEAR_LAUNCH_PF(1, 1, 2);
        } else {
            BITLINEAR_LAUNCH_PF(1, 1, 1);
        }
    } else if (tile == 1) {
        BITLINEAR_LAUNCH_PF(4, 2, 1);
    } else if (tile == 3) {
        BITLINEAR_LAUNCH_PF(2, 4, 1);
    } else if (tile == 2) {
        if (ks == 2) {
            BITLINEAR_LAUNCH_PF(2, 2, 2);
        } else if (dma && dma_fits) {
            g_last_kernel = "gemm_i2_prefill_dma_kernel";
            if (K % 256 == 0) BITLINEAR_LAUNCH_PFX(2, 256);
            else BITLINEAR_LAUNCH_PFX(2, 128);
        } else {
            BITLINEAR_LAUNCH_PF(2, 2, 1);
        }
    } else if (ks == 2) {
        BITLINEAR_LAUNCH_PF(2, 1, 2);
    } else {
        BITLINEAR_LAUNCH_PF(2, 1, 1);
    }
#undef BITLINEAR_LAUNCH_PF
#undef BITLINEAR_LAUNCH_PFX
    return launch_status();
}

// Streaming kernel: applicability and launch.  D (loads in flight per lane) is chosen so that the
// rounds of D steps cover the ceil(K / 256) steps of a row block with the fewest idle steps.
bool stream_applicable(int M, int N, int K, const ScaleMap& smap) {
    if (M < 1 || M > kStreamMaxTokens) return false;
    if ((long long)M * K > kStreamMaxActBytes) return false;  // the activation block lives in LDS
    for (int j = 0; j < smap.nseg; ++j)
        if (smap.ends[j] % 16) return false;  // the kernel takes one scale slot per 16-row block
    (void)N;
    return true;
}

int launch_stream(const StreamProblem* probs, int nprob, int M, int N, int K, const ScaleMap& smap, int32_t* acc_out,
                  hipStream_t stream, bool compute = true, uint32_t* sink = nullptr) {
    if (nprob < 1 || nprob > kStreamMaxProblems) return BITLINEAR_ERR_ARG;
    const int steps = (K + 255) / 256;
    // D (loads in flight per lane): the rounds of D steps should cover the steps of a row block with few
    // idle steps; among equals the first of this list
    const int depths[6] = {5, 6, 7, 4, 8, 10};
    int depth = 5, best = 1 << 30;
    for (int i = 0; i < 6; ++i) {
        const int rounds = (steps + depths[i] - 1) / depths[i];
        const int waste = rounds * depths[i] - steps;
        if (waste < best) {
            best = waste;
            depth = depths[i];
        }
    }
    if (t_tune.stream_depth > 0) depth = t_tune.stream_depth;
    StreamArgs a;
    a.M = M;
    a.N = N;
    a.K = K;
    a.blocks16 = N / 16;
    a.steps = steps;
    a.pad_ = 0;
    // waves the launch is sized for, over all problems: a run of row blocks per wave
    const int waves_per_cu = t_tune.stream_waves > 0 ? t_tune.stream_waves : 8;
    const long long total_items = (long long)nprob * a.blocks16;
    const int max_waves = 256 * waves_per_cu;
    a.ipw = (int)((total_items + max_waves - 1) / max_waves);
    a.rounds = (steps + depth - 1) / depth;
    a.acc_out = acc_out;
    a.smap = smap;
    for (int i = 0; i < kStreamMaxProblems; ++i) a.p[i] = probs[i < nprob ? i : 0];
    const int waves = (a.blocks16 + a.ipw - 1) / a.ipw;  // per problem
    const dim3 grid((waves + 3) / 4, nprob, 1), block(256, 1, 1);
    const size_t lds = compute ? (size_t)M * (K + kStreamRowPad) + 256 : 0;
    g_last_kernel = "gemv_i2_stream_kernel";
#define BITLINEAR_LAUNCH_STREAM(DD)                                                                      \
    if (compute)                                                                                         \
        BL_LAUNCH((gemv_i2_stream_kernel<DD, true>), grid, block, lds, stream, a, sink);        \
    else                                                                                                 \
        BL_LAUNCH((gemv_i2_stream_kernel<DD, false>), grid, block, lds, stream, a, sink)
    switch (depth) {
        case 4: BITLINEAR_LAUNCH_STREAM(4); break;
        case 6: BITLINEAR_LAUNCH_STREAM(6); break;
        case 7: BITLINEAR_LAUNCH_STREAM(7); break;
        case 8: BITLINEAR_LAUNCH_STREAM(8); break;
        case 10: BITLINEAR_LAUNCH_STREAM(10); break;
        default: BITLINEAR_LAUNCH_STREAM(5); break;
    }
#undef BITLINEAR_LAUNCH_STREAM
    return launch_status();
}

int launch_gemv(const int8_t* act, const int8_t* packed, uint16_t* out, int32_t* acc_out, const uint16_t* s,
                const uint16_t* ws, const ScaleMap& smap, int M, int N, int K, hipStream_t stream,
                const uint16_t* residual = nullptr) {
    // vector loads: 16-byte groups of both operands must be 16-byte aligned
    if ((((uintptr_t)act) | ((uintptr_t)packed)) & 15u) return BITLINEAR_ERR_ARG;
    if (M > kPrefillMinTokens && t_tune.path != 2) {
        // A few dozen tokens on a narrow matrix leave most CUs without a GEMM tile, and a tile's
        // chain of 256-k chunks is then pure latency (about 0.64 us each).  There the split-K kernel,
        // run once per 16 tokens and re-reading the weights from L2 (about 1.45 TB/s measured),
        // finishes earlier.  Both estimates in microseconds, fitted to measurements at the 2B shapes.
        bool gemm = true;
        if (M <= kSplitKMaxTokens && t_tune.path == 0) {
            const double groups = (M + 15) / 16;
            const double splitk_us = 3.5 + groups * ((double)N * K / 4.0) / 1.45e6;
            const double tiles = ((N + 127) / 128) * (double)((M + 63) / 64);
            const double tiles32 = ((N + 127) / 128) * (double)((M + 31) / 32);
            const double gemm_us = tiles32 <= kPrefillSplit2Tiles
                                       ? 5.1 + ((tiles32 <= kPrefillSplit4Tiles && K >= kPrefillSplit4MinK) ? 0.267 : 0.29) * (K / 256.0)
                                       : (tiles <= kPrefillFewTiles
                                              ? 4.4 + 0.45 * (K / 256.0) * (tiles32 > 400.0 ? tiles32 / 400.0 : 1.0)
                                              : 4.0 + 0.64 * (K / 256.0) * (tiles > 256.0 ? tiles / 256.0 : 1.0));
            gemm = gemm_us <= splitk_us;
        }
        if (gemm) return launch_prefill(act, packed, out, acc_out, s, ws, smap, M, N, K, stream, residual);
        return launch_splitk(act, packed, out, acc_out, s, ws, smap, M, N, K, stream, residual);
    }
    // The kernel that stages the int8 rows in LDS once per workgroup and shares
    // them between several row blocks: fewer activation bytes through L2 than
    // the kernels below, which read their B operands straight from global.
    // Bandwidth-bound sizes at up to four tokens: waves that stream whole row blocks
    if (t_tune.stream != 2 && t_tune.path == 0 && !residual && stream_applicable(M, N, K, smap)) {
        const bool wanted = t_tune.stream == 1 || (N / 16) >= kStreamMinBlocks;
        if (wanted) {
            const StreamProblem one = {act, packed, out, out ? s : (const uint16_t*)packed, out ? ws : (const uint16_t*)packed};
            return launch_stream(&one, 1, M, N, K, smap, acc_out, stream);
        }
    }
    // Up to 16 tokens through the kernel without staging, where it measured faster than the kernels below (LDS-staged
    // up to four tokens, split-K beyond): many row blocks (13824 x 2560: 4.46 -> 4.19 us at one token, 4.88 -> 4.62
    // at eight, 6.00 -> 5.15 at sixteen) and more than four tokens (3840 x 2560: 3.40 -> 3.34 at eight, 3.83 -> 3.72
    // at sixteen; 2560 x 6912: 4.90 -> 4.71 and 6.11 -> 5.89); elsewhere the staged kernel stays (2.89 against 2.95
    // at 3840 x 2560 and 3.65 against 4.06 at 2560 x 6912, one token)
    // (from 1024 row blocks on the staged kernel's many small workgroups stay: 20480 x 3200 5.0 us against 5.9)
    const bool prod_solo_wanted = t_tune.prod_solo == 1 || (t_tune.prod_solo == 0 && t_tune.staged == 0 && ((N / 16) >= kManyBlocks || M > kDecodeMaxTokens) &&
                                                            (N / 16) < kSmallWorkgroupBlocks);
    if (prod_solo_wanted && t_tune.path != 2 && M <= 16) {
        const ProdPlan pp = plan_prod_solo(M, N, K);
        if (pp.ok && slot_rule(smap, N).ok)
            return launch_prod_solo(act, packed, out, acc_out, out ? s : (const uint16_t*)packed, out ? ws : (const uint16_t*)packed,
                                    smap, M, N, K, pp, stream, residual);
    }
    // (The accumulator export takes the same kernel choice as the drop-in call, so what the parity
    // tests read is what the drop-in entry computes.  Without an output there are no scales: the
    // kernel's unconditional scale requests then go to an address that exists.)
    if (t_tune.staged != 2 && t_tune.path != 2) {
        const FusedPlan pl = plan_fused(M, N, K, 3);
        // measured: up to 4 tokens staging always wins (2.8-4.5 us against 3.1-5.1 at the 2B shapes);
        // beyond, it pays once a workgroup shares the rows between two or more row blocks
        const bool wanted = t_tune.staged == 1 || M <= kDecodeMaxTokens || (N / 16) >= kManyBlocks;
        if (pl.ok && wanted)
            return launch_fused((const uint16_t*)act, packed, out, out ? ws : (const uint16_t*)packed, smap, nullptr,
                                nullptr, FusedExtras{nullptr, residual, 0.0f, 0, out ? s : (const uint16_t*)packed, acc_out},
                                M, N, K, 0, pl, stream);
    }
    return launch_splitk(act, packed, out, acc_out, s, ws, smap, M, N, K, stream, residual);
}

ScaleMap equal_slots(int N, int ws_num) {
    ScaleMap sm;
    sm.nseg = ws_num;
    for (int j = 0; j < kMaxSeg; ++j) sm.ends[j] = (j < ws_num) ? (j + 1) * (N / ws_num) : N;
    sm.ends[ws_num - 1] = N;
    return sm;
}

// What the matrix pipe sustains on this machine for given operand VALUES: a register-only loop of
// v_mfma_i32_32x32x32_i8 (three waves per SIMD on every CU, four accumulators per wave, no memory traffic).
// mode 0: all operands zero; 1: random int8 activations x random codes 1..3 (the products this library
// computes), eight operand pairs in rotation so that the inputs change with every MFMA.  The rate depends on
// the values: switching activity decides the power the pipe draws and with it the clock it is given.
__device__ __forceinline__ unsigned probe_hash32(unsigned x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

template <int MODE>
__global__ __launch_bounds__(256) void probe_mfma_i8_kernel(int iters, uint32_t* sink) {
    v16i acc[4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][r] = 0;
    v4i act[8], code[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const unsigned seed = (threadIdx.x * 8 + i) * 4 + blockIdx.x * 977;
        act[i] = v4i{0, 0, 0, 0};
        code[i] = v4i{0, 0, 0, 0};
        if (MODE == 1) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                act[i][j] = (int)probe_hash32(seed + j);
                const unsigned h = probe_hash32(seed + 50 + j);
                unsigned c = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) c |= (1u + ((h >> (8 * b)) & 0xffu) % 3u) << (8 * b);
                code[i][j] = (int)c;
            }
        }
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int a = 0; a < 4; ++a)
                acc[a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(code[(u * 3 + a) & 7], act[(u + 2 * a) & 7], acc[a], 0, 0, 0);
    }
    int x = 0;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) x ^= acc[a][r];
    if (sink && x == 0x12345678) sink[0] = (uint32_t)x;  // keeps the loop alive; practically never true
}

}  // namespace

extern "C" {

// Measurement probes (declared in include/bitlinear_probes.h): what a launch costs when the kernel does
// nothing, and when it only requests a matrix's bytes with the streaming kernel's access pattern.
__global__ void probe_empty_kernel() {}

// Two workgroups of one launch hand a counter back and forth through device memory: workgroup wa stores round r
// into its word and polls the other's word until it reads r, workgroup wb polls first and then stores.  Stores and
// loads are relaxed device-scope accesses (write-through, read past the caches), the cheapest form in which one
// workgroup can see another's data inside a launch.  Every poll is bounded: a side that runs out sets *gave_up
// and both sides stop after their own bound.
__global__ void probe_flag_roundtrip_kernel(uint32_t* flags, int wa, int wb, int rounds, int spin_limit, int* gave_up) {
    const int w = blockIdx.x;
    if (threadIdx.x != 0 || (w != wa && w != wb)) return;
    uint32_t* mine = flags + (w == wa ? 0 : 64);      // 256 bytes apart: different cache lines
    uint32_t* theirs = flags + (w == wa ? 64 : 0);
    bool bad = false;
    for (int r = 1; r <= rounds && !bad; ++r) {
        if (w == wa) __hip_atomic_store(mine, (uint32_t)r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int spins = 0;
        while (__hip_atomic_load(theirs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != (uint32_t)r)
            if (++spins > spin_limit) {
                bad = true;
                break;
            }
        if (w != wa && !bad) __hip_atomic_store(mine, (uint32_t)r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (bad) __hip_atomic_store(gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

int bitlinear_probe_empty(int blocks, int threads, void* stream) {
    if (blocks < 1 || threads < 1 || threads > 1024) return BITLINEAR_ERR_ARG;
    hipLaunchKernelGGL(probe_empty_kernel, dim3(blocks), dim3(threads), 0, (hipStream_t)stream);
    return hipGetLastError() == hipSuccess ? BITLINEAR_OK : BITLINEAR_ERR_LAUNCH;
}

int bitlinear_probe_flag_roundtrip(uint32_t* flags, int wg_a, int wg_b, int rounds, int* gave_up, void* stream) {
    if (!flags || !gave_up) return BITLINEAR_ERR_NULL;
    if (wg_a < 0 || wg_b < 0 || wg_a == wg_b || wg_a > 4095 || wg_b > 4095 || rounds < 1 || rounds > (1 << 20)) return BITLINEAR_ERR_ARG;
    const int blocks = (wg_a > wg_b ? wg_a : wg_b) + 1;
    // both workgroups must be resident at once: one wave each, far below what the machine holds
    hipLaunchKernelGGL(probe_flag_roundtrip_kernel, dim3(blocks), dim3(64), 0, (hipStream_t)stream, flags, wg_a, wg_b, rounds,
                       1 << 20, gave_up);
    return hipGetLastError() == hipSuccess ? BITLINEAR_OK : BITLINEAR_ERR_LAUNCH;
}

int bitlinear_probe_mfma_i8(int mode, int iters, uint32_t* sink, long long* ops, void* stream) {
    if ((mode != 0 && mode != 1) || iters < 1 || iters > (1 << 20)) return BITLINEAR_ERR_ARG;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return BITLINEAR_ERR_LAUNCH;
    const int blocks = 3 * cus;  // one wave per SIMD and workgroup, three workgroups per CU
    if (mode == 0)
        hipLaunchKernelGGL(probe_mfma_i8_kernel<0>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, iters, sink);
    else
        hipLaunchKernelGGL(probe_mfma_i8_kernel<1>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, iters, sink);
    if (ops) *ops = 2ll * 32 * 32 * 32 * 32 * (long long)iters * 4 * blocks;  // 32 MFMAs per iteration and wave
    return hipGetLastError() == hipSuccess ? BITLINEAR_OK : BITLINEAR_ERR_LAUNCH;
}

int bitlinear_probe_weight_stream(const int8_t* const* packed, int count, int N, int K, uint32_t* sink, void* stream) {
    refresh_tuning();
    if (!shape_ok(1, N, K)) return BITLINEAR_ERR_SHAPE;
    if (!packed || count < 1 || count > kStreamMaxProblems) return BITLINEAR_ERR_ARG;
    StreamProblem sp[kStreamMaxProblems];
    for (int i = 0; i < count; ++i) {
        if (!packed[i] || (((uintptr_t)packed[i]) & 15u)) return BITLINEAR_ERR_ARG;
        sp[i] = StreamProblem{packed[i], packed[i], nullptr, nullptr, nullptr};
    }
    // Nothing is multiplied, so a row block need not be a real one: with few row blocks the same bytes are
    // read as more, shorter pieces (a row block cut into 2, 4, ... runs of k), so that the probe stands for
    // the fastest way of requesting these bytes, not for one kernel's decomposition.
    while ((long long)count * (N / 16) < 2048 && (K % 128) == 0 && K >= 2048) {
        N *= 2;
        K /= 2;
    }
    return launch_stream(sp, count, 1, N, K, equal_slots(N, 1), nullptr, (hipStream_t)stream, false, sink);
}

int bitlinear_last_status(void) { return g_status; }

const char* bitlinear_last_kernel(void) { return g_last_kernel; }

const char* bitlinear_status_string(int status) {
    switch (status) {
        case BITLINEAR_OK: return "ok";
        case BITLINEAR_ERR_SHAPE: return "unsupported shape (need M >= 1, N % 16 == 0, K % 64 == 0)";
        case BITLINEAR_ERR_NULL: return "null pointer";
        case BITLINEAR_ERR_LAUNCH: return "kernel launch failed";
        case BITLINEAR_ERR_ARG: return "invalid argument";
        case BITLINEAR_ERR_SCRATCH:
            return "activation block beyond the static scratch (need M <= 16384 and M * K <= 16744448)";
        case BITLINEAR_ERR_CAPTURE:
            return "bitlinear_forward_bf16_static: the first call on a device must come from outside a stream capture";
        default: return "unknown status";
    }
}

int bitlinear_ws_num(int N, int K) {
    for (const ShapeWs& e : kShapeTable)
        if (e.n == N && e.k == K) return e.ws_num;
    return 1;
}

int bitlinear_set_tuning(int kernel, int a, int b, int c) {
    std::lock_guard<std::mutex> lock(g_tuning_mutex);
    Tuning& g = g_tuning_shared;
    if (kernel == 0) {
        g.path = g.waves = g.upw = g.staged = g.stream = g.stream_depth = g.stream_waves = g.solo = g.solo_coop = g.solo_rpw = g.prod_solo = g.tok = 0;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 6) {
        if (a < 0 || a > 2) return set_status(BITLINEAR_ERR_ARG);
        g.staged = a;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 7) {
        const bool depth_ok = b == 0 || b == 4 || b == 5 || b == 6 || b == 7 || b == 8 || b == 10;
        if (a < 0 || a > 2 || !depth_ok || c < 0 || c > 32) return set_status(BITLINEAR_ERR_ARG);
        g.stream = a;
        g.stream_depth = b;
        g.stream_waves = c;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 9) {
        if (a < 0 || a > 2 || b < 0 || b > 4) return set_status(BITLINEAR_ERR_ARG);
        g.solo_coop = a;
        g.solo_rpw = b;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 11) {
        if (a < 0 || a > 2) return set_status(BITLINEAR_ERR_ARG);
        g.tok = a;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 10) {
        if (a == 0 || a == 2) {
            g.prod_solo = a;
            return set_status(BITLINEAR_OK);
        }
        const bool upw_ok = c == 4 || c == 5 || c == 7 || c == 8;
        if (a != 1 || b < 1 || b > kMaxWaves || !upw_ok) return set_status(BITLINEAR_ERR_ARG);
        g.prod_solo = 1;
        g.prod_s = b;
        g.prod_upw = c;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 8) {
        if (a == 0 || a == 5) {
            g.solo = a;
            return set_status(BITLINEAR_OK);
        }
        const bool upw_ok = c == 4 || c == 5 || c == 7 || c == 8;
        if (a < 1 || a > kFusedMaxRB || b < 1 || a * b > kMaxWaves || !upw_ok) return set_status(BITLINEAR_ERR_ARG);
        g.solo = a;
        g.solo_s = b;
        g.solo_upw = c;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 2) {
        if (a == 0 && b == 0) {  // split-K kernel always, launch shape left to the library
            g.path = 2;
            g.waves = g.upw = 0;
            return set_status(BITLINEAR_OK);
        }
        if (a < 1 || a > kMaxWaves || !(b == 1 || b == 2 || b == 4 || b == 8))
            return set_status(BITLINEAR_ERR_ARG);
        g.path = 2;
        g.waves = a;
        g.upw = b;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 3) {
        const bool upw_ok = c == 4 || c == 5 || c == 8 || c == 10 || c == 16;
        if (a < 1 || a > kFusedMaxRB || b < 1 || a * b > kMaxWaves || !upw_ok) return set_status(BITLINEAR_ERR_ARG);
        g.path = 3;
        g.fused[0] = a;
        g.fused[1] = b;
        g.fused[2] = c;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 4) {
        g.path = 4;
        return set_status(BITLINEAR_OK);
    }
    if (kernel == 5) {
        if (a < 0 || a > 8 || b < 0 || b > 64 || (c != 0 && c != 1 && c != 2 && c != 4)) return set_status(BITLINEAR_ERR_ARG);
        g.path = 5;
        g.prefill_big = a;
        g.prefill_band = b;
        g.prefill_ks = c;
        return set_status(BITLINEAR_OK);
    }
    return set_status(BITLINEAR_ERR_ARG);
}

int bitlinear_int8xint2_acc_i32(const int8_t* input0, const int8_t* input1, int32_t* acc_out, uint16_t* output0,
                                const uint16_t* s, const uint16_t* ws, int M, int N, int K, void* stream) {
    refresh_tuning();
    if (!shape_ok(M, N, K)) return set_status(BITLINEAR_ERR_SHAPE);
    if (!input0 || !input1 || (!acc_out && !output0) || (output0 && (!s || !ws))) return set_status(BITLINEAR_ERR_NULL);
    return set_status(launch_gemv(input0, input1, output0, acc_out, s, ws, equal_slots(N, bitlinear_ws_num(N, K)), M,
                                  N, K, (hipStream_t)stream));
}

void bitlinear_int8xint2(int8_t* input0, int8_t* input1, uint16_t* output0, uint16_t* s, uint16_t* ws, int M, int N,
                         int K, void* stream) {
    refresh_tuning();
    if (!shape_ok(M, N, K)) {
        // same line the reference prints for a shape it has no kernel for (bitnet_kernels.cu:35)
        printf("required ladder gemm kernel: M %d, N %d, K %d\n", M, N, K);
        fflush(stdout);
        set_status(BITLINEAR_ERR_SHAPE);
        return;
    }
    if (!input0 || !input1 || !output0 || !s || !ws) {
        set_status(BITLINEAR_ERR_NULL);
        return;
    }
    set_status(launch_gemv(input0, input1, output0, nullptr, s, ws, equal_slots(N, bitlinear_ws_num(N, K)), M, N, K,
                           (hipStream_t)stream));
}

int bitlinear_int8xint2_grouped(const bitlinear_problem* problems, int count, void* stream) {
    refresh_tuning();
    if (count < 0) return set_status(BITLINEAR_ERR_ARG);
    if (count == 0) return set_status(BITLINEAR_OK);
    if (!problems) return set_status(BITLINEAR_ERR_NULL);
    // everything is checked before anything is launched
    for (int i = 0; i < count; ++i) {
        const bitlinear_problem& p = problems[i];
        if (!shape_ok(p.M, p.N, p.K)) return set_status(BITLINEAR_ERR_SHAPE);
        if (!p.input0 || !p.input1 || !p.output0 || !p.s || !p.ws) return set_status(BITLINEAR_ERR_NULL);
        if ((((uintptr_t)p.input0) | ((uintptr_t)p.input1)) & 15u) return set_status(BITLINEAR_ERR_ARG);
    }
    int i = 0;
    while (i < count) {
        const bitlinear_problem& p0 = problems[i];
        const ScaleMap sm = equal_slots(p0.N, bitlinear_ws_num(p0.N, p0.K));
        // a run of problems of one shape is one launch of the streaming kernel (one flat list of row blocks)
        int j = i + 1;
        while (j < count && j - i < kStreamMaxProblems && problems[j].M == p0.M && problems[j].N == p0.N &&
               problems[j].K == p0.K)
            ++j;
        const bool grouped = t_tune.stream != 2 && t_tune.path == 0 && stream_applicable(p0.M, p0.N, p0.K, sm) &&
                             (j - i > 1 || t_tune.stream == 1 || (p0.N / 16) >= kStreamMinBlocks);
        if (grouped) {
            StreamProblem sp[kStreamMaxProblems];
            for (int k = i; k < j; ++k)
                sp[k - i] = StreamProblem{problems[k].input0, problems[k].input1, problems[k].output0, problems[k].s, problems[k].ws};
            const int st = launch_stream(sp, j - i, p0.M, p0.N, p0.K, sm, nullptr, (hipStream_t)stream);
            if (st != BITLINEAR_OK) return set_status(st);
        } else {
            for (int k = i; k < j; ++k) {
                const bitlinear_problem& p = problems[k];
                const int st = launch_gemv(p.input0, p.input1, p.output0, nullptr, p.s, p.ws, sm, p.M, p.N, p.K,
                                           (hipStream_t)stream);
                if (st != BITLINEAR_OK) return set_status(st);
            }
        }
        i = j;
    }
    return set_status(BITLINEAR_OK);
}

// seg_ends[0 .. nseg) -> the kernels' table: strictly increasing, the last one N
static int segment_map(const int* seg_ends, int nseg, int N, ScaleMap* sm) {
    if (!seg_ends) return BITLINEAR_ERR_NULL;
    if (nseg < 1 || nseg > kMaxSeg) return BITLINEAR_ERR_ARG;
    sm->nseg = nseg;
    int prev = 0;
    for (int j = 0; j < kMaxSeg; ++j) {
        if (j < nseg) {
            if (seg_ends[j] <= prev || seg_ends[j] > N) return BITLINEAR_ERR_ARG;
            prev = seg_ends[j];
        }
        sm->ends[j] = (j < nseg) ? seg_ends[j] : N;
    }
    return prev == N ? BITLINEAR_OK : BITLINEAR_ERR_ARG;
}

int bitlinear_int8xint2_seg(const int8_t* input0, const int8_t* input1, uint16_t* output0, const uint16_t* s,
                            const uint16_t* ws, const int* seg_ends, int nseg, int M, int N, int K, void* stream) {
    refresh_tuning();
    if (!shape_ok(M, N, K)) return set_status(BITLINEAR_ERR_SHAPE);
    if (!input0 || !input1 || !output0 || !s || !ws || !seg_ends) return set_status(BITLINEAR_ERR_NULL);
    ScaleMap sm;
    const int st = segment_map(seg_ends, nseg, N, &sm);
    if (st != BITLINEAR_OK) return set_status(st);
    return set_status(launch_gemv(input0, input1, output0, nullptr, s, ws, sm, M, N, K, (hipStream_t)stream));
}

static int quant_absmax_impl(const uint16_t* x, int8_t* q, uint16_t* s, int32_t* rowsum, int M, int K, int mode, void* stream);

int bitlinear_quant_absmax(const uint16_t* x, int8_t* q, uint16_t* s, int M, int K, int mode, void* stream) {
    return quant_absmax_impl(x, q, s, nullptr, M, K, mode, stream);
}

int bitlinear_quant_absmax_rowsum(const uint16_t* x, int8_t* q, uint16_t* s, int32_t* rowsum, int M, int K, int mode,
                                  void* stream) {
    if (!rowsum) return set_status(BITLINEAR_ERR_NULL);
    return quant_absmax_impl(x, q, s, rowsum, M, K, mode, stream);
}

size_t bitlinear_repacked_size(int N, int K) {
    if (N < 16 || K < 64 || (N % 16) != 0 || (K % 64) != 0) return 0;
    return (size_t)N * (size_t)K / 4;
}

int bitlinear_repack(const int8_t* packed_ref, void* packed_out, int N, int K, void* stream) {
    const size_t bytes = bitlinear_repacked_size(N, K);
    if (bytes == 0) return set_status(BITLINEAR_ERR_SHAPE);
    if (!packed_ref || !packed_out) return set_status(BITLINEAR_ERR_NULL);
    if (packed_ref == packed_out) return set_status(BITLINEAR_OK);  // in place: nothing to do
    // the kernels consume the reference's layout as it is: the converter is a copy
    return set_status(hipMemcpyAsync(packed_out, packed_ref, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream) == hipSuccess
                          ? BITLINEAR_OK
                          : BITLINEAR_ERR_LAUNCH);
}

static int quant_absmax_impl(const uint16_t* x, int8_t* q, uint16_t* s, int32_t* rowsum, int M, int K, int mode, void* stream) {
    if (M < 1 || K < 8 || (K % 8) != 0) return set_status(BITLINEAR_ERR_SHAPE);
    if (!x || !q || !s) return set_status(BITLINEAR_ERR_NULL);
    if (mode != 0 && mode != 1) return set_status(BITLINEAR_ERR_ARG);
    // 256 threads keep rows of up to 8192 elements in registers between the two passes; longer rows
    // get more threads (a second pass that re-reads the row costs a chain of dependent loads)
    // two rows or more: a wave per row while a lane holds at most 8 vectors of the row (measured at K = 2560: 2.41 -> 2.18 us
    // at 8 rows, 2.45 -> 2.26 at 16, 4.49 -> 3.66 at 64, 5.79 -> 5.39 at 2048, 14.7 -> 12.4 at 8192; longer rows keep the
    // kernel below)
    if (M >= kQuantRowsMin && K <= 8 * 64 * 8) {
        const int per_lane = (K / 8 + 63) / 64;
        const dim3 grid((M + 3) / 4, 1, 1), block(256, 1, 1);
#define BITLINEAR_LAUNCH_QR(MODE_, V_) \
    BL_LAUNCH((quant_absmax_rows_kernel<MODE_, V_>), grid, block, 0, (hipStream_t)stream, x, q, s, M, K, rowsum)
#define BITLINEAR_LAUNCH_QR_V(V_)          \
    if (mode == 0) BITLINEAR_LAUNCH_QR(0, V_); \
    else BITLINEAR_LAUNCH_QR(1, V_)
        if (per_lane <= 2) { BITLINEAR_LAUNCH_QR_V(2); }
        else if (per_lane <= 5) { BITLINEAR_LAUNCH_QR_V(5); }
        else { BITLINEAR_LAUNCH_QR_V(8); }
#undef BITLINEAR_LAUNCH_QR_V
#undef BITLINEAR_LAUNCH_QR
        return set_status(launch_status());
    }
    int threads = kQuantThreads;
    while (threads < kQuantMaxThreads && K > threads * kQuantRegVecs * 8) threads *= 2;
    const dim3 grid(M, 1, 1), block(threads, 1, 1);
    if (mode == 0)
        BL_LAUNCH(quant_absmax_kernel<0>, grid, block, 0, (hipStream_t)stream, x, q, s, K, rowsum);
    else
        BL_LAUNCH(quant_absmax_kernel<1>, grid, block, 0, (hipStream_t)stream, x, q, s, K, rowsum);
    return set_status(launch_status());
}

// seg_ends == nullptr: the reference's equal slots (bitnet_kernels.h:80); otherwise the caller's segments
static int forward_impl(const uint16_t* x, const int8_t* packed, uint16_t* output0, int32_t* acc_out, const uint16_t* ws,
                        int8_t* q_ws, uint16_t* s_ws, int M, int N, int K, int mode, void* stream,
                        const int* seg_ends = nullptr, int nseg = 0) {
    refresh_tuning();
    if (!shape_ok(M, N, K)) return set_status(BITLINEAR_ERR_SHAPE);
    if (!x || !packed || !output0 || !ws) return set_status(BITLINEAR_ERR_NULL);
    if (mode != 0 && mode != 1) return set_status(BITLINEAR_ERR_ARG);
    if ((((uintptr_t)x) | ((uintptr_t)packed) | ((uintptr_t)q_ws)) & 15u) return set_status(BITLINEAR_ERR_ARG);
    ScaleMap sm = equal_slots(N, bitlinear_ws_num(N, K));
    if (seg_ends) {
        const int st = segment_map(seg_ends, nseg, N, &sm);
        if (st != BITLINEAR_OK) return set_status(st);
    }
    // up to four tokens: the kernel whose waves quantize their own slices
    if (mode == 0 && t_tune.path == 0 && t_tune.solo != 5 && M <= kSoloMaxTokens && slot_rule(sm, N).ok) {
        const SoloPlan sp = plan_solo(M, N, K);
        if (sp.ok && (t_tune.solo >= 1 || solo_wanted(M, N, K)))
            return set_status(launch_solo(x, packed, output0, acc_out, ws, sm, q_ws, s_ws, M, N, K, sp, (hipStream_t)stream));
    }
    // five to eight tokens, rows of up to 3200 values: the kernel whose lanes quantize for their own token
    if (mode == 0 && t_tune.path == 0 && t_tune.tok != 2 && M <= kTokMaxTokens && (t_tune.tok == 1 || (M >= kTokMinTokens && K <= kTokMaxK)) &&
        (long long)M * K * 2 < 0x7ffffff0ll && slot_rule(sm, N).ok) {
        const ProdPlan tp = plan_prod_solo(M, N, K);
        if (tok_plan_ok(M, tp) && (t_tune.tok == 1 || (N / 16 + tp.rpw - 1) / tp.rpw <= kTokMaxWorkgroups))
            return set_status(launch_solo_tok(x, packed, output0, acc_out, ws, sm, q_ws, s_ws, M, N, K, tp, (hipStream_t)stream));
    }
    const FusedPlan pl = plan_fused(M, N, K);
    // one kernel while the activation block is small enough for every workgroup to quantize it
    // again (or when the caller gave no workspaces for the two-kernel path)
    const bool small = (long long)M * K <= kFuseMaxElems || t_tune.path == 3 || !q_ws || !s_ws;
    if (pl.ok && small && t_tune.path != 4)
        return set_status(launch_fused(x, packed, output0, ws, sm, q_ws, s_ws,
                                       FusedExtras{nullptr, nullptr, 0.0f, 0, nullptr, acc_out}, M, N, K, mode, pl,
                                       (hipStream_t)stream));
    // larger blocks: the quantizer once, in a kernel of its own, then the product
    if (!q_ws || !s_ws) return set_status(BITLINEAR_ERR_NULL);
    const int st = bitlinear_quant_absmax(x, q_ws, s_ws, M, K, mode, stream);
    if (st != BITLINEAR_OK) return st;
    return set_status(launch_gemv(q_ws, packed, output0, acc_out, s_ws, ws, sm, M, N, K, (hipStream_t)stream));
}

int bitlinear_forward_bf16(const uint16_t* x, const int8_t* packed, uint16_t* output0, const uint16_t* ws,
                           int8_t* q_ws, uint16_t* s_ws, int M, int N, int K, int mode, void* stream) {
    return forward_impl(x, packed, output0, nullptr, ws, q_ws, s_ws, M, N, K, mode, stream);
}

int bitlinear_forward_bf16_seg(const uint16_t* x, const int8_t* packed, uint16_t* output0, const uint16_t* ws,
                               const int* seg_ends, int nseg, int8_t* q_ws, uint16_t* s_ws, int M, int N, int K, int mode,
                               void* stream) {
    if (!seg_ends) return set_status(BITLINEAR_ERR_NULL);
    return forward_impl(x, packed, output0, nullptr, ws, q_ws, s_ws, M, N, K, mode, stream, seg_ends, nseg);
}

// The array's name is only a handle on the host: its device address is looked up once per device
// (each GPU has its own copy) and kept.
static unsigned char* static_scratch_ptr(hipError_t* err, hipStream_t stream, bool* refused_under_capture) {
    static std::once_flag flags[bitnet_host::kMaxDevices];
    static unsigned char* ptrs[bitnet_host::kMaxDevices];
    static hipError_t results[bitnet_host::kMaxDevices];
    static std::atomic<bool> known[bitnet_host::kMaxDevices];
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= bitnet_host::kMaxDevices) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    if (!known[dev].load()) {
        // the look-up below is a host call that a stream capture in progress may refuse: the first call on a
        // device has to come from outside a capture, and says so instead of failing in some other way
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) {
            *refused_under_capture = true;
            return nullptr;
        }
    }
    std::call_once(flags[dev], [dev] {
        void* p = nullptr;
        results[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        ptrs[dev] = results[dev] == hipSuccess ? (unsigned char*)p : nullptr;
        known[dev].store(results[dev] == hipSuccess);
    });
    *err = results[dev];
    return ptrs[dev];
}

int bitlinear_forward_bf16_static(const uint16_t* x, const int8_t* packed, uint16_t* output0, const uint16_t* ws, int M,
                                  int N, int K, int mode, void* stream) {
    if (!shape_ok(M, N, K)) return set_status(BITLINEAR_ERR_SHAPE);
    if (M > kStaticMaxTokens || (size_t)M * (size_t)K > kStaticMaxElems) return set_status(BITLINEAR_ERR_SCRATCH);
    if (!x || !packed || !output0 || !ws) return set_status(BITLINEAR_ERR_NULL);
    hipError_t err = hipSuccess;
    bool under_capture = false;
    unsigned char* base = static_scratch_ptr(&err, (hipStream_t)stream, &under_capture);
    if (under_capture) return set_status(BITLINEAR_ERR_CAPTURE);
    if (err != hipSuccess || !base) return set_status(BITLINEAR_ERR_LAUNCH);
    return forward_impl(x, packed, output0, nullptr, ws, (int8_t*)(base + kStaticScaleBytes), (uint16_t*)base, M, N, K, mode,
                        stream);
}

int bitlinear_forward_bf16_acc_i32(const uint16_t* x, const int8_t* packed, int32_t* acc_out, uint16_t* output0,
                                   const uint16_t* ws, int8_t* q_ws, uint16_t* s_ws, int M, int N, int K, int mode,
                                   void* stream) {
    if (!acc_out) return set_status(BITLINEAR_ERR_NULL);
    return forward_impl(x, packed, output0, acc_out, ws, q_ws, s_ws, M, N, K, mode, stream);
}

static int norm_forward_impl(const uint16_t* x, const uint16_t* norm_weight, float eps, int glu, const int8_t* packed,
                             const uint16_t* ws, const uint16_t* residual, uint16_t* output0, int8_t* q_ws, uint16_t* s_ws,
                             int M, int N, int K, int mode, void* stream, const int* seg_ends, int nseg);

int bitlinear_norm_forward_bf16(const uint16_t* x, const uint16_t* norm_weight, float eps, int glu,
                                const int8_t* packed, const uint16_t* ws, const uint16_t* residual, uint16_t* output0,
                                int8_t* q_ws, uint16_t* s_ws, int M, int N, int K, int mode, void* stream) {
    return norm_forward_impl(x, norm_weight, eps, glu, packed, ws, residual, output0, q_ws, s_ws, M, N, K, mode, stream,
                             nullptr, 0);
}

int bitlinear_norm_forward_bf16_seg(const uint16_t* x, const uint16_t* norm_weight, float eps, int glu,
                                    const int8_t* packed, const uint16_t* ws, const int* seg_ends, int nseg,
                                    const uint16_t* residual, uint16_t* output0, int8_t* q_ws, uint16_t* s_ws, int M, int N,
                                    int K, int mode, void* stream) {
    if (!seg_ends) return set_status(BITLINEAR_ERR_NULL);
    return norm_forward_impl(x, norm_weight, eps, glu, packed, ws, residual, output0, q_ws, s_ws, M, N, K, mode, stream,
                             seg_ends, nseg);
}

static int norm_forward_impl(const uint16_t* x, const uint16_t* norm_weight, float eps, int glu, const int8_t* packed,
                             const uint16_t* ws, const uint16_t* residual, uint16_t* output0, int8_t* q_ws, uint16_t* s_ws,
                             int M, int N, int K, int mode, void* stream, const int* seg_ends, int nseg) {
    refresh_tuning();
    if (!shape_ok(M, N, K)) return set_status(BITLINEAR_ERR_SHAPE);
    if (!x || !norm_weight || !packed || !ws || !output0) return set_status(BITLINEAR_ERR_NULL);
    if (mode != 0 && mode != 1) return set_status(BITLINEAR_ERR_ARG);
    if ((((uintptr_t)x) | ((uintptr_t)packed) | ((uintptr_t)norm_weight) | ((uintptr_t)q_ws)) & 15u)
        return set_status(BITLINEAR_ERR_ARG);
    ScaleMap sm = equal_slots(N, bitlinear_ws_num(N, K));
    if (seg_ends) {
        const int st = segment_map(seg_ends, nseg, N, &sm);
        if (st != BITLINEAR_OK) return set_status(st);
    }
    // up to four tokens: the kernel whose waves prepare their own slices
    if (mode == 0 && t_tune.path == 0 && t_tune.solo != 5 && M <= kSoloMaxTokens && slot_rule(sm, N).ok) {
        const SoloPlan sp = plan_solo(M, N, K, glu ? 2 : 1, residual != nullptr);
        if (sp.ok && (t_tune.solo >= 1 || solo_norm_wanted(M, N, K, glu ? 2 : 1)))
            return set_status(launch_solo(x, packed, output0, nullptr, ws, sm, nullptr, nullptr, M, N, K, sp,
                                          (hipStream_t)stream, glu ? 2 : 1, norm_weight, eps, residual));
    }
    const FusedPlan pl = plan_fused(M, N, K, glu ? 2 : 1);
    const bool small = (long long)M * K <= kFuseMaxElemsNorm || t_tune.path == 3 || !q_ws || !s_ws;
    if (pl.ok && small && t_tune.path != 4) {
        const FusedExtras ex = {norm_weight, residual, eps, glu ? 1 : 0, nullptr, nullptr};
        return set_status(launch_fused(x, packed, output0, ws, sm, nullptr, nullptr, ex, M, N, K, mode, pl,
                                       (hipStream_t)stream));
    }
    // larger blocks: gate / norm / quantizer once per token row, then the product with the residual epilogue
    if (!q_ws || !s_ws) return set_status(pl.ok ? BITLINEAR_ERR_NULL : BITLINEAR_ERR_SHAPE);
    if (K > kPreThreads * kPreVecs * 8) return set_status(BITLINEAR_ERR_SHAPE);
    // very many rows, no gate, short rows: a wave per row (norm + product at K = 2560: 32.2 -> 30.1 us at 2048 rows,
    // 53.6 -> 48.7 at 4096; below 1024 rows 0.2-0.9 us behind, with the gate at K = 6912 4-7 us behind: not taken)
    if (M >= kNormRowsPerWaveMinRows && !glu && K <= 8 * 64 * 8) {
        const int per_lane = (K / 8 + 63) / 64;
        const dim3 rgrid((M + 3) / 4, 1, 1), rblock(256, 1, 1);
#define BITLINEAR_LAUNCH_NR(P, V) \
    BL_LAUNCH((norm_quant_rows_kernel<P, V>), rgrid, rblock, 0, (hipStream_t)stream, x, norm_weight, eps, q_ws, s_ws, M, K, mode)
#define BITLINEAR_LAUNCH_NR_V(V) BITLINEAR_LAUNCH_NR(1, V)
        if (per_lane <= 2) { BITLINEAR_LAUNCH_NR_V(2); }
        else if (per_lane <= 5) { BITLINEAR_LAUNCH_NR_V(5); }
        else { BITLINEAR_LAUNCH_NR_V(8); }
#undef BITLINEAR_LAUNCH_NR_V
#undef BITLINEAR_LAUNCH_NR
        if (launch_status() != BITLINEAR_OK) return set_status(BITLINEAR_ERR_LAUNCH);
        return set_status(launch_gemv(q_ws, packed, output0, nullptr, s_ws, ws, sm, M, N, K, (hipStream_t)stream, residual));
    }
    const dim3 grid(M, 1, 1), block(kPreThreads, 1, 1);
    const int per_thread = (K / 8 + kPreThreads - 1) / kPreThreads;
#define BITLINEAR_LAUNCH_PRE(P, V) \
    BL_LAUNCH((norm_quant_kernel<P, V>), grid, block, 0, (hipStream_t)stream, x, norm_weight, eps, q_ws, s_ws, K, mode)
#define BITLINEAR_LAUNCH_PRE_V(V)    \
    if (glu)                         \
        BITLINEAR_LAUNCH_PRE(2, V);  \
    else                             \
        BITLINEAR_LAUNCH_PRE(1, V)
    if (per_thread <= 1) {
        BITLINEAR_LAUNCH_PRE_V(1);
    } else if (per_thread <= 2) {
        BITLINEAR_LAUNCH_PRE_V(2);
    } else if (per_thread <= 4) {
        BITLINEAR_LAUNCH_PRE_V(4);
    } else {
        BITLINEAR_LAUNCH_PRE_V(8);
    }
#undef BITLINEAR_LAUNCH_PRE_V
#undef BITLINEAR_LAUNCH_PRE
    if (launch_status() != BITLINEAR_OK) return set_status(BITLINEAR_ERR_LAUNCH);
    return set_status(launch_gemv(q_ws, packed, output0, nullptr, s_ws, ws, sm, M, N, K, (hipStream_t)stream, residual));
}

int bitlinear_plan_name(int entry, int M, int N, int K, char* buf, int buflen) {
    if (!buf || buflen < 1) return set_status(BITLINEAR_ERR_NULL);
    buf[0] = 0;
    if (entry < 0 || entry > 4) return set_status(BITLINEAR_ERR_ARG);
    // operands of a planning call are never dereferenced, on the host or anywhere: any aligned address does
    uint16_t* const h = reinterpret_cast<uint16_t*>((uintptr_t)0x100000);
    int8_t* const b = reinterpret_cast<int8_t*>((uintptr_t)0x100000);
    t_plan.active = true;
    t_plan.text.clear();
    int st = BITLINEAR_OK;
    switch (entry) {
        case 0:
            bitlinear_int8xint2(b, b, h, h, h, M, N, K, nullptr);
            st = g_status;
            break;
        case 1: st = forward_impl(h, b, h, nullptr, h, b, h, M, N, K, 0, nullptr); break;
        default:
            st = norm_forward_impl(h, h, 1e-5f, entry == 4 ? 1 : 0, b, h, entry >= 3 ? h : nullptr, h, b, h, M, N, K, 0, nullptr,
                                   nullptr, 0);
            break;
    }
    t_plan.active = false;
    snprintf(buf, (size_t)buflen, "%s", t_plan.text.c_str());
    return set_status(st);
}

}  // extern "C"
