/*
 * CPU restatement of the reference's I2_S ternary dot kernels (x86 / AVX2
 * path, ACT_PARALLEL configuration).
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker and the timed CPU
 * baseline.  Nothing in the product library links or calls it.
 *
 * What it follows (paths relative to the reference tree):
 *   layout        src/ggml-bitnet-mad.cpp:51-92   quantize_i2_s, x86 ACT_PARALLEL
 *   1x1 dot       src/ggml-bitnet-mad.cpp:198-296 ggml_vec_dot_i2_i8_s_1x1
 *   Nx1 dot       src/ggml-bitnet-mad.cpp:791-887 ggml_vec_dot_i2_i8_s_Nx1
 *   dispatch      src/ggml-bitnet-mad.cpp:1043-1056
 *   tiling        utils/test_gemm_kernel.sh:137-154 (ggml_gemm_i2_i8_s)
 *   tile sizes    include/gemm-config.h:1-11 (ROW 4, COL 128, PARALLEL 4)
 *
 * Layout: a weight row of n ternary values is n/128 blocks of 32 bytes; byte
 * p of a block holds elements p, 32+p, 64+p, 96+p of the block as unsigned
 * codes q = w + 1 in bit pairs 7:6, 5:4, 3:2, 1:0.
 *
 * The dot functions return sum_k q[k] * y[k] (as float, like the reference);
 * the caller owes the "- sum_k y[k]" that turns q back into w.  The wrapper
 * that does so in the reference lives in a submodule that is not part of the
 * reference tree, so i2s_bitlinear_* below applies it explicitly.
 *
 * Arithmetic detail kept from the reference: products are formed by
 * maddubs (u8 x s8 -> saturating s16 pair sums) and summed in int16 lanes
 * for up to 32 blocks before widening to int32, so the result equals the
 * exact integer sum whenever no int16 lane overflows (always true for
 * |y| <= 127 and codes <= 2 with up to 32 blocks: 32*4*2*2*127 = 65024 can
 * exceed 32767 only for adversarial same-sign data).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__AVX2__)
#include <immintrin.h>
#endif

#define I2S_BLOCK 128     /* QK_I2_S on x86 */
#define I2S_PARALLEL 4    /* PARALLEL_SIZE  */
#define I2S_ROW_TILE 4    /* ROW_BLOCK_SIZE */
#define I2S_COL_TILE 128  /* COL_BLOCK_SIZE */

/* ---- layout --------------------------------------------------------------*/

/* Ternary int8 [n] -> n/4 bytes in the x86 I2_S layout. */
void i2s_pack_row(const int8_t* w, uint8_t* dst, int64_t n) {
    memset(dst, 0, (size_t)(n / 4));
    for (int64_t blk = 0; blk < n / I2S_BLOCK; ++blk)
        for (int e = 0; e < I2S_BLOCK; ++e) {
            const uint8_t code = (uint8_t)(w[blk * I2S_BLOCK + e] + 1);
            dst[blk * 32 + (e % 32)] |= (uint8_t)(code << (6 - 2 * (e / 32)));
        }
}

/* Float weights -> codes the way the reference quantizer classifies them:
 * |x| < 1e-6 -> 0, otherwise the sign.  Returns the tensor scale (max |x|),
 * which the reference appends after the packed bytes. */
float i2s_quantize(const float* src, uint8_t* dst, int64_t nrow, int64_t n_per_row) {
    const int64_t n = nrow * n_per_row;
    double mx = 0.0;
    for (int64_t i = 0; i < n; ++i) {
        const double a = src[i] < 0 ? -(double)src[i] : (double)src[i];
        if (a > mx) mx = a;
    }
    int8_t* t = (int8_t*)malloc((size_t)n);
    for (int64_t i = 0; i < n; ++i) {
        const double a = src[i] < 0 ? -(double)src[i] : (double)src[i];
        t[i] = a < 1e-6 ? 0 : ((double)src[i] * mx > 0 ? 1 : -1);
    }
    i2s_pack_row(t, dst, n); /* blocks never straddle rows when n_per_row % 128 == 0 */
    free(t);
    return (float)mx;
}

/* ---- dot kernels ---------------------------------------------------------*/

#if defined(__AVX2__)
static inline int hsum8_i32(__m256i v) {
    __m128i s = _mm_add_epi32(_mm256_castsi256_si128(v), _mm256_extracti128_si256(v, 1));
    s = _mm_add_epi32(s, _mm_unpackhi_epi64(s, s));
    s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0xB1));
    return _mm_cvtsi128_si32(s);
}

/* One 128-element block: 32 packed bytes against 128 int8, int16 lane sums. */
static inline __m256i block_i16(const uint8_t* px, const int8_t* py) {
    const __m256i m3 = _mm256_set1_epi8(3);
    const __m256i x = _mm256_loadu_si256((const __m256i*)px);
    const __m256i g0 = _mm256_and_si256(_mm256_srli_epi16(x, 6), m3); /* elements   0..31  */
    const __m256i g1 = _mm256_and_si256(_mm256_srli_epi16(x, 4), m3); /* elements  32..63  */
    const __m256i g2 = _mm256_and_si256(_mm256_srli_epi16(x, 2), m3); /* elements  64..95  */
    const __m256i g3 = _mm256_and_si256(x, m3);                       /* elements  96..127 */
    const __m256i p0 = _mm256_maddubs_epi16(g0, _mm256_loadu_si256((const __m256i*)(py)));
    const __m256i p1 = _mm256_maddubs_epi16(g1, _mm256_loadu_si256((const __m256i*)(py + 32)));
    const __m256i p2 = _mm256_maddubs_epi16(g2, _mm256_loadu_si256((const __m256i*)(py + 64)));
    const __m256i p3 = _mm256_maddubs_epi16(g3, _mm256_loadu_si256((const __m256i*)(py + 96)));
    return _mm256_add_epi16(_mm256_add_epi16(p0, p1), _mm256_add_epi16(p2, p3));
}

/* sum over all blocks of one weight row against one activation row */
static int dot_row(const uint8_t* x, const int8_t* y, int nblocks) {
    const __m256i ones = _mm256_set1_epi16(1);
    __m256i acc32 = _mm256_setzero_si256();
    int done = 0;
    while (done < nblocks) { /* widen every 32 blocks, as the reference does */
        const int chunk = nblocks - done < 32 ? nblocks - done : 32;
        __m256i acc16 = _mm256_setzero_si256();
        for (int j = 0; j < chunk; ++j)
            acc16 = _mm256_add_epi16(acc16, block_i16(x + (size_t)(done + j) * 32, y + (size_t)(done + j) * 128));
        acc32 = _mm256_add_epi32(acc32, _mm256_madd_epi16(acc16, ones));
        done += chunk;
    }
    return hsum8_i32(acc32);
}
#else
static int dot_row(const uint8_t* x, const int8_t* y, int nblocks) {
    int sum = 0;
    for (int b = 0; b < nblocks; ++b)
        for (int p = 0; p < 32; ++p) {
            const uint8_t v = x[b * 32 + p];
            sum += ((v >> 6) & 3) * y[b * 128 + p] + ((v >> 4) & 3) * y[b * 128 + 32 + p] +
                   ((v >> 2) & 3) * y[b * 128 + 64 + p] + (v & 3) * y[b * 128 + 96 + p];
        }
    return sum;
}
#endif

/* _1x1: nrc weight rows (stride bx/4 bytes) against one activation row. */
void i2s_vec_dot_1x1(int n, float* s, size_t bs, const void* vx, size_t bx, const void* vy, size_t by, int nrc) {
    (void)bs;
    (void)by;
    const uint8_t* x = (const uint8_t*)vx;
    for (int row = 0; row < nrc; ++row)
        s[row] = (float)dot_row(x + (size_t)row * bx / 4, (const int8_t*)vy, n / I2S_BLOCK);
}

/* _Nx1: one weight row against nrc activation rows (stride by bytes), four
 * activation rows at a time sharing each decoded weight block; result for
 * activation row c goes to s[c * bs]. */
void i2s_vec_dot_Nx1(int n, float* s, size_t bs, const void* vx, size_t bx, const void* vy, size_t by, int nrc) {
    (void)bx;
    const uint8_t* x = (const uint8_t*)vx;
    const int8_t* y = (const int8_t*)vy;
    const int nblocks = n / I2S_BLOCK;
#if defined(__AVX2__)
    const __m256i ones = _mm256_set1_epi16(1);
    const __m256i m3 = _mm256_set1_epi8(3);
    for (int col = 0; col < nrc; col += I2S_PARALLEL) {
        __m256i acc32[I2S_PARALLEL];
        for (int t = 0; t < I2S_PARALLEL; ++t) acc32[t] = _mm256_setzero_si256();
        int done = 0;
        while (done < nblocks) {
            const int chunk = nblocks - done < 32 ? nblocks - done : 32;
            __m256i acc16[I2S_PARALLEL];
            for (int t = 0; t < I2S_PARALLEL; ++t) acc16[t] = _mm256_setzero_si256();
            for (int j = 0; j < chunk; ++j) {
                const __m256i xv = _mm256_loadu_si256((const __m256i*)(x + (size_t)(done + j) * 32));
                const __m256i g0 = _mm256_and_si256(_mm256_srli_epi16(xv, 6), m3);
                const __m256i g1 = _mm256_and_si256(_mm256_srli_epi16(xv, 4), m3);
                const __m256i g2 = _mm256_and_si256(_mm256_srli_epi16(xv, 2), m3);
                const __m256i g3 = _mm256_and_si256(xv, m3);
                for (int t = 0; t < I2S_PARALLEL; ++t) {
                    const int8_t* py = y + (size_t)(col + t) * by + (size_t)(done + j) * 128;
                    const __m256i a = _mm256_add_epi16(
                        _mm256_maddubs_epi16(g0, _mm256_loadu_si256((const __m256i*)(py))),
                        _mm256_maddubs_epi16(g1, _mm256_loadu_si256((const __m256i*)(py + 32))));
                    const __m256i b = _mm256_add_epi16(
                        _mm256_maddubs_epi16(g2, _mm256_loadu_si256((const __m256i*)(py + 64))),
                        _mm256_maddubs_epi16(g3, _mm256_loadu_si256((const __m256i*)(py + 96))));
                    acc16[t] = _mm256_add_epi16(acc16[t], _mm256_add_epi16(a, b));
                }
            }
            for (int t = 0; t < I2S_PARALLEL; ++t)
                acc32[t] = _mm256_add_epi32(acc32[t], _mm256_madd_epi16(acc16[t], ones));
            done += chunk;
        }
        for (int t = 0; t < I2S_PARALLEL; ++t) s[(size_t)(col + t) * bs] = (float)hsum8_i32(acc32[t]);
    }
#else
    for (int col = 0; col < nrc; ++col) s[(size_t)col * bs] = (float)dot_row(x, y + (size_t)col * by, nblocks);
#endif
}

/* Dispatcher: multiples of PARALLEL_SIZE take the Nx1 kernel (ACT_PARALLEL),
 * anything else the 1x1 kernel -- note the two interpret nrc differently. */
void i2s_vec_dot(int n, float* s, size_t bs, const void* vx, size_t bx, const void* vy, size_t by, int nrc) {
    if (nrc % I2S_PARALLEL == 0)
        i2s_vec_dot_Nx1(n, s, bs, vx, bx, vy, by, nrc);
    else
        i2s_vec_dot_1x1(n, s, bs, vx, bx, vy, by, nrc);
}

/* Tiled GEMM driver: s[r * bs + c] = dot(weight row c, activation row r) for
 * c in [c_begin, c_end), r in [0, nr); column tiles of 128 outermost, row
 * tiles of 4 inside, one dispatcher call per weight row and row tile. */
static void gemm_cols(int n, float* s, size_t bs, const uint8_t* vx, const int8_t* vy, int nr, int c_begin, int c_end) {
    for (int c0 = c_begin; c0 < c_end; c0 += I2S_COL_TILE) {
        const int c1 = c0 + I2S_COL_TILE < c_end ? c0 + I2S_COL_TILE : c_end;
        for (int r0 = 0; r0 < nr; r0 += I2S_ROW_TILE) {
            const int cur_r = r0 + I2S_ROW_TILE <= nr ? I2S_ROW_TILE : nr - r0;
            for (int c = c0; c < c1; ++c)
                i2s_vec_dot(n, s + c + (size_t)r0 * bs, bs, vx + (size_t)c * n / 4, (size_t)n,
                            vy + (size_t)r0 * n, (size_t)n, cur_r);
        }
    }
}

void i2s_gemm(int n, float* s, size_t bs, const void* vx, const void* vy, int nr, int nc) {
    /* A row tail that is not a multiple of 4 goes through the 1x1 kernel, whose nrc
     * counts WEIGHT rows; the reference harness only uses nr % 4 == 0 or nr == 1.
     * For other tails each remaining activation row is issued on its own. */
    const int nr4 = nr == 1 ? 1 : nr - nr % I2S_ROW_TILE;
    gemm_cols(n, s, bs, (const uint8_t*)vx, (const int8_t*)vy, nr4, 0, nc);
    for (int r = nr4; r < nr; ++r)
        gemm_cols(n, s + (size_t)r * bs, bs, (const uint8_t*)vx, (const int8_t*)vy + (size_t)r * n, 1, 0, nc);
}

/* ---- BitLinear on top of the dot kernels ----------------------------------*/

/* Weight rows [c_begin, c_end) of the product for all M activation rows. */
static void bitlinear_cols(const uint8_t* x, const int8_t* y, int32_t* acc, float* tmp, int M, int N, int K,
                           int c_begin, int c_end) {
    const int nr4 = M == 1 ? 1 : M - M % I2S_ROW_TILE;
    gemm_cols(K, tmp, (size_t)N, x, y, nr4, c_begin, c_end);
    for (int r = nr4; r < M; ++r) gemm_cols(K, tmp + (size_t)r * N, (size_t)N, x, y + (size_t)r * K, 1, c_begin, c_end);
    for (int m = 0; m < M; ++m) {
        int ysum = 0;
        for (int k = 0; k < K; ++k) ysum += y[(size_t)m * K + k];
        for (int c = c_begin; c < c_end; ++c)
            acc[(size_t)m * N + c] = (int32_t)tmp[(size_t)m * N + c] - ysum; /* q = w + 1 */
    }
}

/* acc[m, n] = sum_k w[n, k] * y[m, k] from I2_S-packed weights, weight rows
 * split contiguously over nthreads OpenMP threads (ggml splits the rows of
 * the weight matrix across its thread pool in the same way; the reference's
 * own harness is built with -fopenmp, utils/test_gemm_kernel.sh:392-397).
 * tmp is float [M, N]. */
void i2s_bitlinear_acc(const void* packed, const int8_t* y, int32_t* acc, float* tmp, int M, int N, int K, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    const int per = (N + nthreads - 1) / nthreads;
    if (nthreads == 1) {
        bitlinear_cols((const uint8_t*)packed, y, acc, tmp, M, N, K, 0, N);
        return;
    }
#pragma omp parallel for num_threads(nthreads) schedule(static, 1)
    for (int t = 0; t < nthreads; ++t) {
        const int b = t * per, e = b + per < N ? b + per : N;
        if (b < e) bitlinear_cols((const uint8_t*)packed, y, acc, tmp, M, N, K, b, e);
    }
}

int i2s_has_avx2(void) {
#if defined(__AVX2__)
    return 1;
#else
    return 0;
#endif
}
