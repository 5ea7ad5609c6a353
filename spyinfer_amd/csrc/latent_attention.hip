// Attention over a cache of latent vectors: per token the cache holds one row [c (R) | kr (DR)] shared by all heads,
// c a normed low-rank vector from which keys and values are expanded (k_h = Wuk_h c, v_h = Wuv_h c) and kr a rotated key
// part.  The expansion is never formed: with qa_h = Wuk_h^T q_h the score is (qa_h . c + qr_h . kr) * scale, and the
// head's output is Wuv_h (sum_j p_j c_j).  So the kernels here see one "key" row of R + DR values and one "value" row of
// R values (its first part) per token and H query rows per token against them.
//
//   spy_latent_prepare         c = rmsnorm(dkv[:R]) * w and kr = rotate(dkv[R:]) into the pages; the heads' rotated query
//                              parts into the absorbed query rows
//   spy_head_products          the per-head products with Wuk and Wuv on MFMA, few rows (many rows: the library's batched product)
//   spy_latent_attention_mfma  bfloat16: 64 or 128 query rows a block against key chunks staged once in LDS; keys in parts for
//                              steps of single tokens, merged by a second kernel
//   spy_latent_attention       plain kernel, float32: one block per (token, head); the same window and sink
//   spy_gemm_strided           batched product with element strides, float32 sums (the float32 path's per-head products)
#include "common.h"
#include <math.h>

// ---------------------------------------------------------------------------------------------
// Rotation: pair (i, i + dims/2), i < dims/2, of the rotated part; angle = position * freq[i] in float32, cos and sin
// times `mag`.  Values beyond `dims` pass unchanged.
#define LP_MAX_PAIRS 512
template <typename TA, typename TW, typename TQ>
__global__ void latent_prepare_kernel(TQ* __restrict__ qa, const TA* __restrict__ q, int ldq, const TA* __restrict__ dkv, int ldd,
                                      TA* __restrict__ cache, const int* __restrict__ slot_mapping, long long cache_rows,
                                      const TW* __restrict__ w_norm, float eps, const float* __restrict__ freq, float mag,
                                      int dims, const int* __restrict__ positions, int H, int DN, int DR, int R, int interleaved) {
    // interleaved: pair j of the rotated dims is (2 j, 2 j + 1) instead of (j, j + dims / 2)
    __shared__ float red[16];
    __shared__ float cs[LP_MAX_PAIRS], sn[LP_MAX_PAIRS];
    const int t = blockIdx.x;
    const float p = (float)positions[t];
    const int half = dims / 2;
    // the token's cos and sin of every rotated pair, once for the block (all heads and the shared key part use them)
    for (int j = threadIdx.x; j < half; j += blockDim.x) {
        const float ang = p * freq[j];
        cs[j] = cosf(ang) * mag;
        sn[j] = sinf(ang) * mag;
    }
    __syncthreads();
    // the heads' rotated parts -> qa[t, h, R ..]
    for (int idx = threadIdx.x; idx < H * DR; idx += blockDim.x) {
        const int h = idx / DR, i = idx - h * DR;
        const TA* src = q + (size_t)t * ldq + (size_t)h * (DN + DR) + DN;
        float v = to_f32<TA>(src[i]);
        if (i < dims) {
            const bool first = interleaved ? !(i & 1) : i < half;
            const int j = interleaved ? i >> 1 : (i < half ? i : i - half);
            const float a = to_f32<TA>(src[interleaved ? 2 * j : j]), b = to_f32<TA>(src[interleaved ? 2 * j + 1 : j + half]);
            v = first ? a * cs[j] - b * sn[j] : b * cs[j] + a * sn[j];
        }
        qa[((size_t)t * H + h) * (R + DR) + R + i] = from_f32<TQ>(v);
    }
    if (!dkv) return;
    const long long slot = slot_mapping[t];
    const TA* d = dkv + (size_t)t * ldd;
    float ss = 0.f;
    for (int i = threadIdx.x; i < R; i += blockDim.x) { const float v = to_f32<TA>(d[i]); ss += v * v; }
    ss = block_sum(ss, red);
    if (slot < 0 || slot >= cache_rows) return;
    TA* row = cache + (size_t)slot * (R + DR);
    const float scale = 1.0f / sqrtf(ss / (float)R + eps);
    for (int i = threadIdx.x; i < R; i += blockDim.x) row[i] = from_f32<TA>((scale * to_f32<TA>(d[i])) * to_f32<TW>(w_norm[i]));
    for (int i = threadIdx.x; i < DR; i += blockDim.x) {
        float v = to_f32<TA>(d[R + i]);
        if (i < dims) {
            const bool first = interleaved ? !(i & 1) : i < half;
            const int j = interleaved ? i >> 1 : (i < half ? i : i - half);
            const float a = to_f32<TA>(d[R + (interleaved ? 2 * j : j)]), b = to_f32<TA>(d[R + (interleaved ? 2 * j + 1 : j + half)]);
            v = first ? a * cs[j] - b * sn[j] : b * cs[j] + a * sn[j];
        }
        row[R + i] = from_f32<TA>(v);
    }
}

extern "C" int spy_latent_prepare(void* qa, int qa_dtype, const void* q, int ldq, const void* dkv, int ldd, int dtype, void* cache,
                                  const int* slot_mapping, long long cache_rows, const void* w_norm, int w_dtype, float eps,
                                  const float* freq, float mag, int dims, const int* positions, int T, int H, int DN, int DR, int R,
                                  int interleaved, hipStream_t st) {
    SPY_REQUIRE(T > 0 && H > 0 && DN >= 0 && DR >= 0 && R > 0, "spy_latent_prepare: empty operand");
    SPY_REQUIRE(dims >= 0 && dims <= DR && dims % 2 == 0 && (dims == 0 || freq) && dims / 2 <= LP_MAX_PAIRS,
                "spy_latent_prepare: %d rotated dims of %d (an even number up to %d)", dims, DR, 2 * LP_MAX_PAIRS);
    SPY_REQUIRE(!dkv || (cache && slot_mapping && w_norm), "spy_latent_prepare: storing needs the cache, the tokens' slots and the norm weight");
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, SPY_DISPATCH(qa_dtype, TQ, (latent_prepare_kernel<TA, TW, TQ><<<T, 256, 0, st>>>(
        (TQ*)qa, (const TA*)q, ldq, (const TA*)dkv, ldd, (TA*)cache, slot_mapping, cache_rows, (const TW*)w_norm, eps, freq, mag, dims,
        positions, H, DN, DR, R, interleaved)))));
    SPY_CHECK_LAUNCH("spy_latent_prepare");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// C[b][m][n] = sum_k A[b][m][k] * B[b][n][k], element strides for every index, float32 products and sums in ascending k.
// A 64 x 64 tile of C per block as in the plain product; blockIdx.z = b.
#define GS_T 64
#define GS_K 16
template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(256) void gemm_strided_kernel(const TA* __restrict__ A, long long ab, long long am, long long ak,
                                                           const TB* __restrict__ B, long long bb, long long bn, long long bk,
                                                           TC* __restrict__ C, long long cb, long long cm, long long cn, int M, int N, int K) {
    __shared__ float As[GS_K][GS_T + 4];
    __shared__ float Bs[GS_K][GS_T + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GS_T, n0 = blockIdx.x * GS_T;
    A += (size_t)blockIdx.z * ab; B += (size_t)blockIdx.z * bb; C += (size_t)blockIdx.z * cb;
    float acc[4][4] = {};
    // A's k is the fast index of its loads where ak == 1 (rows of 16 k values), B's n or k whichever has stride 1
    const int lr = threadIdx.x >> 2, lk = (threadIdx.x & 3) * 4;
    for (int k0 = 0; k0 < K; k0 += GS_K) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e;
            const int m = m0 + lr, n = n0 + lr;
            As[lk + e][lr] = (m < M && k < K) ? to_f32<TA>(A[(size_t)m * am + (size_t)k * ak]) : 0.f;
            Bs[lk + e][lr] = (n < N && k < K) ? to_f32<TB>(B[(size_t)n * bn + (size_t)k * bk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GS_K; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[k][ty * 4 + i]; b[i] = Bs[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[(size_t)m * cm + (size_t)n * cn] = from_f32<TC>(acc[i][j]);
        }
    }
}

extern "C" int spy_gemm_strided(const void* A, int a_dtype, long long ab, long long am, long long ak, const void* B, int b_dtype,
                                long long bb, long long bn, long long bk, void* C, int c_dtype, long long cb, long long cm,
                                long long cn, int batch, int M, int N, int K, hipStream_t st) {
    SPY_REQUIRE(batch > 0 && M > 0 && N > 0 && K > 0, "spy_gemm_strided: empty operand");
    const dim3 grid((N + GS_T - 1) / GS_T, (M + GS_T - 1) / GS_T, batch);
    SPY_REQUIRE(grid.y <= 65535 && batch <= 65535, "spy_gemm_strided: M = %d or batch = %d is too large for this kernel", M, batch);
    SPY_DISPATCH(a_dtype, TA, SPY_DISPATCH(b_dtype, TB, SPY_DISPATCH(c_dtype, TC, (gemm_strided_kernel<TA, TB, TC><<<grid, 256, 0, st>>>(
        (const TA*)A, ab, am, ak, (const TB*)B, bb, bn, bk, (TC*)C, cb, cm, cn, M, N, K)))));
    SPY_CHECK_LAUNCH("spy_gemm_strided");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Plain attention over latent rows: one block per (token, head).  qa [T, H, R + DR] float32; cache [pages, P, R + DR];
// out [T, H, R] = sum_j p_j c_j with p = softmax over the keys the token sees and one more term, exp(sink_h), that has no
// key and no value.  Position i sees j with 0 <= i - j < window (window <= 0: all j <= i).  Keys in chunks of
// LA_THREADS with a running maximum that starts at the sink (so the denominator starts at 1).
#define LA_THREADS 256
#define LA_MAX_D 1024
template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(LA_THREADS) void latent_attention_kernel(
    TO* __restrict__ out, const float* __restrict__ qa, const TA* __restrict__ cache, int P, int num_pages,
    const int* __restrict__ kv_len, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_entry,
    const int* __restrict__ positions, const TW* __restrict__ sink, int H, int R, int DR, float scale, int window) {
    __shared__ float qs[LA_MAX_D];
    __shared__ float ps[LA_THREADS];
    __shared__ long long ro[LA_THREADS];
    __shared__ float red[4];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int D = R + DR;
    const int s = token_entry[t];
    const int p = positions[t];
    int hi = p;
    if (hi > kv_len[s] - 1) hi = kv_len[s] - 1;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const float* qv = qa + ((size_t)t * H + h) * D;
    for (int j = tid; j < D; j += LA_THREADS) qs[j] = qv[j];
    float acc[LA_MAX_D / LA_THREADS] = {};
    float m = sink ? to_f32<TW>(sink[h]) : -INFINITY;
    float l = sink ? 1.f : 0.f;
    const int* bt = block_table + (size_t)s * max_blocks;
    __syncthreads();
    for (int c0 = lo; c0 <= hi; c0 += LA_THREADS) {
        const int c = c0 + tid;
        float sc = -INFINITY;
        long long row = -1;
        if (c <= hi) {
            const int page = bt[c / P];
            if (page >= 0 && page < num_pages) {
                row = ((long long)page * P + c % P) * D;
                const TA* kr = cache + row;
                float dot = 0.f;
                for (int j = 0; j < D; ++j) dot = fmaf(qs[j], to_f32<TA>(kr[j]), dot);
                sc = dot * scale;
            }
        }
        const float cm = block_max(sc, red);
        const float m_new = fmaxf(m, cm);
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float pr = (sc == -INFINITY) ? 0.f : expf(sc - m_new);
        ps[tid] = pr; ro[tid] = row;
        const float csum = block_sum(pr, red);      // has the barriers that publish ps and ro
        l = l * alpha + csum;
        m = m_new;
        const int nk = min(LA_THREADS, hi - c0 + 1);
#pragma unroll
        for (int r = 0; r < LA_MAX_D / LA_THREADS; ++r) {
            const int j = tid + r * LA_THREADS;
            if (j < R) {
                float a = acc[r] * alpha;
                for (int i = 0; i < nk; ++i)
                    if (ro[i] >= 0) a = fmaf(ps[i], to_f32<TA>(cache[ro[i] + j]), a);
                acc[r] = a;
            }
        }
        __syncthreads();
    }
    TO* o = out + ((size_t)t * H + h) * R;
#pragma unroll
    for (int r = 0; r < LA_MAX_D / LA_THREADS; ++r) {
        const int j = tid + r * LA_THREADS;
        if (j < R) o[j] = from_f32<TO>(l > 0.f ? acc[r] / l : 0.f);
    }
}

extern "C" int spy_latent_attention(void* out, int out_dtype, const float* qa, const void* cache, int dtype, int P, int num_pages,
                                    const int* kv_len, const int* block_table, int max_blocks, const int* token_entry,
                                    const int* positions, const void* sink, int sink_dtype, int S, int T, int H, int R, int DR,
                                    float scale, int window, hipStream_t st) {
    SPY_REQUIRE(T > 0 && S > 0 && H > 0 && R > 0 && DR >= 0 && P > 0 && num_pages > 0 && max_blocks > 0,
                "spy_latent_attention: empty operand");
    SPY_REQUIRE(R + DR <= LA_MAX_D, "spy_latent_attention: rows of %d values exceed the supported %d", R + DR, LA_MAX_D);
    SPY_REQUIRE(H <= 65535, "spy_latent_attention: too many heads");
    const dim3 grid(T, H);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(sink_dtype, TW, SPY_DISPATCH(out_dtype, TO, (latent_attention_kernel<TA, TW, TO><<<grid, LA_THREADS, 0, st>>>(
        (TO*)out, qa, (const TA*)cache, P, num_pages, kv_len, block_table, max_blocks, token_entry, positions, (const TW*)sink, H, R,
        DR, scale, window)))));
    SPY_CHECK_LAUNCH("spy_latent_attention");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// The same attention on MFMA for bfloat16 caches.  All heads of a token read the same latent rows, so the query rows of
// an entry, (token, head) pairs, token major, are one long list against one "kv head": a block of LW waves takes
// 16 LW consecutive rows of bfloat16 queries (a row tile per wave), walks the keys that its rows' tokens see in chunks of 32, and stages every
// chunk in LDS ONCE for all its waves (two buffers in turn), in two forms: rows [key][D] for S^T = K . Q^T and, for the first R values, the
// transpose [d][key] for O^T += V^T . P^T (the values are the keys' first part: no second read of memory).  With
// v_mfma_f32_16x16x32_bf16 tile a of S^T takes keys 8 (r / 4) + r % 4 and tile b those + 4, so that lane (q row, g) holds
// the scores of keys 8 g .. 8 g + 7, exactly the 8 k values of its P^T operand.  Softmax float32, online, the sink in
// the first part's start (m = sink, l = 1).  grid.y parts of the keys (steps of single tokens): the parts' (O, m, l) go
// to a workspace and a second kernel adds them.
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short lbf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float lf32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t lu32x4_t;

#define LKPAD 8       // bf16 of padding per staged key row
#define LVROW 40      // bf16 per row of the transposed values (32 keys + 8 of padding)

// QS: most 32-wide steps of D; RT: most 16-wide tiles of R (both bound the registers)
template <int QS, int RT, int NW, typename TW>
__global__ __launch_bounds__(NW * 64) void latent_attention_mfma_kernel(
    bf16_t* __restrict__ out, float* __restrict__ ws, const bf16_t* __restrict__ qa, const bf16_t* __restrict__ cache, int P,
    int num_pages, const int* __restrict__ cu_q, const int* __restrict__ pos0, const int* __restrict__ kv_len,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tile_entry, const int* __restrict__ tile_row0,
    const TW* __restrict__ sink, int H, int R, int D, float scale, int window) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    const int tile = blockIdx.x, sp = blockIdx.y, splits = gridDim.y;
    const int e = tile_entry[tile];
    if (e < 0) return;
    const int q0 = cu_q[e];
    const int n_rows = (cu_q[e + 1] - q0) * H;
    const int r_lo = tile_row0[tile];
    if (r_lo >= n_rows) return;
    const int r_hi = min(r_lo + 16 * NW, n_rows) - 1;
    const int p0 = pos0[e], kvl = kv_len[e];
    const int p_lo = p0 + r_lo / H, p_hi = min(p0 + r_hi / H, kvl - 1);
    const int lo = window > 0 ? max(0, p_lo - window + 1) : 0;
    const int c_start = lo & ~31;
    const int n_chunks = (p_hi - c_start) / 32 + 1;
    const int c_begin = (int)((long long)n_chunks * sp / splits), c_end = (int)((long long)n_chunks * (sp + 1) / splits);
    const int q_steps = (D + 31) / 32, r_tiles = (R + 15) / 16;
    const int Dp = q_steps * 32, krow = Dp + LKPAD;
    bf16_t* Ks = reinterpret_cast<bf16_t*>(lds_raw);                  // two buffers of { keys [32][krow], values [r_tiles * 16][LVROW] }
    // this lane's query row
    const int row = r_lo + 16 * wave + r16;
    const bool row_ok = row <= r_hi;
    const int prow = p0 + row / H, head = row % H;
    const int lo_row = window > 0 ? prow - window + 1 : 0;
    lbf16x8_t bq[QS];
    {
        const bf16_t* qv = qa + ((size_t)q0 * H + row) * D;
#pragma unroll
        for (int s = 0; s < QS; ++s) {
            const int d0 = 32 * s + 8 * g;
            lu32x4_t packed = {0u, 0u, 0u, 0u};
            if (s < q_steps && row_ok && d0 < D) packed = *reinterpret_cast<const lu32x4_t*>(qv + d0);
            bq[s] = __builtin_bit_cast(lbf16x8_t, packed);
        }
    }
    const bool with_sink = sink != nullptr && sp == 0;
    float m = with_sink && row_ok ? to_f32<TW>(sink[head]) : -INFINITY;
    float l = with_sink && row_ok && g == 0 ? 1.f : 0.f;          // a row's sum is spread over its four lanes
    lf32x4_t acc[RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) acc[i] = lf32x4_t{0.f, 0.f, 0.f, 0.f};
    const int* bt = block_table + (size_t)e * max_blocks;
    const int ka_row = 8 * (r16 >> 2) + (r16 & 3);                  // tile a's key of this lane's operand row; tile b: + 4
    // Staging.  A thread takes ONE key of a chunk (tid % 32) and every eighth 16-byte piece of its row: a wave's lanes are
    // the 32 keys of two neighbouring pieces, so its transposed 2-byte stores fall into 16 neighbouring LDS words (lanes
    // along d would all hit one bank), and a thread looks up one page per chunk.  The pieces of chunk c + 2 are asked for
    // (into registers) before chunk c is multiplied, and chunk c + 1 is written to the second LDS buffer before that: one
    // barrier per chunk, and no wave waits for memory while another has products to do.
    constexpr int NP = (QS * 4 + NW * 2 - 1) / (NW * 2);             // 16-byte pieces of a key's row per thread
    const int sk = tid & 31, sd0 = (tid >> 5) * 8;
    const int buf_elems = 32 * krow + r_tiles * 16 * LVROW;
    lu32x4_t pf[NP];
    auto fetch = [&](int c) {
        const int key = c_start + 32 * c + sk;
        const bf16_t* src = nullptr;
        if (c < c_end && key >= lo && key <= p_hi) {
            const int page = bt[key / P];
            if (page >= 0 && page < num_pages) src = cache + ((size_t)page * P + key % P) * D;
        }
#pragma unroll
        for (int it = 0; it < NP; ++it) {
            const int d8 = sd0 + 16 * NW * it;
            pf[it] = lu32x4_t{0u, 0u, 0u, 0u};
            if (src && d8 < D) pf[it] = *reinterpret_cast<const lu32x4_t*>(src + d8);
        }
    };
    auto stage = [&](int c) {
        bf16_t* ks = Ks + (c & 1) * buf_elems;
        bf16_t* vt = ks + 32 * krow;
#pragma unroll
        for (int it = 0; it < NP; ++it) {
            const int d8 = sd0 + 16 * NW * it;
            if (d8 < Dp) {
                *reinterpret_cast<lu32x4_t*>(ks + sk * krow + d8) = pf[it];
                if (d8 < r_tiles * 16) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        vt[(d8 + 2 * j) * LVROW + sk] = (bf16_t)(pf[it][j] & 0xffffu);
                        vt[(d8 + 2 * j + 1) * LVROW + sk] = (bf16_t)(pf[it][j] >> 16);
                    }
                }
            }
        }
    };
    if (c_begin < c_end) {
        fetch(c_begin);
        stage(c_begin);
        fetch(c_begin + 1);
    }
    __syncthreads();
    for (int c = c_begin; c < c_end; ++c) {
        const int key0 = c_start + 32 * c;
        if (c + 1 < c_end) stage(c + 1);                             // into the buffer that chunk c - 1 was read from, before the barrier below
        fetch(c + 2);
        const bf16_t* Kc = Ks + (c & 1) * buf_elems;
        const bf16_t* Vc = Kc + 32 * krow;
        // ---- S^T = K . Q^T ----
        lf32x4_t sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < QS; ++s) {
            if (s < q_steps) {
                const lbf16x8_t ka = *reinterpret_cast<const lbf16x8_t*>(Kc + ka_row * krow + 32 * s + 8 * g);
                const lbf16x8_t kb = *reinterpret_cast<const lbf16x8_t*>(Kc + (ka_row + 4) * krow + 32 * s + 8 * g);
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, bq[s], sa, 0, 0, 0);
                sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, bq[s], sb, 0, 0, 0);
            }
        }
        // ---- softmax over this lane's 8 keys of its row ----
        float sc[8];
        float bmax = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int key = key0 + 8 * g + j;
            const float v = (j < 4 ? sa[j] : sb[j - 4]) * scale;
            const bool ok = row_ok && key <= prow && key >= lo_row && key < kvl;
            sc[j] = ok ? v : -INFINITY;
            bmax = fmaxf(bmax, sc[j]);
        }
        bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
        bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
        const float m_new = fmaxf(m, bmax);
        float alpha = 1.f;
        lbf16x8_t pb = {0, 0, 0, 0, 0, 0, 0, 0};
        if (m_new != -INFINITY) {
            alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
            float psum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float pj = (sc[j] == -INFINITY) ? 0.f : __expf(sc[j] - m_new);
                psum += pj;
                pb[j] = (short)f32_to_bf16(pj);
            }
            l = l * alpha + psum;
            m = m_new;
        }
        // ---- O^T = O^T * alpha + V^T . P^T ----
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            if (i < r_tiles) {
                const lbf16x8_t vt = *reinterpret_cast<const lbf16x8_t*>(Vc + (16 * i + r16) * LVROW + 8 * g);
                acc[i] *= alpha;
                acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, pb, acc[i], 0, 0, 0);
            }
        }
        __syncthreads();                                             // chunk c is read by all, chunk c + 1 is written by all
    }
    // the row's sum over its four lanes
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!row_ok) return;
    // lane (row r16, g) holds O^T[v = 16 i + 4 g + j][row], j < 4
    if (splits == 1) {
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16_t* o = out + ((size_t)q0 * H + row) * R;
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const int v0 = 16 * i + 4 * g;
            if (i < r_tiles && v0 < R) {               // R % 4 == 0 (checked by the launcher)
                uint2 w;
                w.x = pack_bf16x2(acc[i][0] * inv, acc[i][1] * inv);
                w.y = pack_bf16x2(acc[i][2] * inv, acc[i][3] * inv);
                *reinterpret_cast<uint2*>(o + v0) = w;
            }
        }
        return;
    }
    // parts: ws[(global row * splits + part)] = { O[R] unnormalised, m, l }
    float* w = ws + (((size_t)q0 * H + row) * splits + sp) * (R + 2);
#pragma unroll
    for (int i = 0; i < RT; ++i) {
        const int v0 = 16 * i + 4 * g;
        if (i < r_tiles && v0 < R) {
#pragma unroll
            for (int j = 0; j < 4; ++j) w[v0 + j] = acc[i][j];
        }
    }
    if (g == 0) { w[R] = m; w[R + 1] = l; }
}

// out[row] = sum_i O_i e^(m_i - M) / sum_i l_i e^(m_i - M) over the parts i of a row, added in ascending i
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ ws, int R, int splits) {
    __shared__ float wgt[64];
    __shared__ float inv_l;
    const size_t row = blockIdx.x;
    const float* base = ws + row * splits * (R + 2);
    if (threadIdx.x < 64) {                        // the parts' maxima and sums, one lane each (at most 64 parts)
        const int i = threadIdx.x;
        const float mi = i < splits ? base[(size_t)i * (R + 2) + R] : -INFINITY;
        const float li = i < splits ? base[(size_t)i * (R + 2) + R + 1] : 0.f;
        const float M = wave_max(mi);
        const float e = (mi == -INFINITY) ? 0.f : __expf(mi - M);
        wgt[i] = e;
        const float L = wave_sum(li * e);
        if (i == 0) inv_l = L > 0.f ? 1.0f / L : 0.f;
    }
    __syncthreads();
    for (int j = threadIdx.x; j < R; j += blockDim.x) {
        float o = 0.f;
#pragma unroll 8
        for (int i = 0; i < splits; ++i) o = fmaf(base[(size_t)i * (R + 2) + j], wgt[i], o);      // (unrolled: the parts' loads go out together)
        out[row * R + j] = f32_to_bf16(o * inv_l);
    }
}

extern "C" long long spy_latent_attention_mfma_workspace(int T, int H, int R, int splits) {
    return splits > 1 ? (long long)T * H * splits * (R + 2) : 0;
}

// tiles: num_tiles records (entry, first row) of tile_rows (64 or 128) rows each: a block of 4 or 8 waves.  ws: float32, spy_latent_attention_mfma_workspace values.
extern "C" int spy_latent_attention_mfma(void* out, float* ws, const void* qa, const void* cache, int P, int num_pages,
                                         const int* cu_q, const int* pos0, const int* kv_len, const int* block_table,
                                         int max_blocks, const int* tile_entry, const int* tile_row0, int num_tiles,
                                         const void* sink, int sink_dtype, int T, int H, int R, int DR, float scale, int window,
                                         int splits, int tile_rows, hipStream_t st) {
    const int D = R + DR;
    SPY_REQUIRE(T > 0 && H > 0 && R > 0 && DR >= 0 && P > 0 && num_pages > 0 && max_blocks > 0 && num_tiles > 0,
                "spy_latent_attention_mfma: empty operand");
    SPY_REQUIRE(D % 8 == 0 && R % 8 == 0 && D <= 576 && R <= 512, "spy_latent_attention_mfma: rows of %d + %d values are not taken", R, DR);
    SPY_REQUIRE(tile_rows == 64 || tile_rows == 128, "spy_latent_attention_mfma: tiles of %d rows (64 or 128)", tile_rows);
    SPY_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || ws), "spy_latent_attention_mfma: %d parts (1..64, with a workspace)", splits);
    SPY_REQUIRE(((uintptr_t)qa % 16) == 0 && ((uintptr_t)cache % 16) == 0 && ((uintptr_t)out % 8) == 0, "spy_latent_attention_mfma: operands are not aligned");
    const int q_steps = (D + 31) / 32, r_tiles = (R + 15) / 16;
    const size_t lds = 2 * ((size_t)32 * (q_steps * 32 + LKPAD) + (size_t)r_tiles * 16 * LVROW) * sizeof(bf16_t);
    SPY_REQUIRE(lds <= 160 * 1024, "spy_latent_attention_mfma: two staged chunks of %d + %d values take %zu bytes of LDS", R, DR, lds);
    const dim3 grid(num_tiles, splits);
#define SPY_LA_LAUNCH_W(QS, RT, NW)                                                                                             \
    SPY_DISPATCH(sink_dtype, TW, {                                                                                              \
        auto kernel = latent_attention_mfma_kernel<QS, RT, NW, TW>;                                                             \
        if (lds > 48 * 1024) {                                                                                                  \
            hipError_t e_ = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);      \
            if (e_ != hipSuccess) return spy_fail("spy_latent_attention_mfma: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e_)); \
        }                                                                                                                       \
        kernel<<<grid, NW * 64, lds, st>>>((bf16_t*)out, ws, (const bf16_t*)qa, (const bf16_t*)cache, P, num_pages, cu_q, pos0, kv_len, \
                                           block_table, max_blocks, tile_entry, tile_row0, (const TW*)sink, H, R, D, scale, window); \
    })
#define SPY_LA_LAUNCH(QS, RT) if (tile_rows == 128) { SPY_LA_LAUNCH_W(QS, RT, 8); } else { SPY_LA_LAUNCH_W(QS, RT, 4); }
    if (q_steps <= 8 && r_tiles <= 8) { SPY_LA_LAUNCH(8, 8); }
    else if (q_steps <= 12 && r_tiles <= 16) { SPY_LA_LAUNCH(12, 16); }
    else { SPY_LA_LAUNCH(18, 32); }
#undef SPY_LA_LAUNCH_W
#undef SPY_LA_LAUNCH
    SPY_CHECK_LAUNCH("spy_latent_attention_mfma");
    if (splits > 1) {
        latent_attention_merge_kernel<<<(unsigned)((size_t)T * H), R > 128 ? 256 : 64, 0, st>>>((bf16_t*)out, ws, R, splits);
        SPY_CHECK_LAUNCH("spy_latent_attention_mfma (merge)");
    }
    return 0;
}

// ---------------------------------------------------------------------------------------------
// Per-head products of few rows on MFMA: C[t, h, n] = sum_k X[t, h, k] W[h, n, k], bfloat16 operands with k innermost
// (X with element strides between tokens and heads, W [H][N][K] in one piece), float32 sums.  A wave owns 16 columns n
// of one head, holds their part of W in registers (KS steps of 32 k values) and walks the tokens in tiles of 16: W is
// read once.  This is the step of single tokens' form of the products with the keys' and the values' expansion matrices;
// many rows take the library's batched product.
template <int KS, typename TC>
__global__ __launch_bounds__(256) void head_products_kernel(TC* __restrict__ C, long long ct, long long ch, const bf16_t* __restrict__ X,
                                                            long long xt, long long xh, const bf16_t* __restrict__ W, int T, int N, int K) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
    const int n0 = (blockIdx.x * 4 + wave) * 16, h = blockIdx.y;
    if (n0 >= N) return;
    lbf16x8_t wr[KS];
    const int n = n0 + r16;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int k0 = 32 * s + 8 * g;
        lu32x4_t v = {0u, 0u, 0u, 0u};
        if (n < N && k0 < K) v = *reinterpret_cast<const lu32x4_t*>(W + ((size_t)h * N + n) * K + k0);
        wr[s] = __builtin_bit_cast(lbf16x8_t, v);
    }
    for (int t0 = blockIdx.z * 16; t0 < T; t0 += gridDim.z * 16) {
        const int t = t0 + r16;
        lf32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        const bf16_t* x = X + (size_t)t * xt + (size_t)h * xh;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int k0 = 32 * s + 8 * g;
            lu32x4_t v = {0u, 0u, 0u, 0u};
            if (t < T && k0 < K) v = *reinterpret_cast<const lu32x4_t*>(x + k0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wr[s], __builtin_bit_cast(lbf16x8_t, v), acc, 0, 0, 0);
        }
        // lane (t = r16, g) holds C[t][h][n0 + 4 g + j], j < 4
        if (t < T) {
            TC* c = C + (size_t)t * ct + (size_t)h * ch + n0 + 4 * g;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n0 + 4 * g + j < N) c[j] = from_f32<TC>(acc[j]);
        }
    }
}

extern "C" int spy_head_products(void* C, int c_dtype, long long ct, long long ch, const void* X, long long xt, long long xh,
                                 const void* W, int T, int H, int N, int K, hipStream_t st) {
    SPY_REQUIRE(T > 0 && H > 0 && N > 0 && K > 0 && H <= 65535, "spy_head_products: empty operand");
    SPY_REQUIRE(K % 8 == 0 && K <= 512 && xt % 8 == 0 && xh % 8 == 0 && ((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0,
                "spy_head_products: K = %d (a multiple of 8 up to 512) and 16-byte pieces of the operands expected", K);
    const int t_tiles = (T + 15) / 16;
    const dim3 grid((N + 63) / 64, H, t_tiles < 8 ? t_tiles : 8);
#define SPY_HP_LAUNCH(KS) SPY_DISPATCH(c_dtype, TC, (head_products_kernel<KS, TC><<<grid, 256, 0, st>>>((TC*)C, ct, ch, (const bf16_t*)X, xt, xh, (const bf16_t*)W, T, N, K)))
    if (K <= 128) { SPY_HP_LAUNCH(4); } else if (K <= 256) { SPY_HP_LAUNCH(8); } else { SPY_HP_LAUNCH(16); }
#undef SPY_HP_LAUNCH
    SPY_CHECK_LAUNCH("spy_head_products");
    return 0;
}
