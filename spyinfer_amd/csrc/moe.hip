// Mixture of experts: the router's choice, the (token, choice) pairs sorted by expert, the experts' products over the
// sorted rows, and the weighted sum of a token's results.  Nothing here needs the host to know how many tokens an
// expert got: the sizes of all arrays follow the number of tokens alone, and blocks whose tile holds no rows leave.
//
//   route:   s = softmax(z) over all experts (float32); choice = s + correction; the experts form `groups` equal runs of
//            neighbours, a group's score is its largest choice, only experts of the `keep` best groups can be chosen (the
//            others count as minus infinity); the `top` largest choices are taken; their weights are s (without the
//            correction) over their sum (+ 1e-20), times `scale`.
//   align:   rows of the sorted order: expert e's pairs in a run that starts at a multiple of MOE_TM rows, padded with -1.
//   gemm:    C[row] = A[source of row] . W[expert of the row's tile]^T, float32 products and sums; optionally gated:
//            W = [gate rows | up rows], C = silu(gate) * up; or (MoeAct kind 1) with the row's weight w multiplied into both
//            sums first, g = min(w gate, limit), u = clamp(w up, -limit, limit), C = g sigmoid(1.702 g) (u + 1).
//   combine: out[t] = sum_k weight[t, k] * Y[row of pair (t, k)].
#include "common.h"
#include <math.h>

#define MOE_TM 16
#define MOE_MAX_EXPERTS 1024

// What a gated product does with its two sums (see the top).  pair_w: the weight of every (token, choice) pair, or null.
struct MoeAct {
    int kind;
    float limit;
    const float* pair_w;
};
__device__ __forceinline__ float moe_gated(float g, float u, const MoeAct& a, float w) {
    if (a.kind == 0) return g / (1.0f + expf(-g)) * u;
    g = fminf(g * w, a.limit);
    u = fminf(fmaxf(u * w, -a.limit), a.limit);
    return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
}

// one wave per token
__global__ __launch_bounds__(64) void moe_route_kernel(int* __restrict__ ids, float* __restrict__ weights, const float* __restrict__ z,
                                                       const float* __restrict__ correction, int E, int top, int groups, int keep,
                                                       float scale, int sigmoid, int renorm, const float* __restrict__ zbias) {
    // zbias != null: a bias [E] that is part of the logits (it moves the scores and with them the weights, where the
    // correction moves the choice alone)
    __shared__ float sc[MOE_MAX_EXPERTS], ch[MOE_MAX_EXPERTS], gsc[MOE_MAX_EXPERTS];
    __shared__ float zb[MOE_MAX_EXPERTS];
    __shared__ int allowed[MOE_MAX_EXPERTS], sel[MOE_MAX_EXPERTS];
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* zr = z + (size_t)t * E;
    if (zbias) {
        for (int e = lane; e < E; e += 64) zb[e] = zr[e] + zbias[e];     // (a lane reads back only what it wrote: no barrier)
        zr = zb;
    }
    if (sigmoid) {
        // every logit by itself
        for (int e = lane; e < E; e += 64) {
            sc[e] = 1.0f / (1.0f + expf(-zr[e]));
            ch[e] = sc[e] + (correction ? correction[e] : 0.f);
        }
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, zr[e]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += 64) {
            const float p = expf(zr[e] - mx);
            sc[e] = p;
            sum += p;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += 64) {
            sc[e] = sc[e] / sum;
            ch[e] = sc[e] + (correction ? correction[e] : 0.f);
        }
    }
    __syncthreads();
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
        float best = -INFINITY;
        for (int i = 0; i < per; ++i) best = fmaxf(best, ch[g * per + i]);
        gsc[g] = best;
        allowed[g] = 0;
    }
    __syncthreads();
    for (int r = 0; r < keep; ++r) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int g = lane; g < groups; g += 64)
            if (!allowed[g] && (gsc[g] > bv || (gsc[g] == bv && g < bi))) { bv = gsc[g]; bi = g; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (lane == 0 && bi < groups) allowed[bi] = 1;
        __syncthreads();
    }
    for (int e = lane; e < E; e += 64)
        if (!allowed[e / per]) ch[e] = -INFINITY;
    __syncthreads();
    float wsum = 0.f;
    for (int r = 0; r < top; ++r) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int e = lane; e < E; e += 64)
            if (ch[e] > bv) { bv = ch[e]; bi = e; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (bi >= E) bi = 0;                       // fewer allowed experts than choices: never the case for a checked configuration
        wsum += sc[bi];
        __syncthreads();
        if (lane == 0) { ch[bi] = -INFINITY; sel[r] = bi; }
        __syncthreads();
    }
    const float norm = renorm ? scale / (wsum + 1e-20f) : scale;
    for (int r = lane; r < top; r += 64) {
        ids[(size_t)t * top + r] = sel[r];
        weights[(size_t)t * top + r] = sc[sel[r]] * norm;
    }
}

extern "C" int spy_moe_route(int* ids, float* weights, const float* z, const float* correction, int T, int E, int top, int groups,
                             int keep, float scale, int sigmoid, int renorm, const float* zbias, hipStream_t st) {
    SPY_REQUIRE(T > 0 && E > 0 && E <= MOE_MAX_EXPERTS, "spy_moe_route: %d experts (1..%d)", E, MOE_MAX_EXPERTS);
    SPY_REQUIRE(groups > 0 && E % groups == 0 && keep > 0 && keep <= groups && top > 0 && top <= keep * (E / groups),
                "spy_moe_route: %d of %d groups of %d experts cannot give %d choices", keep, groups, E / (groups > 0 ? groups : 1), top);
    moe_route_kernel<<<T, 64, 0, st>>>(ids, weights, z, correction, E, top, groups, keep, scale, sigmoid, renorm, zbias);
    SPY_CHECK_LAUNCH("spy_moe_route");
    return 0;
}

// One block.  ids [P] -> sorted_pair [max_tiles MOE_TM] (pair or -1), pair_row [P], tile_expert [max_tiles] (expert or -1).
__global__ __launch_bounds__(1024) void moe_align_kernel(int* __restrict__ sorted_pair, int* __restrict__ pair_row,
                                                         int* __restrict__ tile_expert, const int* __restrict__ ids, int P, int E,
                                                         int max_tiles) {
    __shared__ int count[MOE_MAX_EXPERTS], first[MOE_MAX_EXPERTS], cursor[MOE_MAX_EXPERTS];
    __shared__ int total_tiles;
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += blockDim.x) { count[e] = 0; cursor[e] = 0; }
    __syncthreads();
    for (int p = tid; p < P; p += blockDim.x) {
        const int e = ids[p];
        if (e >= 0 && e < E) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int tiles = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = tiles;
            tiles += (count[e] + MOE_TM - 1) / MOE_TM;
        }
        total_tiles = tiles;
    }
    __syncthreads();
    for (int e = tid; e < E; e += blockDim.x) {
        const int nt = (count[e] + MOE_TM - 1) / MOE_TM;
        for (int i = 0; i < nt && first[e] + i < max_tiles; ++i) tile_expert[first[e] + i] = e;
        for (int r = count[e]; r < nt * MOE_TM; ++r)
            if (first[e] * MOE_TM + r < max_tiles * MOE_TM) sorted_pair[first[e] * MOE_TM + r] = -1;
    }
    for (int i = total_tiles + tid; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
    for (int r = total_tiles * MOE_TM + tid; r < max_tiles * MOE_TM; r += blockDim.x) sorted_pair[r] = -1;
    for (int p = tid; p < P; p += blockDim.x) {
        const int e = ids[p];
        if (e < 0 || e >= E) { pair_row[p] = -1; continue; }
        const int row = first[e] * MOE_TM + atomicAdd(&cursor[e], 1);
        if (row < max_tiles * MOE_TM) sorted_pair[row] = p;
        pair_row[p] = row < max_tiles * MOE_TM ? row : -1;
    }
}

extern "C" int spy_moe_align(int* sorted_pair, int* pair_row, int* tile_expert, const int* ids, int P, int E, int max_tiles,
                             hipStream_t st) {
    SPY_REQUIRE(P > 0 && E > 0 && E <= MOE_MAX_EXPERTS, "spy_moe_align: %d experts (1..%d)", E, MOE_MAX_EXPERTS);
    SPY_REQUIRE(max_tiles >= P / MOE_TM + (E < P ? E : P), "spy_moe_align: %d tiles are too few for %d pairs of %d experts", max_tiles, P, E);
    moe_align_kernel<<<1, 1024, 0, st>>>(sorted_pair, pair_row, tile_expert, ids, P, E, max_tiles);
    SPY_CHECK_LAUNCH("spy_moe_align");
    return 0;
}

extern "C" int spy_moe_tile_rows() { return MOE_TM; }

// A tile of MOE_TM sorted rows x 64 columns per block; 256 threads, thread (ty, tx) has row ty and columns 4 tx .. + 3.
// gather > 0: row r reads A[sorted_pair[r] / gather] (the token of the pair); 0: A[r].
#define MG_TN 64
#define MG_K 16
template <typename TA, typename TW, typename TC, bool GATED>
__global__ __launch_bounds__(256) void moe_gemm_kernel(TC* __restrict__ C, const TA* __restrict__ A, const TW* __restrict__ W,
                                                       const int* __restrict__ tile_expert, const int* __restrict__ sorted_pair,
                                                       int gather, int N, int K, long long w_stride, MoeAct act) {
    __shared__ float As[MG_K][MOE_TM + 1];
    __shared__ float Ws[GATED ? 2 : 1][MG_K][MG_TN + 4];
    __shared__ int src[MOE_TM];
    const int tile = blockIdx.y;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int n0 = blockIdx.x * MG_TN;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    if (threadIdx.x < MOE_TM) {
        const int p = sorted_pair[tile * MOE_TM + threadIdx.x];
        src[threadIdx.x] = p < 0 ? -1 : (gather > 0 ? p / gather : tile * MOE_TM + (int)threadIdx.x);
    }
    __syncthreads();
    const TW* We = W + (size_t)e * w_stride;
    float acc[4] = {}, acc2[4] = {};
    // staging: A 16 x 16 values, one per thread; W 64 x 16 values, four per thread
    const int ar = threadIdx.x >> 4, ak = threadIdx.x & 15;
    const int wr = threadIdx.x >> 2, wk = (threadIdx.x & 3) * 4;
    for (int k0 = 0; k0 < K; k0 += MG_K) {
        {
            const int sr = src[ar], k = k0 + ak;
            As[ak][ar] = (sr >= 0 && k < K) ? to_f32<TA>(A[(size_t)sr * K + k]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + wk + i, n = n0 + wr;
            Ws[0][wk + i][wr] = (n < N && k < K) ? to_f32<TW>(We[(size_t)n * K + k]) : 0.f;
            if (GATED) Ws[GATED ? 1 : 0][wk + i][wr] = (n < N && k < K) ? to_f32<TW>(We[(size_t)(N + n) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < MG_K; ++k) {
            const float a = As[k][ty];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[i] = fmaf(a, Ws[0][k][tx * 4 + i], acc[i]);
                if (GATED) acc2[i] = fmaf(a, Ws[GATED ? 1 : 0][k][tx * 4 + i], acc2[i]);
            }
        }
        __syncthreads();
    }
    if (src[ty] < 0) return;
    const size_t row = (size_t)tile * MOE_TM + ty;
    const float rw = (GATED && act.pair_w) ? act.pair_w[sorted_pair[row]] : 1.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int n = n0 + tx * 4 + i;
        if (n >= N) continue;
        float v = acc[i];
        if (GATED) {
            v = moe_gated(acc[i], acc2[i], act, rw);
        }
        C[row * N + n] = from_f32<TC>(v);
    }
}


// The same product on the matrix cores, bfloat16 operands and float32 sums (v_mfma_f32_16x16x32_bf16).  A block of four
// waves takes up to MT neighbouring row tiles (16 sorted rows each) that belong to one expert, and a group of columns:
// every wave owns its columns' rows of W (gated: 16 gate rows and the 16 up rows of the same columns; else 32 rows) and
// walks K, loading its W fragments once per step and using them for all the row tiles, whose rows of A are gathered
// through the pairs' tokens.  Operands go from memory straight into MFMA operand registers: lane (r = lane % 16,
// g = lane / 16) holds row r, values k + 8 g .. + 7; the result tile is C^T: lane (r, g) holds C[row r][column 4 g + i].
// A block whose MT tiles belong to several experts takes their runs in turn.
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short moe_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float moe_f32x4_t;

template <int MT, bool GATED, typename TC>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(TC* __restrict__ C, const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                            const int* __restrict__ tile_expert, const int* __restrict__ sorted_pair,
                                                            int gather, int max_tiles, int N, int K, long long w_stride, MoeAct act) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    constexpr int NT = 2;
    const int n0 = (blockIdx.y * 4 + wave) * (GATED ? 16 : 32);
    if (n0 >= N) return;
    int t = blockIdx.x * MT;
    const int t_end = min(t + MT, max_tiles);
    const moe_bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    while (t < t_end) {
        const int e = __builtin_amdgcn_readfirstlane(tile_expert[t]);
        if (e < 0) break;
        int run = 1;
        while (t + run < t_end && __builtin_amdgcn_readfirstlane(tile_expert[t + run]) == e) ++run;
        const bf16_t* xrow[MT];
        bool xok[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            xok[mt] = false;
            xrow[mt] = A;
            if (mt < run) {
                const int row = (t + mt) * MOE_TM + r;
                const int p = sorted_pair[row];
                xok[mt] = p >= 0;
                const int src = gather > 0 ? p / gather : row;
                xrow[mt] = A + (size_t)(p >= 0 ? src : 0) * K + 8 * g;
            }
        }
        const bf16_t* We = W + (size_t)e * w_stride;
        const bf16_t* wrow[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int row = GATED ? nt * N + min(n0 + r, N - 1) : min(n0 + nt * 16 + r, N - 1);
            wrow[nt] = We + (size_t)row * K + 8 * g;
        }
        moe_f32x4_t acc[NT][MT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
        int k = 0;
        auto fetch = [&](moe_bf16x8_t (&a)[NT][4], moe_bf16x8_t (&b)[MT][4], int k0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) a[nt][j] = *reinterpret_cast<const moe_bf16x8_t*>(wrow[nt] + k0 + 32 * j);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) b[mt][j] = xok[mt] ? *reinterpret_cast<const moe_bf16x8_t*>(xrow[mt] + k0 + 32 * j) : zero8;
            }
        };
        auto products = [&](const moe_bf16x8_t (&a)[NT][4], const moe_bf16x8_t (&b)[MT][4]) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    if (mt < run) {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][j], b[mt][j], acc[nt][mt], 0, 0, 0);
                    }
        };
        if constexpr (MT == 1) {
            // a block with one row tile is bound by the memory's round trips: the operands of the step after this one
            // are asked for before this step's products (two sets of operand registers, taken in turn)
            const int steps = K / 128;
            moe_bf16x8_t a0[NT][4], b0[MT][4], a1[NT][4], b1[MT][4];
            if (steps > 0) fetch(a0, b0, 0);
            for (int s = 0; s < steps; s += 2) {
                if (s + 1 < steps) fetch(a1, b1, (s + 1) * 128);
                products(a0, b0);
                if (s + 1 < steps) {
                    if (s + 2 < steps) fetch(a0, b0, (s + 2) * 128);
                    products(a1, b1);
                }
            }
            k = steps * 128;
        } else {
            for (; k + 128 <= K; k += 128) {
                moe_bf16x8_t a[NT][4], b[MT][4];
                fetch(a, b, k);
                products(a, b);
            }
        }
        for (; k < K; k += 32) {                  // the rest of K (a multiple of 8)
            const bool kok = k + 8 * g < K;
            moe_bf16x8_t a[NT], b[MT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) a[nt] = kok ? *reinterpret_cast<const moe_bf16x8_t*>(wrow[nt] + k) : zero8;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) b[mt] = (kok && xok[mt]) ? *reinterpret_cast<const moe_bf16x8_t*>(xrow[mt] + k) : zero8;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                if (mt < run) {
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt], b[mt], acc[nt][mt], 0, 0, 0);
                }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (mt >= run || !xok[mt]) continue;
            const size_t row = (size_t)(t + mt) * MOE_TM + r;
            if (GATED) {
                const float rw = act.pair_w ? act.pair_w[sorted_pair[row]] : 1.f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int col = n0 + 4 * g + i;
                    if (col < N) C[row * N + col] = from_f32<TC>(moe_gated(acc[0][mt][i], acc[1][mt][i], act, rw));
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int col = n0 + nt * 16 + 4 * g + i;
                        if (col < N) C[row * N + col] = from_f32<TC>(acc[nt][mt][i]);
                    }
            }
        }
        t += run;
    }
}


// Many rows per expert: the same tiles, but the gathered rows of A go through LDS once per block and step of 128 of K
// (the four waves read the same rows; loaded by each of them they swept the first-level cache), while every wave's W
// fragments still come straight from memory, asked for before the block waits for the staged rows.
#define MOE_ROWS 128                 // 8 row tiles
#define MOE_LDS_STRIDE (128 + 8)     // values per staged row (16-byte pieces; the pad spreads the rows over the banks)
template <bool GATED, typename TC>
__global__ __launch_bounds__(256) void moe_gemm_mfma_lds_kernel(TC* __restrict__ C, const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                                                                const int* __restrict__ tile_expert, const int* __restrict__ sorted_pair,
                                                                int gather, int max_tiles, int N, int K, long long w_stride, MoeAct act) {
    constexpr int MT = 8, NT = 2;
    __shared__ __align__(16) bf16_t xs[MOE_ROWS * MOE_LDS_STRIDE];
    __shared__ int src_row[MOE_ROWS];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = (blockIdx.y * 4 + wave) * (GATED ? 16 : 32);
    const bool cols = n0 < N;                        // (a wave without columns still helps to stage)
    int t = blockIdx.x * MT;
    const int t_end = min(t + MT, max_tiles);
    const moe_bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const int srow = threadIdx.x >> 4, spiece = threadIdx.x & 15;      // staging: rows srow + 16 i, 16-byte piece spiece
    while (t < t_end) {
        const int e = __builtin_amdgcn_readfirstlane(tile_expert[t]);
        if (e < 0) break;
        int run = 1;
        while (t + run < t_end && __builtin_amdgcn_readfirstlane(tile_expert[t + run]) == e) ++run;
        __syncthreads();                             // the run before has read its rows
        if (threadIdx.x < MOE_ROWS) {
            int src = -1;
            if ((int)threadIdx.x < run * MOE_TM) {
                const int row = t * MOE_TM + threadIdx.x;
                const int p = sorted_pair[row];
                src = p < 0 ? -1 : (gather > 0 ? p / gather : row);
            }
            src_row[threadIdx.x] = src;
        }
        __syncthreads();
        int srcs[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i) srcs[i] = src_row[srow + 16 * i];
        bool xok[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xok[mt] = mt < run && src_row[mt * 16 + r] >= 0;
        const bf16_t* We = W + (size_t)e * w_stride;
        const bf16_t* wrow[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int row = GATED ? nt * N + min(n0 + r, N - 1) : min(n0 + nt * 16 + r, N - 1);
            wrow[nt] = We + (size_t)(cols ? row : 0) * K + 8 * g;
        }
        moe_f32x4_t acc[NT][MT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
        // the operands of a step are asked for one step ahead: W fragments into registers, the rows of A into registers
        // on their way to LDS, both in flight while the matrix cores work on the step before
        moe_bf16x8_t a[NT][4], stage[MT];
#define MOE_ASK(KK)                                                                                                            \
        {                                                                                                                      \
            _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                                      \
                _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                                              \
                    a[nt][j] = (cols && (KK) + 32 * j + 8 * g < K) ? *reinterpret_cast<const moe_bf16x8_t*>(wrow[nt] + (KK) + 32 * j) : zero8; \
            const bool kin_ = (KK) + 8 * spiece < K;                                                                           \
            _Pragma("unroll") for (int i = 0; i < MT; ++i)                                                                     \
                stage[i] = (i < run && srcs[i] >= 0 && kin_) ? *reinterpret_cast<const moe_bf16x8_t*>(A + (size_t)srcs[i] * K + (KK) + 8 * spiece) : zero8; \
        }
        MOE_ASK(0)
        for (int k = 0; k < K; k += 128) {
            moe_bf16x8_t ac[NT][4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) ac[nt][j] = a[nt][j];
            __syncthreads();                         // the step before has read its rows
#pragma unroll
            for (int i = 0; i < MT; ++i)
                if (i < run) *reinterpret_cast<moe_bf16x8_t*>(xs + (srow + 16 * i) * MOE_LDS_STRIDE + 8 * spiece) = stage[i];
            __syncthreads();
            if (k + 128 < K) MOE_ASK(k + 128)
            if (cols) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        if (mt < run) {
                            const moe_bf16x8_t b = *reinterpret_cast<const moe_bf16x8_t*>(xs + (mt * 16 + r) * MOE_LDS_STRIDE + 32 * j + 8 * g);
#pragma unroll
                            for (int nt = 0; nt < NT; ++nt) acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ac[nt][j], b, acc[nt][mt], 0, 0, 0);
                        }
            }
        }
#undef MOE_ASK
        if (cols) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (mt >= run || !xok[mt]) continue;
                const size_t row = (size_t)(t + mt) * MOE_TM + r;
                if (GATED) {
                    const float rw = act.pair_w ? act.pair_w[sorted_pair[row]] : 1.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int col = n0 + 4 * g + i;
                        if (col < N) C[row * N + col] = from_f32<TC>(moe_gated(acc[0][mt][i], acc[1][mt][i], act, rw));
                    }
                } else {
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int col = n0 + nt * 16 + 4 * g + i;
                            if (col < N) C[row * N + col] = from_f32<TC>(acc[nt][mt][i]);
                        }
                }
            }
        }
        t += run;
    }
}

template <int MT>
static int moe_gemm_mfma_launch(void* C, int c_dtype, const void* A, const void* W, const int* tile_expert, const int* sorted_pair,
                                int gather, int gated, int max_tiles, int N, int K, MoeAct act, hipStream_t st) {
    const long long ws = (long long)(gated ? 2 : 1) * N * K;
    const int cols = gated ? 64 : 128;
    const dim3 grid((max_tiles + MT - 1) / MT, (N + cols - 1) / cols);
    SPY_REQUIRE(grid.y <= 65535, "spy_moe_gemm: too many columns");
    if (MT == 8) {
        if (gated) {
            SPY_DISPATCH(c_dtype, TC, (moe_gemm_mfma_lds_kernel<true, TC><<<grid, 256, 0, st>>>((TC*)C, (const bf16_t*)A, (const bf16_t*)W, tile_expert,
                                                                                               sorted_pair, gather, max_tiles, N, K, ws, act)));
        } else {
            SPY_DISPATCH(c_dtype, TC, (moe_gemm_mfma_lds_kernel<false, TC><<<grid, 256, 0, st>>>((TC*)C, (const bf16_t*)A, (const bf16_t*)W, tile_expert,
                                                                                                sorted_pair, gather, max_tiles, N, K, ws, act)));
        }
    } else if (gated) {
        SPY_DISPATCH(c_dtype, TC, (moe_gemm_mfma_kernel<MT, true, TC><<<grid, 256, 0, st>>>((TC*)C, (const bf16_t*)A, (const bf16_t*)W, tile_expert,
                                                                                           sorted_pair, gather, max_tiles, N, K, ws, act)));
    } else {
        SPY_DISPATCH(c_dtype, TC, (moe_gemm_mfma_kernel<MT, false, TC><<<grid, 256, 0, st>>>((TC*)C, (const bf16_t*)A, (const bf16_t*)W, tile_expert,
                                                                                            sorted_pair, gather, max_tiles, N, K, ws, act)));
    }
    return 0;
}

extern "C" int spy_moe_gemm(void* C, int c_dtype, const void* A, int a_dtype, const void* W, int w_dtype, const int* tile_expert,
                            const int* sorted_pair, int gather, int gated, int max_tiles, int E, int N, int K, int tiles_per_block,
                            int act_kind, float limit, const float* pair_w, hipStream_t st) {
    SPY_REQUIRE(max_tiles > 0 && E > 0 && N > 0 && K > 0 && gather >= 0, "spy_moe_gemm: bad sizes (%d tiles)", max_tiles);
    SPY_REQUIRE((act_kind == 0 && !pair_w) || (act_kind == 1 && gated && limit > 0.f), "spy_moe_gemm: activation %d with limit %g", act_kind, (double)limit);
    const MoeAct act = {act_kind, limit, pair_w};
    // bfloat16 operands in 16-byte pieces: the matrix cores; tiles_per_block: 0 = the plain float32 kernel
    if (tiles_per_block > 0 && a_dtype == SPY_BF16 && w_dtype == SPY_BF16 && K % 8 == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0) {
        const int rc = tiles_per_block >= 8 ? moe_gemm_mfma_launch<8>(C, c_dtype, A, W, tile_expert, sorted_pair, gather, gated, max_tiles, N, K, act, st)
                                            : moe_gemm_mfma_launch<1>(C, c_dtype, A, W, tile_expert, sorted_pair, gather, gated, max_tiles, N, K, act, st);
        if (rc) return rc;
        SPY_CHECK_LAUNCH("spy_moe_gemm (mfma)");
        return 0;
    }
    SPY_REQUIRE(max_tiles <= 65535, "spy_moe_gemm: %d tiles are too many for the plain kernel", max_tiles);
    const dim3 grid((N + MG_TN - 1) / MG_TN, max_tiles);
    const long long ws = (long long)(gated ? 2 : 1) * N * K;
    if (gated) {
        SPY_DISPATCH(a_dtype, TA, SPY_DISPATCH(w_dtype, TW, SPY_DISPATCH(c_dtype, TC, (moe_gemm_kernel<TA, TW, TC, true><<<grid, 256, 0, st>>>(
            (TC*)C, (const TA*)A, (const TW*)W, tile_expert, sorted_pair, gather, N, K, ws, act)))));
    } else {
        SPY_DISPATCH(a_dtype, TA, SPY_DISPATCH(w_dtype, TW, SPY_DISPATCH(c_dtype, TC, (moe_gemm_kernel<TA, TW, TC, false><<<grid, 256, 0, st>>>(
            (TC*)C, (const TA*)A, (const TW*)W, tile_expert, sorted_pair, gather, N, K, ws, act)))));
    }
    SPY_CHECK_LAUNCH("spy_moe_gemm");
    return 0;
}

// out[t, :] = sum_k weights[t, k] * Y[pair_row[t top + k], :], added in ascending k (no weights: all one); add != null:
// plus add[t, :], the result of a layer that every token uses, in the same pass
template <typename TC, bool VEC>
__global__ void moe_combine_kernel(TC* __restrict__ out, const float* __restrict__ Y, const float* __restrict__ weights,
                                   const int* __restrict__ pair_row, int top, int H, const TC* __restrict__ add) {
    // a block has one token and a run of columns (blockIdx.y): few tokens still spread over the device.  VEC: a thread has
    // four neighbouring columns (H % 4 == 0 and 16-byte aligned rows, checked by the launcher), else one.
    constexpr int N = VEC ? 4 : 1;
    const int t = blockIdx.x;
    const int c = (blockIdx.y * blockDim.x + threadIdx.x) * N;
    if (c >= H) return;
    float acc[N] = {};
    for (int k = 0; k < top; ++k) {
        const int row = pair_row[(size_t)t * top + k];
        if (row < 0) continue;
        const float w = weights ? weights[(size_t)t * top + k] : 1.f;
        float y[N];
        if (VEC) Vec4<float>::load(Y + (size_t)row * H + c, y); else y[0] = Y[(size_t)row * H + c];
#pragma unroll
        for (int e = 0; e < N; ++e) acc[e] = fmaf(w, y[e], acc[e]);
    }
    if (add) {
        float a[N];
        if (VEC) Vec4<TC>::load(add + (size_t)t * H + c, a); else a[0] = to_f32<TC>(add[(size_t)t * H + c]);
#pragma unroll
        for (int e = 0; e < N; ++e) acc[e] += a[e];
    }
    if (VEC) Vec4<TC>::store(out + (size_t)t * H + c, acc); else out[(size_t)t * H + c] = from_f32<TC>(acc[0]);
}

extern "C" int spy_moe_combine(void* out, int dtype, const float* Y, const float* weights, const int* pair_row, int T, int top, int H,
                               const void* add, hipStream_t st) {
    SPY_REQUIRE(T > 0 && top > 0 && H > 0, "spy_moe_combine: empty operand");
    const bool vec = H % 4 == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)Y % 16) == 0 && ((uintptr_t)add % 16) == 0;
    const int per_block = vec ? 512 : 128;
    const dim3 grid(T, (H + per_block - 1) / per_block);
    SPY_REQUIRE(grid.y <= 65535, "spy_moe_combine: rows of %d values are too long", H);
    if (vec) {
        SPY_DISPATCH(dtype, TC, (moe_combine_kernel<TC, true><<<grid, 128, 0, st>>>((TC*)out, Y, weights, pair_row, top, H, (const TC*)add)));
    } else {
        SPY_DISPATCH(dtype, TC, (moe_combine_kernel<TC, false><<<grid, 128, 0, st>>>((TC*)out, Y, weights, pair_row, top, H, (const TC*)add)));
    }
    SPY_CHECK_LAUNCH("spy_moe_combine");
    return 0;
}
