// Recurrent mixers whose state is a matrix per head, S [d, dv] in float32 in the request's slot: a write k v^T per
// token, a read-out S^T q.  One wave per (entry, head, slice of 16 value channels): four neighbouring lanes share a
// column of S, each with a quarter of its d rows in registers, and add their parts of a sum with two DPP exchanges
// inside the quad (no LDS, no barrier); the wave walks the entry's tokens; the token's key and query go through LDS,
// and the operands of the next four tokens are in flight ahead of this token's arithmetic.  The read-outs leave as
// float32; a second kernel norms every head over all its slices, applies weight and gate and rounds once.
// Everything behind the projections is float32.
//
//   mlstm:       S = a S + b k v^T, n = a n + b k with a = exp(f + m' - m), b = exp(i - m), m = max(f + m', i) (m starts at
//                0), i and f capped log gates; o = S^T q / (max(|n . q|, exp(-m)) + 1e-6); then o / rms(o) * w * sigmoid(g).
//   delta rule:  S = diag(g) S; u = beta (v - S^T k); S = S + k u^T; o = S^T q, g a decay per key channel, q and k unit
//                vectors; then o / rms(o) * w * sigmoid(gate).
//   causal_conv_silu: the short convolution over time that feeds the delta rule, with its last inputs kept per request.
#include "common.h"
#include <math.h>

__device__ __forceinline__ float mm_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float mm_logsigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

#define MM_SLICE 64          // lanes of a block (one wave)
#define MM_COLS 16           // value channels of a wave: four lanes a column

// Between a wave's LDS writes and its own LDS reads: a block here is ONE wave, whose LDS operations run in program order,
// so no barrier is needed.  What is needed is that the compiler keeps the order.
__device__ __forceinline__ void mm_wave_order() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// sum over the four lanes of a quad, in every one of them
__device__ __forceinline__ float quad_sum(float x) {
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0xB1, 0xF, 0xF, true));      // lanes 1 0 3 2
    x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), 0x4E, 0xF, 0xF, true));      // lanes 2 3 0 1
    return x;
}

// out[t, h, j] = o[t, h, j] / sqrt(mean_j(o[t, h, :]^2) + eps) * w[(per_head ? h dv : 0) + j] * sigmoid(gate[t, h dv + j])
// (silu != 0: times silu(gate) = gate sigmoid(gate)); one block per (token, head)
template <typename TA, typename TW>
__global__ void head_norm_gate_kernel(TA* __restrict__ out, const float* __restrict__ o, const TA* __restrict__ gate, long long gs,
                                      const TW* __restrict__ w, int per_head, float eps, int H, int dv, int silu = 0) {
    __shared__ float red[16];
    const int t = blockIdx.x, h = blockIdx.y;
    const float* row = o + ((size_t)t * H + h) * dv;
    float ss = 0.f;
    for (int j = threadIdx.x; j < dv; j += blockDim.x) ss += row[j] * row[j];
    ss = block_sum(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)dv + eps);
    const TA* g = gate + (size_t)t * gs + (size_t)h * dv;
    const TW* wr = w + (per_head ? (size_t)h * dv : 0);
    TA* dst = out + ((size_t)t * H + h) * dv;
    for (int j = threadIdx.x; j < dv; j += blockDim.x) {
        const float gj = to_f32<TA>(g[j]);
        dst[j] = from_f32<TA>(((row[j] * r) * to_f32<TW>(wr[j])) * (silu ? gj * mm_sigmoid(gj) : mm_sigmoid(gj)));
    }
}

// ---- mLSTM ----------------------------------------------------------------------------------------------------------
// In place over the gates' raw products [T, 2 H]: the capped log gates i = cap tanh((. + bi) / cap) and
// f = logsigmoid(cap tanh((. + bf) / cap)), for all tokens at once (the walk below has only the running maximum left).
template <typename TW>
__global__ void mlstm_gates_kernel(float* __restrict__ gates, const TW* __restrict__ bi, const TW* __restrict__ bf, float cap, int T, int H) {
    const size_t total = (size_t)T * 2 * H;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int c = (int)(i % (2 * H));
        if (c < H) gates[i] = cap * tanhf((gates[i] + to_f32<TW>(bi[c])) / cap);
        else gates[i] = mm_logsigmoid(cap * tanhf((gates[i] + to_f32<TW>(bf[c - H])) / cap));
    }
}

// x: rows of the fused projection, xs values apart; q at column q_off (H heads of d), k at k_off, v at v_off (H heads of
// dv).  gates [T, 2 H] float32: the log input and forget gates (mlstm_gates_kernel).  state [slots][H][d dv + NS (d + 1)]:
// S (row dd, column j at dd dv + j), then for every slice of 16 columns its own copy of n and m (the slices' waves do
// not wait for each other, so none may read what another has already moved on).
#define MM_AHEAD 4          // tokens whose operands are in flight ahead of the one being worked on
// MODE 0: block x is an entry, walked whole from the request's state, which is left at the end.
// Entries of many tokens are cut into pieces (block x is a piece then): with the running maximum known for every token
// (mlstm_scalars_kernel: a, b and exp(-m) per token in `gates` [T, 3 H]) the state is linear in itself with scalar
// coefficients, S_end = A S_start + B with A the product of the piece's a.  MODE 1 walks a piece from zero and leaves
// (B, A) in the piece's record of `work` (laid out as a request's state, A where m lies); MODE 2 folds the records of
// the entry's pieces before its own into the request's state, walks its piece from there and writes the read-outs;
// mlstm_keep_kernel folds all of an entry's records into the state afterwards.
template <typename TA, typename TW, int DR, int MODE>
__global__ __launch_bounds__(MM_SLICE) void mlstm_kernel(
    float* __restrict__ o_out, float* __restrict__ state, const TA* __restrict__ x, long long xs, int q_off, int k_off, int v_off,
    const float* __restrict__ gates, const int* __restrict__ cu_q,
    const int* __restrict__ slot_ids, int num_slots, int H, int d, int dv, int NS,
    float* __restrict__ work, const int* __restrict__ piece_entry, const int* __restrict__ piece_t0, const int* __restrict__ piece_t1,
    const int* __restrict__ piece_first) {
    constexpr int R = (DR + MM_SLICE - 1) / MM_SLICE, LD = R * MM_SLICE, DQ = DR / 4;
    constexpr int GS = MODE == 0 ? 2 : 3;             // scalars a token and head in `gates`
    __shared__ __align__(16) float ks[LD], qs[LD];
    const int h = blockIdx.y, c = blockIdx.z, lane = threadIdx.x;
    const int s = MODE == 0 ? (int)blockIdx.x : piece_entry[blockIdx.x];
    const int part = lane & 3, j = c * MM_COLS + (lane >> 2);
    const int row0 = part * DQ;                       // this lane's rows of S: row0 .. row0 + DQ - 1
    const int slot = slot_ids[s];
    if (slot < 0 || slot >= num_slots) return;
    const size_t head_state = (size_t)d * dv + (size_t)NS * (d + 1);
    float* st = state + ((size_t)slot * H + h) * head_state;
    float* nm = st + (size_t)d * dv + (size_t)c * (d + 1);
    const bool col = j < dv;
    // rows of S beyond d stay zero, and so do the staged k and q there: the loops below run over all of a lane's rows
    // without conditions (straight-line code, so that the LDS reads go out ahead of the arithmetic)
    float S[DQ], n[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) {
        S[i] = (MODE != 1 && col && row0 + i < d) ? st[(size_t)(row0 + i) * dv + j] : 0.f;
        n[i] = (MODE != 1 && row0 + i < d) ? nm[row0 + i] : 0.f;
    }
    if (MODE == 2) {
        const int jc = min(j, dv - 1);
        for (int q = piece_first[blockIdx.x]; q < (int)blockIdx.x; ++q) {
            const float* ws = work + ((size_t)q * H + h) * head_state;
            const float* wn = ws + (size_t)d * dv + (size_t)c * (d + 1);
            const float A = wn[d];
            // (loads without conditions, from clamped places, so that they all go out together; rows and columns that do
            // not exist keep their zeros)
            float ws_[DQ], wn_[DQ];
#pragma unroll
            for (int i = 0; i < DQ; ++i) {
                ws_[i] = ws[(size_t)min(row0 + i, d - 1) * dv + jc];
                wn_[i] = wn[min(row0 + i, d - 1)];
            }
#pragma unroll
            for (int i = 0; i < DQ; ++i) {
                const bool rok = row0 + i < d;
                S[i] = (col && rok) ? fmaf(A, S[i], ws_[i]) : S[i];
                n[i] = rok ? fmaf(A, n[i], wn_[i]) : n[i];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        ks[lane + MM_SLICE * i] = 0.f;
        qs[lane + MM_SLICE * i] = 0.f;
    }
    float m = MODE == 0 ? nm[d] : 0.f;
    float Aprod = 1.f;
    const float qscale = 1.0f / sqrtf((float)d);
    const int t0 = MODE == 0 ? cu_q[s] : piece_t0[blockIdx.x], t1 = MODE == 0 ? cu_q[s + 1] : piece_t1[blockIdx.x];
    float kr[MM_AHEAD][R], qr[MM_AHEAD][R], vr[MM_AHEAD], gir[MM_AHEAD], gfr[MM_AHEAD], ger[MM_AHEAD];
#define MLSTM_LOAD(U, TT)                                                                        \
    if ((TT) < t1) {                                                                             \
        const TA* xr_ = x + (size_t)(TT) * xs;                                                   \
        _Pragma("unroll") for (int i = 0; i < R; ++i) {                                          \
            const int idx = lane + MM_SLICE * i;                                                 \
            kr[U][i] = idx < d ? to_f32<TA>(xr_[k_off + (size_t)h * d + idx]) : 0.f;             \
            qr[U][i] = idx < d ? to_f32<TA>(xr_[q_off + (size_t)h * d + idx]) * qscale : 0.f;    \
        }                                                                                        \
        vr[U] = col ? to_f32<TA>(xr_[v_off + (size_t)h * dv + j]) : 0.f;                         \
        gir[U] = gates[(size_t)(TT) * GS * H + h];                                               \
        gfr[U] = gates[(size_t)(TT) * GS * H + H + h];                                           \
        ger[U] = MODE == 0 ? 0.f : gates[(size_t)(TT) * GS * H + 2 * H + h];                     \
    }
#pragma unroll
    for (int u = 0; u < MM_AHEAD; ++u) MLSTM_LOAD(u, t0 + u)
    for (int tb = t0; tb < t1; tb += MM_AHEAD) {
#pragma unroll
        for (int u = 0; u < MM_AHEAD; ++u) {
            const int t = tb + u;
            if (t < t1) {
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const int idx = lane + MM_SLICE * i;
                    if (idx < d) { ks[idx] = kr[u][i]; qs[idx] = qr[u][i]; }
                }
                float a, b, em;
                if (MODE == 0) {
                    const float ig = gir[u], fg = gfr[u];
                    const float m_new = fmaxf(fg + m, ig);
                    a = expf(fg + m - m_new);
                    b = expf(ig - m_new);
                    m = m_new;
                    em = expf(-m);
                } else {
                    a = gir[u];
                    b = gfr[u];
                    em = ger[u];
                    Aprod *= a;
                }
                mm_wave_order();
                float acc = 0.f, acc2 = 0.f, nq = 0.f, nq2 = 0.f;
                const float bv = b * vr[u];
#pragma unroll
                for (int i = 0; i < DQ; i += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + row0 + i), q4 = *reinterpret_cast<const float4*>(qs + row0 + i);
                    S[i] = fmaf(a, S[i], k4.x * bv);         acc = fmaf(S[i], q4.x, acc);
                    S[i + 1] = fmaf(a, S[i + 1], k4.y * bv); acc2 = fmaf(S[i + 1], q4.y, acc2);
                    S[i + 2] = fmaf(a, S[i + 2], k4.z * bv); acc = fmaf(S[i + 2], q4.z, acc);
                    S[i + 3] = fmaf(a, S[i + 3], k4.w * bv); acc2 = fmaf(S[i + 3], q4.w, acc2);
                    n[i] = fmaf(a, n[i], b * k4.x);         nq = fmaf(n[i], q4.x, nq);
                    n[i + 1] = fmaf(a, n[i + 1], b * k4.y); nq2 = fmaf(n[i + 1], q4.y, nq2);
                    n[i + 2] = fmaf(a, n[i + 2], b * k4.z); nq = fmaf(n[i + 2], q4.z, nq);
                    n[i + 3] = fmaf(a, n[i + 3], b * k4.w); nq2 = fmaf(n[i + 3], q4.w, nq2);
                }
                acc = quad_sum(acc + acc2);
                nq = quad_sum(nq + nq2);
                const float den = fmaxf(fabsf(nq), em) + 1e-6f;
                if (MODE != 1 && col && part == 0) o_out[((size_t)t * H + h) * dv + j] = acc / den;
                mm_wave_order();
                MLSTM_LOAD(u, t + MM_AHEAD)
            }
        }
    }
#undef MLSTM_LOAD
    if (MODE == 2) return;
    if (MODE == 1) {
        st = work + ((size_t)blockIdx.x * H + h) * head_state;
        nm = st + (size_t)d * dv + (size_t)c * (d + 1);
        m = Aprod;
    }
#pragma unroll
    for (int i = 0; i < DQ; ++i) {
        if (col && row0 + i < d) st[(size_t)(row0 + i) * dv + j] = S[i];
        if (lane < 4 && row0 + i < d) nm[row0 + i] = n[i];
    }
    if (lane == 0) nm[d] = m;
}

// One thread per (entry, head): the running maximum over the entry's tokens, from the request's state, before and after
// every token in abe [T, 3 H]; the last maximum goes to mfin [S, H].
__global__ void mlstm_scalars_kernel(float* __restrict__ abe, float* __restrict__ mfin, const float* __restrict__ lg,
                                     const float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ slot_ids,
                                     int num_slots, int S, int H, int d, int dv, int NS) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= S * H) return;
    const int s = i / H, h = i - s * H;
    const int slot = slot_ids[s];
    if (slot < 0 || slot >= num_slots) return;
    const size_t head_state = (size_t)d * dv + (size_t)NS * (d + 1);
    float m = state[((size_t)slot * H + h) * head_state + (size_t)d * dv + d];
    const int t1 = cu_q[s + 1];
    // (the gates of 16 tokens are asked for together: the loads do not depend on the maximum, only the arithmetic does)
    for (int tb = cu_q[s]; tb < t1; tb += 16) {
        float ig[16], fg[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int t = tb + u < t1 ? tb + u : t1 - 1;
            ig[u] = lg[(size_t)t * 2 * H + h];
            fg[u] = lg[(size_t)t * 2 * H + H + h];
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int t = tb + u;
            if (t < t1) {
                const float m_new = fmaxf(fg[u] + m, ig[u]);
                abe[(size_t)t * 3 * H + h] = m;                      // (the exponentials follow for all tokens at once)
                abe[(size_t)t * 3 * H + H + h] = m_new;
                m = m_new;
            }
        }
    }
    mfin[i] = m;
}

// abe [T, 3 H] holds the maximum before and after every token (mlstm_scalars_kernel); with the log gates lg [T, 2 H] it
// becomes a = exp(f + m' - m), b = exp(i - m) and exp(-m).
__global__ void mlstm_abe_kernel(float* __restrict__ abe, const float* __restrict__ lg, int T, int H) {
    const size_t total = (size_t)T * H;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / H, h = i - t * H;
        const float mp = abe[t * 3 * H + h], mn = abe[t * 3 * H + H + h];
        const float ig = lg[t * 2 * H + h], fg = lg[t * 2 * H + H + h];
        abe[t * 3 * H + h] = expf(fg + mp - mn);
        abe[t * 3 * H + H + h] = expf(ig - mn);
        abe[t * 3 * H + 2 * H + h] = expf(-mn);
    }
}

// Block x is a piece; the last piece of an entry folds all of the entry's records into the request's state.
template <int DR>
__global__ __launch_bounds__(MM_SLICE) void mlstm_keep_kernel(float* __restrict__ state, const float* __restrict__ work,
                                                              const float* __restrict__ mfin, const int* __restrict__ piece_entry,
                                                              const int* __restrict__ piece_first, int n_pieces,
                                                              const int* __restrict__ slot_ids, int num_slots, int H, int d, int dv, int NS) {
    constexpr int DQ = DR / 4;
    const int k = blockIdx.x, h = blockIdx.y, c = blockIdx.z, lane = threadIdx.x;
    if (!(k + 1 == n_pieces || piece_first[k + 1] == k + 1)) return;
    const int s = piece_entry[k];
    const int slot = slot_ids[s];
    if (slot < 0 || slot >= num_slots) return;
    const int part = lane & 3, j = c * MM_COLS + (lane >> 2), row0 = part * DQ;
    const bool col = j < dv;
    const size_t head_state = (size_t)d * dv + (size_t)NS * (d + 1);
    float* st = state + ((size_t)slot * H + h) * head_state;
    float* nm = st + (size_t)d * dv + (size_t)c * (d + 1);
    float S[DQ], n[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) {
        S[i] = (col && row0 + i < d) ? st[(size_t)(row0 + i) * dv + j] : 0.f;
        n[i] = row0 + i < d ? nm[row0 + i] : 0.f;
    }
    const int jc = min(j, dv - 1);
    for (int q = piece_first[k]; q <= k; ++q) {
        const float* ws = work + ((size_t)q * H + h) * head_state;
        const float* wn = ws + (size_t)d * dv + (size_t)c * (d + 1);
        const float A = wn[d];
        float ws_[DQ], wn_[DQ];
#pragma unroll
        for (int i = 0; i < DQ; ++i) {
            ws_[i] = ws[(size_t)min(row0 + i, d - 1) * dv + jc];
            wn_[i] = wn[min(row0 + i, d - 1)];
        }
#pragma unroll
        for (int i = 0; i < DQ; ++i) {
            const bool rok = row0 + i < d;
            S[i] = (col && rok) ? fmaf(A, S[i], ws_[i]) : S[i];
            n[i] = rok ? fmaf(A, n[i], wn_[i]) : n[i];
        }
    }
#pragma unroll
    for (int i = 0; i < DQ; ++i) {
        if (col && row0 + i < d) st[(size_t)(row0 + i) * dv + j] = S[i];
        if (lane < 4 && row0 + i < d) nm[row0 + i] = n[i];
    }
    if (lane == 0) nm[d] = mfin[(size_t)s * H + h];
}

#define MM_LAUNCH(KERNEL, ...)                                                              \
    do {                                                                                    \
        if (d <= 32) KERNEL<TA, TW, 32><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);            \
        else if (d <= 64) KERNEL<TA, TW, 64><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);       \
        else if (d <= 128) KERNEL<TA, TW, 128><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);     \
        else KERNEL<TA, TW, 256><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);                   \
    } while (0)

#define MM_LAUNCH_MODE(KERNEL, MODE, ...)                                                          \
    do {                                                                                           \
        if (d <= 32) KERNEL<TA, TW, 32, MODE><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);             \
        else if (d <= 64) KERNEL<TA, TW, 64, MODE><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);        \
        else if (d <= 128) KERNEL<TA, TW, 128, MODE><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);      \
        else KERNEL<TA, TW, 256, MODE><<<grid, MM_SLICE, 0, st>>>(__VA_ARGS__);                    \
    } while (0)

// pieces: int32 [4][n_pieces] (entry, first row, end row, index of the entry's first piece), used when `multi` says that an
// entry has several; then work [n_pieces][state of a request], abe [T][3 H] and mfin [S][H] are scratch.
extern "C" int spy_mlstm(void* out, float* o_tmp, float* state, const void* x, long long xs, int dtype, int q_off, int k_off, int v_off,
                         int g_off, float* gates, const void* bi, const void* bf, int w_dtype, float cap, const void* norm_w,
                         float eps, const int* cu_q, const int* slot_ids, int num_slots, int S, int T, int H, int d, int dv,
                         const int* pieces, int n_pieces, int multi, float* work, float* abe, float* mfin, hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && H > 0 && d > 0 && dv > 0 && num_slots > 0 && o_tmp, "spy_mlstm: empty operand");
    SPY_REQUIRE(d <= 256 && dv <= 1024 && H <= 65535, "spy_mlstm: heads of %d x %d (key size up to 256, value size up to 1024)", d, dv);
    SPY_REQUIRE(cap > 0.f, "spy_mlstm: the gates' cap must be positive");
    const int NS = (dv + MM_COLS - 1) / MM_COLS;
    const dim3 grid(S, H, NS);
    {
        const size_t total = (size_t)T * 2 * H;
        const unsigned blocks = (unsigned)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
        SPY_DISPATCH(w_dtype, TW, (mlstm_gates_kernel<TW><<<blocks, 256, 0, st>>>(gates, (const TW*)bi, (const TW*)bf, cap, T, H)));
        SPY_CHECK_LAUNCH("spy_mlstm (gates)");
    }
    if (!multi) {
        SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, MM_LAUNCH_MODE(mlstm_kernel, 0, o_tmp, state, (const TA*)x, xs, q_off, k_off, v_off,
            gates, cu_q, slot_ids, num_slots, H, d, dv, NS, nullptr, nullptr, nullptr, nullptr, nullptr)));
        SPY_CHECK_LAUNCH("spy_mlstm");
    } else {
        SPY_REQUIRE(pieces && n_pieces > 0 && work && abe && mfin, "spy_mlstm: entries in several pieces need their scratch memory");
        const int* pe = pieces;
        const int* p0 = pieces + n_pieces;
        const int* p1 = pieces + 2 * (size_t)n_pieces;
        const int* pf = pieces + 3 * (size_t)n_pieces;
        mlstm_scalars_kernel<<<(S * H + 63) / 64, 64, 0, st>>>(abe, mfin, gates, state, cu_q, slot_ids, num_slots, S, H, d, dv, NS);
        SPY_CHECK_LAUNCH("spy_mlstm (running maximum)");
        {
            const size_t total = (size_t)T * H;
            const unsigned blocks = (unsigned)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
            mlstm_abe_kernel<<<blocks, 256, 0, st>>>(abe, gates, T, H);
            SPY_CHECK_LAUNCH("spy_mlstm (decays)");
        }
        const dim3 grid(n_pieces, H, NS);
        SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, MM_LAUNCH_MODE(mlstm_kernel, 1, o_tmp, state, (const TA*)x, xs, q_off, k_off, v_off,
            abe, cu_q, slot_ids, num_slots, H, d, dv, NS, work, pe, p0, p1, pf)));
        SPY_CHECK_LAUNCH("spy_mlstm (pieces)");
        SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, MM_LAUNCH_MODE(mlstm_kernel, 2, o_tmp, state, (const TA*)x, xs, q_off, k_off, v_off,
            abe, cu_q, slot_ids, num_slots, H, d, dv, NS, work, pe, p0, p1, pf)));
        SPY_CHECK_LAUNCH("spy_mlstm (walk)");
        if (d <= 32) mlstm_keep_kernel<32><<<grid, MM_SLICE, 0, st>>>(state, work, mfin, pe, pf, n_pieces, slot_ids, num_slots, H, d, dv, NS);
        else if (d <= 64) mlstm_keep_kernel<64><<<grid, MM_SLICE, 0, st>>>(state, work, mfin, pe, pf, n_pieces, slot_ids, num_slots, H, d, dv, NS);
        else if (d <= 128) mlstm_keep_kernel<128><<<grid, MM_SLICE, 0, st>>>(state, work, mfin, pe, pf, n_pieces, slot_ids, num_slots, H, d, dv, NS);
        else mlstm_keep_kernel<256><<<grid, MM_SLICE, 0, st>>>(state, work, mfin, pe, pf, n_pieces, slot_ids, num_slots, H, d, dv, NS);
        SPY_CHECK_LAUNCH("spy_mlstm (state)");
    }
    const dim3 ngrid(T, H);
    const int nthreads = dv >= 256 ? 256 : 64;
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (head_norm_gate_kernel<TA, TW><<<ngrid, nthreads, 0, st>>>(
        (TA*)out, o_tmp, (const TA*)x + g_off, xs, (const TW*)norm_w, 1, eps, H, dv))));
    SPY_CHECK_LAUNCH("spy_mlstm (norm and gate)");
    return 0;
}

// ---- short causal convolution + silu -----------------------------------------------------------------------------------
// y[t, c] = silu(sum_j taps[c, j] x[t - (n - 1) + j, c]); inputs before the entry's first token come from the request's
// kept inputs keep[slot][n - 1][C] (index n - 2 the newest), which are zero for a new request.
template <typename TA, typename TW>
__global__ void causal_conv_silu_kernel(TA* __restrict__ y, const TA* __restrict__ x, long long xs, const TW* __restrict__ taps,
                                        const float* __restrict__ keep, long long keep_stride, const int* __restrict__ token_entry,
                                        const int* __restrict__ cu_q, const int* __restrict__ slot_ids, int num_slots, int T, int C,
                                        int n) {
    const size_t total = (size_t)T * C;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int t = (int)(i / C), c = (int)(i - (size_t)t * C);
        const int e = token_entry[t];
        const int t0 = cu_q[e];
        const int slot = slot_ids[e];
        const bool ok = slot >= 0 && slot < num_slots;
        float acc = 0.f;
        for (int j = 0; j < n; ++j) {
            const int src = t - (n - 1) + j;
            float v;
            if (src >= t0) v = to_f32<TA>(x[(size_t)src * xs + c]);
            else v = ok ? keep[(size_t)slot * keep_stride + (size_t)((n - 1) + (src - t0)) * C + c] : 0.f;
            acc = fmaf(to_f32<TW>(taps[(size_t)c * n + j]), v, acc);
        }
        y[i] = from_f32<TA>(acc * mm_sigmoid(acc));
    }
}

// after the convolution has read them: the kept inputs move on by the entry's tokens
#define CONV_MAX_TAPS 8
template <typename TA>
__global__ void conv_keep_kernel(float* __restrict__ keep, long long keep_stride, const TA* __restrict__ x, long long xs,
                                 const int* __restrict__ cu_q, const int* __restrict__ slot_ids, int num_slots, int C, int n) {
    const int e = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int slot = slot_ids[e];
    if (slot < 0 || slot >= num_slots) return;
    const int t0 = cu_q[e], L = cu_q[e + 1] - t0;
    float* kp = keep + (size_t)slot * keep_stride;
    float v[CONV_MAX_TAPS];
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i) {
        if (i < n - 1) {
            const int rel = L - (n - 1) + i;
            v[i] = rel >= 0 ? to_f32<TA>(x[(size_t)(t0 + rel) * xs + c]) : kp[(size_t)(i + L) * C + c];
        }
    }
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS - 1; ++i)
        if (i < n - 1) kp[(size_t)i * C + c] = v[i];
}

extern "C" int spy_causal_conv_silu(void* y, const void* x, long long xs, int dtype, const void* taps, int w_dtype, float* keep,
                                    long long keep_stride, const int* token_entry, const int* cu_q, const int* slot_ids,
                                    int num_slots, int S, int T, int C, int n, hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && C > 0 && num_slots > 0 && xs >= C, "spy_causal_conv_silu: empty operand");
    SPY_REQUIRE(n >= 1 && n <= CONV_MAX_TAPS && keep_stride >= (long long)(n - 1) * C && S <= 65535, "spy_causal_conv_silu: %d taps (1..%d)", n, CONV_MAX_TAPS);
    const size_t total = (size_t)T * C;
    const unsigned blocks = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (causal_conv_silu_kernel<TA, TW><<<blocks, 256, 0, st>>>(
        (TA*)y, (const TA*)x, xs, (const TW*)taps, keep, keep_stride, token_entry, cu_q, slot_ids, num_slots, T, C, n))));
    SPY_CHECK_LAUNCH("spy_causal_conv_silu");
    if (n > 1) {
        const dim3 grid((C + 255) / 256, S);
        SPY_DISPATCH(dtype, TA, (conv_keep_kernel<TA><<<grid, 256, 0, st>>>(keep, keep_stride, (const TA*)x, xs, cu_q, slot_ids, num_slots, C, n)));
        SPY_CHECK_LAUNCH("spy_causal_conv_silu (kept inputs)");
    }
    return 0;
}

// ---- gated delta rule with a decay per key channel ----------------------------------------------------------------------
// qkv [T, 2 G d + H dv]: the convolved, activated q (G heads of d), k (G heads of d), v (H heads of dv).  beta_pre [T, H]
// and dec_pre [T, H d] float32: raw products.  gate: rows of H dv values, gs apart.  state [slots][stride]: S of head h at
// h d dv, row dd and column j at dd dv + j.
// For all tokens at once, one wave per (token, unit): units 0 .. G - 1 turn head g's q and k into unit vectors (q also
// times d^-1/2) in qk [T, 2 G d] float32; units G .. G + H - 1 turn head h's raw decay products into the decays
// exp(-exp(a_log) softplus(. + dt_bias)) and its raw beta product into sigmoid(.), both in place.
template <typename TA, typename TW>
__global__ __launch_bounds__(64) void delta_prepare_kernel(float* __restrict__ qk, const TA* __restrict__ qkv, float* __restrict__ beta,
                                                          float* __restrict__ dec, const TW* __restrict__ a_log,
                                                          const TW* __restrict__ dt_bias, int H, int G, int d, int dv, int dd,
                                                          long long bs, long long zs) {
    // dd: decays per head, d (one per key channel) or 1 (one for the head); bs, zs: values from one token's row of beta
    // and of the decays to the next (both may be columns of one wider product)
    const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int C = 2 * G * d + H * dv;
    if (unit < G) {
        const TA* q = qkv + (size_t)t * C + (size_t)unit * d;
        const TA* k = qkv + (size_t)t * C + (size_t)(G + unit) * d;
        float sq = 0.f, sk = 0.f;
        for (int i = lane; i < d; i += 64) {
            const float a = to_f32<TA>(q[i]), b = to_f32<TA>(k[i]);
            sq = fmaf(a, a, sq);
            sk = fmaf(b, b, sk);
        }
        sq = wave_sum(sq);
        sk = wave_sum(sk);
        const float rq = 1.0f / sqrtf(sq + 1e-6f) / sqrtf((float)d), rk = 1.0f / sqrtf(sk + 1e-6f);
        float* oq = qk + (size_t)t * 2 * G * d + (size_t)unit * d;
        float* ok = qk + (size_t)t * 2 * G * d + (size_t)(G + unit) * d;
        for (int i = lane; i < d; i += 64) {
            oq[i] = to_f32<TA>(q[i]) * rq;
            ok[i] = to_f32<TA>(k[i]) * rk;
        }
        return;
    }
    const int h = unit - G;
    const float rate = expf(to_f32<TW>(a_log[h]));
    float* z = dec + (size_t)t * zs + (size_t)h * dd;
    for (int i = lane; i < dd; i += 64) z[i] = expf(-rate * softplus_f(z[i] + to_f32<TW>(dt_bias[(size_t)h * dd + i])));
    if (lane == 0) beta[(size_t)t * bs + h] = mm_sigmoid(beta[(size_t)t * bs + h]);
}

template <typename TA, typename TW, int DR>
__global__ __launch_bounds__(MM_SLICE) void delta_rule_kernel(
    float* __restrict__ o_out, float* __restrict__ state, long long state_stride, const TA* __restrict__ qkv, const float* __restrict__ qk,
    const float* __restrict__ beta_pre, const float* __restrict__ dec_pre, const int* __restrict__ cu_q,
    const int* __restrict__ slot_ids, int num_slots, int H, int G, int d, int dv, int dd, long long bs, long long zs) {
    constexpr int R = (DR + MM_SLICE - 1) / MM_SLICE, LD = R * MM_SLICE, DQ = DR / 4;
    __shared__ __align__(16) float ks[LD], qs[LD], dec[LD];
    const int s = blockIdx.x, h = blockIdx.y, c = blockIdx.z, lane = threadIdx.x;
    const int part = lane & 3, j = c * MM_COLS + (lane >> 2);
    const int row0 = part * DQ;
    const int slot = slot_ids[s];
    if (slot < 0 || slot >= num_slots) return;
    const int g = h / (H / G);
    float* st = state + (size_t)slot * state_stride + (size_t)h * d * dv;
    const bool col = j < dv;
    // (rows beyond d: S zero, staged k and q zero, decay one; the loops run over all of a lane's rows without conditions)
    float S[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) S[i] = (col && row0 + i < d) ? st[(size_t)(row0 + i) * dv + j] : 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        ks[lane + MM_SLICE * i] = 0.f;
        qs[lane + MM_SLICE * i] = 0.f;
        dec[lane + MM_SLICE * i] = 1.f;
    }
    const int C = 2 * G * d + H * dv;
    const int t0 = cu_q[s], t1 = cu_q[s + 1];
    float kr[MM_AHEAD][R], qr[MM_AHEAD][R], zr[MM_AHEAD][R], vr[MM_AHEAD], br[MM_AHEAD];
#define DELTA_LOAD(U, TT)                                                                        \
    if ((TT) < t1) {                                                                             \
        const float* qk_ = qk + (size_t)(TT) * 2 * G * d;                                        \
        _Pragma("unroll") for (int i = 0; i < R; ++i) {                                          \
            const int idx = lane + MM_SLICE * i;                                                 \
            qr[U][i] = idx < d ? qk_[(size_t)g * d + idx] : 0.f;                                 \
            kr[U][i] = idx < d ? qk_[(size_t)(G + g) * d + idx] : 0.f;                           \
            zr[U][i] = idx < d ? dec_pre[(size_t)(TT) * zs + (size_t)h * dd + (dd == 1 ? 0 : idx)] : 1.f; \
        }                                                                                        \
        vr[U] = col ? to_f32<TA>(qkv[(size_t)(TT) * C + (size_t)2 * G * d + (size_t)h * dv + j]) : 0.f; \
        br[U] = beta_pre[(size_t)(TT) * bs + h];                                                 \
    }
#pragma unroll
    for (int u = 0; u < MM_AHEAD; ++u) DELTA_LOAD(u, t0 + u)
    for (int tb = t0; tb < t1; tb += MM_AHEAD) {
#pragma unroll
        for (int u = 0; u < MM_AHEAD; ++u) {
            const int t = tb + u;
            if (t < t1) {
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const int idx = lane + MM_SLICE * i;
                    if (idx < d) { qs[idx] = qr[u][i]; ks[idx] = kr[u][i]; dec[idx] = zr[u][i]; }
                }
                const float beta = br[u];
                mm_wave_order();
                float r = 0.f, r2 = 0.f;
#pragma unroll
                for (int i = 0; i < DQ; i += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + row0 + i), g4 = *reinterpret_cast<const float4*>(dec + row0 + i);
                    S[i] *= g4.x;     r = fmaf(S[i], k4.x, r);
                    S[i + 1] *= g4.y; r2 = fmaf(S[i + 1], k4.y, r2);
                    S[i + 2] *= g4.z; r = fmaf(S[i + 2], k4.z, r);
                    S[i + 3] *= g4.w; r2 = fmaf(S[i + 3], k4.w, r2);
                }
                const float uu = beta * (vr[u] - quad_sum(r + r2));
                float acc = 0.f, acc2 = 0.f;
#pragma unroll
                for (int i = 0; i < DQ; i += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + row0 + i), q4 = *reinterpret_cast<const float4*>(qs + row0 + i);
                    S[i] = fmaf(k4.x, uu, S[i]);         acc = fmaf(S[i], q4.x, acc);
                    S[i + 1] = fmaf(k4.y, uu, S[i + 1]); acc2 = fmaf(S[i + 1], q4.y, acc2);
                    S[i + 2] = fmaf(k4.z, uu, S[i + 2]); acc = fmaf(S[i + 2], q4.z, acc);
                    S[i + 3] = fmaf(k4.w, uu, S[i + 3]); acc2 = fmaf(S[i + 3], q4.w, acc2);
                }
                acc = quad_sum(acc + acc2);
                if (col && part == 0) o_out[((size_t)t * H + h) * dv + j] = acc;
                mm_wave_order();
                DELTA_LOAD(u, t + MM_AHEAD)
            }
        }
    }
#undef DELTA_LOAD
#pragma unroll
    for (int i = 0; i < DQ; ++i)
        if (col && row0 + i < d) st[(size_t)(row0 + i) * dv + j] = S[i];
}

extern "C" int spy_delta_rule(void* out, float* o_tmp, float* qk_tmp, float* state, long long state_stride, const void* qkv, int dtype,
                              float* beta_pre, float* dec_pre, const void* a_log, const void* dt_bias, int w_dtype, const void* gate, long long gs,
                              const void* norm_w, float eps, const int* cu_q, const int* slot_ids, int num_slots, int S, int T, int H,
                              int G, int d, int dv, int dd, int silu_gate, long long bs, long long zs, hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0 && num_slots > 0 && o_tmp, "spy_delta_rule: empty operand");
    SPY_REQUIRE(dd == d || dd == 1, "spy_delta_rule: %d decays for a head of %d key channels (one, or one per channel)", dd, d);
    SPY_REQUIRE(bs >= H && zs >= (long long)H * dd, "spy_delta_rule: rows of beta or of the decays are too short");
    SPY_REQUIRE(d <= 256 && dv <= 1024 && H <= 65535, "spy_delta_rule: heads of %d x %d (key size up to 256, value size up to 1024)", d, dv);
    SPY_REQUIRE(state_stride >= (long long)H * d * dv && gs >= (long long)H * dv, "spy_delta_rule: the state or the gate rows are too short");
    SPY_REQUIRE(qk_tmp && G + H <= 65535, "spy_delta_rule: no room for the unit vectors");
    const dim3 pgrid(T, G + H);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (delta_prepare_kernel<TA, TW><<<pgrid, 64, 0, st>>>(
        qk_tmp, (const TA*)qkv, beta_pre, dec_pre, (const TW*)a_log, (const TW*)dt_bias, H, G, d, dv, dd, bs, zs))));
    SPY_CHECK_LAUNCH("spy_delta_rule (unit vectors and decays)");
    const dim3 grid(S, H, (dv + MM_COLS - 1) / MM_COLS);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, MM_LAUNCH(delta_rule_kernel, o_tmp, state, state_stride, (const TA*)qkv, qk_tmp, beta_pre,
        dec_pre, cu_q, slot_ids, num_slots, H, G, d, dv, dd, bs, zs)));
    SPY_CHECK_LAUNCH("spy_delta_rule");
    const dim3 ngrid(T, H);
    const int nthreads = dv >= 256 ? 256 : 64;
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (head_norm_gate_kernel<TA, TW><<<ngrid, nthreads, 0, st>>>(
        (TA*)out, o_tmp, (const TA*)gate, gs, (const TW*)norm_w, 0, eps, H, dv, silu_gate))));
    SPY_CHECK_LAUNCH("spy_delta_rule (norm and gate)");
    return 0;
}

// ---- token shift -------------------------------------------------------------------------------------------------------
// out[s][t][c] = x[t][c] + (x'[t][c] - x[t][c]) mu[s][c], x' the row before t in its request: the entry's row before, or,
// for an entry's first token, the request's kept row (float32, `keep_stride` values from slot to slot).  A second kernel
// then leaves every entry's last row as the request's kept row (after all reads of the old one: the next launch).
template <typename TA, typename TW>
__global__ void token_shift_kernel(TA* __restrict__ out, const TA* __restrict__ x, const TW* __restrict__ mu, int n,
                                   const float* __restrict__ keep, long long keep_stride, const int* __restrict__ token_entry,
                                   const int* __restrict__ cu_q, const int* __restrict__ slot_ids, int num_slots, int T, int W) {
    const size_t total = (size_t)T * W;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int t = (int)(i / W), c = (int)(i - (size_t)t * W);
        const int e = token_entry[t];
        float prev;
        if (t > cu_q[e]) prev = to_f32<TA>(x[i - W]);
        else {
            const int slot = slot_ids[e];
            prev = (slot >= 0 && slot < num_slots) ? keep[(size_t)slot * keep_stride + c] : 0.f;
        }
        const float cur = to_f32<TA>(x[i]);
        for (int s = 0; s < n; ++s) out[(size_t)s * total + i] = from_f32<TA>(fmaf(prev - cur, to_f32<TW>(mu[(size_t)s * W + c]), cur));
    }
}

template <typename TA>
__global__ void shift_keep_kernel(float* __restrict__ keep, long long keep_stride, const TA* __restrict__ x, const int* __restrict__ cu_q,
                                  const int* __restrict__ slot_ids, int num_slots, int W) {
    const int s = blockIdx.y;
    const int slot = slot_ids[s];
    const int last = cu_q[s + 1] - 1;
    if (slot < 0 || slot >= num_slots || last < cu_q[s]) return;
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < W; c += gridDim.x * blockDim.x)
        keep[(size_t)slot * keep_stride + c] = to_f32<TA>(x[(size_t)last * W + c]);
}

extern "C" int spy_token_shift(void* out, const void* x, int dtype, const void* mu, int w_dtype, int n, float* keep, long long keep_stride,
                               const int* token_entry, const int* cu_q, const int* slot_ids, int num_slots, int S, int T, int W,
                               hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && W > 0 && n > 0 && num_slots > 0 && keep && keep_stride >= W && S <= 65535, "spy_token_shift: bad sizes");
    const size_t total = (size_t)T * W;
    const unsigned blocks = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (token_shift_kernel<TA, TW><<<blocks, 256, 0, st>>>(
        (TA*)out, (const TA*)x, (const TW*)mu, n, keep, keep_stride, token_entry, cu_q, slot_ids, num_slots, T, W))));
    SPY_CHECK_LAUNCH("spy_token_shift");
    const dim3 kgrid((W + 255) / 256, S);
    SPY_DISPATCH(dtype, TA, (shift_keep_kernel<TA><<<kgrid, 256, 0, st>>>(keep, keep_stride, (const TA*)x, cu_q, slot_ids, num_slots, W)));
    SPY_CHECK_LAUNCH("spy_token_shift (kept row)");
    return 0;
}

template <typename TC>
__global__ void tanh_kernel(TC* __restrict__ out, const float* __restrict__ x, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        out[i] = from_f32<TC>(tanhf(x[i]));
}

// out = tanh(x) of float32 sums, rounded once to the dtype that the next product reads
extern "C" int spy_tanh(void* out, int dtype, const float* x, long long n, hipStream_t st) {
    SPY_REQUIRE(n > 0, "spy_tanh: empty operand");
    const unsigned blocks = (unsigned)((n + 255) / 256 > 65536 ? 65536 : (n + 255) / 256);
    SPY_DISPATCH(dtype, TC, (tanh_kernel<TC><<<blocks, 256, 0, st>>>((TC*)out, x, n)));
    SPY_CHECK_LAUNCH("spy_tanh");
    return 0;
}

// ---- a state with a decay per key channel, read before the write, and a bonus for the token's own pair ------------------
// r, k, v, gate [T, H d]; dec [T, H d] float32: raw products, turned in place into the decays w = exp(-exp(. + w0));
// bonus [T, H] = sum_i r_i u_i k_i.  Per head: o_j = sum_i r_i S_ij + bonus v_j; S_ij = w_i S_ij + k_i v_j.
// state [slots][stride]: S of head h at h d d, row (key channel) i and column j at i d + j.
// The preparation, for all tokens at once: one wave per (token, head).
template <typename TA, typename TW>
__global__ __launch_bounds__(64) void time_mix_prepare_kernel(float* __restrict__ dec, float* __restrict__ bonus, const TA* __restrict__ r,
                                                             const TA* __restrict__ k, const TW* __restrict__ w0, const TW* __restrict__ u,
                                                             int H, int d) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const size_t at = ((size_t)t * H + h) * d;
    float b = 0.f;
    for (int i = lane; i < d; i += 64) {
        dec[at + i] = expf(-expf(dec[at + i] + to_f32<TW>(w0[(size_t)h * d + i])));
        b = fmaf(to_f32<TA>(r[at + i]) * to_f32<TW>(u[(size_t)h * d + i]), to_f32<TA>(k[at + i]), b);
    }
    b = wave_sum(b);
    if (lane == 0) bonus[(size_t)t * H + h] = b;
}

// The walk: one wave per (entry, head, slice of 16 value channels), four lanes a column, as the delta rule's.
template <typename TA, typename TW, int DR>
__global__ __launch_bounds__(MM_SLICE) void time_mix_kernel(
    float* __restrict__ o_out, float* __restrict__ state, long long state_stride, const TA* __restrict__ r, const TA* __restrict__ k,
    const TA* __restrict__ v, const float* __restrict__ dec_in, const float* __restrict__ bonus, const int* __restrict__ cu_q,
    const int* __restrict__ slot_ids, int num_slots, int H, int d) {
    constexpr int R = (DR + MM_SLICE - 1) / MM_SLICE, LD = R * MM_SLICE, DQ = DR / 4;
    __shared__ __align__(16) float ks[LD], rs[LD], dec[LD];
    const int s = blockIdx.x, h = blockIdx.y, c = blockIdx.z, lane = threadIdx.x;
    const int part = lane & 3, j = c * MM_COLS + (lane >> 2);
    const int row0 = part * DQ;
    const int slot = slot_ids[s];
    if (slot < 0 || slot >= num_slots) return;
    float* st = state + (size_t)slot * state_stride + (size_t)h * d * d;
    const bool col = j < d;
    // (rows beyond d: S zero, staged k and r zero, decay one; the loops run over all of a lane's rows without conditions)
    float S[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i) S[i] = (col && row0 + i < d) ? st[(size_t)(row0 + i) * d + j] : 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        ks[lane + MM_SLICE * i] = 0.f;
        rs[lane + MM_SLICE * i] = 0.f;
        dec[lane + MM_SLICE * i] = 1.f;
    }
    const int N = H * d;
    const int t0 = cu_q[s], t1 = cu_q[s + 1];
    float kr[MM_AHEAD][R], rr[MM_AHEAD][R], zr[MM_AHEAD][R], vr[MM_AHEAD], br[MM_AHEAD];
#define TMIX_LOAD(U, TT)                                                                         \
    if ((TT) < t1) {                                                                             \
        const size_t at_ = (size_t)(TT) * N + (size_t)h * d;                                     \
        _Pragma("unroll") for (int i = 0; i < R; ++i) {                                          \
            const int idx = lane + MM_SLICE * i;                                                 \
            rr[U][i] = idx < d ? to_f32<TA>(r[at_ + idx]) : 0.f;                                 \
            kr[U][i] = idx < d ? to_f32<TA>(k[at_ + idx]) : 0.f;                                 \
            zr[U][i] = idx < d ? dec_in[at_ + idx] : 1.f;                                        \
        }                                                                                        \
        vr[U] = col ? to_f32<TA>(v[at_ + j]) : 0.f;                                              \
        br[U] = bonus[(size_t)(TT) * H + h];                                                     \
    }
#pragma unroll
    for (int u = 0; u < MM_AHEAD; ++u) TMIX_LOAD(u, t0 + u)
    for (int tb = t0; tb < t1; tb += MM_AHEAD) {
#pragma unroll
        for (int u = 0; u < MM_AHEAD; ++u) {
            const int t = tb + u;
            if (t < t1) {
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const int idx = lane + MM_SLICE * i;
                    if (idx < d) { rs[idx] = rr[u][i]; ks[idx] = kr[u][i]; dec[idx] = zr[u][i]; }
                }
                const float vj = vr[u];
                mm_wave_order();
                float acc = 0.f, acc2 = 0.f;
#pragma unroll
                for (int i = 0; i < DQ; i += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + row0 + i), g4 = *reinterpret_cast<const float4*>(dec + row0 + i);
                    const float4 r4 = *reinterpret_cast<const float4*>(rs + row0 + i);
                    acc = fmaf(S[i], r4.x, acc);          S[i] = fmaf(S[i], g4.x, k4.x * vj);
                    acc2 = fmaf(S[i + 1], r4.y, acc2);    S[i + 1] = fmaf(S[i + 1], g4.y, k4.y * vj);
                    acc = fmaf(S[i + 2], r4.z, acc);      S[i + 2] = fmaf(S[i + 2], g4.z, k4.z * vj);
                    acc2 = fmaf(S[i + 3], r4.w, acc2);    S[i + 3] = fmaf(S[i + 3], g4.w, k4.w * vj);
                }
                acc = quad_sum(acc + acc2);
                if (col && part == 0) o_out[(size_t)t * N + (size_t)h * d + j] = fmaf(br[u], vj, acc);
                mm_wave_order();
                TMIX_LOAD(u, t + MM_AHEAD)
            }
        }
    }
#undef TMIX_LOAD
#pragma unroll
    for (int i = 0; i < DQ; ++i)
        if (col && row0 + i < d) st[(size_t)(row0 + i) * d + j] = S[i];
}

extern "C" int spy_time_mix(void* out, float* o_tmp, float* bonus, float* state, long long state_stride, const void* r, const void* k,
                            const void* v, const void* gate, int dtype, float* dec_pre, const void* w0, const void* u, const void* norm_w,
                            int w_dtype, float eps, const int* cu_q, const int* slot_ids, int num_slots, int S, int T, int H, int d,
                            hipStream_t st) {
    SPY_REQUIRE(S > 0 && T > 0 && H > 0 && d > 0 && num_slots > 0 && o_tmp && bonus, "spy_time_mix: empty operand");
    SPY_REQUIRE(d <= 256 && H <= 65535, "spy_time_mix: heads of %d (up to 256)", d);
    SPY_REQUIRE(state_stride >= (long long)H * d * d, "spy_time_mix: the state is too short");
    const dim3 pgrid(T, H);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (time_mix_prepare_kernel<TA, TW><<<pgrid, 64, 0, st>>>(
        dec_pre, bonus, (const TA*)r, (const TA*)k, (const TW*)w0, (const TW*)u, H, d))));
    SPY_CHECK_LAUNCH("spy_time_mix (decays and bonus)");
    const dim3 grid(S, H, (d + MM_COLS - 1) / MM_COLS);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, MM_LAUNCH(time_mix_kernel, o_tmp, state, state_stride, (const TA*)r, (const TA*)k,
        (const TA*)v, dec_pre, bonus, cu_q, slot_ids, num_slots, H, d)));
    SPY_CHECK_LAUNCH("spy_time_mix");
    const dim3 ngrid(T, H);
    const int nthreads = d >= 256 ? 256 : 64;
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (head_norm_gate_kernel<TA, TW><<<ngrid, nthreads, 0, st>>>(
        (TA*)out, o_tmp, (const TA*)gate, (long long)H * d, (const TW*)norm_w, 1, eps, H, d, 1))));
    SPY_CHECK_LAUNCH("spy_time_mix (norm and gate)");
    return 0;
}

// ---- two results normed over the width and averaged ----------------------------------------------------------------------
// out[t] = (a[t] / rms(a[t]) * wa + b[t] / rms(b[t]) * wb) / 2; one block per row.  VEC: W % 4 == 0, aligned rows, and a row
// fits PAIR_PASSES passes of four values a thread: both rows are read once and stay in registers
#define PAIR_PASSES 4
template <typename TA, typename TW, bool VEC>
__global__ void norm_pair_mean_kernel(TA* __restrict__ out, const TA* __restrict__ a, const TA* __restrict__ b, const TW* __restrict__ wa,
                                      const TW* __restrict__ wb, float eps, int W) {
    __shared__ float red[16], red2[16];
    const TA* ar = a + (size_t)blockIdx.x * W;
    const TA* br = b + (size_t)blockIdx.x * W;
    TA* o = out + (size_t)blockIdx.x * W;
    float sa = 0.f, sb = 0.f;
    if (VEC) {
        float x[PAIR_PASSES][4], y[PAIR_PASSES][4];
#pragma unroll
        for (int p = 0; p < PAIR_PASSES; ++p) {
            const int i = (p * blockDim.x + threadIdx.x) * 4;
            if (i < W) {
                Vec4<TA>::load(ar + i, x[p]);
                Vec4<TA>::load(br + i, y[p]);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sa = fmaf(x[p][e], x[p][e], sa);
                    sb = fmaf(y[p][e], y[p][e], sb);
                }
            }
        }
        sa = block_sum(sa, red);
        sb = block_sum(sb, red2);
        const float ra = 0.5f / sqrtf(sa / (float)W + eps), rb = 0.5f / sqrtf(sb / (float)W + eps);
#pragma unroll
        for (int p = 0; p < PAIR_PASSES; ++p) {
            const int i = (p * blockDim.x + threadIdx.x) * 4;
            if (i < W) {
                float u4[4], v4[4], r4[4];
                Vec4<TW>::load(wa + i, u4);
                Vec4<TW>::load(wb + i, v4);
#pragma unroll
                for (int e = 0; e < 4; ++e) r4[e] = fmaf(x[p][e] * ra, u4[e], (y[p][e] * rb) * v4[e]);
                Vec4<TA>::store(o + i, r4);
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float x = to_f32<TA>(ar[i]), y = to_f32<TA>(br[i]);
        sa = fmaf(x, x, sa);
        sb = fmaf(y, y, sb);
    }
    sa = block_sum(sa, red);
    sb = block_sum(sb, red2);
    const float ra = 0.5f / sqrtf(sa / (float)W + eps), rb = 0.5f / sqrtf(sb / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x)
        o[i] = from_f32<TA>(fmaf(to_f32<TA>(ar[i]) * ra, to_f32<TW>(wa[i]), (to_f32<TA>(br[i]) * rb) * to_f32<TW>(wb[i])));
}

extern "C" int spy_norm_pair_mean(void* out, const void* a, const void* b, int dtype, const void* wa, const void* wb, int w_dtype, float eps,
                                  int T, int W, hipStream_t st) {
    SPY_REQUIRE(T > 0 && W > 0, "spy_norm_pair_mean: empty operand");
    const int threads = W >= 2048 ? 256 : (W >= 512 ? 128 : 64);
    const bool vec = W % 4 == 0 && W <= threads * 4 * PAIR_PASSES && ((uintptr_t)out % 16) == 0 && ((uintptr_t)a % 16) == 0 &&
                     ((uintptr_t)b % 16) == 0 && ((uintptr_t)wa % 16) == 0 && ((uintptr_t)wb % 16) == 0;
    if (vec) {
        SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (norm_pair_mean_kernel<TA, TW, true><<<T, threads, 0, st>>>(
            (TA*)out, (const TA*)a, (const TA*)b, (const TW*)wa, (const TW*)wb, eps, W))));
    } else {
        SPY_DISPATCH(dtype, TA, SPY_DISPATCH(w_dtype, TW, (norm_pair_mean_kernel<TA, TW, false><<<T, 256, 0, st>>>(
            (TA*)out, (const TA*)a, (const TA*)b, (const TW*)wa, (const TW*)wb, eps, W))));
    }
    SPY_CHECK_LAUNCH("spy_norm_pair_mean");
    return 0;
}
