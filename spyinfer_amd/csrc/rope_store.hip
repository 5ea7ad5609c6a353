// Projection biases, rotation by angles formed in the kernel, and the store of keys and values into their pages, for
// attention layers whose heads are rotated in part and whose frequencies are rescaled (no table: the angle of pair j at
// position p is float(p) * freq[j], float32, and its cosine and sine come from the full-range functions).  And the
// sigmoid gate that such a layer multiplies into its result.
//
// The projections come as rows of a wider product: [q heads | k heads | v heads] of `d` values each, `xs` values from
// one token's row to the next.  One wave per (token, head).  q -> q_out[t, h, :]; k -> K[page, h, off, :];
// v -> V[page, h, :, off] (values lie transposed in a page).
#include "common.h"
#include <math.h>

#define RS_MAX_D 512
#define RS_WAVES 4

template <typename TA, typename TW>
__global__ __launch_bounds__(RS_WAVES * 64) void bias_rope_store_kernel(
    const TA* __restrict__ x, long long xs, TA* __restrict__ q_out, int n_q, int n_kv, int d, const TW* __restrict__ bias,
    const float* __restrict__ freq, int rot, const int* __restrict__ positions, TA* __restrict__ kc, TA* __restrict__ vc, int P,
    int num_pages, const int* __restrict__ slots, float mag, float v_eps, int v_n, float qt_coef, int qt_every) {
    // qt_every > 0: a query is multiplied by 1 + qt_coef ln(floor((position + 1) / qt_every) + 1), float32 (queries that grow
    // with the logarithm of the position, in steps of qt_every positions)
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int h = blockIdx.y * RS_WAVES + (threadIdx.x >> 6);
    const int heads = n_q + 2 * n_kv;
    if (h >= heads) return;
    const TA* row = x + (size_t)t * xs + (size_t)h * d;
    const TW* b = bias ? bias + (size_t)h * d : nullptr;
    const bool is_q = h < n_q, is_k = !is_q && h < n_q + n_kv;
    int page = -1, off = 0;
    if (!is_q) {
        if (!slots) return;
        const int slot = slots[t];
        if (slot < 0 || slot >= num_pages * P) return;
        page = slot / P;
        off = slot - page * P;
    }
    if (!is_q && !is_k) {
        const int hv = h - n_q - n_kv;
        TA* dst = vc + ((size_t)page * n_kv + hv) * d * P + off;
        float r = 1.f;
        if (v_n > 0) {
            // the value head over its root mean square (its first v_n values: the rest is padding)
            float ss = 0.f;
            for (int j = lane; j < v_n; j += 64) {
                const float v = to_f32<TA>(row[j]) + (b ? to_f32<TW>(b[j]) : 0.f);
                ss = fmaf(v, v, ss);
            }
            r = 1.0f / sqrtf(wave_sum(ss) / (float)v_n + v_eps);
        }
        for (int j = lane; j < d; j += 64) dst[(size_t)j * P] = from_f32<TA>((to_f32<TA>(row[j]) + (b ? to_f32<TW>(b[j]) : 0.f)) * r);
        return;
    }
    const int half = rot >> 1;
    const float p = (float)positions[t];
    const float qt = (is_q && qt_every > 0) ? 1.0f + qt_coef * logf((float)((positions[t] + 1) / qt_every) + 1.0f) : 1.0f;
    TA* dst = is_q ? q_out + ((size_t)t * n_q + h) * d : kc + (((size_t)page * n_kv + (h - n_q)) * P + off) * d;
    for (int j = lane; j < half; j += 64) {
        const float a = to_f32<TA>(row[j]) + (b ? to_f32<TW>(b[j]) : 0.f);
        const float c = to_f32<TA>(row[j + half]) + (b ? to_f32<TW>(b[j + half]) : 0.f);
        const float ang = p * freq[j];
        const float cs = cosf(ang) * mag, sn = sinf(ang) * mag;
        dst[j] = from_f32<TA>((a * cs - c * sn) * qt);
        dst[j + half] = from_f32<TA>((c * cs + a * sn) * qt);
    }
    for (int j = rot + lane; j < d; j += 64) dst[j] = from_f32<TA>((to_f32<TA>(row[j]) + (b ? to_f32<TW>(b[j]) : 0.f)) * qt);
}

extern "C" int spy_bias_rope_store(const void* x, long long xs, int dtype, void* q_out, int T, int n_q, int n_kv, int d,
                                   const void* bias, int b_dtype, const float* freq, int rot, const int* positions, void* kc,
                                   void* vc, int P, int num_pages, const int* slots, float mag, float v_eps, int v_n, float qt_coef, int qt_every,
                                   hipStream_t st) {
    SPY_REQUIRE(T > 0 && n_q > 0 && n_kv > 0 && d > 0 && xs >= (long long)(n_q + 2 * n_kv) * d, "spy_bias_rope_store: bad sizes");
    SPY_REQUIRE(d <= RS_MAX_D, "spy_bias_rope_store: head size %d exceeds the supported %d", d, RS_MAX_D);
    SPY_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0 && (rot == 0 || freq), "spy_bias_rope_store: %d rotated dims do not fit a head of %d", rot, d);
    SPY_REQUIRE(!slots || (kc && vc && P > 0 && num_pages > 0), "spy_bias_rope_store: slots without a cache");
    SPY_REQUIRE(n_q + 2 * n_kv <= 65535 * RS_WAVES, "spy_bias_rope_store: too many heads");
    SPY_REQUIRE(v_n >= 0 && v_n <= d, "spy_bias_rope_store: a value norm over %d of %d values", v_n, d);
    const dim3 grid(T, (n_q + 2 * n_kv + RS_WAVES - 1) / RS_WAVES);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(b_dtype, TW, (bias_rope_store_kernel<TA, TW><<<grid, RS_WAVES * 64, 0, st>>>(
        (const TA*)x, xs, (TA*)q_out, n_q, n_kv, d, (const TW*)bias, freq, rot, positions, (TA*)kc, (TA*)vc, P, num_pages, slots, mag, v_eps, v_n,
        qt_coef, qt_every))));
    SPY_CHECK_LAUNCH("spy_bias_rope_store");
    return 0;
}

// y[t, j] *= mult * sigmoid(g[t, j / per] + bias[j / per]) in place; the gate's rows may be part of a wider product (`gs`
// values from row to row); the bias may be absent.  per: columns of y that share one gate value (1: a gate per column;
// a head's size: one number per head).
template <typename TA, typename TW>
__global__ void sigmoid_gate_kernel(TA* __restrict__ y, const TA* __restrict__ g, long long gs, const TW* __restrict__ bias, float mult,
                                    int T, int N, int per) {
    const size_t total = (size_t)T * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / N, j = i - t * N;
        const size_t c = per > 1 ? j / per : j;
        const float gate = to_f32<TA>(g[t * gs + c]) + (bias ? to_f32<TW>(bias[c]) : 0.f);
        y[i] = from_f32<TA>(to_f32<TA>(y[i]) * mult / (1.0f + expf(-gate)));
    }
}

extern "C" int spy_sigmoid_gate(void* y, const void* g, long long gs, int dtype, const void* bias, int b_dtype, float mult, int T, int N,
                                int per, hipStream_t st) {
    SPY_REQUIRE(T > 0 && N > 0 && per > 0 && N % per == 0 && gs >= N / per, "spy_sigmoid_gate: bad sizes");
    const size_t total = (size_t)T * N;
    const unsigned blocks = (unsigned)((total + 255) / 256 > 65536 ? 65536 : (total + 255) / 256);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(b_dtype, TW, (sigmoid_gate_kernel<TA, TW><<<blocks, 256, 0, st>>>((TA*)y, (const TA*)g, gs,
        (const TW*)bias, mult, T, N, per))));
    SPY_CHECK_LAUNCH("spy_sigmoid_gate");
    return 0;
}
