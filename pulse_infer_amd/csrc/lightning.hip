// Linear attention with a constant decay per head ("lightning attention").
//
// Every head keeps a state S [d, dv] in float32 for each request:
//     S_t = decay_h * S_(t-1) + k_t v_t^T          o_t = S_t^T q_t
// q, k [heads, d] and v [heads, dv] are columns of one projection output, with an
// activation (silu) applied as they are read.  The state of a request lives in its
// slot and is taken as zero when the request's portion starts at position 0.
//
// pulse_lightning_scan walks the tokens of an entry in order (a single decoded token
// is the walk of one), so a prompt cut into portions, or decoded token by token, goes
// through the same arithmetic in the same order.  A wavefront owns 64 / R columns of
// one head's state; a lane holds d / R rows of one column in registers, and the R
// partial sums of an output meet through lane exchanges.  R is chosen on the host so
// that the launch has enough wavefronts.  q, k and v of 16 tokens at a time go
// through LDS.
//
// pulse_gated_rmsnorm finishes the mixer: the heads' outputs of a token, taken
// together, are divided by their root mean square, multiplied by a weight and by
// sigmoid(gate), and rounded once.
#include "common.h"

#include <math.h>

namespace {

struct ScanArgs {
    int heads, d, dv;
    int64_t x_stride, o_stride;
    int q0, k0, v0;   // first columns of q, k and v in a row of x
    int act;          // 0: none, 1: silu
};

__device__ __forceinline__ float activate(float z, int act) { return act == 1 ? z / (1.0f + expf(-z)) : z; }

constexpr int SCAN_TOKENS = 16;

template <typename TX, int D, int R>
__global__ __launch_bounds__(64) void lightning_scan_kernel(const TX* __restrict__ x, float* __restrict__ out,
                                                            float* __restrict__ state, const float* __restrict__ decay,
                                                            const int* __restrict__ entry_first_row,
                                                            const int* __restrict__ entry_start,
                                                            const int* __restrict__ entry_slot, ScanArgs a) {
    constexpr int CW = PULSE_WAVE / R;   // columns of the state a wavefront owns
    constexpr int DR = D / R;            // rows a lane holds
    __shared__ float q_s[SCAN_TOKENS][D];
    __shared__ float k_s[SCAN_TOKENS][D];
    __shared__ float v_s[SCAN_TOKENS][CW];
    const int e = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x;
    const int cl = lane % CW, rg = lane / CW;
    const int c = blockIdx.z * CW + cl;
    const int i0 = rg * DR;
    const bool live = c < a.dv;
    const int row0 = entry_first_row[e];
    const int n = entry_first_row[e + 1] - row0;
    float* S = state + (static_cast<int64_t>(entry_slot[e]) * a.heads + h) * a.d * a.dv;
    float s[DR];
    const bool fresh = entry_start[e] == 0;
#pragma unroll
    for (int i = 0; i < DR; ++i)
        s[i] = (!fresh && live && i0 + i < a.d) ? S[static_cast<int64_t>(i0 + i) * a.dv + c] : 0.f;
    const float lam = decay[h];
    for (int t0 = 0; t0 < n; t0 += SCAN_TOKENS) {
        const int nb = min(SCAN_TOKENS, n - t0);
        __syncthreads();
        for (int idx = lane; idx < nb * D; idx += PULSE_WAVE) {
            const int tt = idx / D, i = idx % D;
            float qv = 0.f, kv = 0.f;
            if (i < a.d) {
                const TX* row = x + static_cast<int64_t>(row0 + t0 + tt) * a.x_stride;
                qv = activate(to_f32<TX>(row[a.q0 + h * a.d + i]), a.act);
                kv = activate(to_f32<TX>(row[a.k0 + h * a.d + i]), a.act);
            }
            q_s[tt][i] = qv;
            k_s[tt][i] = kv;
        }
        for (int idx = lane; idx < nb * CW; idx += PULSE_WAVE) {
            const int tt = idx / CW, cc = blockIdx.z * CW + idx % CW;
            const TX* row = x + static_cast<int64_t>(row0 + t0 + tt) * a.x_stride;
            v_s[tt][idx % CW] = cc < a.dv ? activate(to_f32<TX>(row[a.v0 + h * a.dv + cc]), a.act) : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < nb; ++tt) {
            const float v = v_s[tt][cl];
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < DR; ++i) {
                s[i] = fmaf(lam, s[i], k_s[tt][i0 + i] * v);
                o = fmaf(s[i], q_s[tt][i0 + i], o);
            }
#pragma unroll
            for (int off = CW; off < PULSE_WAVE; off <<= 1) o += __shfl_xor(o, off, PULSE_WAVE);
            if (live && rg == 0) out[static_cast<int64_t>(row0 + t0 + tt) * a.o_stride + h * a.dv + c] = o;
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DR; ++i)
            if (i0 + i < a.d) S[static_cast<int64_t>(i0 + i) * a.dv + c] = s[i];
    }
}

// ------------------------------------------------------- gated norm of heads
template <typename TX, typename TW>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, int64_t o_stride, const TW* __restrict__ w,
                                     const TX* __restrict__ gate, int64_t gate_stride, TX* __restrict__ y,
                                     int64_t y_stride, int n, float eps, float scale) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const float* row = o + static_cast<int64_t>(t) * o_stride;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(row[i], row[i], ss);
    const float total = block_sum(ss, scratch);
    const float inv = scale / sqrtf(total / static_cast<float>(n) + eps);
    const TX* g = gate ? gate + static_cast<int64_t>(t) * gate_stride : nullptr;
    TX* dst = y + static_cast<int64_t>(t) * y_stride;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = row[i] * inv * to_f32<TW>(w[i]);
        if (g) v *= 1.0f / (1.0f + expf(-to_f32<TX>(g[i])));
        dst[i] = from_f32<TX>(v);
    }
}

template <typename TX, int D, int R>
int launch_scan(const void* x, float* out, float* state, const float* decay, const int* first_row, const int* start,
                const int* slot, int entries, const ScanArgs& a, hipStream_t stream) {
    constexpr int CW = PULSE_WAVE / R;
    const dim3 grid(entries, a.heads, (a.dv + CW - 1) / CW);
    hipLaunchKernelGGL((lightning_scan_kernel<TX, D, R>), grid, dim3(64), 0, stream, static_cast<const TX*>(x), out, state,
                       decay, first_row, start, slot, a);
    return 0;
}

template <typename TX, int D>
int launch_scan_d(int r, const void* x, float* out, float* state, const float* decay, const int* first_row,
                  const int* start, const int* slot, int entries, const ScanArgs& a, hipStream_t stream) {
    if constexpr (D >= 64) {
        if (r >= 16) return launch_scan<TX, D, 16>(x, out, state, decay, first_row, start, slot, entries, a, stream);
    }
    if (r >= 4) return launch_scan<TX, D, 4>(x, out, state, decay, first_row, start, slot, entries, a, stream);
    return launch_scan<TX, D, 1>(x, out, state, decay, first_row, start, slot, entries, a, stream);
}

}  // namespace

// x [T, x_stride]: the projection output that holds q, k (heads x d each) and v (heads x dv) from columns q0, k0, v0;
// out [T, o_stride] float32 receives the heads' outputs (heads x dv); state [slots, heads, d, dv] float32;
// decay [heads] float32; the entries' first rows [entries + 1], start positions and slots are read on the device.
// row_groups: over how many lanes a column's rows are shared out (1, 4 or 16; 16 from 64 key channels a head on).
extern "C" int pulse_lightning_scan(const void* x, int x_dtype, int64_t x_stride, int q0, int k0, int v0, float* out,
                                    int64_t o_stride, float* state, int slots, const float* decay,
                                    const int* entry_first_row, const int* entry_start, const int* entry_slot,
                                    int entries, int heads, int d, int dv, int act, int row_groups, hipStream_t stream) {
    PULSE_REQUIRE(entries >= 0 && heads > 0 && d > 0 && dv > 0 && slots > 0, "lightning_scan: bad sizes");
    PULSE_REQUIRE(d <= 256, "lightning_scan: at most 256 key channels a head, got %d", d);
    PULSE_REQUIRE(heads < 65536 && dv < 65536 * 4, "lightning_scan: too many heads or value channels");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && (act == 0 || act == 1), "lightning_scan: bad dtype tag or activation");
    PULSE_REQUIRE(x && out && state && decay && entry_first_row && entry_start && entry_slot, "lightning_scan: null pointer");
    PULSE_REQUIRE(q0 >= 0 && k0 >= 0 && v0 >= 0 && x_stride >= static_cast<int64_t>(q0) + heads * d &&
                  x_stride >= static_cast<int64_t>(k0) + heads * d && x_stride >= static_cast<int64_t>(v0) + heads * dv &&
                  o_stride >= static_cast<int64_t>(heads) * dv, "lightning_scan: rows are too short for their columns");
    if (entries == 0) return 0;
    ScanArgs a;
    a.heads = heads; a.d = d; a.dv = dv; a.x_stride = x_stride; a.o_stride = o_stride;
    a.q0 = q0; a.k0 = k0; a.v0 = v0; a.act = act;
    int rc = 0;
#define PULSE_SCAN_CASE(DD)                                                                                            \
    PULSE_DISPATCH_DTYPE(x_dtype, TX, rc = launch_scan_d<TX, DD>(row_groups, x, out, state, decay, entry_first_row,     \
                                                                 entry_start, entry_slot, entries, a, stream))
    if (d <= 16) PULSE_SCAN_CASE(16);
    else if (d <= 32) PULSE_SCAN_CASE(32);
    else if (d <= 64) PULSE_SCAN_CASE(64);
    else if (d <= 128) PULSE_SCAN_CASE(128);
    else PULSE_SCAN_CASE(256);
#undef PULSE_SCAN_CASE
    if (rc) return rc;
    PULSE_LAUNCH_CHECK("lightning_scan");
    return 0;
}

// y[t, i] = scale * o[t, i] / sqrt(mean_i(o[t]^2) + eps) * w[i] * sigmoid(gate[t, i]), one rounding; gate may be null.
extern "C" int pulse_gated_rmsnorm(const float* o, int64_t o_stride, const void* w, int w_dtype, const void* gate,
                                   int64_t gate_stride, void* y, int64_t y_stride, int x_dtype, int tokens, int n,
                                   float eps, float scale, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && n > 0 && o && w && y, "gated_rmsnorm: bad arguments");
    PULSE_REQUIRE(pulse_dtype_ok(w_dtype) && pulse_dtype_ok(x_dtype), "gated_rmsnorm: bad dtype tag");
    PULSE_REQUIRE(o_stride >= n && y_stride >= n && (!gate || gate_stride >= n), "gated_rmsnorm: rows are too short");
    if (tokens == 0) return 0;
    const int threads = n >= 1024 ? 256 : 128;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((gated_rmsnorm_kernel<TX, TW>), dim3(tokens), dim3(threads), 0, stream, o, o_stride,
                           static_cast<const TW*>(w), static_cast<const TX*>(gate), gate_stride, static_cast<TX*>(y),
                           y_stride, n, eps, scale)));
    PULSE_LAUNCH_CHECK("gated_rmsnorm");
    return 0;
}
