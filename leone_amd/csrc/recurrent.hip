// Mixers that keep a matrix memory per request and head instead of a cache of keys: S is [dim, vdim] float,
// carried from token to token in the request's state slot.
//
//   outer_scan   S_t = a_t S_(t-1) + b_t k_t v_t^T,  o_t = S_t^T q_t
//                a_t, b_t per head and token: a fixed decay with b = 1 (retention), or exponential gates with a
//                running maximum m_t = max(f_t + m_(t-1), i_t), a_t = exp(f_t + m_(t-1) - m_t),
//                b_t = exp(i_t - m_t), together with the normaliser n_t = a_t n_(t-1) + b_t k_t carried as one
//                more column of S (a value that is always 1), whose read-out n_t . q_t and m_t go out beside o
//                for the division that follows.  Rotary positions on q and k if tables come.
//   delta_scan   S <- g_t * S (g per key channel);  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//                with q and k made unit vectors per head first.
//
// One wave owns 64 columns of one head of one entry (a request's rows in the step), a lane one column with its
// dim elements in registers, and walks the entry's rows in order: a single decoded token and a prompt portion
// are the same kernel.  The vectors every lane needs (q_t, k_t, the decays) are prepared 16 tokens at a time in
// shared memory.  Everything here is float.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kScanTokens = 16;

struct OuterScanArgs {
    const float* proj;          // [rows, stride]
    long stride;
    int q_off, k_off, v_off;    // columns of head 0; head h of q and k at + h * dim, of v at + h * vdim
    int i_off, f_off;           // columns of the gates' pre-activations (one a head), -1: fixed decay
    AnyVec i_bias, f_bias;      // [heads]
    float cap;                  // gates go through cap * tanh(. / cap)
    const float* decay;         // [heads] for the fixed decay
    float q_scale, k_scale;
    const float* cos_table;     // [table_positions, rot_half] or null
    const float* sin_table;
    int rot_half, table_positions;
    float* state;               // [slots, heads, per_head]
    long slot_stride;
    int write_state;
    const int* spans;           // [entries, 2] first row and end
    const int* entry_slots;
    const int* positions;
    float* out;                 // [rows, heads, vdim]
    float* dot;                 // [rows, heads] n_t . q_t   (gated form only)
    float* top;                 // [rows, heads] m_t
    int heads, dim, vdim;
};

__device__ inline float rotated(const float* src, int i, int dim, const float* cos_row, const float* sin_row, int rot_half) {
    const float x = src[i];
    if (!cos_row || i >= 2 * rot_half) return x;
    if (i < rot_half) return x * cos_row[i] - src[i + rot_half] * sin_row[i];
    return x * cos_row[i - rot_half] + src[i - rot_half] * sin_row[i - rot_half];
}

__device__ inline float soft_cap_f(float z, float cap) { return cap * tanhf(z / cap); }
__device__ inline float log_sigmoid_f(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

template <int DKP>
__global__ void __launch_bounds__(kWave) outer_scan_kernel(OuterScanArgs p) {
    __shared__ __align__(16) float sq[kScanTokens][DKP];
    __shared__ __align__(16) float sk[kScanTokens][DKP];
    __shared__ float sa[kScanTokens], sb[kScanTokens], sm[kScanTokens], sli[kScanTokens], slf[kScanTokens];
    const int e = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const bool gated = p.i_off >= 0;
    const int col = blockIdx.z * kWave + lane;
    const int cols = p.vdim + (gated ? 1 : 0);
    const bool is_value = col < p.vdim, is_norm = gated && col == p.vdim;
    const int first = p.spans[2 * e], n = p.spans[2 * e + 1] - first;
    const bool fresh = p.positions[first] == 0;
    const long per_head = static_cast<long>(p.dim) * p.vdim + (gated ? p.dim + 1 : 0);
    float* mine = p.state + p.entry_slots[e] * p.slot_stride + head * per_head;

    float S[DKP];
#pragma unroll
    for (int i = 0; i < DKP; ++i) {
        float v = 0.f;
        if (!fresh && i < p.dim) {
            if (is_value) v = mine[static_cast<long>(i) * p.vdim + col];
            else if (is_norm) v = mine[static_cast<long>(p.dim) * p.vdim + i];
        }
        S[i] = v;
    }
    float m = (gated && !fresh) ? mine[static_cast<long>(p.dim) * p.vdim + p.dim] : 0.f;
    const float fixed = gated ? 0.f : p.decay[head];

    for (int t0 = 0; t0 < n; t0 += kScanTokens) {
        const int here = min(kScanTokens, n - t0);
        for (int idx = lane; idx < here * DKP; idx += kWave) {
            const int t = idx / DKP, i = idx % DKP;
            const long row = first + t0 + t;
            float qv = 0.f, kv = 0.f;
            if (i < p.dim) {
                const int pos = min(p.positions[row], p.table_positions - 1);
                const float* c = p.cos_table ? p.cos_table + static_cast<long>(pos) * p.rot_half : nullptr;
                const float* s = p.cos_table ? p.sin_table + static_cast<long>(pos) * p.rot_half : nullptr;
                const float* base = p.proj + row * p.stride;
                qv = rotated(base + p.q_off + head * p.dim, i, p.dim, c, s, p.rot_half) * p.q_scale;
                kv = rotated(base + p.k_off + head * p.dim, i, p.dim, c, s, p.rot_half) * p.k_scale;
            }
            sq[t][i] = qv;
            sk[t][i] = kv;
        }
        if (gated) {
            if (lane < here) {
                const float* base = p.proj + static_cast<long>(first + t0 + lane) * p.stride;
                sli[lane] = soft_cap_f(base[p.i_off + head] + load_any(p.i_bias, head), p.cap);                 // log input gate
                slf[lane] = log_sigmoid_f(soft_cap_f(base[p.f_off + head] + load_any(p.f_bias, head), p.cap));  // log forget gate
            }
            __syncthreads();
            // the running maximum goes from token to token: every lane walks it by itself, lane 0 notes the weights
            float walk = m;
            for (int t = 0; t < here; ++t) {
                const float li = sli[t], lf = slf[t];
                const float next = fmaxf(lf + walk, li);
                if (lane == 0) {
                    sm[t] = next;
                    sa[t] = expf(lf + walk - next);
                    sb[t] = expf(li - next);
                }
                walk = next;
            }
            m = walk;
        }
        __syncthreads();
        if (col < cols) {
            for (int t = 0; t < here; ++t) {
                const long row = first + t0 + t;
                const float a = gated ? sa[t] : fixed;
                const float b = gated ? sb[t] : 1.f;
                const float v = is_value ? p.proj[row * p.stride + p.v_off + head * p.vdim + col] : 1.f;
                const float bv = b * v;
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < DKP; ++i) {
                    S[i] = fmaf(a, S[i], sk[t][i] * bv);
                    acc = fmaf(S[i], sq[t][i], acc);
                }
                const long at = row * p.heads + head;
                if (is_value) p.out[at * p.vdim + col] = acc;
                else {
                    p.dot[at] = acc;
                    p.top[at] = sm[t];
                }
            }
        }
        __syncthreads();
    }
    if (!p.write_state || col >= cols) return;
#pragma unroll
    for (int i = 0; i < DKP; ++i) {
        if (i < p.dim) {
            if (is_value) mine[static_cast<long>(i) * p.vdim + col] = S[i];
            else mine[static_cast<long>(p.dim) * p.vdim + i] = S[i];
        }
    }
    if (is_norm) mine[static_cast<long>(p.dim) * p.vdim + p.dim] = m;
}

struct DeltaScanArgs {
    const float* qkv;           // [rows, stride]: q and k heads (kv_heads x dim each), then v heads (heads x vdim)
    long stride;
    int q_off, k_off, v_off;
    const float* beta;          // [rows, beta_stride]: pre-activation of the write strength, one a head
    long beta_stride;
    const float* step;          // [rows, step_stride]: pre-activation of the step size, heads x dim
    long step_stride;
    AnyVec rate_log;            // [heads]: decay = exp(-exp(rate_log) * softplus(step + step_bias))
    AnyVec step_bias;           // [heads * dim]
    float q_scale, unit_eps;
    float* state;               // [slots, heads, dim, vdim]
    long slot_stride;
    int write_state;
    const int* spans;
    const int* entry_slots;
    const int* positions;
    float* out;                 // [rows, heads, vdim]
    int heads, kv_heads, dim, vdim;
};

__device__ inline float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <int DKP>
__global__ void __launch_bounds__(kWave) delta_scan_kernel(DeltaScanArgs p) {
    __shared__ __align__(16) float sq[kScanTokens][DKP];
    __shared__ __align__(16) float sk[kScanTokens][DKP];
    __shared__ __align__(16) float sg[kScanTokens][DKP];
    __shared__ float sbeta[kScanTokens];
    const int e = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int kvh = head / (p.heads / p.kv_heads);
    const int col = blockIdx.z * kWave + lane;
    const bool live = col < p.vdim;
    const int first = p.spans[2 * e], n = p.spans[2 * e + 1] - first;
    const bool fresh = p.positions[first] == 0;
    float* mine = p.state + p.entry_slots[e] * p.slot_stride + static_cast<long>(head) * p.dim * p.vdim;
    const float rate = expf(load_any(p.rate_log, head));

    float S[DKP];
#pragma unroll
    for (int i = 0; i < DKP; ++i) S[i] = (!fresh && live && i < p.dim) ? mine[static_cast<long>(i) * p.vdim + col] : 0.f;

    for (int t0 = 0; t0 < n; t0 += kScanTokens) {
        const int here = min(kScanTokens, n - t0);
        for (int t = 0; t < here; ++t) {
            const long row = first + t0 + t;
            const float* base = p.qkv + row * p.stride;
            const float* qs = base + p.q_off + kvh * p.dim;
            const float* ks = base + p.k_off + kvh * p.dim;
            float qq = 0.f, kk = 0.f;
            for (int i = lane; i < p.dim; i += kWave) {
                qq = fmaf(qs[i], qs[i], qq);
                kk = fmaf(ks[i], ks[i], kk);
            }
            const float qinv = p.q_scale / sqrtf(wave_sum(qq) + p.unit_eps);
            const float kinv = 1.0f / sqrtf(wave_sum(kk) + p.unit_eps);
            for (int i = lane; i < DKP; i += kWave) {
                const bool in = i < p.dim;
                sq[t][i] = in ? qs[i] * qinv : 0.f;
                sk[t][i] = in ? ks[i] * kinv : 0.f;
                const long ch = static_cast<long>(head) * p.dim + i;
                sg[t][i] = in ? expf(-rate * softplus_f(p.step[row * p.step_stride + ch] + load_any(p.step_bias, ch))) : 1.f;
            }
            if (lane == 0) sbeta[t] = 1.0f / (1.0f + expf(-p.beta[row * p.beta_stride + head]));
        }
        __syncthreads();
        if (live) {
            for (int t = 0; t < here; ++t) {
                const long row = first + t0 + t;
                const float v = p.qkv[row * p.stride + p.v_off + head * p.vdim + col];
                float seen = 0.f;
#pragma unroll
                for (int i = 0; i < DKP; ++i) {
                    S[i] *= sg[t][i];
                    seen = fmaf(S[i], sk[t][i], seen);
                }
                const float u = sbeta[t] * (v - seen);
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < DKP; ++i) {
                    S[i] = fmaf(sk[t][i], u, S[i]);
                    acc = fmaf(S[i], sq[t][i], acc);
                }
                p.out[(row * p.heads + head) * p.vdim + col] = acc;
            }
        }
        __syncthreads();
    }
    if (!p.write_state || !live) return;
#pragma unroll
    for (int i = 0; i < DKP; ++i)
        if (i < p.dim) mine[static_cast<long>(i) * p.vdim + col] = S[i];
}

static bool known_vec(int dtype) { return dtype == kF32 || dtype == kBF16; }

}  // namespace leone

using namespace leone;

extern "C" int leone_scan_max_dim() { return 256; }

#define LEONE_SCAN_DISPATCH(KERNEL, ARGS, DIM, GRID)                                  \
    do {                                                                              \
        if (DIM <= 32) KERNEL<32><<<GRID, kWave, 0, stream>>>(ARGS);                  \
        else if (DIM <= 64) KERNEL<64><<<GRID, kWave, 0, stream>>>(ARGS);             \
        else if (DIM <= 96) KERNEL<96><<<GRID, kWave, 0, stream>>>(ARGS);             \
        else if (DIM <= 128) KERNEL<128><<<GRID, kWave, 0, stream>>>(ARGS);           \
        else if (DIM <= 192) KERNEL<192><<<GRID, kWave, 0, stream>>>(ARGS);           \
        else KERNEL<256><<<GRID, kWave, 0, stream>>>(ARGS);                           \
    } while (0)

extern "C" int leone_outer_scan(const float* proj, long stride, int q_off, int k_off, int v_off, int i_off, int f_off,
                                const void* i_bias, const void* f_bias, int bias_dtype, float cap, const float* decay,
                                float q_scale, float k_scale, const float* cos_table, const float* sin_table, int rotary_dim,
                                int table_positions, float* state, long slot_stride, int write_state, const int* spans,
                                const int* entry_slots, const int* positions, int entries, float* out, float* dot, float* top,
                                int heads, int dim, int vdim, hipStream_t stream) {
    LEONE_REQUIRE(proj && state && spans && entry_slots && positions && out, "outer_scan: null pointer");
    LEONE_REQUIRE(entries > 0 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0, "outer_scan: %d entries, %d heads of %d x %d",
                  entries, heads, dim, vdim);
    LEONE_REQUIRE(dim <= leone_scan_max_dim(), "outer_scan: heads of %d key channels, the kernel takes up to %d", dim, leone_scan_max_dim());
    const bool gated = i_off >= 0;
    LEONE_REQUIRE(gated == (f_off >= 0), "outer_scan: the two gates come together");
    LEONE_REQUIRE(!gated || (i_bias && f_bias && known_vec(bias_dtype) && cap > 0.f && dot && top),
                  "outer_scan: gates need their biases, a positive cap and room for the denominator's parts");
    LEONE_REQUIRE(gated || decay, "outer_scan: neither gates nor a fixed decay");
    LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "outer_scan: cos and sin tables come together");
    LEONE_REQUIRE(!cos_table || (rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= dim && table_positions > 0),
                  "outer_scan: rotary_dim %d must be even, positive and at most %d", rotary_dim, dim);
    const long per_head = static_cast<long>(dim) * vdim + (gated ? dim + 1 : 0);
    LEONE_REQUIRE(slot_stride >= heads * per_head, "outer_scan: a state slot of %ld floats is too small", slot_stride);
    LEONE_REQUIRE(stride >= q_off + heads * dim && stride >= k_off + heads * dim && stride >= v_off + heads * vdim &&
                  (!gated || (stride >= i_off + heads && stride >= f_off + heads)) && q_off >= 0 && k_off >= 0 && v_off >= 0,
                  "outer_scan: the projection's rows of %ld do not hold the named columns", stride);
    OuterScanArgs a{proj, stride, q_off, k_off, v_off, gated ? i_off : -1, gated ? f_off : -1, AnyVec{i_bias, bias_dtype},
                    AnyVec{f_bias, bias_dtype}, cap, decay, q_scale, k_scale, cos_table, sin_table,
                    cos_table ? rotary_dim / 2 : 0, cos_table ? table_positions : 1, state, slot_stride, write_state, spans,
                    entry_slots, positions, out, dot, top, heads, dim, vdim};
    const dim3 grid(entries, heads, ceil_div(vdim + (gated ? 1 : 0), kWave));
    LEONE_SCAN_DISPATCH(outer_scan_kernel, a, dim, grid);
    LEONE_LAUNCH_CHECK("outer_scan");
    return 0;
}

extern "C" int leone_delta_scan(const float* qkv, long stride, int q_off, int k_off, int v_off, const float* beta,
                                long beta_stride, const float* step, long step_stride, const void* rate_log,
                                const void* step_bias, int vec_dtype, float q_scale, float unit_eps, float* state,
                                long slot_stride, int write_state, const int* spans, const int* entry_slots,
                                const int* positions, int entries, float* out, int heads, int kv_heads, int dim, int vdim,
                                hipStream_t stream) {
    LEONE_REQUIRE(qkv && beta && step && rate_log && step_bias && state && spans && entry_slots && positions && out,
                  "delta_scan: null pointer");
    LEONE_REQUIRE(known_vec(vec_dtype), "delta_scan: unknown element type");
    LEONE_REQUIRE(entries > 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
                  "delta_scan: %d entries, %d heads over %d key heads of %d x %d", entries, heads, kv_heads, dim, vdim);
    LEONE_REQUIRE(dim <= leone_scan_max_dim(), "delta_scan: heads of %d key channels, the kernel takes up to %d", dim, leone_scan_max_dim());
    LEONE_REQUIRE(slot_stride >= static_cast<long>(heads) * dim * vdim, "delta_scan: a state slot of %ld floats is too small", slot_stride);
    LEONE_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && stride >= q_off + kv_heads * dim && stride >= k_off + kv_heads * dim &&
                  stride >= v_off + heads * vdim && beta_stride >= heads && step_stride >= static_cast<long>(heads) * dim,
                  "delta_scan: rows too short for the named columns");
    DeltaScanArgs a{qkv, stride, q_off, k_off, v_off, beta, beta_stride, step, step_stride, AnyVec{rate_log, vec_dtype},
                    AnyVec{step_bias, vec_dtype}, q_scale, unit_eps, state, slot_stride, write_state, spans, entry_slots,
                    positions, out, heads, kv_heads, dim, vdim};
    const dim3 grid(entries, heads, ceil_div(vdim, kWave));
    LEONE_SCAN_DISPATCH(delta_scan_kernel, a, dim, grid);
    LEONE_LAUNCH_CHECK("delta_scan");
    return 0;
}
