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
// A workgroup of four waves owns a run of columns of one head of one segment (a request's rows in the step, or a
// chunk of them) and walks the segment's rows in order: a single decoded token and a prompt portion are the same
// kernel.  A column's dim elements are spread over 1, 2, 4 or 8 lanes, 32 to a lane in registers (so that several
// waves fit a SIMD and hide each other's waits); the lanes of a column add their parts of a read-out by shuffles.
// The vectors every lane needs (q_t, k_t, the decays) are prepared 16 tokens at a time in shared memory.
// Everything here is float.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kScanTokens = 16;
constexpr int kLaneRows = 32;       // key channels a lane holds
constexpr int kScanThreads = 256;
constexpr int kLaneCols = 2;        // columns a lane holds in the outer-product scan: every q and k it reads serves both

// Over how many lanes a column of `dim` key channels is spread: 1, 2, 4 or 8 (dim up to 256).
inline int lane_groups(int dim) { return dim <= 32 ? 1 : dim <= 64 ? 2 : dim <= 128 ? 4 : 8; }

// A segment is a run of consecutive rows of one request that one wave walks in order: rows [first, end), the
// state it starts from (index `in` into the launch's input states, negative: zeros) and where the state it ends
// with goes (index `out` into the launch's output states, negative: nowhere).  A decoded token or a short portion
// is one segment from and into the request's state slot.  A long portion is cut into chunks that are walked side
// by side, three launches instead of one: every chunk from zeros (what the chunk's own rows write, and what they
// read of it), then the chunks' end states chained into the state each chunk starts from (outer_chain), then every
// chunk once more from that state with nothing written into it (`no_input`), added to the first walk's read-outs.
struct Segment {
    int first, end, in, out;
};

struct OuterScanArgs {
    const float* proj;          // [rows, stride]
    long stride;
    int q_off, k_off, v_off;    // columns of head 0; head h of q and k at + h * dim, of v at + h * vdim
    const float* coef;          // [rows, heads, 2]: a_t and b_t, or null: a = decay[head], b = 1
    const float* decay;         // [heads]
    int no_input;               // b is taken as 0: the state is only carried through the rows and read
    int accumulate;             // read-outs are added to what out and dot hold
    int norm_column;            // one more column whose value is always 1 (the normaliser), read out into dot
    float q_scale, k_scale;
    const float* cos_table;     // [table_positions, rot_half] or null
    const float* sin_table;
    int rot_half, table_positions;
    const int* positions;
    const Segment* segments;
    const float* state_in;      // [index, heads, head_stride]
    long in_stride;
    float* state_out;
    long out_stride;
    long head_stride;           // floats from head to head in a state: S [dim, vdim], then the normaliser [dim]
    float* decay_product;       // [segments, heads]: the product of a_t over the segment's rows, or null
    float* out;                 // [rows, heads, vdim]
    float* dot;                 // [rows, heads]
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

// The exponential gates of an entry's rows, one wave per (entry, head): log gates i_t = soft_cap(pre_i + bias_i),
// f_t = logsigmoid(soft_cap(pre_f + bias_f)); running maximum m_t = max(f_t + m_(t-1), i_t) from the request's
// state (0 at a sequence's start); a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t).  coef[row, head] = (a, b),
// top[row, head] = m_t; the last m goes back into the state.
__global__ void __launch_bounds__(kScanThreads)
exp_gates_kernel(const float* __restrict__ proj, long stride, int i_off, int f_off, AnyVec i_bias, AnyVec f_bias, float cap,
                 const int* __restrict__ spans, float* __restrict__ state, long slot_stride, long head_stride, long top_at,
                 int write_state, float* __restrict__ coef, float* __restrict__ top, int heads) {
    __shared__ float sli[kScanThreads], slf[kScanThreads];
    const int e = blockIdx.x, head = blockIdx.y, tid = threadIdx.x, lane = tid % kWave;
    const int first = spans[4 * e], end = spans[4 * e + 1], in = spans[4 * e + 2], out = spans[4 * e + 3];
    float m = in < 0 ? 0.f : state[in * slot_stride + head * head_stride + top_at];
    const float bi = load_any(i_bias, head), bf = load_any(f_bias, head);
    // m -> max(A + m, B) is what a row does to the maximum; rows compose as (A2, B2) after (A1, B1) =
    // (A1 + A2, max(A2 + B1, B2)), so 64 rows are walked by a prefix scan over the lanes instead of one by one.
    // All four waves make the log gates of 256 rows; the first wave then walks them 64 at a time.
    for (int r0 = first; r0 < end; r0 += kScanThreads) {
        float li = -INFINITY, lf = 0.f;
        if (r0 + tid < end) {
            const float* base = proj + static_cast<long>(r0 + tid) * stride;
            li = soft_cap_f(base[i_off + head] + bi, cap);
            lf = log_sigmoid_f(soft_cap_f(base[f_off + head] + bf, cap));
        }
        sli[tid] = li;
        slf[tid] = lf;
        __syncthreads();
        if (tid < kWave) {
            for (int t0 = r0; t0 < min(end, r0 + kScanThreads); t0 += kWave) {
                const int here = min(kWave, end - t0);
                li = sli[t0 - r0 + lane];
                lf = slf[t0 - r0 + lane];
                float A = lf, B = li;
#pragma unroll
                for (int off = 1; off < kWave; off <<= 1) {
                    const float Ap = __shfl_up(A, off, kWave), Bp = __shfl_up(B, off, kWave);
                    if (lane >= off) {
                        B = fmaxf(A + Bp, B);
                        A = A + Ap;
                    }
                }
                const float mine_m = fmaxf(A + m, B);
                float before = __shfl_up(mine_m, 1, kWave);
                if (lane == 0) before = m;
                if (lane < here) {
                    const long at = static_cast<long>(t0 + lane) * heads + head;
                    coef[2 * at] = expf(lf + before - mine_m);
                    coef[2 * at + 1] = expf(li - mine_m);
                    top[at] = mine_m;
                }
                m = __shfl(mine_m, here - 1, kWave);
            }
        }
        __syncthreads();
    }
    if (write_state && out >= 0 && tid == 0) state[out * slot_stride + head * head_stride + top_at] = m;
}

__global__ void __launch_bounds__(kScanThreads) outer_scan_kernel(OuterScanArgs p, int groups) {
    extern __shared__ __align__(16) float scan_lds[];
    const int dkp = groups * kLaneRows;
    float* sq = scan_lds;                       // [kScanTokens][dkp]
    float* sk = sq + kScanTokens * dkp;
    float* sa = sk + kScanTokens * dkp;         // [kScanTokens]
    float* sb = sa + kScanTokens;
    const int head = blockIdx.y, tid = threadIdx.x, lane = tid % kWave;
    const Segment seg = p.segments[blockIdx.x];
    const int per_wave = kWave / groups;                       // lanes a wave has for columns; each holds kLaneCols of them
    const int part = lane / per_wave;                          // which 32 key channels of its columns this lane holds
    const int cols = p.vdim + (p.norm_column ? 1 : 0);
    int col[kLaneCols];
    bool is_value[kLaneCols], is_norm[kLaneCols];
#pragma unroll
    for (int c = 0; c < kLaneCols; ++c) {
        col[c] = ((blockIdx.z * (kScanThreads / kWave) + tid / kWave) * kLaneCols + c) * per_wave + lane % per_wave;
        is_value[c] = col[c] < p.vdim;
        is_norm[c] = p.norm_column && col[c] == p.vdim;
    }
    const int first = seg.first, n = seg.end - seg.first;
    const int ch0 = part * kLaneRows;
    const float* from = seg.in < 0 ? nullptr : p.state_in + seg.in * p.in_stride + head * p.head_stride;

    float S[kLaneCols][kLaneRows];
#pragma unroll
    for (int c = 0; c < kLaneCols; ++c) {
#pragma unroll
        for (int i = 0; i < kLaneRows; ++i) {
            float v = 0.f;
            if (from && ch0 + i < p.dim) {
                if (is_value[c]) v = from[static_cast<long>(ch0 + i) * p.vdim + col[c]];
                else if (is_norm[c]) v = from[static_cast<long>(p.dim) * p.vdim + ch0 + i];
            }
            S[c][i] = v;
        }
    }
    const float fixed = p.coef ? 0.f : p.decay[head];
    float carried = 1.f;                                      // the product of the segment's decays

    for (int t0 = 0; t0 < n; t0 += kScanTokens) {
        const int here = min(kScanTokens, n - t0);
        for (int idx = tid; idx < here * dkp; idx += kScanThreads) {
            const int t = idx / dkp, i = idx % dkp;
            const long row = first + t0 + t;
            float qv = 0.f, kv = 0.f;
            if (i < p.dim) {
                const int pos = min(p.positions[row], p.table_positions - 1);
                const float* c = p.cos_table ? p.cos_table + static_cast<long>(pos) * p.rot_half : nullptr;
                const float* s = p.cos_table ? p.sin_table + static_cast<long>(pos) * p.rot_half : nullptr;
                const float* base = p.proj + row * p.stride;
                qv = rotated(base + p.q_off + head * p.dim, i, p.dim, c, s, p.rot_half) * p.q_scale;
                if (!p.no_input) kv = rotated(base + p.k_off + head * p.dim, i, p.dim, c, s, p.rot_half) * p.k_scale;
            }
            sq[idx] = qv;
            sk[idx] = kv;
        }
        if (tid < here) {
            const long at = static_cast<long>(first + t0 + tid) * p.heads + head;
            sa[tid] = p.coef ? p.coef[2 * at] : fixed;
            sb[tid] = p.no_input ? 0.f : (p.coef ? p.coef[2 * at + 1] : 1.f);
        }
        __syncthreads();
        if (col[0] < cols) {                                   // the lanes of a column are in or out together
            for (int t = 0; t < here; ++t) {
                const long row = first + t0 + t;
                const float a = sa[t];
                const float* kt = sk + t * dkp + ch0;
                const float* qt = sq + t * dkp + ch0;
                float acc[kLaneCols];
                if (p.no_input) {                              // nothing is written: the state decays and is read
#pragma unroll
                    for (int c = 0; c < kLaneCols; ++c) acc[c] = 0.f;
#pragma unroll
                    for (int i = 0; i < kLaneRows; ++i) {
                        const float q = qt[i];
#pragma unroll
                        for (int c = 0; c < kLaneCols; ++c) {
                            S[c][i] *= a;
                            acc[c] = fmaf(S[c][i], q, acc[c]);
                        }
                    }
                } else {
                    float bv[kLaneCols];
#pragma unroll
                    for (int c = 0; c < kLaneCols; ++c) {
                        const float v = is_value[c] ? p.proj[row * p.stride + p.v_off + head * p.vdim + col[c]] : 1.f;
                        bv[c] = sb[t] * v;
                        acc[c] = 0.f;
                    }
#pragma unroll
                    for (int i = 0; i < kLaneRows; ++i) {
                        const float k = kt[i], q = qt[i];
#pragma unroll
                        for (int c = 0; c < kLaneCols; ++c) {
                            S[c][i] = fmaf(a, S[c][i], k * bv[c]);
                            acc[c] = fmaf(S[c][i], q, acc[c]);
                        }
                    }
                }
                carried *= a;
#pragma unroll
                for (int c = 0; c < kLaneCols; ++c) {
                    for (int off = per_wave; off < kWave; off <<= 1) acc[c] += __shfl_xor(acc[c], off, kWave);
                    if (part == 0 && col[c] < cols) {
                        const long at = row * p.heads + head;
                        float* dst = is_value[c] ? p.out + at * p.vdim + col[c] : p.dot + at;
                        *dst = p.accumulate ? *dst + acc[c] : acc[c];
                    }
                }
            }
        }
        __syncthreads();
    }
    if (p.decay_product && blockIdx.z == 0 && tid == 0) p.decay_product[static_cast<long>(blockIdx.x) * p.heads + head] = carried;
    if (!p.state_out || seg.out < 0) return;
    float* to = p.state_out + seg.out * p.out_stride + head * p.head_stride;
#pragma unroll
    for (int c = 0; c < kLaneCols; ++c) {
        if (col[c] >= cols) continue;
#pragma unroll
        for (int i = 0; i < kLaneRows; ++i) {
            if (ch0 + i < p.dim) {
                if (is_value[c]) to[static_cast<long>(ch0 + i) * p.vdim + col[c]] = S[c][i];
                else to[static_cast<long>(p.dim) * p.vdim + ch0 + i] = S[c][i];
            }
        }
    }
}

// The chunks' end states chained: for a long portion whose chunks are [g0, g1) of `work` (each holding what its
// own rows wrote, from zeros), S = the request's state (zeros at a sequence's start); for every chunk in order:
// what the chunk holds is replaced by S (the state it starts from), and S <- product[chunk] * S + what it held.
// The last S is the request's new state.  links[l] = (slot, fresh, g0, g1).
__global__ void outer_chain_kernel(const int* __restrict__ links, float* __restrict__ work, long work_stride,
                                   const float* __restrict__ product, float* __restrict__ state, long slot_stride,
                                   long head_stride, int per_head, int heads, int write_state) {
    const int l = blockIdx.x, head = blockIdx.y;
    const int el = blockIdx.z * blockDim.x + threadIdx.x;
    if (el >= per_head) return;
    const int slot = links[4 * l], fresh = links[4 * l + 1], g0 = links[4 * l + 2], g1 = links[4 * l + 3];
    float* mine = state + slot * slot_stride + head * head_stride + el;
    float S = fresh ? 0.f : *mine;
    for (int g = g0; g < g1; ++g) {
        float* at = work + g * work_stride + head * head_stride + el;
        const float wrote = *at;
        *at = S;
        S = fmaf(product[static_cast<long>(g) * heads + head], S, wrote);
    }
    if (write_state) *mine = S;
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
    int no_input;               // v is taken as 0: what a state carries through the rows, and what is read of it
    int accumulate;             // read-outs are added to what out holds
    const Segment* segments;
    const float* state_in;      // [index, heads, dim, vdim]
    long in_stride;
    float* state_out;
    long out_stride;
    float* transition;          // [segments, heads, dim, dim] or null: what the segment's rows do to a state that comes
                                // in, as a matrix: dim more columns that start as the unit vectors and are given v = 0;
                                // stored [unit vector j][channel i], the order in which the chain reads it
    float* out;                 // [rows, heads, vdim]
    int heads, kv_heads, dim, vdim;
};

__device__ inline float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

__global__ void __launch_bounds__(kScanThreads) delta_scan_kernel(DeltaScanArgs p, int groups) {
    extern __shared__ __align__(16) float scan_lds[];
    const int dkp = groups * kLaneRows;
    float* sq = scan_lds;                       // [kScanTokens][dkp] each
    float* sk = sq + kScanTokens * dkp;
    float* sg = sk + kScanTokens * dkp;
    float* sbeta = sg + kScanTokens * dkp;      // [kScanTokens]
    const int head = blockIdx.y, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const Segment seg = p.segments[blockIdx.x];
    const int kvh = head / (p.heads / p.kv_heads);
    const int per_wave = kWave / groups;
    const int part = lane / per_wave;
    const int col = (blockIdx.z * (kScanThreads / kWave) + wave) * per_wave + lane % per_wave;
    const bool is_value = col < p.vdim;
    const int unit = (p.transition && !is_value && col < p.vdim + p.dim) ? col - p.vdim : -1;   // a unit vector's column
    const bool live = is_value || unit >= 0;
    const int ch0 = part * kLaneRows;
    const int first = seg.first, n = seg.end - seg.first;
    const long head_size = static_cast<long>(p.dim) * p.vdim;
    const float* from = seg.in < 0 ? nullptr : p.state_in + seg.in * p.in_stride + head * head_size;
    const float rate = expf(load_any(p.rate_log, head));

    float S[kLaneRows];
#pragma unroll
    for (int i = 0; i < kLaneRows; ++i) {
        float v = 0.f;
        if (is_value && from && ch0 + i < p.dim) v = from[static_cast<long>(ch0 + i) * p.vdim + col];
        if (unit >= 0 && ch0 + i == unit) v = 1.f;
        S[i] = v;
    }

    for (int t0 = 0; t0 < n; t0 += kScanTokens) {
        const int here = min(kScanTokens, n - t0);
        {   // sixteen lanes prepare a row's vectors, all rows of the chunk at once
            constexpr int kRowLanes = kScanThreads / kScanTokens;
            const int t = tid / kRowLanes, sub = tid % kRowLanes;
            if (t < here) {
                const long row = first + t0 + t;
                const float* base = p.qkv + row * p.stride;
                const float* qs = base + p.q_off + kvh * p.dim;
                const float* ks = base + p.k_off + kvh * p.dim;
                float qq = 0.f, kk = 0.f;
                for (int i = sub; i < p.dim; i += kRowLanes) {
                    qq = fmaf(qs[i], qs[i], qq);
                    kk = fmaf(ks[i], ks[i], kk);
                }
#pragma unroll
                for (int off = kRowLanes / 2; off > 0; off >>= 1) {
                    qq += __shfl_xor(qq, off, kWave);
                    kk += __shfl_xor(kk, off, kWave);
                }
                const float qinv = p.q_scale / sqrtf(qq + p.unit_eps);
                const float kinv = 1.0f / sqrtf(kk + p.unit_eps);
                for (int i = sub; i < dkp; i += kRowLanes) {
                    const bool in = i < p.dim;
                    sq[t * dkp + i] = in ? qs[i] * qinv : 0.f;
                    sk[t * dkp + i] = in ? ks[i] * kinv : 0.f;
                    const long ch = static_cast<long>(head) * p.dim + i;
                    sg[t * dkp + i] = in ? expf(-rate * softplus_f(p.step[row * p.step_stride + ch] + load_any(p.step_bias, ch))) : 1.f;
                }
                if (sub == 0) sbeta[t] = 1.0f / (1.0f + expf(-p.beta[row * p.beta_stride + head]));
            }
        }
        __syncthreads();
        if (live) {                                            // the lanes of a column are in or out together
            for (int t = 0; t < here; ++t) {
                const long row = first + t0 + t;
                const float v = (is_value && !p.no_input) ? p.qkv[row * p.stride + p.v_off + head * p.vdim + col] : 0.f;
                const float* gt = sg + t * dkp + ch0;
                const float* kt = sk + t * dkp + ch0;
                const float* qt = sq + t * dkp + ch0;
                float seen = 0.f;
#pragma unroll
                for (int i = 0; i < kLaneRows; ++i) {
                    S[i] *= gt[i];
                    seen = fmaf(S[i], kt[i], seen);
                }
                for (int off = per_wave; off < kWave; off <<= 1) seen += __shfl_xor(seen, off, kWave);
                const float u = sbeta[t] * (v - seen);
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < kLaneRows; ++i) {
                    S[i] = fmaf(kt[i], u, S[i]);
                    acc = fmaf(S[i], qt[i], acc);
                }
                for (int off = per_wave; off < kWave; off <<= 1) acc += __shfl_xor(acc, off, kWave);
                if (part == 0 && is_value) {
                    float* dst = p.out + (row * p.heads + head) * p.vdim + col;
                    *dst = p.accumulate ? *dst + acc : acc;
                }
            }
        }
        __syncthreads();
    }
    if (unit >= 0) {
        float* to = p.transition + (static_cast<long>(blockIdx.x) * p.heads + head) * p.dim * p.dim;
#pragma unroll
        for (int i = 0; i < kLaneRows; ++i)
            if (ch0 + i < p.dim) to[static_cast<long>(unit) * p.dim + ch0 + i] = S[i];
        return;
    }
    if (!p.state_out || seg.out < 0 || !is_value) return;
    float* to = p.state_out + seg.out * p.out_stride + head * head_size;
#pragma unroll
    for (int i = 0; i < kLaneRows; ++i)
        if (ch0 + i < p.dim) to[static_cast<long>(ch0 + i) * p.vdim + col] = S[i];
}

// The chunks of a long portion chained for the delta rule: a chunk's rows turn a state S that comes in into
// transition[chunk] . S + (what the chunk holds: its end state from zeros).  As in outer_chain_kernel every chunk's
// place in `work` ends up holding the state the chunk starts from, and the last state is the request's new one.
// A workgroup owns a run of columns of one head; a column's channels are spread over lanes as in the scans, and
// the whole column passes through shared memory so that every lane sees all of it.
__global__ void __launch_bounds__(kScanThreads)
delta_chain_kernel(const int* __restrict__ links, float* __restrict__ work, long work_stride, const float* __restrict__ transition,
                   float* __restrict__ state, long slot_stride, int heads, int dim, int vdim, int groups, int tile, int write_state) {
    extern __shared__ __align__(16) float chain_lds[];
    const int dkp = groups * kLaneRows;
    const int l = blockIdx.x, head = blockIdx.y, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int per_wave = kWave / groups, per_block = (kScanThreads / kWave) * per_wave;
    float* sS = chain_lds;                      // [dkp][columns a workgroup]: the state that comes in
    float* sT = chain_lds + dkp * per_block;    // [tile][dkp]: `tile` columns of the transition, turned
    const int part = lane / per_wave, local = wave * per_wave + lane % per_wave;
    const int col = blockIdx.z * per_block + local;
    const bool live = col < vdim;
    const int ch0 = part * kLaneRows;
    const int slot = links[4 * l], fresh = links[4 * l + 1], g0 = links[4 * l + 2], g1 = links[4 * l + 3];
    const long head_size = static_cast<long>(dim) * vdim;
    float* mine = state + slot * slot_stride + head * head_size;
    float S[kLaneRows];
#pragma unroll
    for (int i = 0; i < kLaneRows; ++i)
        S[i] = (!fresh && live && ch0 + i < dim) ? mine[static_cast<long>(ch0 + i) * vdim + col] : 0.f;
    for (int g = g0; g < g1; ++g) {
        float* held = work + g * work_stride + head * head_size;
        const float* T = transition + (static_cast<long>(g) * heads + head) * dim * dim;
        float next[kLaneRows];
#pragma unroll
        for (int i = 0; i < kLaneRows; ++i) {
            const bool in = live && ch0 + i < dim;
            next[i] = in ? held[static_cast<long>(ch0 + i) * vdim + col] : 0.f;
            if (in) held[static_cast<long>(ch0 + i) * vdim + col] = S[i];
            sS[(ch0 + i) * per_block + local] = S[i];
        }
        for (int j0 = 0; j0 < dim; j0 += tile) {
            __syncthreads();
            for (int idx = tid; idx < tile * dkp; idx += kScanThreads) {
                const int jj = idx / dkp, i = idx % dkp;
                sT[idx] = (i < dim && j0 + jj < dim) ? T[static_cast<long>(j0 + jj) * dim + i] : 0.f;
            }
            __syncthreads();
            const int width = min(tile, dim - j0);
            for (int jj = 0; jj < width; ++jj) {
                const float s = sS[(j0 + jj) * per_block + local];
                const float* column = sT + jj * dkp + ch0;
#pragma unroll
                for (int i = 0; i < kLaneRows; ++i) next[i] = fmaf(column[i], s, next[i]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < kLaneRows; ++i) S[i] = next[i];
    }
    if (!write_state || !live) return;
#pragma unroll
    for (int i = 0; i < kLaneRows; ++i)
        if (ch0 + i < dim) mine[static_cast<long>(ch0 + i) * vdim + col] = S[i];
}

static bool known_vec(int dtype) { return dtype == kF32 || dtype == kBF16; }

}  // namespace leone

using namespace leone;

extern "C" int leone_scan_max_dim() { return 256; }

extern "C" int leone_exp_gates(const float* proj, long stride, int i_off, int f_off, const void* i_bias, const void* f_bias,
                               int bias_dtype, float cap, const int* spans, int entries, float* state, long slot_stride,
                               long head_stride, long top_at, int write_state, float* coef, float* top, int heads,
                               hipStream_t stream) {
    LEONE_REQUIRE(proj && i_bias && f_bias && spans && state && coef && top, "exp_gates: null pointer");
    LEONE_REQUIRE(known_vec(bias_dtype) && cap > 0.f, "exp_gates: unknown bias type or cap %g", cap);
    LEONE_REQUIRE(entries > 0 && heads > 0 && heads <= 65535 && i_off >= 0 && f_off >= 0 && stride >= i_off + heads &&
                  stride >= f_off + heads, "exp_gates: %d entries, %d heads, rows of %ld", entries, heads, stride);
    LEONE_REQUIRE(top_at >= 0 && top_at < head_stride && slot_stride >= heads * head_stride, "exp_gates: the maximum's place %ld", top_at);
    exp_gates_kernel<<<dim3(entries, heads), kScanThreads, 0, stream>>>(proj, stride, i_off, f_off, AnyVec{i_bias, bias_dtype},
                                                                 AnyVec{f_bias, bias_dtype}, cap, spans, state, slot_stride,
                                                                 head_stride, top_at, write_state, coef, top, heads);
    LEONE_LAUNCH_CHECK("exp_gates");
    return 0;
}

extern "C" int leone_outer_scan(const float* proj, long stride, int q_off, int k_off, int v_off, const float* coef,
                                const float* decay, int no_input, int accumulate, int norm_column, float q_scale,
                                float k_scale, const float* cos_table, const float* sin_table, int rotary_dim,
                                int table_positions, const int* positions, const int* segments, int n_segments,
                                const float* state_in, long in_stride, float* state_out, long out_stride, long head_stride,
                                float* decay_product, float* out, float* dot, int heads, int dim, int vdim,
                                hipStream_t stream) {
    LEONE_REQUIRE(proj && positions && segments && out, "outer_scan: null pointer");
    LEONE_REQUIRE(n_segments > 0 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0, "outer_scan: %d segments, %d heads of %d x %d",
                  n_segments, heads, dim, vdim);
    LEONE_REQUIRE(dim <= leone_scan_max_dim(), "outer_scan: heads of %d key channels, the kernel takes up to %d", dim, leone_scan_max_dim());
    LEONE_REQUIRE(coef || decay, "outer_scan: neither per-row coefficients nor a fixed decay");
    LEONE_REQUIRE(!norm_column || dot, "outer_scan: the normaliser's read-out needs a place");
    LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "outer_scan: cos and sin tables come together");
    LEONE_REQUIRE(!cos_table || (rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= dim && table_positions > 0),
                  "outer_scan: rotary_dim %d must be even, positive and at most %d", rotary_dim, dim);
    const long per_head = static_cast<long>(dim) * vdim + (norm_column ? dim : 0);
    LEONE_REQUIRE(head_stride >= per_head && (!state_in || in_stride >= heads * head_stride) &&
                  (!state_out || out_stride >= heads * head_stride), "outer_scan: states of %ld floats a head do not fit", head_stride);
    LEONE_REQUIRE(stride >= q_off + heads * dim && stride >= k_off + heads * dim && stride >= v_off + heads * vdim &&
                  q_off >= 0 && k_off >= 0 && v_off >= 0, "outer_scan: the projection's rows of %ld do not hold the named columns", stride);
    OuterScanArgs a{proj, stride, q_off, k_off, v_off, coef, decay, no_input, accumulate, norm_column, q_scale, k_scale,
                    cos_table, sin_table, cos_table ? rotary_dim / 2 : 0, cos_table ? table_positions : 1, positions,
                    reinterpret_cast<const Segment*>(segments), state_in, in_stride, state_out, out_stride, head_stride,
                    decay_product, out, dot, heads, dim, vdim};
    const int groups = lane_groups(dim);
    const int per_block = (kScanThreads / kWave) * (kWave / groups) * kLaneCols;          // columns a workgroup
    const dim3 grid(n_segments, heads, ceil_div(vdim + (norm_column ? 1 : 0), per_block));
    const size_t shared = (2 * kScanTokens * groups * kLaneRows + 2 * kScanTokens) * sizeof(float);
    outer_scan_kernel<<<grid, kScanThreads, shared, stream>>>(a, groups);
    LEONE_LAUNCH_CHECK("outer_scan");
    return 0;
}

extern "C" int leone_outer_chain(const int* links, int n_links, float* work, long work_stride, const float* product,
                                 float* state, long slot_stride, long head_stride, int per_head, int heads, int write_state,
                                 hipStream_t stream) {
    LEONE_REQUIRE(links && work && product && state && n_links > 0 && heads > 0 && heads <= 65535 && per_head > 0,
                  "outer_chain: null pointer or empty sizes");
    LEONE_REQUIRE(head_stride >= per_head && work_stride >= heads * head_stride && slot_stride >= heads * head_stride &&
                  ceil_div(per_head, 256) <= 65535, "outer_chain: states of %ld floats a head do not fit", head_stride);
    outer_chain_kernel<<<dim3(n_links, heads, ceil_div(per_head, 256)), 256, 0, stream>>>(
        links, work, work_stride, product, state, slot_stride, head_stride, per_head, heads, write_state);
    LEONE_LAUNCH_CHECK("outer_chain");
    return 0;
}

extern "C" int leone_delta_scan(const float* qkv, long stride, int q_off, int k_off, int v_off, const float* beta,
                                long beta_stride, const float* step, long step_stride, const void* rate_log,
                                const void* step_bias, int vec_dtype, float q_scale, float unit_eps, int no_input,
                                int accumulate, const int* segments, int n_segments, const float* state_in, long in_stride,
                                float* state_out, long out_stride, float* transition, float* out, int heads, int kv_heads,
                                int dim, int vdim, hipStream_t stream) {
    LEONE_REQUIRE(qkv && beta && step && rate_log && step_bias && segments && out, "delta_scan: null pointer");
    LEONE_REQUIRE(known_vec(vec_dtype), "delta_scan: unknown element type");
    LEONE_REQUIRE(n_segments > 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0,
                  "delta_scan: %d segments, %d heads over %d key heads of %d x %d", n_segments, heads, kv_heads, dim, vdim);
    LEONE_REQUIRE(dim <= leone_scan_max_dim(), "delta_scan: heads of %d key channels, the kernel takes up to %d", dim, leone_scan_max_dim());
    const long per_slot = static_cast<long>(heads) * dim * vdim;
    LEONE_REQUIRE((!state_in || in_stride >= per_slot) && (!state_out || out_stride >= per_slot),
                  "delta_scan: states of %ld floats do not fit", per_slot);
    LEONE_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && stride >= q_off + kv_heads * dim && stride >= k_off + kv_heads * dim &&
                  stride >= v_off + heads * vdim && beta_stride >= heads && step_stride >= static_cast<long>(heads) * dim,
                  "delta_scan: rows too short for the named columns");
    DeltaScanArgs a{qkv, stride, q_off, k_off, v_off, beta, beta_stride, step, step_stride, AnyVec{rate_log, vec_dtype},
                    AnyVec{step_bias, vec_dtype}, q_scale, unit_eps, no_input, accumulate,
                    reinterpret_cast<const Segment*>(segments), state_in, in_stride, state_out, out_stride, transition, out,
                    heads, kv_heads, dim, vdim};
    const int groups = lane_groups(dim);
    const dim3 grid(n_segments, heads, ceil_div(vdim + (transition ? dim : 0), (kScanThreads / kWave) * (kWave / groups)));
    const size_t shared = (3 * kScanTokens * groups * kLaneRows + kScanTokens) * sizeof(float);
    delta_scan_kernel<<<grid, kScanThreads, shared, stream>>>(a, groups);
    LEONE_LAUNCH_CHECK("delta_scan");
    return 0;
}

extern "C" int leone_delta_chain(const int* links, int n_links, float* work, long work_stride, const float* transition,
                                 float* state, long slot_stride, int heads, int dim, int vdim, int write_state,
                                 hipStream_t stream) {
    LEONE_REQUIRE(links && work && transition && state && n_links > 0 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0,
                  "delta_chain: null pointer or empty sizes");
    LEONE_REQUIRE(dim <= leone_scan_max_dim(), "delta_chain: heads of %d key channels, the kernel takes up to %d", dim, leone_scan_max_dim());
    const long per_slot = static_cast<long>(heads) * dim * vdim;
    LEONE_REQUIRE(work_stride >= per_slot && slot_stride >= per_slot, "delta_chain: states of %ld floats do not fit", per_slot);
    const int groups = lane_groups(dim);
    const int per_block = (kScanThreads / kWave) * (kWave / groups);
    const int dkp = groups * kLaneRows;
    const int tile = 8192 / dkp;                                   // 32 KB of the transition at a time
    const size_t shared = static_cast<size_t>(dkp) * (per_block + tile) * sizeof(float);
    delta_chain_kernel<<<dim3(n_links, heads, ceil_div(vdim, per_block)), kScanThreads, shared, stream>>>(
        links, work, work_stride, transition, state, slot_stride, heads, dim, vdim, groups, tile, write_state);
    LEONE_LAUNCH_CHECK("delta_chain");
    return 0;
}
