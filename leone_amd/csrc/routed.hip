// A feed-forward of routed experts: the router's choice, the rows sorted by expert, the experts' products.
//
//   route_topk   scores s = softmax(z) over all router outputs (float); choice scores s + correction; experts in
//                equal groups of neighbours, a group's score its best choice score, only the best `keep` groups
//                stay open (the others count as minus infinity); the `top` best open choice scores win; the
//                weights are the winners' s over their sum (+ 1e-20).
//   moe_plan     the (row, place) pairs of every expert gathered into tiles of kTilePairs pairs of one expert.
//   moe_up       act(W_gate h) * (W_up h) of every pair, by its expert's matrices.
//   moe_down     W_down of that, times the pair's weight, float.
//   moe_combine  a row's pairs summed in the order of its places; a router output beyond the experts with
//                matrices hands the row itself on (times its weight); a delta that comes along is added.
//
// Every grid is fixed by the step's row count alone (tiles that turn out unused end at once), so a step that is
// recorded once can be replayed with other choices.  Products accumulate in float from operands of the engine's
// type; the router, its softmax and the weights are float.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kRouteSlots = 8;                 // router outputs a lane holds: up to 512 experts
constexpr int kTilePairs = 8;                  // pairs of one expert a workgroup of the products takes
constexpr int kMoeThreads = 256;
constexpr int kMoeWaves = kMoeThreads / kWave;
constexpr int kColsPerWave = 4;
constexpr int kMoeCols = kMoeWaves * kColsPerWave;

// The better of two (value, index): the larger value, the lower index among equals.
__device__ inline void wave_best(float& v, int& at) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float v2 = __shfl_xor(v, off, kWave);
        const int at2 = __shfl_xor(at, off, kWave);
        if (v2 > v || (v2 == v && at2 < at)) {
            v = v2;
            at = at2;
        }
    }
}

// One wave a row.
__global__ void __launch_bounds__(kWave)
route_topk_kernel(const float* __restrict__ logits, AnyVec correction, int* __restrict__ chosen, float* __restrict__ weight,
                  int total, int top, int group_count, int group_keep) {
    const int row = blockIdx.x;
    const int lane = threadIdx.x;
    const float* z = logits + static_cast<long>(row) * total;
    float s[kRouteSlots], choice[kRouteSlots];
    bool taken[kRouteSlots];
    float top_z = -INFINITY;
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i) {
        const int e = lane + i * kWave;
        s[i] = e < total ? z[e] : -INFINITY;
        top_z = fmaxf(top_z, s[i]);
    }
    top_z = wave_max(top_z);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i) {
        const int e = lane + i * kWave;
        s[i] = e < total ? expf(s[i] - top_z) : 0.f;
        sum += s[i];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < kRouteSlots; ++i) {
        const int e = lane + i * kWave;
        s[i] = s[i] / sum;
        choice[i] = e < total ? s[i] + (correction.ptr ? load_any(correction, e) : 0.f) : -INFINITY;
        taken[i] = e >= total;
    }
    if (group_count > 1) {
        // a group's score; lane g keeps group g's (group_count <= 64)
        const int size = total / group_count;
        float mine = -INFINITY;
        for (int g = 0; g < group_count; ++g) {
            float best = -INFINITY;
#pragma unroll
            for (int i = 0; i < kRouteSlots; ++i) {
                const int e = lane + i * kWave;
                if (e < total && e / size == g) best = fmaxf(best, choice[i]);
            }
            best = wave_max(best);
            if (lane == g) mine = best;
        }
        unsigned long long open = 0ull;
        bool mine_taken = lane >= group_count;
        for (int n = 0; n < group_keep; ++n) {
            float v = mine_taken ? -INFINITY : mine;
            int at = mine_taken ? 0x7fffffff : lane;
            wave_best(v, at);
            if (at == 0x7fffffff) break;
            open |= 1ull << at;
            if (lane == at) mine_taken = true;
        }
#pragma unroll
        for (int i = 0; i < kRouteSlots; ++i) {
            const int e = lane + i * kWave;
            if (e < total && !((open >> (e / size)) & 1ull)) choice[i] = -INFINITY;
        }
    }
    float picked_sum = 0.f;
    float my_s = 0.f;
    int my_e = 0;
    for (int n = 0; n < top; ++n) {
        float v = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < kRouteSlots; ++i) {
            const int e = lane + i * kWave;
            if (!taken[i] && (at == 0x7fffffff || choice[i] > v)) {
                v = choice[i];
                at = e;
            }
        }
        wave_best(v, at);
        float got = 0.f;
#pragma unroll
        for (int i = 0; i < kRouteSlots; ++i) {
            const int e = lane + i * kWave;
            if (e == at) {
                taken[i] = true;
                got = s[i];
            }
        }
        got = wave_sum(got);               // one lane held it
        picked_sum += got;
        if (lane == n % kWave && n < kWave) {
            my_s = got;
            my_e = at;
        }
        if (n >= kWave && lane == 0) {       // more than 64 places: written as they come, scaled below
            chosen[static_cast<long>(row) * top + n] = at;
            weight[static_cast<long>(row) * top + n] = got;
        }
    }
    const float denom = picked_sum + 1e-20f;
    if (lane < top && lane < kWave) {
        chosen[static_cast<long>(row) * top + lane] = my_e;
        weight[static_cast<long>(row) * top + lane] = my_s / denom;
    }
    if (top > kWave && lane == 0)
        for (int n = kWave; n < top; ++n) weight[static_cast<long>(row) * top + n] /= denom;
}

// One workgroup.  counts and places live in shared memory (experts <= 1024).
__global__ void __launch_bounds__(1024)
moe_plan_kernel(const int* __restrict__ chosen, int pairs, int experts, int* __restrict__ tile_expert,
                int* __restrict__ tile_pairs, int max_tiles) {
    __shared__ int count[1024];
    __shared__ int first_tile[1024];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
    for (int t = threadIdx.x; t < max_tiles; t += blockDim.x) tile_expert[t] = -1;
    for (long i = threadIdx.x; i < static_cast<long>(max_tiles) * kTilePairs; i += blockDim.x) tile_pairs[i] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            first_tile[e] = at;
            const int tiles = (count[e] + kTilePairs - 1) / kTilePairs;
            for (int t = 0; t < tiles && at + t < max_tiles; ++t) tile_expert[at + t] = e;
            at += tiles;
            count[e] = 0;
        }
    }
    __syncthreads();
    // Which place of its expert's tiles a pair gets does not matter to its result: every pair is worked out by itself.
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < experts) {
            const int at = atomicAdd(&count[e], 1);
            const long place = static_cast<long>(first_tile[e]) * kTilePairs + at;
            if (place < static_cast<long>(max_tiles) * kTilePairs) tile_pairs[place] = p;
        }
    }
}

template <typename T>
__device__ inline void load8f(const T* __restrict__ p, int k, int limit, bool runs, float out[8]);

template <>
__device__ inline void load8f<float>(const float* __restrict__ p, int k, int limit, bool runs, float out[8]) {
    if (runs && k + 8 <= limit) {
        const float4 a = *reinterpret_cast<const float4*>(p + k);
        const float4 b = *reinterpret_cast<const float4*>(p + k + 4);
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
        return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = k + i < limit ? p[k + i] : 0.f;
}

template <>
__device__ inline void load8f<bf16_t>(const bf16_t* __restrict__ p, int k, int limit, bool runs, float out[8]) {
    if (runs && k + 8 <= limit) {
        const uint4 t = *reinterpret_cast<const uint4*>(p + k);
        const unsigned w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = k + i < limit ? to_float(p[k + i]) : 0.f;
}

// A tile's pairs against kMoeCols rows of its expert's matrices: a wave takes kColsPerWave rows, its lanes runs of
// eight elements of the inner size; sums over the lanes at the end.
//   kGated: w = [experts][2][n][k] (gate rows, then up rows), y[pair][col] = act(gate) * up in T
//   else:   w = [experts][n][k], y[pair][col] = weight[pair] * product in float
// x: kGated: row pair / top of [rows][k]; else row pair of [pairs][k].
template <typename T, bool kGated>
__global__ void __launch_bounds__(kMoeThreads)
moe_product_kernel(const T* __restrict__ x, const T* __restrict__ w, void* __restrict__ y, const float* __restrict__ pair_weight,
                   const int* __restrict__ tile_expert, const int* __restrict__ tile_pairs, int top, int n, int k, int act,
                   int runs) {
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int col0 = blockIdx.y * kMoeCols + wave * kColsPerWave;
    if (col0 >= n) return;
    int pair[kTilePairs];
#pragma unroll
    for (int p = 0; p < kTilePairs; ++p) pair[p] = tile_pairs[static_cast<long>(tile) * kTilePairs + p];
    float acc[kColsPerWave][kTilePairs], acc2[kGated ? kColsPerWave : 1][kTilePairs];
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c)
#pragma unroll
        for (int p = 0; p < kTilePairs; ++p) {
            acc[c][p] = 0.f;
            if constexpr (kGated) acc2[c][p] = 0.f;
        }
    const long matrix = static_cast<long>(n) * k;
    const T* w_first = w + static_cast<long>(e) * (kGated ? 2 : 1) * matrix;
    for (int at = 8 * lane; at < k; at += 8 * kWave) {
        float xv[kTilePairs][8];
#pragma unroll
        for (int p = 0; p < kTilePairs; ++p) {
            if (pair[p] >= 0) {
                load8f<T>(x + static_cast<long>(kGated ? pair[p] / top : pair[p]) * k, at, k, runs != 0, xv[p]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) xv[p][i] = 0.f;
            }
        }
#pragma unroll
        for (int c = 0; c < kColsPerWave; ++c) {
            const int col = col0 + c;
            if (col >= n) continue;
            float wv[8], wv2[8];
            load8f<T>(w_first + static_cast<long>(col) * k, at, k, runs != 0, wv);
            if constexpr (kGated) load8f<T>(w_first + matrix + static_cast<long>(col) * k, at, k, runs != 0, wv2);
#pragma unroll
            for (int p = 0; p < kTilePairs; ++p)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    acc[c][p] = fmaf(wv[i], xv[p][i], acc[c][p]);
                    if constexpr (kGated) acc2[c][p] = fmaf(wv2[i], xv[p][i], acc2[c][p]);
                }
        }
    }
    // lane c * kTilePairs + p writes (column c, pair p)
    float mine = 0.f, mine2 = 0.f;
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c)
#pragma unroll
        for (int p = 0; p < kTilePairs; ++p) {
            const float total = wave_sum(acc[c][p]);
            float total2 = 0.f;
            if constexpr (kGated) total2 = wave_sum(acc2[c][p]);
            if (lane == c * kTilePairs + p) {
                mine = total;
                mine2 = total2;
            }
        }
    if (lane < kColsPerWave * kTilePairs) {
        const int c = lane / kTilePairs, p = lane % kTilePairs;
        const int col = col0 + c;
        // the pair of this lane, without indexing the register array by a lane's value
        int which = -1;
#pragma unroll
        for (int q = 0; q < kTilePairs; ++q)
            if (q == p) which = pair[q];
        if (col < n && which >= 0) {
            if constexpr (kGated)
                static_cast<T*>(y)[static_cast<long>(which) * n + col] = from_float<T>(gate_act(mine, act) * mine2);
            else
                static_cast<float*>(y)[static_cast<long>(which) * n + col] = mine * pair_weight[which];
        }
    }
}

// One workgroup a row.
template <typename T>
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ pair_out, const int* __restrict__ chosen, const float* __restrict__ weight,
                   const T* __restrict__ x, const float* __restrict__ extra, float* __restrict__ out, int top, int experts,
                   int hidden) {
    const int row = blockIdx.x;
    const int* ch = chosen + static_cast<long>(row) * top;
    const float* wt = weight + static_cast<long>(row) * top;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
        float sum = 0.f;
        for (int j = 0; j < top; ++j) {
            const int e = ch[j];
            if (e >= experts)
                sum += wt[j] * to_float(x[static_cast<long>(row) * hidden + c]);    // hands the row on as it came
            else if (e >= 0)
                sum += pair_out[(static_cast<long>(row) * top + j) * hidden + c];
        }
        if (extra != nullptr) sum += extra[static_cast<long>(row) * hidden + c];
        out[static_cast<long>(row) * hidden + c] = sum;
    }
}

}  // namespace leone

using namespace leone;

extern "C" int leone_moe_tile_pairs() { return kTilePairs; }
extern "C" int leone_route_max_outputs() { return kRouteSlots * kWave; }

extern "C" int leone_route_topk(const float* logits, const void* correction, int correction_dtype, int* chosen, float* weight,
                                int rows, int total, int top, int group_count, int group_keep, hipStream_t stream) {
    LEONE_REQUIRE(logits && chosen && weight, "route_topk: null pointer");
    LEONE_REQUIRE(rows > 0 && total > 0 && total <= kRouteSlots * kWave, "route_topk: rows %d, %d router outputs (at most %d)",
                  rows, total, kRouteSlots * kWave);
    LEONE_REQUIRE(top > 0 && top <= total, "route_topk: %d of %d outputs", top, total);
    LEONE_REQUIRE(!correction || correction_dtype == kF32 || correction_dtype == kBF16, "route_topk: unknown type of the correction");
    LEONE_REQUIRE(group_count >= 1 && group_count <= kWave && total % group_count == 0 && group_keep >= 1 && group_keep <= group_count,
                  "route_topk: %d groups (at most %d, dividing %d outputs), %d kept", group_count, kWave, total, group_keep);
    route_topk_kernel<<<rows, kWave, 0, stream>>>(logits, AnyVec{correction, correction_dtype}, chosen, weight, total, top,
                                                  group_count, group_keep);
    LEONE_LAUNCH_CHECK("route_topk");
    return 0;
}

extern "C" int leone_moe_plan(const int* chosen, int pairs, int experts, int* tile_expert, int* tile_pairs, int max_tiles,
                              hipStream_t stream) {
    LEONE_REQUIRE(chosen && tile_expert && tile_pairs, "moe_plan: null pointer");
    LEONE_REQUIRE(pairs > 0 && experts > 0 && experts <= 1024, "moe_plan: %d pairs, %d experts (at most 1024)", pairs, experts);
    const long needed = static_cast<long>(pairs) / kTilePairs + experts;
    LEONE_REQUIRE(max_tiles >= (needed < pairs ? needed : pairs), "moe_plan: %d tiles cannot hold %d pairs of %d experts", max_tiles,
                  pairs, experts);
    moe_plan_kernel<<<1, 1024, 0, stream>>>(chosen, pairs, experts, tile_expert, tile_pairs, max_tiles);
    LEONE_LAUNCH_CHECK("moe_plan");
    return 0;
}

// gated != 0: x [rows, k], w [experts, 2, n, k], y [pairs, n] of dtype = act(gate) * up (act: GateAct).
// gated == 0: x [pairs, k], w [experts, n, k], y float32 [pairs, n] = pair_weight[pair] * product.
extern "C" int leone_moe_product(const void* x, const void* w, void* y, const float* pair_weight, int dtype, int gated,
                                 const int* tile_expert, const int* tile_pairs, int max_tiles, int top, int n, int k, int act,
                                 hipStream_t stream) {
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_product: unknown element type %d", dtype);
    LEONE_REQUIRE(x && w && y && tile_expert && tile_pairs && (gated || pair_weight), "moe_product: null pointer");
    LEONE_REQUIRE(max_tiles > 0 && top > 0 && n > 0 && k > 0, "moe_product: %d tiles, sizes %d x %d", max_tiles, n, k);
    LEONE_REQUIRE(act == kGateSilu || act == kGateGeluTanh, "moe_product: unknown activation %d", act);
    const uintptr_t run = 8 * (dtype == kF32 ? sizeof(float) : sizeof(bf16_t));
    const int runs = k % 8 == 0 && reinterpret_cast<uintptr_t>(x) % run == 0 && reinterpret_cast<uintptr_t>(w) % run == 0;
    const dim3 grid(max_tiles, ceil_div(n, kMoeCols));
    LEONE_REQUIRE(grid.y <= 65535, "moe_product: %d rows of a matrix are too many", n);
#define LEONE_MOE(T, G)                                                                                                   \
    moe_product_kernel<T, G><<<grid, kMoeThreads, 0, stream>>>(static_cast<const T*>(x), static_cast<const T*>(w), y, pair_weight, \
                                                               tile_expert, tile_pairs, top, n, k, act, runs)
    if (dtype == kF32) {
        if (gated) LEONE_MOE(float, true);
        else LEONE_MOE(float, false);
    } else {
        if (gated) LEONE_MOE(bf16_t, true);
        else LEONE_MOE(bf16_t, false);
    }
#undef LEONE_MOE
    LEONE_LAUNCH_CHECK("moe_product");
    return 0;
}

extern "C" int leone_moe_combine(const float* pair_out, const int* chosen, const float* weight, const void* x, int dtype,
                                 const float* extra, float* out, int rows, int top, int experts, int hidden, hipStream_t stream) {
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_combine: unknown element type %d", dtype);
    LEONE_REQUIRE(pair_out && chosen && weight && x && out, "moe_combine: null pointer");
    LEONE_REQUIRE(rows > 0 && top > 0 && experts >= 0 && hidden > 0, "moe_combine: rows %d, top %d, hidden %d", rows, top, hidden);
    if (dtype == kF32)
        moe_combine_kernel<float><<<rows, 256, 0, stream>>>(pair_out, chosen, weight, static_cast<const float*>(x), extra, out, top,
                                                            experts, hidden);
    else
        moe_combine_kernel<bf16_t><<<rows, 256, 0, stream>>>(pair_out, chosen, weight, static_cast<const bf16_t*>(x), extra, out, top,
                                                             experts, hidden);
    LEONE_LAUNCH_CHECK("moe_combine");
    return 0;
}
