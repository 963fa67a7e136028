// A norm on what a sublayer hands back, folded into the residual sum.
//
// A block whose norms stand behind its sublayers (x <- x + norm(sublayer(x)), the sublayer reading x itself)
// needs, between two sublayers, the RMS norm of the sublayer's result, the sum into the float32 stream and
// the stream's rows in the type the next product reads.  One launch does all three; for the model's last rows
// it also does the norm that stands before the output head.  Sums of squares, the scaling and the residual
// sum are float whatever the type that is written.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kPostThreads = 256;

// One workgroup a row.  `row` (dynamic shared memory, `hidden` floats) holds the summed planes of the delta,
// then the new row of the stream.
//   x[r] += (delta[r] / sqrt(mean(delta[r]^2) + eps)) * gain          (delta == nullptr: nothing is added)
//   gain2 == nullptr:  y[r] = x[r] in TY                               (y == nullptr: nothing is written)
//   gain2 != nullptr:  y[i] = (x[r] / sqrt(mean(x[r]^2) + eps2)) * gain2, r = rows ? rows[i] : i
// With `rows` the stream itself is left as it was (only some rows are looked at).
// kVec: elements a thread takes at a time (4 where the row's length and the addresses allow whole 16-byte runs).
template <int kVec>
__device__ inline void load_run(const float* p, float out[kVec]) {
    if constexpr (kVec == 4) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    } else {
        out[0] = p[0];
    }
}
template <int kVec>
__device__ inline void store_run(float* p, const float v[kVec]) {
    if constexpr (kVec == 4) *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
    else p[0] = v[0];
}
template <int kVec>
__device__ inline void store_run(bf16_t* p, const float v[kVec]) {
    if constexpr (kVec == 4) {
        uint2 packed;
        packed.x = bf16_bits_from_float(v[0]) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
        packed.y = bf16_bits_from_float(v[2]) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
        *reinterpret_cast<uint2*>(p) = packed;
    } else {
        p[0] = from_float<bf16_t>(v[0]);
    }
}

template <typename TY, int kVec>
__global__ void __launch_bounds__(kPostThreads)
add_normed_kernel(float* __restrict__ x, const float* __restrict__ delta, int planes, long plane, AnyVec gain, float eps,
                  TY* __restrict__ y, AnyVec gain2, float eps2, const int* __restrict__ rows, int hidden) {
    extern __shared__ float row[];
    __shared__ float scratch[kPostThreads / kWave];
    const int out_row = blockIdx.x;
    const long in_row = rows ? rows[out_row] : out_row;
    float* xr = x + in_row * hidden;
    float inv = 0.f;
    if (delta != nullptr) {
        const float* dr = delta + in_row * hidden;
        float ss = 0.f;
        for (int c = kVec * threadIdx.x; c < hidden; c += kVec * kPostThreads) {
            float d[kVec];
            load_run<kVec>(dr + c, d);
            for (int p = 1; p < planes; ++p) {                 // planes of a product cut along K, in order
                float more[kVec];
                load_run<kVec>(dr + p * plane + c, more);
#pragma unroll
                for (int i = 0; i < kVec; ++i) d[i] += more[i];
            }
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                row[c + i] = d[i];
                ss = fmaf(d[i], d[i], ss);
            }
        }
        inv = 1.0f / sqrtf(block_sum<kPostThreads>(ss, scratch) / static_cast<float>(hidden) + eps);
    }
    float ss2 = 0.f;
    for (int c = kVec * threadIdx.x; c < hidden; c += kVec * kPostThreads) {
        float v[kVec];
        load_run<kVec>(xr + c, v);
        if (delta != nullptr) {
#pragma unroll
            for (int i = 0; i < kVec; ++i) v[i] += (row[c + i] * inv) * load_any(gain, c + i);
            if (!rows) store_run<kVec>(xr + c, v);
        }
        if (gain2.ptr != nullptr) {
#pragma unroll
            for (int i = 0; i < kVec; ++i) {
                row[c + i] = v[i];
                ss2 = fmaf(v[i], v[i], ss2);
            }
        } else if (y != nullptr) {
            store_run<kVec>(y + static_cast<long>(out_row) * hidden + c, v);
        }
    }
    if (gain2.ptr == nullptr) return;
    const float inv2 = 1.0f / sqrtf(block_sum<kPostThreads>(ss2, scratch) / static_cast<float>(hidden) + eps2);
    for (int c = kVec * threadIdx.x; c < hidden; c += kVec * kPostThreads) {
        float v[kVec];
#pragma unroll
        for (int i = 0; i < kVec; ++i) v[i] = (row[c + i] * inv2) * load_any(gain2, c + i);
        store_run<kVec>(y + static_cast<long>(out_row) * hidden + c, v);
    }
}

}  // namespace leone

using namespace leone;

extern "C" int leone_add_normed(float* x, const float* delta, int delta_planes, long delta_plane, const void* gain,
                                int gain_dtype, float eps, void* y, int y_dtype, const void* gain2, int gain2_dtype,
                                float eps2, const int* rows, int n_rows, int hidden, hipStream_t stream) {
    LEONE_REQUIRE(x, "add_normed: null pointer");
    LEONE_REQUIRE(n_rows > 0 && hidden > 0 && hidden <= 12288, "add_normed: rows %d, hidden %d (at most 12288)", n_rows, hidden);
    LEONE_REQUIRE(!delta || (gain && eps > 0.f && eps == eps && (gain_dtype == kF32 || gain_dtype == kBF16)),
                  "add_normed: a delta needs its norm's gain and a positive eps");
    LEONE_REQUIRE(!delta || (delta_planes >= 1 && delta_planes <= 64 && (delta_planes == 1 || delta_plane >= static_cast<long>(n_rows) * hidden)),
                  "add_normed: %d planes of what is to be added", delta_planes);
    LEONE_REQUIRE(!gain2 || (y && eps2 > 0.f && eps2 == eps2 && (gain2_dtype == kF32 || gain2_dtype == kBF16)),
                  "add_normed: the second norm needs an output, a gain and a positive eps");
    LEONE_REQUIRE(!y || y_dtype == kF32 || y_dtype == kBF16, "add_normed: unknown output type %d", y_dtype);
    LEONE_REQUIRE(!rows || gain2, "add_normed: picked rows come with the second norm");
    LEONE_REQUIRE(delta || y, "add_normed: nothing to do");
    const AnyVec g1{gain, gain_dtype}, g2{gain2, gain2_dtype};
    const size_t shared = static_cast<size_t>(hidden) * sizeof(float);
    // whole 16-byte runs where the row's length, the planes' distance and every address allow them
    const bool runs = hidden % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                      (!delta || (reinterpret_cast<uintptr_t>(delta) % 16 == 0 && (delta_planes == 1 || delta_plane % 4 == 0))) &&
                      (!y || reinterpret_cast<uintptr_t>(y) % 16 == 0);
#define LEONE_ADD_NORMED(TY, V)                                                                                        \
    add_normed_kernel<TY, V><<<n_rows, kPostThreads, shared, stream>>>(x, delta, delta_planes, delta_plane, g1, eps,  \
                                                                       static_cast<TY*>(y), g2, eps2, rows, hidden)
    if (y_dtype == kBF16 && y) {
        if (runs) LEONE_ADD_NORMED(bf16_t, 4);
        else LEONE_ADD_NORMED(bf16_t, 1);
    } else {
        if (runs) LEONE_ADD_NORMED(float, 4);
        else LEONE_ADD_NORMED(float, 1);
    }
#undef LEONE_ADD_NORMED
    LEONE_LAUNCH_CHECK("add_normed");
    return 0;
}
