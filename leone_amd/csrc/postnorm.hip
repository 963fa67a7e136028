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
template <typename TY>
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
        for (int c = threadIdx.x; c < hidden; c += kPostThreads) {
            float d = dr[c];
            for (int p = 1; p < planes; ++p) d += dr[p * plane + c];      // planes of a product cut along K, in order
            row[c] = d;
            ss = fmaf(d, d, ss);
        }
        inv = 1.0f / sqrtf(block_sum<kPostThreads>(ss, scratch) / static_cast<float>(hidden) + eps);
    }
    float ss2 = 0.f;
    for (int c = threadIdx.x; c < hidden; c += kPostThreads) {
        float v = xr[c];
        if (delta != nullptr) {
            v += (row[c] * inv) * load_any(gain, c);
            if (!rows) xr[c] = v;
        }
        if (gain2.ptr != nullptr) {
            row[c] = v;
            ss2 = fmaf(v, v, ss2);
        } else if (y != nullptr) {
            y[static_cast<long>(out_row) * hidden + c] = from_float<TY>(v);
        }
    }
    if (gain2.ptr == nullptr) return;
    const float inv2 = 1.0f / sqrtf(block_sum<kPostThreads>(ss2, scratch) / static_cast<float>(hidden) + eps2);
    for (int c = threadIdx.x; c < hidden; c += kPostThreads)
        y[static_cast<long>(out_row) * hidden + c] = from_float<TY>((row[c] * inv2) * load_any(gain2, c));
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
    if (y_dtype == kBF16 && y)
        add_normed_kernel<bf16_t><<<n_rows, kPostThreads, shared, stream>>>(x, delta, delta_planes, delta_plane, g1, eps,
                                                                           static_cast<bf16_t*>(y), g2, eps2, rows, hidden);
    else
        add_normed_kernel<float><<<n_rows, kPostThreads, shared, stream>>>(x, delta, delta_planes, delta_plane, g1, eps,
                                                                          static_cast<float*>(y), g2, eps2, rows, hidden);
    LEONE_LAUNCH_CHECK("add_normed");
    return 0;
}
