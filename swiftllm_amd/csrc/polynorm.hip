// polynorm.hip — row-wise feed-forward activations whose statistics span the whole row.
//
// PolyNorm: out = a * N(z) + b * N(z^2) + c * N(z^3) + e, powers taken element by element, N(v) = v / sqrt(mean(v^2) + eps)
// over the row's ff values. The three mean squares (of z, z^2, z^3) are accumulated in fp32 in one pass over the row.
//
// Clamped gated unit (mixture-of-experts experts): g = min(gate, limit), u = clamp(up, -limit, limit),
// y = g * sigmoid(1.702 g) * (u + 1).
#include "swl_common.h"

namespace swl {

constexpr int kPnThreads = 256;

template <typename T>
__global__ __launch_bounds__(kPnThreads) void polynorm_kernel(T *out, const T *z, float a, float b, float c, float e,
                                                              float eps, int ff) {
    __shared__ float red[3][kPnThreads / 64];
    const int64_t r = blockIdx.x;
    const T *zr = z + r * ff;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    // 16-bit rows whose length is a multiple of 8 move 16 bytes per lane
    bool wide = false;
    if constexpr (sizeof(T) == 2) wide = (ff & 7) == 0 && ((reinterpret_cast<uintptr_t>(z) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if constexpr (sizeof(T) == 2) {
        if (wide) {
            for (int i = threadIdx.x * 8; i < ff; i += kPnThreads * 8) {
                const vec8_t<T> zv = load8(zr + i);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float v = to_f(zv[j]);
                    const float v2 = v * v, v3 = v2 * v;
                    s1 += v2;
                    s2 += v2 * v2;
                    s3 += v3 * v3;
                }
            }
        }
    }
    if (!wide) {
        for (int i = threadIdx.x; i < ff; i += kPnThreads) {
            const float v = to_f(zr[i]);
            const float v2 = v * v, v3 = v2 * v;
            s1 += v2;
            s2 += v2 * v2;
            s3 += v3 * v3;
        }
    }
    s1 = wave_allreduce_sum(s1);
    s2 = wave_allreduce_sum(s2);
    s3 = wave_allreduce_sum(s3);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) {
        red[0][wave] = s1;
        red[1][wave] = s2;
        red[2][wave] = s3;
    }
    __syncthreads();
    s1 = s2 = s3 = 0.f;
#pragma unroll
    for (int w = 0; w < kPnThreads / 64; ++w) {
        s1 += red[0][w];
        s2 += red[1][w];
        s3 += red[2][w];
    }
    const float n = static_cast<float>(ff);
    const float r1 = a / sqrtf(s1 / n + eps), r2 = b / sqrtf(s2 / n + eps), r3 = c / sqrtf(s3 / n + eps);
    T *orow = out + r * ff;
    if constexpr (sizeof(T) == 2) {
        if (wide) {
            for (int i = threadIdx.x * 8; i < ff; i += kPnThreads * 8) {
                const vec8_t<T> zv = load8(zr + i);
                vec8_t<T> ov;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float v = to_f(zv[j]);
                    const float v2 = v * v;
                    ov[j] = to_t<T>(r1 * v + r2 * v2 + r3 * (v2 * v) + e);
                }
                store8(orow + i, ov);
            }
            return;
        }
    }
    for (int i = threadIdx.x; i < ff; i += kPnThreads) {
        const float v = to_f(zr[i]);
        const float v2 = v * v;
        orow[i] = to_t<T>(r1 * v + r2 * v2 + r3 * (v2 * v) + e);
    }
}

} // namespace swl

extern "C" int swl_polynorm(void *out, const void *z, float a, float b, float c, float e, float eps, int64_t num_rows,
                            int32_t ff, int32_t dtype, swl_stream_t stream) {
    if (num_rows < 0 || ff <= 0) return SWL_ERR_BAD_ARG;
    if (num_rows == 0) return SWL_OK;
    if (!out || !z) return SWL_ERR_BAD_ARG;
    if (num_rows > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::polynorm_kernel<T>), dim3(static_cast<unsigned>(num_rows)), dim3(swl::kPnThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(out), static_cast<const T *>(z), a, b, c, e,
                           eps, ff);
    });
    return swl::check_launch();
}
