// conv_tail.h — the carried inputs of a short causal convolution over time, shared by the kernels that convolve.
//
// A sequence's state slot keeps the last R = taps - 1 inputs of every channel, twice: buffer `parity` is what earlier steps
// left, the other buffer receives what this step leaves (written by the workgroup of the portion's last token). Entry r of a
// buffer holds the input at position (tokens consumed so far) - R + r; entries of positions before the sequence's start are
// never read (those inputs are zero by definition), so a slot needs no clearing when it changes hands.
#pragma once

#include "swl_common.h"

namespace swl {

struct ConvTail {
    const float *old_tail;
    float *new_tail;
    int64_t t;
    int R, C, taps, pos, start;
    bool last;

    __device__ ConvTail(float *state, int64_t slot_stride, int64_t tail_off, const int32_t *tok_pos,
                        const int32_t *tok_start, const int32_t *tok_state, const int32_t *tok_seq, int64_t num_tokens,
                        int channels, int taps_, int64_t token)
        : old_tail(nullptr), new_tail(nullptr), t(token), R(taps_ - 1), C(channels), taps(taps_) {
        pos = tok_pos[t];
        start = tok_start[t];
        last = (t + 1 == num_tokens) || tok_seq[t + 1] != tok_seq[t];
        if (R > 0) {
            const int code = tok_state[t];      // slot * 2 + parity
            float *base = state + static_cast<int64_t>(code >> 1) * slot_stride + tail_off;
            const int par = code & 1;
            old_tail = base + static_cast<int64_t>(par) * R * C;
            new_tail = base + static_cast<int64_t>(1 - par) * R * C;
        }
    }

    // input of channel c at position q < pos: zero before the sequence, a row of this step, or the carried tail
    template <typename T>
    __device__ __forceinline__ float at(const T *h, int64_t h_stride, int c, int q) const {
        if (q < 0) return 0.f;
        if (q >= start) return to_f(h[(t - (pos - q)) * h_stride + c]);
        return old_tail[static_cast<int64_t>(R - (start - q)) * C + c];
    }

    // sum_j w[j][c] * input(pos - taps + 1 + j); w is tap-major [taps, channels], the last tap multiplies the current input
    template <typename T>
    __device__ __forceinline__ float conv(const T *h, int64_t h_stride, const float *w, int c, float cur) const {
        float a = 0.f;
        for (int k = taps - 1; k >= 1; --k) a += w[static_cast<int64_t>(taps - 1 - k) * C + c] * at(h, h_stride, c, pos - k);
        return a + w[static_cast<int64_t>(taps - 1) * C + c] * cur;
    }

    // the portion's last token leaves the sequence's new tail (channel c)
    template <typename T>
    __device__ __forceinline__ void save(const T *h, int64_t h_stride, int c, float cur) const {
        if (!last || R == 0) return;
        for (int r = 0; r < R; ++r) {
            const int q = pos + 1 - R + r;
            if (q < 0) continue;
            new_tail[static_cast<int64_t>(r) * C + c] = q == pos ? cur : at(h, h_stride, c, q);
        }
    }

    // ---- the same for 8 consecutive channels of 16-bit rows (16-byte loads; c a multiple of 8, rows 16-byte aligned) ----
    template <typename T>
    __device__ __forceinline__ void at8(const T *h, int64_t h_stride, int c, int q, float (&v)[8]) const {
        if (q < 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = 0.f;
        } else if (q >= start) {
            const vec8_t<T> x = load8(h + (t - (pos - q)) * h_stride + c);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = to_f(x[j]);
        } else {
            const float *p = old_tail + static_cast<int64_t>(R - (start - q)) * C + c;
            const float4_t a = *reinterpret_cast<const float4_t *>(p), b = *reinterpret_cast<const float4_t *>(p + 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[j] = a[j];
                v[4 + j] = b[j];
            }
        }
    }

    // same sums in the same order as conv()
    template <typename T>
    __device__ __forceinline__ void conv8(const T *h, int64_t h_stride, const float *w, int c, const float (&cur)[8],
                                          float (&a)[8]) const {
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = 0.f;
        for (int k = taps - 1; k >= 1; --k) {
            float v[8];
            at8(h, h_stride, c, pos - k, v);
            const float *wk = w + static_cast<int64_t>(taps - 1 - k) * C + c;
            const float4_t w0 = *reinterpret_cast<const float4_t *>(wk), w1 = *reinterpret_cast<const float4_t *>(wk + 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                a[j] += w0[j] * v[j];
                a[4 + j] += w1[j] * v[4 + j];
            }
        }
        const float *wl = w + static_cast<int64_t>(taps - 1) * C + c;
        const float4_t w0 = *reinterpret_cast<const float4_t *>(wl), w1 = *reinterpret_cast<const float4_t *>(wl + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] += w0[j] * cur[j];
            a[4 + j] += w1[j] * cur[4 + j];
        }
    }

    template <typename T>
    __device__ __forceinline__ void save8(const T *h, int64_t h_stride, int c, const float (&cur)[8]) const {
        if (!last || R == 0) return;
        for (int r = 0; r < R; ++r) {
            const int q = pos + 1 - R + r;
            if (q < 0) continue;
            float v[8];
            if (q == pos) {
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = cur[j];
            } else {
                at8(h, h_stride, c, q, v);
            }
            float *p = new_tail + static_cast<int64_t>(r) * C + c;
            *reinterpret_cast<float4_t *>(p) = float4_t{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<float4_t *>(p + 4) = float4_t{v[4], v[5], v[6], v[7]};
        }
    }

    // whether the 8-channel forms may be used for rows of h (and a state region) laid out like this
    template <typename T>
    static __device__ __forceinline__ bool wide_ok(const T *h, int64_t h_stride, const float *w, const float *state,
                                                   int64_t slot_stride, int64_t tail_off, int channels) {
        if constexpr (sizeof(T) != 2) return false;
        return (channels & 7) == 0 && (h_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(h) & 15) == 0 &&
               (reinterpret_cast<uintptr_t>(w) & 15) == 0 && (reinterpret_cast<uintptr_t>(state) & 15) == 0 &&
               (slot_stride & 3) == 0 && (tail_off & 3) == 0;
    }
};

} // namespace swl
