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

    // sum_j w[c][j] * input(pos - taps + 1 + j); the last tap multiplies the current input `cur`
    template <typename T>
    __device__ __forceinline__ float conv(const T *h, int64_t h_stride, const float *w, int c, float cur) const {
        const float *wc = w + static_cast<int64_t>(c) * taps;
        float a = 0.f;
        for (int k = taps - 1; k >= 1; --k) a += wc[taps - 1 - k] * at(h, h_stride, c, pos - k);
        return a + wc[taps - 1] * cur;
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
};

} // namespace swl
