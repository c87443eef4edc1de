// delta_rule.hip — the gated delta rule as a recurrent mixer, for any mixture of prompt portions and decoded tokens.
//
// Per head a state S [dim, vdim] (fp32, in the sequence's state slot) is carried from token to token:
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with unit vectors q (scaled by dim^-1/2) and k, beta in (0, 1) and a decay g in (0, 1).
//
//   swl_delta_prep:  one workgroup per token. The fused input projection row [q | k | v | gate | b | a] -> short causal
//                    convolution + SiLU on q, k, v (carried inputs: conv_tail.h), unit norms of the q / k heads,
//                    beta = sigmoid(b), g = exp(-exp(A_log) softplus(a + dt_bias)); everything after the loads is fp32.
//   swl_delta_rule:  one workgroup per (portion, head). The columns of S are independent recurrences, so a column belongs
//                    to L adjacent lanes, each holding dim / L of its elements in registers; per token the lanes exchange
//                    two partial dot products (S^T k, S^T q) through DPP and o = S^T q + u (k . q, from the prep) needs no second
//                    pass over the state. q, k, v, beta, g of 16 tokens at a time are staged in LDS. The token loop is
//                    sequential whatever the cut of the sequence into steps: the same operations in the same order. When
//                    a step has few (portion, head) pairs the columns of a head are shared out over several workgroups. A
//                    wave of loaders stages the next 16 tokens into a second LDS buffer while the others walk the current ones.
//   swl_gated_head_rmsnorm: out = o / rms(o over vdim) * w * silu(gate), per head.
#include "swl_common.h"
#include "conv_tail.h"

namespace swl {

constexpr int kDpThreads = 256;
constexpr int kDrChunk = 16;        // tokens staged at a time

__device__ __forceinline__ float dr_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <typename T>
__global__ __launch_bounds__(kDpThreads) void delta_prep_kernel(
    float *qn, float *kn, float *kq, float *vv, float *beta, float *decay, const T *proj, int64_t proj_stride,
    const float *conv_w, const float *a_log, const float *dt_bias, float *state, int64_t slot_stride, int64_t tail_off, const int32_t *tok_pos,
    const int32_t *tok_start, const int32_t *tok_state, const int32_t *tok_seq, int64_t num_tokens, int H, int G, int d,
    int dv, int taps) {
    extern __shared__ float act[];      // [2 G d + H dv] convolved, activated channels
    const int64_t t = blockIdx.x;
    const int qk = G * d, C = 2 * qk + H * dv;
    const T *row = proj + t * proj_stride;
    const ConvTail tail(state, slot_stride, tail_off, tok_pos, tok_start, tok_state, tok_seq, num_tokens, C, taps, t);
    bool wide = false;
    if constexpr (sizeof(T) == 2) wide = ConvTail::wide_ok(proj, proj_stride, conv_w, state, slot_stride, tail_off, C);
    if (wide) {
        if constexpr (sizeof(T) == 2) {
            for (int c = threadIdx.x * 8; c < C; c += kDpThreads * 8) {
                const vec8_t<T> x = load8(row + c);
                float cur[8], a[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) cur[j] = to_f(x[j]);
                tail.conv8(proj, proj_stride, conv_w, c, cur, a);
#pragma unroll
                for (int j = 0; j < 8; ++j) act[c + j] = a[j] * dr_sigmoid(a[j]);
                tail.save8(proj, proj_stride, c, cur);
            }
        }
    } else {
        for (int c = threadIdx.x; c < C; c += kDpThreads) {
            const float cur = to_f(row[c]);
            const float a = tail.conv(proj, proj_stride, conv_w, c, cur);
            act[c] = a * dr_sigmoid(a);
            tail.save(proj, proj_stride, c, cur);
        }
    }
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const float qscale = 1.0f / sqrtf(static_cast<float>(d));
    for (int g = wave; g < G; g += kDpThreads / 64) {       // q head g and k head g: unit norms and their dot product
        const float *qsrc = act + g * d, *ksrc = act + qk + g * d;
        float sq = 0.f, sk = 0.f, dot = 0.f;
        for (int e = lane; e < d; e += 64) {
            sq += qsrc[e] * qsrc[e];
            sk += ksrc[e] * ksrc[e];
            dot += qsrc[e] * ksrc[e];
        }
        sq = wave_allreduce_sum(sq);
        sk = wave_allreduce_sum(sk);
        dot = wave_allreduce_sum(dot);
        const float rq = qscale / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
        float *qdst = qn + t * qk + g * d, *kdst = kn + t * qk + g * d;
        for (int e = lane; e < d; e += 64) {
            qdst[e] = qsrc[e] * rq;
            kdst[e] = ksrc[e] * rk;
        }
        if (lane == 0) kq[t * G + g] = dot * rq * rk;
    }
    for (int i = threadIdx.x; i < H * dv; i += kDpThreads) vv[t * H * dv + i] = act[2 * qk + i];
    for (int h = threadIdx.x; h < H; h += kDpThreads) {
        const float b = to_f(row[C + H * dv + h]), a = to_f(row[C + H * dv + H + h]);
        beta[t * H + h] = dr_sigmoid(b);
        const float z = a + dt_bias[h];
        const float sp = z > 20.f ? z : log1pf(expf(z));
        decay[t * H + h] = expf(-expf(a_log[h]) * sp);
    }
}

template <int L>
__device__ __forceinline__ float dr_group_sum(float v) {
    return group_allreduce_sum<L>(v);
}

// LDS rows of q and k are padded by 4 floats per lane slice: the L lanes of a column read L different 16-byte pieces at
// once, and without the padding slices of 8 / 16 / 32 floats start in the same banks.
__host__ __device__ inline int dr_row_floats(int d, int L) { return d + 4 * L; }

template <int MAXDS, int L, bool EXACT>
__global__ __launch_bounds__(1024) void delta_rule_kernel(float *o, const float *qn, const float *kn, const float *kqn,
                                                          const float *vv, const float *beta, const float *decay,
                                                          float *state, int64_t slot_stride, int64_t s_off,
                                                          const int32_t *seq_row0, const int32_t *seq_cnt,
                                                          const int32_t *tok_pos, const int32_t *tok_state, int H, int G,
                                                          int d, int dv, int cpw, int nload) {
    // nload > 0: the last nload threads of the workgroup only LOAD — they stage chunk c + 1 into the other LDS buffer while
    // the first cpw * L threads walk the tokens of chunk c, one barrier per chunk. nload = 0: everybody stages, then walks.
    extern __shared__ float lds[];
    const int dp = dr_row_floats(d, L);
    const int buf_floats = kDrChunk * (2 * dp + cpw + 3);
    const int seq = blockIdx.x, h = blockIdx.y;
    const int col0 = blockIdx.z * cpw;      // this workgroup's columns of the state (independent recurrences)
    const int row0 = seq_row0[seq], cnt = seq_cnt[seq];
    const int kvh = h / (H / G);
    const int ncomp = static_cast<int>(blockDim.x) - nload;
    const bool computes = static_cast<int>(threadIdx.x) < ncomp;
    const int lc = computes ? threadIdx.x / L : 0, l = threadIdx.x % L;
    const int col = col0 + lc;
    const int ds = EXACT ? MAXDS : d / L, i0 = l * ds;      // (EXACT: the slice fills the register array, no predicates)
    const int qk = G * d, hv = H * dv;
    float *S = state + static_cast<int64_t>(tok_state[row0] >> 1) * slot_stride + s_off + static_cast<int64_t>(h) * d * dv;
    float s[MAXDS];
    const bool fresh = tok_pos[row0] == 0;      // a sequence starts from the zero state whatever the slot held
#pragma unroll
    for (int i = 0; i < MAXDS; ++i) s[i] = (computes && i < ds && !fresh) ? S[static_cast<int64_t>(i0 + i) * dv + col] : 0.f;
    const bool quads = EXACT || (ds & 3) == 0;  // 16-byte LDS reads

    // Stage the chunk at c0 into `buf` with threads sid, sid + sn, ...: all of the chunk's loads are issued before the first
    // one is waited for — one memory round trip per chunk (load by load, with an LDS store between two loads, the round
    // trips of a chunk line up one after the other).
    auto stage = [&](int c0, float *buf, int sid, int sn) {
        const int cn = min(kDrChunk, cnt - c0);
        float *qs = buf, *ks = qs + kDrChunk * dp, *vs = ks + kDrChunk * dp, *bs = vs + kDrChunk * cpw;
        float *gs = bs + kDrChunk, *kqs = gs + kDrChunk;
        for (int e = sid; e < d; e += sn) {
            float tq[kDrChunk], tk[kDrChunk];
            const float *qsrc = qn + static_cast<int64_t>(row0 + c0) * qk + kvh * d + e;
            const float *ksrc = kn + static_cast<int64_t>(row0 + c0) * qk + kvh * d + e;
#pragma unroll
            for (int j = 0; j < kDrChunk; ++j) {
                const int64_t jj = min(j, cn - 1);      // (rows past the chunk's end re-read its last row: never stored)
                tq[j] = qsrc[jj * qk];
                tk[j] = ksrc[jj * qk];
            }
            const int at = e + 4 * (EXACT ? e / MAXDS : e / ds);
#pragma unroll
            for (int j = 0; j < kDrChunk; ++j) {
                if (j < cn) {
                    qs[j * dp + at] = tq[j];
                    ks[j * dp + at] = tk[j];
                }
            }
        }
        for (int e = sid; e < cpw; e += sn) {
            float tv[kDrChunk];
            const float *vsrc = vv + static_cast<int64_t>(row0 + c0) * hv + h * dv + col0 + e;
#pragma unroll
            for (int j = 0; j < kDrChunk; ++j) tv[j] = vsrc[static_cast<int64_t>(min(j, cn - 1)) * hv];
#pragma unroll
            for (int j = 0; j < kDrChunk; ++j)
                if (j < cn) vs[j * cpw + e] = tv[j];
        }
        for (int j = sid; j < cn; j += sn) {
            bs[j] = beta[static_cast<int64_t>(row0 + c0 + j) * H + h];
            gs[j] = decay[static_cast<int64_t>(row0 + c0 + j) * H + h];
            kqs[j] = kqn[static_cast<int64_t>(row0 + c0 + j) * G + kvh];
        }
    };

    // Walk the tokens of the chunk at c0 (staged in `buf`): the sequential part.
    auto walk = [&](int c0, const float *buf) {
        const int cn = min(kDrChunk, cnt - c0);
        const float *qs = buf, *ks = qs + kDrChunk * dp, *vs = ks + kDrChunk * dp, *bs = vs + kDrChunk * cpw;
        const float *gs = bs + kDrChunk, *kqs = gs + kDrChunk;
#pragma unroll 2
        for (int j = 0; j < cn; ++j) {
            const float g = gs[j], b = bs[j], kq = kqs[j];
            const float *kj = ks + j * dp + l * (ds + 4), *qj = qs + j * dp + l * (ds + 4);
            float kr[MAXDS], qr[MAXDS];
            if (quads) {
#pragma unroll
                for (int i = 0; i < MAXDS; i += 4) {
                    if (EXACT || i < ds) {
                        const float4_t k4 = *reinterpret_cast<const float4_t *>(kj + i);
                        const float4_t q4 = *reinterpret_cast<const float4_t *>(qj + i);
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            kr[i + c] = k4[c];
                            qr[i + c] = q4[c];
                        }
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < MAXDS; ++i) {
                    kr[i] = i < ds ? kj[i] : 0.f;
                    qr[i] = i < ds ? qj[i] : 0.f;
                }
            }
            float sk = 0.f, sq = 0.f;
#pragma unroll
            for (int i = 0; i < MAXDS; ++i) {
                if (EXACT || i < ds) {
                    s[i] *= g;
                    sk = fmaf(s[i], kr[i], sk);
                    sq = fmaf(s[i], qr[i], sq);
                }
            }
            sk = dr_group_sum<L>(sk);
            sq = dr_group_sum<L>(sq);
            const float u = b * (vs[j * cpw + lc] - sk);
#pragma unroll
            for (int i = 0; i < MAXDS; ++i)
                if (EXACT || i < ds) s[i] = fmaf(kr[i], u, s[i]);
            if (l == 0) o[static_cast<int64_t>(row0 + c0 + j) * hv + h * dv + col] = fmaf(u, kq, sq);
        }
    };

    if (nload > 0) {
        if (!computes) stage(0, lds, static_cast<int>(threadIdx.x) - ncomp, nload);
        __syncthreads();
        int c = 0;
        for (int c0 = 0; c0 < cnt; c0 += kDrChunk, ++c) {
            if (computes) walk(c0, lds + (c & 1) * buf_floats);
            else if (c0 + kDrChunk < cnt) stage(c0 + kDrChunk, lds + ((c + 1) & 1) * buf_floats, static_cast<int>(threadIdx.x) - ncomp, nload);
            __syncthreads();    // chunk c has been walked and chunk c + 1 is in place
        }
    } else {
        for (int c0 = 0; c0 < cnt; c0 += kDrChunk) {
            __syncthreads();    // the previous chunk has been consumed
            stage(c0, lds, threadIdx.x, blockDim.x);
            __syncthreads();
            walk(c0, lds);
        }
    }
    if (!computes) return;
#pragma unroll
    for (int i = 0; i < MAXDS; ++i)
        if (i < ds) S[static_cast<int64_t>(i0 + i) * dv + col] = s[i];
}

template <typename T>
__global__ __launch_bounds__(256) void gated_head_rmsnorm_kernel(T *out, const float *o, const T *gate, int64_t gate_stride,
                                                                 const float *w, float eps, int H, int dv) {
    const int64_t t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int h = wave; h < H; h += 4) {
        const float *src = o + (t * H + h) * dv;
        float ss = 0.f;
        for (int e = lane; e < dv; e += 64) ss += src[e] * src[e];
        ss = wave_allreduce_sum(ss);
        const float r = 1.0f / sqrtf(ss / static_cast<float>(dv) + eps);
        for (int e = lane; e < dv; e += 64) {
            const float z = to_f(gate[t * gate_stride + h * dv + e]);
            out[(t * H + h) * dv + e] = to_t<T>(src[e] * r * w[e] * (z * dr_sigmoid(z)));
        }
    }
}

// lanes per state column: as many as keep at least 16 elements per lane (measured: slices of 8 do not shorten a prompt's walk
// and cost a decode launch 1.6x, slices of 32 cost a prompt 1.5x), a power of two that divides dim, at most 16 and at most
// 1024 threads per workgroup of `cols` columns
inline int dr_lanes(int d, int cols) {
    int L = 16;
    while (L > 1 && (d % L || d / L < 16 || static_cast<int64_t>(cols) * L > 1024)) L >>= 1;
    return L;
}

template <int L>
int launch_dr(int ds, dim3 grid, dim3 block, size_t lds, hipStream_t s, float *o, const float *qn, const float *kn,
              const float *kq, const float *vv, const float *beta, const float *decay, float *state, int64_t slot_stride, int64_t s_off,
              const int32_t *seq_row0, const int32_t *seq_cnt, const int32_t *tok_pos, const int32_t *tok_state, int H,
              int G, int d, int dv, int cpw, int nload) {
#define SWL_DR_LAUNCH1(M, X)                                                                                                 \
    hipLaunchKernelGGL((delta_rule_kernel<M, L, X>), grid, block, lds, s, o, qn, kn, kq, vv, beta, decay, state, slot_stride, \
                       s_off, seq_row0, seq_cnt, tok_pos, tok_state, H, G, d, dv, cpw, nload)
#define SWL_DR_LAUNCH(M)                   \
    if (ds == M) SWL_DR_LAUNCH1(M, true);  \
    else SWL_DR_LAUNCH1(M, false)
    if (ds <= 8) { SWL_DR_LAUNCH(8); }
    else if (ds <= 16) { SWL_DR_LAUNCH(16); }
    else if (ds <= 32) { SWL_DR_LAUNCH(32); }
    else if (ds <= 64) { SWL_DR_LAUNCH(64); }
    else if (ds <= 128) { SWL_DR_LAUNCH(128); }
    else return SWL_ERR_UNSUPPORTED;
#undef SWL_DR_LAUNCH
#undef SWL_DR_LAUNCH1
    return check_launch();
}

} // namespace swl

extern "C" int swl_delta_prep(float *qn, float *kn, float *kq, float *vv, float *beta, float *decay, const void *proj,
                              int64_t proj_stride, const float *conv_w, const float *a_log, const float *dt_bias,
                              float *state, int64_t slot_stride, int64_t tail_off, const int32_t *tok_pos,
                              const int32_t *tok_start, const int32_t *tok_state, const int32_t *tok_seq,
                              int64_t num_tokens, int32_t num_heads, int32_t num_qk_heads, int32_t dim, int32_t vdim,
                              int32_t taps, int32_t dtype, swl_stream_t stream) {
    if (num_tokens < 0 || num_heads <= 0 || num_qk_heads <= 0 || dim <= 0 || vdim <= 0 || taps < 1) return SWL_ERR_BAD_ARG;
    if (num_heads % num_qk_heads) return SWL_ERR_BAD_ARG;
    const int64_t C = 2LL * num_qk_heads * dim + static_cast<int64_t>(num_heads) * vdim;
    if (proj_stride < C + static_cast<int64_t>(num_heads) * vdim + 2 * num_heads) return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!qn || !kn || !kq || !vv || !beta || !decay || !proj || !conv_w || !a_log || !dt_bias || !tok_pos || !tok_start || !tok_seq)
        return SWL_ERR_BAD_ARG;
    if (taps > 1 && (!state || !tok_state)) return SWL_ERR_BAD_ARG;
    const size_t lds = static_cast<size_t>(C) * sizeof(float);
    if (num_tokens > 0x7fffffffLL || lds > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::delta_prep_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(swl::kDpThreads), lds,
                           static_cast<hipStream_t>(stream), qn, kn, kq, vv, beta, decay, static_cast<const T *>(proj),
                           proj_stride, conv_w, a_log, dt_bias, state, slot_stride, tail_off, tok_pos, tok_start,
                           tok_state, tok_seq, num_tokens, num_heads, num_qk_heads, dim, vdim, taps);
    });
    return swl::check_launch();
}

extern "C" int swl_delta_rule(float *o, const float *qn, const float *kn, const float *kq, const float *vv,
                              const float *beta,
                              const float *decay, float *state, int64_t slot_stride, int64_t s_off,
                              const int32_t *seq_row0, const int32_t *seq_cnt, const int32_t *tok_pos,
                              const int32_t *tok_state, int32_t num_seqs, int32_t num_heads, int32_t num_qk_heads,
                              int32_t dim, int32_t vdim, swl_stream_t stream) {
    if (num_seqs < 0 || num_heads <= 0 || num_qk_heads <= 0 || dim <= 0 || vdim <= 0 || num_heads % num_qk_heads)
        return SWL_ERR_BAD_ARG;
    if (num_seqs == 0) return SWL_OK;
    if (!o || !qn || !kn || !kq || !vv || !beta || !decay || !state || !seq_row0 || !seq_cnt || !tok_pos || !tok_state)
        return SWL_ERR_BAD_ARG;
    if (vdim > 1024 || num_heads > 65535) return SWL_ERR_UNSUPPORTED;
    // columns per workgroup: all of them when there are (portion, head) pairs enough to fill the chip (decode batches); a
    // long prompt alone is a sequential walk, so its columns are shared out over more workgroups (down to 16 columns each)
    int cpw = vdim;
    while (static_cast<int64_t>(num_seqs) * num_heads * (vdim / cpw) < 512 && cpw % 2 == 0 && cpw > 16) cpw /= 2;
    const int L = swl::dr_lanes(dim, cpw);
    const int ds = dim / L;
    const size_t one = (static_cast<size_t>(swl::kDrChunk) * (2 * swl::dr_row_floats(dim, L) + cpw + 3)) * sizeof(float);
    if (one > 64 * 1024) return SWL_ERR_UNSUPPORTED;
    // a wave of loaders and a second LDS buffer when both fit and there is more than one chunk's worth of tokens to gain from
    const int nload = (cpw * L + 64 <= 1024 && 2 * one <= 64 * 1024) ? 64 : 0;
    const size_t lds = nload ? 2 * one : one;
    const dim3 grid(static_cast<unsigned>(num_seqs), static_cast<unsigned>(num_heads), static_cast<unsigned>(vdim / cpw));
    const dim3 block(static_cast<unsigned>(cpw * L + nload));
    hipStream_t s = static_cast<hipStream_t>(stream);
#define SWL_DR_L(LL)                                                                                                         \
    case LL: return swl::launch_dr<LL>(ds, grid, block, lds, s, o, qn, kn, kq, vv, beta, decay, state, slot_stride, s_off,       \
                                       seq_row0, seq_cnt, tok_pos, tok_state, num_heads, num_qk_heads, dim, vdim, cpw, nload)
    switch (L) {
        SWL_DR_L(1);
        SWL_DR_L(2);
        SWL_DR_L(4);
        SWL_DR_L(8);
        SWL_DR_L(16);
    }
#undef SWL_DR_L
    return SWL_ERR_UNSUPPORTED;
}

extern "C" int swl_gated_head_rmsnorm(void *out, const float *o, const void *gate, int64_t gate_stride, const float *w,
                                      float eps, int64_t num_tokens, int32_t num_heads, int32_t vdim, int32_t dtype,
                                      swl_stream_t stream) {
    if (num_tokens < 0 || num_heads <= 0 || vdim <= 0 || gate_stride < static_cast<int64_t>(num_heads) * vdim)
        return SWL_ERR_BAD_ARG;
    if (num_tokens == 0) return SWL_OK;
    if (!out || !o || !gate || !w) return SWL_ERR_BAD_ARG;
    if (num_tokens > 0x7fffffffLL) return SWL_ERR_UNSUPPORTED;
    SWL_DISPATCH_DTYPE3(dtype, T, {
        hipLaunchKernelGGL((swl::gated_head_rmsnorm_kernel<T>), dim3(static_cast<unsigned>(num_tokens)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), static_cast<T *>(out), o, static_cast<const T *>(gate),
                           gate_stride, w, eps, num_heads, vdim);
    });
    return swl::check_launch();
}
