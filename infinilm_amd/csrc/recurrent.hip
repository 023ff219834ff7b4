// Kernels of the mixers that carry a fixed-size state from token to token (linear attention with a decay,
// selective state spaces) and of the small steps around them: activations, rotation by computed angles,
// norms in groups with a gate, the short causal convolution, unit-norm queries and keys with a
// position-dependent temperature, and a weighted sum of two branches.
//
// Everything that enters a recurrence is float: states, decays, step sizes, rotated queries and keys.  A
// request's state passes from step to step through a row of a float pool, so cutting a prompt into portions
// changes no bit: a token's result is a function of the state before it and of its own row.
#include "common.h"

__device__ __forceinline__ float ldf(const void* p, int dt, size_t i) {
    return dt == ILM_DTYPE_F32 ? ((const float*)p)[i] : bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
__device__ __forceinline__ void stf(void* p, int dt, size_t i, float v) {
    if (dt == ILM_DTYPE_F32) ((float*)p)[i] = v;
    else ((uint16_t*)p)[i] = __builtin_bit_cast(uint16_t, (__bf16)v);
}
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

#define RC_ACT_NONE 0
#define RC_ACT_SILU 1
#define RC_ACT_SIGMOID 2
#define RC_ACT_RELU2 3
#define RC_ACT_GELU_TANH 4

__device__ __forceinline__ float act_f(float x, int kind) {
    switch (kind) {
        case RC_ACT_SILU: return silu_f(x);
        case RC_ACT_SIGMOID: return sigmoid_f(x);
        case RC_ACT_RELU2: { const float r = fmaxf(x, 0.f); return r * r; }
        case RC_ACT_GELU_TANH: return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
        default: return x;
    }
}

// eight consecutive elements as floats / from floats (16-byte accesses for bfloat16, two for float)
__device__ __forceinline__ void ld8(const void* p, int dt, size_t i, float (&v)[8]) {
    if (dt == ILM_DTYPE_F32) {
        const float4 a = *reinterpret_cast<const float4*>((const float*)p + i), b = *reinterpret_cast<const float4*>((const float*)p + i + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        uint16_t t[8];
        *reinterpret_cast<uint4*>(t) = *reinterpret_cast<const uint4*>((const uint16_t*)p + i);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = bf16_bits_to_f32(t[e]);
    }
}
__device__ __forceinline__ void st8(void* p, int dt, size_t i, const float (&v)[8]) {
    if (dt == ILM_DTYPE_F32) {
        *reinterpret_cast<float4*>((float*)p + i) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>((float*)p + i + 4) = make_float4(v[4], v[5], v[6], v[7]);
    } else {
        uint16_t t[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = __builtin_bit_cast(uint16_t, (__bf16)v[e]);
        *reinterpret_cast<uint4*>((uint16_t*)p + i) = *reinterpret_cast<uint4*>(t);
    }
}

// ------------------------------------------------------------------------------------------
// out[t, j] = act(in[t, j]), rows of n elements with their own strides
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
unary_kernel(void* __restrict__ out, const void* __restrict__ in, int n, int out_stride, int in_stride, int kind,
             int out_dt, int in_dt) {
    const int t = blockIdx.y;
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    stf(out, out_dt, (size_t)t * out_stride + j, act_f(ldf(in, in_dt, (size_t)t * in_stride + j), kind));
}

// bfloat16 rows, eight elements a thread (16-byte accesses): n and the strides multiples of 8, rows 16 bytes aligned
__global__ void __launch_bounds__(256)
unary_vec_kernel(uint16_t* __restrict__ out, const uint16_t* __restrict__ in, int n, int out_stride, int in_stride, int kind) {
    const int t = blockIdx.y;
    const int j = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (j >= n) return;
    uint16_t a[8], r[8];
    *reinterpret_cast<uint4*>(a) = *reinterpret_cast<const uint4*>(in + (size_t)t * in_stride + j);
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = __builtin_bit_cast(uint16_t, (__bf16)act_f(bf16_bits_to_f32(a[e]), kind));
    *reinterpret_cast<uint4*>(out + (size_t)t * out_stride + j) = *reinterpret_cast<uint4*>(r);
}

extern "C" int ilm_unary(void* out, const void* in, int T_, int n, int out_stride, int in_stride, int kind, int out_dt,
                         int in_dt, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && n > 0 && T_ <= 65535 * 32768, "unary: bad sizes T=%d n=%d", T_, n);
    ILM_REQUIRE(kind >= 0 && kind <= RC_ACT_GELU_TANH, "unary: unknown activation %d", kind);
    if (out_dt == ILM_DTYPE_BF16 && in_dt == ILM_DTYPE_BF16 && n % 8 == 0 && out_stride % 8 == 0 && in_stride % 8 == 0
        && ((uintptr_t)out & 15) == 0 && ((uintptr_t)in & 15) == 0) {
        for (int t0 = 0; t0 < T_; t0 += 65535) {
            const int rows = T_ - t0 < 65535 ? T_ - t0 : 65535;
            unary_vec_kernel<<<dim3((n / 8 + 255) / 256, rows), 256, 0, stream>>>(
                (uint16_t*)out + (size_t)t0 * out_stride, (const uint16_t*)in + (size_t)t0 * in_stride, n, out_stride, in_stride, kind);
        }
        ILM_LAUNCH_CHECK("unary");
        return 0;
    }
    for (int t0 = 0; t0 < T_; t0 += 65535) {
        const int rows = T_ - t0 < 65535 ? T_ - t0 : 65535;
        const size_t eo = out_dt == ILM_DTYPE_F32 ? 4 : 2, ei = in_dt == ILM_DTYPE_F32 ? 4 : 2;
        unary_kernel<<<dim3((n + 255) / 256, rows), 256, 0, stream>>>((char*)out + (size_t)t0 * out_stride * eo,
                                                                      (const char*)in + (size_t)t0 * in_stride * ei, n,
                                                                      out_stride, in_stride, kind, out_dt, in_dt);
    }
    ILM_LAUNCH_CHECK("unary");
    return 0;
}

// ------------------------------------------------------------------------------------------
// Decays of a gated recurrence from their raw rows: out[t, j] = sigmoid(z[t, j] + b[j])^inv_tau = exp(inv_tau * log
// sigmoid(.)), the logarithm in its stable form (-log1p(exp(-x)) for x >= 0, x - log1p(exp(x)) below); float results.
// ------------------------------------------------------------------------------------------
template <typename T, typename TB>
__global__ void __launch_bounds__(256)
sigmoid_root_kernel(float* __restrict__ out, const T* __restrict__ z, const TB* __restrict__ bias, int n, int out_stride,
                    int in_stride, float inv_tau) {
    const int t = blockIdx.y, j = blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    const float x = to_f32(z[(size_t)t * in_stride + j]) + (bias != nullptr ? to_f32(bias[j]) : 0.f);
    const float ls = x >= 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x));
    out[(size_t)t * out_stride + j] = expf(inv_tau * ls);
}

extern "C" int ilm_sigmoid_root(void* out, const void* z, const void* bias, int T_, int n, int out_stride, int in_stride,
                                float inv_tau, int z_dt, int b_dt, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && n > 0, "sigmoid_root: bad sizes");
    ILM_REQUIRE(z_dt == ILM_DTYPE_F32 || z_dt == ILM_DTYPE_BF16, "sigmoid_root: unknown dtype %d", z_dt);
    ILM_REQUIRE(bias == nullptr || b_dt == ILM_DTYPE_F32 || b_dt == ILM_DTYPE_BF16, "sigmoid_root: unknown bias dtype %d", b_dt);
    for (int t0 = 0; t0 < T_; t0 += 65535) {
        const int rows = T_ - t0 < 65535 ? T_ - t0 : 65535;
        dim3 grid((n + 255) / 256, rows);
        float* o = (float*)out + (size_t)t0 * out_stride;
#define SR_LAUNCH(T__, TB__)                                                                                          \
    sigmoid_root_kernel<T__, TB__><<<grid, 256, 0, stream>>>(o, (const T__*)z + (size_t)t0 * in_stride, (const TB__*)bias, n, \
                                                             out_stride, in_stride, inv_tau)
        if (z_dt == ILM_DTYPE_F32) {
            if (b_dt == ILM_DTYPE_BF16) SR_LAUNCH(float, bf16); else SR_LAUNCH(float, float);
        } else {
            if (b_dt == ILM_DTYPE_BF16) SR_LAUNCH(bf16, bf16); else SR_LAUNCH(bf16, float);
        }
#undef SR_LAUNCH
    }
    ILM_LAUNCH_CHECK("sigmoid_root");
    return 0;
}

// ------------------------------------------------------------------------------------------
// Queries, keys and values of a linear-attention mixer made ready for the recurrence, as floats:
// rows [q: heads*dk | k: heads*dk | v: heads*dv] of the fused projection -> the same layout in float, with an
// activation on all three, then the first `rd` entries of each q and k head turned by the angle pos * freq[i]
// (entry i paired with entry i + rd/2), then k times k_scale.  One block a token.
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
lin_prep_kernel(float* __restrict__ out, const void* __restrict__ in, const int* __restrict__ pos,
                const float* __restrict__ freq, int heads, int dk, int dv, int rd, int in_stride, int act, float k_scale,
                int in_dt) {
    const int t = blockIdx.x;
    const int nqk = heads * dk, n = 2 * nqk + heads * dv;
    const size_t ib = (size_t)t * in_stride, ob = (size_t)t * n;
    const int half = rd >> 1;
    const float p = (float)pos[t];
    // the turned pairs
    const int pairs = 2 * heads * half;
    for (int it = threadIdx.x; it < pairs; it += 256) {
        const int hs = it / half, i = it % half;   // hs: q heads, then k heads
        const size_t c = (size_t)hs * dk + i;
        const float a = act_f(ldf(in, in_dt, ib + c), act), b = act_f(ldf(in, in_dt, ib + c + half), act);
        const float ang = p * freq[i];
        float sn, cs;
        sincosf(ang, &sn, &cs);
        const float sc = hs >= heads ? k_scale : 1.0f;
        out[ob + c] = (a * cs - b * sn) * sc;
        out[ob + c + half] = (b * cs + a * sn) * sc;
    }
    // what passes: the rest of the q and k heads, and v
    const int rest = dk - rd;
    for (int it = threadIdx.x; it < 2 * heads * rest; it += 256) {
        const int hs = it / rest, i = rd + it % rest;
        const size_t c = (size_t)hs * dk + i;
        out[ob + c] = act_f(ldf(in, in_dt, ib + c), act) * (hs >= heads ? k_scale : 1.0f);
    }
    for (int j = 2 * nqk + threadIdx.x; j < n; j += 256) out[ob + j] = act_f(ldf(in, in_dt, ib + j), act);
}

// The same with eight elements a thread: head sizes and half the turned entries in multiples of 8, rows 16 bytes aligned.
__global__ void __launch_bounds__(256)
lin_prep_vec_kernel(float* __restrict__ out, const void* __restrict__ in, const int* __restrict__ pos,
                    const float* __restrict__ freq, int heads, int dk, int dv, int rd, int in_stride, int act, float k_scale,
                    int in_dt) {
    const int t = blockIdx.x;
    const int nqk = heads * dk, n = 2 * nqk + heads * dv;
    const size_t ib = (size_t)t * in_stride, ob = (size_t)t * n;
    const int half = rd >> 1, hp = half >> 3, rest = (dk - rd) >> 3;
    const int per_head = hp + rest;                       // work items of a q or k head: turned pairs of pieces, then passing pieces
    const int n_qk = 2 * heads * per_head, n_items = n_qk + (heads * dv >> 3);
    const float p = rd > 0 ? (float)pos[t] : 0.f;
    for (int it = threadIdx.x; it < n_items; it += 256) {
        float a[8], o8[8];
        if (it >= n_qk) {                                  // values
            const size_t c = 2 * (size_t)nqk + (size_t)(it - n_qk) * 8;
            ld8(in, in_dt, ib + c, a);
#pragma unroll
            for (int e = 0; e < 8; ++e) o8[e] = act_f(a[e], act);
            st8(out, ILM_DTYPE_F32, ob + c, o8);
            continue;
        }
        const int hs = it / per_head, piece = it % per_head;
        const float sc = hs >= heads ? k_scale : 1.0f;
        if (piece >= hp) {                                 // entries that pass
            const size_t c = (size_t)hs * dk + rd + (size_t)(piece - hp) * 8;
            ld8(in, in_dt, ib + c, a);
#pragma unroll
            for (int e = 0; e < 8; ++e) o8[e] = act_f(a[e], act) * sc;
            st8(out, ILM_DTYPE_F32, ob + c, o8);
            continue;
        }
        const int i0 = piece * 8;
        const size_t c = (size_t)hs * dk + i0;
        float b[8], o9[8];
        ld8(in, in_dt, ib + c, a);
        ld8(in, in_dt, ib + c + half, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float u = act_f(a[e], act), w = act_f(b[e], act);
            float sn, cs;
            sincosf(p * freq[i0 + e], &sn, &cs);
            o8[e] = (u * cs - w * sn) * sc;
            o9[e] = (w * cs + u * sn) * sc;
        }
        st8(out, ILM_DTYPE_F32, ob + c, o8);
        st8(out, ILM_DTYPE_F32, ob + c + half, o9);
    }
}

extern "C" int ilm_lin_prep(void* out, const void* in, const void* pos, const void* freq, int T_, int heads, int dk, int dv,
                            int rd, int in_stride, int act, float k_scale, int in_dt, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && heads > 0 && dk > 0 && dv > 0, "lin_prep: bad sizes");
    ILM_REQUIRE(rd >= 0 && rd <= dk && rd % 2 == 0, "lin_prep: %d turned entries do not fit a head of %d", rd, dk);
    ILM_REQUIRE(rd == 0 || (freq != nullptr && pos != nullptr), "lin_prep: a rotation needs positions and frequencies");
    ILM_REQUIRE(in_stride >= 2 * heads * dk + heads * dv, "lin_prep: rows of %d elements are too short", in_stride);
    if (dk % 8 == 0 && dv % 8 == 0 && rd % 16 == 0 && in_stride % 8 == 0 && (((uintptr_t)out | (uintptr_t)in) & 15) == 0) {
        lin_prep_vec_kernel<<<T_, 256, 0, stream>>>((float*)out, in, (const int*)pos, (const float*)freq, heads, dk, dv, rd,
                                                    in_stride, act, k_scale, in_dt);
        ILM_LAUNCH_CHECK("lin_prep");
        return 0;
    }
    lin_prep_kernel<<<T_, 256, 0, stream>>>((float*)out, in, (const int*)pos, (const float*)freq, heads, dk, dv, rd, in_stride,
                                            act, k_scale, in_dt);
    ILM_LAUNCH_CHECK("lin_prep");
    return 0;
}

// ------------------------------------------------------------------------------------------
// The recurrence  S_t = a_t S_(t-1) + (b_t k_t) v_t^T,  o_t = S_t^T q_t + skip v_t  per (request, head), token by token.
//
// A block of 256 threads owns a head's state for VT = 256 / KP value columns: thread (kp, column) keeps the
// SC_NK entries kp, kp + KP, kp + 2 KP, ... of the column's dk state entries in registers; a token's output is
// the sum over the KP threads of a column (lanes of one wave, folded by shuffles).  The state pool holds a
// head's state as [dv][dk] (the key index fastest), so a column's KP threads read consecutive floats.
// a_t comes per head (decay_h) or per token and head (decay_t [T, heads]); b_t (kscale_t [T, heads]) and skip
// (skip_h [heads]) may be absent.  Head h reads the q and k of group h / q_div.
// Requests are the segments of the step: seg_offsets [R + 1] rows, state_in / state_out [R] pool rows.
//
// Long segments (portions of prompts) are cut into pieces of `piece` tokens that run side by side, in three launches:
//   SC_LOCAL    every piece runs its tokens from a zero state and leaves that local state, and the product of its
//               decays, in a workspace slot;
//   (combine)   per segment, piece after piece: the state at a piece's start = decay product of the piece before x the
//               state at that piece's start + its local state, written over the local states; the state after the last
//               piece goes to the pool;
//   SC_FROM     every piece runs its tokens again from its start state and writes the outputs.
// Twice the arithmetic of one pass, and as many blocks as the step has pieces.  Piece p of segment r has the slot
// floor(first row of r / piece) + r + p: slots of different segments never meet, and floor(T / piece) + R slots hold all.
// A block finds its (segment, piece) from its slot by bisection over the segments' first slots.
// ------------------------------------------------------------------------------------------
// Sums over the KP lanes of a column group, for the four columns a thread holds: two exchanges halve the columns a lane
// goes on with (lanes with bit 0 clear keep columns 0 and 1, then bit 1 picks one of the two), the remaining steps fold
// one number.  At the end lane kp (kp < 4) of the group holds the sum of column 2 * (kp & 1) + ((kp >> 1) & 1): five
// exchanges for 16 lanes where four separate folds take sixteen.  KP >= 4.
__device__ __forceinline__ float sc_fold4(const float (&acc)[4], int kp, int KP) {
    const bool b0 = kp & 1, b1 = kp & 2;
    const float s0 = __shfl_xor(b0 ? acc[0] : acc[2], 1, 64), s1 = __shfl_xor(b0 ? acc[1] : acc[3], 1, 64);
    const float k0 = (b0 ? acc[2] : acc[0]) + s0, k1 = (b0 ? acc[3] : acc[1]) + s1;
    float v = (b1 ? k1 : k0) + __shfl_xor(b1 ? k0 : k1, 2, 64);
    for (int off = 4; off < KP; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}

#define SC_NK 8
#define SC_LOCAL 1
#define SC_FROM 2

// the segment whose slots hold slot s (-1: none), its piece p
__device__ __forceinline__ int sc_find(const int* __restrict__ seg_offsets, int R, int piece, int s, int& p) {
    int lo = 0, hi = R - 1;     // the last segment whose first slot is <= s
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (seg_offsets[mid] / piece + mid <= s) lo = mid; else hi = mid - 1;
    }
    p = s - (seg_offsets[lo] / piece + lo);
    const int len = seg_offsets[lo + 1] - seg_offsets[lo];
    return (p >= 0 && p * piece < len) ? lo : -1;
}

// CH: the decay comes per token, head and key channel (decay_c, rows of heads * dk floats dc_stride apart) and acts on the
// state's rows: S_t = diag(a_t) S_(t-1) + ...
template <int VC, bool CH = false>   // VC: value columns a thread (the q and k a thread loads serve all of them)
__global__ void __launch_bounds__(256)
decay_scan_kernel(float* __restrict__ o, int o_stride, const float* __restrict__ q, const float* __restrict__ k,
                  int qk_stride, int q_div, const float* __restrict__ v, int v_stride,
                  const float* __restrict__ decay_h, const float* __restrict__ decay_t,
                  const float* __restrict__ kscale_t, const float* __restrict__ skip_h, float* __restrict__ pool,
                  const int* __restrict__ state_in, const int* __restrict__ state_out,
                  const int* __restrict__ seg_offsets, int heads, int dk, int dv, int KP,
                  const float* __restrict__ decay_c = nullptr, int dc_stride = 0) {
    const int h = blockIdx.y, r = blockIdx.z;
    const int t0 = seg_offsets[r], t1 = seg_offsets[r + 1];
    if (t0 >= t1) return;
    const int VT = 256 / KP;                                 // column groups a block
    const int kp = threadIdx.x % KP, vc0 = (blockIdx.x * VT + threadIdx.x / KP) * VC;
    const size_t hs = (size_t)dk * dv;                       // floats of a head's state
    const float* src = pool + ((size_t)state_in[r] * heads + h) * hs;
    float S[VC][SC_NK];
#pragma unroll
    for (int c = 0; c < VC; ++c)
#pragma unroll
        for (int i = 0; i < SC_NK; ++i) {
            const int ki = i * KP + kp;
            S[c][i] = (vc0 + c < dv && ki < dk) ? src[(size_t)(vc0 + c) * dk + ki] : 0.f;
        }
    const int qoff = (h / q_div) * dk;
    const float a_h = decay_h != nullptr ? decay_h[h] : 1.0f;
    const float skip = skip_h != nullptr ? skip_h[h] : 0.f;
    float qn[SC_NK], kn[SC_NK], vn[VC], an, bn, acn[CH ? SC_NK : 1];
#define SC_LOAD(T_)                                                                              \
    {                                                                                            \
        const float* qr = q + (size_t)(T_) * qk_stride + qoff;                                   \
        const float* kr = k + (size_t)(T_) * qk_stride + qoff;                                   \
        _Pragma("unroll") for (int i = 0; i < SC_NK; ++i) {                                      \
            const int ki = i * KP + kp;                                                          \
            qn[i] = ki < dk ? qr[ki] : 0.f;                                                      \
            kn[i] = ki < dk ? kr[ki] : 0.f;                                                      \
            if (CH) acn[CH ? i : 0] = ki < dk ? decay_c[(size_t)(T_) * dc_stride + (size_t)h * dk + ki] : 0.f; \
        }                                                                                        \
        _Pragma("unroll") for (int c = 0; c < VC; ++c)                                           \
            vn[c] = vc0 + c < dv ? v[(size_t)(T_) * v_stride + (size_t)h * dv + vc0 + c] : 0.f;  \
        an = decay_t != nullptr ? decay_t[(size_t)(T_) * heads + h] : a_h;                       \
        bn = kscale_t != nullptr ? kscale_t[(size_t)(T_) * heads + h] : 1.0f;                    \
    }
    SC_LOAD(t0)
    for (int t = t0; t < t1; ++t) {
        float qc[SC_NK], kc[SC_NK], vcur[VC], ac[SC_NK];
        const float a = an, b = bn;
#pragma unroll
        for (int i = 0; i < SC_NK; ++i) {
            qc[i] = qn[i];
            kc[i] = kn[i] * b;
            ac[i] = CH ? acn[CH ? i : 0] : a;
        }
#pragma unroll
        for (int c = 0; c < VC; ++c) vcur[c] = vn[c];
        if (t + 1 < t1) SC_LOAD(t + 1)      // the next token's operands are on their way while this one is computed
        float acc[VC];
#pragma unroll
        for (int c = 0; c < VC; ++c) {
            acc[c] = 0.f;
#pragma unroll
            for (int i = 0; i < SC_NK; ++i) {
                S[c][i] = fmaf(ac[i], S[c][i], kc[i] * vcur[c]);
                acc[c] = fmaf(S[c][i], qc[i], acc[c]);
            }
        }
        if (VC == 4 && KP >= 4) {
            const float (&a4)[4] = reinterpret_cast<const float (&)[4]>(acc);
            const float tot = sc_fold4(a4, kp, KP);
            const int c = 2 * (kp & 1) + ((kp >> 1) & 1);
            const float vsel = c == 0 ? vcur[0] : c == 1 ? vcur[VC > 1 ? 1 : 0] : c == 2 ? vcur[VC > 2 ? 2 : 0] : vcur[VC > 3 ? 3 : 0];
            if (kp < 4 && vc0 + c < dv) o[(size_t)t * o_stride + (size_t)h * dv + vc0 + c] = fmaf(skip, vsel, tot);
        } else {
#pragma unroll
            for (int c = 0; c < VC; ++c) {
                for (int off = 1; off < KP; off <<= 1) acc[c] += __shfl_xor(acc[c], off, 64);
                if (kp == 0 && vc0 + c < dv) o[(size_t)t * o_stride + (size_t)h * dv + vc0 + c] = fmaf(skip, vcur[c], acc[c]);
            }
        }
    }
#undef SC_LOAD
    float* dst = pool + ((size_t)state_out[r] * heads + h) * hs;
#pragma unroll
    for (int c = 0; c < VC; ++c)
#pragma unroll
        for (int i = 0; i < SC_NK; ++i) {
            const int ki = i * KP + kp;
            if (vc0 + c < dv && ki < dk) dst[(size_t)(vc0 + c) * dk + ki] = S[c][i];
        }
}

// The pieces' form (SC_LOCAL: local states, SC_FROM: outputs from given start states): a token's q, k, v, decay and scale reach the threads through
// LDS in tiles of TB tokens that the block loads together, the next tile on its way from memory while this one is
// computed (one barrier a tile), instead of every thread loading its own entries token by token: a wave then waits for
// memory once a tile, not once a token.  Thread (kp, column group) owns the SC_NK consecutive state entries
// kp * SC_NK ... of its VC columns.  LDS: 2 buffers x TB x (2 dkp + columns + 2) floats, dkp = KP * SC_NK.
// CH: a decay per token, head and key channel (decay_c, rows dc_stride apart): the tile holds the decays beside q and k,
// and a piece's product of decays is a vector of dk numbers a head (ws_decay [slots][heads][dk]).
template <int MODE, int VC, bool CH = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3)))   // (three blocks a compute unit: 168 registers)
decay_scan_tiled_kernel(float* __restrict__ o, int o_stride, const float* __restrict__ q, const float* __restrict__ k,
                        int qk_stride, int q_div, const float* __restrict__ v, int v_stride,
                        const float* __restrict__ decay_h, const float* __restrict__ decay_t,
                        const float* __restrict__ kscale_t, const float* __restrict__ skip_h,
                        const int* __restrict__ seg_offsets, int heads, int dk, int dv, int KP, int R, int piece, int TB,
                        float* __restrict__ ws_state, float* __restrict__ ws_decay, const float* __restrict__ decay_c = nullptr,
                        int dc_stride = 0) {
    extern __shared__ float lds[];
    const int h = blockIdx.y, slot = blockIdx.z;
    int p;
    const int r = sc_find(seg_offsets, R, piece, slot, p);
    if (r < 0) return;
    const int t0 = seg_offsets[r] + p * piece, t1 = min(t0 + piece, seg_offsets[r + 1]);
    const int VT = 256 / KP, cols = VT * VC, dkp = KP * SC_NK;
    const int kp = threadIdx.x % KP, cl = (threadIdx.x / KP) * VC;   // first column of the thread inside the block
    const int vb = blockIdx.x * cols;                                 // first column of the block
    const size_t hs = (size_t)dk * dv;
    float* st = ws_state + ((size_t)slot * heads + h) * hs;
    const int per = TB * ((CH ? 3 : 2) * dkp + cols + 2);             // floats of one buffer: q | k | v | a | b (| decays per channel)
    float S[VC][SC_NK];
#pragma unroll
    for (int c = 0; c < VC; ++c)
#pragma unroll
        for (int i = 0; i < SC_NK; ++i) {
            const int ki = kp * SC_NK + i, vc = vb + cl + c;
            S[c][i] = (MODE == SC_FROM && vc < dv && ki < dk) ? st[(size_t)vc * dk + ki] : 0.f;
        }
    const int qoff = (h / q_div) * dk;
    const float a_h = decay_h != nullptr ? decay_h[h] : 1.0f;
    const float skip = skip_h != nullptr ? skip_h[h] : 0.f;
    float rq[8], rk[8], rv[8], rc[CH ? 8 : 1], ra = 1.f, rb = 1.f;     // a tile on its way: TB * dkp <= 2048 and TB * cols <= 2048
#define SCT_FETCH(T0_)                                                                                       \
    {                                                                                                        \
        _Pragma("unroll") for (int i = 0; i < 8; ++i) {                                                      \
            const int idx = threadIdx.x + i * 256, tt = idx / dkp, ki = idx % dkp;                           \
            const bool ok = idx < TB * dkp && (T0_) + tt < t1 && ki < dk;                                    \
            const size_t at = (size_t)((T0_) + tt) * qk_stride + qoff + ki;                                  \
            rq[i] = (MODE == SC_FROM && ok) ? q[at] : 0.f;                                                   \
            rk[i] = ok ? k[at] : 0.f;                                                                        \
            if (CH) rc[CH ? i : 0] = ok ? decay_c[(size_t)((T0_) + tt) * dc_stride + (size_t)h * dk + ki] : 1.f; \
        }                                                                                                    \
        _Pragma("unroll") for (int i = 0; i < 8; ++i) {                                                      \
            const int idx = threadIdx.x + i * 256, tt = idx / cols, c = idx % cols;                          \
            const bool ok = idx < TB * cols && (T0_) + tt < t1 && vb + c < dv;                               \
            rv[i] = ok ? v[(size_t)((T0_) + tt) * v_stride + (size_t)h * dv + vb + c] : 0.f;                 \
        }                                                                                                    \
        if (threadIdx.x < TB && (T0_) + threadIdx.x < t1) {                                                  \
            ra = decay_t != nullptr ? decay_t[(size_t)((T0_) + threadIdx.x) * heads + h] : a_h;              \
            rb = kscale_t != nullptr ? kscale_t[(size_t)((T0_) + threadIdx.x) * heads + h] : 1.0f;           \
        }                                                                                                    \
    }
#define SCT_STORE(BUF_)                                                                                      \
    {                                                                                                        \
        float* b_ = lds + (BUF_) * per;                                                                      \
        _Pragma("unroll") for (int i = 0; i < 8; ++i) {                                                      \
            const int idx = threadIdx.x + i * 256;                                                           \
            if (idx < TB * dkp) {                                                                            \
                b_[idx] = rq[i];                                                                             \
                b_[TB * dkp + idx] = rk[i];                                                                  \
                if (CH) b_[TB * (2 * dkp + cols + 2) + idx] = rc[CH ? i : 0];                                \
            }                                                                                                \
            if (idx < TB * cols) b_[2 * TB * dkp + idx] = rv[i];                                             \
        }                                                                                                    \
        if (threadIdx.x < TB) {                                                                              \
            b_[TB * (2 * dkp + cols) + threadIdx.x] = ra;                                                    \
            b_[TB * (2 * dkp + cols + 1) + threadIdx.x] = rb;                                                \
        }                                                                                                    \
    }
    SCT_FETCH(t0)
    SCT_STORE(0)
    __syncthreads();
    float aprod = 1.0f, aprodc[CH ? SC_NK : 1];
#pragma unroll
    for (int i = 0; i < (CH ? SC_NK : 1); ++i) aprodc[i] = 1.0f;
    int buf = 0;
    for (int tb = t0; tb < t1; tb += TB, buf ^= 1) {
        const bool more = tb + TB < t1;
        if (more) SCT_FETCH(tb + TB)
        const float* b_ = lds + buf * per;
        const int n = min(TB, t1 - tb);
#pragma unroll 2
        for (int tt = 0; tt < n; ++tt) {
            float qc[SC_NK], kc[SC_NK], vcur[VC], ac[SC_NK];
            const float a = b_[TB * (2 * dkp + cols) + tt], bsc = b_[TB * (2 * dkp + cols + 1) + tt];
#pragma unroll
            for (int i4 = 0; i4 < SC_NK; i4 += 4) {
                if (MODE == SC_FROM) {
                    const float4 t4 = *reinterpret_cast<const float4*>(b_ + tt * dkp + kp * SC_NK + i4);
                    qc[i4] = t4.x; qc[i4 + 1] = t4.y; qc[i4 + 2] = t4.z; qc[i4 + 3] = t4.w;
                }
                const float4 u4 = *reinterpret_cast<const float4*>(b_ + TB * dkp + tt * dkp + kp * SC_NK + i4);
                kc[i4] = u4.x * bsc; kc[i4 + 1] = u4.y * bsc; kc[i4 + 2] = u4.z * bsc; kc[i4 + 3] = u4.w * bsc;
                if (CH) {
                    const float4 w4 = *reinterpret_cast<const float4*>(b_ + TB * (2 * dkp + cols + 2) + tt * dkp + kp * SC_NK + i4);
                    ac[i4] = w4.x; ac[i4 + 1] = w4.y; ac[i4 + 2] = w4.z; ac[i4 + 3] = w4.w;
                } else {
                    ac[i4] = ac[i4 + 1] = ac[i4 + 2] = ac[i4 + 3] = a;
                }
            }
#pragma unroll
            for (int c = 0; c < VC; ++c) vcur[c] = b_[2 * TB * dkp + tt * cols + cl + c];
            float acc[VC];
#pragma unroll
            for (int c = 0; c < VC; ++c) {
                acc[c] = 0.f;
#pragma unroll
                for (int i = 0; i < SC_NK; ++i) {
                    S[c][i] = fmaf(ac[i], S[c][i], kc[i] * vcur[c]);
                    if (MODE == SC_FROM) acc[c] = fmaf(S[c][i], qc[i], acc[c]);
                }
            }
            if (MODE == SC_LOCAL) {
                aprod *= a;
                if (CH) {
#pragma unroll
                    for (int i = 0; i < SC_NK; ++i) aprodc[CH ? i : 0] *= ac[i];
                }
            } else {
                if (VC == 4 && KP >= 4) {
                    const float (&a4)[4] = reinterpret_cast<const float (&)[4]>(acc);
                    const float tot = sc_fold4(a4, kp, KP);
                    const int c = 2 * (kp & 1) + ((kp >> 1) & 1);
                    const float vsel = c == 0 ? vcur[0] : c == 1 ? vcur[VC > 1 ? 1 : 0] : c == 2 ? vcur[VC > 2 ? 2 : 0] : vcur[VC > 3 ? 3 : 0];
                    if (kp < 4 && vb + cl + c < dv)
                        o[(size_t)(tb + tt) * o_stride + (size_t)h * dv + vb + cl + c] = fmaf(skip, vsel, tot);
                } else {
#pragma unroll
                    for (int c = 0; c < VC; ++c) {
                        for (int off = 1; off < KP; off <<= 1) acc[c] += __shfl_xor(acc[c], off, 64);
                        if (kp == 0 && vb + cl + c < dv)
                            o[(size_t)(tb + tt) * o_stride + (size_t)h * dv + vb + cl + c] = fmaf(skip, vcur[c], acc[c]);
                    }
                }
            }
        }
        if (more) SCT_STORE(buf ^ 1)
        __syncthreads();
    }
#undef SCT_FETCH
#undef SCT_STORE
    if (MODE == SC_FROM) return;
#pragma unroll
    for (int c = 0; c < VC; ++c)
#pragma unroll
        for (int i = 0; i < SC_NK; ++i) {
            const int ki = kp * SC_NK + i, vc = vb + cl + c;
            if (vc < dv && ki < dk) st[(size_t)vc * dk + ki] = S[c][i];
        }
    if (CH) {
        if (blockIdx.x == 0 && threadIdx.x < KP)
#pragma unroll
            for (int i = 0; i < SC_NK; ++i) {
                const int ki = kp * SC_NK + i;
                if (ki < dk) ws_decay[((size_t)slot * heads + h) * dk + ki] = aprodc[CH ? i : 0];
            }
    } else if (blockIdx.x == 0 && threadIdx.x == 0) {
        ws_decay[(size_t)slot * heads + h] = aprod;
    }
}

// per (segment, head), piece after piece: ws_state[slot] <- the state at the piece's start; the pool gets the last state
__global__ void __launch_bounds__(256)
decay_scan_combine_kernel(float* __restrict__ ws_state, const float* __restrict__ ws_decay, float* __restrict__ pool,
                          const int* __restrict__ state_in, const int* __restrict__ state_out,
                          const int* __restrict__ seg_offsets, int heads, int hs, int piece, int dk_c) {
    const int r = blockIdx.z, h = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
    const int t0 = seg_offsets[r], len = seg_offsets[r + 1] - t0;
    if (len <= 0 || e >= hs) return;
    const int pieces = (len + piece - 1) / piece, base = t0 / piece + r;
    float S = pool[((size_t)state_in[r] * heads + h) * hs + e];
    for (int p = 0; p < pieces; ++p) {
        float* at = ws_state + ((size_t)(base + p) * heads + h) * hs + e;
        const float local = *at;
        *at = S;
        // (dk_c > 0: a product of decays per key channel, the fastest index of a head's state [dv][dk])
        const float a = dk_c > 0 ? ws_decay[((size_t)(base + p) * heads + h) * dk_c + e % dk_c] : ws_decay[(size_t)(base + p) * heads + h];
        S = fmaf(a, S, local);
    }
    pool[((size_t)state_out[r] * heads + h) * hs + e] = S;
}

extern "C" int ilm_decay_scan_max_dk() { return SC_NK * 64; }

// piece == 0: one pass, a block a (segment, head, columns).  piece > 0: segments in pieces of that many tokens (see
// above); ws_state holds (T / piece + R) * heads * dk * dv floats, ws_decay (T / piece + R) * heads.
extern "C" int ilm_decay_scan(void* o, int o_stride, const void* q, const void* k, int qk_stride, int q_div, const void* v,
                              int v_stride, const void* decay_h, const void* decay_t, const void* kscale_t,
                              const void* skip_h, void* pool, const void* state_in, const void* state_out,
                              const void* seg_offsets, int R, int heads, int dk, int dv, int T_, int piece, void* ws_state,
                              void* ws_decay, const void* decay_c, int dc_stride, hipStream_t stream) {
    ILM_REQUIRE(R > 0 && heads > 0 && dk > 0 && dv > 0 && T_ > 0, "decay_scan: bad sizes");
    if (decay_c != nullptr) {
        ILM_REQUIRE(decay_h == nullptr && decay_t == nullptr, "decay_scan: a decay per channel stands alone");
        ILM_REQUIRE(dc_stride >= heads * dk, "decay_scan: a decay per channel comes in rows of heads * dk");
    }
    ILM_REQUIRE(dk <= SC_NK * 64, "decay_scan: %d state entries a column, at most %d", dk, SC_NK * 64);
    ILM_REQUIRE(q_div > 0 && heads % q_div == 0, "decay_scan: %d heads do not divide into groups of %d", heads, q_div);
    ILM_REQUIRE(decay_c != nullptr || (decay_h != nullptr) != (decay_t != nullptr), "decay_scan: a decay per head or per token, one of them");
    ILM_REQUIRE(R <= 65535 && heads <= 65535, "decay_scan: too many requests or heads");
    ILM_REQUIRE(piece >= 0 && (piece == 0 || (ws_state != nullptr && ws_decay != nullptr)), "decay_scan: pieces need a workspace");
    int KP = 1;
    while (KP * SC_NK < dk) KP <<= 1;
    const int VT = 256 / KP;
#define SC_ARGS (float*)o, o_stride, (const float*)q, (const float*)k, qk_stride, q_div, (const float*)v, v_stride,              \
                (const float*)decay_h, (const float*)decay_t, (const float*)kscale_t, (const float*)skip_h, (float*)pool,        \
                (const int*)state_in, (const int*)state_out, (const int*)seg_offsets, heads, dk, dv, KP
    // four columns a thread where that still leaves two blocks a compute unit (long prompts in pieces, large batches):
    // a thread's loads of q and k then serve four columns; one column a thread where blocks are few (small batches)
    const int cus = ilm_num_cus();
    if (piece == 0 && decay_c != nullptr) {
        const int g4 = (dv + 4 * VT - 1) / (4 * VT);
        if ((long)g4 * heads * R >= 2L * cus && dv >= 4)
            decay_scan_kernel<4, true><<<dim3(g4, heads, R), 256, 0, stream>>>(SC_ARGS, (const float*)decay_c, dc_stride);
        else
            decay_scan_kernel<1, true><<<dim3((dv + VT - 1) / VT, heads, R), 256, 0, stream>>>(SC_ARGS, (const float*)decay_c, dc_stride);
        ILM_LAUNCH_CHECK("decay_scan (decay per channel)");
        return 0;
    }
    if (piece == 0) {
        const int g4 = (dv + 4 * VT - 1) / (4 * VT);
        if ((long)g4 * heads * R >= 2L * cus && dv >= 4) decay_scan_kernel<4><<<dim3(g4, heads, R), 256, 0, stream>>>(SC_ARGS);
        else decay_scan_kernel<1><<<dim3((dv + VT - 1) / VT, heads, R), 256, 0, stream>>>(SC_ARGS);
        ILM_LAUNCH_CHECK("decay_scan");
        return 0;
    }
    const int slots = T_ / piece + R;
    ILM_REQUIRE(slots <= 65535, "decay_scan: %d pieces in a step, at most 65535", slots);
    const int g4 = (dv + 4 * VT - 1) / (4 * VT);
    const bool four = (long)g4 * heads * (T_ / piece + 1) >= 2L * cus && dv >= 4;
    const int cols = VT * (four ? 4 : 1), dkp = KP * SC_NK;
    int TB = 16;
    while (TB > 1 && (TB * dkp > 2048 || TB * cols > 2048)) TB >>= 1;
    const size_t shm = (size_t)2 * TB * ((decay_c != nullptr ? 3 : 2) * dkp + cols + 2) * sizeof(float);
    ILM_REQUIRE(shm <= 64 * 1024, "decay_scan: a tile of %zu bytes does not fit LDS", shm);
    dim3 grid(four ? g4 : (dv + VT - 1) / VT, heads, slots);
#define SCT_ARGS (float*)o, o_stride, (const float*)q, (const float*)k, qk_stride, q_div, (const float*)v, v_stride,             \
                 (const float*)decay_h, (const float*)decay_t, (const float*)kscale_t, (const float*)skip_h,                    \
                 (const int*)seg_offsets, heads, dk, dv, KP, R, piece, TB, (float*)ws_state, (float*)ws_decay
    if (decay_c != nullptr) {
        if (four) decay_scan_tiled_kernel<SC_LOCAL, 4, true><<<grid, 256, shm, stream>>>(SCT_ARGS, (const float*)decay_c, dc_stride);
        else decay_scan_tiled_kernel<SC_LOCAL, 1, true><<<grid, 256, shm, stream>>>(SCT_ARGS, (const float*)decay_c, dc_stride);
    } else if (four) decay_scan_tiled_kernel<SC_LOCAL, 4><<<grid, 256, shm, stream>>>(SCT_ARGS);
    else decay_scan_tiled_kernel<SC_LOCAL, 1><<<grid, 256, shm, stream>>>(SCT_ARGS);
    ILM_LAUNCH_CHECK("decay_scan (local states)");
    decay_scan_combine_kernel<<<dim3((dk * dv + 255) / 256, heads, R), 256, 0, stream>>>(
        (float*)ws_state, (const float*)ws_decay, (float*)pool, (const int*)state_in, (const int*)state_out,
        (const int*)seg_offsets, heads, dk * dv, piece, decay_c != nullptr ? dk : 0);
    ILM_LAUNCH_CHECK("decay_scan (combine)");
    if (decay_c != nullptr) {
        if (four) decay_scan_tiled_kernel<SC_FROM, 4, true><<<grid, 256, shm, stream>>>(SCT_ARGS, (const float*)decay_c, dc_stride);
        else decay_scan_tiled_kernel<SC_FROM, 1, true><<<grid, 256, shm, stream>>>(SCT_ARGS, (const float*)decay_c, dc_stride);
    } else if (four) decay_scan_tiled_kernel<SC_FROM, 4><<<grid, 256, shm, stream>>>(SCT_ARGS);
    else decay_scan_tiled_kernel<SC_FROM, 1><<<grid, 256, shm, stream>>>(SCT_ARGS);
    ILM_LAUNCH_CHECK("decay_scan (outputs)");
#undef SCT_ARGS
#undef SC_ARGS
    return 0;
}

// ------------------------------------------------------------------------------------------
// RMS norm in groups with an optional gate, one wave (groups up to 512 elements) or one block a (row, group):
//   y = x * act(gate)            (gate_before)
//   y = y / sqrt(mean_group(y^2) + eps) * w       (w may be absent)
//   y = y * act(gate)            (otherwise)
// Sums run over a group in an order that depends on its size only.
// ------------------------------------------------------------------------------------------
template <int LANES>   // threads an item: 64 (four items a block) or 256
__global__ void __launch_bounds__(256)
group_norm_gate_kernel(void* __restrict__ out, const void* __restrict__ x, const void* __restrict__ gate,
                       const void* __restrict__ w, int rows, int n, int groups, int x_stride, int gate_stride,
                       int out_stride, float eps, int gate_act, int gate_before, int out_dt, int x_dt, int gate_dt, int w_dt,
                       int parts, size_t pstride) {
    __shared__ float red[4];
    const int item = LANES == 64 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
    const int lane = LANES == 64 ? (threadIdx.x & 63) : threadIdx.x;
    if (item >= rows * groups) return;     // (whole waves; with 256 lanes an item every block has one)
    const int t = item / groups, g = item % groups, gs = n / groups;
    const size_t xb = (size_t)t * x_stride + (size_t)g * gs, gb = (size_t)t * gate_stride + (size_t)g * gs;
    const size_t ob = (size_t)t * out_stride + (size_t)g * gs;
    const bool pre = gate != nullptr && gate_before;
    float ss = 0.f;
    for (int j = lane; j < gs; j += LANES) {
        float y = ldf(x, x_dt, xb + j);
        for (int p = 1; p < parts; ++p) y += ldf(x, x_dt, p * pstride + xb + j);
        if (pre) y *= act_f(ldf(gate, gate_dt, gb + j), gate_act);
        ss = fmaf(y, y, ss);
    }
    ss = LANES == 64 ? wave_sum(ss) : block_sum<4>(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int j = lane; j < gs; j += LANES) {
        float y = ldf(x, x_dt, xb + j);
        for (int p = 1; p < parts; ++p) y += ldf(x, x_dt, p * pstride + xb + j);
        if (pre) y *= act_f(ldf(gate, gate_dt, gb + j), gate_act);
        y *= rstd;
        if (w != nullptr) y *= ldf(w, w_dt, (size_t)g * gs + j);
        if (gate != nullptr && !gate_before) y *= act_f(ldf(gate, gate_dt, gb + j), gate_act);
        stf(out, out_dt, ob + j, y);
    }
}

// The same with eight elements a thread and the group in registers between the sum and the stores: groups in multiples
// of 8 up to 8 * LANES * NITER elements, rows 16 bytes aligned.
template <int LANES, int NITER>
__global__ void __launch_bounds__(256)
group_norm_gate_vec_kernel(void* __restrict__ out, const void* __restrict__ x, const void* __restrict__ gate,
                           const void* __restrict__ w, int rows, int n, int groups, int x_stride, int gate_stride,
                           int out_stride, float eps, int gate_act, int gate_before, int out_dt, int x_dt, int gate_dt, int w_dt,
                           int parts, size_t pstride) {
    __shared__ float red[4];
    const int item = LANES == 64 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
    const int lane = LANES == 64 ? (threadIdx.x & 63) : threadIdx.x;
    if (item >= rows * groups) return;
    const int t = item / groups, g = item % groups, gs = n / groups;
    const size_t xb = (size_t)t * x_stride + (size_t)g * gs, gb = (size_t)t * gate_stride + (size_t)g * gs;
    const size_t ob = (size_t)t * out_stride + (size_t)g * gs;
    const bool pre = gate != nullptr && gate_before;
    float v[NITER][8];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * LANES + lane) * 8;
        if (j < gs) {
            ld8(x, x_dt, xb + j, v[it]);
            for (int p = 1; p < parts; ++p) {
                float more[8];
                ld8(x, x_dt, p * pstride + xb + j, more);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[it][e] += more[e];
            }
            if (pre) {
                float gt[8];
                ld8(gate, gate_dt, gb + j, gt);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[it][e] *= act_f(gt[e], gate_act);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) ss = fmaf(v[it][e], v[it][e], ss);
        }
    }
    ss = LANES == 64 ? wave_sum(ss) : block_sum<4>(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)gs + eps);
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * LANES + lane) * 8;
        if (j < gs) {
            float o8[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o8[e] = v[it][e] * rstd;
            if (w != nullptr) {
                float wt[8];
                ld8(w, w_dt, (size_t)g * gs + j, wt);
#pragma unroll
                for (int e = 0; e < 8; ++e) o8[e] *= wt[e];
            }
            if (gate != nullptr && !gate_before) {
                float gt[8];
                ld8(gate, gate_dt, gb + j, gt);
#pragma unroll
                for (int e = 0; e < 8; ++e) o8[e] *= act_f(gt[e], gate_act);
            }
            st8(out, out_dt, ob + j, o8);
        }
    }
}

extern "C" int ilm_group_norm_gate(void* out, const void* x, const void* gate, const void* w, int rows, int n, int groups,
                                   int x_stride, int gate_stride, int out_stride, float eps, int gate_act, int gate_before,
                                   int out_dt, int x_dt, int gate_dt, int w_dt, int parts, long pstride, hipStream_t stream) {
    ILM_REQUIRE(parts >= 1, "group_norm_gate: %d parts", parts);
    ILM_REQUIRE(rows > 0 && n > 0 && groups > 0 && n % groups == 0, "group_norm_gate: %d elements do not divide into %d groups", n, groups);
    ILM_REQUIRE((long)rows * groups < (1L << 31) - 4, "group_norm_gate: too many rows");
    const int gs_ = n / groups;
    const bool al = gs_ % 8 == 0 && x_stride % 8 == 0 && out_stride % 8 == 0 && (gate == nullptr || gate_stride % 8 == 0) && pstride % 8 == 0
                    && (((uintptr_t)out | (uintptr_t)x | (uintptr_t)gate | (uintptr_t)w) & 15) == 0;
    if (al && gs_ <= 8192) {
#define GN_ARGS out, x, gate, w, rows, n, groups, x_stride, gate_stride, out_stride, eps, gate_act, gate_before, out_dt, x_dt, gate_dt, \
                w_dt, parts, (size_t)pstride
        if (gs_ <= 512) group_norm_gate_vec_kernel<64, 1><<<(rows * groups + 3) / 4, 256, 0, stream>>>(GN_ARGS);
        else if (gs_ <= 2048) group_norm_gate_vec_kernel<256, 1><<<rows * groups, 256, 0, stream>>>(GN_ARGS);
        else if (gs_ <= 4096) group_norm_gate_vec_kernel<256, 2><<<rows * groups, 256, 0, stream>>>(GN_ARGS);
        else group_norm_gate_vec_kernel<256, 4><<<rows * groups, 256, 0, stream>>>(GN_ARGS);
#undef GN_ARGS
        ILM_LAUNCH_CHECK("group_norm_gate");
        return 0;
    }
    if (n / groups > 512) {
        group_norm_gate_kernel<256><<<rows * groups, 256, 0, stream>>>(out, x, gate, w, rows, n, groups, x_stride, gate_stride,
                                                                       out_stride, eps, gate_act, gate_before, out_dt, x_dt, gate_dt, w_dt, parts, (size_t)pstride);
    } else {
        const int blocks = (int)(((long)rows * groups + 3) / 4);
        group_norm_gate_kernel<64><<<blocks, 256, 0, stream>>>(out, x, gate, w, rows, n, groups, x_stride, gate_stride, out_stride,
                                                               eps, gate_act, gate_before, out_dt, x_dt, gate_dt, w_dt, parts, (size_t)pstride);
    }
    ILM_LAUNCH_CHECK("group_norm_gate");
    return 0;
}

// ------------------------------------------------------------------------------------------
// A branch's output normed, added to the residual stream, and the stream normed for the next sublayer, in one pass:
//   r += alpha * (y / sqrt(mean(y^2) + eps_b) * wb);   x = r / sqrt(mean(r^2) + eps) * w
// One block a row; r is float, y and x have their own types.  Sums in an order that depends on the width only.
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
norm_add_norm_kernel(void* __restrict__ x, float* __restrict__ r, const void* __restrict__ y, const void* __restrict__ wb,
                     const void* __restrict__ w, int H, float alpha, float eps_b, float eps, int x_dt, int y_dt, int wb_dt, int w_dt,
                     int parts, size_t pstride) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * H;
    float ss = 0.f;
    for (int j = threadIdx.x; j < H; j += 256) {
        float v = ldf(y, y_dt, base + j);
        for (int p = 1; p < parts; ++p) v += ldf(y, y_dt, p * pstride + base + j);
        ss = fmaf(v, v, ss);
    }
    const float rb = alpha / sqrtf(block_sum<4>(ss, red) / (float)H + eps_b);
    ss = 0.f;
    for (int j = threadIdx.x; j < H; j += 256) {
        float yv = ldf(y, y_dt, base + j);
        for (int p = 1; p < parts; ++p) yv += ldf(y, y_dt, p * pstride + base + j);
        const float v = fmaf(yv * rb, ldf(wb, wb_dt, j), r[base + j]);
        r[base + j] = v;
        ss = fmaf(v, v, ss);
    }
    const float rs = 1.0f / sqrtf(block_sum<4>(ss, red) / (float)H + eps);
    for (int j = threadIdx.x; j < H; j += 256) stf(x, x_dt, base + j, r[base + j] * rs * ldf(w, w_dt, j));
}

// The same for widths that are multiples of 8 up to 8 * 256 * NITER: a thread keeps its pieces of the row in registers
// from the first sum to the last store, so y is read once, r read and written once, x written once.
template <int NITER>
__global__ void __launch_bounds__(256)
norm_add_norm_vec_kernel(void* __restrict__ x, float* __restrict__ r, const void* __restrict__ y, const void* __restrict__ wb,
                         const void* __restrict__ w, int H, float alpha, float eps_b, float eps, int x_dt, int y_dt, int wb_dt, int w_dt,
                         int parts, size_t pstride) {
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * H;
    float v[NITER][8];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * 256 + threadIdx.x) * 8;
        if (j < H) {
            ld8(y, y_dt, base + j, v[it]);
            for (int p = 1; p < parts; ++p) {      // the parts of a product that was split over K, summed in order
                float more[8];
                ld8(y, y_dt, p * pstride + base + j, more);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[it][e] += more[e];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) ss = fmaf(v[it][e], v[it][e], ss);
        }
    }
    const float rb = alpha / sqrtf(block_sum<4>(ss, red) / (float)H + eps_b);
    ss = 0.f;
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * 256 + threadIdx.x) * 8;
        if (j < H) {
            float g[8], q[8];
            ld8(wb, wb_dt, j, g);
            ld8(r, ILM_DTYPE_F32, base + j, q);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                v[it][e] = fmaf(v[it][e] * rb, g[e], q[e]);
                ss = fmaf(v[it][e], v[it][e], ss);
            }
            st8(r, ILM_DTYPE_F32, base + j, v[it]);
        }
    }
    const float rs = 1.0f / sqrtf(block_sum<4>(ss, red) / (float)H + eps);
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int j = (it * 256 + threadIdx.x) * 8;
        if (j < H) {
            float g[8], out[8];
            ld8(w, w_dt, j, g);
#pragma unroll
            for (int e = 0; e < 8; ++e) out[e] = v[it][e] * rs * g[e];
            st8(x, x_dt, base + j, out);
        }
    }
}

extern "C" int ilm_norm_add_norm(void* x, void* r, const void* y, const void* wb, const void* w, int rows, int H, float alpha,
                                 float eps_b, float eps, int x_dt, int y_dt, int wb_dt, int w_dt, int parts, long pstride,
                                 hipStream_t stream) {
    ILM_REQUIRE(rows > 0 && H > 0 && parts >= 1, "norm_add_norm: bad sizes");
    const bool al = pstride % 8 == 0 && (((uintptr_t)x | (uintptr_t)r | (uintptr_t)y | (uintptr_t)wb | (uintptr_t)w) & 15) == 0;
    if (al && H % 8 == 0 && H <= 8192) {
#define NAN_ARGS x, (float*)r, y, wb, w, H, alpha, eps_b, eps, x_dt, y_dt, wb_dt, w_dt, parts, (size_t)pstride
        if (H <= 2048) norm_add_norm_vec_kernel<1><<<rows, 256, 0, stream>>>(NAN_ARGS);
        else if (H <= 4096) norm_add_norm_vec_kernel<2><<<rows, 256, 0, stream>>>(NAN_ARGS);
        else norm_add_norm_vec_kernel<4><<<rows, 256, 0, stream>>>(NAN_ARGS);
#undef NAN_ARGS
        ILM_LAUNCH_CHECK("norm_add_norm");
        return 0;
    }
    norm_add_norm_kernel<<<rows, 256, 0, stream>>>(x, (float*)r, y, wb, w, H, alpha, eps_b, eps, x_dt, y_dt, wb_dt, w_dt, parts,
                                                   (size_t)pstride);
    ILM_LAUNCH_CHECK("norm_add_norm");
    return 0;
}

// ------------------------------------------------------------------------------------------
// Short causal convolution over the tokens of each request, per channel, with bias and activation:
//   y[t, c] = act(b[c] + sum_i w[c, i] * x[t - (taps - 1) + i, c]),   the last tap is the token's own input.
// Inputs before a request's first token of this step come from its state row (the last taps - 1 inputs of the
// steps before, oldest first; zeros for a new request).  One thread a (token, channel); a second launch, one thread a
// (request, channel), then writes the state row anew from the old row and the step's inputs (it reads what it
// overwrites into registers first, and no other thread touches its entries).
// ------------------------------------------------------------------------------------------
#define CV_MAX_TAPS 8

__global__ void __launch_bounds__(256)
causal_conv_kernel(float* __restrict__ y, const void* __restrict__ x, const void* __restrict__ w, const void* __restrict__ b,
                   const float* __restrict__ pool, const int* __restrict__ state_in, const int* __restrict__ seg_of_token,
                   const int* __restrict__ seg_offsets, int C, int taps, int x_stride, int y_stride, int act, int x_dt, int w_dt,
                   int t_first) {
    const int t = t_first + blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int r = seg_of_token[t];
    const int j = t - seg_offsets[r];                       // the token's place in its segment
    const size_t sin = (size_t)state_in[r] * (taps - 1) * C;
    float s = b != nullptr ? ldf(b, w_dt, c) : 0.f;
#pragma unroll
    for (int i = 0; i < CV_MAX_TAPS; ++i) {
        if (i < taps) {
            const int back = taps - 1 - i;                  // tap i reads the input `back` tokens before
            const float xv = back <= j ? ldf(x, x_dt, (size_t)(t - back) * x_stride + c)
                                       : pool[sin + (size_t)(taps - 1 - (back - j)) * C + c];
            s = fmaf(ldf(w, w_dt, (size_t)c * taps + i), xv, s);
        }
    }
    y[(size_t)t * y_stride + c] = act_f(s, act);
}

// Eight channels a thread (16-byte loads of the inputs, 32-byte stores): channels and the row stride in multiples of 8,
// bfloat16 inputs, rows 16 bytes aligned.  The taps of a thread's eight channels are 8 * taps consecutive weights.
template <int TAPS>
__global__ void __launch_bounds__(256)
causal_conv_vec_kernel(float* __restrict__ y, const uint16_t* __restrict__ x, const void* __restrict__ w, const void* __restrict__ b,
                       const float* __restrict__ pool, const int* __restrict__ state_in, const int* __restrict__ seg_of_token,
                       const int* __restrict__ seg_offsets, int C, int taps, int x_stride, int y_stride, int act, int w_dt,
                       int t_first) {
    const int t = t_first + blockIdx.y, c = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (c >= C) return;
    const int r = seg_of_token[t];
    const int j = t - seg_offsets[r];
    const size_t sin = (size_t)state_in[r] * (taps - 1) * C;
    float s[8], wt[TAPS][8];     // wt[m][.]: the weights c * TAPS + 8 m ... of the thread's 8 * TAPS consecutive ones
    if (b != nullptr) ld8(b, w_dt, c, s);
    else {
#pragma unroll
        for (int e = 0; e < 8; ++e) s[e] = 0.f;
    }
#pragma unroll
    for (int m = 0; m < TAPS; ++m) ld8(w, w_dt, (size_t)c * TAPS + 8 * m, wt[m]);
#pragma unroll
    for (int i = 0; i < TAPS; ++i) {
        const int back = TAPS - 1 - i;
        float xv[8];
        if (back <= j) ld8(x, ILM_DTYPE_BF16, (size_t)(t - back) * x_stride + c, xv);
        else ld8(pool, ILM_DTYPE_F32, sin + (size_t)(TAPS - 1 - (back - j)) * C + c, xv);
#pragma unroll
        for (int e = 0; e < 8; ++e) s[e] = fmaf(wt[(e * TAPS + i) / 8][(e * TAPS + i) % 8], xv[e], s[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] = act_f(s[e], act);
    st8(y, ILM_DTYPE_F32, (size_t)t * y_stride + c, s);
}

__global__ void __launch_bounds__(256)
causal_conv_state_kernel(const void* __restrict__ x, float* __restrict__ pool, const int* __restrict__ state_in,
                         const int* __restrict__ state_out, const int* __restrict__ seg_offsets, int C, int taps,
                         int x_stride, int x_dt) {
    const int r = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int t0 = seg_offsets[r], len = seg_offsets[r + 1] - t0;
    if (len <= 0) return;
    const size_t sin = (size_t)state_in[r] * (taps - 1) * C, sout = (size_t)state_out[r] * (taps - 1) * C;
    float win[CV_MAX_TAPS];
#pragma unroll
    for (int i = 0; i < CV_MAX_TAPS; ++i) {
        // entry i of the new row: the input taps - 1 - i tokens before the segment's end
        const int back = taps - 1 - i;
        win[i] = 0.f;
        if (i < taps - 1) win[i] = back <= len ? ldf(x, x_dt, (size_t)(t0 + len - back) * x_stride + c)
                                               : pool[sin + (size_t)(i + len) * C + c];
    }
#pragma unroll
    for (int i = 0; i < CV_MAX_TAPS; ++i)
        if (i < taps - 1) pool[sout + (size_t)i * C + c] = win[i];
}

extern "C" int ilm_causal_conv_max_taps() { return CV_MAX_TAPS; }

extern "C" int ilm_causal_conv(void* y, const void* x, const void* w, const void* b, void* pool, const void* state_in,
                               const void* state_out, const void* seg_of_token, const void* seg_offsets, int T_, int R, int C,
                               int taps, int x_stride, int y_stride, int act, int x_dt, int w_dt, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && R > 0 && C > 0 && R <= 65535, "causal_conv: bad sizes");
    ILM_REQUIRE(taps >= 1 && taps <= CV_MAX_TAPS, "causal_conv: %d taps, at most %d", taps, CV_MAX_TAPS);
    // (few rows, decoded tokens: one channel a thread gives more blocks and measured faster: 5.4 against 6.9 us at 64 rows)
    const bool vec = T_ >= 256 && taps >= 2 && taps <= 4 && ((uintptr_t)w & 15) == 0 && x_dt == ILM_DTYPE_BF16 && C % 8 == 0 && x_stride % 8 == 0 && y_stride % 8 == 0
                     && (((uintptr_t)x | (uintptr_t)y | (uintptr_t)pool | (uintptr_t)b) & 15) == 0;
    for (int t0 = 0; vec && t0 < T_; t0 += 65535) {
        const int rows = T_ - t0 < 65535 ? T_ - t0 : 65535;
#define CV_ARGS (float*)y, (const uint16_t*)x, w, b, (const float*)pool, (const int*)state_in, (const int*)seg_of_token,   \
                (const int*)seg_offsets, C, taps, x_stride, y_stride, act, w_dt, t0
        const dim3 vg((C / 8 + 255) / 256, rows);
        if (taps == 2) causal_conv_vec_kernel<2><<<vg, 256, 0, stream>>>(CV_ARGS);
        else if (taps == 3) causal_conv_vec_kernel<3><<<vg, 256, 0, stream>>>(CV_ARGS);
        else causal_conv_vec_kernel<4><<<vg, 256, 0, stream>>>(CV_ARGS);
#undef CV_ARGS
    }
    for (int t0 = 0; !vec && t0 < T_; t0 += 65535) {
        const int rows = T_ - t0 < 65535 ? T_ - t0 : 65535;
        causal_conv_kernel<<<dim3((C + 255) / 256, rows), 256, 0, stream>>>(
            (float*)y, x, w, b, (const float*)pool, (const int*)state_in, (const int*)seg_of_token, (const int*)seg_offsets, C, taps,
            x_stride, y_stride, act, x_dt, w_dt, t0);
    }
    ILM_LAUNCH_CHECK("causal_conv");
    if (taps > 1) {
        causal_conv_state_kernel<<<dim3((C + 255) / 256, R), 256, 0, stream>>>(x, (float*)pool, (const int*)state_in,
                                                                                (const int*)state_out, (const int*)seg_offsets, C,
                                                                                taps, x_stride, x_dt);
        ILM_LAUNCH_CHECK("causal_conv_state");
    }
    return 0;
}

// ------------------------------------------------------------------------------------------
// Step sizes and decays of a selective state space: dt = softplus(raw + bias[h]), decay = exp(-exp(A_log[h]) dt).
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
ssm_steps_kernel(float* __restrict__ dt, float* __restrict__ decay, const void* __restrict__ raw,
                 const float* __restrict__ bias, const float* __restrict__ a_log, int T_, int heads, int raw_stride, int raw_dt) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= T_ * heads) return;
    const int t = i / heads, h = i % heads;
    const float z = ldf(raw, raw_dt, (size_t)t * raw_stride + h) + bias[h];
    const float d = z > 20.0f ? z : log1pf(expf(z));
    dt[i] = d;
    decay[i] = expf(-expf(a_log[h]) * d);
}

extern "C" int ilm_ssm_steps(void* dt, void* decay, const void* raw, const void* bias, const void* a_log, int T_, int heads,
                             int raw_stride, int raw_dt, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && heads > 0, "ssm_steps: bad sizes");
    ssm_steps_kernel<<<(T_ * heads + 255) / 256, 256, 0, stream>>>((float*)dt, (float*)decay, raw, (const float*)bias,
                                                                   (const float*)a_log, T_, heads, raw_stride, raw_dt);
    ILM_LAUNCH_CHECK("ssm_steps");
    return 0;
}

// ------------------------------------------------------------------------------------------
// Queries and keys of unit root mean square with a temperature on the queries, inside the fused projection
// rows [T, (nh + 2 nkv) d], and k, v into the paged cache (keys [pages, nkv, page, d], values [pages, nkv, d, page]).
// A head has `dn` entries that count (the rest up to d are zeros that only fill the head up):
//   q <- q / sqrt(sum(q^2) / dn + eps) * (1 + coef * ln(floor((pos + 1) / every) + 1)),  k <- k / sqrt(sum(k^2) / dn + eps).
// normed == 0: no division.  every <= 0: no temperature.  One wave a (token, head).
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(64)
unit_qk_kvwrite_kernel(T* __restrict__ qkv, const int* __restrict__ pos, T* __restrict__ kc, T* __restrict__ vc,
                       const int* __restrict__ slots, int nh, int nkv, int d, int dn, int row_stride, int page, int normed,
                       float eps, float coef, int every) {
    const int t = blockIdx.x, hs = blockIdx.y, lane = threadIdx.x;
    T* p = qkv + (size_t)t * row_stride + (size_t)hs * d;
    const int slot = slots != nullptr ? slots[t] : -1;
    if (hs >= nh + nkv) {
        if (slot >= 0) {
            T* vdst = vc + ((size_t)(slot / page) * nkv + (hs - nh - nkv)) * d * page + (slot % page);
            for (int i = lane; i < d; i += 64) vdst[(size_t)i * page] = p[i];
        }
        return;
    }
    const bool is_k = hs >= nh;
    float f = 1.0f;
    if (normed) {
        float ss = 0.f;
        for (int i = lane; i < d; i += 64) {
            const float x = to_f32(p[i]);
            ss = fmaf(x, x, ss);
        }
        f = 1.0f / sqrtf(wave_sum(ss) / (float)dn + eps);
    }
    if (!is_k && every > 0) f *= 1.0f + coef * logf((float)((pos[t] + 1) / every) + 1.0f);
    T* dst = (is_k && slot >= 0) ? kc + (((size_t)(slot / page) * nkv + (hs - nh)) * page + (slot % page)) * d : nullptr;
    for (int i = lane; i < d; i += 64) {
        const T y = from_f32<T>(to_f32(p[i]) * f);
        p[i] = y;
        if (dst != nullptr) dst[i] = y;
    }
}

extern "C" int ilm_unit_qk_kvwrite(void* qkv, const void* pos, void* kc, void* vc, const void* slots, int T_, int nh, int nkv,
                                   int d, int dn, int row_stride, int page, int normed, float eps, float coef, int every,
                                   int dtype, hipStream_t stream) {
    ILM_REQUIRE(T_ > 0 && nh > 0 && nkv > 0 && d > 0 && dn > 0 && dn <= d, "unit_qk_kvwrite: bad sizes");
    ILM_REQUIRE(nh + 2 * nkv <= 65535, "unit_qk_kvwrite: too many heads");
    ILM_REQUIRE(slots == nullptr || (kc != nullptr && vc != nullptr && page > 0), "unit_qk_kvwrite: slots without a cache");
    dim3 grid(T_, nh + 2 * nkv);
    if (dtype == ILM_DTYPE_F32)
        unit_qk_kvwrite_kernel<float><<<grid, 64, 0, stream>>>((float*)qkv, (const int*)pos, (float*)kc, (float*)vc,
                                                              (const int*)slots, nh, nkv, d, dn, row_stride, page, normed, eps,
                                                              coef, every);
    else if (dtype == ILM_DTYPE_BF16)
        unit_qk_kvwrite_kernel<bf16><<<grid, 64, 0, stream>>>((bf16*)qkv, (const int*)pos, (bf16*)kc, (bf16*)vc,
                                                             (const int*)slots, nh, nkv, d, dn, row_stride, page, normed, eps,
                                                             coef, every);
    else
        ILM_REQUIRE(false, "unit_qk_kvwrite: unknown dtype %d", dtype);
    ILM_LAUNCH_CHECK("unit_qk_kvwrite");
    return 0;
}

// ------------------------------------------------------------------------------------------
// out = a x + b y, element by element (the branches of a mixer that runs two side by side)
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
weighted_sum_kernel(void* __restrict__ out, const void* __restrict__ x, const void* __restrict__ y, long n, float a, float b,
                    int out_dt, int x_dt, int y_dt) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    stf(out, out_dt, i, fmaf(a, ldf(x, x_dt, i), b * ldf(y, y_dt, i)));
}

__global__ void __launch_bounds__(256)
weighted_sum_vec_kernel(void* __restrict__ out, const void* __restrict__ x, const void* __restrict__ y, long n, float a, float b,
                        int out_dt, int x_dt, int y_dt) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= n) return;
    float p[8], q[8], r[8];
    ld8(x, x_dt, i, p);
    ld8(y, y_dt, i, q);
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = fmaf(a, p[e], b * q[e]);
    st8(out, out_dt, i, r);
}

extern "C" int ilm_weighted_sum(void* out, const void* x, const void* y, long n, float a, float b, int out_dt, int x_dt,
                                int y_dt, hipStream_t stream) {
    ILM_REQUIRE(n > 0 && (n + 255) / 256 < (1L << 31), "weighted_sum: bad size");
    if (n % 8 == 0 && (((uintptr_t)out | (uintptr_t)x | (uintptr_t)y) & 15) == 0) {
        weighted_sum_vec_kernel<<<(unsigned)((n / 8 + 255) / 256), 256, 0, stream>>>(out, x, y, n, a, b, out_dt, x_dt, y_dt);
        ILM_LAUNCH_CHECK("weighted_sum");
        return 0;
    }
    weighted_sum_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(out, x, y, n, a, b, out_dt, x_dt, y_dt);
    ILM_LAUNCH_CHECK("weighted_sum");
    return 0;
}
