// Sum of everything that is due to the residual stream, and a layer norm of the result, in one pass over a row:
//   r += sum_i scale_i * a_i        (r float, in place; up to LN_MAX_ADD addends)
//   x = (r - mean(r)) / sqrt(mean((r - mean)^2) + eps) * w + b
// An addend is [rows, H] in float or bfloat16, possibly as float parts [P, rows, H] of a product that was split
// over K (summed in order), or one row [H] that is added to every row (row stride 0).  Without w the kernel
// only sums.  One block a row; the row stays in LDS between the three passes (sum, deviations, result), so the
// variance is the mean of the squared deviations from the mean, not a difference of sums.
#include "common.h"

#define LN_MAX_ADD 4

struct LnAddends {
    const void* p[LN_MAX_ADD];
    long pstride[LN_MAX_ADD];   // elements between parts
    long rstride[LN_MAX_ADD];   // elements between rows (0: one row for all)
    float scale[LN_MAX_ADD];
    int dt[LN_MAX_ADD];
    int parts[LN_MAX_ADD];
    int n;
};

__device__ __forceinline__ float ln_load(const void* p, int dt, size_t i) {
    return dt == ILM_DTYPE_F32 ? ((const float*)p)[i] : to_f32(((const bf16*)p)[i]);
}

__device__ __forceinline__ float4 ln_load4(const void* p, int dt, size_t i) {
    if (dt == ILM_DTYPE_F32) return *reinterpret_cast<const float4*>((const float*)p + i);
    const uint2 t = *reinterpret_cast<const uint2*>((const bf16*)p + i);
    return make_float4(__uint_as_float(t.x << 16), __uint_as_float(t.x & 0xffff0000u), __uint_as_float(t.y << 16),
                       __uint_as_float(t.y & 0xffff0000u));
}
template <typename T>
__device__ __forceinline__ float4 ln_get4(const T* p) { return ln_load4(p, sizeof(T) == 4 ? ILM_DTYPE_F32 : ILM_DTYPE_BF16, 0); }
__device__ __forceinline__ void ln_put4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void ln_put4(bf16* p, float4 v) {
    const bf16 a = from_f32<bf16>(v.x), b = from_f32<bf16>(v.y), c = from_f32<bf16>(v.z), d = from_f32<bf16>(v.w);
    *reinterpret_cast<uint2*>(p) = make_uint2((uint32_t)a.bits | ((uint32_t)b.bits << 16), (uint32_t)c.bits | ((uint32_t)d.bits << 16));
}

// NT threads a row: 256, or 1024 for wide rows in steps of up to LN_WIDE_ROWS rows (few rows of a block each would leave
// most of the chip idle).  VEC: four elements a thread and access (H, the strides and the parts' distances multiples of 4,
// everything 16 bytes aligned).  The order of a row's sums follows H, NT and VEC: a wide row's mean and variance may round
// differently in a step of few rows and in one of many (float rounding, both modes).
template <typename TO, typename TW, int NT, bool VEC>
__global__ void __launch_bounds__(NT)
add_layernorm_kernel(TO* __restrict__ x, float* __restrict__ r, LnAddends a, const TW* __restrict__ w,
                     const TW* __restrict__ b, int H, float eps) {
    extern __shared__ float row[];
    __shared__ float red[NT / 64];
    const int t = blockIdx.x;
    float* rr = r + (size_t)t * H;
    float s = 0.f;
    if (VEC) {
        for (int j = threadIdx.x * 4; j < H; j += NT * 4) {
            float4 v = *reinterpret_cast<const float4*>(rr + j);
            for (int i = 0; i < a.n; ++i) {
                float4 u = make_float4(0.f, 0.f, 0.f, 0.f);
                for (int p = 0; p < a.parts[i]; ++p) {
                    const float4 q = ln_load4(a.p[i], a.dt[i], (size_t)p * a.pstride[i] + (size_t)t * a.rstride[i] + j);
                    u.x += q.x; u.y += q.y; u.z += q.z; u.w += q.w;
                }
                v.x = fmaf(a.scale[i], u.x, v.x); v.y = fmaf(a.scale[i], u.y, v.y);
                v.z = fmaf(a.scale[i], u.z, v.z); v.w = fmaf(a.scale[i], u.w, v.w);
            }
            if (a.n > 0) *reinterpret_cast<float4*>(rr + j) = v;
            *reinterpret_cast<float4*>(row + j) = v;
            s += (v.x + v.y) + (v.z + v.w);
        }
    } else {
        for (int j = threadIdx.x; j < H; j += NT) {
            float v = rr[j];
            for (int i = 0; i < a.n; ++i) {
                float u = 0.f;
                for (int p = 0; p < a.parts[i]; ++p) u += ln_load(a.p[i], a.dt[i], (size_t)p * a.pstride[i] + (size_t)t * a.rstride[i] + j);
                v = fmaf(a.scale[i], u, v);
            }
            if (a.n > 0) rr[j] = v;
            row[j] = v;
            s += v;
        }
    }
    if (w == nullptr) return;
    const float mean = block_sum<NT / 64>(s, red) / (float)H;
    float q = 0.f;
    for (int j = threadIdx.x; j < H; j += NT) {
        const float d = row[j] - mean;
        q = fmaf(d, d, q);
    }
    const float rstd = 1.0f / sqrtf(block_sum<NT / 64>(q, red) / (float)H + eps);
    TO* xr = x + (size_t)t * H;
    if (VEC) {
        for (int j = threadIdx.x * 4; j < H; j += NT * 4) {
            const float4 v = *reinterpret_cast<const float4*>(row + j), ww = ln_get4(w + j);
            const float4 bb = b != nullptr ? ln_get4(b + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            ln_put4(xr + j, make_float4((v.x - mean) * rstd * ww.x + bb.x, (v.y - mean) * rstd * ww.y + bb.y,
                                        (v.z - mean) * rstd * ww.z + bb.z, (v.w - mean) * rstd * ww.w + bb.w));
        }
    } else {
        for (int j = threadIdx.x; j < H; j += NT) {
            const float y = (row[j] - mean) * rstd * to_f32(w[j]) + (b != nullptr ? to_f32(b[j]) : 0.f);
            xr[j] = from_f32<TO>(y);
        }
    }
}

#define LN_WIDE_ROWS 512

extern "C" int ilm_add_layernorm_max_addends() { return LN_MAX_ADD; }

// x: [rows, H] of out_dt (ignored without w); r: float [rows, H]; w, b: [H] of w_dt (b may be null)
extern "C" int ilm_add_layernorm(void* x, void* r, const void* w, const void* b, int rows, int H, float eps, int out_dt,
                                 int w_dt, int n_add,
                                 const void* p0, int dt0, int parts0, long ps0, long rs0, float sc0,
                                 const void* p1, int dt1, int parts1, long ps1, long rs1, float sc1,
                                 const void* p2, int dt2, int parts2, long ps2, long rs2, float sc2,
                                 const void* p3, int dt3, int parts3, long ps3, long rs3, float sc3, hipStream_t stream) {
    ILM_REQUIRE(rows > 0 && H > 0 && H <= 16384, "add_layernorm: bad sizes rows=%d H=%d", rows, H);
    ILM_REQUIRE(n_add >= 0 && n_add <= LN_MAX_ADD, "add_layernorm: %d addends, at most %d", n_add, LN_MAX_ADD);
    LnAddends a;
    const void* ps[4] = {p0, p1, p2, p3};
    const int dts[4] = {dt0, dt1, dt2, dt3}, parts[4] = {parts0, parts1, parts2, parts3};
    const long pss[4] = {ps0, ps1, ps2, ps3}, rss[4] = {rs0, rs1, rs2, rs3};
    const float scs[4] = {sc0, sc1, sc2, sc3};
    a.n = n_add;
    for (int i = 0; i < LN_MAX_ADD; ++i) {
        a.p[i] = ps[i]; a.dt[i] = dts[i]; a.parts[i] = parts[i]; a.pstride[i] = pss[i]; a.rstride[i] = rss[i]; a.scale[i] = scs[i];
        if (i < n_add) {
            ILM_REQUIRE(ps[i] != nullptr && parts[i] >= 1, "add_layernorm: addend %d is empty", i);
            ILM_REQUIRE(dts[i] == ILM_DTYPE_F32 || dts[i] == ILM_DTYPE_BF16, "add_layernorm: addend %d has unknown dtype %d", i, dts[i]);
        }
    }
    const size_t shm = (size_t)H * sizeof(float);
    bool vec = H % 4 == 0 && ((uintptr_t)r & 15) == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)b & 15) == 0;
    for (int i = 0; i < n_add; ++i)
        vec = vec && ((uintptr_t)ps[i] & 15) == 0 && pss[i] % 4 == 0 && rss[i] % 4 == 0;
    const bool wide = rows <= LN_WIDE_ROWS && H >= 1024;
#define LN_LAUNCH_NV(TO_, TW_, NT_, VEC_)                                                                        \
    add_layernorm_kernel<TO_, TW_, NT_, VEC_><<<rows, NT_, shm, stream>>>((TO_*)x, (float*)r, a, (const TW_*)w, (const TW_*)b, H, eps)
#define LN_LAUNCH(TO_, TW_)                                                                                      \
    {                                                                                                            \
        if (wide) { if (vec) LN_LAUNCH_NV(TO_, TW_, 1024, true); else LN_LAUNCH_NV(TO_, TW_, 1024, false); }     \
        else { if (vec) LN_LAUNCH_NV(TO_, TW_, 256, true); else LN_LAUNCH_NV(TO_, TW_, 256, false); }            \
    }
    if (w == nullptr) LN_LAUNCH(float, float)
    else if (out_dt == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) LN_LAUNCH(float, float)
    else if (out_dt == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) LN_LAUNCH(bf16, bf16)
    else if (out_dt == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) LN_LAUNCH(bf16, float)
    else if (out_dt == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_BF16) LN_LAUNCH(float, bf16)
    else ILM_REQUIRE(false, "add_layernorm: unknown dtypes %d / %d", out_dt, w_dt);
#undef LN_LAUNCH
#undef LN_LAUNCH_NV
    ILM_LAUNCH_CHECK("add_layernorm");
    return 0;
}
