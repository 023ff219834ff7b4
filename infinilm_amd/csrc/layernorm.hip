// Sum of everything that is due to the residual stream, and a layer norm of the result, in one pass over a row:
//   r += sum_i scale_i * a_i        (r float, in place; up to LN_MAX_ADD addends)
//   x = (r - mean(r)) / sqrt(mean((r - mean)^2) + eps) * w + b
// An addend is [rows, H] in float or bfloat16, possibly as float parts [P, rows, H] of a product that was split
// over K (summed in order), or one row [H] that is added to every row (row stride 0).  Without w the kernel
// only sums.  One block a row; the row stays in LDS between the three passes (sum, deviations, result), so the
// variance is the mean of the squared deviations from the mean, not a difference of sums.  Sums run in an order
// that depends on H only.
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

template <typename TO, typename TW>
__global__ void __launch_bounds__(256)
add_layernorm_kernel(TO* __restrict__ x, float* __restrict__ r, LnAddends a, const TW* __restrict__ w,
                     const TW* __restrict__ b, int H, float eps) {
    extern __shared__ float row[];
    __shared__ float red[4];
    const int t = blockIdx.x;
    float* rr = r + (size_t)t * H;
    float s = 0.f;
    for (int j = threadIdx.x; j < H; j += 256) {
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
    if (w == nullptr) return;
    const float mean = block_sum<4>(s, red) / (float)H;
    float q = 0.f;
    for (int j = threadIdx.x; j < H; j += 256) {
        const float d = row[j] - mean;
        q = fmaf(d, d, q);
    }
    const float rstd = 1.0f / sqrtf(block_sum<4>(q, red) / (float)H + eps);
    TO* xr = x + (size_t)t * H;
    for (int j = threadIdx.x; j < H; j += 256) {
        const float y = (row[j] - mean) * rstd * to_f32(w[j]) + (b != nullptr ? to_f32(b[j]) : 0.f);
        xr[j] = from_f32<TO>(y);
    }
}

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
#define LN_LAUNCH(TO_, TW_)                                                                                     \
    add_layernorm_kernel<TO_, TW_><<<rows, 256, shm, stream>>>((TO_*)x, (float*)r, a, (const TW_*)w, (const TW_*)b, H, eps)
    if (w == nullptr) LN_LAUNCH(float, float);
    else if (out_dt == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_F32) LN_LAUNCH(float, float);
    else if (out_dt == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_BF16) LN_LAUNCH(bf16, bf16);
    else if (out_dt == ILM_DTYPE_BF16 && w_dt == ILM_DTYPE_F32) LN_LAUNCH(bf16, float);
    else if (out_dt == ILM_DTYPE_F32 && w_dt == ILM_DTYPE_BF16) LN_LAUNCH(float, bf16);
    else ILM_REQUIRE(false, "add_layernorm: unknown dtypes %d / %d", out_dt, w_dt);
#undef LN_LAUNCH
    ILM_LAUNCH_CHECK("add_layernorm");
    return 0;
}
