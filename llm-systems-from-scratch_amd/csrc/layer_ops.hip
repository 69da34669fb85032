// The two fused elementwise/normalisation ops that sit next to attention in a transformer
// block: RMSNorm forward (optionally fused with the residual add in front of it) and
// silu(gate) * up.  Both are streaming kernels: HBM-bound, 16-byte accesses, fp32 math,
// one rounding to bf16 per stored value.
#include "common.hpp"
#include "launch.hpp"

namespace mi355 {

struct RmsNormParams {
    const __bf16* x;
    const __bf16* residual;      // optional: h = bf16(x + residual) is normalised instead of x
    const void* weight;          // bf16 or fp32 (n_cols)
    __bf16* y;
    __bf16* sum_out;             // optional (with residual): receives h
    float* rstd_out;             // optional (n_rows)
    int64_t n_rows;
    int64_t xs, rs, ys, ss;      // row strides in elements
    int n_cols;
    float eps;
    bool weight_fp32;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ void load_weight8(const RmsNormParams& p, int col, float (&w)[8]) {
    if (p.weight_fp32) {
        const f32x4* wp = reinterpret_cast<const f32x4*>(static_cast<const float*>(p.weight) + col);
        const f32x4 a = wp[0], b = wp[1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            w[e] = a[e];
            w[4 + e] = b[e];
        }
    } else {
        const bf16x8 a = as_bf16x8(*reinterpret_cast<const u32x4*>(static_cast<const __bf16*>(p.weight) + col));
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = (float)a[e];
    }
}

// One wavefront per row, the row held in registers: NCHUNK chunks of 512 elements (8 per lane).
// Requires n_cols % 8 == 0, n_cols <= 512 * NCHUNK, 16-byte aligned rows.
// The occupancy attribute caps the registers at 128: without it the compiler hoists every weight load
// of the 8-chunk instance (232 registers, two wavefronts per SIMD) and the kernel streams 15 % slower.
template <int NCHUNK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8))) void rms_norm_rows_kernel(RmsNormParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.n_rows) return;
    const __bf16* xr = p.x + row * p.xs;
    const __bf16* rr = p.residual ? p.residual + row * p.rs : nullptr;
    u32x4 raw[NCHUNK];
    float ssq = 0.f;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
        const int col = c * 512 + lane * 8;
        raw[c] = u32x4{0u, 0u, 0u, 0u};
        if (col < p.n_cols) {
            raw[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xr + col));
            if (rr) {
                const u32x4 rw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rr + col));
                const bf16x8 a = as_bf16x8(raw[c]), b = as_bf16x8(rw);
                u32x4 s;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s[e] = pack_bf16((float)a[2 * e] + (float)b[2 * e], (float)a[2 * e + 1] + (float)b[2 * e + 1]);
                raw[c] = s;
                if (p.sum_out) __builtin_nontemporal_store(s, reinterpret_cast<u32x4*>(p.sum_out + row * p.ss + col));
            }
            const bf16x8 v = as_bf16x8(raw[c]);
#pragma unroll
            for (int e = 0; e < 8; ++e) ssq += (float)v[e] * (float)v[e];
        }
    }
    ssq = wave_sum(ssq);
    const float rstd = 1.0f / sqrtf(ssq / (float)p.n_cols + p.eps);
    if (p.rstd_out && lane == 0) p.rstd_out[row] = rstd;
    __bf16* yr = p.y + row * p.ys;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
        const int col = c * 512 + lane * 8;
        if (col < p.n_cols) {
            float w[8];
            load_weight8(p, col, w);
            const bf16x8 v = as_bf16x8(raw[c]);
            u32x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                o[e] = pack_bf16(w[2 * e] * ((float)v[2 * e] * rstd), w[2 * e + 1] * ((float)v[2 * e + 1] * rstd));
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(yr + col));
        }
    }
}

// Any n_cols, any alignment: one wavefront per row, two passes over the row, scalar accesses.
__global__ __launch_bounds__(256) void rms_norm_generic_kernel(RmsNormParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= p.n_rows) return;
    const __bf16* xr = p.x + row * p.xs;
    const __bf16* rr = p.residual ? p.residual + row * p.rs : nullptr;
    __bf16* sr = (rr && p.sum_out) ? p.sum_out + row * p.ss : nullptr;
    float ssq = 0.f;
    for (int col = lane; col < p.n_cols; col += 64) {
        float v = (float)xr[col];
        if (rr) {
            v = (float)(__bf16)(v + (float)rr[col]);
            if (sr) sr[col] = (__bf16)v;
        }
        ssq += v * v;
    }
    ssq = wave_sum(ssq);
    const float rstd = 1.0f / sqrtf(ssq / (float)p.n_cols + p.eps);
    if (p.rstd_out && lane == 0) p.rstd_out[row] = rstd;
    __bf16* yr = p.y + row * p.ys;
    for (int col = lane; col < p.n_cols; col += 64) {
        float v = (float)xr[col];
        if (rr) v = (float)(__bf16)(v + (float)rr[col]);
        const float w = p.weight_fp32 ? static_cast<const float*>(p.weight)[col]
                                      : (float)static_cast<const __bf16*>(p.weight)[col];
        yr[col] = (__bf16)(w * (v * rstd));
    }
}

struct SiluMulParams {
    const __bf16* gate;
    const __bf16* up;
    __bf16* out;
    int64_t n_rows;
    int64_t gs, us, os;          // row strides in elements
    int n_cols;
};

// silu in fp32, rounded to bf16, then multiplied by `up` (product rounded to bf16): the order of
// roundings of a bf16 tensor program silu(gate).to(bf16) * up.
__device__ __forceinline__ float silu_mul_one(float g, float u) {
    const float s = g / (1.0f + __expf(-g));
    return (float)(__bf16)s * u;
}

// One thread per 8 adjacent elements of a row.  Requires n_cols % 8 == 0 and 16-byte aligned rows.
// The grid covers the tensor once (the loop only runs again beyond 2^31 workgroups): workgroups are
// dispatched in order, so the accesses in flight at any time form one window that moves through the
// tensor, which DRAM serves faster than the scattered windows of a small persistent grid (measured:
// 6.4 against 4.9 TB/s for a two-reads-one-write stream of this size).
__global__ __launch_bounds__(256) void silu_mul_vec8_kernel(SiluMulParams p) {
    const int groups = p.n_cols / 8;
    const int64_t total = p.n_rows * groups;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = idx / groups;
        const int col = (int)(idx % groups) * 8;
        const bf16x8 g = as_bf16x8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.gate + row * p.gs + col)));
        const bf16x8 u = as_bf16x8(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.up + row * p.us + col)));
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            o[e] = pack_bf16(silu_mul_one((float)g[2 * e], (float)u[2 * e]),
                             silu_mul_one((float)g[2 * e + 1], (float)u[2 * e + 1]));
        __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(p.out + row * p.os + col));
    }
}

__global__ __launch_bounds__(256) void silu_mul_generic_kernel(SiluMulParams p) {
    const int64_t total = p.n_rows * p.n_cols;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = idx / p.n_cols;
        const int col = (int)(idx % p.n_cols);
        p.out[row * p.os + col] = (__bf16)silu_mul_one((float)p.gate[row * p.gs + col], (float)p.up[row * p.us + col]);
    }
}

}  // namespace mi355

using namespace mi355;

static bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

extern "C" int mi355_rms_norm_fwd(const void* x, const void* residual, const void* weight, void* y, void* sum_out,
                                  float* rstd_out, int64_t n_rows, int n_cols, int64_t x_row_stride,
                                  int64_t residual_row_stride, int64_t y_row_stride, int64_t sum_row_stride, float eps,
                                  int weight_dtype, void* stream) {
    if (!x || !weight || !y) return set_error(MI355_EINVAL, "rms_norm: null pointer argument");
    if (sum_out && !residual) return set_error(MI355_EINVAL, "rms_norm: sum_out given without residual");
    if (n_rows < 0 || n_cols <= 0) return set_error(MI355_EINVAL, "rms_norm: n_rows, n_cols out of range");
    if (weight_dtype != MI355_BF16 && weight_dtype != MI355_FP32)
        return set_error(MI355_EDTYPE, "rms_norm: weight dtype must be MI355_BF16 or MI355_FP32");
    if (!(eps >= 0.f)) return set_error(MI355_EINVAL, "rms_norm: eps must be >= 0");
    if (n_rows == 0) return MI355_OK;
    RmsNormParams p;
    p.x = (const __bf16*)x;
    p.residual = (const __bf16*)residual;
    p.weight = weight;
    p.y = (__bf16*)y;
    p.sum_out = (__bf16*)sum_out;
    p.rstd_out = rstd_out;
    p.n_rows = n_rows;
    p.xs = x_row_stride;
    p.rs = residual_row_stride;
    p.ys = y_row_stride;
    p.ss = sum_row_stride;
    p.n_cols = n_cols;
    p.eps = eps;
    p.weight_fp32 = weight_dtype == MI355_FP32;
    const int64_t wgs = (n_rows + 3) / 4;
    if (wgs > 0x7fffffffLL) return set_error(MI355_EINVAL, "rms_norm: too many rows");
    const bool vec = n_cols % 8 == 0 && n_cols <= 8192 && aligned16(x) && aligned16(y) && aligned16(weight) &&
                     (!residual || aligned16(residual)) && (!sum_out || aligned16(sum_out)) &&
                     ((x_row_stride | y_row_stride) & 7) == 0 && (!residual || (residual_row_stride & 7) == 0) &&
                     (!sum_out || (sum_row_stride & 7) == 0);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)wgs), block(256);
    if (!vec) hipLaunchKernelGGL(rms_norm_generic_kernel, grid, block, 0, s, p);
    else if (n_cols <= 512) hipLaunchKernelGGL(rms_norm_rows_kernel<1>, grid, block, 0, s, p);
    else if (n_cols <= 1024) hipLaunchKernelGGL(rms_norm_rows_kernel<2>, grid, block, 0, s, p);
    else if (n_cols <= 2048) hipLaunchKernelGGL(rms_norm_rows_kernel<4>, grid, block, 0, s, p);
    else if (n_cols <= 4096) hipLaunchKernelGGL(rms_norm_rows_kernel<8>, grid, block, 0, s, p);
    else hipLaunchKernelGGL(rms_norm_rows_kernel<16>, grid, block, 0, s, p);
    const int rc = (int)hipGetLastError();
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}

extern "C" int mi355_silu_mul_fwd(const void* gate, const void* up, void* out, int64_t n_rows, int n_cols,
                                  int64_t gate_row_stride, int64_t up_row_stride, int64_t out_row_stride, void* stream) {
    if (!gate || !up || !out) return set_error(MI355_EINVAL, "silu_mul: null pointer argument");
    if (n_rows < 0 || n_cols <= 0) return set_error(MI355_EINVAL, "silu_mul: n_rows, n_cols out of range");
    if (n_rows == 0) return MI355_OK;
    SiluMulParams p;
    p.gate = (const __bf16*)gate;
    p.up = (const __bf16*)up;
    p.out = (__bf16*)out;
    p.n_rows = n_rows;
    p.gs = gate_row_stride;
    p.us = up_row_stride;
    p.os = out_row_stride;
    p.n_cols = n_cols;
    const bool vec = n_cols % 8 == 0 && aligned16(gate) && aligned16(up) && aligned16(out) &&
                     ((gate_row_stride | up_row_stride | out_row_stride) & 7) == 0;
    const int64_t total = vec ? n_rows * (n_cols / 8) : n_rows * (int64_t)n_cols;
    const int64_t blocks = (total + 255) / 256;
    const unsigned grid = (unsigned)(blocks < 0x7fffffffLL ? blocks : 0x7fffffffLL);
    hipStream_t s = (hipStream_t)stream;
    if (vec) hipLaunchKernelGGL(silu_mul_vec8_kernel, dim3(grid), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(silu_mul_generic_kernel, dim3(grid), dim3(256), 0, s, p);
    const int rc = (int)hipGetLastError();
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}
