// Residual add fused with LayerNorm for the Swin block around the attention operator (gfx950).
//
// The block (Swin3D/modules/swin3d_layers.py:617-623) computes
//   feats = short_cut + attn(norm1(feats));  feats = feats + mlp(norm2(feats))
// on an fp32 residual stream whose normalised copies feed fp16 GEMMs under autocast.  As separate torch kernels
// that is an add (read two rows, write one), a LayerNorm (read one, write one in fp32) and a cast (read fp32,
// write fp16) per use; this kernel reads the row and the branch output once and writes the updated residual
// row and the normalised row in the GEMM's input type.  Memory bound: 4*C (+2*C) bytes in, 4*C + 2*C out per row.
//
// One group of G lanes per row (G = 16, 32 or 64 by row length), 16-byte loads, two-pass mean / variance in
// registers (the row stays in registers between the passes), fp32 arithmetic.
#include "s3d_common.h"

#include <hip/hip_fp16.h>

namespace s3d {
namespace {

constexpr int kLnThreads = 256;
constexpr int kMaxChunks = 4;   // float4 chunks per lane: rows of up to 4 * 4 * 64 = 1024 channels

template <int G> __device__ __forceinline__ float group_sum(float v)
{
#pragma unroll
    for (int off = 1; off < G; off <<= 1) v += __shfl_xor(v, off, G);
    return v;
}

// RES: 0 = no residual, 1 = fp32 residual, 2 = fp16 residual.  OUT16: normalised rows in fp16 (else fp32).
template <int G, int RES, bool OUT16>
__global__ __launch_bounds__(kLnThreads) void add_layernorm_kernel(const float *__restrict__ x, const void *__restrict__ residual,
                                                                   const float *__restrict__ gamma,
                                                                   const float *__restrict__ beta, float eps,
                                                                   float *__restrict__ x_out, void *__restrict__ y,
                                                                   int64_t N, int C)
{
    const int lane = threadIdx.x % G;
    const int64_t row = (static_cast<int64_t>(blockIdx.x) * kLnThreads + threadIdx.x) / G;
    if (row >= N) return;   // whole groups leave together: the shuffles below stay inside a group
    const int chunks = C / 4;   // C is a multiple of 4
    const float *xr = x + row * C;
    float4 v[kMaxChunks];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ch = lane + i * G;
        v[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (ch < chunks) {
            v[i] = *reinterpret_cast<const float4 *>(xr + 4 * ch);
            if (RES == 1) {
                const float4 r = *reinterpret_cast<const float4 *>(static_cast<const float *>(residual) + row * C + 4 * ch);
                v[i].x += r.x; v[i].y += r.y; v[i].z += r.z; v[i].w += r.w;
            } else if (RES == 2) {
                const uint2 raw = *reinterpret_cast<const uint2 *>(static_cast<const __half *>(residual) + row * C + 4 * ch);
                const float2 lo = __half22float2(*reinterpret_cast<const __half2 *>(&raw.x));
                const float2 hi = __half22float2(*reinterpret_cast<const __half2 *>(&raw.y));
                v[i].x += lo.x; v[i].y += lo.y; v[i].z += hi.x; v[i].w += hi.y;
            }
            if (RES != 0 && x_out) *reinterpret_cast<float4 *>(x_out + row * C + 4 * ch) = v[i];
            sum += (v[i].x + v[i].y) + (v[i].z + v[i].w);
        }
    }
    const float mean = group_sum<G>(sum) / static_cast<float>(C);
    float sq = 0.0f;
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ch = lane + i * G;
        if (ch < chunks) {
            const float a = v[i].x - mean, b = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
            sq += (a * a + b * b) + (c * c + d * d);
        }
    }
    const float rstd = rsqrtf(group_sum<G>(sq) / static_cast<float>(C) + eps);
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ch = lane + i * G;
        if (ch < chunks) {
            const float4 g = *reinterpret_cast<const float4 *>(gamma + 4 * ch);
            const float4 b = *reinterpret_cast<const float4 *>(beta + 4 * ch);
            float4 o;
            o.x = (v[i].x - mean) * rstd * g.x + b.x;
            o.y = (v[i].y - mean) * rstd * g.y + b.y;
            o.z = (v[i].z - mean) * rstd * g.z + b.z;
            o.w = (v[i].w - mean) * rstd * g.w + b.w;
            if (OUT16) {
                uint2 packed;
                *reinterpret_cast<__half2 *>(&packed.x) = __floats2half2_rn(o.x, o.y);
                *reinterpret_cast<__half2 *>(&packed.y) = __floats2half2_rn(o.z, o.w);
                *reinterpret_cast<uint2 *>(static_cast<__half *>(y) + row * C + 4 * ch) = packed;
            } else {
                *reinterpret_cast<float4 *>(static_cast<float *>(y) + row * C + 4 * ch) = o;
            }
        }
    }
}

template <int G, int RES>
void launch_ln(bool out16, const float *x, const void *residual, const float *gamma, const float *beta, float eps,
               float *x_out, void *y, int64_t N, int C, hipStream_t stream)
{
    const int64_t threads = N * G;
    const dim3 grid(static_cast<unsigned>((threads + kLnThreads - 1) / kLnThreads));
    if (out16)
        hipLaunchKernelGGL((add_layernorm_kernel<G, RES, true>), grid, dim3(kLnThreads), 0, stream, x, residual, gamma, beta,
                           eps, x_out, y, N, C);
    else
        hipLaunchKernelGGL((add_layernorm_kernel<G, RES, false>), grid, dim3(kLnThreads), 0, stream, x, residual, gamma, beta,
                           eps, x_out, y, N, C);
}

template <int G>
void launch_ln_res(int res, bool out16, const float *x, const void *residual, const float *gamma, const float *beta,
                   float eps, float *x_out, void *y, int64_t N, int C, hipStream_t stream)
{
    if (res == 0) launch_ln<G, 0>(out16, x, residual, gamma, beta, eps, x_out, y, N, C, stream);
    else if (res == 1) launch_ln<G, 1>(out16, x, residual, gamma, beta, eps, x_out, y, N, C, stream);
    else launch_ln<G, 2>(out16, x, residual, gamma, beta, eps, x_out, y, N, C, stream);
}

}  // namespace
}  // namespace s3d

extern "C" __attribute__((visibility("default"))) int s3d_add_layernorm(
    const float *x, const void *residual, int32_t residual_dtype, const float *gamma, const float *beta, float eps,
    float *x_out, void *y, int32_t y_dtype, int64_t N, int32_t C, void *stream)
{
    using namespace s3d;
    if (N < 0 || C < 4 || C % 4 != 0 || C > 4 * kMaxChunks * 64)
        return fail(S3D_ERR_BAD_SHAPE, "s3d_add_layernorm: N=%lld C=%d (C a multiple of 4, 4..%d)", (long long)N, C,
                    4 * kMaxChunks * 64);
    if (y_dtype != S3D_DTYPE_F32 && y_dtype != S3D_DTYPE_F16)
        return fail(S3D_ERR_BAD_DTYPE, "s3d_add_layernorm: y_dtype %d (0 = fp32, 1 = fp16)", y_dtype);
    if (residual && residual_dtype != S3D_DTYPE_F32 && residual_dtype != S3D_DTYPE_F16)
        return fail(S3D_ERR_BAD_DTYPE, "s3d_add_layernorm: residual_dtype %d (0 = fp32, 1 = fp16)", residual_dtype);
    if (N == 0) return S3D_OK;
    if (!x || !gamma || !beta || !y) return fail(S3D_ERR_NULL_POINTER, "s3d_add_layernorm: null device pointer");
    const int res = !residual ? 0 : (residual_dtype == S3D_DTYPE_F32 ? 1 : 2);
    const bool out16 = y_dtype == S3D_DTYPE_F16;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int chunks = C / 4;
    if (chunks <= 16 * kMaxChunks / 2) launch_ln_res<16>(res, out16, x, residual, gamma, beta, eps, x_out, y, N, C, s);
    else if (chunks <= 32 * kMaxChunks / 2) launch_ln_res<32>(res, out16, x, residual, gamma, beta, eps, x_out, y, N, C, s);
    else launch_ln_res<64>(res, out16, x, residual, gamma, beta, eps, x_out, y, N, C, s);
    S3D_HIP_CHECK(hipGetLastError());
    return S3D_OK;
}
