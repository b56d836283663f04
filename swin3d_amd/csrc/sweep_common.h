// Pieces shared by the sweep kernels of the attention forward and backward (gfx950): work-queue layout,
// row loads and stores, (row, head) slices in registers, the cRSE row quantiser, LDS table rows.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdint>

namespace s3d {
namespace sweep {

// Work distribution.  Atomics on one cache line retire one after the other (about 12 ns each on this part),
// so a single counter per head bounds a launch of 50 000 units to 0.6 ms whatever the units cost.  Every head
// has kQueues counters, each on a cache line of its own; unit u belongs to queue u % kQueues; a wavefront
// draws from the queue it starts on and moves to the next one when that is empty.
// The chip has eight XCDs with an L2 each: a wavefront starts on the queue of the XCD it runs on, so all heads
// of a unit are served from the same XCD and the unit's q, k, v rows and coordinates reach that L2 once.
constexpr int kQueues = 8;
constexpr int kCounterStride = 64;   // ints between counters (256 bytes)

// id of the XCD (accelerator complex die) the wavefront runs on
__device__ __forceinline__ int xcd_id()
{
    int id;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(id));
    return id;
}

template <int D> __device__ __forceinline__ void load_row(const float *p, float *dst)
{
#pragma unroll
    for (int c = 0; c < D; c += 4) {
        const float4 x = *reinterpret_cast<const float4 *>(p + c);
        dst[c] = x.x; dst[c + 1] = x.y; dst[c + 2] = x.z; dst[c + 3] = x.w;
    }
}
template <int D> __device__ __forceinline__ void load_row(const __half *p, float *dst)
{
#pragma unroll
    for (int c = 0; c < D; c += 8) {
        const uint4 x = *reinterpret_cast<const uint4 *>(p + c);
        const __half2 *hh = reinterpret_cast<const __half2 *>(&x);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float2 f = __half22float2(hh[e]);
            dst[c + 2 * e] = f.x;
            dst[c + 2 * e + 1] = f.y;
        }
    }
}
template <int D> __device__ __forceinline__ void store_row(float *p, const float *src)
{
#pragma unroll
    for (int c = 0; c < D; c += 4) *reinterpret_cast<float4 *>(p + c) = make_float4(src[c], src[c + 1], src[c + 2], src[c + 3]);
}
template <int D> __device__ __forceinline__ void store_row(__half *p, const float *src)
{
#pragma unroll
    for (int c = 0; c < D; c += 8) {
        uint4 x;
        __half2 *hh = reinterpret_cast<__half2 *>(&x);
#pragma unroll
        for (int e = 0; e < 4; ++e) hh[e] = __floats2half2_rn(src[c + 2 * e], src[c + 2 * e + 1]);
        *reinterpret_cast<uint4 *>(p + c) = x;
    }
}
__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(__half x) { return __half2float(x); }

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// 16-byte LDS reads at a 32-bit LDS address (pointer arithmetic on generic pointers is 64-bit, which costs a
// 64-bit multiply-add per gathered row)
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const u32x4_t lds_uint4_t;
typedef __attribute__((address_space(3))) const f32x4_t lds_float4_t;
// a * b + c with 24-bit factors: one full-rate instruction (the compiler's choice for a 32-bit multiply-add,
// v_mad_u64_u32, issues at a quarter of the rate)
__device__ __forceinline__ uint32_t mad_u24(uint32_t a, uint32_t b, uint32_t c)
{
    uint32_t d;
    asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "s"(c));
    return d;
}
__device__ __forceinline__ uint32_t lds_address(const void *p)
{
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p));   // low half of a flat LDS address
}

// One (row, head) slice of D channels in registers.  fp32: D floats, products by FMA.  fp16: D/2 packed pairs
// kept as loaded; dot products with v_dot2_f32_f16 (exact fp16 products, fp32 accumulation), widening only
// where a sum of rows is needed.
template <typename T, int D> struct Slice;
template <int D> struct Slice<float, D> {
    float x[D];
    __device__ __forceinline__ void load(const float *p) { load_row<D>(p, x); }
    // a row stored in fp16, widened as it is loaded (fp32 arithmetic on fp16 features)
    __device__ __forceinline__ void load(const __half *p) { load_row<D>(p, x); }
    __device__ __forceinline__ void load_lds(uint32_t addr)
    {
#pragma unroll
        for (int c = 0; c < D; c += 4) {
            const f32x4_t v = *(lds_float4_t *)(addr + 4 * c);
            x[c] = v[0]; x[c + 1] = v[1]; x[c + 2] = v[2]; x[c + 3] = v[3];
        }
    }
    __device__ __forceinline__ float dot(const Slice &o, float acc) const
    {
#pragma unroll
        for (int c = 0; c < D; ++c) acc += x[c] * o.x[c];
        return acc;
    }
    // acc += p * x
    __device__ __forceinline__ void fma_to(float *acc, float p) const
    {
#pragma unroll
        for (int c = 0; c < D; ++c) acc[c] += p * x[c];
    }
    // x += o
    __device__ __forceinline__ void add(const Slice &o)
    {
#pragma unroll
        for (int c = 0; c < D; ++c) x[c] += o.x[c];
    }
    // acc + sum_c x[c] * y[c]
    __device__ __forceinline__ float dot_f32(const float *y, float acc) const
    {
#pragma unroll
        for (int c = 0; c < D; ++c) acc += x[c] * y[c];
        return acc;
    }
    // the slice held by lane `src` (src uniform): scalar reads instead of LDS permutes
    __device__ __forceinline__ Slice lane(int src) const
    {
        Slice r;
#pragma unroll
        for (int c = 0; c < D; ++c) r.x[c] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x[c]), src));
        return r;
    }
    // out[c4] = channel 4 c4 + lane % 4 (the B operand of a 4x4x1 MFMA whose 1 x 4 row is this slice's quad c4)
    __device__ __forceinline__ void quad_channels(int lane, float *out) const
    {
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            const float lo = (lane & 1) ? x[4 * c + 1] : x[4 * c];
            const float hi = (lane & 1) ? x[4 * c + 3] : x[4 * c + 2];
            out[c] = (lane & 2) ? hi : lo;
        }
    }
    // fp32 logits: one short partial sum per table row keeps the rounding of the (2*D*ND + D)-term sum at the
    // level of a tree sum
    static constexpr bool kChainLogit = false;
};
template <int D> struct Slice<__half, D> {
    half2_t x[D / 2];
    __device__ __forceinline__ void load(const __half *p)
    {
#pragma unroll
        for (int c = 0; c < D; c += 8) *reinterpret_cast<uint4 *>(&x[c / 2]) = *reinterpret_cast<const uint4 *>(p + c);
    }
    __device__ __forceinline__ void load_lds(uint32_t addr)
    {
#pragma unroll
        for (int c = 0; c < D; c += 8) *reinterpret_cast<u32x4_t *>(&x[c / 2]) = *(lds_uint4_t *)(addr + 2 * c);
    }
    __device__ __forceinline__ float dot(const Slice &o, float acc) const
    {
#pragma unroll
        for (int e = 0; e < D / 2; ++e) acc = __builtin_amdgcn_fdot2(x[e], o.x[e], acc, false);
        return acc;
    }
    // acc += p * x, widened inside a mixed-precision FMA
    __device__ __forceinline__ void fma_to(float *acc, float p) const
    {
#pragma unroll
        for (int e = 0; e < D / 2; ++e) {
            acc[2 * e] = __builtin_fmaf(static_cast<float>(x[e][0]), p, acc[2 * e]);
            acc[2 * e + 1] = __builtin_fmaf(static_cast<float>(x[e][1]), p, acc[2 * e + 1]);
        }
    }
    // x += o in packed fp16 (two channels per instruction)
    __device__ __forceinline__ void add(const Slice &o)
    {
#pragma unroll
        for (int e = 0; e < D / 2; ++e) x[e] = x[e] + o.x[e];
    }
    // acc + sum_c x[c] * y[c], x widened inside the FMAs
    __device__ __forceinline__ float dot_f32(const float *y, float acc) const
    {
#pragma unroll
        for (int e = 0; e < D / 2; ++e) {
            acc = __builtin_fmaf(static_cast<float>(x[e][0]), y[2 * e], acc);
            acc = __builtin_fmaf(static_cast<float>(x[e][1]), y[2 * e + 1], acc);
        }
        return acc;
    }
    // the slice held by lane `src` (src uniform): scalar reads instead of LDS permutes
    __device__ __forceinline__ Slice lane(int src) const
    {
        Slice r;
#pragma unroll
        for (int e = 0; e < D / 2; ++e)
            r.x[e] = __builtin_bit_cast(half2_t, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x[e]), src));
        return r;
    }
    // out[c4] = channel 4 c4 + lane % 4 (the B operand of a 4x4x1 MFMA whose 1 x 4 row is this slice's quad c4)
    __device__ __forceinline__ void quad_channels(int lane, float *out) const
    {
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            const uint32_t pair = (lane & 2) ? __builtin_bit_cast(uint32_t, x[2 * c + 1]) : __builtin_bit_cast(uint32_t, x[2 * c]);
            const uint32_t bits = pair >> ((lane & 1) * 16);
            out[c] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(bits)));
        }
    }
    // fp16 I/O: the whole logit is one chain of dot-product accumulations
    static constexpr bool kChainLogit = true;
};

// Row of the axis table hit by a pair; fp32 arithmetic in the reference's operation order (subtract, add
// half the row count, clamp, truncate).  The reference clamps to [0, rows] and folds the upper edge onto
// the last row after truncation; clamping to [0, largest float below rows] gives the same row for every
// input with one median-of-three and no integer minimum.
__device__ __forceinline__ float crse_upper(int rows)
{
    return __int_as_float(__float_as_int(static_cast<float>(rows)) - 1);
}
__device__ __forceinline__ int crse_row(float ci, float cj, float half_rows, float upper)
{
    float rel = ci - cj;
    rel = rel + half_rows;
    return static_cast<int>(__builtin_amdgcn_fmed3f(rel, 0.0f, upper));
}

// Elements of T between table rows in LDS.  A row holds the head's slices of the three tables back to back
// (q-side, k-side, v-side: one address per pair and axis); a row length that is a multiple of 32 bytes is
// padded by 16 bytes so that a wavefront's 16-byte gathers of different rows spread over all bank groups.
template <typename T, int D> __host__ __device__ constexpr int table_row_stride()
{
    return 3 * D + ((3 * D * static_cast<int>(sizeof(T)) / 4) % 8 == 0 ? 16 / static_cast<int>(sizeof(T)) : 0);
}

}  // namespace sweep
}  // namespace s3d
