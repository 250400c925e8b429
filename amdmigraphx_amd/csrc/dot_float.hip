// Float `dot` and the strided copy: the two operators a quantized graph still needs around
// the quantized GEMMs (calibration runs of the unquantized graph, the dot behind a per-tensor
// int4 dequantizelinear, `contiguous` of a transposed view).
//
// mi355_dot reproduces op::dot::compute -> gemm_naive (src/include/migraphx/op/dot.hpp:102-107,
// src/gemm.cpp:42-63) bit for bit: every output accumulates double(a) * double(b) for k ascending
// in a double, then casts once to the tensor's type.  The product of two floats is exact in a
// double, so the fused multiply-add used here rounds exactly as the reference's separate multiply
// and add do.
#include "common.h"

namespace {

struct dot_params
{
    const void* a;
    const void* b;
    void* c;
    int64_t m, n, k;
    int64_t a_sm, a_sk, b_sk, b_sn, ldc;
    int64_t stride_a, stride_b, stride_c;
    int type;
};

MI355_DEVINL float load_f32(const void* p, int type, int64_t i)
{
    switch(type)
    {
    case MI355_F32: return ((const float*)p)[i];
    case MI355_F16: return half_to_f32(((const uint16_t*)p)[i]);
    default: return bf16_to_f32(((const uint16_t*)p)[i]);
    }
}

// 64 x 64 outputs per workgroup of 256 threads, 4 x 4 per thread, K in steps of 16 through LDS.
__global__ __launch_bounds__(256) void dot_float_kernel(dot_params p)
{
    __shared__ float as[16][65];
    __shared__ float bs[16][65];
    const int tid = threadIdx.x;
    const int tx  = tid & 15;
    const int ty  = tid >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * 64;
    const int64_t col0 = (int64_t)blockIdx.x * 64;
    const int64_t ao   = (int64_t)blockIdx.z * p.stride_a;
    const int64_t bo   = (int64_t)blockIdx.z * p.stride_b;
    double acc[4][4];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
            acc[i][j] = 0.0;

    for(int64_t k0 = 0; k0 < p.k; k0 += 16)
    {
#pragma unroll
        for(int e = 0; e < 4; e++)
        {
            const int idx = tid + e * 256; // 0..1023
            // A tile: element (r, kk) with kk fastest so that K-contiguous rows coalesce
            {
                const int r  = idx >> 4;
                const int kk = idx & 15;
                float v      = 0.f;
                if(row0 + r < p.m && k0 + kk < p.k)
                    v = load_f32(p.a, p.type, ao + (row0 + r) * p.a_sm + (k0 + kk) * p.a_sk);
                as[kk][r] = v;
            }
            // B tile: element (kk, c) with c fastest (row-major B coalesces)
            {
                const int kk = idx >> 6;
                const int c  = idx & 63;
                float v      = 0.f;
                if(col0 + c < p.n && k0 + kk < p.k)
                    v = load_f32(p.b, p.type, bo + (k0 + kk) * p.b_sk + (col0 + c) * p.b_sn);
                bs[kk][c] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for(int kk = 0; kk < 16; kk++)
        {
            double av[4], bv[4];
#pragma unroll
            for(int i = 0; i < 4; i++)
                av[i] = (double)as[kk][ty * 4 + i];
#pragma unroll
            for(int j = 0; j < 4; j++)
                bv[j] = (double)bs[kk][tx + 16 * j];
#pragma unroll
            for(int i = 0; i < 4; i++)
#pragma unroll
                for(int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_fma(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for(int i = 0; i < 4; i++)
    {
        const int64_t row = row0 + ty * 4 + i;
        if(row >= p.m)
            continue;
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            const int64_t col = col0 + tx + 16 * j;
            if(col >= p.n)
                continue;
            const int64_t idx = (int64_t)blockIdx.z * p.stride_c + row * p.ldc + col;
            // static_cast<T>(double): double -> float (nearest even), then float -> 16-bit
            // float by truncation for half and bf16
            const float f = (float)acc[i][j];
            if(p.type == MI355_F32)
                ((float*)p.c)[idx] = f;
            else if(p.type == MI355_F16)
                ((uint16_t*)p.c)[idx] = f32_to_half_rtz(f);
            else
                ((uint16_t*)p.c)[idx] = f32_to_bf16_rtz(f);
        }
    }
}

struct gather_params
{
    const uint8_t* in;
    uint8_t* out;
    int64_t lens[MI355_MAX_DIMS];
    int64_t strides[MI355_MAX_DIMS];
    int64_t total;
    int ndim;
    int elem_size;
};

template <class T>
__global__ __launch_bounds__(256) void gather_kernel(gather_params p)
{
    const int64_t step = (int64_t)gridDim.x * 256;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += step)
    {
        int64_t rem = i;
        int64_t off = 0;
        for(int d = p.ndim - 1; d >= 0; d--)
        {
            off += (rem % p.lens[d]) * p.strides[d];
            rem /= p.lens[d];
        }
        ((T*)p.out)[i] = ((const T*)p.in)[off];
    }
}

} // namespace

extern "C" int mi355_dot(const void* a,
                         const void* b,
                         void* c,
                         int32_t type,
                         int64_t m,
                         int64_t n,
                         int64_t k,
                         int64_t a_stride_m,
                         int64_t a_stride_k,
                         int64_t b_stride_k,
                         int64_t b_stride_n,
                         int64_t ldc,
                         int64_t batch,
                         int64_t stride_a,
                         int64_t stride_b,
                         int64_t stride_c,
                         void* stream)
{
    if(type != MI355_F32 && type != MI355_F16 && type != MI355_BF16)
        return MI355_ERR_BAD_ARG;
    if(m < 0 || n < 0 || k < 0 || batch < 0 || a_stride_m < 0 || a_stride_k < 0 || b_stride_k < 0 ||
       b_stride_n < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0 || ldc < n)
        return MI355_ERR_BAD_ARG;
    if(m == 0 || n == 0 || batch == 0)
        return MI355_OK;
    if(c == nullptr || (k > 0 && (a == nullptr || b == nullptr)))
        return MI355_ERR_BAD_ARG;
    const int64_t gx = (n + 63) / 64, gy = (m + 63) / 64;
    if(gy > 65535 || batch > 65535)
        return MI355_ERR_UNSUPPORTED;
    dot_params p{a, b, c, m, n, k, a_stride_m, a_stride_k, b_stride_k, b_stride_n, ldc,
                 stride_a, stride_b, stride_c, type};
    hipLaunchKernelGGL(dot_float_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)batch), dim3(256),
                       0, static_cast<hipStream_t>(stream), p);
    return mi355_launch_status();
}

extern "C" int mi355_contiguous(const void* in,
                                void* out,
                                int32_t elem_size,
                                int32_t ndim,
                                const int64_t* lens,
                                const int64_t* strides,
                                void* stream)
{
    if(ndim < 1 || ndim > MI355_MAX_DIMS || lens == nullptr || strides == nullptr)
        return MI355_ERR_BAD_ARG;
    if(elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8)
        return MI355_ERR_BAD_ARG;
    gather_params p{};
    p.total = 1;
    for(int d = 0; d < ndim; d++)
    {
        if(lens[d] < 0 || strides[d] < 0)
            return MI355_ERR_BAD_ARG;
        p.lens[d]    = lens[d];
        p.strides[d] = strides[d];
        p.total *= lens[d];
    }
    if(p.total == 0)
        return MI355_OK;
    if(in == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    p.in        = static_cast<const uint8_t*>(in);
    p.out       = static_cast<uint8_t*>(out);
    p.ndim      = ndim;
    p.elem_size = elem_size;
    int64_t blocks = (p.total + 255) / 256;
    if(blocks > 256 * 16)
        blocks = 256 * 16;
    const dim3 grid((unsigned)blocks);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch(elem_size)
    {
    case 1: hipLaunchKernelGGL(gather_kernel<uint8_t>, grid, dim3(256), 0, s, p); break;
    case 2: hipLaunchKernelGGL(gather_kernel<uint16_t>, grid, dim3(256), 0, s, p); break;
    case 4: hipLaunchKernelGGL(gather_kernel<uint32_t>, grid, dim3(256), 0, s, p); break;
    default: hipLaunchKernelGGL(gather_kernel<uint64_t>, grid, dim3(256), 0, s, p); break;
    }
    return mi355_launch_status();
}
