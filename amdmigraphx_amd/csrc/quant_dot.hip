// mi355_quant_dot: argument checking, kernel selection, and the any-stride
// kernel that serves the shapes the MFMA kernel's load pattern does not fit
// (transposed A, K not a multiple of 16, odd leading dimensions, tiny cases).
#include "common.h"
#include <atomic>
#include <mutex>

bool mi355_mfma_gemm_supported(const mi355_quant_dot_desc*, const void*, const void*, const void*);
int mi355_mfma_gemm_launch(const mi355_quant_dot_desc*,
                           const void*,
                           const void*,
                           void*,
                           const float*,
                           const float*,
                           const int32_t*,
                           const int32_t*,
                           const float*,
                           hipStream_t);
bool mi355_dma_gemm_supported(const mi355_quant_dot_desc*, const void*, const void*);
int mi355_dma_gemm_launch(const mi355_quant_dot_desc*,
                          const void*,
                          const void*,
                          void*,
                          const float*,
                          const float*,
                          const int32_t*,
                          const int32_t*,
                          const float*,
                          void*,
                          size_t,
                          hipStream_t);
size_t mi355_dma_gemm_workspace(const mi355_quant_dot_desc*);

namespace {

struct generic_params
{
    const uint8_t* a;
    const uint8_t* b;
    void* c;
    int64_t m, n, k;
    int64_t a_sm, a_sk, b_sk, b_sn, ldc;
    int64_t stride_a, stride_b, stride_c;
    const float* scale_a;
    const float* scale_b;
    const int32_t* colsum_b;
    const int32_t* rowsum_a;
    const float* bias;
    int scale_a_mode, scale_b_mode, zp_a, zp_b;
    int fp8, dequant, out_type; // fp8: 0 integers, 1 e4m3fn, 2 e5m2
    int is_unsigned; // uint8 operands (bare quant_dot only)
};

MI355_DEVINL float decode_operand(uint8_t raw, const generic_params& p)
{
    if(p.fp8 == 1)
        return fp8_to_f32(raw);
    if(p.fp8 == 2)
        return bf8_to_f32(raw);
    return p.is_unsigned ? (float)raw : (float)(int8_t)raw;
}

// 16 x 16 outputs per workgroup, K walked in steps of 16 through LDS.  int8
// accumulates in int32 (exact); fp8 accumulates in double, which holds the
// sum exactly for any K this path sees, as the ref target's double
// accumulator does.
__global__ __launch_bounds__(256) void quant_dot_generic_kernel(generic_params p)
{
    __shared__ float as[16][17];
    __shared__ float bs[16][17];
    const int tx = threadIdx.x & 15;
    const int ty = threadIdx.x >> 4;
    const int64_t row = (int64_t)blockIdx.y * 16 + ty;
    const int64_t col = (int64_t)blockIdx.x * 16 + tx;
    const uint8_t* a  = p.a + (int64_t)blockIdx.z * p.stride_a;
    const uint8_t* b  = p.b + (int64_t)blockIdx.z * p.stride_b;
    int32_t iacc = 0;
    double facc  = 0.0;
    for(int64_t k0 = 0; k0 < p.k; k0 += 16)
    {
        // as[ty][tx] = A[row, k0 + tx];  bs[ty][tx] = B[k0 + ty, col]
        float av = 0.f, bv = 0.f;
        if(row < p.m && k0 + tx < p.k)
        {
            uint8_t raw = a[row * p.a_sm + (k0 + tx) * p.a_sk];
            av          = decode_operand(raw, p);
        }
        if(col < p.n && k0 + ty < p.k)
        {
            uint8_t raw = b[(k0 + ty) * p.b_sk + col * p.b_sn];
            bv          = decode_operand(raw, p);
        }
        as[ty][tx] = av;
        bs[ty][tx] = bv;
        __syncthreads();
        if(p.fp8)
        {
#pragma unroll
            for(int kk = 0; kk < 16; kk++)
                facc += (double)as[ty][kk] * (double)bs[kk][tx];
        }
        else
        {
#pragma unroll
            for(int kk = 0; kk < 16; kk++)
                iacc += (int32_t)as[ty][kk] * (int32_t)bs[kk][tx];
        }
        __syncthreads();
    }
    if(row >= p.m || col >= p.n)
        return;
    const int64_t idx = (int64_t)blockIdx.z * p.stride_c + row * p.ldc + col;
    if(!p.dequant)
    {
        if(p.fp8)
            static_cast<float*>(p.c)[idx] = (float)facc;
        else
            static_cast<int32_t*>(p.c)[idx] = iacc;
        return;
    }
    float sa = 1.f, sb = 1.f;
    if(p.scale_a_mode == MI355_QP_PER_TENSOR)
        sa = p.scale_a[0];
    else if(p.scale_a_mode == MI355_QP_PER_ROW)
        sa = p.scale_a[row];
    if(p.scale_b_mode == MI355_QP_PER_TENSOR)
        sb = p.scale_b[0];
    else if(p.scale_b_mode == MI355_QP_PER_COL)
        sb = p.scale_b[col];
    const float s = sa * sb;
    double d;
    if(p.fp8)
    {
        // the ref target rounds the accumulator to float (quant_dot's output
        // type) before dequantizelinear reads it
        d = (double)(float)facc;
    }
    else
    {
        int64_t zp = 0;
        if(p.zp_a != 0)
            zp += (int64_t)p.zp_a * p.colsum_b[col];
        if(p.zp_b != 0)
            zp += (int64_t)p.zp_b * p.rowsum_a[row];
        if(p.zp_a != 0 && p.zp_b != 0)
            zp -= p.k * (int64_t)p.zp_a * p.zp_b;
        d = (double)iacc - (double)(int32_t)zp;
    }
    float v = (float)(d * (double)s);
    if(p.bias != nullptr)
        v = add_bias(v, p.bias[col]);
    switch(p.out_type)
    {
    case MI355_F32: static_cast<float*>(p.c)[idx] = v; break;
    case MI355_F16: static_cast<uint16_t*>(p.c)[idx] = convert_f32_to_half(v); break;
    case MI355_BF16: static_cast<uint16_t*>(p.c)[idx] = convert_f32_to_bf16(v); break;
    default: break;
    }
}

// out[i] = sum over `len` int8 elements, element j of vector i at
// base + i*stride_i + j*stride_j.  One wave per output.
__global__ __launch_bounds__(256) void sum_i8_kernel(
    const int8_t* base, int64_t count, int64_t len, int64_t stride_i, int64_t stride_j, int32_t* out)
{
    const int lane    = threadIdx.x & 63;
    const int64_t vec = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if(vec >= count)
        return;
    const int8_t* p = base + vec * stride_i;
    int32_t s       = 0;
    for(int64_t j = lane; j < len; j += 64)
        s += p[j * stride_j];
#pragma unroll
    for(int off = 32; off > 0; off >>= 1)
        s += __shfl_xor(s, off, 64);
    if(lane == 0)
        out[vec] = s;
}

// column sums of row-major [K, N]: consecutive threads take consecutive
// columns so every row read is coalesced; K is split over blockIdx.y slices
// that combine with integer atomics (exact, order independent).
__global__ __launch_bounds__(256) void colsum_rowmajor_kernel(
    const int8_t* b, int64_t k, int64_t n, int64_t ldb, int64_t k_per_slice, int32_t* out)
{
    const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(col >= n)
        return;
    const int64_t k0 = (int64_t)blockIdx.y * k_per_slice;
    const int64_t k1 = min(k, k0 + k_per_slice);
    int32_t s        = 0;
    for(int64_t kk = k0; kk < k1; kk++)
        s += b[kk * ldb + col];
    atomicAdd(out + col, s);
}

__global__ void zero_i32_kernel(int32_t* p, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if(i < n)
        p[i] = 0;
}

} // namespace

extern "C" int mi355_quant_dot(const mi355_quant_dot_desc* d,
                               const void* a,
                               const void* b,
                               void* c,
                               const float* scale_a,
                               const float* scale_b,
                               const int32_t* colsum_b,
                               const int32_t* rowsum_a,
                               void* stream)
{
    return mi355_quant_dot_bias(d, a, b, c, scale_a, scale_b, colsum_b, rowsum_a, nullptr, stream);
}

extern "C" int mi355_quant_dot_bias(const mi355_quant_dot_desc* d,
                                    const void* a,
                                    const void* b,
                                    void* c,
                                    const float* scale_a,
                                    const float* scale_b,
                                    const int32_t* colsum_b,
                                    const int32_t* rowsum_a,
                                    const float* bias,
                                    void* stream)
{
    return mi355_quant_dot_ws(d, a, b, c, scale_a, scale_b, colsum_b, rowsum_a, bias, nullptr, 0, stream);
}

extern "C" size_t mi355_quant_dot_workspace_size(const mi355_quant_dot_desc* d)
{
    return d == nullptr ? 0 : mi355_dma_gemm_workspace(d);
}

extern "C" int mi355_quant_dot_ws(const mi355_quant_dot_desc* d,
                                  const void* a,
                                  const void* b,
                                  void* c,
                                  const float* scale_a,
                                  const float* scale_b,
                                  const int32_t* colsum_b,
                                  const int32_t* rowsum_a,
                                  const float* bias,
                                  void* workspace,
                                  size_t workspace_bytes,
                                  void* stream)
{
    if(d == nullptr)
        return MI355_ERR_BAD_ARG;
    if(d->m < 0 || d->n < 0 || d->k < 0 || d->batch < 0)
        return MI355_ERR_BAD_ARG;
    const bool empty = d->m == 0 || d->n == 0 || d->batch == 0;
    if(!empty && (a == nullptr || b == nullptr || c == nullptr))
        return MI355_ERR_BAD_ARG;
    if(d->in_type != MI355_I8 && d->in_type != MI355_FP8 && d->in_type != MI355_U8 &&
       d->in_type != MI355_BF8)
        return MI355_ERR_UNSUPPORTED;
    // e5m2 x e5m2 -> float (op/quant_dot.hpp:62-66 takes every fp8 type): the 16x16x128 MFMA
    // kernel or the generic one
    const bool bf8 = d->in_type == MI355_BF8;
    const bool fp8 = d->in_type == MI355_FP8 || bf8;
    // uint8 x uint8 -> int32 (op/quant_dot.hpp:62-64 lists it): bare result only, correctness path
    const bool u8 = d->in_type == MI355_U8;
    if(u8 && d->dequant)
        return MI355_ERR_UNSUPPORTED;
    if(bias != nullptr && !d->dequant)
        return MI355_ERR_BAD_ARG; // the bias is a float added to the dequantized value
    if(d->dequant)
    {
        if(d->out_type != MI355_F32 && d->out_type != MI355_F16 && d->out_type != MI355_BF16)
            return MI355_ERR_BAD_ARG;
        if(d->scale_a_mode != MI355_QP_NONE && d->scale_a_mode != MI355_QP_PER_TENSOR &&
           d->scale_a_mode != MI355_QP_PER_ROW)
            return MI355_ERR_BAD_ARG;
        if(d->scale_b_mode != MI355_QP_NONE && d->scale_b_mode != MI355_QP_PER_TENSOR &&
           d->scale_b_mode != MI355_QP_PER_COL && d->scale_b_mode != MI355_QP_PER_COL_BATCH)
            return MI355_ERR_BAD_ARG;
        if(d->scale_a_mode != MI355_QP_NONE && scale_a == nullptr)
            return MI355_ERR_BAD_ARG;
        if(d->scale_b_mode != MI355_QP_NONE && scale_b == nullptr)
            return MI355_ERR_BAD_ARG;
        if(fp8 && (d->zp_a != 0 || d->zp_b != 0))
            return MI355_ERR_UNSUPPORTED;
        if(d->zp_a != 0 && colsum_b == nullptr)
            return MI355_ERR_BAD_ARG;
        if(d->zp_b != 0 && rowsum_a == nullptr)
            return MI355_ERR_BAD_ARG;
        if(d->zp_a < -128 || d->zp_a > 127 || d->zp_b < -128 || d->zp_b > 127)
            return MI355_ERR_BAD_ARG;
        if((d->zp_a != 0 || d->zp_b != 0) && d->batch > 1)
            return MI355_ERR_UNSUPPORTED; // sums are given for one matrix
    }
    else
    {
        if(d->out_type != (fp8 ? MI355_F32 : MI355_I32))
            return MI355_ERR_BAD_ARG;
    }
    if(empty)
        return MI355_OK;
    if(d->ldc < d->n)
        return MI355_ERR_BAD_ARG;
    if((d->trans_a ? d->lda < d->m : d->lda < d->k) || (d->trans_b ? d->ldb < d->k : d->ldb < d->n))
        return MI355_ERR_BAD_ARG;
    if(d->batch > 65535)
        return MI355_ERR_UNSUPPORTED;

    hipStream_t s = static_cast<hipStream_t>(stream);
    // int8 with N % 4 != 0 would take the DMA path's 32 x 32 kernel, which applies no bias
    const bool dma_has_bias = bias == nullptr || fp8 || d->n % 4 == 0;
    if(!u8 && !bf8 && d->k > 0 && dma_has_bias && mi355_dma_gemm_supported(d, a, b))
        return mi355_dma_gemm_launch(d, a, b, c, scale_a, scale_b, colsum_b, rowsum_a, bias, workspace, workspace_bytes, s);
    // a vector of column scales per batch entry exists in the kernels above only
    if(d->dequant && d->scale_b_mode == MI355_QP_PER_COL_BATCH)
        return MI355_ERR_UNSUPPORTED;
    if(!u8 && d->k > 0 && mi355_mfma_gemm_supported(d, a, b, c))
        return mi355_mfma_gemm_launch(d, a, b, c, scale_a, scale_b, colsum_b, rowsum_a, bias, s);

    generic_params p;
    p.a            = static_cast<const uint8_t*>(a);
    p.b            = static_cast<const uint8_t*>(b);
    p.c            = c;
    p.m            = d->m;
    p.n            = d->n;
    p.k            = d->k;
    p.a_sm         = d->trans_a ? 1 : d->lda;
    p.a_sk         = d->trans_a ? d->lda : 1;
    p.b_sk         = d->trans_b ? 1 : d->ldb;
    p.b_sn         = d->trans_b ? d->ldb : 1;
    p.ldc          = d->ldc;
    p.stride_a     = d->stride_a;
    p.stride_b     = d->stride_b;
    p.stride_c     = d->stride_c;
    p.scale_a      = scale_a;
    p.scale_b      = scale_b;
    p.colsum_b     = colsum_b;
    p.rowsum_a     = rowsum_a;
    p.bias         = bias;
    p.scale_a_mode = d->scale_a_mode;
    p.scale_b_mode = d->scale_b_mode;
    p.zp_a         = d->zp_a;
    p.zp_b         = d->zp_b;
    p.fp8          = bf8 ? 2 : (fp8 ? 1 : 0);
    p.is_unsigned  = u8;
    p.dequant      = d->dequant;
    p.out_type     = d->out_type;
    const int64_t gx = (d->n + 15) / 16, gy = (d->m + 15) / 16;
    if(gy > 65535)
        return MI355_ERR_UNSUPPORTED;
    dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)d->batch);
    hipLaunchKernelGGL(quant_dot_generic_kernel, grid, dim3(256), 0, s, p);
    return mi355_launch_status();
}

// ---- quant_dot that allocates nothing and takes no workspace -------------------------------
// The split-K partial sums of mi355_quant_dot_ws go to a device array that is part of the
// library's code object: every GPU the library runs on holds its own copy from the moment the
// module is loaded there until the process ends.  In host code the array's name only stands for
// the symbol; the memory is reached through the address hipGetSymbolAddress reports on the
// device that is current, looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[MI355_QUANT_DOT_STATIC_SCRATCH_BYTES];

namespace {
constexpr int max_devices = 64;
std::atomic<void*> scratch_of_device[max_devices];
std::mutex scratch_lookup;

// address of this device's copy of `scratch`; null with *status set when HIP reports an error
void* device_scratch(int* status)
{
    int dev = -1;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= max_devices)
    {
        *status = MI355_ERR_LAUNCH;
        return nullptr;
    }
    void* ptr = scratch_of_device[dev].load(std::memory_order_acquire);
    if(ptr != nullptr)
        return ptr;
    std::lock_guard<std::mutex> guard(scratch_lookup);
    ptr = scratch_of_device[dev].load(std::memory_order_acquire);
    if(ptr != nullptr)
        return ptr;
    if(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr)
    {
        (void)hipGetLastError();
        *status = MI355_ERR_LAUNCH;
        return nullptr;
    }
    scratch_of_device[dev].store(ptr, std::memory_order_release);
    return ptr;
}
} // namespace

extern "C" int mi355_quant_dot_static(const mi355_quant_dot_desc* d,
                                      const void* a,
                                      const void* b,
                                      void* c,
                                      const float* scale_a,
                                      const float* scale_b,
                                      const int32_t* colsum_b,
                                      const int32_t* rowsum_a,
                                      const float* bias,
                                      void* stream)
{
    if(d == nullptr)
        return MI355_ERR_BAD_ARG;
    const size_t need = mi355_quant_dot_workspace_size(d);
    if(need > MI355_QUANT_DOT_STATIC_SCRATCH_BYTES)
        return MI355_ERR_SCRATCH_TOO_SMALL;
    if(need == 0) // no split for this description: the one-pass kernels use no scratch memory
        return mi355_quant_dot_ws(d, a, b, c, scale_a, scale_b, colsum_b, rowsum_a, bias, nullptr, 0, stream);
    int status = MI355_OK;
    void* ptr  = device_scratch(&status);
    if(ptr == nullptr)
        return status;
    // every element of the partial sums that the second kernel reads is stored by the first one in
    // the same call, so nothing has to be cleared between calls
    return mi355_quant_dot_ws(d, a, b, c, scale_a, scale_b, colsum_b, rowsum_a, bias, ptr, need, stream);
}

extern "C" int mi355_colsum_i8(const void* b,
                               int64_t k,
                               int64_t n,
                               int64_t ldb,
                               int32_t trans_b,
                               int32_t* out,
                               void* stream)
{
    if(b == nullptr || out == nullptr || k < 0 || n < 0)
        return MI355_ERR_BAD_ARG;
    if(n == 0)
        return MI355_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if(trans_b)
    {
        // [N, K] storage: each column is a contiguous K run
        hipLaunchKernelGGL(sum_i8_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, s,
                           static_cast<const int8_t*>(b), n, k, ldb, (int64_t)1, out);
        return mi355_launch_status();
    }
    hipLaunchKernelGGL(zero_i32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, out, n);
    if(k == 0)
        return mi355_launch_status();
    int64_t slices      = (k + 255) / 256;
    if(slices > 64)
        slices = 64;
    int64_t k_per_slice = (k + slices - 1) / slices;
    slices              = (k + k_per_slice - 1) / k_per_slice;
    hipLaunchKernelGGL(colsum_rowmajor_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)slices),
                       dim3(256), 0, s, static_cast<const int8_t*>(b), k, n, ldb, k_per_slice, out);
    return mi355_launch_status();
}

extern "C" int mi355_rowsum_i8(const void* a,
                               int64_t m,
                               int64_t k,
                               int64_t lda,
                               int32_t trans_a,
                               int32_t* out,
                               void* stream)
{
    if(a == nullptr || out == nullptr || k < 0 || m < 0)
        return MI355_ERR_BAD_ARG;
    if(m == 0)
        return MI355_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if(trans_a)
    {
        // [K, M] storage: identical to column sums of a row-major matrix
        return mi355_colsum_i8(a, k, m, lda, 0, out, stream);
    }
    hipLaunchKernelGGL(sum_i8_kernel, dim3((unsigned)((m + 3) / 4)), dim3(256), 0, s,
                       static_cast<const int8_t*>(a), m, k, lda, (int64_t)1, out);
    return mi355_launch_status();
}

extern "C" const char* mi355_status_string(int status)
{
    switch(status)
    {
    case MI355_OK: return "ok";
    case MI355_ERR_BAD_ARG: return "bad argument";
    case MI355_ERR_UNSUPPORTED: return "unsupported configuration";
    case MI355_ERR_LAUNCH: return "HIP launch error";
    case MI355_ERR_SCRATCH_TOO_SMALL: return "the problem needs more scratch memory than the library's static buffer holds";
    default: return "unknown status";
    }
}

extern "C" int mi355_version(void) { return 100; }
