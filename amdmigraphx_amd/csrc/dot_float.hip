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
#include <type_traits>

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
    const float* scale; // fp32 only: the result is multiplied by scale[0] (a `mul` behind the dot); null = none
    // batch index z = zo * batch_inner + zi: operand z starts at zo * stride_?_outer + zi * stride_?
    // (two batch axes with strides of their own, e.g. the [batch, head] axes of a transposed view);
    // one batch axis: batch_inner = the batch count, outer strides 0
    int64_t batch_inner     = 1;
    int64_t stride_a_outer  = 0;
    int64_t stride_b_outer  = 0;
    int64_t stride_c_outer  = 0; // C likewise: zo * stride_c_outer + zi * stride_c
};

MI355_DEVINL void batch_offsets(const dot_params& p, int64_t& ao, int64_t& bo, int64_t& co)
{
    const int64_t z  = blockIdx.z;
    const int64_t zo = z / p.batch_inner;
    const int64_t zi = z - zo * p.batch_inner;
    ao               = zo * p.stride_a_outer + zi * p.stride_a;
    bo               = zo * p.stride_b_outer + zi * p.stride_b;
    co               = zo * p.stride_c_outer + zi * p.stride_c;
}

MI355_DEVINL float load_f32(const void* p, int type, int64_t i)
{
    switch(type)
    {
    case MI355_F32: return ((const float*)p)[i];
    case MI355_F16: return half_to_f32(((const uint16_t*)p)[i]);
    default: return bf16_to_f32(((const uint16_t*)p)[i]);
    }
}

typedef double v4d __attribute__((ext_vector_type(4)));

// The sums run on the fp64 matrix cores.  v_mfma_f64_16x16x4_f64 adds its four products to the
// accumulator one after the other, k ascending, each as a fused multiply-add in double -- the
// order and the rounding of the reference's loop -- so the results are the same bits (the tests
// compare them with the CPU restatement).  Operand layout (probed): lane l supplies A[l % 16][l / 16] and
// B[l / 16][l % 16]; register r of lane l holds D[4*r + l / 16][l % 16].
// 64 x 64 outputs per workgroup of four waves (2 x 2, each 32 x 32 = 2 x 2 instruction tiles), K in
// steps of 16 through LDS, where the tiles are kept as doubles (converted once, when staged).  The
// row pitch of 80 doubles puts the two k rows a half wave reads into disjoint halves of the banks.
__global__ __launch_bounds__(256) void dot_float_mfma_kernel(dot_params p)
{
    constexpr int PITCH = 80;
    __shared__ double as[16][PITCH];
    __shared__ double bs[16][PITCH];
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm   = wave >> 1;
    const int wn   = wave & 1;
    const int l16  = lane & 15;
    const int lk   = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * 64;
    const int64_t col0 = (int64_t)blockIdx.x * 64;
    int64_t ao, bo, co;
    batch_offsets(p, ao, bo, co);
    v4d acc[2][2];
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < 2; j++)
            acc[i][j] = v4d{0.0, 0.0, 0.0, 0.0};

    for(int64_t k0 = 0; k0 < p.k; k0 += 16)
    {
#pragma unroll
        for(int e = 0; e < 4; e++)
        {
            const int idx = tid + e * 256; // 0..1023
            {
                const int r  = idx >> 4;
                const int kk = idx & 15;
                float v      = 0.f;
                if(row0 + r < p.m && k0 + kk < p.k)
                    v = load_f32(p.a, p.type, ao + (row0 + r) * p.a_sm + (k0 + kk) * p.a_sk);
                as[kk][r] = (double)v;
            }
            {
                const int kk = idx >> 6;
                const int c  = idx & 63;
                float v      = 0.f;
                if(col0 + c < p.n && k0 + kk < p.k)
                    v = load_f32(p.b, p.type, bo + (k0 + kk) * p.b_sk + (col0 + c) * p.b_sn);
                bs[kk][c] = (double)v;
            }
        }
        __syncthreads();
#pragma unroll
        for(int kk0 = 0; kk0 < 16; kk0 += 4)
        {
            double av[2], bv[2];
#pragma unroll
            for(int i = 0; i < 2; i++)
                av[i] = as[kk0 + lk][wm * 32 + i * 16 + l16];
#pragma unroll
            for(int j = 0; j < 2; j++)
                bv[j] = bs[kk0 + lk][wn * 32 + j * 16 + l16];
#pragma unroll
            for(int i = 0; i < 2; i++)
#pragma unroll
                for(int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int r = 0; r < 4; r++)
        {
            const int64_t row = row0 + wm * 32 + i * 16 + 4 * r + lk;
            if(row >= p.m)
                continue;
#pragma unroll
            for(int j = 0; j < 2; j++)
            {
                const int64_t col = col0 + wn * 32 + j * 16 + l16;
                if(col >= p.n)
                    continue;
                const int64_t idx = co + row * p.ldc + col;
                const float f     = (float)acc[i][j][r];
                if(p.type == MI355_F32)
                    ((float*)p.c)[idx] = p.scale != nullptr ? f * p.scale[0] : f;
                else if(p.type == MI355_F16)
                    ((uint16_t*)p.c)[idx] = f32_to_half_rtz(f);
                else
                    ((uint16_t*)p.c)[idx] = f32_to_bf16_rtz(f);
            }
        }
}

// fp32 operands whose rows or columns are contiguous: the same kernel with 16-byte loads (one per
// thread and operand per K step) that are issued one step ahead, so that their latency runs under
// the matrix instructions.  A_KCONT: A's K stride is 1 (else its row stride is 1); B_NCONT: B's
// column stride is 1 (else its K stride is 1).  The host checks the alignment the vector loads need;
// a vector that would cross the matrix edge is read element by element with zero fill.
// FP32ACC: the sums run on the fp32 matrix cores instead (v_mfma_f32_16x16x4_f32, twice the rate):
// fp32 products and fp32 accumulation, no longer the bits of the reference's double sum but within
// K * 2^-24 of sum|a||b| of them.  Register r of lane l then holds D[4 * (l / 16) + r][l % 16].
template <bool A_KCONT, bool B_NCONT, bool FP32ACC = false>
__global__ __launch_bounds__(256) void dot_f32_mfma_kernel(dot_params p)
{
    constexpr int PITCH = 80;
    using stage_t = std::conditional_t<FP32ACC, float, double>;
    using acc_t   = std::conditional_t<FP32ACC, v4f, v4d>;
    __shared__ stage_t as[16][PITCH];
    __shared__ stage_t bs[16][PITCH];
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm   = wave >> 1;
    const int wn   = wave & 1;
    const int l16  = lane & 15;
    const int lk   = lane >> 4;
    const int64_t row0 = (int64_t)blockIdx.y * 64;
    const int64_t col0 = (int64_t)blockIdx.x * 64;
    int64_t ao, bo, co;
    batch_offsets(p, ao, bo, co);
    const float* a = static_cast<const float*>(p.a) + ao;
    const float* b = static_cast<const float*>(p.b) + bo;
    // this thread's piece of each tile: `major` indexes the strided dimension, `minor` the
    // contiguous one (4 elements)
    const int a_major = A_KCONT ? tid >> 2 : tid >> 4;        // row       | k
    const int a_minor = A_KCONT ? (tid & 3) * 4 : (tid & 15) * 4; // k     | row
    const int b_major = B_NCONT ? tid >> 4 : tid >> 2;        // k         | column
    const int b_minor = B_NCONT ? (tid & 15) * 4 : (tid & 3) * 4; // column | k

    auto load_a = [&](int64_t k0) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        const int64_t row = row0 + (A_KCONT ? a_major : a_minor);
        const int64_t kk  = k0 + (A_KCONT ? a_minor : a_major);
        const float* src  = a + row * p.a_sm + kk * p.a_sk;
        const int64_t lim = A_KCONT ? p.k - kk : p.m - row; // elements left along the contiguous axis
        const bool inside = A_KCONT ? row < p.m : kk < p.k;
        if(inside && lim >= 4)
            v = *reinterpret_cast<const v4f*>(src);
        else if(inside)
        {
#pragma unroll
            for(int e = 0; e < 4; e++)
                if(e < lim)
                    v[e] = src[e];
        }
        return v;
    };
    auto load_b = [&](int64_t k0) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        const int64_t col = col0 + (B_NCONT ? b_minor : b_major);
        const int64_t kk  = k0 + (B_NCONT ? b_major : b_minor);
        const float* src  = b + kk * p.b_sk + col * p.b_sn;
        const int64_t lim = B_NCONT ? p.n - col : p.k - kk;
        const bool inside = B_NCONT ? kk < p.k : col < p.n;
        if(inside && lim >= 4)
            v = *reinterpret_cast<const v4f*>(src);
        else if(inside)
        {
#pragma unroll
            for(int e = 0; e < 4; e++)
                if(e < lim)
                    v[e] = src[e];
        }
        return v;
    };

    acc_t acc[2][2];
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < 2; j++)
            acc[i][j] = acc_t{0, 0, 0, 0};

    // x * 1.0f is x for every float, so "no scale" needs no second code path
    const float alpha = p.scale != nullptr ? p.scale[0] : 1.0f;
    auto stage = [&](const v4f& va, const v4f& vb) {
#pragma unroll
        for(int e = 0; e < 4; e++)
        {
            if(A_KCONT)
                as[a_minor + e][a_major] = (stage_t)va[e];
            else
                as[a_major][a_minor + e] = (stage_t)va[e];
            if(B_NCONT)
                bs[b_major][b_minor + e] = (stage_t)vb[e];
            else
                bs[b_minor + e][b_major] = (stage_t)vb[e];
        }
    };
    auto multiply = [&] {
#pragma unroll
        for(int kk0 = 0; kk0 < 16; kk0 += 4)
        {
            stage_t av[2], bv[2];
#pragma unroll
            for(int i = 0; i < 2; i++)
                av[i] = as[kk0 + lk][wm * 32 + i * 16 + l16];
#pragma unroll
            for(int j = 0; j < 2; j++)
                bv[j] = bs[kk0 + lk][wn * 32 + j * 16 + l16];
#pragma unroll
            for(int i = 0; i < 2; i++)
#pragma unroll
                for(int j = 0; j < 2; j++)
                {
                    if constexpr(FP32ACC)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[j], acc[i][j], 0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[i], bv[j], acc[i][j], 0, 0, 0);
                }
        }
    };

    if(row0 + 64 <= p.m && col0 + 64 <= p.n && p.k % 16 == 0 && p.k >= 96)
    {
        // A tile inside the matrices and a K long enough to gain by it: every load is one whole
        // vector, so the loads carry no branches and three K steps of operands can be in flight (the
        // sixteen matrix instructions of a step last less than a load from memory does).  The three
        // register sets take turns; a load past the last step reads the last step again and is not
        // used.
        const float* a_at = a + (row0 + (A_KCONT ? a_major : a_minor)) * p.a_sm + (A_KCONT ? a_minor : a_major) * p.a_sk;
        const float* b_at = b + (col0 + (B_NCONT ? b_minor : b_major)) * p.b_sn + (B_NCONT ? b_major : b_minor) * p.b_sk;
        const int64_t k_last = p.k - 16;
        auto fetch_a = [&](int64_t k0) {
            return *reinterpret_cast<const v4f*>(a_at + (k0 < k_last ? k0 : k_last) * p.a_sk);
        };
        auto fetch_b = [&](int64_t k0) {
            return *reinterpret_cast<const v4f*>(b_at + (k0 < k_last ? k0 : k_last) * p.b_sk);
        };
        v4f va0 = fetch_a(0), vb0 = fetch_b(0);
        v4f va1 = fetch_a(16), vb1 = fetch_b(16);
        v4f va2 = fetch_a(32), vb2 = fetch_b(32);
        int64_t k0 = 0;
        auto step = [&](v4f& va, v4f& vb) {
            stage(va, vb);
            __syncthreads();
            va = fetch_a(k0 + 48);
            vb = fetch_b(k0 + 48);
            multiply();
            __syncthreads();
            k0 += 16;
        };
        auto last_step = [&](const v4f& va, const v4f& vb) {
            stage(va, vb);
            __syncthreads();
            multiply();
            __syncthreads();
        };
        int64_t steps = p.k / 16;
        for(; steps >= 3; steps -= 3)
        {
            step(va0, vb0);
            step(va1, vb1);
            step(va2, vb2);
        }
        if(steps >= 1)
            last_step(va0, vb0);
        if(steps == 2)
            last_step(va1, vb1);
    }
    else
    {
        v4f va = load_a(0);
        v4f vb = load_b(0);
        for(int64_t k0 = 0; k0 < p.k; k0 += 16)
        {
            stage(va, vb);
            __syncthreads();
            if(k0 + 16 < p.k)
            {
                va = load_a(k0 + 16);
                vb = load_b(k0 + 16);
            }
            multiply();
            __syncthreads();
        }
    }
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int r = 0; r < 4; r++)
        {
            const int64_t row = row0 + wm * 32 + i * 16 + (FP32ACC ? 4 * lk + r : 4 * r + lk);
            if(row >= p.m)
                continue;
#pragma unroll
            for(int j = 0; j < 2; j++)
            {
                const int64_t col = col0 + wn * 32 + j * 16 + l16;
                if(col < p.n)
                    static_cast<float*>(p.c)[co + row * p.ldc + col] =
                        (float)acc[i][j][r] * alpha;
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

// The innermost dimension is contiguous in the input too (a permutation of the outer dimensions, a
// slice): rows of `run` 16-byte pieces are copied whole; only the row index is decomposed, in 32-bit
// arithmetic, once per piece.
struct row_copy_params
{
    const uint8_t* in;
    uint8_t* out;
    uint32_t lens[MI355_MAX_DIMS]; // outer dimensions
    int64_t strides[MI355_MAX_DIMS]; // their input strides in bytes
    uint32_t rows, run;              // run = 16-byte pieces per row
    int ndim;                        // number of outer dimensions
};

__global__ __launch_bounds__(256) void row_copy_kernel(row_copy_params p)
{
    const uint64_t total = (uint64_t)p.rows * p.run;
    const uint64_t step  = (uint64_t)gridDim.x * 256;
    for(uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step)
    {
        uint32_t row       = (uint32_t)(i / p.run);
        const uint32_t pc  = (uint32_t)(i - (uint64_t)row * p.run);
        int64_t off        = 0;
        for(int d = p.ndim - 1; d >= 0; d--)
        {
            const uint32_t q = row / p.lens[d];
            off += (int64_t)(row - q * p.lens[d]) * p.strides[d];
            row = q;
        }
        reinterpret_cast<v4u*>(p.out)[i] = *reinterpret_cast<const v4u*>(p.in + off + (int64_t)pc * 16);
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
    return mi355_dot_scaled(a, b, c, type, m, n, k, a_stride_m, a_stride_k, b_stride_k, b_stride_n, ldc, batch,
                            stride_a, stride_b, stride_c, nullptr, stream);
}

static int dot_launch(bool fp32acc,
                      const void* a,
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
                                const float* scale,
                                void* stream,
                                int64_t batch_inner    = 0,
                                int64_t stride_a_outer = 0,
                                int64_t stride_b_outer = 0,
                                int64_t stride_c_outer = -1) // -1: batch_inner dense blocks of stride_c
{
    if(type != MI355_F32 && type != MI355_F16 && type != MI355_BF16)
        return MI355_ERR_BAD_ARG;
    if(batch_inner < 0 || stride_a_outer < 0 || stride_b_outer < 0 || (batch_inner > 0 && batch % batch_inner != 0))
        return MI355_ERR_BAD_ARG;
    if((scale != nullptr || fp32acc) && type != MI355_F32)
        return MI355_ERR_UNSUPPORTED;
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
                 stride_a, stride_b, stride_c, type, scale};
    p.batch_inner    = batch_inner > 0 ? batch_inner : batch;
    p.stride_a_outer = stride_a_outer;
    p.stride_b_outer = stride_b_outer;
    p.stride_c_outer = stride_c_outer >= 0 ? stride_c_outer : p.batch_inner * stride_c;
    const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)batch);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // fp32 with contiguous rows or columns, everything the 16-byte loads touch aligned
    auto aligned4 = [](int64_t x) { return x % 4 == 0; };
    const bool a_k = a_stride_k == 1 && aligned4(a_stride_m);
    const bool a_m = a_stride_m == 1 && aligned4(a_stride_k);
    const bool b_n = b_stride_n == 1 && aligned4(b_stride_k);
    const bool b_k = b_stride_k == 1 && aligned4(b_stride_n);
    if(type == MI355_F32 && k > 0 && (a_k || a_m) && (b_n || b_k) && aligned4(stride_a) && aligned4(stride_b) &&
       aligned4(stride_a_outer) && aligned4(stride_b_outer) &&
       reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0)
    {
        if(fp32acc)
        {
            if(a_k && b_n)
                hipLaunchKernelGGL((dot_f32_mfma_kernel<true, true, true>), grid, dim3(256), 0, s, p);
            else if(a_k)
                hipLaunchKernelGGL((dot_f32_mfma_kernel<true, false, true>), grid, dim3(256), 0, s, p);
            else if(b_n)
                hipLaunchKernelGGL((dot_f32_mfma_kernel<false, true, true>), grid, dim3(256), 0, s, p);
            else
                hipLaunchKernelGGL((dot_f32_mfma_kernel<false, false, true>), grid, dim3(256), 0, s, p);
            return mi355_launch_status();
        }
        if(a_k && b_n)
            hipLaunchKernelGGL((dot_f32_mfma_kernel<true, true>), grid, dim3(256), 0, s, p);
        else if(a_k)
            hipLaunchKernelGGL((dot_f32_mfma_kernel<true, false>), grid, dim3(256), 0, s, p);
        else if(b_n)
            hipLaunchKernelGGL((dot_f32_mfma_kernel<false, true>), grid, dim3(256), 0, s, p);
        else
            hipLaunchKernelGGL((dot_f32_mfma_kernel<false, false>), grid, dim3(256), 0, s, p);
        return mi355_launch_status();
    }
    hipLaunchKernelGGL(dot_float_mfma_kernel, grid, dim3(256), 0, s, p);
    return mi355_launch_status();
}

extern "C" int mi355_dot_scaled(const void* a,
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
                                const float* scale,
                                void* stream)
{
    return dot_launch(false, a, b, c, type, m, n, k, a_stride_m, a_stride_k, b_stride_k, b_stride_n, ldc, batch,
                      stride_a, stride_b, stride_c, scale, stream);
}

extern "C" int mi355_dot_fp32acc(const void* a,
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
                                 const float* scale,
                                 void* stream)
{
    return dot_launch(true, a, b, c, type, m, n, k, a_stride_m, a_stride_k, b_stride_k, b_stride_n, ldc, batch,
                      stride_a, stride_b, stride_c, scale, stream);
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
    hipStream_t s = static_cast<hipStream_t>(stream);
    // last dimension contiguous in the input, rows a whole number of aligned 16-byte pieces
    {
        int last = ndim - 1;
        while(last > 0 && lens[last] == 1)
            last--;
        const int64_t row_bytes = lens[last] * elem_size;
        bool ok = strides[last] == 1 && row_bytes % 16 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(out) % 16 == 0 && p.total / lens[last] < (1ll << 31) &&
                  row_bytes / 16 < (1ll << 31);
        row_copy_params q{};
        q.ndim = 0;
        for(int d = 0; d < last && ok; d++)
        {
            if(lens[d] == 1)
                continue;
            ok = (strides[d] * elem_size) % 16 == 0 && lens[d] < (1ll << 31);
            q.lens[q.ndim]    = (uint32_t)lens[d];
            q.strides[q.ndim] = strides[d] * elem_size;
            q.ndim++;
        }
        if(ok)
        {
            q.in   = p.in;
            q.out  = p.out;
            q.rows = (uint32_t)(p.total / lens[last]);
            q.run  = (uint32_t)(row_bytes / 16);
            int64_t nb = ((int64_t)q.rows * q.run + 255) / 256;
            if(nb > 256 * 16)
                nb = 256 * 16;
            hipLaunchKernelGGL(row_copy_kernel, dim3((unsigned)nb), dim3(256), 0, s, q);
            return mi355_launch_status();
        }
    }
    int64_t blocks = (p.total + 255) / 256;
    if(blocks > 256 * 16)
        blocks = 256 * 16;
    const dim3 grid((unsigned)blocks);
    switch(elem_size)
    {
    case 1: hipLaunchKernelGGL(gather_kernel<uint8_t>, grid, dim3(256), 0, s, p); break;
    case 2: hipLaunchKernelGGL(gather_kernel<uint16_t>, grid, dim3(256), 0, s, p); break;
    case 4: hipLaunchKernelGGL(gather_kernel<uint32_t>, grid, dim3(256), 0, s, p); break;
    default: hipLaunchKernelGGL(gather_kernel<uint64_t>, grid, dim3(256), 0, s, p); break;
    }
    return mi355_launch_status();
}

extern "C" int mi355_dot_batch2(const void* a,
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
                                int64_t batch_outer,
                                int64_t batch_inner,
                                int64_t stride_a_outer,
                                int64_t stride_a_inner,
                                int64_t stride_b_outer,
                                int64_t stride_b_inner,
                                const float* scale,
                                int32_t fp32acc,
                                void* stream)
{
    if(batch_outer < 0 || batch_inner < 0)
        return MI355_ERR_BAD_ARG;
    if(batch_outer == 0 || batch_inner == 0)
        return MI355_OK;
    if(batch_outer > 65535 / batch_inner)
        return MI355_ERR_UNSUPPORTED;
    return dot_launch(fp32acc != 0, a, b, c, type, m, n, k, a_stride_m, a_stride_k, b_stride_k, b_stride_n, n,
                      batch_outer * batch_inner, stride_a_inner, stride_b_inner, m * n, scale, stream, batch_inner,
                      stride_a_outer, stride_b_outer);
}

extern "C" int mi355_dot_batch2_strided(const void* a,
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
                                        int64_t batch_outer,
                                        int64_t batch_inner,
                                        int64_t stride_a_outer,
                                        int64_t stride_a_inner,
                                        int64_t stride_b_outer,
                                        int64_t stride_b_inner,
                                        int64_t stride_c_outer,
                                        int64_t stride_c_inner,
                                        const float* scale,
                                        int32_t fp32acc,
                                        void* stream)
{
    if(batch_outer < 0 || batch_inner < 0 || stride_c_outer < 0 || stride_c_inner < 0)
        return MI355_ERR_BAD_ARG;
    if(batch_outer == 0 || batch_inner == 0)
        return MI355_OK;
    if(batch_outer > 65535 / batch_inner)
        return MI355_ERR_UNSUPPORTED;
    return dot_launch(fp32acc != 0, a, b, c, type, m, n, k, a_stride_m, a_stride_k, b_stride_k, b_stride_n, ldc,
                      batch_outer * batch_inner, stride_a_inner, stride_b_inner, stride_c_inner, scale, stream,
                      batch_inner, stride_a_outer, stride_b_outer, stride_c_outer);
}
