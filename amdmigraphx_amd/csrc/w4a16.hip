// int4 weight-only GEMM / GEMV with group-wise fp16 scales.
//
// Decode shapes (small M) move K*N/2 bytes of weights for 2*M*N*K flops, i.e.
// they are bound by HBM, not by arithmetic: the kernel streams the packed
// nibbles with 16-byte loads (one wave reads 1 KiB of one weight row per
// instruction), unpacks and dequantizes in registers, multiplies into fp32
// partial sums per lane and reduces across the wave at the end of the row.
//
// Arithmetic contract (ref target, op by op):
//   w[n,k] = half_rtz( float( (q - zp) * scale ) )      exact product, RTZ to half
//   out    = half_rtz( float( sum_k double(a) * double(w) ) )
// The products a*w are exact in fp32 (11 x 11 significant bits); only the
// running sum differs from the reference's double accumulator in the last
// bits, which the parity tolerance covers.
#include "common.h"

namespace {

constexpr int W4_THREADS = 256;

struct w4_params
{
    const uint16_t* a;
    int64_t lda;
    const uint8_t* w;
    const uint16_t* scales;
    const uint8_t* zp;
    int zp_mode, zp_scalar;
    uint16_t* out;
    int64_t ldc;
    int m, n, k, group;
};

MI355_DEVINL float wave_sum(float v)
{
#pragma unroll
    for(int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}

MI355_DEVINL float dequant_weight(int q, int zp, float scale)
{
    // (q - zp) * scale is exact in fp32; the reference stores it as half (RTZ)
    return half_to_f32(f32_to_half_rtz((float)(q - zp) * scale));
}

// One wave per weight row n; MB activation rows per pass.
template <int MB>
__global__ __launch_bounds__(W4_THREADS) void w4a16_gemv_kernel(w4_params p)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n    = blockIdx.x * (W4_THREADS / 64) + wave;
    if(n >= p.n)
        return;
    const int kbytes        = p.k >> 1;
    const int groups        = p.k / p.group;
    const uint8_t* wrow     = p.w + (int64_t)n * kbytes;
    const uint16_t* srow    = p.scales + (int64_t)n * groups;

    for(int mb = 0; mb < p.m; mb += MB)
    {
        float acc[MB];
#pragma unroll
        for(int i = 0; i < MB; i++)
            acc[i] = 0.f;

        for(int kb = lane * 16; kb < kbytes; kb += 64 * 16)
        {
            const uint4 wv  = *reinterpret_cast<const uint4*>(wrow + kb);
            const int k0    = kb * 2; // first k of this lane's 32 weights
            const int g     = k0 / p.group;
            const float sc  = half_to_f32(srow[g]);
            int zp          = p.zp_scalar;
            if(p.zp_mode == MI355_W4_ZP_GROUP)
                zp = p.zp[(int64_t)n * groups + g];
            else if(p.zp_mode == MI355_W4_ZP_PACKED)
            {
                uint8_t zb = p.zp[(int64_t)n * ((groups + 1) / 2) + (g >> 1)];
                zp         = (g & 1) ? (zb >> 4) : (zb & 0xf);
            }
            const uint32_t words[4] = {wv.x, wv.y, wv.z, wv.w};
            float wf[32];
#pragma unroll
            for(int d = 0; d < 4; d++)
#pragma unroll
                for(int e = 0; e < 8; e++)
                    wf[d * 8 + e] = dequant_weight((words[d] >> (4 * e)) & 0xf, zp, sc);
#pragma unroll
            for(int i = 0; i < MB; i++)
            {
                if(mb + i < p.m)
                {
                    const uint4* ap =
                        reinterpret_cast<const uint4*>(p.a + (int64_t)(mb + i) * p.lda + k0);
#pragma unroll
                    for(int c = 0; c < 4; c++)
                    {
                        const uint4 av         = ap[c];
                        const uint32_t aw[4]   = {av.x, av.y, av.z, av.w};
#pragma unroll
                        for(int e = 0; e < 4; e++)
                        {
                            acc[i] += half_to_f32((uint16_t)(aw[e] & 0xffff)) * wf[c * 8 + 2 * e];
                            acc[i] += half_to_f32((uint16_t)(aw[e] >> 16)) * wf[c * 8 + 2 * e + 1];
                        }
                    }
                }
            }
        }
#pragma unroll
        for(int i = 0; i < MB; i++)
        {
            float s = wave_sum(acc[i]);
            if(lane == 0 && mb + i < p.m)
                p.out[(int64_t)(mb + i) * p.ldc + n] = f32_to_half_rtz(s);
        }
    }
}

} // namespace

extern "C" int mi355_w4a16_gemm(const void* a,
                                int64_t lda,
                                const void* w_packed,
                                const void* scales,
                                const void* zp,
                                int32_t zp_mode,
                                int32_t zp_scalar,
                                void* out,
                                int64_t ldc,
                                int64_t m,
                                int64_t n,
                                int64_t k,
                                int64_t group,
                                void* stream)
{
    if(a == nullptr || w_packed == nullptr || scales == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    if(m < 0 || n < 0 || k <= 0 || group <= 0)
        return MI355_ERR_BAD_ARG;
    if(zp_mode != MI355_W4_ZP_SCALAR && zp_mode != MI355_W4_ZP_GROUP &&
       zp_mode != MI355_W4_ZP_PACKED)
        return MI355_ERR_BAD_ARG;
    if(zp_mode != MI355_W4_ZP_SCALAR && zp == nullptr)
        return MI355_ERR_BAD_ARG;
    if(zp_mode == MI355_W4_ZP_SCALAR && (zp_scalar < 0 || zp_scalar > 15))
        return MI355_ERR_BAD_ARG;
    if(lda < k || ldc < n)
        return MI355_ERR_BAD_ARG;
    // a lane owns 32 consecutive weights (16 bytes) that must share one scale,
    // and reads its activations as 16-byte vectors
    if(group % 32 != 0 || k % group != 0 || lda % 8 != 0 ||
       reinterpret_cast<uintptr_t>(a) % 16 != 0 || reinterpret_cast<uintptr_t>(w_packed) % 16 != 0)
        return MI355_ERR_UNSUPPORTED;
    if(k > (1 << 30) || n > (1 << 30) || m > (1 << 30))
        return MI355_ERR_UNSUPPORTED;
    if(m == 0 || n == 0)
        return MI355_OK;
    w4_params p;
    p.a         = static_cast<const uint16_t*>(a);
    p.lda       = lda;
    p.w         = static_cast<const uint8_t*>(w_packed);
    p.scales    = static_cast<const uint16_t*>(scales);
    p.zp        = static_cast<const uint8_t*>(zp);
    p.zp_mode   = zp_mode;
    p.zp_scalar = zp_scalar;
    p.out       = static_cast<uint16_t*>(out);
    p.ldc       = ldc;
    p.m         = (int)m;
    p.n         = (int)n;
    p.k         = (int)k;
    p.group     = (int)group;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid((unsigned)((n + 3) / 4));
    if(m == 1)
        hipLaunchKernelGGL(w4a16_gemv_kernel<1>, grid, dim3(W4_THREADS), 0, s, p);
    else if(m == 2)
        hipLaunchKernelGGL(w4a16_gemv_kernel<2>, grid, dim3(W4_THREADS), 0, s, p);
    else
        hipLaunchKernelGGL(w4a16_gemv_kernel<4>, grid, dim3(W4_THREADS), 0, s, p);
    return mi355_launch_status();
}
