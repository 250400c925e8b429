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
#include <type_traits>
#include <utility>
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
    float* partial;        // room for split-K partial sums (null: none)
    size_t partial_bytes;  // host side only
    int chunks_per_share;  // set by the launcher when it splits
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


// ---------------------------------------------------------------------------
// M = 1 streaming GEMV.
//
// A workgroup of 8 waves keeps the activation vector in LDS; each wave owns
// one weight row at a time.  Lane l reads the 16-byte runs (c*64 + l) of the
// packed row, c = 0..NCH-1, so one load instruction covers 1 KiB of contiguous
// weights and the whole row (NCH KiB) is in flight at once; the loads of the
// wave's next row are issued before the current row is consumed.
//
// Dequantization runs on packed halves, one fused multiply-add per pair of
// weights.  The nibbles k and k+4 of a dword are masked in place at bits 4..7
// of the two halves of a register: read as half-precision subnormals they are
// q * 2^-20 exactly.  fma(q * 2^-20, scale * 2^20, -zp * scale) then forms
// (q - zp) * scale exactly inside the FMA and rounds it once -- the one rounding
// of the reference's float -> half store -- with the half-precision rounding
// mode of the wave set to round-toward-zero so that it matches that truncation
// bit for bit.  This needs scale * 2^20 and zp * scale to be exact halves: zp
// in {0, 1, 2, 4, 8} and |scale| below 2^-5; a lane whose scale is outside
// that range (or is not finite) takes the three-instruction form instead
// (1024 + q built in the mantissa, minus 1024 + zp, times scale).
// v_dot2_f32_f16 then multiplies by the matching activation pair and
// accumulates in fp32.
// The activations sit in LDS already paired (k, k+4) and laid out
// [chunk][dword][lane] so a wave's 16-byte reads are conflict free.
// Each row's 64 partial sums are reduced with DPP row operations.
// ---------------------------------------------------------------------------
constexpr int GV_THREADS = 512;
constexpr int GV_WAVES   = GV_THREADS / 64;

MI355_DEVINL float dpp_row_sum(float v)
{
    // 16-lane sums in every lane of each DPP row
    int x = __builtin_bit_cast(int, v);
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xf, 0xf, false));
    x = __builtin_bit_cast(int, v);
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xf, 0xf, false));
    x = __builtin_bit_cast(int, v);
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, x, 0x141, 0xf, 0xf, false));
    x = __builtin_bit_cast(int, v);
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, x, 0x140, 0xf, 0xf, false));
    return v;
}

MI355_DEVINL float wave_sum_dpp(float v)
{
    v        = dpp_row_sum(v);
    int x    = __builtin_bit_cast(int, v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 48));
    return (r0 + r1) + (r2 + r3);
}

MI355_DEVINL uint32_t and_or(uint32_t x, uint32_t mask, uint32_t bits)
{
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(mask), "v"(bits));
    return r;
}

constexpr int GV_DEPTH = 4; // 16-byte runs per lane kept in flight

__global__ __launch_bounds__(GV_THREADS) void w4a16_gemv_m1_kernel(w4_params p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t gv_lds[];
    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    // wave-uniform values are pinned to scalar registers so that the loop
    // control around the pipeline below is scalar branches, not exec masking
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kbytes = p.k >> 1;
    const int groups = p.k / p.group;
    const int nch    = p.k >> 11; // 1 KiB runs per packed row
    // scale index of this lane inside a run: the group size divides 2048
    const int gshift = __builtin_ctz(p.group);
    const int lane_g = (lane * 32) >> gshift;
    const int run_g  = 2048 >> gshift;

    // Half-precision arithmetic of this wave rounds toward zero from here on
    // (MODE.fp_round bits 3:2); fp32 rounding is untouched.  Written as inline
    // assembly: the compiler tracks s_setreg it emits itself and would put the
    // default mode back in front of the first packed-half instruction.  All
    // half arithmetic below sits behind the workgroup barrier, which this
    // statement cannot move across.
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 2, 2), 3" ::: "memory");

    // The activation loads go out first so that they are not queued behind the
    // weight stream.  Slot s = (c*4 + d)*64 + l of the LDS copy holds the 8
    // halves a[k0 .. k0+7], k0 = (c*64 + l)*32 + 8*d, reordered to
    // (0,4,1,5,2,6,3,7).
    const int a_slots = p.k >> 3;
    uint4 areg[4];
#pragma unroll
    for(int it = 0; it < 4; it++)
    {
        const int s  = tid + it * GV_THREADS;
        const int l  = s & 63;
        const int cd = s >> 6;
        const int k0 = ((cd >> 2) * 64 + l) * 32 + 8 * (cd & 3);
        if(s < a_slots)
            areg[it] = *reinterpret_cast<const uint4*>(p.a + k0);
    }

    // this wave's rows: row0, row0 + stride, ...; its work items are the 1 KiB
    // runs of those rows in order
    const int stride = gridDim.x * GV_WAVES;
    const int row0   = blockIdx.x * GV_WAVES + wave;
    const int nrows  = row0 < p.n ? (p.n - 1 - row0) / stride + 1 : 0;
    const int total  = __builtin_amdgcn_readfirstlane(nrows * nch);

    v4u wbuf[GV_DEPTH];
    uint16_t sbuf[GV_DEPTH];
    int ld_row = row0, ld_c = 0; // item the next issue() fetches
    auto issue = [&](int slot) {
        const uint8_t* q = p.w + (int64_t)ld_row * kbytes + ld_c * 1024 + lane * 16;
        wbuf[slot]       = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(q));
        sbuf[slot]       = p.scales[(int64_t)ld_row * groups + ld_c * run_g + lane_g];
        if(++ld_c == nch)
        {
            ld_c = 0;
            ld_row += stride;
        }
    };
#pragma unroll
    for(int u = 0; u < GV_DEPTH; u++)
        if(u < total)
            issue(u);

#pragma unroll
    for(int it = 0; it < 4; it++)
    {
        const int s = tid + it * GV_THREADS;
        if(s < a_slots)
        {
            const uint4 v = areg[it];
            uint4 o;
            o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
            o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
            o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
            o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
            *reinterpret_cast<uint4*>(gv_lds + s * 16) = o;
        }
    }
    __syncthreads();

    // 1024 + zp as half bits (zp in 0..15 sits in the low mantissa bits); built
    // from integers so that no float -> half conversion instruction appears in
    // this kernel: the compiler resets the rounding mode in front of those.
    const uint32_t zbits = 0x6400u | (uint32_t)p.zp_scalar;
    const h2 zoff2       = __builtin_bit_cast(h2, zbits | (zbits << 16));
    // mask and magic live in registers so that (w & mask) | magic is one
    // v_and_or_b32 (the three-operand form takes no literal constants here)
    uint32_t nib_mask = 0x000F000Fu, magic = 0x64006400u;
    asm volatile("" : "+v"(nib_mask), "+v"(magic));
    const int zpv      = p.zp_scalar;
    const bool zp_pow2 = (zpv & (zpv - 1)) == 0; // 0, 1, 2, 4, 8
    const int zp_log2  = zpv <= 1 ? 0 : (zpv == 2 ? 1 : (zpv == 4 ? 2 : 3));

    float acc[4] = {0.f, 0.f, 0.f, 0.f}; // independent chains for the dot units
    int cs_row = row0, cs_c = 0;         // item being consumed

    auto consume = [&](int slot) {
        const uint16_t sb    = sbuf[slot];
        const _Float16 sc    = __builtin_bit_cast(_Float16, sb);
        const h2 scv         = {sc, sc};
        const uint32_t wa[4] = {wbuf[slot].x, wbuf[slot].y, wbuf[slot].z, wbuf[slot].w};
        // scale * 2^20 by adding 20 to the exponent field; exact for normal
        // scales below 2^-5 (exponent field 1..10)
        const uint32_t sexp = (sb >> 10) & 0x1fu;
        // taken by the whole wave or not at all: the general form is right for
        // every lane, so one out-of-range scale just costs the wave speed
        const bool fast =
            __builtin_amdgcn_ballot_w64(zp_pow2 && sexp >= 1 && sexp <= 10) == ~0ull;
        const uint8_t* abase = gv_lds + (cs_c * 256 + lane) * 16;
        if(fast)
        {
            const uint32_t sup = (uint32_t)sb + (20u << 10);
            const h2 scv_up    = __builtin_bit_cast(h2, sup | (sup << 16));
            // -zp * scale: exponent raised by log2(zp), sign flipped (zp == 0: +0)
            const uint32_t zsb =
                zpv == 0 ? 0u : (((uint32_t)sb + ((uint32_t)zp_log2 << 10)) ^ 0x8000u);
            const h2 zs = __builtin_bit_cast(h2, zsb | (zsb << 16));
#pragma unroll
            for(int d = 0; d < 4; d++)
            {
                const uint4 av       = *reinterpret_cast<const uint4*>(abase + d * 1024);
                const uint32_t ap[4] = {av.x, av.y, av.z, av.w};
                // the four nibble pairs of the dword advance in lock step so that
                // dependent packed-half instructions are never back to back
                h2 x[4];
                x[0] = __builtin_bit_cast(h2, (wa[d] << 4) & 0x00F000F0u);
                x[1] = __builtin_bit_cast(h2, wa[d] & 0x00F000F0u);
                x[2] = __builtin_bit_cast(h2, (wa[d] >> 4) & 0x00F000F0u);
                x[3] = __builtin_bit_cast(h2, (wa[d] >> 8) & 0x00F000F0u);
#pragma unroll
                for(int j = 0; j < 4; j++)
                    x[j] = __builtin_elementwise_fma(x[j], scv_up, zs);
#pragma unroll
                for(int j = 0; j < 4; j++)
                    acc[j] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, ap[j]), x[j], acc[j],
                                                    false);
            }
        }
        else
        {
#pragma unroll
            for(int d = 0; d < 4; d++)
            {
                const uint4 av       = *reinterpret_cast<const uint4*>(abase + d * 1024);
                const uint32_t ap[4] = {av.x, av.y, av.z, av.w};
                h2 x[4];
#pragma unroll
                for(int j = 0; j < 4; j++)
                    x[j] = __builtin_bit_cast(h2, and_or(wa[d] >> (4 * j), nib_mask, magic));
#pragma unroll
                for(int j = 0; j < 4; j++)
                    x[j] = x[j] - zoff2;
#pragma unroll
                for(int j = 0; j < 4; j++)
                    x[j] = x[j] * scv;
#pragma unroll
                for(int j = 0; j < 4; j++)
                    acc[j] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, ap[j]), x[j], acc[j],
                                                    false);
            }
        }
        if(++cs_c == nch)
        {
            const float t = wave_sum_dpp((acc[0] + acc[1]) + (acc[2] + acc[3]));
            if(lane == 0)
                p.out[cs_row] = f32_to_half_rtz(t);
            acc[0] = acc[1] = acc[2] = acc[3] = 0.f;
            cs_c                              = 0;
            cs_row += stride;
        }
    };

    // GV_DEPTH register slots rotate: a slot is refilled with the item
    // GV_DEPTH ahead as soon as it has been consumed
    for(int base = 0; base < total; base += GV_DEPTH)
    {
#pragma unroll
        for(int u = 0; u < GV_DEPTH; u++)
        {
            if(base + u < total)
            {
                consume(u);
                if(base + u + GV_DEPTH < total)
                    issue(u);
            }
        }
    }
}

constexpr int GV_MAX_K = 16384; // activations staged in LDS: 4 slots of 8 halves per thread, 512 threads

int launch_gemv_m1(const w4_params& p, hipStream_t s)
{
    const int lds    = p.k * 2;
    const int blocks = (p.n + GV_WAVES - 1) / GV_WAVES;
    // one resident set of workgroups: every wave walks several rows with its
    // next runs in flight, instead of a second round of workgroups starting cold
    const int per_cu = lds <= 16384 ? 4 : 2;
    const int grid   = min(blocks, 256 * per_cu);
    hipLaunchKernelGGL(w4a16_gemv_m1_kernel, dim3(grid), dim3(GV_THREADS), lds, s, p);
    return mi355_launch_status();
}

#include "w4a16_mfma.h"
#include "w4a16_tile.h"

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
    return mi355_w4a16_gemm_ws(a, lda, w_packed, scales, zp, zp_mode, zp_scalar, out, ldc, m, n, k, group, nullptr,
                               0, stream);
}

extern "C" size_t mi355_w4a16_gemm_workspace_size(int64_t m, int64_t n, int64_t k, int64_t group)
{
    if(m < 2 || n <= 0 || k <= 0 || group <= 0 || k % 128 != 0 || n % 16 != 0 || k > (1 << 30) || n > (1 << 30) ||
       m > (1 << 30))
        return 0;
    if(m > 32 && n % TL_BN == 0)
    {
        const int shares = tile_gemm_shares((int)m, (int)n, (int)k);
        return shares > 1 ? (size_t)shares * m * n * 4 : 0;
    }
    // the matrix-core kernel for few rows: the widest column tile any zero-point form may take
    // (an upper bound for the others)
    int shares = 1;
    if(m <= 32)
        shares = mfma_gemm_shares<4>((int)n, (int)k);
    else if(m <= 64)
        shares = mfma_gemm_shares<2>((int)n, (int)k);
    return shares > 1 ? (size_t)shares * m * n * 4 : 0;
}

extern "C" int mi355_w4a16_gemm_ws(const void* a,
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
                                   void* workspace,
                                   size_t workspace_bytes,
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
    p.partial   = reinterpret_cast<uintptr_t>(workspace) % 16 == 0 ? static_cast<float*>(workspace) : nullptr;
    p.partial_bytes    = p.partial != nullptr ? workspace_bytes : 0;
    p.chunks_per_share = 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if(m == 1 && zp_mode == MI355_W4_ZP_SCALAR && k % 2048 == 0 && k <= GV_MAX_K &&
       (group & (group - 1)) == 0 && group <= 2048)
        return launch_gemv_m1(p, s);
    if(m >= 2 && mfma_gemm_supported(p))
        return launch_mfma_gemm(p, s);
    dim3 grid((unsigned)((n + 3) / 4));
    if(m == 1)
        hipLaunchKernelGGL(w4a16_gemv_kernel<1>, grid, dim3(W4_THREADS), 0, s, p);
    else if(m == 2)
        hipLaunchKernelGGL(w4a16_gemv_kernel<2>, grid, dim3(W4_THREADS), 0, s, p);
    else
        hipLaunchKernelGGL(w4a16_gemv_kernel<4>, grid, dim3(W4_THREADS), 0, s, p);
    return mi355_launch_status();
}
