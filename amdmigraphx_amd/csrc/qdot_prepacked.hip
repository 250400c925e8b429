// quant_dot with few rows (M <= 16) over a constant B reordered once, ahead of time.
//
// A linear layer applied to a handful of rows streams its whole weight matrix for almost no
// arithmetic: the time is the time to read B once.  The weights are constants of the graph, so
// their layout in memory is free, and the reordering stores B as the matrix-core operands
// themselves:
//
//   tile (T, S) = columns 16T .. 16T+15 against k = 64S .. 64S+63, 1 KiB:
//     lane l = 16*kq + c holds the 16 bytes B[64S + 16kq .. +16, 16T + c].
//   Tiles lie in (T, S) order, so what one wave reads is one contiguous run.
//
// A wave owns one tile column T and a share of K.  Per step it loads 1 KiB of B with one
// instruction (every byte of every 128-byte line used, nothing staged through the LDS, no
// transposing reads), the matching 16 x 64 piece of A straight from the row-major activations
// (lane l: row l % 16, 16 bytes at k = 64S + 16*(l / 16): the other operand as it stands; A is
// small and stays in the caches), and issues one v_mfma_i32_16x16x64_i8 -- or two
// v_mfma_f32_16x16x32_{fp8_fp8, bf8_bf8} on the low and high halves of the same registers.  B is
// the instruction's first operand, so a lane ends up with 4 consecutive columns of one row of C
// and stores them with one instruction.  The waves that share a tile column add their partial
// sums through the LDS in a fixed order and the first of them applies the dequantizing epilogue
// (the arithmetic of reduce_partials_kernel / the one-pass kernels): one launch, no workspace,
// nothing to clear.
#include "common.h"
#include <type_traits>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

constexpr int QDP_WAVES = 16; // waves per workgroup

struct qdp_params
{
    const uint8_t* a;
    const uint8_t* b; // reordered tiles
    void* c;
    int m, n, k;
    int64_t lda, ldc;
    const float* scale_a;
    const float* scale_b;
    const int32_t* colsum_b;
    const int32_t* rowsum_a;
    const float* bias;
    int scale_a_mode, scale_b_mode, zp_a, zp_b;
    int n_tiles, ksteps;
    int wk;           // waves that share one tile column (split K among them)
    int per;          // K steps per wave
    int tiles_per_wg; // QDP_WAVES / wk: tile columns per workgroup, at most
    int grid;         // workgroups; workgroup g takes tile columns [g * n_tiles / grid, (g + 1) * n_tiles / grid)
    int vec_store;    // C takes aligned stores of 4 outputs
    uint32_t k16_magic; // floor(2^32 / (K / 16)) + 1: i / (K / 16) = umulhi(i, magic) for the i used here
};

// one thread per 16-byte piece of the reordered matrix; B is addressed by element strides, so
// [K, N] and [N, K] sources (and views of them) need no copy first
__global__ __launch_bounds__(256) void qdp_prepack_kernel(
    const uint8_t* b, int64_t b_sk, int64_t b_sn, uint4* out, int n_tiles, int ksteps)
{
    const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(piece >= (int64_t)n_tiles * ksteps * 64)
        return;
    const int l       = (int)(piece & 63);
    const int64_t ts  = piece >> 6;
    const int64_t t   = ts / ksteps;
    const int64_t s   = ts - t * ksteps;
    const int64_t col = 16 * t + (l & 15);
    const int64_t k0  = 64 * s + 16 * (l >> 4);
    uint32_t w[4];
#pragma unroll
    for(int d = 0; d < 4; d++)
    {
        uint32_t v = 0;
#pragma unroll
        for(int j = 0; j < 4; j++)
            v |= (uint32_t)b[(k0 + 4 * d + j) * b_sk + col * b_sn] << (8 * j);
        w[d] = v;
    }
    out[piece] = make_uint4(w[0], w[1], w[2], w[3]);
}

template <int FMT>
struct qdp_acc
{
    using scalar = float;
    using type   = v4f;
};
template <>
struct qdp_acc<0>
{
    using scalar = int32_t;
    using type   = v4i;
};

// FMT: 0 int8, 1 fp8 e4m3fn, 2 fp8 e5m2
template <int FMT>
MI355_DEVINL typename qdp_acc<FMT>::type qdp_mma(const v4u& bq, const v4u& aq, typename qdp_acc<FMT>::type acc)
{
    if constexpr(FMT == 0)
    {
        const v4i bv = {(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w};
        const v4i av = {(int)aq.x, (int)aq.y, (int)aq.z, (int)aq.w};
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(bv, av, acc, 0, 0, 0);
    }
    else
    {
        // K = 32 per instruction, 8 bytes per lane: the low halves of the two 16-byte pieces hold
        // the same k on both sides, and so do the high halves
        const long b0 = (long)(((uint64_t)bq.y << 32) | bq.x), b1 = (long)(((uint64_t)bq.w << 32) | bq.z);
        const long a0 = (long)(((uint64_t)aq.y << 32) | aq.x), a1 = (long)(((uint64_t)aq.w << 32) | aq.z);
        if constexpr(FMT == 1)
        {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(b0, a0, acc, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(b1, a1, acc, 0, 0, 0);
        }
        else
        {
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(b0, a0, acc, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(b1, a1, acc, 0, 0, 0);
        }
    }
}

template <int OUT>
MI355_DEVINL void qdp_store1(void* c, int64_t idx, float v)
{
    if constexpr(OUT == MI355_F32)
        static_cast<float*>(c)[idx] = v;
    else if constexpr(OUT == MI355_F16)
        static_cast<uint16_t*>(c)[idx] = convert_f32_to_half(v);
    else
        static_cast<uint16_t*>(c)[idx] = convert_f32_to_bf16(v);
}

// C = epilogue(sum) for the lane's 4 outputs: lane l holds row l % 16 of C, columns
// 16 * tile + 4 * (l / 16) .. + 3
template <int FMT, bool DEQ, int OUT>
MI355_DEVINL void qdp_finish(const qdp_params& p, typename qdp_acc<FMT>::type sum, int tile, int lane)
{
    using acc_t    = typename qdp_acc<FMT>::type;
    using scalar_t = typename qdp_acc<FMT>::scalar;
    const int m = lane & 15;
    if(m >= p.m)
        return;
    const int col     = 16 * tile + 4 * (lane >> 4);
    const int64_t idx = (int64_t)m * p.ldc + col;
    if constexpr(!DEQ)
    {
        if(p.vec_store)
            *reinterpret_cast<acc_t*>(static_cast<scalar_t*>(p.c) + idx) = sum;
        else
        {
#pragma unroll
            for(int e = 0; e < 4; e++)
                static_cast<scalar_t*>(p.c)[idx + e] = sum[e];
        }
    }
    else
    {
        float sa = 1.f;
        if(p.scale_a_mode == MI355_QP_PER_TENSOR)
            sa = p.scale_a[0];
        else if(p.scale_a_mode == MI355_QP_PER_ROW)
            sa = p.scale_a[m];
        int64_t zrow = 0;
        if constexpr(FMT == 0)
            zrow = p.zp_b != 0 ? (int64_t)p.zp_b * p.rowsum_a[m] - (int64_t)p.k * p.zp_a * p.zp_b : 0;
        float v[4];
#pragma unroll
        for(int e = 0; e < 4; e++)
        {
            const int c = col + e;
            float sb    = 1.f;
            if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                sb = p.scale_b[0];
            else if(p.scale_b_mode == MI355_QP_PER_COL)
                sb = p.scale_b[c];
            const float bias = p.bias != nullptr ? p.bias[c] : -0.0f;
            const float s    = sa * sb;
            if constexpr(FMT != 0)
                v[e] = add_bias((float)sum[e] * s, bias);
            else
            {
                const int32_t cs = p.zp_a != 0 ? p.colsum_b[c] : 0;
                const double d   = (double)sum[e] - (double)(int32_t)(zrow + (int64_t)p.zp_a * cs);
                v[e]             = add_bias((float)(d * (double)s), bias);
            }
        }
        if(!p.vec_store)
        {
#pragma unroll
            for(int e = 0; e < 4; e++)
                qdp_store1<OUT>(p.c, idx + e, v[e]);
        }
        else if constexpr(OUT == MI355_F32)
            *reinterpret_cast<v4f*>(static_cast<float*>(p.c) + idx) = v4f{v[0], v[1], v[2], v[3]};
        else if constexpr(OUT == MI355_F16)
        {
            uint2 o;
            o.x = convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16);
            o.y = convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16);
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = o;
        }
        else
        {
            uint2 o;
            o.x = convert_f32_to_bf16x2(v[0], v[1]);
            o.y = convert_f32_to_bf16x2(v[2], v[3]);
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = o;
        }
    }
}

// D: K steps whose loads are issued together
template <int FMT, bool DEQ, int OUT, int D>
__global__ __launch_bounds__(QDP_WAVES * 64) void qdp_kernel(qdp_params p)
{
    using acc_t    = typename qdp_acc<FMT>::type;
    __shared__ acc_t red[QDP_WAVES][64];

    const int lane  = threadIdx.x & 63;
    const int wave  = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int slot  = wave / p.wk;
    const int kpart = wave - slot * p.wk;
    const int tile  = (int)((int64_t)blockIdx.x * p.n_tiles / p.grid) + slot;
    const bool live = slot < p.tiles_per_wg && tile < (int)((int64_t)(blockIdx.x + 1) * p.n_tiles / p.grid);

    acc_t acc = {0, 0, 0, 0};
    if(live)
    {
        const int s0 = kpart * p.per;
        const int s1 = min(p.ksteps, s0 + p.per);
        const v4u* bp = reinterpret_cast<const v4u*>(p.b) + ((int64_t)tile * p.ksteps + s0) * 64 + lane;
        // rows past M read row M - 1 again: their results are columns of the instruction's
        // output that nobody stores
        const int row     = min(lane & 15, p.m - 1);
        const uint8_t* ap = p.a + (int64_t)row * p.lda + 16 * (lane >> 4) + (int64_t)64 * s0;
        int s = s0;
        for(; s + D <= s1; s += D)
        {
            v4u bv[D], av[D];
#pragma unroll
            for(int d = 0; d < D; d++)
                bv[d] = __builtin_nontemporal_load(bp + d * 64);
#pragma unroll
            for(int d = 0; d < D; d++)
                av[d] = *reinterpret_cast<const v4u*>(ap + d * 64);
#pragma unroll
            for(int d = 0; d < D; d++)
                acc = qdp_mma<FMT>(bv[d], av[d], acc);
            bp += D * 64;
            ap += D * 64;
        }
        for(; s < s1; s++)
        {
            const v4u bv = __builtin_nontemporal_load(bp);
            const v4u av = *reinterpret_cast<const v4u*>(ap);
            acc            = qdp_mma<FMT>(bv, av, acc);
            bp += 64;
            ap += 64;
        }
    }
    red[wave][lane] = acc;
    __syncthreads();
    if(!live || kpart != 0)
        return;
    // int8: integer sums, any order gives the same bits.  fp8: this fixed order, the same bits on
    // every call.
    acc_t sum = red[wave][lane];
    for(int j = 1; j < p.wk; j++)
        sum += red[wave + j][lane];

    qdp_finish<FMT, DEQ, OUT>(p, sum, tile, lane);
}

// The same product with the rows of A resident in the LDS and every B tile of the wave requested
// before anything else happens.  A workgroup covers all of K, so it needs all of A: M rows of
// K + 16 bytes (the 16 spare bytes spread the 16 rows of one fragment read over all banks),
// copied once by the whole workgroup, instead of one read from the caches per wave and step.
// STEPS = K steps per wave, exactly: the loads of a wave are STEPS instructions issued back to
// back (16 KiB in flight per wave at 16), consumed in order with a counted wait each.
constexpr int QDP_RED_BYTES = QDP_WAVES * 1024;
constexpr int QDP_LDS_LIMIT = 160 * 1024;

template <int FMT, bool DEQ, int OUT, int STEPS>
__global__ __launch_bounds__(QDP_WAVES * 64) void qdp_lds_kernel(qdp_params p)
{
    using acc_t = typename qdp_acc<FMT>::type;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    acc_t* red     = reinterpret_cast<acc_t*>(lds); // [wave][lane]
    uint8_t* arows = lds + QDP_RED_BYTES;

    const int tid      = threadIdx.x;
    const int nthreads = blockDim.x;
    const int lane     = tid & 63;
    const int wave     = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int slot     = wave / p.wk;
    const int kpart    = wave - slot * p.wk;
    const int tile     = (int)((int64_t)blockIdx.x * p.n_tiles / p.grid) + slot;
    const bool live    = tile < (int)((int64_t)(blockIdx.x + 1) * p.n_tiles / p.grid);

    // A: 16-byte pieces, piece i = row i / (K / 16), bytes 16 * (i % (K / 16)) ..
    const int k16    = p.k >> 4;
    const int pieces = p.m * k16;
    const int pitch  = p.k + 16;
    constexpr int CH = 8;
    v4u t[CH];
#pragma unroll
    for(int j = 0; j < CH; j++)
    {
        t[j] = v4u{0, 0, 0, 0};
        if(j * nthreads < pieces) // the same for the whole workgroup
        {
            // a thread past the end reads what it read one round earlier: some valid address that
            // is not the same one for every such thread of every workgroup
            int i = tid + j * nthreads;
            i     = i < pieces ? i : (j > 0 ? i - nthreads : i % pieces);
            const int r = (int)__umulhi((uint32_t)i, p.k16_magic);
            t[j]        = *reinterpret_cast<const v4u*>(p.a + (int64_t)r * p.lda + 16 * (i - r * k16));
        }
    }
    // B: all of the wave's tiles (a wave past the last tile column reads the last one again, so
    // that every wave has the same number of loads in flight at every point of the program)
    const int s0  = kpart * STEPS;
    const v4u* bp = reinterpret_cast<const v4u*>(p.b) + ((int64_t)min(tile, p.n_tiles - 1) * p.ksteps + s0) * 64 + lane;
    v4u bv[STEPS];
#pragma unroll
    for(int d = 0; d < STEPS; d++)
        bv[d] = __builtin_nontemporal_load(bp + d * 64);
#pragma unroll
    for(int j = 0; j < CH; j++)
    {
        const int i = tid + j * nthreads;
        const int r = (int)__umulhi((uint32_t)i, p.k16_magic);
        if(i < pieces)
            *reinterpret_cast<v4u*>(arows + r * pitch + 16 * (i - r * k16)) = t[j];
    }
    for(int i = tid + CH * nthreads; i < pieces; i += nthreads)
    {
        const int r = (int)__umulhi((uint32_t)i, p.k16_magic);
        *reinterpret_cast<v4u*>(arows + r * pitch + 16 * (i - r * k16)) =
            *reinterpret_cast<const v4u*>(p.a + (int64_t)r * p.lda + 16 * (i - r * k16));
    }
    __syncthreads();

    // rows past M read row M - 1 again: columns of the instruction's output that nobody stores
    const uint8_t* ap = arows + min(lane & 15, p.m - 1) * pitch + 16 * (lane >> 4) + 64 * s0;
    acc_t acc         = {0, 0, 0, 0};
#pragma unroll
    for(int d = 0; d < STEPS; d++)
        acc = qdp_mma<FMT>(bv[d], *reinterpret_cast<const v4u*>(ap + 64 * d), acc);
    red[wave * 64 + lane] = acc;
    __syncthreads();
    if(!live || kpart != 0)
        return;
    acc_t sum = red[wave * 64 + lane];
    for(int j = 1; j < p.wk; j++)
        sum += red[(wave + j) * 64 + lane];
    qdp_finish<FMT, DEQ, OUT>(p, sum, tile, lane);
}

template <int FMT, bool DEQ, int OUT, int STEPS>
int qdp_launch_lds(const qdp_params& p, int grid, int waves, size_t lds_bytes, hipStream_t s)
{
    auto kern = qdp_lds_kernel<FMT, DEQ, OUT, STEPS>;
    // above the 64 KiB default: opt in once per kernel instantiation
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, QDP_LDS_LIMIT);
    if(attr != hipSuccess)
        return MI355_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(waves * 64), lds_bytes, s, p);
    return mi355_launch_status();
}

// Workgroups for tile columns handed out at most `per_wg` each: the fewest that cover them, raised
// to the next multiple of the 256 compute units where there are enough columns, so that the
// columns spread evenly (3 and 4 per workgroup rather than 4 for most and none for the rest).
int qdp_grid(int n_tiles, int per_wg)
{
    const int least = (n_tiles + per_wg - 1) / per_wg;
    const int even  = (least + 255) / 256 * 256;
    return even <= n_tiles ? even : least;
}

// steps per wave of the LDS form for this shape (0: the shape takes the other kernel): every wave
// gets exactly that many, at most 16 waves share a tile column, A and the partial sums fit the LDS.
// The largest count that still gives every SIMD two waves; failing that, the most waves.
int qdp_lds_steps(const qdp_params& p)
{
    if((int64_t)p.m * (p.k + 16) + QDP_RED_BYTES > QDP_LDS_LIMIT)
        return 0;
    // One workgroup per compute unit at a time.  Fewest rounds of 256 workgroups first, then the
    // most waves at work per workgroup, then the longer run per wave (measured on 4096^2,
    // 8192^2 and 14336 x 4096: 5.9 / 8.0 / 12.8, - / 16.1 / 14.3 and 18.2 / 15.0 / 13.4 us for
    // 4 / 8 / 16 steps).
    int best = 0, best_rounds = 0;
    double best_live = 0.0;
    for(int steps : {16, 8, 4})
    {
        if(p.ksteps % steps != 0 || p.ksteps / steps > QDP_WAVES)
            continue;
        const int wk      = p.ksteps / steps;
        const int g       = qdp_grid(p.n_tiles, QDP_WAVES / wk);
        const int rounds  = (g + 255) / 256;
        const double live = (double)p.n_tiles / g * wk;
        if(best == 0 || rounds < best_rounds || (rounds == best_rounds && live > best_live + 1e-9))
        {
            best        = steps;
            best_rounds = rounds;
            best_live   = live;
        }
    }
    return best;
}

template <int FMT, bool DEQ, int OUT>
int qdp_launch_d(qdp_params p, int grid, hipStream_t s)
{
    if(const int steps = qdp_lds_steps(p))
    {
        p.wk               = p.ksteps / steps;
        p.per              = steps;
        p.tiles_per_wg     = QDP_WAVES / p.wk;
        const int waves    = p.wk * p.tiles_per_wg;
        const int g        = qdp_grid(p.n_tiles, p.tiles_per_wg);
        p.grid             = g;
        const size_t bytes = (size_t)QDP_RED_BYTES + (size_t)p.m * (p.k + 16);
        switch(steps)
        {
        case 16: return qdp_launch_lds<FMT, DEQ, OUT, 16>(p, g, waves, bytes, s);
        case 8: return qdp_launch_lds<FMT, DEQ, OUT, 8>(p, g, waves, bytes, s);
        default: return qdp_launch_lds<FMT, DEQ, OUT, 4>(p, g, waves, bytes, s);
        }
    }
    if(p.per >= 8)
        hipLaunchKernelGGL((qdp_kernel<FMT, DEQ, OUT, 8>), dim3(grid), dim3(QDP_WAVES * 64), 0, s, p);
    else
        hipLaunchKernelGGL((qdp_kernel<FMT, DEQ, OUT, 4>), dim3(grid), dim3(QDP_WAVES * 64), 0, s, p);
    return mi355_launch_status();
}

template <int FMT>
int qdp_launch(const qdp_params& p, int grid, bool deq, int out, hipStream_t s)
{
    if(!deq)
        return qdp_launch_d<FMT, false, MI355_F32>(p, grid, s);
    switch(out)
    {
    case MI355_F32: return qdp_launch_d<FMT, true, MI355_F32>(p, grid, s);
    case MI355_F16: return qdp_launch_d<FMT, true, MI355_F16>(p, grid, s);
    case MI355_BF16: return qdp_launch_d<FMT, true, MI355_BF16>(p, grid, s);
    default: return MI355_ERR_UNSUPPORTED;
    }
}

bool qdp_shape_ok(int32_t in_type, int64_t n, int64_t k)
{
    if(in_type != MI355_I8 && in_type != MI355_FP8 && in_type != MI355_BF8)
        return false;
    return n > 0 && k > 0 && n % 16 == 0 && k % 64 == 0 && n <= (1 << 30) && k <= (1 << 30);
}

} // namespace

extern "C" size_t mi355_quant_dot_prepacked_size(int32_t in_type, int64_t n, int64_t k)
{
    return qdp_shape_ok(in_type, n, k) ? (size_t)n * (size_t)k : 0;
}

extern "C" int mi355_quant_dot_prepack(const void* b,
                                       int32_t in_type,
                                       int64_t n,
                                       int64_t k,
                                       int64_t stride_k,
                                       int64_t stride_n,
                                       void* prepacked,
                                       void* stream)
{
    if(b == nullptr || prepacked == nullptr)
        return MI355_ERR_BAD_ARG;
    if(!qdp_shape_ok(in_type, n, k))
        return MI355_ERR_UNSUPPORTED;
    if(reinterpret_cast<uintptr_t>(prepacked) % 16 != 0)
        return MI355_ERR_BAD_ARG;
    const int n_tiles = (int)(n / 16), ksteps = (int)(k / 64);
    const int64_t pieces = (int64_t)n_tiles * ksteps * 64;
    hipLaunchKernelGGL(qdp_prepack_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(b), stride_k, stride_n,
                       static_cast<uint4*>(prepacked), n_tiles, ksteps);
    return mi355_launch_status();
}

extern "C" int mi355_quant_dot_prepacked(const mi355_quant_dot_desc* d,
                                         const void* a,
                                         const void* b_prepacked,
                                         void* c,
                                         const float* scale_a,
                                         const float* scale_b,
                                         const int32_t* colsum_b,
                                         const int32_t* rowsum_a,
                                         const float* bias,
                                         void* stream)
{
    if(d == nullptr || a == nullptr || b_prepacked == nullptr || c == nullptr)
        return MI355_ERR_BAD_ARG;
    if(d->m <= 0 || d->n <= 0 || d->k <= 0)
        return MI355_ERR_BAD_ARG;
    if(!qdp_shape_ok(d->in_type, d->n, d->k) || d->m > 16 || d->batch != 1 || d->trans_a)
        return MI355_ERR_UNSUPPORTED;
    const bool fp8 = d->in_type != MI355_I8;
    if(bias != nullptr && !d->dequant)
        return MI355_ERR_BAD_ARG;
    if(d->dequant)
    {
        if(d->out_type != MI355_F32 && d->out_type != MI355_F16 && d->out_type != MI355_BF16)
            return MI355_ERR_BAD_ARG;
        if(d->scale_a_mode != MI355_QP_NONE && d->scale_a_mode != MI355_QP_PER_TENSOR &&
           d->scale_a_mode != MI355_QP_PER_ROW)
            return MI355_ERR_BAD_ARG;
        if(d->scale_b_mode != MI355_QP_NONE && d->scale_b_mode != MI355_QP_PER_TENSOR &&
           d->scale_b_mode != MI355_QP_PER_COL)
            return MI355_ERR_BAD_ARG;
        if((d->scale_a_mode != MI355_QP_NONE && scale_a == nullptr) ||
           (d->scale_b_mode != MI355_QP_NONE && scale_b == nullptr))
            return MI355_ERR_BAD_ARG;
        if(fp8 && (d->zp_a != 0 || d->zp_b != 0))
            return MI355_ERR_UNSUPPORTED;
        if((d->zp_a != 0 && colsum_b == nullptr) || (d->zp_b != 0 && rowsum_a == nullptr))
            return MI355_ERR_BAD_ARG;
        if(d->zp_a < -128 || d->zp_a > 127 || d->zp_b < -128 || d->zp_b > 127)
            return MI355_ERR_BAD_ARG;
    }
    else if(d->out_type != (fp8 ? MI355_F32 : MI355_I32))
        return MI355_ERR_BAD_ARG;
    if(d->ldc < d->n || d->lda < d->k)
        return MI355_ERR_BAD_ARG;
    // 16-byte loads of A and of the reordered B
    if(d->lda % 16 != 0 || reinterpret_cast<uintptr_t>(a) % 16 != 0 ||
       reinterpret_cast<uintptr_t>(b_prepacked) % 16 != 0)
        return MI355_ERR_UNSUPPORTED;

    qdp_params p;
    p.a            = static_cast<const uint8_t*>(a);
    p.b            = static_cast<const uint8_t*>(b_prepacked);
    p.c            = c;
    p.m            = (int)d->m;
    p.n            = (int)d->n;
    p.k            = (int)d->k;
    p.lda          = d->lda;
    p.ldc          = d->ldc;
    p.scale_a      = scale_a;
    p.scale_b      = scale_b;
    p.colsum_b     = colsum_b;
    p.rowsum_a     = rowsum_a;
    p.bias         = bias;
    p.scale_a_mode = d->scale_a_mode;
    p.scale_b_mode = d->scale_b_mode;
    p.zp_a         = d->zp_a;
    p.zp_b         = d->zp_b;
    p.n_tiles      = (int)(d->n / 16);
    p.k16_magic    = (uint32_t)((((uint64_t)1 << 32) / (uint64_t)(d->k / 16)) + 1);
    p.ksteps       = (int)(d->k / 64);
    // enough waves for every SIMD of the chip to hold four, each with at least two K steps
    int wk = 1;
    while(wk < QDP_WAVES && (int64_t)p.n_tiles * wk * 2 <= 256 * QDP_WAVES && p.ksteps >= wk * 4)
        wk *= 2;
    p.wk           = wk;
    p.per          = (p.ksteps + wk - 1) / wk;
    p.tiles_per_wg = QDP_WAVES / wk;
    const size_t esz = d->dequant ? mi355_dtype_size(d->out_type) : 4;
    p.vec_store      = d->ldc % 4 == 0 && reinterpret_cast<uintptr_t>(c) % (4 * esz) == 0;
    const int grid   = qdp_grid(p.n_tiles, p.tiles_per_wg);
    p.grid           = grid;
    hipStream_t s    = static_cast<hipStream_t>(stream);
    const bool deq   = d->dequant != 0;
    switch(d->in_type)
    {
    case MI355_I8:
        return qdp_launch<0>(p, grid, deq, d->out_type, s);
    case MI355_FP8: return qdp_launch<1>(p, grid, deq, d->out_type, s);
    default: return qdp_launch<2>(p, grid, deq, d->out_type, s);
    }
}
