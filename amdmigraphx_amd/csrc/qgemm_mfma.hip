// quant_dot on the gfx950 matrix cores: int8 x int8 -> int32 with
// v_mfma_i32_16x16x64_i8 and e4m3fn x e4m3fn -> fp32 with
// v_mfma_f32_16x16x128_f8f6f4, with the dequantizelinear / convert epilogue
// applied to the accumulators in registers.
//
// Tiling: one workgroup of 8 waves computes a 256 x 256 tile of C, stepping
// through K in slabs of 128 bytes.  Waves are arranged 2 (M) x 4 (N); each owns
// 128 x 64 of the tile as 8 x 4 MFMA tiles of 16 x 16 (128 accumulator
// registers).  A and B slabs are staged in LDS, K-contiguous, with rows padded
// from 128 to 144 bytes so that the 16 lanes of an MFMA operand read hit 64
// distinct banks.  Two LDS stages: the next slab is fetched from global memory
// into registers while the current one feeds the MFMAs, then written to the
// other stage; one barrier per slab.
//
// B arrives either K-contiguous ([N, K] storage, the transpose view) or row
// major [K, N].  The row-major form is transposed on its way to LDS: each lane
// reads one dword (4 consecutive n) from 16 consecutive k rows, transposes the
// 16 x 4 bytes with v_perm_b32 and writes four 16-byte K-runs.
//
// Column assignment: the column of C that MFMA tile j, lane column i computes is
// n = 4*i + j (not 16*j + i).  A lane then holds 4 consecutive n of one row
// across its 4 N-tiles and stores them with one 16-byte write; 16 lanes cover
// 256 contiguous bytes of a C row.  In LDS the B rows are permuted to match
// (row j*64 + q holds column 4*q + j), which also makes the transposed
// row-major store conflict free.
#include "common.h"

namespace {

constexpr int BM       = 256;
constexpr int BN       = 256;
constexpr int BK       = 128; // bytes of K per slab
constexpr int LDS_ROW  = BK + 16;
constexpr int NTHREADS = 512;
constexpr int STAGE_BYTES = (BM + BN) * LDS_ROW;
constexpr int LDS_BYTES   = 2 * STAGE_BYTES;

struct gemm_params
{
    const uint8_t* a;
    const uint8_t* b;
    void* c;
    int m, n, k;
    int64_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;
    int tiles_m, tiles_n;
    const float* scale_a;
    const float* scale_b;
    const float* bias; // [N], added after the dequantization; null = none
    const int32_t* colsum_b;
    const int32_t* rowsum_a;
    int scale_a_mode, scale_b_mode;
    int zp_a, zp_b;
};

MI355_DEVINL uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel)
{
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// rows r0..r3 hold bytes [n0 n1 n2 n3] of four consecutive k; returns in c[j]
// the four k bytes of column j (k ascending from byte 0).
MI355_DEVINL void transpose4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t c[4])
{
    uint32_t t01l = perm(r1, r0, 0x05010400u); // r0[0] r1[0] r0[1] r1[1]
    uint32_t t01h = perm(r1, r0, 0x07030602u); // r0[2] r1[2] r0[3] r1[3]
    uint32_t t23l = perm(r3, r2, 0x05010400u);
    uint32_t t23h = perm(r3, r2, 0x07030602u);
    c[0]          = perm(t23l, t01l, 0x05040100u);
    c[1]          = perm(t23l, t01l, 0x07060302u);
    c[2]          = perm(t23h, t01h, 0x05040100u);
    c[3]          = perm(t23h, t01h, 0x07060302u);
}

// XCD-aware tile order.  Workgroup ids are dealt round-robin to the 8 XCDs,
// each with its own L2.  Give every XCD a contiguous run of the tile order, and
// walk that order in column-major bands of 8 tile rows, so the ~32 tiles an
// XCD works on at one time share A row panels and B column panels in its L2.
MI355_DEVINL void tile_coords(int wg, int tiles_m, int tiles_n, int& tm, int& tn)
{
    const int total = tiles_m * tiles_n;
    int v           = wg;
    if(total % 8 == 0)
        v = (wg % 8) * (total / 8) + wg / 8;
    constexpr int band = 8;
    int per_band       = band * tiles_n;
    int b              = v / per_band;
    int first_m        = b * band;
    int rows           = min(band, tiles_m - first_m);
    int r              = v - b * per_band;
    tm                 = first_m + r % rows;
    tn                 = r / rows;
}

template <bool FP8>
struct acc_traits
{
    using type = v4i;
};
template <>
struct acc_traits<true>
{
    using type = v4f;
};

template <bool FP8>
struct frag_traits
{
    using type = v4i;
};
template <>
struct frag_traits<true>
{
    using type = v8i;
};

template <int OUT>
MI355_DEVINL void store4(void* c, int64_t idx, const float v[4])
{
    if constexpr(OUT == MI355_F32)
    {
        *reinterpret_cast<float4*>(static_cast<float*>(c) + idx) =
            make_float4(v[0], v[1], v[2], v[3]);
    }
    else if constexpr(OUT == MI355_F16)
    {
        uint2 o;
        o.x = convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16);
        o.y = convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16);
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(c) + idx) = o;
    }
    else
    {
        uint2 o;
        o.x = convert_f32_to_bf16(v[0]) | ((uint32_t)convert_f32_to_bf16(v[1]) << 16);
        o.y = convert_f32_to_bf16(v[2]) | ((uint32_t)convert_f32_to_bf16(v[3]) << 16);
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(c) + idx) = o;
    }
}

// FMT: element type (0 int8, 1 fp8 e4m3fn, 2 fp8 e5m2); TRANS_B: B stored [N, K]; DEQ: apply the
// epilogue; OUT: output element type; KFULL: K is a multiple of the 128-byte slab, so no
// load needs a bounds predicate (a predicate per load costs a branch each).
template <int FMT, bool TRANS_B, bool DEQ, int OUT, bool KFULL>
__global__ __launch_bounds__(NTHREADS) void qgemm_mfma_kernel(gemm_params p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr bool FP8 = FMT != 0;
    using acc_t  = typename acc_traits<FP8>::type;
    using frag_t = typename frag_traits<FP8>::type;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    // wave-uniform values live in scalar registers: addresses built from them
    // use the scalar-base form of the global loads
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 2; // 0..1
    const int wave_n = wave & 3;  // 0..3

    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const uint8_t* __restrict__ ga = p.a + (int64_t)blockIdx.y * p.stride_a;
    const uint8_t* __restrict__ gb = p.b + (int64_t)blockIdx.y * p.stride_b;

    // ---- global -> register staging -------------------------------------
    // A (and K-contiguous B): 4 passes of 64 rows, 8 lanes x 16 bytes per row.
    // Per-lane byte offsets are 32-bit (the launcher checks the extents);
    // the slab offset k0 goes into the uniform base.
    const int ld_row = tid >> 3;
    const int ld_kc  = (tid & 7) * 16;
    uint32_t a_off[4];
#pragma unroll
    for(int s = 0; s < 4; s++)
    {
        int row  = min(m0 + ld_row + 64 * s, p.m - 1);
        a_off[s] = (uint32_t)row * (uint32_t)p.lda + ld_kc;
    }
    uint32_t bt_off[4]; // K-contiguous B: same pattern over n
    uint32_t b_off = 0; // row-major B: lane l reads the dword at column 4l
    if constexpr(TRANS_B)
    {
#pragma unroll
        for(int s = 0; s < 4; s++)
        {
            int col   = min(n0 + ld_row + 64 * s, p.n - 1);
            bt_off[s] = (uint32_t)col * (uint32_t)p.ldb + ld_kc;
        }
    }
    else
    {
        b_off = (uint32_t)min(n0 + 4 * lane, p.n - 4);
    }

    uint4 ra[4];
    uint4 rbt[4];
    uint32_t rb[16];

    auto load_slab = [&](int k0) {
        const bool kin        = KFULL || (k0 + ld_kc) < p.k;
        const uint8_t* a_base = ga + k0;
#pragma unroll
        for(int s = 0; s < 4; s++)
            ra[s] = kin ? *reinterpret_cast<const uint4*>(a_base + a_off[s])
                        : make_uint4(0, 0, 0, 0);
        if constexpr(TRANS_B)
        {
            const uint8_t* b_base = gb + k0;
#pragma unroll
            for(int s = 0; s < 4; s++)
                rbt[s] = kin ? *reinterpret_cast<const uint4*>(b_base + bt_off[s])
                             : make_uint4(0, 0, 0, 0);
        }
        else
        {
            // wave w reads k rows 16w..16w+15 of the slab
            const uint8_t* b_base = gb + (int64_t)(k0 + 16 * wave) * p.ldb;
#pragma unroll
            for(int i = 0; i < 16; i++)
            {
                const int kk = k0 + 16 * wave + i;
                rb[i]        = (KFULL || kk < p.k)
                                   ? *reinterpret_cast<const uint32_t*>(b_base + (int64_t)i * p.ldb + b_off)
                                   : 0u;
            }
        }
    };

    auto store_slab = [&](int stage) {
        uint8_t* as = lds + stage * STAGE_BYTES;
        uint8_t* bs = as + BM * LDS_ROW;
#pragma unroll
        for(int s = 0; s < 4; s++)
            *reinterpret_cast<uint4*>(as + (ld_row + 64 * s) * LDS_ROW + ld_kc) = ra[s];
        if constexpr(TRANS_B)
        {
#pragma unroll
            for(int s = 0; s < 4; s++)
            {
                int nl  = ld_row + 64 * s;           // column within the tile
                int row = (nl & 3) * 64 + (nl >> 2); // permuted LDS row
                *reinterpret_cast<uint4*>(bs + row * LDS_ROW + ld_kc) = rbt[s];
            }
        }
        else
        {
            uint32_t c0[4], c1[4], c2[4], c3[4];
            transpose4x4(rb[0], rb[1], rb[2], rb[3], c0);
            transpose4x4(rb[4], rb[5], rb[6], rb[7], c1);
            transpose4x4(rb[8], rb[9], rb[10], rb[11], c2);
            transpose4x4(rb[12], rb[13], rb[14], rb[15], c3);
#pragma unroll
            for(int j = 0; j < 4; j++)
            {
                // column 4*lane + j -> LDS row j*64 + lane, k bytes 16*wave..+15
                *reinterpret_cast<uint4*>(bs + (j * 64 + lane) * LDS_ROW + 16 * wave) =
                    make_uint4(c0[j], c1[j], c2[j], c3[j]);
            }
        }
    };

    acc_t acc[8][4];
#pragma unroll
    for(int i = 0; i < 8; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
            acc[i][j] = acc_t{0, 0, 0, 0};

    // ---- LDS -> MFMA operand fragments ------------------------------------
    // Lane l supplies row (l % 16) of a 16-row operand tile and the K bytes of
    // lane group l / 16: 16 bytes per group for the K = 64 int8 instruction,
    // 32 for the K = 128 fp8 one.  A and B use the same K assignment, which is
    // all the dot product needs.
    constexpr int FRAG_BYTES = FP8 ? 32 : 16;
    const int frag_off = (lane & 15) * LDS_ROW + (lane >> 4) * FRAG_BYTES;
    auto read_frag = [&](const uint8_t* q) -> frag_t {
        if constexpr(FP8)
        {
            v4i lo = *reinterpret_cast<const v4i*>(q);
            v4i hi = *reinterpret_cast<const v4i*>(q + 16);
            return v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
        else
        {
            return *reinterpret_cast<const v4i*>(q);
        }
    };
    // half h of a slab: int8 -> K bytes 64h..64h+63 with all 8 A tiles;
    //                   fp8  -> all 128 K bytes with A tiles 4h..4h+3.
    auto a_frag = [&](int stage, int h, int i) -> frag_t {
        const uint8_t* q = lds + stage * STAGE_BYTES + frag_off;
        if constexpr(FP8)
            return read_frag(q + (wave_m * 128 + (4 * h + i) * 16) * LDS_ROW);
        else
            return read_frag(q + (wave_m * 128 + i * 16) * LDS_ROW + h * 64);
    };
    auto b_frag = [&](int stage, int h, int j) -> frag_t {
        const uint8_t* q =
            lds + stage * STAGE_BYTES + BM * LDS_ROW + frag_off + (j * 64 + wave_n * 16) * LDS_ROW;
        if constexpr(FP8)
            return read_frag(q);
        else
            return read_frag(q + h * 64);
    };
    auto mfma = [&](const frag_t& a, const frag_t& b, acc_t c) -> acc_t {
        if constexpr(FMT == 2)
            // cbsz = blgp = 1: e5m2 for both operands
            return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 1, 1, 0, 0, 0, 0);
        else if constexpr(FP8)
            // zero scale operands select the unscaled v_mfma_f32_16x16x128_f8f6f4;
            // cbsz = blgp = 0 means e4m3 for both operands
            return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
    };

    constexpr int A_STEPS = FP8 ? 4 : 8; // A tiles per half slab
    frag_t af[2];                        // A fragments, double buffered
    frag_t bf[FP8 ? 1 : 2][4];           // B fragments (int8: one set per half)

    // The fragments a half starts with are read ahead of it; inside a half the
    // next A fragment is requested before the four MFMAs of the current one
    // issue, so the matrix pipe does not wait on LDS latency.
    auto first_frags = [&](int stage) {
#pragma unroll
        for(int j = 0; j < 4; j++)
            bf[0][j] = b_frag(stage, 0, j);
        af[0] = a_frag(stage, 0, 0);
    };
    auto compute_half = [&](int stage, int h) {
#pragma unroll
        for(int i = 0; i < A_STEPS; i++)
        {
            const int cur = i & 1;
            if(i + 1 < A_STEPS)
                af[cur ^ 1] = a_frag(stage, h, i + 1);
            else if(h == 0)
                af[cur ^ 1] = a_frag(stage, 1, 0);
            if constexpr(!FP8)
            {
                if(h == 0 && i >= A_STEPS - 4)
                    bf[1][i - (A_STEPS - 4)] = b_frag(stage, 1, i - (A_STEPS - 4));
            }
            const int row = FP8 ? 4 * h + i : i;
            const int bh  = FP8 ? 0 : h;
#pragma unroll
            for(int j = 0; j < 4; j++)
                acc[row][j] = mfma(af[cur], bf[bh][j], acc[row][j]);
            // keep "LDS reads of the next step, then this step's MFMAs" as the
            // issue order instead of letting the reads sink to their first use
            __builtin_amdgcn_sched_group_barrier(0x100, FP8 ? 2 : 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        }
    };

    // ---- main loop ------------------------------------------------------------
    // Slab kt+1 is fetched into registers at the top of iteration kt, written to
    // the other LDS stage between the two halves of slab kt (that stage was last
    // read before the previous barrier), and is visible after the barrier that
    // ends the iteration.
    const int nk = (p.k + BK - 1) / BK;
    load_slab(0);
    store_slab(0);
    __syncthreads();
    first_frags(0);
    for(int kt = 0; kt < nk; kt++)
    {
        const bool more = kt + 1 < nk;
        const int stage = kt & 1;
        if(more)
            load_slab((kt + 1) * BK);
        compute_half(stage, 0);
        if(more)
            store_slab(stage ^ 1);
        compute_half(stage, 1);
        __syncthreads();
        if(more)
            first_frags(stage ^ 1);
    }

    // ---- epilogue -------------------------------------------------------------
    // acc[i][j][r]: row 16*i + 4*(lane/16) + r, column 4*(lane%16) + j of the
    // wave's 128 x 64 block.
    const int col = n0 + wave_n * 64 + 4 * (lane & 15);
    if(col >= p.n)
        return;
    float sb[4]  = {1.f, 1.f, 1.f, 1.f};
    int32_t cs[4] = {0, 0, 0, 0};
    float bias[4] = {-0.0f, -0.0f, -0.0f, -0.0f};
    if constexpr(DEQ)
    {
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                sb[j] = p.scale_b[0];
            else if(p.scale_b_mode == MI355_QP_PER_COL)
                sb[j] = p.scale_b[col + j];
            if(p.zp_a != 0)
                cs[j] = p.colsum_b[col + j];
            if(p.bias != nullptr)
                bias[j] = p.bias[col + j];
        }
    }
    uint8_t* cbase = static_cast<uint8_t*>(p.c);
#pragma unroll
    for(int i = 0; i < 8; i++)
    {
#pragma unroll
        for(int r = 0; r < 4; r++)
        {
            int row = m0 + wave_m * 128 + 16 * i + 4 * (lane >> 4) + r;
            if(row >= p.m)
                continue;
            int64_t idx = (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
            if constexpr(!DEQ)
            {
                if constexpr(FP8)
                {
                    *reinterpret_cast<float4*>(reinterpret_cast<float*>(cbase) + idx) =
                        make_float4(acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]);
                }
                else
                {
                    *reinterpret_cast<int4*>(reinterpret_cast<int32_t*>(cbase) + idx) =
                        make_int4(acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]);
                }
            }
            else
            {
                float sa = 1.f;
                if(p.scale_a_mode == MI355_QP_PER_TENSOR)
                    sa = p.scale_a[0];
                else if(p.scale_a_mode == MI355_QP_PER_ROW)
                    sa = p.scale_a[row];
                int64_t zrow = 0;
                if constexpr(!FP8)
                {
                    if(p.zp_b != 0)
                        zrow = (int64_t)p.zp_b * p.rowsum_a[row] -
                               (int64_t)p.k * p.zp_a * p.zp_b;
                }
                float v[4];
#pragma unroll
                for(int j = 0; j < 4; j++)
                {
                    // scale = fp32 product of the two scales (the graph's `mul`),
                    // then (double(acc) - double(zp)) * scale in double, one
                    // rounding to float (dequantizelinear).
                    float s = sa * sb[j];
                    double d;
                    if constexpr(FP8)
                        d = (double)acc[i][j][r];
                    else
                        d = (double)acc[i][j][r] -
                            (double)(int32_t)(zrow + (int64_t)p.zp_a * cs[j]);
                    v[j] = add_bias((float)(d * (double)s), bias[j]);
                }
                store4<OUT>(p.c, idx, v);
            }
        }
    }
}

template <int FMT, bool TRANS_B, bool DEQ, int OUT, bool KFULL>
int launch_k(const gemm_params& p, int batch, hipStream_t stream)
{
    auto kern = qgemm_mfma_kernel<FMT, TRANS_B, DEQ, OUT, KFULL>;
    // above the 64 KiB default: opt in once per kernel instantiation
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if(attr != hipSuccess)
        return MI355_ERR_LAUNCH;
    dim3 grid(p.tiles_m * p.tiles_n, batch);
    hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), LDS_BYTES, stream, p);
    return mi355_launch_status();
}

template <int FMT, bool TRANS_B, bool DEQ, int OUT>
int launch_one(const gemm_params& p, int batch, hipStream_t stream)
{
    return p.k % BK == 0 ? launch_k<FMT, TRANS_B, DEQ, OUT, true>(p, batch, stream)
                         : launch_k<FMT, TRANS_B, DEQ, OUT, false>(p, batch, stream);
}

template <int FMT, bool TRANS_B>
int launch_out(const gemm_params& p, int batch, bool deq, int out, hipStream_t s)
{
    if(!deq)
        return launch_one<FMT, TRANS_B, false, MI355_F32>(p, batch, s);
    switch(out)
    {
    case MI355_F32: return launch_one<FMT, TRANS_B, true, MI355_F32>(p, batch, s);
    case MI355_F16: return launch_one<FMT, TRANS_B, true, MI355_F16>(p, batch, s);
    case MI355_BF16: return launch_one<FMT, TRANS_B, true, MI355_BF16>(p, batch, s);
    default: return MI355_ERR_UNSUPPORTED;
    }
}

} // namespace

// Whether the MFMA kernel's load pattern fits this problem: 16-byte K runs for
// A (and K-contiguous B), dword n runs for row-major B, 16-byte stores of C.
bool mi355_mfma_gemm_supported(const mi355_quant_dot_desc* d,
                               const void* a,
                               const void* b,
                               const void* c)
{
    if(d->trans_a)
        return false;
    if(d->k % 16 != 0 || d->lda % 16 != 0 || d->stride_a % 16 != 0)
        return false;
    if(reinterpret_cast<uintptr_t>(a) % 16 != 0)
        return false;
    if(d->n % 4 != 0 || d->n < 4)
        return false;
    if(d->trans_b)
    {
        if(d->ldb % 16 != 0 || d->stride_b % 16 != 0 || reinterpret_cast<uintptr_t>(b) % 16 != 0)
            return false;
    }
    else
    {
        if(d->ldb % 4 != 0 || d->stride_b % 4 != 0 || reinterpret_cast<uintptr_t>(b) % 4 != 0)
            return false;
    }
    size_t osz = 4;
    if(d->dequant)
        osz = mi355_dtype_size(d->out_type);
    // 4 consecutive outputs are written with one store
    if((d->ldc * osz) % (4 * osz) != 0 || (d->stride_c * osz) % (4 * osz) != 0 ||
       reinterpret_cast<uintptr_t>(c) % (4 * osz) != 0)
        return false;
    if(d->m > (1 << 30) || d->n > (1 << 30) || d->k > (1 << 30))
        return false;
    // per-lane byte offsets inside one matrix are kept in 32 bits
    const int64_t lim = (int64_t)1 << 31;
    if(d->m * d->lda >= lim || (d->trans_b ? d->n * d->ldb : d->k * d->ldb) >= lim)
        return false;
    return true;
}

int mi355_mfma_gemm_launch(const mi355_quant_dot_desc* d,
                           const void* a,
                           const void* b,
                           void* c,
                           const float* scale_a,
                           const float* scale_b,
                           const int32_t* colsum_b,
                           const int32_t* rowsum_a,
                           const float* bias,
                           hipStream_t stream)
{
    gemm_params p;
    p.bias         = bias;
    p.a            = static_cast<const uint8_t*>(a);
    p.b            = static_cast<const uint8_t*>(b);
    p.c            = c;
    p.m            = (int)d->m;
    p.n            = (int)d->n;
    p.k            = (int)d->k;
    p.lda          = d->lda;
    p.ldb          = d->ldb;
    p.ldc          = d->ldc;
    p.stride_a     = d->stride_a;
    p.stride_b     = d->stride_b;
    p.stride_c     = d->stride_c;
    p.tiles_m      = (p.m + BM - 1) / BM;
    p.tiles_n      = (p.n + BN - 1) / BN;
    p.scale_a      = scale_a;
    p.scale_b      = scale_b;
    p.colsum_b     = colsum_b;
    p.rowsum_a     = rowsum_a;
    p.scale_a_mode = d->scale_a_mode;
    p.scale_b_mode = d->scale_b_mode;
    p.zp_a         = d->zp_a;
    p.zp_b         = d->zp_b;
    const bool deq = d->dequant != 0;
    if(d->in_type == MI355_BF8)
        return d->trans_b ? launch_out<2, true>(p, (int)d->batch, deq, d->out_type, stream)
                          : launch_out<2, false>(p, (int)d->batch, deq, d->out_type, stream);
    if(d->in_type == MI355_FP8)
        return d->trans_b ? launch_out<1, true>(p, (int)d->batch, deq, d->out_type, stream)
                          : launch_out<1, false>(p, (int)d->batch, deq, d->out_type, stream);
    return d->trans_b ? launch_out<0, true>(p, (int)d->batch, deq, d->out_type, stream)
                      : launch_out<0, false>(p, (int)d->batch, deq, d->out_type, stream);
}
