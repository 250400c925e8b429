// int4 weight-only GEMV (one activation row) over weights reordered once, ahead of time.
//
// Weights of a weight-only layer are constants of the graph, so their layout in memory is free.
// The reordering puts everything one wave instruction needs side by side and spares the kernel
// all the per-weight bit shuffling that the operator's own layout ([N, K/2] rows, two nibbles per
// byte along K, scales in a second tensor) costs:
//
//   block (R, S) = weight rows 16R .. 16R+15 against k = 512S .. 512S+511:
//     128 bytes of scales:  lane l = 16*kg + nl reads scale[16R + nl, 4S + kg] (group size 128),
//     4 x 1 KiB of nibbles: piece i of lane l is the 32 weights
//                           W[16R + nl, 512S + 128kg + 32i .. +32), i.e. one 16-byte load.
//   Blocks lie in (R, S) order behind a 256-byte header.
//
// The product runs on the matrix cores: the 8 halves a lane feeds to one
// v_mfma_f32_16x16x32_f16 as the second operand are 8 dequantized weights of its row, the first
// operand is the matching 8 activations (a broadcast 16-byte LDS read per lane group), and row 0
// of the result is 16 outputs: the instruction adds over the lane groups, so there is no
// cross-lane reduction and no per-weight multiply on the vector ALU.
//
// Dequantization is one packed-half fused multiply-add per two weights, with nibbles used where
// they lie.  A nibble at bits 4..7 of a half reads as the subnormal q * 2^-20, one at bits 0..3
// as q * 2^-24.  With S = scale * 2^20, fma(q * 2^-20, S, -zp * scale) forms (q - zp) * scale
// exactly and rounds it once, toward zero (the wave's half rounding mode), which is the
// reference's half((q - zp) * scale) bit for bit; fma(q * 2^-24, S, -zp * scale / 16) gives the
// same weight divided by 16 (same significand, exponent lower by 4).  The weights of the odd
// nibble positions (bits 4..7, and 12..15 after one shift by 8) and those of the even positions
// therefore go to different matrix-core instructions and different accumulators, and the sum
// of the second kind is multiplied by 16 (exact) at the end.  The nibble order inside a 16-byte
// piece is chosen so that the packed results are the instruction operands as they stand.
// This needs every scale to be positive with exponent field 5..10 (2^-10 <= scale < 2^-4) and the
// zero point to be 0 or a power of two; the reordering kernel checks that and records it in the
// header, and the GEMV takes the general form (1024 + q in the mantissa, minus 1024 + zp, times
// scale: three instructions per pair) for the whole matrix otherwise.
#include "common.h"
#include <type_traits>

namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr uint32_t W4P_MAGIC  = 0x31503457u; // "W4P1"
constexpr int W4P_HEADER      = 256;
constexpr int W4P_BLOCK       = 128 + 4096;
constexpr int W4P_GROUP       = 128;
constexpr int W4P_SUPER_K     = 512; // k per block
constexpr int W4P_MAX_WAVES   = 16;
constexpr int W4P_A_SLOTS     = 4;   // 16-byte pieces of the activation row per thread, at most
constexpr uint32_t W4P_FLAG_GENERAL = 1u;

struct w4p_header
{
    uint32_t magic, n, k, group, zp, flags;
};

// nibble of weight k_local = 8j + e (j: instruction 0..3, e: element 0..7) inside a lane's
// 16-byte piece: dword d, half h, position p (bit 16h + 4p).  Instructions 0 and 1 take the odd
// positions (read as q * 2^-20), 2 and 3 the even ones (q * 2^-24).
__host__ __device__ inline void w4p_place(int k_local, int& d, int& h, int& p)
{
    const int j = k_local >> 3, e = k_local & 7;
    const int v = e >> 1;           // operand register 0..3
    h           = e & 1;
    d           = 2 * (j & 1) + (v >> 1);
    p           = 2 * (v & 1) + (j < 2 ? 1 : 0);
}

__global__ void w4p_header_kernel(uint8_t* out, uint32_t n, uint32_t k, uint32_t zp)
{
    if(threadIdx.x == 0 && blockIdx.x == 0)
    {
        auto* h  = reinterpret_cast<w4p_header*>(out);
        h->magic = W4P_MAGIC;
        h->n     = n;
        h->k     = k;
        h->group = W4P_GROUP;
        h->zp    = zp;
        // zero points other than 0 / powers of two have no exact -zp * scale
        h->flags = (zp & (zp - 1)) == 0 ? 0u : W4P_FLAG_GENERAL;
    }
}

// one thread per 16-byte piece (and, for i == 0, per scale)
__global__ __launch_bounds__(256) void w4p_prepack_kernel(const uint8_t* w, const uint16_t* scales, uint8_t* out,
                                                           int n, int k)
{
    const int nss        = k / W4P_SUPER_K;
    const int64_t pieces = (int64_t)(n / 16) * nss * 256;
    const int64_t t      = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(t >= pieces)
        return;
    const int l        = (int)(t & 63);
    const int i        = (int)((t >> 6) & 3);
    const int64_t blk  = t >> 8;
    const int s        = (int)(blk % nss);
    const int64_t r    = blk / nss;
    const int nl       = l & 15, kg = l >> 4;
    const int64_t row  = r * 16 + nl;
    const int k0       = s * W4P_SUPER_K + kg * 128 + i * 32;
    const uint8_t* src = w + row * (k / 2) + k0 / 2;
    uint32_t o[4]      = {0, 0, 0, 0};
    for(int kl = 0; kl < 32; kl++)
    {
        const uint32_t q = (src[kl >> 1] >> (4 * (kl & 1))) & 0xfu;
        int d, h, p;
        w4p_place(kl, d, h, p);
        o[d] |= q << (16 * h + 4 * p);
    }
    uint8_t* b = out + W4P_HEADER + blk * W4P_BLOCK;
    *reinterpret_cast<v4u*>(b + 128 + i * 1024 + l * 16) = v4u{o[0], o[1], o[2], o[3]};
    if(i == 0)
    {
        const uint16_t sb = scales[row * (k / W4P_GROUP) + s * 4 + kg];
        *reinterpret_cast<uint16_t*>(b + l * 2) = sb;
        const uint32_t e = (sb >> 10) & 0x1fu;
        if((sb & 0x8000u) != 0 || e < 5 || e > 10)
            atomicOr(&reinterpret_cast<w4p_header*>(out)->flags, W4P_FLAG_GENERAL);
    }
}

struct w4p_params
{
    const uint8_t* pk;   // reordered weights (header + blocks)
    const uint16_t* a;   // activation row, k halves
    uint16_t* out;       // n halves
    int n, k;
    int nss;             // blocks along K
    int nrg;             // groups of 16 weight rows
    int wk;              // waves that share a row group (they split its blocks)
    int teams;           // row groups a workgroup works on at a time
    int iters_s;         // blocks per wave and row group
    int iters_r;         // row groups per team
    int rg_stride;       // distance between a team's row groups
    int rg_base;         // first row group of this launch
    // several activation rows (the MR = 16 kernels)
    int m;               // activation rows, 1 .. 16
    int lda, ldc;        // halves between rows of a and of out
    int a_pitch;         // bytes between activation rows in the LDS: 2 k + 16
    uint32_t row_magic;  // i / (k / 8)        = umulhi(i, row_magic)   for the piece numbers staged
    uint32_t all_magic;  // i / (m * (k / 8))  = umulhi(i, all_magic)
};


struct w4p_item
{
    v4u w[4];
    uint32_t sb;
};

// Vector-memory loads of the GEMV kernel are assembly statements with explicit waits.  A wave's
// loads return in the order they were issued; the kernel keeps the activation row's loads, then
// two blocks of weights, in flight and waits for exactly the piece it is about to use.  Left to
// the compiler, the loads are reordered and every wait behind a branch becomes a wait for all of
// them.  The registers a load writes are operands of the wait statement in front of their first
// use, so nothing reads them earlier -- as long as the compiler has no reason to copy them on the
// way, which is why the kernel's blocks are written out in a straight line (their number is a
// template parameter): around a loop the copies of loop-carried registers land in front of the
// wait.
template <int OFF>
MI355_DEVINL void w4p_load16_nt(v4u& r, const uint8_t* base, uint32_t voff)
{
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3 nt" : "=&v"(r) : "v"(voff), "s"(base), "n"(OFF));
}

// five loads: the scales first, the four pieces behind them (loads FROM .. TO - 1 of the five)
template <int FROM = 0, int TO = 5>
MI355_DEVINL void w4p_issue(w4p_item& it, const uint8_t* block, uint32_t lane16, uint32_t lane2)
{
    if constexpr(FROM <= 0 && 0 < TO)
        asm volatile("global_load_ushort %0, %1, %2 nt" : "=&v"(it.sb) : "v"(lane2), "s"(block));
    if constexpr(FROM <= 1 && 1 < TO)
        w4p_load16_nt<128>(it.w[0], block, lane16);
    if constexpr(FROM <= 2 && 2 < TO)
        w4p_load16_nt<128 + 1024>(it.w[1], block, lane16);
    if constexpr(FROM <= 3 && 3 < TO)
        w4p_load16_nt<128 + 2048>(it.w[2], block, lane16);
    if constexpr(FROM <= 4 && 4 < TO)
        w4p_load16_nt<128 + 3072>(it.w[3], block, lane16);
}

// piece I of a block has arrived: BEHIND loads were issued after it
template <int BEHIND>
MI355_DEVINL void w4p_wait_piece(v4u& w)
{
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(w) : "n"(BEHIND));
}
template <int BEHIND>
MI355_DEVINL void w4p_wait_piece(v4u& w, uint32_t& sb)
{
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(w), "+v"(sb) : "n"(BEHIND));
}

MI355_DEVINL v8h w4p_pack(h2 a, h2 b, h2 c, h2 d)
{
    return __builtin_bit_cast(v8h, v4u{__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b),
                                       __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, d)});
}

struct w4p_consts
{
    h2 mul, add_n, add_s;
};

template <bool FAST>
MI355_DEVINL w4p_consts w4p_scale_consts(uint32_t sb, int zp, int zp_log2)
{
    const uint32_t spl = sb | (sb << 16);
    w4p_consts c;
    if(FAST)
    {
        // S = scale * 2^20 (exponent field + 20), -zp * scale (exponent + log2 zp, sign set; the
        // scale is positive), and the same / 16
        c.mul            = __builtin_bit_cast(h2, spl + 0x50005000u);
        const uint32_t z = zp == 0 ? 0u : spl + (((uint32_t)zp_log2 << 10) | 0x8000u) * 0x10001u;
        c.add_n          = __builtin_bit_cast(h2, z);
        c.add_s          = __builtin_bit_cast(h2, zp == 0 ? 0u : z - 0x10001000u);
    }
    else
    {
        c.mul                = __builtin_bit_cast(h2, spl);
        const uint32_t zbits = 0x6400u | (uint32_t)zp;
        c.add_n = c.add_s    = __builtin_bit_cast(h2, zbits | (zbits << 16));
    }
    return c;
}

// one piece: 16 rows x 128 k (32 per lane group) against the 32 activations of each lane group at
// `a_piece` (64 bytes, natural order)
template <bool FAST>
MI355_DEVINL void w4p_piece(const v4u& w, const w4p_consts& c, const uint8_t* a_piece, v4f (&acc)[4])
{
    const uint32_t d[4] = {w.x, w.y, w.z, w.w};
    h2 xn[4][2], xs[4][2];
#pragma unroll
    for(int j = 0; j < 4; j++)
    {
        const uint32_t t = d[j] >> 8;
        if(FAST)
        {
            xn[j][0] = __builtin_elementwise_fma(__builtin_bit_cast(h2, d[j] & 0x00F000F0u), c.mul, c.add_n);
            xn[j][1] = __builtin_elementwise_fma(__builtin_bit_cast(h2, t & 0x00F000F0u), c.mul, c.add_n);
            xs[j][0] = __builtin_elementwise_fma(__builtin_bit_cast(h2, d[j] & 0x000F000Fu), c.mul, c.add_s);
            xs[j][1] = __builtin_elementwise_fma(__builtin_bit_cast(h2, t & 0x000F000Fu), c.mul, c.add_s);
        }
        else
        {
            auto one = [&](uint32_t bits) {
                const h2 x = __builtin_bit_cast(h2, (bits & 0x000F000Fu) | 0x64006400u);
                return (x - c.add_n) * c.mul;
            };
            xn[j][0] = one(d[j] >> 4);
            xn[j][1] = one(t >> 4);
            xs[j][0] = one(d[j]);
            xs[j][1] = one(t);
        }
    }
    const v8h a0 = *reinterpret_cast<const v8h*>(a_piece);
    const v8h a1 = *reinterpret_cast<const v8h*>(a_piece + 16);
    const v8h a2 = *reinterpret_cast<const v8h*>(a_piece + 32);
    const v8h a3 = *reinterpret_cast<const v8h*>(a_piece + 48);
    acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, w4p_pack(xn[0][0], xn[0][1], xn[1][0], xn[1][1]), acc[0], 0,
                                                    0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, w4p_pack(xn[2][0], xn[2][1], xn[3][0], xn[3][1]), acc[1], 0,
                                                    0, 0);
    acc[2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a2, w4p_pack(xs[0][0], xs[0][1], xs[1][0], xs[1][1]), acc[2], 0,
                                                    0, 0);
    acc[3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a3, w4p_pack(xs[2][0], xs[2][1], xs[3][0], xs[3][1]), acc[3], 0,
                                                    0, 0);
}

// The blocks of one wave, written out in a straight line.  FAST: every scale is in the range of the
// fused-multiply-add form; a block that is not the wave's to take (a team past the last row group,
// a wave past the last block of its row group) is multiplied like any other, against a stretch of
// zero activations, so that the code has no branch and the compiler can overlap the LDS reads and
// the matrix-core latency of one piece with the vector work of the next.  The general form may
// meet scales that are not finite and skips such blocks instead.
// block idx of a wave: row group rg0 + (idx / IS) * rg_stride, block w + (idx % IS) * wk of it (a
// team past the last row group, or a wave past the last block, reads the last one and drops it)
template <int IS>
MI355_DEVINL const uint8_t* w4p_block_at(const w4p_params& p, int rg0, int w, int idx)
{
    const int rg = min(rg0 + (idx / IS) * p.rg_stride, p.nrg - 1);
    const int s  = min(w + (idx % IS) * p.wk, p.nss - 1);
    return p.pk + W4P_HEADER + ((int64_t)rg * p.nss + s) * W4P_BLOCK;
}

template <bool FAST, int MR, int IR, int IS>
MI355_DEVINL void w4p_blocks(const w4p_params& p, uint8_t* lds, const uint8_t* zeros, float* red, int rg0, int team,
                             int w, int lane, int zp)
{
    // MR = 16: lane l multiplies activation row l % 16 (rows past the last read the last one
    // again: rows of the result tile that nobody stores)
    const uint8_t* a_rows = MR == 1 ? lds : lds + min(lane & 15, p.m - 1) * p.a_pitch;
    constexpr int TOTAL = IR * IS;
    static_assert(TOTAL >= 1 && TOTAL <= 4);
    const int zp_log2 = zp <= 1 ? 0 : (zp == 2 ? 1 : (zp == 4 ? 2 : 3));
    // all of the wave's blocks are asked for at once
    w4p_item it[TOTAL];
#pragma unroll
    for(int i = 0; i < TOTAL; i++)
        w4p_issue(it[i], w4p_block_at<IS>(p, rg0, w, i), lane * 16, lane * 2);

    v4f acc[4];
#pragma unroll
    for(int c = 0; c < 4; c++)
        acc[c] = v4f{0.f, 0.f, 0.f, 0.f};
    auto block = [&](auto idx_tag) __attribute__((always_inline)) {
        constexpr int IDX = decltype(idx_tag)::value;
        // loads behind this block's: five for every later block
        constexpr int NEXT     = 5 * (TOTAL - 1 - IDX);
        w4p_item& b            = it[IDX];
        const int rg           = rg0 + (IDX / IS) * p.rg_stride;
        const int s            = w + (IDX % IS) * p.wk;
        const bool live        = rg < p.nrg && s < p.nss;
        const uint8_t* a_block = live || !FAST ? a_rows + s * 1024 + (lane >> 4) * 256 : zeros;
        w4p_wait_piece<3 + NEXT>(b.w[0], b.sb);
        const w4p_consts c = w4p_scale_consts<FAST>(b.sb, zp, zp_log2);
        if(FAST || live)
            w4p_piece<FAST>(b.w[0], c, a_block, acc);
        w4p_wait_piece<2 + NEXT>(b.w[1]);
        if(FAST || live)
            w4p_piece<FAST>(b.w[1], c, a_block + 64, acc);
        w4p_wait_piece<1 + NEXT>(b.w[2]);
        if(FAST || live)
            w4p_piece<FAST>(b.w[2], c, a_block + 128, acc);
        w4p_wait_piece<0 + NEXT>(b.w[3]);
        if(FAST || live)
            w4p_piece<FAST>(b.w[3], c, a_block + 192, acc);
        if constexpr(IDX % IS == IS - 1 && MR != 1)
        {
            // the whole result tile: lane l holds column l % 16 (a weight row) of activation rows
            // 4 * (l / 16) .. + 3.  One buffer for the partial sums, so a second barrier keeps the
            // next row group's sums out of it until the first wave has read these.
            const v4f mine = (acc[0] + acc[1]) + (acc[2] + acc[3]) * (FAST ? 16.0f : 1.0f);
            v4f* slot      = reinterpret_cast<v4f*>(red) + team * p.wk * 64;
            slot[w * 64 + lane] = mine;
            __syncthreads();
            if(w == 0 && rg < p.nrg)
            {
                v4f sum = slot[lane];
                for(int j = 1; j < p.wk; j++)
                    sum += slot[j * 64 + lane];
#pragma unroll
                for(int r = 0; r < 4; r++)
                {
                    const int row = 4 * (lane >> 4) + r;
                    if(row < p.m)
                        p.out[(int64_t)row * p.ldc + rg * 16 + (lane & 15)] = f32_to_half_rtz(sum[r]);
                }
            }
            __syncthreads();
#pragma unroll
            for(int c2 = 0; c2 < 4; c2++)
                acc[c2] = v4f{0.f, 0.f, 0.f, 0.f};
        }
        else if constexpr(IDX % IS == IS - 1)
        {
            // row 0 of the result tile: register 0 of lanes 0..15
            const float mine = (acc[0][0] + acc[1][0]) + (acc[2][0] + acc[3][0]) * (FAST ? 16.0f : 1.0f);
            float* slot      = red + (((IDX / IS) & 1) * p.teams + team) * (W4P_MAX_WAVES * 16);
            if(lane < 16)
                slot[w * 16 + lane] = mine;
            __syncthreads();
            if(w == 0 && lane < 16 && rg < p.nrg)
            {
                float sum = slot[lane];
                for(int j = 1; j < p.wk; j++)
                    sum += slot[j * 16 + lane];
                p.out[rg * 16 + lane] = f32_to_half_rtz(sum);
            }
#pragma unroll
            for(int c2 = 0; c2 < 4; c2++)
                acc[c2] = v4f{0.f, 0.f, 0.f, 0.f};
        }
    };
    block(std::integral_constant<int, 0>{});
    if constexpr(TOTAL > 1)
        block(std::integral_constant<int, 1>{});
    if constexpr(TOTAL > 2)
        block(std::integral_constant<int, 2>{});
    if constexpr(TOTAL > 3)
        block(std::integral_constant<int, 3>{});
}

// Workgroup = `teams` x `wk` waves.  A team works on one group of 16 weight rows at a time, its
// waves taking every wk-th block of it: IS blocks per wave and row group, IR row groups per team,
// IR * IS blocks per wave in all, two of them in flight.  At the end of a row group the team's
// partial sums meet in LDS and its first wave adds them in wave order (so the result does not
// depend on timing) and stores 16 outputs.
//
// The activation row is staged in LDS first and the weights are asked for behind the workgroup's
// barrier.  A CU takes load instructions only at the rate the memory returns data, so a wave with
// many loads to issue sits at its issue for microseconds; with the weights' loads in front of the
// barrier the workgroup could not start to multiply until its last wave had issued its last load.
template <int MR, int SLOTS, int IR, int IS>
__global__ __launch_bounds__(W4P_MAX_WAVES * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void
w4p_gemv_kernel(w4p_params p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int team = 0, w = wave;
    while(w >= p.wk)   // wave-uniform: at most `teams` - 1 rounds
    {
        w -= p.wk;
        team++;
    }
    const int nthreads = p.teams * p.wk * 64;
    uint8_t* zeros     = lds + (MR == 1 ? p.k * 2 : p.m * p.a_pitch); // 256 bytes
    float* red         = reinterpret_cast<float*>(zeros + 256);

    // half-precision arithmetic of this wave truncates from here on (MODE.fp_round bits 3:2); the
    // fp32 accumulation of the matrix cores is not affected.  Inline assembly: the compiler tracks a
    // mode change it emits itself and would restore the default in front of the packed-half code.
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 2, 2), 3" ::: "memory");

    // the header's zero point and flags (words 4 and 5), through the scalar cache
    uint64_t zp_flags;
    asm volatile("s_load_dwordx2 %0, %1, 0x10" : "=s"(zp_flags) : "s"(p.pk) : "memory");

    // The activations, 16-byte pieces: loads and LDS stores are unconditional.  A thread past the
    // end takes piece (number mod count) once more -- not one fixed piece: the same 16 bytes asked
    // for by half the threads of every workgroup on the chip queue up at one cache channel.
    const int row_pieces = p.k >> 3;
    const int a_pieces   = MR == 1 ? row_pieces : p.m * row_pieces;
    v4u areg[SLOTS];
    int aslot[SLOTS]; // byte offset of the piece in the LDS
#pragma unroll
    for(int s = 0; s < SLOTS; s++)
    {
        int i = tid + s * nthreads;
        i -= (int)__umulhi((uint32_t)i, p.all_magic) * a_pieces;
        int goff;
        if constexpr(MR == 1)
        {
            goff     = i * 16;
            aslot[s] = i * 16;
        }
        else
        {
            const int row = (int)__umulhi((uint32_t)i, p.row_magic);
            const int col = i - row * row_pieces;
            goff          = row * p.lda * 2 + col * 16;
            aslot[s]      = row * p.a_pitch + col * 16;
        }
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(areg[s]) : "v"(goff), "s"(p.a) : "memory");
    }
    const int rg0 = p.rg_base + blockIdx.x * p.teams + team;
    if(tid < 16)
        *reinterpret_cast<v4u*>(zeros + tid * 16) = v4u{0, 0, 0, 0};
    if constexpr(SLOTS == 1)
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(areg[0])::"memory");
    else if constexpr(SLOTS == 2)
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(areg[0]), "+v"(areg[1])::"memory");
    else if constexpr(SLOTS == 4)
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(areg[0]), "+v"(areg[1]), "+v"(areg[2]), "+v"(areg[3])::"memory");
    else
    {
        static_assert(SLOTS == 8);
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(areg[0]), "+v"(areg[1]), "+v"(areg[2]), "+v"(areg[3]), "+v"(areg[4]), "+v"(areg[5]),
                       "+v"(areg[6]), "+v"(areg[7])::"memory");
    }
#pragma unroll
    for(int s = 0; s < SLOTS; s++)
        *reinterpret_cast<v4u*>(lds + aslot[s]) = areg[s];
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(zp_flags)::"memory");
    const uint32_t flags = (uint32_t)(zp_flags >> 32);
    const int zp         = (int)(uint32_t)zp_flags;
    __syncthreads();

    // two separate bodies, each with its own loads and waits: a wait statement in each of two
    // branches for one load makes the compiler copy the loaded register in front of the branch
    if(__builtin_amdgcn_readfirstlane((flags & W4P_FLAG_GENERAL) == 0))
        w4p_blocks<true, MR, IR, IS>(p, lds, zeros, red, rg0, team, w, lane, zp);
    else
        w4p_blocks<false, MR, IR, IS>(p, lds, zeros, red, rg0, team, w, lane, zp);
}

template <int MR, int SLOTS>
int w4p_launch(const w4p_params& p, int grid, int threads, int lds, hipStream_t s)
{
#define W4P_CASE(R, S)                                                                                    \
    if(p.iters_r == R && p.iters_s == S)                                                                  \
    {                                                                                                     \
        auto kern = w4p_gemv_kernel<MR, SLOTS, R, S>;                                                     \
        if(lds > 64 * 1024)                                                                               \
        {                                                                                                 \
            /* above the default limit: opt in once per kernel instantiation */                          \
            static const hipError_t attr = hipFuncSetAttribute(                                           \
                reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            if(attr != hipSuccess)                                                                        \
                return MI355_ERR_LAUNCH;                                                                  \
        }                                                                                                 \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(threads), lds, s, p);                                   \
    }
    W4P_CASE(1, 1)
    W4P_CASE(2, 1)
    W4P_CASE(3, 1)
    W4P_CASE(4, 1)
    W4P_CASE(1, 2)
    W4P_CASE(2, 2)
    W4P_CASE(1, 3)
    W4P_CASE(1, 4)
#undef W4P_CASE
    return MI355_OK;
}

bool w4p_shape_ok(int64_t n, int64_t k, int64_t group)
{
    return group == W4P_GROUP && n > 0 && k > 0 && n % 16 == 0 && k % W4P_SUPER_K == 0 && k <= 28672 &&
           n <= (1 << 24) && (n / 16) * (k / W4P_SUPER_K) * (int64_t)W4P_BLOCK < (1ll << 40);
}

} // namespace

extern "C" size_t mi355_w4a16_prepacked_size(int64_t n, int64_t k, int64_t group)
{
    if(!w4p_shape_ok(n, k, group))
        return 0;
    return (size_t)W4P_HEADER + (size_t)(n / 16) * (size_t)(k / W4P_SUPER_K) * W4P_BLOCK;
}

// rows of activations the reordered form takes for this shape: one always; up to 16 as long as the
// rows (2 k + 16 bytes each), 256 zero bytes and one result tile per wave (16 KiB) fit the LDS
extern "C" int64_t mi355_w4a16_prepacked_max_rows(int64_t n, int64_t k, int64_t group)
{
    if(!w4p_shape_ok(n, k, group))
        return 0;
    const int64_t fit = (160 * 1024 - 256 - W4P_MAX_WAVES * 1024) / (2 * k + 16);
    return fit < 1 ? 1 : (fit > 16 ? 16 : fit);
}

extern "C" int mi355_w4a16_prepack(const void* w_packed,
                                   const void* scales,
                                   int32_t zp_scalar,
                                   int64_t n,
                                   int64_t k,
                                   int64_t group,
                                   void* prepacked,
                                   void* stream)
{
    if(w_packed == nullptr || scales == nullptr || prepacked == nullptr || zp_scalar < 0 || zp_scalar > 15)
        return MI355_ERR_BAD_ARG;
    if(!w4p_shape_ok(n, k, group) || reinterpret_cast<uintptr_t>(prepacked) % 16 != 0)
        return MI355_ERR_UNSUPPORTED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto* out     = static_cast<uint8_t*>(prepacked);
    hipLaunchKernelGGL(w4p_header_kernel, dim3(1), dim3(64), 0, s, out, (uint32_t)n, (uint32_t)k,
                       (uint32_t)zp_scalar);
    const int64_t pieces = (n / 16) * (k / W4P_SUPER_K) * 256;
    hipLaunchKernelGGL(w4p_prepack_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, s,
                       static_cast<const uint8_t*>(w_packed), static_cast<const uint16_t*>(scales), out, (int)n,
                       (int)k);
    return mi355_launch_status();
}

extern "C" int mi355_w4a16_gemm_prepacked(const void* a,
                                          int64_t lda,
                                          const void* prepacked,
                                          void* out,
                                          int64_t ldc,
                                          int64_t m,
                                          int64_t n,
                                          int64_t k,
                                          void* stream)
{
    if(a == nullptr || prepacked == nullptr || out == nullptr || m < 0 || lda < k || ldc < n)
        return MI355_ERR_BAD_ARG;
    if(!w4p_shape_ok(n, k, W4P_GROUP) || reinterpret_cast<uintptr_t>(a) % 16 != 0 ||
       reinterpret_cast<uintptr_t>(prepacked) % 16 != 0)
        return MI355_ERR_UNSUPPORTED;
    if(m == 0)
        return MI355_OK;
    if(m > 16)
        return MI355_ERR_UNSUPPORTED;
    const bool rows = m > 1;
    // several rows: 16-byte loads of every row, 32-bit byte offsets inside a
    if(rows && (lda % 8 != 0 || lda * 2 * 16 >= (1ll << 31) || ldc * 16 >= (1ll << 31)))
        return MI355_ERR_UNSUPPORTED;
    w4p_params p;
    p.pk  = static_cast<const uint8_t*>(prepacked);
    p.a   = static_cast<const uint16_t*>(a);
    p.out = static_cast<uint16_t*>(out);
    p.n   = (int)n;
    p.k   = (int)k;
    p.nss = (int)(k / W4P_SUPER_K);
    p.nrg = (int)(n / 16);
    p.m   = (int)m;
    p.lda = (int)lda;
    p.ldc = (int)ldc;
    p.a_pitch = (int)(2 * k + 16);
    const int row_pieces = (int)(k / 8);
    const int a_pieces   = (int)m * row_pieces;
    p.row_magic = (uint32_t)((((uint64_t)1 << 32) / (uint64_t)row_pieces) + 1);
    p.all_magic = (uint32_t)((((uint64_t)1 << 32) / (uint64_t)a_pieces) + 1);
    // Waves per row group (they split its blocks) and row groups per workgroup.  Measured on the
    // shapes of a Llama-sized layer: two blocks per wave and row group beat one (half as many
    // waves at the workgroup's barriers, one sum per two blocks) as long as the chip still gets
    // some eight waves per CU, and two row groups per workgroup beat one where a row group has
    // only four waves.
    p.iters_s = (p.nss + W4P_MAX_WAVES - 1) / W4P_MAX_WAVES;
    if(p.iters_s == 1 && p.nss >= 8 && p.nrg >= 384)
        p.iters_s = 2;
    p.wk    = (p.nss + p.iters_s - 1) / p.iters_s;
    p.teams = (p.wk <= 4 && p.nrg >= 384) ? 2 : 1;
    // the activations are staged with at most W4P_A_SLOTS (several rows: 8) pieces per thread
    const int max_slots = rows ? 8 : W4P_A_SLOTS;
    while(a_pieces > max_slots * p.teams * p.wk * 64 && (p.teams + 1) * p.wk <= W4P_MAX_WAVES)
        p.teams++;
    if(a_pieces > max_slots * p.teams * p.wk * 64)
        return MI355_ERR_UNSUPPORTED;
    const int threads  = p.teams * p.wk * 64;
    // one row: the row, 256 zero bytes, two buffers of 16 partial sums per wave; several rows: the
    // rows 2 k + 16 bytes apart, the zero bytes, one buffer of a whole result tile per wave
    const int lds = rows ? (int)m * p.a_pitch + 256 + p.teams * p.wk * 1024
                         : p.k * 2 + 256 + 2 * p.teams * W4P_MAX_WAVES * 16 * 4;
    if(lds > 160 * 1024)
        return MI355_ERR_UNSUPPORTED;
    const int wgs      = (p.nrg + p.teams - 1) / p.teams;
    // One resident set of workgroups (the kernel is built for 16 waves per CU), each walking up to
    // 4 / iters_s row groups.  More rows than that: one row group per workgroup and as many
    // workgroups as it takes, which the device deals out as others finish (measured at
    // (8192, 28672): 23.4 us against 29.5 as two launches over two halves of the rows).
    const int per_cu   = max(1, min(W4P_MAX_WAVES * 64 / threads, (160 * 1024) / lds));
    const int resident = 256 * per_cu;
    const int max_r    = 4 / p.iters_s;
    const int slots    = (a_pieces + threads - 1) / threads;
    hipStream_t s      = static_cast<hipStream_t>(stream);
    const bool overflow = wgs > resident * max_r;
    for(int done = 0; done < wgs;)
    {
        const int left = wgs - done;
        p.iters_r      = overflow ? 1 : min(max_r, (left + resident - 1) / resident);
        const int grid = overflow ? left
                                  : (left <= resident * p.iters_r ? (left + p.iters_r - 1) / p.iters_r : resident);
        p.rg_stride    = grid * p.teams;
        p.rg_base      = done * p.teams;
        int st;
        if(rows && slots <= 2)
            st = w4p_launch<16, 2>(p, grid, threads, lds, s);
        else if(rows && slots <= 4)
            st = w4p_launch<16, 4>(p, grid, threads, lds, s);
        else if(rows)
            st = w4p_launch<16, 8>(p, grid, threads, lds, s);
        else if(slots <= 1)
            st = w4p_launch<1, 1>(p, grid, threads, lds, s);
        else if(slots <= 2)
            st = w4p_launch<1, 2>(p, grid, threads, lds, s);
        else
            st = w4p_launch<1, W4P_A_SLOTS>(p, grid, threads, lds, s);
        if(st != MI355_OK)
            return st;
        done += grid * p.iters_r;
    }
    return mi355_launch_status();
}

