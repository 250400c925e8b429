// quant_dot on the gfx950 matrix cores, main kernel: int8 x int8 -> int32
// with v_mfma_i32_32x32x32_i8 and e4m3fn x e4m3fn -> fp32 with
// v_mfma_f32_32x32x64_f8f6f4, dequantizelinear / convert epilogue in registers.
//
// Data path: global memory -> LDS directly (global_load_lds_dwordx4, no
// register staging, no LDS store instructions), LDS -> MFMA operands.
//
// Tiling: a workgroup of 8 waves computes a 256 x 256 tile of C and walks K in
// slabs of 64 bytes.  Waves are arranged 2 (M) x 4 (N), each owning 128 x 64
// of the tile as 4 x 2 MFMA tiles of 32 x 32 (128 accumulator registers).
// LDS holds a ring of 4 slab stages (32 KiB each): the loads of slab kt+3 are
// issued while slab kt is multiplied, so a global load has about three slab
// times to land.  One barrier per slab, placed between the two halves of the
// slab's MFMAs so that the first operand reads of the next slab overlap the
// second half.
//
// LDS layouts (16-byte chunks, XOR swizzled so that operand reads are bank
// conflict free; a direct-to-LDS load writes lane l at base + 16*l, so the
// swizzle is applied to the global address each lane fetches):
//   K-contiguous operand (A, or B given as [N, K]): row r holds its 64 K bytes
//     as 4 chunks; logical chunk c sits at position c ^ ((r >> 2) & 3).
//   row-major B ([K, N]): row k holds 256 N bytes as 16 chunks; logical chunk c
//     sits at position c ^ (k & 7).  MFMA wants K-contiguous bytes per column:
//     ds_read_b64_tr_b8 does that transposition on the way out of LDS (a group
//     of 16 lanes reads an 8 (k) x 16 (n) byte block and each lane receives one
//     column).
#include "common.h"
#include <type_traits>

namespace {

typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM          = 256;
constexpr int BN          = 256;
constexpr int BK          = 64;
constexpr int STAGES      = 4;
constexpr int NTHREADS    = 512;
constexpr int A_BYTES     = BM * BK;
constexpr int STAGE_BYTES = (BM + BN) * BK;
constexpr int LDS_BYTES   = STAGES * STAGE_BYTES;
// The 16 x 16 int8 kernel keeps the K-contiguous A operand in stages of 128 K bytes (two slabs), so
// that every direct-to-LDS load instruction fetches whole 128-byte lines (8 rows x 128 bytes): a
// load of 16 rows x 64 bytes moves the same 16 lines from L2 for half the payload, and with all
// 256 CUs pulling such half lines the L2s deliver 28 instead of 40 bytes per clock and CU.
constexpr int A2_STAGES   = 2;
constexpr int A2_BYTES    = BM * 2 * BK; // one stage of A: 256 rows x 128 bytes
constexpr int B_BYTES     = BN * BK;     // one stage of B: one slab
constexpr int I8_B_BASE   = A2_STAGES * A2_BYTES;
constexpr int I8_LDS_BYTES = I8_B_BASE + STAGES * B_BYTES;

struct dma_params
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
    const int32_t* colsum_b;
    const int32_t* rowsum_a;
    const float* bias; // [N], added after the dequantization; null = none
    int scale_a_mode, scale_b_mode;
    int zp_a, zp_b;
    int ksplit; // workgroups along K per output tile (blockIdx.z), int8 split-K kernel only
    int32_t* partial; // split-K with a workspace: share z of batch b writes its tile sums to
                      // partial[(b * ksplit + z)][m][partial_ld] with plain stores; null = atomic adds
                      // into C
    int partial_ld;   // n rounded up to 4: a group of 4 columns that starts inside n is stored whole
    int vec_store; // rows of C keep groups of 4 outputs aligned to 4 elements
    int vec8_store; // 16-bit outputs: N % 8 == 0 and rows of C keep groups of 8 aligned to 16 bytes
    int stream_c;   // C is far larger than the caches: streaming stores
    int vec_cols;   // the per-column arrays in use (scale_b, colsum_b, bias) are 16-byte aligned and
                    // N % 4 == 0: four columns' values come with one load
    int64_t stride_cols = 0; // MI355_QP_PER_COL_BATCH: scale_b and bias hold one [N] vector per batch entry,
                             // this many elements apart (the dense int8 kernels only)
    // block-scaled operands (qgemm_dma_kernel<.., MX>): exponent bytes of the scales as
    // [batch][slab][rows rounded up to 256][4] (a slab of 64 operand bytes is 128 fp4 elements = 4
    // blocks of 32, or 64 fp8 elements = 2 blocks in bytes 0 and 1), and a word that, when it holds
    // this call's number, says the scales are not such exponents
    const uint8_t* mx_ea  = nullptr;
    const uint8_t* mx_eb  = nullptr;
    const uint32_t* mx_flag = nullptr;
    uint32_t mx_ticket      = 0; // the value of *mx_flag that says so
    int mx_rows_a = 0, mx_rows_b = 0;
};

// s_waitcnt with only the vector-memory counter constrained
template <int N>
MI355_DEVINL void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64);
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// s_barrier alone: __syncthreads() would also drain the vector-memory counter
// and with it the slabs that are meant to stay in flight.  The empty asm
// statements keep the compiler from moving LDS accesses across it.
MI355_DEVINL void block_barrier()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

MI355_DEVINL void load_to_lds(const uint8_t* g, uint8_t* l)
{
    // generic -> global / LDS address-space pointers need C-style casts
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g),
                                     (__attribute__((address_space(3))) void*)(l),
                                     16,
                                     0,
                                     0);
}

MI355_DEVINL v2i read_tr8(const uint8_t* l)
{
    return __builtin_amdgcn_ds_read_tr8_b64_v2i32((v2i __attribute__((address_space(3)))*)(l));
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
struct types
{
    using acc  = v16i;
    using frag = v4i;
};
template <>
struct types<true>
{
    using acc  = v16f;
    using frag = v8i;
};

// 16 bytes of C.  store_c: straight from the accumulators, where an instruction writes 32 or 64
// bytes of each of 16 or 32 rows.  store_rows: from the row-major copy in the LDS, where it writes
// whole 128-byte lines; `stream`: the result is large against the last-level cache and is written
// once, so a streaming (nontemporal) store keeps it from pushing out the operand panels that every L2
// miss of the main loop is served from (fp8 4096 x 28672 x 4096 -> fp32: 475 -> 461 us; no
// difference at 8192^3).  Only there: nontemporal stores of pieces of lines are far slower than
// plain ones (block-scaled 8192^3 through the eight-wave kernel: 376 -> 630 us).  Assembly: the
// compiler folds a nontemporal and a plain store of the same value behind a branch into one plain
// store.
template <class V>
MI355_DEVINL void store_c(V* dst, V v, bool)
{
    *dst = v;
}

template <class V>
MI355_DEVINL void store_rows(V* dst, V v, bool stream)
{
    static_assert(sizeof(V) == 16);
    if(stream)
        asm volatile("global_store_dwordx4 %0, %1, off nt" : : "v"(dst), "v"(v) : "memory");
    else
        *dst = v;
}

// two outputs of a 16-bit type in one word, the first in the low half
template <int OUT>
MI355_DEVINL uint32_t pack16(float lo, float hi)
{
    if constexpr(OUT == MI355_F16)
        return convert_f32_to_half(lo) | ((uint32_t)convert_f32_to_half(hi) << 16);
    else
        return convert_f32_to_bf16x2(lo, hi);
}

template <int OUT>
MI355_DEVINL void store1(void* c, int64_t idx, float v)
{
    if constexpr(OUT == MI355_F32)
        static_cast<float*>(c)[idx] = v;
    else if constexpr(OUT == MI355_F16)
        static_cast<uint16_t*>(c)[idx] = convert_f32_to_half(v);
    else
        static_cast<uint16_t*>(c)[idx] = convert_f32_to_bf16(v);
}

// MX = 4 or 8: the operands are packed fp4 (e2m1) or fp8 (e4m3fn) codes with one power-of-two scale
// per 32 elements along K, both K-contiguous.  Bytes are bytes: the loads, the LDS layout and the
// fragment reads are those of fp8 with B as [N, K].  fp4: a lane's two 16-byte chunks of a slab are
// two scale blocks, multiplied by two v_mfma_scale_f32_32x32x64_f8f6f4 (32 elements per lane each);
// fp8: its 32 bytes are one block and one instruction.  The exponent bytes of a row's slab (four,
// or two and two unused) travel through the LDS with the operands (2 KiB more per stage: one more
// load per wave and slab, sixteen lanes of it), and a lane shifts its own down to byte 0 (and 1).
// VIA_LDS: the result leaves through a row-major copy in the LDS (see the epilogue).  A separate
// instantiation: compiled into the same kernel behind a run-time choice, the copy's code made the
// direct stores of a large result 25 % slower (8192^3 block-scaled fp4: 382 -> 479 us) although the
// main loop and the direct epilogue came out instruction for instruction the same.
template <bool FP8, bool TRANS_B, bool DEQ, int OUT, int MX = 0, bool VIA_LDS = false>
__global__ __launch_bounds__(NTHREADS) void qgemm_dma_kernel(dma_params p)
{
    static_assert(MX == 0 || ((MX == 4 || MX == 8) && FP8 && TRANS_B && !DEQ),
                  "block scales: K-contiguous operands, bare result");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    using acc_t  = typename types<FP8>::acc;
    using frag_t = typename types<FP8>::frag;
    constexpr int ST        = MX ? STAGE_BYTES + 2048 : STAGE_BYTES; // bytes of one stage
    constexpr int PER_SLAB  = MX ? 5 : 4;                            // loads per wave and slab
    if constexpr(MX)
    {
        if(*p.mx_flag == p.mx_ticket)
            return;
    }

    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 2; // 0..1
    const int wave_n = wave & 3;  // 0..3

    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const uint8_t* __restrict__ ga = p.a + (int64_t)blockIdx.y * p.stride_a;
    const uint8_t* __restrict__ gb = p.b + (int64_t)blockIdx.y * p.stride_b;

    // ---- global -> LDS ----------------------------------------------------------
    // Each wave issues 4 loads of 1 KiB per slab: A row blocks {wave, wave+8}
    // (16 rows x 64 bytes each) and B blocks {wave, wave+8} (16 rows x 64 bytes
    // of [N, K] storage, or 4 rows x 256 bytes of [K, N] storage).
    uint32_t a_off[2], b_off[2];
#pragma unroll
    for(int h = 0; h < 2; h++)
    {
        const int blk = wave + 8 * h;
        {
            const int r     = 16 * blk + (lane >> 2);
            const int chunk = (lane & 3) ^ ((r >> 2) & 3);
            const int row   = min(m0 + r, p.m - 1);
            a_off[h]        = (uint32_t)row * (uint32_t)p.lda + chunk * 16;
        }
        if constexpr(TRANS_B)
        {
            const int r     = 16 * blk + (lane >> 2);
            const int chunk = (lane & 3) ^ ((r >> 2) & 3);
            const int col   = min(n0 + r, p.n - 1);
            b_off[h]        = (uint32_t)col * (uint32_t)p.ldb + chunk * 16;
        }
        else
        {
            const int k     = 4 * blk + (lane >> 4);
            const int chunk = (lane & 15) ^ (k & 7);
            const int col   = min(n0 + chunk * 16, p.n - 16);
            b_off[h]        = (uint32_t)k * (uint32_t)p.ldb + col;
        }
    }
    // one load at a time, so that the main loop can deal them out between runs of MFMAs (a load
    // occupies the CU's memory pipeline for about 47 cycles; 32 issued together stall every wave)
    auto issue_a = [&](int kt, int h) {
        uint8_t* st           = lds + (kt & (STAGES - 1)) * ST;
        const uint8_t* a_base = ga + (int64_t)kt * BK;
        load_to_lds(a_base + a_off[h], st + (wave + 8 * h) * 1024);
    };
    auto issue_b = [&](int kt, int h) {
        uint8_t* st           = lds + (kt & (STAGES - 1)) * ST;
        const uint8_t* b_base = TRANS_B ? gb + (int64_t)kt * BK : gb + (int64_t)kt * BK * p.ldb;
        load_to_lds(b_base + b_off[h], st + A_BYTES + (wave + 8 * h) * 1024);
    };
    // MX: the slab's exponent bytes, 1 KiB for the 256 rows of A (waves 0..3, a quarter each) and
    // 1 KiB for B (waves 4..7); issued with the B blocks
    const uint8_t* gs = nullptr;
    if constexpr(MX)
    {
        const bool for_b   = wave >= 4;
        const int rows     = for_b ? p.mx_rows_b : p.mx_rows_a;
        const int64_t per  = (int64_t)(p.k / BK) * rows * 4; // one batch
        gs = (for_b ? p.mx_eb : p.mx_ea) + (int64_t)blockIdx.y * per +
             ((int64_t)(for_b ? n0 : m0) + 64 * (wave & 3)) * 4 + (lane & 15) * 16;
    }
    auto issue_s = [&](int kt) {
        if constexpr(MX)
        {
            uint8_t* st    = lds + (kt & (STAGES - 1)) * ST + STAGE_BYTES + (wave >= 4 ? 1024 : 0) + (wave & 3) * 256;
            const int rows = wave >= 4 ? p.mx_rows_b : p.mx_rows_a;
            if(lane < 16)
                load_to_lds(gs + (int64_t)kt * rows * 4, st);
        }
    };
    auto issue_slab = [&](int kt) {
        issue_a(kt, 0);
        issue_a(kt, 1);
        issue_b(kt, 0);
        issue_b(kt, 1);
        issue_s(kt);
    };

    // ---- LDS -> operand fragments --------------------------------------------
    // A 32-row operand tile: lane l supplies row l % 32 and the K bytes of lane
    // group l / 32 (16 bytes per group for the K = 32 int8 instruction, 32 for
    // the K = 64 fp8 one).  A and B use the same K assignment.
    //
    // A slab is multiplied in two steps.  int8: step s is K bytes 32s..32s+31
    // against all 4 A tiles.  fp8: step s is all 64 K bytes against A tiles
    // 2s, 2s+1.
    //
    // The reads are inline assembly on purpose.  The compiler keeps no alias
    // information for direct-to-LDS loads, so in front of every LDS read it can
    // see it waits for ALL outstanding ones (vmcnt(0)), which would serialise
    // the slab pipeline; reads it cannot see leave the counters to the explicit
    // waits below.  Each fragment is tied ("+v") into the s_waitcnt statement
    // that must precede its first use, which is what orders the MFMAs.
    constexpr int A_TILES = FP8 ? 2 : 4;
    const int lrow        = lane & 31;
    const int lgrp        = lane >> 5;
    const int tr_i        = lane & 15;
    const int tr_g        = lane >> 4;
    const uint32_t lds0   = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);

    // per-lane byte offsets inside a stage, [step or part]
    uint32_t a_lane[2], b_lane[2];
    {
        const int sw = (lrow >> 2) & 3;
#pragma unroll
        for(int x = 0; x < 2; x++)
        {
            // int8: x = step (chunk 2x + lgrp); fp8: x = part (chunk 2*lgrp + x).  Block-scaled fp8:
            // the instruction takes K [16 g, 16 g + 16) and [32 + 16 g, ..) from lane group g and
            // scales K [32 g, 32 g + 32) by that group's exponent, so the group holds chunks g and
            // 2 + g, and the two groups' first halves are the block whose scale group 0 supplies.
            const int chunk = FP8 && MX != 8 ? 2 * lgrp + x : 2 * x + lgrp;
            a_lane[x]       = (wave_m * 128 + lrow) * BK + ((chunk ^ sw) << 4);
            if constexpr(TRANS_B)
                b_lane[x] = A_BYTES + (wave_n * 64 + lrow) * BK + ((chunk ^ sw) << 4);
        }
        if constexpr(!TRANS_B)
        {
            // lane 16g + i supplies the address of row k = kbase + (i >> 1), byte
            // half (i & 1) of the 16-byte chunk holding columns 16*(g & 1).. of
            // the tile, and receives column 16*(g & 1) + i with 8 consecutive k
            const int krow = (tr_g >> 1) * (FP8 ? 32 : 16) + (tr_i >> 1);
#pragma unroll
            for(int j = 0; j < 2; j++)
            {
                const int chunk = wave_n * 4 + j * 2 + (tr_g & 1);
                b_lane[j] = A_BYTES + krow * BN + ((chunk ^ (krow & 7)) << 4) + 8 * (tr_i & 1);
            }
        }
    }

    frag_t fa[2][A_TILES];
    frag_t fb[2][2];
    // MX: the exponent bytes of the lane's rows, [step][tile of the step]
    int sca[2][2] = {{0, 0}, {0, 0}}, scb[2][2] = {{0, 0}, {0, 0}};
    const uint32_t sa_lane = STAGE_BYTES + (wave_m * 128 + lrow) * 4;
    const uint32_t sb_lane = STAGE_BYTES + 1024 + (wave_n * 64 + lrow) * 4;
    const int sc_shift     = (MX == 4 ? 16 : 8) * lgrp;
    (void)sa_lane; (void)sb_lane; (void)sc_shift;

    auto rd128 = [](uint32_t addr, auto imm) -> v4i {
        v4i r;
        asm volatile("ds_read_b128 %0, %1 offset:%2"
                     : "=v"(r)
                     : "v"(addr), "n"(decltype(imm)::value)
                     : "memory");
        return r;
    };
    auto rdtr8 = [](uint32_t addr, auto imm) -> v2i {
        v2i r;
        asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2"
                     : "=v"(r)
                     : "v"(addr), "n"(decltype(imm)::value)
                     : "memory");
        return r;
    };
    auto rd32 = [](uint32_t addr, auto imm) -> int {
        int r;
        asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(decltype(imm)::value) : "memory");
        return r;
    };
#define IMM(x) std::integral_constant<int, (x)>{}

    // Issues the LDS reads of step S of the slab in `stage` into fa[S], fb[S].
    auto read_step = [&](int stage, auto step) {
        constexpr int S     = decltype(step)::value;
        const uint32_t base = lds0 + stage * ST;
        if constexpr(FP8)
        {
            const uint32_t a0 = base + a_lane[0], a1 = base + a_lane[1];
#pragma unroll
            for(int i = 0; i < 2; i++)
            {
                v4i lo, hi;
                if(i == 0)
                {
                    lo = rd128(a0, IMM((2 * S) * 32 * BK));
                    hi = rd128(a1, IMM((2 * S) * 32 * BK));
                }
                else
                {
                    lo = rd128(a0, IMM((2 * S + 1) * 32 * BK));
                    hi = rd128(a1, IMM((2 * S + 1) * 32 * BK));
                }
                fa[S][i] = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            }
            if constexpr(TRANS_B)
            {
                const uint32_t b0 = base + b_lane[0], b1 = base + b_lane[1];
                v4i lo0 = rd128(b0, IMM(0)), hi0 = rd128(b1, IMM(0));
                v4i lo1 = rd128(b0, IMM(32 * BK)), hi1 = rd128(b1, IMM(32 * BK));
                fb[S][0] = v8i{lo0.x, lo0.y, lo0.z, lo0.w, hi0.x, hi0.y, hi0.z, hi0.w};
                fb[S][1] = v8i{lo1.x, lo1.y, lo1.z, lo1.w, hi1.x, hi1.y, hi1.z, hi1.w};
                if constexpr(MX)
                {
                    sca[S][0] = rd32(base + sa_lane, IMM((2 * S) * 128));
                    sca[S][1] = rd32(base + sa_lane, IMM((2 * S + 1) * 128));
                    scb[S][0] = rd32(base + sb_lane, IMM(0));
                    scb[S][1] = rd32(base + sb_lane, IMM(128));
                }
            }
            else
            {
#pragma unroll
                for(int j = 0; j < 2; j++)
                {
                    const uint32_t bj = base + b_lane[j];
                    v2i p0 = rdtr8(bj, IMM(0)), p1 = rdtr8(bj, IMM(8 * BN));
                    v2i p2 = rdtr8(bj, IMM(16 * BN)), p3 = rdtr8(bj, IMM(24 * BN));
                    fb[S][j] = v8i{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
                }
            }
        }
        else
        {
            const uint32_t as = base + a_lane[S];
            fa[S][0]          = rd128(as, IMM(0));
            fa[S][1]          = rd128(as, IMM(32 * BK));
            fa[S][2]          = rd128(as, IMM(64 * BK));
            fa[S][3]          = rd128(as, IMM(96 * BK));
            if constexpr(TRANS_B)
            {
                const uint32_t bs = base + b_lane[S];
                fb[S][0]          = rd128(bs, IMM(0));
                fb[S][1]          = rd128(bs, IMM(32 * BK));
            }
            else
            {
#pragma unroll
                for(int j = 0; j < 2; j++)
                {
                    const uint32_t bj = base + b_lane[j];
                    v2i p0 = rdtr8(bj, IMM(S * 32 * BN)), p1 = rdtr8(bj, IMM(S * 32 * BN + 8 * BN));
                    fb[S][j] = v4i{p0.x, p0.y, p1.x, p1.y};
                }
            }
        }
    };
    // s_waitcnt lgkmcnt(0) that "produces" the fragments of step S: everything
    // that uses them is ordered behind it.  (A macro: asm operands that name
    // captured arrays do not compile inside a generic lambda.)
#define WAIT_STEP(S)                                                                            \
    do                                                                                          \
    {                                                                                           \
        if constexpr(MX)                                                                        \
        {                                                                                       \
            asm volatile("s_waitcnt lgkmcnt(0)"                                                 \
                         : "+v"(fa[S][0]), "+v"(fa[S][1]), "+v"(fb[S][0]), "+v"(fb[S][1]),      \
                           "+v"(sca[S][0]), "+v"(sca[S][1]), "+v"(scb[S][0]), "+v"(scb[S][1])   \
                         :                                                                      \
                         : "memory");                                                           \
            sca[S][0] >>= sc_shift; sca[S][1] >>= sc_shift;                                     \
            scb[S][0] >>= sc_shift; scb[S][1] >>= sc_shift;                                     \
        }                                                                                       \
        else if constexpr(FP8)                                                                  \
            asm volatile("s_waitcnt lgkmcnt(0)"                                                 \
                         : "+v"(fa[S][0]), "+v"(fa[S][1]), "+v"(fb[S][0]), "+v"(fb[S][1])       \
                         :                                                                      \
                         : "memory");                                                           \
        else                                                                                    \
            asm volatile("s_waitcnt lgkmcnt(0)"                                                 \
                         : "+v"(fa[S][0]), "+v"(fa[S][1]), "+v"(fa[S][A_TILES - 2]),            \
                           "+v"(fa[S][A_TILES - 1]), "+v"(fb[S][0]), "+v"(fb[S][1])             \
                         :                                                                      \
                         : "memory");                                                           \
    } while(0)
    auto mfma = [&](const frag_t& a, const frag_t& b, acc_t c) -> acc_t {
        if constexpr(FP8)
            // zero scale operands select the unscaled v_mfma_f32_32x32x64_f8f6f4;
            // cbsz = blgp = 0 means e4m3 for both operands
            return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    };

    acc_t acc[4][2];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 2; j++)
#pragma unroll
            for(int e = 0; e < 16; e++)
                acc[i][j][e] = 0;

    // half H (0, 1) of the MFMAs of step S
    auto mfma_half = [&](auto step, auto half) {
        constexpr int S = decltype(step)::value;
        constexpr int H = decltype(half)::value;
#pragma unroll
        for(int i = H * (A_TILES / 2); i < (H + 1) * (A_TILES / 2); i++)
#pragma unroll
            for(int j = 0; j < 2; j++)
            {
                const int tile = FP8 ? 2 * S + i : i;
                // B tile first: the accumulator holds the tile transposed, so that a lane owns
                // runs of 4 consecutive columns of C (see the epilogue)
                if constexpr(MX == 8)
                    acc[tile][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                        fb[S][j], fa[S][i], acc[tile][j], 0, 0, 0, scb[S][j], 0, sca[S][i]);
                else if constexpr(MX == 4)
                {
                    // chunk 0 of both lanes' pairs, then chunk 1: for 4-bit codes the instruction reads
                    // four registers per operand, so registers 4..7 serve as they are (the upper half
                    // of the shuffled vector is left undefined, which costs no copies)
                    acc[tile][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                        fb[S][j], fa[S][i], acc[tile][j], 4, 4, 0, scb[S][j], 0, sca[S][i]);
                    acc[tile][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                        __builtin_shufflevector(fb[S][j], fb[S][j], 4, 5, 6, 7, -1, -1, -1, -1),
                        __builtin_shufflevector(fa[S][i], fa[S][i], 4, 5, 6, 7, -1, -1, -1, -1), acc[tile][j], 4, 4, 1,
                        scb[S][j], 1, sca[S][i]);
                }
                else
                    acc[tile][j] = mfma(fb[S][j], fa[S][i], acc[tile][j]);
            }
    };

    // ---- main loop ---------------------------------------------------------------
    // Per slab: multiply step 0 while the step-1 fragments are read, barrier, multiply step 1 while
    // the first fragments of slab kt+1 are read.  The barrier sits between the two steps so that the
    // LDS latency of the next slab's first reads is covered by MFMAs.  The wave's four loads go out
    // singly behind the four halves of the MFMA work: the B blocks of slab kt+3 in step 0, the A
    // blocks of slab kt+4 in step 1.
    //
    // Slab kt+1 must be complete and visible to every wave, and every wave must have its last
    // fragments of slab kt in registers, before that barrier: the loads issued behind it (A blocks
    // of slab kt+4) overwrite the stage slab kt sits in.  At the wait in front of the barrier the
    // loads in flight are, in issue order, those of slabs kt+1, kt+2, kt+3.
    const int nk = p.k / BK;
#pragma unroll
    for(int s = 0; s < STAGES - 1; s++)
        if(s < nk)
            issue_slab(s);
    // slab 0 has landed when at most the loads of slabs 1 and 2 are outstanding
    if(nk >= 3)
        wait_vmcnt<2 * PER_SLAB>();
    else if(nk == 2)
        wait_vmcnt<PER_SLAB>();
    else
        wait_vmcnt<0>();
    block_barrier();
    if(STAGES - 1 < nk)
    {
        issue_a(STAGES - 1, 0);
        issue_a(STAGES - 1, 1);
    }
    read_step(0, IMM(0));

    for(int kt = 0; kt < nk; kt++)
    {
        const int stage = kt & (STAGES - 1);
        const bool ldb  = kt + STAGES - 1 < nk;
        const bool lda  = kt + STAGES < nk;
        // lgkmcnt counts every outstanding LDS read, so the wait for step 0
        // comes before the step-1 reads are issued, not after
        WAIT_STEP(0);
        read_step(stage, IMM(1));
        mfma_half(IMM(0), IMM(0));
        if(ldb)
            issue_b(kt + STAGES - 1, 0);
        mfma_half(IMM(0), IMM(1));
        if(ldb)
        {
            issue_b(kt + STAGES - 1, 1);
            issue_s(kt + STAGES - 1);
        }
        if(kt + 3 < nk)
            wait_vmcnt<2 * PER_SLAB>();
        else if(kt + 2 < nk)
            wait_vmcnt<PER_SLAB>();
        else
            wait_vmcnt<0>();
        WAIT_STEP(1);
        block_barrier();
        if(kt + 1 < nk)
            read_step((kt + 1) & (STAGES - 1), IMM(0));
        mfma_half(IMM(1), IMM(0));
        if(lda)
            issue_a(kt + STAGES, 0);
        mfma_half(IMM(1), IMM(1));
        if(lda)
            issue_a(kt + STAGES, 1);
    }
#undef IMM
#undef WAIT_STEP

    // ---- epilogue ------------------------------------------------------------------
    // The operands went in swapped, so element e of lane l belongs to row l % 32 of the A tile
    // and column 8*(e/4) + 4*(l/32) + e%4 of the B tile: four groups of 4 consecutive columns,
    // each written with one store when C allows it (p.vec_store).
    // Every scale, column sum and row sum this lane needs is loaded before the first store: a
    // load placed behind a store to C cannot be moved in front of it (C may alias), and 32 groups
    // of "load, wait out the latency, compute, store" in a row cost more than the main loop of a
    // short K.
    float sa_r[4]     = {1.f, 1.f, 1.f, 1.f};
    int64_t zrow_r[4] = {0, 0, 0, 0};
    float sb_c[2][4][4];
    int32_t cs_c[2][4][4];
    float bias_c[2][4][4];
    if constexpr(DEQ)
    {
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            const int row = min(m0 + wave_m * 128 + i * 32 + lrow, p.m - 1);
            if(p.scale_a_mode == MI355_QP_PER_TENSOR)
                sa_r[i] = p.scale_a[0];
            else if(p.scale_a_mode == MI355_QP_PER_ROW)
                sa_r[i] = p.scale_a[row];
            if(!FP8 && p.zp_b != 0)
                zrow_r[i] = (int64_t)p.zp_b * p.rowsum_a[row] - (int64_t)p.k * p.zp_a * p.zp_b;
        }
#pragma unroll
        for(int j = 0; j < 2; j++)
#pragma unroll
            for(int g = 0; g < 4; g++)
#pragma unroll
                for(int e = 0; e < 4; e++)
                {
                    const int c = min(n0 + wave_n * 64 + j * 32 + 8 * g + 4 * lgrp + e, p.n - 1);
                    float sb    = 1.f;
                    if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                        sb = p.scale_b[0];
                    else if(p.scale_b_mode == MI355_QP_PER_COL)
                        sb = p.scale_b[c];
                    sb_c[j][g][e] = sb;
                    cs_c[j][g][e] = (!FP8 && p.zp_a != 0) ? p.colsum_b[c] : 0;
                    if constexpr(FP8)
                        bias_c[j][g][e] = p.bias != nullptr ? p.bias[c] : -0.0f;
                }
    }
    // the int8 form of this kernel has no registers left for a bias: the launcher never sends
    // one here (only matrices whose N is no multiple of 4 come here with int8)
    auto bias_of = [&](int j, int g, int e) __attribute__((always_inline)) {
        if constexpr(FP8)
            return bias_c[j][g][e];
        else
            return -0.0f;
    };
    // fp8 (and the block-scaled products) where C takes whole groups: through a row-major copy in
    // the LDS, 32 rows of the wave's 128 x 64 part at a time (the operand stages are dead behind the
    // barrier).  Straight from the accumulators a store instruction writes 32 bytes of each of 32
    // rows; from the copy, the whole 256 bytes (fp32) of 4 rows or 128 bytes (16-bit) of 8.
    // Measured on this kernel (block-scaled products, whole call): 4096^3 fp4 68 -> 63 us and fp8
    // 96 -> 86 us, but 8192^3 fp4 424 -> 466 us and 4096 x 28672 x 4096 391 -> 423 us: with many
    // rounds of tiles and a result far larger than the caches the direct stores are faster here
    // (unlike in the four-wave kernels), so the launcher takes this form for results that stay
    // cached.  It requires p.vec_store, N % 4 == 0 and, for 16-bit outputs, p.vec8_store.
    if constexpr(FP8 && VIA_LDS)
    {
        constexpr int ESZ = DEQ && (OUT == MI355_F16 || OUT == MI355_BF16) ? 2 : 4;
        {
            block_barrier();
            constexpr int ROWB  = 64 * ESZ + 16;  // rows start 4 banks apart
            constexpr int PER   = 16 / ESZ;       // outputs per 16-byte piece
            constexpr int LANES = 64 / PER;       // lanes per row of the copy
            uint8_t* mine       = lds + wave * 16384;
            const int col       = n0 + wave_n * 64 + (lane % LANES) * PER;
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                const float sa = sa_r[i];
#pragma unroll
                for(int j = 0; j < 2; j++)
#pragma unroll
                    for(int g = 0; g < 4; g++)
                    {
                        float v[4];
#pragma unroll
                        for(int e = 0; e < 4; e++)
                        {
                            v[e] = acc[i][j][4 * g + e];
                            if constexpr(DEQ)
                                v[e] = add_bias(v[e] * (sa * sb_c[j][g][e]), bias_of(j, g, e));
                        }
                        uint8_t* dst = mine + lrow * ROWB + (32 * j + 8 * g + 4 * lgrp) * ESZ;
                        if constexpr(ESZ == 4)
                            *reinterpret_cast<v4f*>(dst) = v4f{v[0], v[1], v[2], v[3]};
                        else
                            *reinterpret_cast<uint2*>(dst) =
                                make_uint2(pack16<OUT>(v[0], v[1]), pack16<OUT>(v[2], v[3]));
                    }
                __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
                // every read before the first store (left to itself the compiler moves each read
                // into the branch of its store: read, wait, store, one at a time)
                constexpr int T = 32 * LANES / 64;
                v4u val[T];
#pragma unroll
                for(int t = 0; t < T; t++)
                    val[t] = *reinterpret_cast<const v4u*>(mine + (t * (64 / LANES) + lane / LANES) * ROWB +
                                                           (lane % LANES) * 16);
#pragma unroll
                for(int t = 0; t < T; t++)
                    asm volatile("" : "+v"(val[t]));
#pragma unroll
                for(int t = 0; t < T; t++)
                {
                    const int row = m0 + wave_m * 128 + 32 * i + t * (64 / LANES) + lane / LANES;
                    if(row < p.m && col < p.n)
                        store_rows(reinterpret_cast<v4u*>(
                                    static_cast<uint8_t*>(p.c) +
                                    ((int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col) * ESZ),
                                val[t], p.stream_c);
                }
            }
            return;
        }
    }
#pragma unroll
    for(int i = 0; i < 4; i++)
    {
        const int row = m0 + wave_m * 128 + i * 32 + lrow;
        if(row >= p.m)
            continue;
        const float sa     = sa_r[i];
        const int64_t zrow = zrow_r[i];
#pragma unroll
        for(int j = 0; j < 2; j++)
        {
            // 16-bit outputs: lanes l and l + 32 hold the two halves of the same 8 columns, for two
            // column groups; one v_permlane32_swap per register gives each of them one whole group,
            // which goes out as a single 16-byte store (half as many store instructions).  N % 8 == 0
            // there, so the two lanes are in or out of the matrix together.
            if constexpr(DEQ && (OUT == MI355_F16 || OUT == MI355_BF16))
            {
                if(p.vec8_store)
                {
#pragma unroll
                    for(int gp = 0; gp < 4; gp += 2)
                    {
                        uint32_t pk[2][2];
#pragma unroll
                        for(int h = 0; h < 2; h++)
                        {
                            float q[4];
#pragma unroll
                            for(int e = 0; e < 4; e++)
                            {
                                const float s = sa * sb_c[j][gp + h][e];
                                float v;
                                if constexpr(FP8)
                                    v = acc[i][j][4 * (gp + h) + e] * s;
                                else
                                {
                                    const int64_t zp = zrow + (int64_t)p.zp_a * cs_c[j][gp + h][e];
                                    const double d =
                                        (double)acc[i][j][4 * (gp + h) + e] - (double)(int32_t)zp;
                                    v = (float)(d * (double)s);
                                }
                                v    = add_bias(v, bias_of(j, gp + h, e));
                                q[e] = v;
                            }
                            pk[h][0] = pack16<OUT>(q[0], q[1]);
                            pk[h][1] = pack16<OUT>(q[2], q[3]);
                        }
                        const auto r0 = __builtin_amdgcn_permlane32_swap(pk[0][0], pk[1][0], false, false);
                        const auto r1 = __builtin_amdgcn_permlane32_swap(pk[0][1], pk[1][1], false, false);
                        const int col = n0 + wave_n * 64 + j * 32 + 8 * (gp + lgrp);
                        if(col < p.n)
                        {
                            const int64_t idx =
                                (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
                            store_c(reinterpret_cast<v4u*>(static_cast<uint16_t*>(p.c) + idx),
                                    v4u{r0[0], r1[0], r0[1], r1[1]}, p.stream_c);
                        }
                    }
                    continue;
                }
            }
#pragma unroll
            for(int g = 0; g < 4; g++)
            {
                const int col = n0 + wave_n * 64 + j * 32 + 8 * g + 4 * lgrp;
                if(col >= p.n)
                    continue;
                const int64_t idx = (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
                const bool whole  = p.vec_store && col + 4 <= p.n;
                float v[4];
                if constexpr(DEQ)
                {
#pragma unroll
                    for(int e = 0; e < 4; e++)
                    {
                        // scale = fp32 product of the two scales (the graph's `mul`), then
                        // (double(acc) - double(zp)) * scale in double, one rounding to float
                        // (dequantizelinear)
                        const float s = sa * sb_c[j][g][e];
                        if constexpr(FP8)
                        {
                            // the accumulator is a float: double(acc) * double(s) rounded once
                            // to float is exactly the correctly rounded fp32 product
                            v[e] = acc[i][j][4 * g + e] * s;
                        }
                        else
                        {
                            const int64_t zp = zrow + (int64_t)p.zp_a * cs_c[j][g][e];
                            const double d   = (double)acc[i][j][4 * g + e] - (double)(int32_t)zp;
                            v[e]             = (float)(d * (double)s);
                        }
                        v[e] = add_bias(v[e], bias_of(j, g, e));
                    }
                }
                if constexpr(!DEQ)
                {
                    using out_t = std::conditional_t<FP8, float, int32_t>;
                    out_t* o    = static_cast<out_t*>(p.c) + idx;
                    if(whole)
                    {
                        using vec_t = out_t __attribute__((ext_vector_type(4)));
                        store_c(reinterpret_cast<vec_t*>(o),
                                vec_t{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                                      acc[i][j][4 * g + 3]},
                                p.stream_c);
                    }
                    else
                    {
#pragma unroll
                        for(int e = 0; e < 4; e++)
                            if(col + e < p.n)
                                o[e] = acc[i][j][4 * g + e];
                    }
                }
                else if(whole)
                {
                    if constexpr(OUT == MI355_F32)
                        store_c(reinterpret_cast<v4f*>(static_cast<float*>(p.c) + idx), v4f{v[0], v[1], v[2], v[3]}, p.stream_c);
                    else if constexpr(OUT == MI355_F16)
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16),
                            convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16));
                    else
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_bf16x2(v[0], v[1]),
                            convert_f32_to_bf16x2(v[2], v[3]));
                }
                else
                {
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        if(col + e < p.n)
                            store1<OUT>(p.c, idx + e, v[e]);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// int8 with v_mfma_i32_16x16x64_i8.  Same data path, LDS layouts and slab ring
// as the kernel above; the wave's 128 x 64 block is 8 x 4 tiles of 16 x 16 and
// one MFMA covers the whole 64-byte slab.  Under uniformly random operands the
// chip is power limited and the 16 x 16 instruction sustains a higher rate than
// the 32 x 32 one, which is why int8 has its own kernel.
//
// The operands are passed swapped (B tile as the instruction's first operand):
// the accumulator then holds C transposed, lane l owning row (l % 16) of the A
// tile and 4 consecutive columns 4*(l / 16).. of the B tile, so C goes out in
// 16-byte stores.
//
// A slab is multiplied in two steps of 16 MFMAs (A tiles 0-3, then 4-7) with
// the barrier between them; the slab's four B fragments are shared by both
// steps and double buffered across slabs, so the loop body exists for both
// slab parities.
// ---------------------------------------------------------------------------
// SPLITK (bare int32 result only): blockIdx.z selects a share of the K slabs and the tile is
// added into a zero-filled C with integer atomics.  Integer addition commutes, so the result is
// the same bits whatever order the workgroups finish in.  This is what fills the machine when a
// skinny problem (few rows of A against a large B) has too few output tiles; 16-row tiles past the
// last row of A are skipped in the MFMA steps.
// VIA_LDS: the result (int32, or dequantized to fp32) leaves through a row-major copy in the LDS, as
// in qgemm_dma_kernel and for the reason given there a separate instantiation.
template <bool TRANS_B, bool DEQ, int OUT, bool VEC_STORE, bool SPLITK = false, bool VIA_LDS = false>
__global__ __launch_bounds__(NTHREADS) void qgemm_dma_i8_kernel(dma_params p)
{
    static_assert(!SPLITK || !DEQ, "split-K adds raw accumulators");
    // (with SPLITK: the partial sums of the workspace form, p.partial set)
    static_assert(!VIA_LDS || (VEC_STORE && (!DEQ || OUT == MI355_F32)), "32-bit results in groups of 4");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // one vector of column scales (and of the bias) per batch entry
    if constexpr(DEQ)
    {
        if(p.stride_cols != 0)
        {
            const int64_t off = (int64_t)blockIdx.y * p.stride_cols;
            p.scale_b += off;
            if(p.bias != nullptr)
                p.bias += off;
        }
    }
    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 2; // 0..1
    const int wave_n = wave & 3;  // 0..3

    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const uint8_t* __restrict__ ga = p.a + (int64_t)blockIdx.y * p.stride_a;
    const uint8_t* __restrict__ gb = p.b + (int64_t)blockIdx.y * p.stride_b;
    int nk = p.k / BK;
    if constexpr(SPLITK)
    {
        // slabs [s0, s1) of this workgroup
        const int per = (nk + p.ksplit - 1) / p.ksplit;
        const int s0  = min((int)blockIdx.z * per, nk);
        const int s1  = min(s0 + per, nk);
        ga += (int64_t)s0 * BK;
        gb += TRANS_B ? (int64_t)s0 * BK : (int64_t)s0 * BK * p.ldb;
        nk = s1 - s0;
        if(nk <= 0)
            return;
    }
    // 16-row tiles of this wave's 128-row block that hold rows of A
    const int live_tiles = SPLITK ? max(0, min(8, (p.m - (m0 + wave_m * 128) + 15) / 16)) : 8;

    // ---- global -> LDS ---------------------------------------------------------
    // A: stages of two slabs (128 K bytes).  One load instruction fetches 8 rows x 128 bytes, whole
    // lines; a wave issues blocks {wave, wave+8, wave+16, wave+24} of a stage.  Row r keeps its 8
    // 16-byte chunks at positions c ^ ((r >> 1) & 7), which makes the 16 rows x one chunk of an
    // operand read fall into 16 different bank groups.  B: one slab per stage as in the kernel above.
    uint32_t a_off[4], b_off[2];
    const int a_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7); // (r >> 1) & 7 of this lane's rows
#pragma unroll
    for(int h = 0; h < 4; h++)
    {
        const int r   = 8 * (wave + 8 * h) + (lane >> 3);
        const int row = min(m0 + r, p.m - 1);
        a_off[h]      = (uint32_t)row * (uint32_t)p.lda + a_chunk * 16;
    }
    // an odd number of slabs leaves the last stage half filled: the lanes of its second half
    // fetch the first half again instead of bytes past the end of the rows
    const uint32_t a_tail_back = a_chunk >= 4 ? 64u : 0u;
#pragma unroll
    for(int h = 0; h < 2; h++)
    {
        const int blk = wave + 8 * h;
        if constexpr(TRANS_B)
        {
            const int r     = 16 * blk + (lane >> 2);
            const int chunk = (lane & 3) ^ ((r >> 2) & 3);
            const int col   = min(n0 + r, p.n - 1);
            b_off[h]        = (uint32_t)col * (uint32_t)p.ldb + chunk * 16;
        }
        else
        {
            const int k     = 4 * blk + (lane >> 4);
            const int chunk = (lane & 15) ^ (k & 7);
            const int col   = min(n0 + chunk * 16, p.n - 16);
            b_off[h]        = (uint32_t)k * (uint32_t)p.ldb + col;
        }
    }
    // Loads go out one at a time, each between two runs of MFMAs: 32 of them issued together at
    // the top of a slab would hold every wave at its issue with the matrix cores idle.
    // ss: index of the 128-byte K step (slabs 2*ss and 2*ss + 1)
    auto issue_a = [&](int ss, int h) {
        uint8_t* st           = lds + (ss % A2_STAGES) * A2_BYTES;
        const uint8_t* a_base = ga + (int64_t)ss * (2 * BK);
        const uint32_t back   = 2 * ss + 1 < nk ? 0u : a_tail_back;
        load_to_lds(a_base + (a_off[h] - back), st + (wave + 8 * h) * 1024);
    };
    auto issue_b = [&](int kt, int h) {
        uint8_t* st           = lds + I8_B_BASE + (kt & (STAGES - 1)) * B_BYTES;
        const uint8_t* b_base = TRANS_B ? gb + (int64_t)kt * BK : gb + (int64_t)kt * BK * p.ldb;
        load_to_lds(b_base + b_off[h], st + (wave + 8 * h) * 1024);
    };

    // ---- LDS -> operand fragments ----------------------------------------------
    // 16-row operand tile: lane l supplies row l % 16 and K bytes 16*(l / 16)..
    const int lrow      = lane & 15;
    const int lgrp      = lane >> 4;
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    const int sw        = (lrow >> 2) & 3;
    // A: row stride 128 bytes; slab parity h reads logical chunks 4h .. 4h+3
    uint32_t a_lane[2];
#pragma unroll
    for(int h = 0; h < 2; h++)
        a_lane[h] = (wave_m * 128 + lrow) * (2 * BK) + (((4 * h + lgrp) ^ ((lrow >> 1) & 7)) << 4);
    uint32_t b_lane[2]; // K-contiguous B: one offset; row-major B: one per 8-row k block
    if constexpr(TRANS_B)
    {
        b_lane[0] = I8_B_BASE + (wave_n * 64 + lrow) * BK + ((lgrp ^ sw) << 4);
        b_lane[1] = 0;
    }
    else
    {
        // transposing read: lane 16g + i supplies row k = 16g + 8r + (i >> 1), byte
        // half (i & 1) of the 16-byte chunk with the tile's 16 columns, and
        // receives column i with 8 consecutive k (r = 0, 1)
#pragma unroll
        for(int r = 0; r < 2; r++)
        {
            const int k = lgrp * 16 + 8 * r + (lrow >> 1);
            // chunk index of tile j is wave_n*4 + j; its low bits are XORed with
            // k & 7, which for j in 0..3 only needs (j ^ x) on the low two bits
            b_lane[r] = I8_B_BASE + k * BN + 8 * (lrow & 1);
        }
    }
    const int bsw = (lrow >> 1) & 7; // k & 7 of this lane's row in the transposing read

    v4i fa[2][4];
    v4i fb[2][4];
    v4i acc[8][4];
#pragma unroll
    for(int i = 0; i < 8; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
            acc[i][j] = v4i{0, 0, 0, 0};

#define RD128(dst, addr, imm) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define RDTR8(dst, addr, imm) \
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")

    // A tile 4*S + E of slab kt (slab parity H = kt & 1, a constant where this is used) -> fa[S][E]
#define READ_A1(kt, H, S, E)                                                                 \
    RD128(fa[S][E], lds0 + (((kt) >> 1) % A2_STAGES) * A2_BYTES + a_lane[H],             \
          (4 * (S) + (E)) * 16 * 2 * BK)
#define READ_A(kt, H, S)      \
    do                        \
    {                         \
        READ_A1(kt, H, S, 0); \
        READ_A1(kt, H, S, 1); \
        READ_A1(kt, H, S, 2); \
        READ_A1(kt, H, S, 3); \
    } while(0)
    // B tile J of the slab in B stage `stage` -> fb[P][J]
#define READ_B1(stage, P, J)                                                               \
    do                                                                                     \
    {                                                                                      \
        const uint32_t s_ = lds0 + (stage) * B_BYTES;                                      \
        if constexpr(TRANS_B)                                                              \
        {                                                                                  \
            RD128(fb[P][J], s_ + b_lane[0], (J) * 16 * BK);                                \
        }                                                                                  \
        else                                                                               \
        {                                                                                  \
            const uint32_t c_ = (uint32_t)(((wave_n * 4 + (J)) ^ bsw) << 4);               \
            v2i lo_, hi_;                                                                  \
            RDTR8(lo_, s_ + b_lane[0] + c_, 0);                                            \
            RDTR8(hi_, s_ + b_lane[1] + c_, 0);                                            \
            fb[P][J] = v4i{lo_.x, lo_.y, hi_.x, hi_.y};                                    \
        }                                                                                  \
    } while(0)
#define READ_B(stage, P)      \
    do                        \
    {                         \
        READ_B1(stage, P, 0); \
        READ_B1(stage, P, 1); \
        READ_B1(stage, P, 2); \
        READ_B1(stage, P, 3); \
    } while(0)
#define WAIT4(x) \
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3])::"memory")
    // one MFMA: A tile 4*S + I against B tile J in fb[P]
#define MF(S, P, I, J)                                                                            \
    do                                                                                            \
    {                                                                                             \
        if(!SPLITK || 4 * (S) + (I) < live_tiles)                                                 \
            acc[4 * (S) + (I)][J] = __builtin_amdgcn_mfma_i32_16x16x64_i8(                        \
                fb[P][J], fa[S][I], acc[4 * (S) + (I)][J], 0, 0, 0);                              \
    } while(0)
    // the instruction order below is the schedule: nothing moves across these
#define SB() __builtin_amdgcn_sched_barrier(0)
    // One slab whose B fragments sit in fb[P]; the next slab's go to fb[1 - P].  P is also the slab's
    // parity, i.e. which half of the A stage it multiplies.  LDS reads and direct-to-LDS loads are
    // dealt out between the MFMAs, one at a time: issued in a bunch (12 reads by each of 8 waves right
    // behind the barrier, as an earlier version did) they fill the LDS and memory queues and every
    // wave sits at its issue with MFMAs waiting behind it in program order.
    //
    // Order of a wave's loads: B blocks of slab kt+3 in the first step of slab kt; the four A blocks
    // of K step s + A2_STAGES behind the barrier of slab 2s+1 (every wave then holds its last
    // fragments of K step s, whose stage they overwrite).  At the wait in front of the barrier of
    // slab kt, slab kt+1 must have landed; behind its last load the wave has issued, with three A
    // stages,
    //   kt even: B(kt+2), A(kt/2+2), B(kt+3)        kt odd: A((kt+3)/2), B(kt+2), B(kt+3)
    // and with two A stages
    //   kt even: B(kt+2), A(kt/2+1), B(kt+3)        kt odd: B(kt+2), B(kt+3)
    // (each where it exists): that many may stay in flight.
#define WAIT_LOADS(P)                                                                 \
    do                                                                                \
    {                                                                                 \
        int cnt_ = (kt_ + 2 < nk ? 2 : 0) + (kt_ + 3 < nk ? 2 : 0);                    \
        if((P) == 0)                                                                  \
            cnt_ += kt_ + 2 * A2_STAGES - 2 < nk ? 4 : 0;                             \
        else if(A2_STAGES == 3)                                                       \
            cnt_ += kt_ + 3 < nk ? 4 : 0;                                             \
        if(cnt_ == 8)      wait_vmcnt<8>();                                           \
        else if(cnt_ == 6) wait_vmcnt<6>();                                           \
        else if(cnt_ == 4) wait_vmcnt<4>();                                           \
        else if(cnt_ == 2) wait_vmcnt<2>();                                           \
        else               wait_vmcnt<0>();                                           \
    } while(0)
#define LOAD_A(h) \
    do { if((P_) == 1 && lda_) issue_a(((kt_) >> 1) + A2_STAGES, h); } while(0)
#define SLAB(kt, P)                                                                   \
    do                                                                                \
    {                                                                                 \
        constexpr int P_  = (P);                                                      \
        const int kt_     = (kt);                                                     \
        const int stage_  = kt_ & (STAGES - 1);                                       \
        const int nstage_ = (kt_ + 1) & (STAGES - 1);                                 \
        const bool more_  = kt_ + 1 < nk;                                             \
        const bool ldb_   = kt_ + STAGES - 1 < nk;                                    \
        const bool lda_   = 2 * ((kt_ >> 1) + A2_STAGES) < nk;                        \
        (void)stage_;                                                                 \
        WAIT4(fa[0]);                                                                 \
        WAIT4(fb[P]);                                                                 \
        SB();                                                                         \
        READ_A1(kt_, P_, 1, 0); SB(); MF(0, P, 0, 0); MF(0, P, 0, 1); SB();           \
        READ_A1(kt_, P_, 1, 1); SB(); MF(0, P, 0, 2); MF(0, P, 0, 3); SB();           \
        READ_A1(kt_, P_, 1, 2); SB(); MF(0, P, 1, 0); MF(0, P, 1, 1); SB();           \
        READ_A1(kt_, P_, 1, 3); SB(); MF(0, P, 1, 2); MF(0, P, 1, 3); SB();           \
        if(ldb_) issue_b(kt_ + STAGES - 1, 0);                                        \
        SB(); MF(0, P, 2, 0); MF(0, P, 2, 1); MF(0, P, 2, 2); MF(0, P, 2, 3); SB();   \
        if(ldb_) issue_b(kt_ + STAGES - 1, 1);                                        \
        SB(); MF(0, P, 3, 0); MF(0, P, 3, 1); MF(0, P, 3, 2); MF(0, P, 3, 3); SB();   \
        WAIT_LOADS(P);                                                                \
        WAIT4(fa[1]);                                                                 \
        block_barrier();                                                              \
        SB();                                                                         \
        if(more_) READ_A1(kt_ + 1, 1 - P_, 0, 0); SB(); MF(1, P, 0, 0); SB();         \
        if(more_) READ_A1(kt_ + 1, 1 - P_, 0, 1); SB(); MF(1, P, 0, 1); SB();         \
        if(more_) READ_A1(kt_ + 1, 1 - P_, 0, 2); SB(); MF(1, P, 0, 2); SB();         \
        if(more_) READ_A1(kt_ + 1, 1 - P_, 0, 3); SB(); MF(1, P, 0, 3); SB();         \
        if(more_) READ_B1(nstage_, 1 - (P), 0); SB(); MF(1, P, 1, 0); MF(1, P, 1, 1); SB(); \
        LOAD_A(0); SB();                                                              \
        if(more_) READ_B1(nstage_, 1 - (P), 1); SB(); MF(1, P, 1, 2); MF(1, P, 1, 3); SB(); \
        LOAD_A(1); SB();                                                              \
        if(more_) READ_B1(nstage_, 1 - (P), 2); SB(); MF(1, P, 2, 0); MF(1, P, 2, 1); SB(); \
        LOAD_A(2); SB();                                                              \
        if(more_) READ_B1(nstage_, 1 - (P), 3); SB(); MF(1, P, 2, 2); MF(1, P, 2, 3); SB(); \
        LOAD_A(3);                                                                    \
        SB(); MF(1, P, 3, 0); MF(1, P, 3, 1); MF(1, P, 3, 2); MF(1, P, 3, 3); SB();   \
    } while(0)

    // ---- main loop -----------------------------------------------------------------
    // Prologue in the order the waits above assume: A(0), B(0), [A(1)], B(1), B(2), A(last stage).
    {
#pragma unroll
        for(int h = 0; h < 4; h++)
            issue_a(0, h);
        issue_b(0, 0);
        issue_b(0, 1);
        if(A2_STAGES == 3 && 2 < nk)
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_a(1, h);
        }
#pragma unroll
        for(int s = 1; s < STAGES - 1; s++)
            if(s < nk)
            {
                issue_b(s, 0);
                issue_b(s, 1);
            }
        if(2 * (A2_STAGES - 1) < nk)
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_a(A2_STAGES - 1, h);
        }
    }
    // slab 0 has landed when only what was issued behind B(0) is outstanding
    {
        const int cnt = (1 < nk ? 2 : 0) + (2 < nk ? 2 : 0) + (A2_STAGES == 3 && 2 < nk ? 4 : 0) +
                        (2 * (A2_STAGES - 1) < nk ? 4 : 0);
        if(cnt == 12)      wait_vmcnt<12>();
        else if(cnt == 8)  wait_vmcnt<8>();
        else if(cnt == 6)  wait_vmcnt<6>();
        else if(cnt == 2)  wait_vmcnt<2>();
        else               wait_vmcnt<0>();
    }
    block_barrier();
    READ_A(0, 0, 0);
    READ_B(0, 0);
    int kt = 0;
    for(; kt + 1 < nk; kt += 2)
    {
        SLAB(kt, 0);
        SLAB(kt + 1, 1);
    }
    if(kt < nk)
        SLAB(kt, 0);
#undef LOAD_A
#undef WAIT_LOADS
#undef SLAB
#undef SB
#undef MF
#undef WAIT4
#undef READ_B
#undef READ_B1
#undef READ_A
#undef READ_A1
#undef RDTR8
#undef RD128

    // ---- epilogue ----------------------------------------------------------------
    // acc[i][j][e]: row 16*i + (l % 16) of the wave's A block, column
    // 16*j + 4*(l / 16) + e of its B block.
    // Scales, column sums and row sums are all loaded before the first store (a load behind a
    // store to C cannot move in front of it, and its latency would be paid once per group).
    float sb_c[4][4];
    int32_t cs_c[4][4];
    float bias_c[4][4];
    float sa_r[8];
    int64_t zrow_r[8];
    if constexpr(DEQ)
    {
#pragma unroll
        for(int j = 0; j < 4; j++)
#pragma unroll
            for(int e = 0; e < 4; e++)
            {
                const int c = min(n0 + wave_n * 64 + j * 16 + 4 * lgrp + e, p.n - 1);
                float sb    = 1.f;
                if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                    sb = p.scale_b[0];
                else if(p.scale_b_mode == MI355_QP_PER_COL)
                    sb = p.scale_b[c];
                sb_c[j][e] = sb;
                cs_c[j][e] = p.zp_a != 0 ? p.colsum_b[c] : 0;
                bias_c[j][e] = p.bias != nullptr ? p.bias[c] : -0.0f;
            }
#pragma unroll
        for(int i = 0; i < 8; i++)
        {
            const int row = min(m0 + wave_m * 128 + i * 16 + lrow, p.m - 1);
            float sa      = 1.f;
            if(p.scale_a_mode == MI355_QP_PER_TENSOR)
                sa = p.scale_a[0];
            else if(p.scale_a_mode == MI355_QP_PER_ROW)
                sa = p.scale_a[row];
            sa_r[i]   = sa;
            zrow_r[i] = p.zp_b != 0 ? (int64_t)p.zp_b * p.rowsum_a[row] - (int64_t)p.k * p.zp_a * p.zp_b : 0;
        }
    }
    if constexpr(VIA_LDS)
    {
        // 32 rows of the wave's 128 x 64 part at a time: written in the accumulators' layout (an
        // instruction's 64 bytes of each of 16 rows), read back along the rows, stored as the whole
        // 256 bytes of 4 rows per instruction.  The operand stages are dead behind the barrier.
        block_barrier();
        constexpr int ROWB = 256 + 16; // rows start 4 banks apart
        uint8_t* mine      = lds + wave * 16384;
        const int col      = n0 + wave_n * 64 + 4 * (lane & 15);
#pragma unroll
        for(int round = 0; round < 4; round++)
        {
#pragma unroll
            for(int i2 = 0; i2 < 2; i2++)
#pragma unroll
                for(int j = 0; j < 4; j++)
                {
                    const int i  = 2 * round + i2;
                    uint8_t* dst = mine + (16 * i2 + lrow) * ROWB + (16 * j + 4 * lgrp) * 4;
                    if constexpr(!DEQ)
                        *reinterpret_cast<v4i*>(dst) = acc[i][j];
                    else
                    {
                        float v[4];
#pragma unroll
                        for(int e = 0; e < 4; e++)
                        {
                            const float s  = sa_r[i] * sb_c[j][e];
                            const double d = (double)acc[i][j][e] -
                                             (double)(int32_t)(zrow_r[i] + (int64_t)p.zp_a * cs_c[j][e]);
                            v[e] = add_bias((float)(d * (double)s), bias_c[j][e]);
                        }
                        *reinterpret_cast<v4f*>(dst) = v4f{v[0], v[1], v[2], v[3]};
                    }
                }
            __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
            v4u val[8];
#pragma unroll
            for(int t = 0; t < 8; t++)
                val[t] = *reinterpret_cast<const v4u*>(mine + (4 * t + (lane >> 4)) * ROWB + (lane & 15) * 16);
#pragma unroll
            for(int t = 0; t < 8; t++)
                asm volatile("" : "+v"(val[t]));
#pragma unroll
            for(int t = 0; t < 8; t++)
            {
                const int row = m0 + wave_m * 128 + 32 * round + 4 * t + (lane >> 4);
                if(row < p.m && col < p.n)
                {
                    if constexpr(SPLITK)
                        *reinterpret_cast<v4u*>(
                            p.partial + (((int64_t)blockIdx.y * p.ksplit + blockIdx.z) * p.m + row) * p.partial_ld +
                            col) = val[t];
                    else
                        store_rows(reinterpret_cast<v4u*>(
                                    static_cast<uint8_t*>(p.c) +
                                    ((int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col) * 4),
                                val[t], p.stream_c);
                }
            }
        }
        return;
    }
#pragma unroll
    for(int j = 0; j < 4; j++)
    {
        const int col = n0 + wave_n * 64 + j * 16 + 4 * lgrp;
        if(col >= p.n)
            continue; // N is a multiple of 4 on this path, so the 4 columns are in or out together
#pragma unroll
        for(int i = 0; i < 8; i++)
        {
            const int row = m0 + wave_m * 128 + i * 16 + lrow;
            if(row >= p.m)
                continue;
            const int64_t idx = (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
            if constexpr(!DEQ)
            {
                int32_t* o = static_cast<int32_t*>(p.c) + idx;
                if constexpr(SPLITK)
                {
                    if(p.partial != nullptr)
                    {
                        int32_t* w = p.partial +
                                     (((int64_t)blockIdx.y * p.ksplit + blockIdx.z) * p.m + row) * p.partial_ld +
                                     col;
                        *reinterpret_cast<v4i*>(w) = acc[i][j];
                    }
                    else
                    {
#pragma unroll
                        for(int e = 0; e < 4; e++)
                            __hip_atomic_fetch_add(o + e, acc[i][j][e], __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
                else if constexpr(VEC_STORE)
                    store_c(reinterpret_cast<v4i*>(o), acc[i][j], p.stream_c);
                else
                {
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        o[e] = acc[i][j][e];
                }
            }
            else
            {
                float v[4];
#pragma unroll
                for(int e = 0; e < 4; e++)
                {
                    // scale = fp32 product of the two scales (the graph's `mul`),
                    // then (double(acc) - double(zp)) * scale in double, one
                    // rounding to float (dequantizelinear)
                    const float s  = sa_r[i] * sb_c[j][e];
                    const double d = (double)acc[i][j][e] -
                                     (double)(int32_t)(zrow_r[i] + (int64_t)p.zp_a * cs_c[j][e]);
                    v[e] = add_bias((float)(d * (double)s), bias_c[j][e]);
                }
                if constexpr(VEC_STORE)
                {
                    if constexpr(OUT == MI355_F32)
                        store_c(reinterpret_cast<v4f*>(static_cast<float*>(p.c) + idx), v4f{v[0], v[1], v[2], v[3]}, p.stream_c);
                    else if constexpr(OUT == MI355_F16)
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16),
                            convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16));
                    else
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_bf16x2(v[0], v[1]),
                            convert_f32_to_bf16x2(v[2], v[3]));
                }
                else
                {
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        store1<OUT>(p.c, idx + e, v[e]);
                }
            }
        }
    }
}


// ---------------------------------------------------------------------------------------------
// The same 256 x 256 tile with four waves, one per SIMD, each owning a 128 x 128 quadrant
// (8 x 8 MFMA tiles of 16 x 16: 256 accumulator registers, which the compiler keeps in the
// accumulation half of the register file).  Against the eight-wave kernel above every operand
// byte in LDS is read by half as many waves: 64 KiB of fragment reads per slab instead of 96,
// next to the 32 KiB the direct-to-LDS loads write.  The LDS serves about 146 bytes per clock to
// both together, so the eight-wave kernel needs 88 % of it at the full MFMA rate, this one 66 %.
//
// A slab's fragments are all in registers when its MFMAs start: they are read (into the other
// half of a double buffer) while the previous slab is multiplied, right behind the one barrier per
// slab.  That barrier tells a wave that slab kt+1 is complete in LDS and that every wave has
// finished reading slab kt, whose B stage then takes the loads of slab kt+4.  A has three stages
// of two slabs each; K step s is loaded in two halves during slabs 2s-5 and 2s-4, so every slab
// issues 4 B and 4 A load instructions per wave.
constexpr int W4_THREADS  = 256;
constexpr int W4_A_STAGES = 3;
constexpr int W4_B_BASE   = W4_A_STAGES * A2_BYTES;
constexpr int W4_LDS_BYTES = W4_B_BASE + STAGES * B_BYTES; // 96 + 64 KiB

// The steady state of the four-wave kernels runs in trips of twelve slabs (see qgemm_w4_i8_kernel).
// For slab U = 0 .. 11 of a trip (kt = 12 t + U), as compile-time constants:
// the A stage slab U is read from,
#define A_STAGE12(U) ((((U) >> 1)) % W4_A_STAGES)
// the A stage that the half K step loaded during slab U goes to (K step (kt + 5) / 2 in an odd
// slab, (kt + 4) / 2 in an even one), and the first of that half's four blocks
#define A_LOAD_STAGE12(U) ((((U) & 1) != 0 ? ((U) + 5) / 2 : ((U) + 4) / 2) % W4_A_STAGES)
#define A_LOAD_BLOCK12(U) (((U) & 1) != 0 ? 0 : 4)
// The trips themselves: SLAB(U) is the kernel's slab body; a trip runs only while every load of
// its slabs' shares exists (slab kt + 15 of B and K step (kt + 16) / 2 of A: kt + 17 < nk).
#define W4_TRIPS_OF_TWELVE(kt, nk, SLAB)                   \
    for(; (kt) + 17 < (nk); (kt) += 12)                    \
    {                                                      \
        SLAB(0); SLAB(1); SLAB(2);  SLAB(3);               \
        SLAB(4); SLAB(5); SLAB(6);  SLAB(7);               \
        SLAB(8); SLAB(9); SLAB(10); SLAB(11);              \
    }

template <bool TRANS_B, bool DEQ, int OUT, bool VEC_STORE>
__global__ __launch_bounds__(W4_THREADS) void qgemm_w4_i8_kernel(dma_params p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // one vector of column scales (and of the bias) per batch entry
    if constexpr(DEQ)
    {
        if(p.stride_cols != 0)
        {
            const int64_t off = (int64_t)blockIdx.y * p.stride_cols;
            p.scale_b += off;
            if(p.bias != nullptr)
                p.bias += off;
        }
    }
    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 1; // 0..1
    const int wave_n = wave & 1;  // 0..1

    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const uint8_t* __restrict__ ga = p.a + (int64_t)blockIdx.y * p.stride_a;
    const uint8_t* __restrict__ gb = p.b + (int64_t)blockIdx.y * p.stride_b;
    const int nk = p.k / BK;

    // ---- global -> LDS: the layouts of the eight-wave kernel, blocks dealt to four waves ----
    uint32_t a_off[8], b_off[4];
    const int a_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7); // (r >> 1) & 7 of this lane's rows
#pragma unroll
    for(int h = 0; h < 8; h++)
    {
        const int r   = 8 * (wave + 4 * h) + (lane >> 3);
        const int row = min(m0 + r, p.m - 1);
        a_off[h]      = (uint32_t)row * (uint32_t)p.lda + a_chunk * 16;
    }
    const uint32_t a_tail_back = a_chunk >= 4 ? 64u : 0u;
#pragma unroll
    for(int h = 0; h < 4; h++)
    {
        const int blk = wave + 4 * h;
        if constexpr(TRANS_B)
        {
            const int r     = 16 * blk + (lane >> 2);
            const int chunk = (lane & 3) ^ ((r >> 2) & 3);
            const int col   = min(n0 + r, p.n - 1);
            b_off[h]        = (uint32_t)col * (uint32_t)p.ldb + chunk * 16;
        }
        else
        {
            const int k     = 4 * blk + (lane >> 4);
            const int chunk = (lane & 15) ^ (k & 7);
            const int col   = min(n0 + chunk * 16, p.n - 16);
            b_off[h]        = (uint32_t)k * (uint32_t)p.ldb + col;
        }
    }
    // ss: index of the 128-byte K step (slabs 2*ss and 2*ss + 1); h: block 0..7 of this wave
    auto issue_a = [&](int ss, int h) {
        uint8_t* st           = lds + (ss % W4_A_STAGES) * A2_BYTES;
        const uint8_t* a_base = ga + (int64_t)ss * (2 * BK);
        const uint32_t back   = 2 * ss + 1 < nk ? 0u : a_tail_back;
        load_to_lds(a_base + (a_off[h] - back), st + (wave + 4 * h) * 1024);
    };
    auto issue_b = [&](int kt, int h) {
        uint8_t* st           = lds + W4_B_BASE + (kt & (STAGES - 1)) * B_BYTES;
        const uint8_t* b_base = TRANS_B ? gb + (int64_t)kt * BK : gb + (int64_t)kt * BK * p.ldb;
        load_to_lds(b_base + b_off[h], st + (wave + 4 * h) * 1024);
    };
    // what a wave issues during slab kt (kt from -4: the prologue runs the same sequence): the B
    // blocks of slab kt+4 and one half of an A step, K step (kt+5)/2 first half when kt is odd,
    // (kt+4)/2 second half when it is even
    auto a_step_of   = [](int kt) { return (kt & 1) != 0 ? (kt + 5) / 2 : (kt + 4) / 2; };
    auto issues_b    = [&](int kt) { return kt + 4 >= 0 && kt + 4 < nk; };
    auto issues_a    = [&](int kt) { const int ss = a_step_of(kt); return ss >= 1 && 2 * ss < nk; };
    auto issued_in   = [&](int kt) { return (issues_b(kt) ? 4 : 0) + (issues_a(kt) ? 4 : 0); };

    // ---- LDS -> operand fragments -------------------------------------------------------------
    const int lrow      = lane & 15;
    const int lgrp      = lane >> 4;
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    const int sw        = (lrow >> 2) & 3;
    uint32_t a_lane[2];
#pragma unroll
    for(int h = 0; h < 2; h++)
        a_lane[h] = (wave_m * 128 + lrow) * (2 * BK) + (((4 * h + lgrp) ^ ((lrow >> 1) & 7)) << 4);
    uint32_t b_lane[2];
    if constexpr(TRANS_B)
    {
        b_lane[0] = W4_B_BASE + (wave_n * 128 + lrow) * BK + ((lgrp ^ sw) << 4);
        b_lane[1] = 0;
    }
    else
    {
#pragma unroll
        for(int r = 0; r < 2; r++)
        {
            const int k = lgrp * 16 + 8 * r + (lrow >> 1);
            b_lane[r]   = W4_B_BASE + k * BN + 8 * (lrow & 1);
        }
    }
    const int bsw = (lrow >> 1) & 7; // k & 7 of this lane's row in the transposing read

    v4i fa[2][8];
    v4i fb[2][8];
    v4i acc[8][8];
#pragma unroll
    for(int i = 0; i < 8; i++)
#pragma unroll
        for(int j = 0; j < 8; j++)
            acc[i][j] = v4i{0, 0, 0, 0};

#define RD128(dst, addr, imm) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define RDTR8(dst, addr, imm) \
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define SB() __builtin_amdgcn_sched_barrier(0)
    // A tile I of slab kt -> fa[Q][I]
#define RA(kt, Q, I) \
    RD128(fa[Q][I], lds0 + (((kt) >> 1) % W4_A_STAGES) * A2_BYTES + a_lane[(kt) & 1], (I) * 16 * 2 * BK)
    // B tile J of slab kt: row-major B takes two reads (R = 0, 1), K-contiguous B one
#define RB(kt, Q, J, R)                                                                        \
    do                                                                                         \
    {                                                                                          \
        const uint32_t s_ = lds0 + ((kt) & (STAGES - 1)) * B_BYTES;                            \
        if constexpr(TRANS_B)                                                                  \
        {                                                                                      \
            if((R) == 0)                                                                       \
                RD128(fb[Q][J], s_ + b_lane[0], (J) * 16 * BK);                                \
        }                                                                                      \
        else                                                                                   \
        {                                                                                      \
            const uint32_t c_ = (uint32_t)(((wave_n * 8 + (J)) ^ bsw) << 4);                   \
            v2i t_;                                                                            \
            if((R) == 0)                                                                       \
            {                                                                                  \
                RDTR8(t_, s_ + b_lane[0] + c_, 0);                                             \
                fb[Q][J].x = t_.x;                                                             \
                fb[Q][J].y = t_.y;                                                             \
            }                                                                                  \
            else                                                                               \
            {                                                                                  \
                RDTR8(t_, s_ + b_lane[1] + c_, 0);                                             \
                fb[Q][J].z = t_.x;                                                             \
                fb[Q][J].w = t_.y;                                                             \
            }                                                                                  \
        }                                                                                      \
    } while(0)
    // every fragment of buffer Q has arrived
#define WAIT_FRAGS(Q)                                                                              \
    do                                                                                             \
    {                                                                                              \
        asm volatile("s_waitcnt lgkmcnt(0)"                                                        \
                     : "+v"(fa[Q][0]), "+v"(fa[Q][1]), "+v"(fa[Q][2]), "+v"(fa[Q][3]),             \
                       "+v"(fa[Q][4]), "+v"(fa[Q][5]), "+v"(fa[Q][6]), "+v"(fa[Q][7]),             \
                       "+v"(fb[Q][0]), "+v"(fb[Q][1]), "+v"(fb[Q][2]), "+v"(fb[Q][3]),             \
                       "+v"(fb[Q][4]), "+v"(fb[Q][5]), "+v"(fb[Q][6]), "+v"(fb[Q][7])::"memory");   \
    } while(0)
    // the same and at most 16 vector-memory operations in flight, as one instruction
#define WAIT_FRAGS_VM16(Q)                                                                         \
    do                                                                                             \
    {                                                                                              \
        asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)"                                              \
                     : "+v"(fa[Q][0]), "+v"(fa[Q][1]), "+v"(fa[Q][2]), "+v"(fa[Q][3]),             \
                       "+v"(fa[Q][4]), "+v"(fa[Q][5]), "+v"(fa[Q][6]), "+v"(fa[Q][7]),             \
                       "+v"(fb[Q][0]), "+v"(fb[Q][1]), "+v"(fb[Q][2]), "+v"(fb[Q][3]),             \
                       "+v"(fb[Q][4]), "+v"(fb[Q][5]), "+v"(fb[Q][6]), "+v"(fb[Q][7])::"memory");   \
    } while(0)
    // The MFMA as an assembly statement with the accumulator tied to the accumulation registers:
    // left to the register allocator, a part of the 256 accumulators ends up in ordinary
    // registers and scratch memory and is copied in and out around every instruction.  The
    // statements are volatile, so together with the LDS reads they stay in program order.
#define MF(Q, I, J)                                                   \
    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0"              \
                 : "+a"(acc[I][J])                                    \
                 : "v"(fb[Q][J]), "v"(fa[Q][I]))
    // two MFMAs, then one other instruction: slot N of 32 in a slab.  Slots 0..23 read the next
    // slab's fragments (8 A tiles, then 8 B tiles in two halves), slots 24..31 issue this slab's
    // share of the loads.
#define OTHER(kt, Q, N)                                                                     \
    do                                                                                      \
    {                                                                                       \
        if constexpr((N) < 8)                                                               \
        {                                                                                   \
            if(fast_ || more_) RA((kt) + 1, 1 - (Q), (N));                                  \
        }                                                                                   \
        else if constexpr((N) < 24)                                                         \
        {                                                                                   \
            if(fast_ || more_) RB((kt) + 1, 1 - (Q), ((N) - 8) >> 1, ((N) - 8) & 1);        \
        }                                                                                   \
        else if constexpr((N) < 28)                                                         \
        {                                                                                   \
            if(fast_ || ldb_) issue_b((kt) + 4, (N) - 24);                                  \
        }                                                                                   \
        else                                                                                \
        {                                                                                   \
            if(fast_ || lda_) issue_a(ass_, (1 - (Q)) * 4 + (N) - 28);                      \
        }                                                                                   \
    } while(0)
#define ROW(kt, Q, I)                                                                       \
    do                                                                                      \
    {                                                                                       \
        SB(); MF(Q, I, 0); MF(Q, I, 1); SB(); OTHER(kt, Q, 4 * (I) + 0);                     \
        SB(); MF(Q, I, 2); MF(Q, I, 3); SB(); OTHER(kt, Q, 4 * (I) + 1);                     \
        SB(); MF(Q, I, 4); MF(Q, I, 5); SB(); OTHER(kt, Q, 4 * (I) + 2);                     \
        SB(); MF(Q, I, 6); MF(Q, I, 7); SB(); OTHER(kt, Q, 4 * (I) + 3);                     \
    } while(0)
    // vector-memory operations that may stay in flight when slab kt+1 must be complete: what the
    // wave issued during slabs kt-2 and kt-1
#define WAIT_SLAB(kt)                                                                       \
    do                                                                                      \
    {                                                                                       \
        const int cnt_ = issued_in((kt) - 2) + issued_in((kt) - 1);                          \
        if(cnt_ >= 16)      wait_vmcnt<16>();                                               \
        else if(cnt_ >= 12) wait_vmcnt<12>();                                               \
        else if(cnt_ >= 8)  wait_vmcnt<8>();                                                \
        else if(cnt_ >= 4)  wait_vmcnt<4>();                                                \
        else                wait_vmcnt<0>();                                                \
    } while(0)
    // Q: the slab's parity (which fragment buffer it multiplies; an even slab issues the second
    // half of an A step, an odd one the first).  FAST: a slab of the steady state, where the next
    // slab and every load of the slab's share exist and the wait is for 16 operations.
#define SLAB(kt, Q, FAST)                                                                   \
    do                                                                                      \
    {                                                                                       \
        constexpr bool fast_ = (FAST);                                                      \
        const int kt_     = (kt);                                                           \
        const bool more_  = kt_ + 1 < nk;                                                   \
        const bool ldb_   = issues_b(kt_);                                                  \
        const bool lda_   = issues_a(kt_);                                                  \
        const int ass_    = a_step_of(kt_);                                                 \
        (void)more_; (void)ldb_; (void)lda_;                                                \
        WAIT_FRAGS(Q);                                                                      \
        if constexpr(fast_)                                                                 \
            wait_vmcnt<16>();                                                               \
        else if(more_)                                                                      \
            WAIT_SLAB(kt_);                                                                 \
        block_barrier();                                                                    \
        ROW(kt_, Q, 0); ROW(kt_, Q, 1); ROW(kt_, Q, 2); ROW(kt_, Q, 3);                     \
        ROW(kt_, Q, 4); ROW(kt_, Q, 5); ROW(kt_, Q, 6); ROW(kt_, Q, 7);                     \
        SB();                                                                               \
    } while(0)

    // ---- the steady state, twelve slabs per trip ---------------------------------------------
    // A wave issues in order and nothing it issues runs in the shadow of its own MFMAs: every
    // other instruction of the loop adds its issue time (about 4 cycles for a vector instruction,
    // 2.6 for a scalar one) to the 1024 cycles of a slab's 64 MFMAs.  The A stage of a slab repeats
    // every six slabs and its B stage every four, so in a trip of twelve every LDS address is a
    // register that never changes plus an immediate, every LDS destination of a load the wave's
    // base plus an immediate (written to M0 ahead of the MFMA pair the load follows, which also
    // covers the wait state between the two), and every global address a scalar base that advances
    // once per slab plus the lane's fixed 32-bit offset: a slab is its 64 MFMAs, 24 LDS reads,
    // 8 loads with their 8 M0 writes, three scalar additions, the waits and the barrier.
    uint32_t a_vaddr[2][2]; // [slab parity][0: stages 0 and 1, 1: stage 2 (beyond a 16-bit immediate)]
#pragma unroll
    for(int h = 0; h < 2; h++)
    {
        a_vaddr[h][0] = lds0 + a_lane[h];
        a_vaddr[h][1] = lds0 + a_lane[h] + 2 * A2_BYTES;
    }
    uint32_t b_vaddr[8][2];
#pragma unroll
    for(int j2 = 0; j2 < 8; j2++)
    {
        if constexpr(TRANS_B)
        {
            b_vaddr[j2][0] = lds0 + b_lane[0];
            b_vaddr[j2][1] = 0;
        }
        else
        {
            const uint32_t c_ = (uint32_t)(((wave_n * 8 + j2) ^ bsw) << 4);
            b_vaddr[j2][0]    = lds0 + b_lane[0] + c_;
            b_vaddr[j2][1]    = lds0 + b_lane[1] + c_;
        }
    }
    const uint32_t wave_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
#define RA12(U1, Q, I)                                                                         \
    RD128(fa[Q][I], a_vaddr[(U1) & 1][A_STAGE12(U1) == 2 ? 1 : 0],                             \
          (A_STAGE12(U1) == 2 ? 0 : A_STAGE12(U1) * A2_BYTES) + (I) * 16 * 2 * BK)
#define RB12(U1, Q, J, R)                                                                      \
    do                                                                                         \
    {                                                                                          \
        if constexpr(TRANS_B)                                                                  \
        {                                                                                      \
            if((R) == 0)                                                                       \
                RD128(fb[Q][J], b_vaddr[0][0], ((U1) & (STAGES - 1)) * B_BYTES + (J) * 16 * BK); \
        }                                                                                      \
        else                                                                                   \
        {                                                                                      \
            v2i t_;                                                                            \
            RDTR8(t_, b_vaddr[J][R], ((U1) & (STAGES - 1)) * B_BYTES);                         \
            if((R) == 0)                                                                       \
            {                                                                                  \
                fb[Q][J].x = t_.x;                                                             \
                fb[Q][J].y = t_.y;                                                             \
            }                                                                                  \
            else                                                                               \
            {                                                                                  \
                fb[Q][J].z = t_.x;                                                             \
                fb[Q][J].w = t_.y;                                                             \
            }                                                                                  \
        }                                                                                      \
    } while(0)
    // a row of eight MFMAs with a load behind every pair; M0 (the load's LDS destination) is
    // written between the two MFMAs of the pair, an MFMA away from the load that uses it and from
    // the load before (one statement: between two statements the compiler puts a wait state)
#define MF8_LOAD4(Q, I, LDS_CONST, OFF0, OFF1, OFF2, OFF3, BASE)                                 \
    asm volatile("v_mfma_i32_16x16x64_i8 %[c0], %[b0], %[a], %[c0]\n\t"                        \
                 "s_add_i32 m0, %[wl], %[lc0]\n\t"                                             \
                 "v_mfma_i32_16x16x64_i8 %[c1], %[b1], %[a], %[c1]\n\t"                        \
                 "global_load_lds_dwordx4 %[o0], %[base]\n\t"                                  \
                 "v_mfma_i32_16x16x64_i8 %[c2], %[b2], %[a], %[c2]\n\t"                        \
                 "s_add_i32 m0, %[wl], %[lc1]\n\t"                                             \
                 "v_mfma_i32_16x16x64_i8 %[c3], %[b3], %[a], %[c3]\n\t"                        \
                 "global_load_lds_dwordx4 %[o1], %[base]\n\t"                                  \
                 "v_mfma_i32_16x16x64_i8 %[c4], %[b4], %[a], %[c4]\n\t"                        \
                 "s_add_i32 m0, %[wl], %[lc2]\n\t"                                             \
                 "v_mfma_i32_16x16x64_i8 %[c5], %[b5], %[a], %[c5]\n\t"                        \
                 "global_load_lds_dwordx4 %[o2], %[base]\n\t"                                  \
                 "v_mfma_i32_16x16x64_i8 %[c6], %[b6], %[a], %[c6]\n\t"                        \
                 "s_add_i32 m0, %[wl], %[lc3]\n\t"                                             \
                 "v_mfma_i32_16x16x64_i8 %[c7], %[b7], %[a], %[c7]\n\t"                        \
                 "global_load_lds_dwordx4 %[o3], %[base]"                                      \
                 : [c0] "+a"(acc[I][0]), [c1] "+a"(acc[I][1]), [c2] "+a"(acc[I][2]),           \
                   [c3] "+a"(acc[I][3]), [c4] "+a"(acc[I][4]), [c5] "+a"(acc[I][5]),           \
                   [c6] "+a"(acc[I][6]), [c7] "+a"(acc[I][7])                                  \
                 : [b0] "v"(fb[Q][0]), [b1] "v"(fb[Q][1]), [b2] "v"(fb[Q][2]),                 \
                   [b3] "v"(fb[Q][3]), [b4] "v"(fb[Q][4]), [b5] "v"(fb[Q][5]),                 \
                   [b6] "v"(fb[Q][6]), [b7] "v"(fb[Q][7]), [a] "v"(fa[Q][I]),                  \
                   [wl] "s"(wave_lds), [lc0] "n"((LDS_CONST) + 0 * 4096),                      \
                   [lc1] "n"((LDS_CONST) + 1 * 4096), [lc2] "n"((LDS_CONST) + 2 * 4096),       \
                   [lc3] "n"((LDS_CONST) + 3 * 4096), [o0] "v"(OFF0), [o1] "v"(OFF1),          \
                   [o2] "v"(OFF2), [o3] "v"(OFF3), [base] "s"(BASE)                            \
                 : "memory", "scc")
#define ROW12_READS(U, Q, I, N0)                                                               \
    do                                                                                         \
    {                                                                                          \
        SB(); MF(Q, I, 0); MF(Q, I, 1); SB(); OTHER12(U, Q, (N0) + 0);                          \
        SB(); MF(Q, I, 2); MF(Q, I, 3); SB(); OTHER12(U, Q, (N0) + 1);                          \
        SB(); MF(Q, I, 4); MF(Q, I, 5); SB(); OTHER12(U, Q, (N0) + 2);                          \
        SB(); MF(Q, I, 6); MF(Q, I, 7); SB(); OTHER12(U, Q, (N0) + 3);                          \
    } while(0)
#define OTHER12(U, Q, N)                                                                       \
    do                                                                                         \
    {                                                                                          \
        if constexpr((N) < 8)                                                                  \
            RA12((U) + 1, 1 - (Q), (N));                                                       \
        else                                                                                   \
            RB12((U) + 1, 1 - (Q), ((N) - 8) >> 1, ((N) - 8) & 1);                             \
    } while(0)
#define SLAB12(U)                                                                              \
    do                                                                                         \
    {                                                                                          \
        constexpr int q_ = (U) & 1;                                                            \
        WAIT_FRAGS_VM16(q_);                                                                   \
        block_barrier();                                                                       \
        ROW12_READS(U, q_, 0, 0);  ROW12_READS(U, q_, 1, 4);  ROW12_READS(U, q_, 2, 8);        \
        ROW12_READS(U, q_, 3, 12); ROW12_READS(U, q_, 4, 16); ROW12_READS(U, q_, 5, 20);       \
        SB();                                                                                  \
        MF8_LOAD4(q_, 6, W4_B_BASE + (((U) + 4) & (STAGES - 1)) * B_BYTES,                     \
                  b_off[0], b_off[1], b_off[2], b_off[3], b_ptr);                              \
        MF8_LOAD4(q_, 7, A_LOAD_STAGE12(U) * A2_BYTES + A_LOAD_BLOCK12(U) * 4096,              \
                  a_off[A_LOAD_BLOCK12(U) + 0], a_off[A_LOAD_BLOCK12(U) + 1],                  \
                  a_off[A_LOAD_BLOCK12(U) + 2], a_off[A_LOAD_BLOCK12(U) + 3], a_ptr);          \
        SB();                                                                                  \
        b_ptr += b_step;                                                                       \
        if constexpr(((U) & 1) == 0)                                                           \
            a_ptr += 2 * BK;                                                                   \
    } while(0)

    // ---- main loop -----------------------------------------------------------------------------
    // Prologue: K step 0 of A, then what slabs -4 .. -1 would have issued.
#pragma unroll
    for(int h = 0; h < 8; h++)
        issue_a(0, h);
#pragma unroll
    for(int kt = -4; kt < 0; kt++)
    {
        if(issues_b(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_b(kt + 4, h);
        }
        if(issues_a(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_a(a_step_of(kt), ((kt & 1) != 0 ? 0 : 4) + h);
        }
    }
    // slab 0 is complete when only what came behind B(0) is in flight
    {
        const int cnt = issued_in(-3) + issued_in(-2) + issued_in(-1);
        if(cnt >= 24)      wait_vmcnt<24>();
        else if(cnt == 20) wait_vmcnt<20>();
        else if(cnt == 16) wait_vmcnt<16>();
        else if(cnt == 12) wait_vmcnt<12>();
        else if(cnt == 8)  wait_vmcnt<8>();
        else if(cnt == 4)  wait_vmcnt<4>();
        else               wait_vmcnt<0>();
    }
    block_barrier();
#pragma unroll
    for(int i = 0; i < 8; i++)
        RA(0, 0, i);
#pragma unroll
    for(int j = 0; j < 8; j++)
    {
        RB(0, 0, j, 0);
        RB(0, 0, j, 1);
    }
    int kt = 0;
    if(nk > 17)
    {
        // b_ptr: slab kt + 4 of B; a_ptr: K step a_step_of(kt) of A; both for the slab about to run
        const int64_t b_step = TRANS_B ? (int64_t)BK : (int64_t)BK * p.ldb;
        const uint8_t* b_ptr = gb + 4 * b_step;
        const uint8_t* a_ptr = ga + 2 * (2 * BK);
        uint32_t m0_saved;
        asm volatile("s_mov_b32 %0, m0" : "=s"(m0_saved));
        W4_TRIPS_OF_TWELVE(kt, nk, SLAB12);
        asm volatile("s_mov_b32 m0, %0" ::"s"(m0_saved));
    }
    for(; kt + 6 < nk; kt += 2)
    {
        SLAB(kt, 0, true);
        SLAB(kt + 1, 1, true);
    }
    for(; kt + 1 < nk; kt += 2)
    {
        SLAB(kt, 0, false);
        SLAB(kt + 1, 1, false);
    }
    if(kt < nk)
        SLAB(kt, 0, false);
    // The last MFMAs' results are read by ordinary instructions next: the wait states the compiler
    // would put behind an MFMA it knows.  The last row of accumulators passes through the statement,
    // so no read of it can move ahead; the rows before are at least eight MFMAs old.
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3"
                 : "+a"(acc[7][0]), "+a"(acc[7][1]), "+a"(acc[7][2]), "+a"(acc[7][3]),
                   "+a"(acc[7][4]), "+a"(acc[7][5]), "+a"(acc[7][6]), "+a"(acc[7][7]));
#undef SLAB12
#undef OTHER12
#undef ROW12_READS
#undef MF8_LOAD4
#undef RB12
#undef RA12
#undef SLAB
#undef WAIT_SLAB
#undef ROW
#undef OTHER
#undef MF
#undef WAIT_FRAGS_VM16
#undef WAIT_FRAGS
#undef RB
#undef RA
#undef SB
#undef RDTR8
#undef RD128

    // ---- epilogue: as in the eight-wave kernel, 8 x 8 tiles per wave ---------------------------
    // acc[i][j][e]: row 16*i + (l % 16) of the wave's A block, column 16*j + 4*(l / 16) + e of its
    // B block.
    if constexpr(!DEQ && VEC_STORE)
    {
        // The bare result through the LDS: stored straight from the accumulators an instruction
        // writes 64 bytes of each of 16 rows; re-read from a row-major copy in the LDS it writes the
        // 512 bytes of two whole rows of the wave's quadrant.  32 rows at a time, in two buffers of
        // the wave's own 40 KiB (the operand stages are dead: every wave is past its last fragment
        // read behind this barrier, and no load is in flight).
        block_barrier();
        constexpr int PITCH = 512 + 16; // bytes per row of the copy: rows start 4 banks apart
        uint8_t* mine       = lds + wave * 40960;
        const int out_col   = n0 + wave_n * 128 + 4 * (lane & 31);
        int32_t* out_base   = static_cast<int32_t*>(p.c) + (int64_t)blockIdx.y * p.stride_c + out_col;
#pragma unroll
        for(int pass = 0; pass < 4; pass++)
        {
            uint8_t* buf = mine + (pass & 1) * (32 * PITCH);
#pragma unroll
            for(int i2 = 0; i2 < 2; i2++)
#pragma unroll
                for(int j = 0; j < 8; j++)
                    *reinterpret_cast<v4i*>(buf + (16 * i2 + lrow) * PITCH + (16 * j + 4 * lgrp) * 4) =
                        acc[2 * pass + i2][j];
            __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): the wave's own writes are in the LDS
            // every read before the first store (left to itself the compiler moves each read into
            // the branch of its store: read, wait, store, one at a time)
            v4i val[16];
#pragma unroll
            for(int t = 0; t < 16; t++)
                val[t] = *reinterpret_cast<const v4i*>(buf + (2 * t + (lane >> 5)) * PITCH + (lane & 31) * 16);
#pragma unroll
            for(int t = 0; t < 16; t++)
                asm volatile("" : "+v"(val[t]));
#pragma unroll
            for(int t = 0; t < 16; t++)
            {
                const int row = m0 + wave_m * 128 + 32 * pass + 2 * t + (lane >> 5);
                if(row < p.m && out_col < p.n)
                    store_rows(reinterpret_cast<v4i*>(out_base + (int64_t)row * p.ldc), val[t], p.stream_c);
            }
        }
        return;
    }
    float sa_r[8];
    int64_t zrow_r[8];
    if constexpr(DEQ)
    {
#pragma unroll
        for(int i = 0; i < 8; i++)
        {
            const int row = min(m0 + wave_m * 128 + i * 16 + lrow, p.m - 1);
            float sa      = 1.f;
            if(p.scale_a_mode == MI355_QP_PER_TENSOR)
                sa = p.scale_a[0];
            else if(p.scale_a_mode == MI355_QP_PER_ROW)
                sa = p.scale_a[row];
            sa_r[i]   = sa;
            zrow_r[i] = p.zp_b != 0 ? (int64_t)p.zp_b * p.rowsum_a[row] - (int64_t)p.k * p.zp_a * p.zp_b : 0;
        }
    }
    // The scales, column sums and biases of a block of 16 columns are loaded ahead of the stores of
    // the block before it: a load issued behind a store waits for it.
    float sb_c[4], bias_c[4], sb_next[4], bias_next[4];
    int32_t cs_c[4], cs_next[4];
    auto load_block = [&](int j, float (&sb_o)[4], int32_t (&cs_o)[4], float (&bias_o)[4]) {
        if(p.vec_cols)
        {
            const int cv = min(n0 + wave_n * 128 + j * 16 + 4 * lgrp, p.n - 4);
            v4f sb4      = {1.f, 1.f, 1.f, 1.f};
            v4f bi4      = {-0.0f, -0.0f, -0.0f, -0.0f};
            v4i cs4      = {0, 0, 0, 0};
            if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                sb4 = v4f{p.scale_b[0], p.scale_b[0], p.scale_b[0], p.scale_b[0]};
            else if(p.scale_b_mode == MI355_QP_PER_COL)
                sb4 = *reinterpret_cast<const v4f*>(p.scale_b + cv);
            if(p.zp_a != 0)
                cs4 = *reinterpret_cast<const v4i*>(p.colsum_b + cv);
            if(p.bias != nullptr)
                bi4 = *reinterpret_cast<const v4f*>(p.bias + cv);
#pragma unroll
            for(int e = 0; e < 4; e++)
            {
                sb_o[e]   = sb4[e];
                cs_o[e]   = cs4[e];
                bias_o[e] = bi4[e];
            }
            return;
        }
#pragma unroll
        for(int e = 0; e < 4; e++)
        {
            const int c = min(n0 + wave_n * 128 + j * 16 + 4 * lgrp + e, p.n - 1);
            float sb    = 1.f;
            if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                sb = p.scale_b[0];
            else if(p.scale_b_mode == MI355_QP_PER_COL)
                sb = p.scale_b[c];
            sb_o[e]   = sb;
            cs_o[e]   = p.zp_a != 0 ? p.colsum_b[c] : 0;
            bias_o[e] = p.bias != nullptr ? p.bias[c] : -0.0f;
        }
    };
    if constexpr(DEQ)
        load_block(0, sb_c, cs_c, bias_c);
    // fp32 outputs, and 16-bit ones in whole groups of 8: through the LDS like the bare result.  The
    // wave's copy holds 256 bytes of each of its 128 rows: all 128 columns of a 16-bit type, or half
    // of them in fp32 (two rounds); an instruction then stores 256 contiguous bytes of 4 rows.
    if constexpr(DEQ && VEC_STORE)
    {
        // (16-bit outputs come here in whole groups of 8 only: launch_i8_one)
        {
            block_barrier();
            constexpr int ROWB = 256 + 16;               // rows start 4 banks apart
            constexpr int ESZ  = OUT == MI355_F32 ? 4 : 2;
            constexpr int JP   = OUT == MI355_F32 ? 4 : 8; // 16-column blocks per round
            uint8_t* mine      = lds + wave * 40960;
#pragma unroll
            for(int round = 0; round < 8 / JP; round++)
            {
#pragma unroll
                for(int jj = 0; jj < JP; jj++)
                {
                    const int j = round * JP + jj;
                    if(j > 0)
                    {
#pragma unroll
                        for(int e = 0; e < 4; e++)
                        {
                            sb_c[e]   = sb_next[e];
                            cs_c[e]   = cs_next[e];
                            bias_c[e] = bias_next[e];
                        }
                    }
                    if(j + 1 < 8)
                        load_block(j + 1, sb_next, cs_next, bias_next);
#pragma unroll
                    for(int i = 0; i < 8; i++)
                    {
                        float v[4];
#pragma unroll
                        for(int e = 0; e < 4; e++)
                        {
                            const float s  = sa_r[i] * sb_c[e];
                            const double d = (double)acc[i][j][e] -
                                             (double)(int32_t)(zrow_r[i] + (int64_t)p.zp_a * cs_c[e]);
                            v[e] = add_bias((float)(d * (double)s), bias_c[e]);
                        }
                        uint8_t* dst = mine + (16 * i + lrow) * ROWB + (16 * jj + 4 * lgrp) * ESZ;
                        if constexpr(OUT == MI355_F32)
                            *reinterpret_cast<v4f*>(dst) = v4f{v[0], v[1], v[2], v[3]};
                        else
                            *reinterpret_cast<uint2*>(dst) =
                                make_uint2(pack16<OUT>(v[0], v[1]), pack16<OUT>(v[2], v[3]));
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
                const int col = n0 + wave_n * 128 + round * (JP * 16) + (lane & 15) * (16 / ESZ);
#pragma unroll
                for(int t8 = 0; t8 < 32; t8 += 8)
                {
                    // eight reads before their eight stores (see the bare result above)
                    v4u val[8];
#pragma unroll
                    for(int t = 0; t < 8; t++)
                        val[t] = *reinterpret_cast<const v4u*>(mine + (4 * (t8 + t) + (lane >> 4)) * ROWB + (lane & 15) * 16);
#pragma unroll
                    for(int t = 0; t < 8; t++)
                        asm volatile("" : "+v"(val[t]));
#pragma unroll
                    for(int t = 0; t < 8; t++)
                    {
                        const int row = m0 + wave_m * 128 + 4 * (t8 + t) + (lane >> 4);
                        if(row < p.m && col < p.n)
                            store_rows(reinterpret_cast<v4u*>(static_cast<uint8_t*>(p.c) +
                                                           ((int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col) * ESZ),
                                    val[t], p.stream_c);
                    }
                }
            }
            return;
        }
    }
#pragma unroll
    for(int j = 0; j < 8; j++)
    {
        if constexpr(DEQ)
        {
            if(j > 0)
            {
#pragma unroll
                for(int e = 0; e < 4; e++)
                {
                    sb_c[e]   = sb_next[e];
                    cs_c[e]   = cs_next[e];
                    bias_c[e] = bias_next[e];
                }
            }
            if(j + 1 < 8)
                load_block(j + 1, sb_next, cs_next, bias_next);
        }
        const int col = n0 + wave_n * 128 + j * 16 + 4 * lgrp;
        if(col >= p.n)
            continue; // N is a multiple of 4 on this path, so the 4 columns are in or out together
#pragma unroll
        for(int i = 0; i < 8; i++)
        {
            const int row = m0 + wave_m * 128 + i * 16 + lrow;
            if(row >= p.m)
                continue;
            const int64_t idx = (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
            if constexpr(!DEQ)
            {
                int32_t* o = static_cast<int32_t*>(p.c) + idx;
                if constexpr(VEC_STORE)
                    store_c(reinterpret_cast<v4i*>(o), acc[i][j], p.stream_c);
                else
                {
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        o[e] = acc[i][j][e];
                }
            }
            else
            {
                float v[4];
#pragma unroll
                for(int e = 0; e < 4; e++)
                {
                    const float s  = sa_r[i] * sb_c[e];
                    const double d = (double)acc[i][j][e] -
                                     (double)(int32_t)(zrow_r[i] + (int64_t)p.zp_a * cs_c[e]);
                    v[e] = add_bias((float)(d * (double)s), bias_c[e]);
                }
                if constexpr(VEC_STORE)
                {
                    if constexpr(OUT == MI355_F32)
                        store_c(reinterpret_cast<v4f*>(static_cast<float*>(p.c) + idx), v4f{v[0], v[1], v[2], v[3]}, p.stream_c);
                    else if constexpr(OUT == MI355_F16)
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16),
                            convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16));
                    else
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_bf16x2(v[0], v[1]),
                            convert_f32_to_bf16x2(v[2], v[3]));
                }
                else
                {
#pragma unroll
                    for(int e = 0; e < 4; e++)
                        store1<OUT>(p.c, idx + e, v[e]);
                }
            }
        }
    }
}

template <bool TRANS_B, bool DEQ, int OUT, bool VEC>
int launch_i8_one(const dma_params& p, int batch, hipStream_t stream)
{
    dim3 grid(p.tiles_m * p.tiles_n, batch);
    // The four-wave kernel pays more per tile (a deeper pipeline to fill, 64 stores per wave at
    // the end) and less per slab: measured against the eight-wave kernel at 8192 x 8192 x K it is
    // 12 % slower at K = 1024, even at 2048, 2-15 % faster from 4096 on.
    constexpr bool half_out = DEQ && (OUT == MI355_F16 || OUT == MI355_BF16);
    if(p.k >= 3072 && (!VEC || !half_out || p.vec8_store))
    {
        auto kern = qgemm_w4_i8_kernel<TRANS_B, DEQ, OUT, VEC>;
        static const hipError_t attr = hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, W4_LDS_BYTES);
        if(attr != hipSuccess)
            return MI355_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, dim3(W4_THREADS), W4_LDS_BYTES, stream, p);
    }
    else
    {
        // 32-bit results in whole groups of 4 leave through the LDS copy
        constexpr bool lds_out = VEC && (!DEQ || OUT == MI355_F32);
        auto kern              = qgemm_dma_i8_kernel<TRANS_B, DEQ, OUT, VEC, false, lds_out>;
        static const hipError_t attr = hipFuncSetAttribute(
            reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, I8_LDS_BYTES);
        if(attr != hipSuccess)
            return MI355_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), I8_LDS_BYTES, stream, p);
    }
    return mi355_launch_status();
}

// zero C ahead of the split-K kernel (a kernel rather than a memset so that a captured graph
// replays it faithfully)
__global__ __launch_bounds__(256) void zero_i32_kernel(int32_t* c, int m, int n, int64_t ldc, int64_t stride_c)
{
    int32_t* base   = c + (int64_t)blockIdx.y * stride_c;
    const int64_t t = (int64_t)m * n;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < t; i += (int64_t)gridDim.x * 256)
        base[(i / n) * ldc + (i % n)] = 0;
}

// Second kernel of the split-K with a workspace: C = epilogue(sum of the shares' partial tiles).
// A thread column (threadIdx.x) owns 4 adjacent outputs; the 4 waves of a workgroup (threadIdx.y)
// each add every fourth share and the first one collects the four sums through the LDS.  int8:
// integer sums, any order gives the same bits, and the dequantizing epilogue is the arithmetic of
// the one-pass kernel's.  fp8: float partial sums added in this fixed order (the same bits on every
// run; not those of the one-pass kernel, whose one accumulator walks K in another order).  VEC: N,
// ldc and the batch stride of C are multiples of 4 and C is aligned for a store of 4 outputs;
// otherwise the outputs leave one by one (the partial rows are padded to a multiple of 4).
template <bool FP8, bool DEQ, int OUT, bool VEC>
__global__ __launch_bounds__(256) void reduce_partials_kernel(dma_params p, int shares)
{
    using acc_t = std::conditional_t<FP8, float, int32_t>;
    using vec_t = acc_t __attribute__((ext_vector_type(4)));
    __shared__ vec_t part[3][64];
    const int64_t mn  = (int64_t)p.m * p.partial_ld;
    const int64_t q   = (int64_t)blockIdx.x * 64 + threadIdx.x;
    const bool inside = 4 * q < mn;
    const acc_t* src  = reinterpret_cast<const acc_t*>(p.partial) + (int64_t)blockIdx.y * p.ksplit * mn + 4 * q;
    vec_t sum         = {0, 0, 0, 0};
    if(inside)
    {
#pragma unroll 4
        for(int z = threadIdx.y; z < shares; z += 4)
            sum += *reinterpret_cast<const vec_t*>(src + (int64_t)z * mn);
    }
    if(threadIdx.y > 0)
        part[threadIdx.y - 1][threadIdx.x] = sum;
    __syncthreads();
    if(threadIdx.y != 0 || !inside)
        return;
    sum               = ((sum + part[0][threadIdx.x]) + part[1][threadIdx.x]) + part[2][threadIdx.x];
    const int row     = (int)(4 * q / p.partial_ld);
    const int col     = (int)(4 * q % p.partial_ld);
    const int64_t idx = (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
    if constexpr(!DEQ)
    {
        if constexpr(VEC)
            *reinterpret_cast<vec_t*>(static_cast<acc_t*>(p.c) + idx) = sum;
        else
        {
#pragma unroll
            for(int e = 0; e < 4; e++)
                if(col + e < p.n)
                    static_cast<acc_t*>(p.c)[idx + e] = sum[e];
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
            zrow = p.zp_b != 0 ? (int64_t)p.zp_b * p.rowsum_a[row] - (int64_t)p.k * p.zp_a * p.zp_b : 0;
        float v[4];
#pragma unroll
        for(int e = 0; e < 4; e++)
        {
            const int c = min(col + e, p.n - 1);
            float sb    = 1.f;
            if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                sb = p.scale_b[0];
            else if(p.scale_b_mode == MI355_QP_PER_COL)
                sb = p.scale_b[c];
            const float bias = p.bias != nullptr ? p.bias[c] : -0.0f;
            const float s    = sa * sb;
            if constexpr(FP8)
                v[e] = add_bias((float)sum[e] * s, bias);
            else
            {
                const int32_t cs = p.zp_a != 0 ? p.colsum_b[c] : 0;
                const double d   = (double)sum[e] - (double)(int32_t)(zrow + (int64_t)p.zp_a * cs);
                v[e]             = add_bias((float)(d * (double)s), bias);
            }
        }
        if constexpr(!VEC)
        {
#pragma unroll
            for(int e = 0; e < 4; e++)
                if(col + e < p.n)
                    store1<OUT>(p.c, idx + e, v[e]);
        }
        else if constexpr(OUT == MI355_F32)
            *reinterpret_cast<v4f*>(static_cast<float*>(p.c) + idx) = v4f{v[0], v[1], v[2], v[3]};
        else if constexpr(OUT == MI355_F16)
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) =
                make_uint2(convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16),
                           convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16));
        else
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) =
                make_uint2(convert_f32_to_bf16x2(v[0], v[1]),
                           convert_f32_to_bf16x2(v[2], v[3]));
    }
}

template <bool FP8, bool VEC>
int launch_reduce_vec(const dma_params& p, int batch, int shares, bool deq, int out_type, hipStream_t stream)
{
    const int64_t quads = (int64_t)p.m * p.partial_ld / 4;
    const dim3 grid((unsigned)((quads + 63) / 64), batch), block(64, 4);
    if(!deq)
        hipLaunchKernelGGL((reduce_partials_kernel<FP8, false, MI355_F32, VEC>), grid, block, 0, stream, p, shares);
    else if(out_type == MI355_F32)
        hipLaunchKernelGGL((reduce_partials_kernel<FP8, true, MI355_F32, VEC>), grid, block, 0, stream, p, shares);
    else if(out_type == MI355_F16)
        hipLaunchKernelGGL((reduce_partials_kernel<FP8, true, MI355_F16, VEC>), grid, block, 0, stream, p, shares);
    else
        hipLaunchKernelGGL((reduce_partials_kernel<FP8, true, MI355_BF16, VEC>), grid, block, 0, stream, p, shares);
    return mi355_launch_status();
}

template <bool FP8>
int launch_reduce(const dma_params& p, int batch, int shares, bool deq, int out_type, hipStream_t stream)
{
    const bool vec = p.vec_store && p.n % 4 == 0;
    return vec ? launch_reduce_vec<FP8, true>(p, batch, shares, deq, out_type, stream)
               : launch_reduce_vec<FP8, false>(p, batch, shares, deq, out_type, stream);
}

// deq / out_type: the epilogue of the second kernel on the workspace path (the atomic path gives
// the bare int32 product only)
template <bool TRANS_B>
int launch_i8_splitk(const dma_params& p, int batch, hipStream_t stream, bool deq = false, int out_type = MI355_F32)
{
    auto kern    = qgemm_dma_i8_kernel<TRANS_B, false, MI355_F32, true, true>;
    auto kern_ws = qgemm_dma_i8_kernel<TRANS_B, false, MI355_F32, true, true, true>;
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, I8_LDS_BYTES);
    static const hipError_t attr_ws = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern_ws), hipFuncAttributeMaxDynamicSharedMemorySize, I8_LDS_BYTES);
    if(attr != hipSuccess || attr_ws != hipSuccess)
        return MI355_ERR_LAUNCH;
    if(p.partial != nullptr)
    {
        // the partial tiles of many rows leave through the LDS copy (whole rows of the wave's part
        // per store: M = 128, N = K = 8192 33.4 -> 32.0 us); a few rows are faster straight from the
        // accumulators (M = 16: 22.3 against 23.7 us with the copy's barrier and round trip)
        dim3 grid(p.tiles_m * p.tiles_n, batch, p.ksplit);
        hipLaunchKernelGGL(p.m > 64 ? kern_ws : kern, grid, dim3(NTHREADS), I8_LDS_BYTES, stream, p);
        // shares that hold slabs: the kernel gives ceil(nk / ksplit) slabs to each, the last ones
        // may be left with none (they write nothing)
        const int nk     = p.k / BK;
        const int per    = (nk + p.ksplit - 1) / p.ksplit;
        const int shares = (nk + per - 1) / per;
        return launch_reduce<false>(p, batch, shares, deq, out_type, stream);
    }
    const int64_t total = (int64_t)p.m * p.n;
    const int zb        = (int)min((int64_t)2048, (total + 255) / 256);
    hipLaunchKernelGGL(zero_i32_kernel, dim3(zb, batch), dim3(256), 0, stream,
                       static_cast<int32_t*>(p.c), p.m, p.n, p.ldc, p.stride_c);
    dim3 grid(p.tiles_m * p.tiles_n, batch, p.ksplit);
    hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), I8_LDS_BYTES, stream, p);
    return mi355_launch_status();
}

// K shares per tile for a bare int8 quant_dot whose tiles alone leave most of the 256 CUs idle;
// 1 = no split.  Measured on this kernel: one workgroup streams its operands at about 25 GB/s, and
// the atomic adds of a share cost about 11.5 us per 2^20 outputs, so the time is roughly
// T1 / S + c * S with T1 = operand bytes / (workgroups * 25 GB/s) and c = 11.5 us * outputs / 2^20;
// the minimum is at sqrt(T1 / c).
int choose_ksplit(int tiles, int batch, int nk, int64_t m, int64_t n, int64_t k)
{
    const int64_t wgs = (int64_t)tiles * batch;
    if(wgs >= 128 || nk < 8)
        return 1;
    const double bytes = (double)batch * ((double)m * k + (double)k * n);
    const double t1_us = bytes / ((double)wgs * 25e3);
    const double c_us  = 11.5 * (double)batch * (double)m * (double)n / 1048576.0;
    int s              = (int)(0.75 * __builtin_sqrt(t1_us / c_us));
    s                  = min(s, nk / 4); // at least four slabs per share keep the LDS ring busy
    s                  = min((int64_t)s, (512 + wgs - 1) / wgs);
    return max(s, 1);
}

// The same choice when the shares write partial tiles to a workspace and a second kernel adds them
// up (no atomics).  A cost model fitted to measurements on the MI355X, in microseconds: a workgroup
// walks a 64-deep slab in 0.74 and spends 12 on its prologue and epilogue; the launch takes
// ceil(workgroups / 256) such walks; the partial sums are written and read once at about 6 TB/s;
// the second kernel adds 6.  The count with the lowest estimate is taken if it beats the one-pass
// estimate by 5 %; every share keeps at least four slabs.
int choose_ksplit_ws(int tiles, int batch, int nk, int64_t m, int64_t n, int64_t k)
{
    (void)k;
    const int64_t wgs = (int64_t)tiles * batch;
    if(wgs >= 256 || nk < 8)
        return 1;
    auto walk = [&](int s) {
        const int per        = (nk + s - 1) / s;
        const int64_t rounds = (wgs * s + 255) / 256;
        return (0.74 * per + 12.0) * (double)rounds;
    };
    const double one_pass = walk(1);
    double best           = one_pass * 0.95;
    int best_s            = 1;
    for(int s = 2; s <= 64 && s <= nk / 4; s++)
    {
        const double partial = (double)s * batch * m * n * 8.0 / 6.0e6;
        const double t       = walk(s) + partial + 6.0;
        if(t < best)
        {
            best   = t;
            best_s = s;
        }
    }
    return best_s;
}

template <bool TRANS_B, bool VEC>
int launch_i8_out(const dma_params& p, int batch, bool deq, int out, hipStream_t s)
{
    if(!deq)
        return launch_i8_one<TRANS_B, false, MI355_F32, VEC>(p, batch, s);
    switch(out)
    {
    case MI355_F32: return launch_i8_one<TRANS_B, true, MI355_F32, VEC>(p, batch, s);
    case MI355_F16: return launch_i8_one<TRANS_B, true, MI355_F16, VEC>(p, batch, s);
    case MI355_BF16: return launch_i8_one<TRANS_B, true, MI355_BF16, VEC>(p, batch, s);
    default: return MI355_ERR_UNSUPPORTED;
    }
}


// ---------------------------------------------------------------------------------------------
// fp8 (e4m3fn) on the four-wave plan: the same loads, LDS stages, barrier and one-slab-ahead
// fragment reads as qgemm_w4_i8_kernel, with v_mfma_f32_32x32x64_f8f6f4.  A wave's 128 x 128
// quadrant is 4 x 4 tiles of 32 x 32 (16 accumulator registers each, 256 in all); a 32-row operand
// tile of one slab is 32 bytes per lane (lane l: row l % 32, K bytes 32 * (l / 32)..), read as two
// 16-byte chunks (A, or B given as [N, K]) or four transposing 8-byte reads (row-major B).
// 16 MFMAs of 64 cycles per slab, two other instructions behind each.
// The kernel is for C whose rows keep groups of 4 outputs whole and aligned (N % 4 == 0 and
// p.vec_store); VEC8: 16-bit outputs in groups of 8 (p.vec8_store).  The way C is stored is fixed at
// compile time: with both ways behind a run-time branch the compiler keeps the accumulators in
// scratch memory across the epilogue.
template <bool TRANS_B, bool DEQ, int OUT, bool VEC8>
__global__ __launch_bounds__(W4_THREADS) void qgemm_w4_f8_kernel(dma_params p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 1; // 0..1
    const int wave_n = wave & 1;  // 0..1

    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const uint8_t* __restrict__ ga = p.a + (int64_t)blockIdx.y * p.stride_a;
    const uint8_t* __restrict__ gb = p.b + (int64_t)blockIdx.y * p.stride_b;
    const int nk = p.k / BK;

    // ---- global -> LDS: exactly as in qgemm_w4_i8_kernel -------------------------------------
    uint32_t a_off[8], b_off[4];
    const int a_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
#pragma unroll
    for(int h = 0; h < 8; h++)
    {
        const int r   = 8 * (wave + 4 * h) + (lane >> 3);
        const int row = min(m0 + r, p.m - 1);
        a_off[h]      = (uint32_t)row * (uint32_t)p.lda + a_chunk * 16;
    }
    const uint32_t a_tail_back = a_chunk >= 4 ? 64u : 0u;
#pragma unroll
    for(int h = 0; h < 4; h++)
    {
        const int blk = wave + 4 * h;
        if constexpr(TRANS_B)
        {
            const int r     = 16 * blk + (lane >> 2);
            const int chunk = (lane & 3) ^ ((r >> 2) & 3);
            const int col   = min(n0 + r, p.n - 1);
            b_off[h]        = (uint32_t)col * (uint32_t)p.ldb + chunk * 16;
        }
        else
        {
            const int k     = 4 * blk + (lane >> 4);
            const int chunk = (lane & 15) ^ (k & 7);
            const int col   = min(n0 + chunk * 16, p.n - 16);
            b_off[h]        = (uint32_t)k * (uint32_t)p.ldb + col;
        }
    }
    auto issue_a = [&](int ss, int h) {
        uint8_t* st           = lds + (ss % W4_A_STAGES) * A2_BYTES;
        const uint8_t* a_base = ga + (int64_t)ss * (2 * BK);
        const uint32_t back   = 2 * ss + 1 < nk ? 0u : a_tail_back;
        load_to_lds(a_base + (a_off[h] - back), st + (wave + 4 * h) * 1024);
    };
    auto issue_b = [&](int kt, int h) {
        uint8_t* st           = lds + W4_B_BASE + (kt & (STAGES - 1)) * B_BYTES;
        const uint8_t* b_base = TRANS_B ? gb + (int64_t)kt * BK : gb + (int64_t)kt * BK * p.ldb;
        load_to_lds(b_base + b_off[h], st + (wave + 4 * h) * 1024);
    };
    auto a_step_of   = [](int kt) { return (kt & 1) != 0 ? (kt + 5) / 2 : (kt + 4) / 2; };
    auto issues_b    = [&](int kt) { return kt + 4 >= 0 && kt + 4 < nk; };
    auto issues_a    = [&](int kt) { const int ss = a_step_of(kt); return ss >= 1 && 2 * ss < nk; };
    auto issued_in   = [&](int kt) { return (issues_b(kt) ? 4 : 0) + (issues_a(kt) ? 4 : 0); };

    // ---- LDS -> operand fragments -------------------------------------------------------------
    const int lrow      = lane & 31;
    const int lgrp      = lane >> 5;
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    // A: rows of 128 bytes (two slabs); slab parity h, chunk x of this lane's 32 bytes is logical
    // chunk 4h + 2*lgrp + x at position c ^ ((row >> 1) & 7)
    uint32_t a_lane[2][2];
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int x = 0; x < 2; x++)
            a_lane[h][x] = (wave_m * 128 + lrow) * (2 * BK) + (((4 * h + 2 * lgrp + x) ^ ((lrow >> 1) & 7)) << 4);
    uint32_t b_lane[2];
    int bsw = 0, bcol = 0;
    if constexpr(TRANS_B)
    {
        const int sw = (lrow >> 2) & 3;
#pragma unroll
        for(int x = 0; x < 2; x++)
            b_lane[x] = W4_B_BASE + (wave_n * 128 + lrow) * BK + (((2 * lgrp + x) ^ sw) << 4);
    }
    else
    {
        // transposing read: lane 16g + i supplies row k = 32 * (g >> 1) + 8r + (i >> 1) (r = 0..3),
        // byte half (i & 1) of the 16-byte chunk with columns 16 * (g & 1).. of the tile, and
        // receives column 16 * (g & 1) + i with 8 consecutive k
        const int tr_i = lane & 15;
        const int tr_g = lane >> 4;
        const int krow = (tr_g >> 1) * 32 + (tr_i >> 1);
        b_lane[0]      = W4_B_BASE + krow * BN + 8 * (tr_i & 1);
        b_lane[1]      = 0;
        bsw            = krow & 7;
        bcol           = tr_g & 1;
    }

    v8i fa[2][4];
    v8i fb[2][4];
    v16f acc[4][4];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
#pragma unroll
            for(int e = 0; e < 16; e++)
                acc[i][j][e] = 0.f;

#define RD128(dst, addr, imm) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define RDTR8(dst, addr, imm) \
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define SB() __builtin_amdgcn_sched_barrier(0)
#define PUT4(frag, X, t)                \
    do                                  \
    {                                   \
        frag[4 * (X) + 0] = t.x;        \
        frag[4 * (X) + 1] = t.y;        \
        frag[4 * (X) + 2] = t.z;        \
        frag[4 * (X) + 3] = t.w;        \
    } while(0)
    // half X of A tile I of slab kt -> fa[Q][I]
#define RA(kt, Q, I, X)                                                                         \
    do                                                                                          \
    {                                                                                           \
        v4i t_;                                                                                 \
        RD128(t_, lds0 + (((kt) >> 1) % W4_A_STAGES) * A2_BYTES + a_lane[(kt) & 1][X],          \
              (I) * 32 * 2 * BK);                                                               \
        PUT4(fa[Q][I], X, t_);                                                                  \
    } while(0)
    // part R of B tile J of slab kt: row-major B four transposing reads, K-contiguous B two
#define RB(kt, Q, J, R)                                                                         \
    do                                                                                          \
    {                                                                                           \
        const uint32_t s_ = lds0 + ((kt) & (STAGES - 1)) * B_BYTES;                             \
        if constexpr(TRANS_B)                                                                   \
        {                                                                                       \
            if((R) < 2)                                                                         \
            {                                                                                   \
                v4i t_;                                                                         \
                RD128(t_, s_ + b_lane[(R) & 1], (J) * 32 * BK);                                 \
                PUT4(fb[Q][J], (R) & 1, t_);                                                    \
            }                                                                                   \
        }                                                                                       \
        else                                                                                    \
        {                                                                                       \
            const uint32_t c_ = (uint32_t)(((wave_n * 8 + (J) * 2 + bcol) ^ bsw) << 4);         \
            v2i t_;                                                                             \
            RDTR8(t_, s_ + b_lane[0] + c_, (R) * 8 * BN);                                       \
            fb[Q][J][2 * (R) + 0] = t_.x;                                                       \
            fb[Q][J][2 * (R) + 1] = t_.y;                                                       \
        }                                                                                       \
    } while(0)
#define WAIT_FRAGS(Q)                                                                           \
    asm volatile("s_waitcnt lgkmcnt(0)"                                                         \
                 : "+v"(fa[Q][0]), "+v"(fa[Q][1]), "+v"(fa[Q][2]), "+v"(fa[Q][3]),              \
                   "+v"(fb[Q][0]), "+v"(fb[Q][1]), "+v"(fb[Q][2]), "+v"(fb[Q][3])::"memory")
    // The B tile goes in first: the accumulator then holds the tile transposed and a lane owns runs
    // of four consecutive columns of C (see the epilogue).  Assembly for the reason given in
    // qgemm_w4_i8_kernel.  The compiler does not know that the statement is an MFMA and adds none
    // of the wait states a 16-pass MFMA needs before its result may be read.  In the steady-state
    // loop nothing reads an accumulator.  In the last slabs, whose loads and reads are conditional,
    // the compiler keeps copies of the accumulators in scratch memory and stores them right behind
    // the MFMA, so there the statement carries the wait states itself.
#define MF(Q, I, J)                                                                        \
    do                                                                                     \
    {                                                                                      \
        if constexpr(fast_)                                                                \
            asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0"                       \
                         : "+a"(acc[I][J])                                                 \
                         : "v"(fb[Q][J]), "v"(fa[Q][I]));                                  \
        else                                                                               \
            asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0\n\t"                   \
                         "s_nop 7\n\ts_nop 7\n\ts_nop 3"                                   \
                         : "+a"(acc[I][J])                                                 \
                         : "v"(fb[Q][J]), "v"(fa[Q][I]));                                  \
    } while(0)
    // slot N of 32: 0..7 A reads, 8..23 B reads (8..15 when B is K-contiguous), 24..31 loads.
#define OTHER(kt, Q, N)                                                                     \
    do                                                                                      \
    {                                                                                       \
        if constexpr((N) < 8)                                                               \
        {                                                                                   \
            if(fast_ || more_) RA((kt) + 1, 1 - (Q), (N) >> 1, (N) & 1);                   \
        }                                                                                   \
        else if constexpr((N) < 24)                                                         \
        {                                                                                   \
            if(fast_ || more_) RB((kt) + 1, 1 - (Q), ((N) - 8) >> 2, ((N) - 8) & 3);       \
        }                                                                                   \
        else if constexpr((N) < 28)                                                         \
        {                                                                                   \
            if(fast_ || ldb_) issue_b((kt) + 4, (N) - 24);                                  \
        }                                                                                   \
        else                                                                                \
        {                                                                                   \
            if(fast_ || lda_) issue_a(ass_, (1 - (Q)) * 4 + (N) - 28);                      \
        }                                                                                   \
    } while(0)
#define ROW(kt, Q, I)                                                                       \
    do                                                                                      \
    {                                                                                       \
        SB(); MF(Q, I, 0); SB(); OTHER(kt, Q, 8 * (I) + 0); SB(); OTHER(kt, Q, 8 * (I) + 1);  \
        SB(); MF(Q, I, 1); SB(); OTHER(kt, Q, 8 * (I) + 2); SB(); OTHER(kt, Q, 8 * (I) + 3);  \
        SB(); MF(Q, I, 2); SB(); OTHER(kt, Q, 8 * (I) + 4); SB(); OTHER(kt, Q, 8 * (I) + 5);  \
        SB(); MF(Q, I, 3); SB(); OTHER(kt, Q, 8 * (I) + 6); SB(); OTHER(kt, Q, 8 * (I) + 7);  \
    } while(0)
#define WAIT_SLAB(kt)                                                                       \
    do                                                                                      \
    {                                                                                       \
        const int cnt_ = issued_in((kt) - 2) + issued_in((kt) - 1);                          \
        if(cnt_ >= 16)      wait_vmcnt<16>();                                               \
        else if(cnt_ >= 12) wait_vmcnt<12>();                                               \
        else if(cnt_ >= 8)  wait_vmcnt<8>();                                                \
        else if(cnt_ >= 4)  wait_vmcnt<4>();                                                \
        else                wait_vmcnt<0>();                                                \
    } while(0)
#define SLAB(kt, Q, FAST)                                                                   \
    do                                                                                      \
    {                                                                                       \
        constexpr bool fast_ = (FAST);                                                      \
        const int kt_     = (kt);                                                           \
        const bool more_  = kt_ + 1 < nk;                                                   \
        const bool ldb_   = issues_b(kt_);                                                  \
        const bool lda_   = issues_a(kt_);                                                  \
        const int ass_    = a_step_of(kt_);                                                 \
        (void)more_; (void)ldb_; (void)lda_;                                                \
        WAIT_FRAGS(Q);                                                                      \
        if constexpr(fast_)                                                                 \
            wait_vmcnt<16>();                                                               \
        else if(more_)                                                                      \
            WAIT_SLAB(kt_);                                                                 \
        block_barrier();                                                                    \
        ROW(kt_, Q, 0); ROW(kt_, Q, 1); ROW(kt_, Q, 2); ROW(kt_, Q, 3);                     \
        SB();                                                                               \
    } while(0)

    // ---- the steady state in trips of twelve slabs, as in qgemm_w4_i8_kernel: LDS addresses that
    // are a fixed register plus an immediate, loads from a scalar base plus the lane's offset with
    // their LDS destination (M0) an immediate away from the wave's base.  The 24 fragment reads
    // follow the first eight MFMAs of a slab (three each), the eight loads the last eight.
    uint32_t a_vaddr[2][2][2]; // [slab parity][half of the lane's 32 bytes][0: stages 0 and 1, 1: stage 2]
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int x = 0; x < 2; x++)
        {
            a_vaddr[h][x][0] = lds0 + a_lane[h][x];
            a_vaddr[h][x][1] = lds0 + a_lane[h][x] + 2 * A2_BYTES;
        }
    uint32_t b_vaddr[4];
#pragma unroll
    for(int j2 = 0; j2 < 4; j2++)
    {
        if constexpr(TRANS_B)
            b_vaddr[j2] = lds0 + b_lane[j2 & 1];
        else
            b_vaddr[j2] = lds0 + b_lane[0] + (uint32_t)(((wave_n * 8 + j2 * 2 + bcol) ^ bsw) << 4);
    }
    const uint32_t wave_lds = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
#define RA12(U1, Q, I, X)                                                                       \
    do                                                                                          \
    {                                                                                           \
        v4i t_;                                                                                 \
        RD128(t_, a_vaddr[(U1) & 1][X][A_STAGE12(U1) == 2 ? 1 : 0],                             \
              (A_STAGE12(U1) == 2 ? 0 : A_STAGE12(U1) * A2_BYTES) + (I) * 32 * 2 * BK);         \
        PUT4(fa[Q][I], X, t_);                                                                  \
    } while(0)
#define RB12(U1, Q, J, R)                                                                       \
    do                                                                                          \
    {                                                                                           \
        if constexpr(TRANS_B)                                                                   \
        {                                                                                       \
            v4i t_;                                                                             \
            RD128(t_, b_vaddr[(R) & 1], ((U1) & (STAGES - 1)) * B_BYTES + (J) * 32 * BK);       \
            PUT4(fb[Q][J], (R) & 1, t_);                                                        \
        }                                                                                       \
        else                                                                                    \
        {                                                                                       \
            v2i t_;                                                                             \
            RDTR8(t_, b_vaddr[J], ((U1) & (STAGES - 1)) * B_BYTES + (R) * 8 * BN);              \
            fb[Q][J][2 * (R) + 0] = t_.x;                                                       \
            fb[Q][J][2 * (R) + 1] = t_.y;                                                       \
        }                                                                                       \
    } while(0)
    // read N of a slab: 0..7 the halves of the A tiles, then the parts of the B tiles (16 for
    // row-major B, 8 for K-contiguous B)
#define READ12(U, Q, N)                                                                         \
    do                                                                                          \
    {                                                                                           \
        if constexpr((N) < 8)                                                                   \
            RA12((U) + 1, 1 - (Q), (N) >> 1, (N) & 1);                                          \
        else if constexpr(!TRANS_B)                                                             \
            RB12((U) + 1, 1 - (Q), ((N) - 8) >> 2, ((N) - 8) & 3);                              \
        else if constexpr((N) < 16)                                                             \
            RB12((U) + 1, 1 - (Q), ((N) - 8) >> 1, ((N) - 8) & 1);                              \
    } while(0)
#define MF12(Q, I, J)                                                                           \
    asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0"                                    \
                 : "+a"(acc[I][J])                                                              \
                 : "v"(fb[Q][J]), "v"(fa[Q][I]))
#define ROW12_READS(U, Q, I, N0)                                                                \
    do                                                                                          \
    {                                                                                           \
        SB(); MF12(Q, I, 0); SB(); READ12(U, Q, (N0) + 0); READ12(U, Q, (N0) + 1); READ12(U, Q, (N0) + 2);   \
        SB(); MF12(Q, I, 1); SB(); READ12(U, Q, (N0) + 3); READ12(U, Q, (N0) + 4); READ12(U, Q, (N0) + 5);   \
        SB(); MF12(Q, I, 2); SB(); READ12(U, Q, (N0) + 6); READ12(U, Q, (N0) + 7); READ12(U, Q, (N0) + 8);   \
        SB(); MF12(Q, I, 3); SB(); READ12(U, Q, (N0) + 9); READ12(U, Q, (N0) + 10); READ12(U, Q, (N0) + 11); \
    } while(0)
    // a row of four MFMAs with a load behind each; M0 (the load's LDS destination) is written
    // ahead of the MFMA, which is the wait state between the two
#define MF4_LOAD4(Q, I, LDS_CONST, OFF0, OFF1, OFF2, OFF3, BASE)                                \
    asm volatile("s_add_i32 m0, %[wl], %[lc0]\n\t"                                              \
                 "v_mfma_f32_32x32x64_f8f6f4 %[c0], %[b0], %[a], %[c0]\n\t"                     \
                 "global_load_lds_dwordx4 %[o0], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc1]\n\t"                                              \
                 "v_mfma_f32_32x32x64_f8f6f4 %[c1], %[b1], %[a], %[c1]\n\t"                     \
                 "global_load_lds_dwordx4 %[o1], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc2]\n\t"                                              \
                 "v_mfma_f32_32x32x64_f8f6f4 %[c2], %[b2], %[a], %[c2]\n\t"                     \
                 "global_load_lds_dwordx4 %[o2], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc3]\n\t"                                              \
                 "v_mfma_f32_32x32x64_f8f6f4 %[c3], %[b3], %[a], %[c3]\n\t"                     \
                 "global_load_lds_dwordx4 %[o3], %[base]"                                       \
                 : [c0] "+a"(acc[I][0]), [c1] "+a"(acc[I][1]), [c2] "+a"(acc[I][2]),            \
                   [c3] "+a"(acc[I][3])                                                         \
                 : [b0] "v"(fb[Q][0]), [b1] "v"(fb[Q][1]), [b2] "v"(fb[Q][2]),                  \
                   [b3] "v"(fb[Q][3]), [a] "v"(fa[Q][I]), [wl] "s"(wave_lds),                   \
                   [lc0] "n"((LDS_CONST) + 0 * 4096), [lc1] "n"((LDS_CONST) + 1 * 4096),        \
                   [lc2] "n"((LDS_CONST) + 2 * 4096), [lc3] "n"((LDS_CONST) + 3 * 4096),        \
                   [o0] "v"(OFF0), [o1] "v"(OFF1), [o2] "v"(OFF2), [o3] "v"(OFF3),              \
                   [base] "s"(BASE)                                                             \
                 : "memory", "scc")
#define SLAB12(U)                                                                               \
    do                                                                                          \
    {                                                                                           \
        constexpr int q_ = (U) & 1;                                                             \
        asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)"                                           \
                     : "+v"(fa[q_][0]), "+v"(fa[q_][1]), "+v"(fa[q_][2]), "+v"(fa[q_][3]),      \
                       "+v"(fb[q_][0]), "+v"(fb[q_][1]), "+v"(fb[q_][2]), "+v"(fb[q_][3])::"memory"); \
        block_barrier();                                                                        \
        ROW12_READS(U, q_, 0, 0);                                                               \
        ROW12_READS(U, q_, 1, 12);                                                              \
        SB();                                                                                   \
        MF4_LOAD4(q_, 2, W4_B_BASE + (((U) + 4) & (STAGES - 1)) * B_BYTES,                      \
                  b_off[0], b_off[1], b_off[2], b_off[3], b_ptr);                               \
        MF4_LOAD4(q_, 3, A_LOAD_STAGE12(U) * A2_BYTES + A_LOAD_BLOCK12(U) * 4096,               \
                  a_off[A_LOAD_BLOCK12(U) + 0], a_off[A_LOAD_BLOCK12(U) + 1],                   \
                  a_off[A_LOAD_BLOCK12(U) + 2], a_off[A_LOAD_BLOCK12(U) + 3], a_ptr);           \
        SB();                                                                                   \
        b_ptr += b_step;                                                                        \
        if constexpr(((U) & 1) == 0)                                                            \
            a_ptr += 2 * BK;                                                                    \
    } while(0)

    // ---- main loop: the schedule of qgemm_w4_i8_kernel ------------------------------------------
#pragma unroll
    for(int h = 0; h < 8; h++)
        issue_a(0, h);
#pragma unroll
    for(int kt = -4; kt < 0; kt++)
    {
        if(issues_b(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_b(kt + 4, h);
        }
        if(issues_a(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_a(a_step_of(kt), ((kt & 1) != 0 ? 0 : 4) + h);
        }
    }
    {
        const int cnt = issued_in(-3) + issued_in(-2) + issued_in(-1);
        if(cnt >= 24)      wait_vmcnt<24>();
        else if(cnt == 20) wait_vmcnt<20>();
        else if(cnt == 16) wait_vmcnt<16>();
        else if(cnt == 12) wait_vmcnt<12>();
        else if(cnt == 8)  wait_vmcnt<8>();
        else if(cnt == 4)  wait_vmcnt<4>();
        else               wait_vmcnt<0>();
    }
    block_barrier();
#pragma unroll
    for(int i = 0; i < 4; i++)
    {
        RA(0, 0, i, 0);
        RA(0, 0, i, 1);
    }
#pragma unroll
    for(int j = 0; j < 4; j++)
    {
        RB(0, 0, j, 0);
        RB(0, 0, j, 1);
        RB(0, 0, j, 2);
        RB(0, 0, j, 3);
    }
    int kt = 0;
    if(nk > 17)
    {
        // b_ptr: slab kt + 4 of B; a_ptr: K step a_step_of(kt) of A; both for the slab about to run
        const int64_t b_step = TRANS_B ? (int64_t)BK : (int64_t)BK * p.ldb;
        const uint8_t* b_ptr = gb + 4 * b_step;
        const uint8_t* a_ptr = ga + 2 * (2 * BK);
        uint32_t m0_saved;
        asm volatile("s_mov_b32 %0, m0" : "=s"(m0_saved));
        W4_TRIPS_OF_TWELVE(kt, nk, SLAB12);
        asm volatile("s_mov_b32 m0, %0" ::"s"(m0_saved));
    }
    for(; kt + 6 < nk; kt += 2)
    {
        SLAB(kt, 0, true);
        SLAB(kt + 1, 1, true);
    }
    // The second half of the accumulators was written last: it passes through a statement that
    // holds the wait states before anything the compiler places here can read it.  The first half
    // is at least eight MFMAs old.
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3"
                 : "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]),
                   "+a"(acc[3][0]), "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3]));
    for(; kt + 1 < nk; kt += 2)
    {
        SLAB(kt, 0, false);
        SLAB(kt + 1, 1, false);
    }
    if(kt < nk)
        SLAB(kt, 0, false);
#undef SLAB12
#undef MF4_LOAD4
#undef ROW12_READS
#undef MF12
#undef READ12
#undef RB12
#undef RA12
#undef SLAB
#undef WAIT_SLAB
#undef ROW
#undef OTHER
#undef MF
#undef WAIT_FRAGS
#undef RB
#undef RA
#undef PUT4
#undef SB
#undef RDTR8
#undef RD128

    // ---- epilogue: the fp8 part of qgemm_dma_kernel's, 4 x 4 tiles per wave ---------------------
    // Element e of lane l belongs to row l % 32 of the A tile and column 8*(e/4) + 4*(l/32) + e%4
    // of the B tile: four groups of 4 consecutive columns, each written with one store.  One block
    // of 32 columns at a time; its scales and biases are loaded ahead of the stores of the block
    // before it (a load issued behind a store waits for it), and no more than two blocks' worth is
    // held in registers.
    float sa_r[4] = {1.f, 1.f, 1.f, 1.f};
    if constexpr(DEQ)
    {
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            const int row = min(m0 + wave_m * 128 + i * 32 + lrow, p.m - 1);
            if(p.scale_a_mode == MI355_QP_PER_TENSOR)
                sa_r[i] = p.scale_a[0];
            else if(p.scale_a_mode == MI355_QP_PER_ROW)
                sa_r[i] = p.scale_a[row];
        }
    }
    if constexpr(!DEQ)
    {
        {
            // The bare result through the LDS, as in qgemm_w4_i8_kernel: straight from the
            // accumulators a store instruction writes 32 bytes of each of 32 rows, from a row-major
            // copy in the LDS the 512 bytes of two whole rows of the wave's quadrant.
            block_barrier();
            constexpr int PITCH = 512 + 16;
            uint8_t* mine       = lds + wave * 40960;
            const int out_col   = n0 + wave_n * 128 + 4 * (lane & 31);
            float* out_base     = static_cast<float*>(p.c) + (int64_t)blockIdx.y * p.stride_c + out_col;
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                uint8_t* buf = mine + (i & 1) * (32 * PITCH);
#pragma unroll
                for(int j = 0; j < 4; j++)
#pragma unroll
                    for(int g = 0; g < 4; g++)
                        *reinterpret_cast<v4f*>(buf + lrow * PITCH + (32 * j + 8 * g + 4 * lgrp) * 4) =
                            v4f{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
                // (every read before the first store, see qgemm_w4_i8_kernel)
                v4f val[16];
#pragma unroll
                for(int t = 0; t < 16; t++)
                    val[t] = *reinterpret_cast<const v4f*>(buf + (2 * t + (lane >> 5)) * PITCH + (lane & 31) * 16);
#pragma unroll
                for(int t = 0; t < 16; t++)
                    asm volatile("" : "+v"(val[t]));
#pragma unroll
                for(int t = 0; t < 16; t++)
                {
                    const int row = m0 + wave_m * 128 + 32 * i + 2 * t + (lane >> 5);
                    if(row < p.m && out_col < p.n)
                        store_rows(reinterpret_cast<v4f*>(out_base + (int64_t)row * p.ldc), val[t], p.stream_c);
                }
            }
            return;
        }
    }
    float sb_c[4][4], bias_c[4][4], sb_next[4][4], bias_next[4][4];
    auto load_block = [&](int j, float (&sb_o)[4][4], float (&bias_o)[4][4]) {
#pragma unroll
        for(int g = 0; g < 4; g++)
        {
            const int c0 = n0 + wave_n * 128 + j * 32 + 8 * g + 4 * lgrp;
            if(p.vec_cols)
            {
                // N % 4 == 0: a group that starts inside N lies inside it
                const int cv = min(c0, p.n - 4);
                v4f sb4      = {1.f, 1.f, 1.f, 1.f};
                v4f bi4      = {-0.0f, -0.0f, -0.0f, -0.0f};
                if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                    sb4 = v4f{p.scale_b[0], p.scale_b[0], p.scale_b[0], p.scale_b[0]};
                else if(p.scale_b_mode == MI355_QP_PER_COL)
                    sb4 = *reinterpret_cast<const v4f*>(p.scale_b + cv);
                if(p.bias != nullptr)
                    bi4 = *reinterpret_cast<const v4f*>(p.bias + cv);
#pragma unroll
                for(int e = 0; e < 4; e++)
                {
                    sb_o[g][e]   = sb4[e];
                    bias_o[g][e] = bi4[e];
                }
                continue;
            }
#pragma unroll
            for(int e = 0; e < 4; e++)
            {
                const int c = min(c0 + e, p.n - 1);
                float sb    = 1.f;
                if(p.scale_b_mode == MI355_QP_PER_TENSOR)
                    sb = p.scale_b[0];
                else if(p.scale_b_mode == MI355_QP_PER_COL)
                    sb = p.scale_b[c];
                sb_o[g][e]   = sb;
                bias_o[g][e] = p.bias != nullptr ? p.bias[c] : -0.0f;
            }
        }
    };
    if constexpr(DEQ)
        load_block(0, sb_c, bias_c);
    // fp32 outputs, and 16-bit ones in whole groups of 8: through the LDS like the bare result.  The
    // wave's copy holds 256 bytes of each of its 128 rows: all 128 columns of a 16-bit type, or half
    // of them in fp32 (two rounds); an instruction then stores 256 contiguous bytes of 4 rows.
    if constexpr(DEQ && (OUT == MI355_F32 || VEC8))
    {
        block_barrier();
        constexpr int ROWB = 256 + 16;               // rows start 4 banks apart
        constexpr int ESZ  = OUT == MI355_F32 ? 4 : 2;
        constexpr int JP   = OUT == MI355_F32 ? 2 : 4; // 32-column blocks per round
        uint8_t* mine      = lds + wave * 40960;
#pragma unroll
        for(int round = 0; round < 4 / JP; round++)
        {
#pragma unroll
            for(int jj = 0; jj < JP; jj++)
            {
                const int j = round * JP + jj;
                if(j + 1 < 4)
                    load_block(j + 1, sb_next, bias_next);
#pragma unroll
                for(int i = 0; i < 4; i++)
                {
                    const float sa = sa_r[i];
#pragma unroll
                    for(int g = 0; g < 4; g++)
                    {
                        float v[4];
#pragma unroll
                        for(int e = 0; e < 4; e++)
                            // the accumulator is a float: double(acc) * double(s) rounded once to
                            // float is exactly the correctly rounded fp32 product
                            v[e] = add_bias(acc[i][j][4 * g + e] * (sa * sb_c[g][e]), bias_c[g][e]);
                        uint8_t* dst = mine + (32 * i + lrow) * ROWB + (32 * jj + 8 * g + 4 * lgrp) * ESZ;
                        if constexpr(OUT == MI355_F32)
                            *reinterpret_cast<v4f*>(dst) = v4f{v[0], v[1], v[2], v[3]};
                        else
                            *reinterpret_cast<uint2*>(dst) =
                                make_uint2(pack16<OUT>(v[0], v[1]), pack16<OUT>(v[2], v[3]));
                    }
                }
                if(j + 1 < 4)
                {
#pragma unroll
                    for(int g = 0; g < 4; g++)
#pragma unroll
                        for(int e = 0; e < 4; e++)
                        {
                            sb_c[g][e]   = sb_next[g][e];
                            bias_c[g][e] = bias_next[g][e];
                        }
                }
            }
            __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
            const int col = n0 + wave_n * 128 + round * (JP * 32) + (lane & 15) * (16 / ESZ);
#pragma unroll
            for(int t8 = 0; t8 < 32; t8 += 8)
            {
                // eight reads before their eight stores (see the bare result above)
                v4u val[8];
#pragma unroll
                for(int t = 0; t < 8; t++)
                    val[t] = *reinterpret_cast<const v4u*>(mine + (4 * (t8 + t) + (lane >> 4)) * ROWB + (lane & 15) * 16);
#pragma unroll
                for(int t = 0; t < 8; t++)
                    asm volatile("" : "+v"(val[t]));
#pragma unroll
                for(int t = 0; t < 8; t++)
                {
                    const int row = m0 + wave_m * 128 + 4 * (t8 + t) + (lane >> 4);
                    if(row < p.m && col < p.n)
                        store_rows(reinterpret_cast<v4u*>(static_cast<uint8_t*>(p.c) +
                                                       ((int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col) * ESZ),
                                val[t], p.stream_c);
                }
            }
        }
        return;
    }
#pragma unroll
    for(int j = 0; j < 4; j++)
    {
        if constexpr(DEQ)
        {
            if(j + 1 < 4)
                load_block(j + 1, sb_next, bias_next);
        }
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            const int row = m0 + wave_m * 128 + i * 32 + lrow;
            if(row >= p.m)
                continue;
            const float sa = sa_r[i];
            // 16-bit outputs: lanes l and l + 32 hold the two halves of the same 8 columns, for two
            // column groups; one v_permlane32_swap per register gives each of them one whole group,
            // which goes out as a single 16-byte store.  N % 8 == 0 there, so the two lanes are in
            // or out of the matrix together (and they share their row).
            if constexpr(VEC8)
            {
                static_assert(!VEC8 || (DEQ && (OUT == MI355_F16 || OUT == MI355_BF16)), "16-bit outputs only");
#pragma unroll
                for(int gp = 0; gp < 4; gp += 2)
                {
                    uint32_t pk[2][2];
#pragma unroll
                    for(int h = 0; h < 2; h++)
                    {
                        float q[4];
#pragma unroll
                        for(int e = 0; e < 4; e++)
                        {
                            float v = acc[i][j][4 * (gp + h) + e] * (sa * sb_c[gp + h][e]);
                            v       = add_bias(v, bias_c[gp + h][e]);
                            q[e]    = v;
                        }
                        pk[h][0] = pack16<OUT>(q[0], q[1]);
                        pk[h][1] = pack16<OUT>(q[2], q[3]);
                    }
                    const auto r0 = __builtin_amdgcn_permlane32_swap(pk[0][0], pk[1][0], false, false);
                    const auto r1 = __builtin_amdgcn_permlane32_swap(pk[0][1], pk[1][1], false, false);
                    const int col = n0 + wave_n * 128 + j * 32 + 8 * (gp + lgrp);
                    if(col < p.n)
                    {
                        const int64_t idx = (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
                        store_c(reinterpret_cast<v4u*>(static_cast<uint16_t*>(p.c) + idx),
                                v4u{r0[0], r1[0], r0[1], r1[1]}, p.stream_c);
                    }
                }
            }
            else
            {
#pragma unroll
                for(int g = 0; g < 4; g++)
                {
                    const int col = n0 + wave_n * 128 + j * 32 + 8 * g + 4 * lgrp;
                    if(col >= p.n)
                        continue;
                    const int64_t idx = (int64_t)blockIdx.y * p.stride_c + (int64_t)row * p.ldc + col;
                    float v[4];
#pragma unroll
                    for(int e = 0; e < 4; e++)
                    {
                        v[e] = acc[i][j][4 * g + e];
                        if constexpr(DEQ)
                            // the accumulator is a float: double(acc) * double(s) rounded once to float
                            // is exactly the correctly rounded fp32 product
                            v[e] = add_bias(v[e] * (sa * sb_c[g][e]), bias_c[g][e]);
                    }
                    if constexpr(!DEQ || OUT == MI355_F32)
                        store_c(reinterpret_cast<v4f*>(static_cast<float*>(p.c) + idx), v4f{v[0], v[1], v[2], v[3]},
                                p.stream_c);
                    else if constexpr(OUT == MI355_F16)
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16),
                            convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16));
                    else
                        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p.c) + idx) = make_uint2(
                            convert_f32_to_bf16x2(v[0], v[1]),
                            convert_f32_to_bf16x2(v[2], v[3]));
                }
            }
        }
        if constexpr(DEQ)
        {
            if(j + 1 < 4)
            {
#pragma unroll
                for(int g = 0; g < 4; g++)
#pragma unroll
                    for(int e = 0; e < 4; e++)
                    {
                        sb_c[g][e]   = sb_next[g][e];
                        bias_c[g][e] = bias_next[g][e];
                    }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Block-scaled packed fp4 x fp4 on the four-wave plan (qgemm_w4_f8_kernel's loads, LDS stages and
// schedule; B is [N, K / 2], the result bare fp32 through the LDS copy).  A 64-byte slab of a row
// is 128 codes in four blocks of 32: lane group g of a 32-row operand tile holds blocks 2 g and
// 2 g + 1 (two 16-byte chunks), and a tile pair takes two v_mfma_scale_f32_32x32x64_f8f6f4 (8 passes
// each, cbsz = blgp = 4), the first over blocks {0, 2}, the second over {1, 3}.  The exponent
// bytes do not pass through the LDS (it is full): every lane loads the word of its row and slab
// -- [slab][row][4 blocks], see dma_params::mx_ea -- two slabs ahead, for its four A and four B
// tiles, shifts it so that bytes 0 and 1 are its group's two blocks, and op_sel picks the byte.
__global__ __launch_bounds__(W4_THREADS) void qgemm_w4_mx4_kernel(dma_params p)
{
    constexpr bool TRANS_B = true;
    constexpr bool DEQ     = false;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    if(*p.mx_flag == p.mx_ticket)
        return;

    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 1; // 0..1
    const int wave_n = wave & 1;  // 0..1

    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const uint8_t* __restrict__ ga = p.a + (int64_t)blockIdx.y * p.stride_a;
    const uint8_t* __restrict__ gb = p.b + (int64_t)blockIdx.y * p.stride_b;
    const int nk = p.k / BK;

    // ---- global -> LDS: exactly as in qgemm_w4_i8_kernel -------------------------------------
    uint32_t a_off[8], b_off[4];
    const int a_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
#pragma unroll
    for(int h = 0; h < 8; h++)
    {
        const int r   = 8 * (wave + 4 * h) + (lane >> 3);
        const int row = min(m0 + r, p.m - 1);
        a_off[h]      = (uint32_t)row * (uint32_t)p.lda + a_chunk * 16;
    }
    const uint32_t a_tail_back = a_chunk >= 4 ? 64u : 0u;
#pragma unroll
    for(int h = 0; h < 4; h++)
    {
        const int blk = wave + 4 * h;
        if constexpr(TRANS_B)
        {
            const int r     = 16 * blk + (lane >> 2);
            const int chunk = (lane & 3) ^ ((r >> 2) & 3);
            const int col   = min(n0 + r, p.n - 1);
            b_off[h]        = (uint32_t)col * (uint32_t)p.ldb + chunk * 16;
        }
        else
        {
            const int k     = 4 * blk + (lane >> 4);
            const int chunk = (lane & 15) ^ (k & 7);
            const int col   = min(n0 + chunk * 16, p.n - 16);
            b_off[h]        = (uint32_t)k * (uint32_t)p.ldb + col;
        }
    }
    auto issue_a = [&](int ss, int h) {
        uint8_t* st           = lds + (ss % W4_A_STAGES) * A2_BYTES;
        const uint8_t* a_base = ga + (int64_t)ss * (2 * BK);
        const uint32_t back   = 2 * ss + 1 < nk ? 0u : a_tail_back;
        load_to_lds(a_base + (a_off[h] - back), st + (wave + 4 * h) * 1024);
    };
    auto issue_b = [&](int kt, int h) {
        uint8_t* st           = lds + W4_B_BASE + (kt & (STAGES - 1)) * B_BYTES;
        const uint8_t* b_base = TRANS_B ? gb + (int64_t)kt * BK : gb + (int64_t)kt * BK * p.ldb;
        load_to_lds(b_base + b_off[h], st + (wave + 4 * h) * 1024);
    };
    auto a_step_of   = [](int kt) { return (kt & 1) != 0 ? (kt + 5) / 2 : (kt + 4) / 2; };
    auto issues_b    = [&](int kt) { return kt + 4 >= 0 && kt + 4 < nk; };
    auto issues_a    = [&](int kt) { const int ss = a_step_of(kt); return ss >= 1 && 2 * ss < nk; };
    auto issued_in   = [&](int kt) { return (issues_b(kt) ? 4 : 0) + (issues_a(kt) ? 4 : 0); };

    // ---- LDS -> operand fragments -------------------------------------------------------------
    const int lrow      = lane & 31;
    const int lgrp      = lane >> 5;
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    // A: rows of 128 bytes (two slabs); slab parity h, chunk x of this lane's 32 bytes is logical
    // chunk 4h + 2*lgrp + x at position c ^ ((row >> 1) & 7)
    uint32_t a_lane[2][2];
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int x = 0; x < 2; x++)
            a_lane[h][x] = (wave_m * 128 + lrow) * (2 * BK) + (((4 * h + 2 * lgrp + x) ^ ((lrow >> 1) & 7)) << 4);
    uint32_t b_lane[2];
    {
        const int sw = (lrow >> 2) & 3;
#pragma unroll
        for(int x = 0; x < 2; x++)
            b_lane[x] = W4_B_BASE + (wave_n * 128 + lrow) * BK + (((2 * lgrp + x) ^ sw) << 4);
    }

    v4i fa[2][4][2]; // [register set][tile][chunk of the lane's 32 bytes]
    v4i fb[2][4][2];
    // exponent bytes of the lane's rows (0..3: A tiles, 4..7: B tiles): in flight, one set per slab
    // parity, and the current slab's, shifted so that bytes 0 and 1 are the lane group's two blocks
    int sin[2][8] = {{0, 0, 0, 0, 0, 0, 0, 0}, {0, 0, 0, 0, 0, 0, 0, 0}};
    int sc[8]     = {0, 0, 0, 0, 0, 0, 0, 0};
    const int sc_shift = 16 * lgrp;
    const uint8_t* sa_ptr = p.mx_ea + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_a * 4 +
                            (int64_t)(m0 + wave_m * 128 + lrow) * 4;
    const uint8_t* sb_ptr = p.mx_eb + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_b * 4 +
                            (int64_t)(n0 + wave_n * 128 + lrow) * 4;
    const int64_t sa_step = (int64_t)p.mx_rows_a * 4, sb_step = (int64_t)p.mx_rows_b * 4;
    v16f acc[4][4];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
#pragma unroll
            for(int e = 0; e < 16; e++)
                acc[i][j][e] = 0.f;

#define RD128(dst, addr, imm) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define RDTR8(dst, addr, imm) \
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define SB() __builtin_amdgcn_sched_barrier(0)
    // the 8 exponent words of slab s -> sin[Q]; inline assembly keeps them out of the compiler's own
    // count of outstanding loads (it would wait for the direct-to-LDS loads with them)
#define LDS1(dst, ptr, imm) \
    asm volatile("global_load_dword %0, %1, off offset:%2" : "=v"(dst) : "v"(ptr), "n"(imm) : "memory")
#define LOAD_SCALES(s, Q)                                                   \
    do                                                                      \
    {                                                                       \
        const int s_          = min((s), nk - 1);                           \
        const uint8_t* pa_    = sa_ptr + (int64_t)s_ * sa_step;             \
        const uint8_t* pb_    = sb_ptr + (int64_t)s_ * sb_step;             \
        LDS1(sin[Q][0], pa_, 0);   LDS1(sin[Q][1], pa_, 128);               \
        LDS1(sin[Q][2], pa_, 256); LDS1(sin[Q][3], pa_, 384);               \
        LDS1(sin[Q][4], pb_, 0);   LDS1(sin[Q][5], pb_, 128);               \
        LDS1(sin[Q][6], pb_, 256); LDS1(sin[Q][7], pb_, 384);               \
    } while(0)
    // half X of A tile I of slab kt -> fa[Q][I]
#define RA(kt, Q, I, X)                                                                         \
    do                                                                                          \
    {                                                                                           \
        RD128(fa[Q][I][X], lds0 + (((kt) >> 1) % W4_A_STAGES) * A2_BYTES + a_lane[(kt) & 1][X], \
              (I) * 32 * 2 * BK);                                                               \
    } while(0)
    // part R of B tile J of slab kt: row-major B four transposing reads, K-contiguous B two
#define RB(kt, Q, J, R)                                                                         \
    do                                                                                          \
    {                                                                                           \
        const uint32_t s_ = lds0 + ((kt) & (STAGES - 1)) * B_BYTES;                             \
        if constexpr(TRANS_B)                                                                   \
        {                                                                                       \
            if((R) < 2)                                                                         \
            {                                                                                   \
                RD128(fb[Q][J][(R) & 1], s_ + b_lane[(R) & 1], (J) * 32 * BK);                  \
            }                                                                                   \
        }                                                                                       \
        else                                                                                    \
        {                                                                                       \
            (void)s_;                                                                           \
        }                                                                                       \
    } while(0)
#define WAIT_FRAGS(Q)                                                                           \
    asm volatile("s_waitcnt lgkmcnt(0)"                                                         \
                 : "+v"(fa[Q][0][0]), "+v"(fa[Q][1][0]), "+v"(fa[Q][2][0]), "+v"(fa[Q][3][0]),  \
                   "+v"(fa[Q][0][1]), "+v"(fa[Q][1][1]), "+v"(fa[Q][2][1]), "+v"(fa[Q][3][1]),  \
                   "+v"(fb[Q][0][0]), "+v"(fb[Q][1][0]), "+v"(fb[Q][2][0]), "+v"(fb[Q][3][0]),  \
                   "+v"(fb[Q][0][1]), "+v"(fb[Q][1][1]), "+v"(fb[Q][2][1]), "+v"(fb[Q][3][1])::"memory")
    // The B tile goes in first: the accumulator then holds the tile transposed and a lane owns runs
    // of four consecutive columns of C (see the epilogue).  Assembly for the reason given in
    // qgemm_w4_i8_kernel.  The compiler does not know that the statement is an MFMA and adds none
    // of the wait states a 16-pass MFMA needs before its result may be read.  In the steady-state
    // loop nothing reads an accumulator.  In the last slabs, whose loads and reads are conditional,
    // the compiler keeps copies of the accumulators in scratch memory and stores them right behind
    // the MFMA, so there the statement carries the wait states itself.
    // X: which of the lane's two chunks (K blocks 2 g + X of lane group g; the scale bytes follow
    // through op_sel).  8 passes each; the two MFMAs of a tile are four instructions apart.
#define MF(Q, I, J, X)                                                                         \
    do                                                                                         \
    {                                                                                          \
        if constexpr((X) == 0 && fast_)                                                        \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 "            \
                         "op_sel_hi:[0,0,0] cbsz:4 blgp:4"                                     \
                         : "+a"(acc[I][J])                                                     \
                         : "v"(fb[Q][J][0]), "v"(fa[Q][I][0]), "v"(sc[4 + (J)]), "v"(sc[I]));  \
        else if constexpr((X) == 0)                                                            \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 "            \
                         "op_sel_hi:[0,0,0] cbsz:4 blgp:4\n\ts_nop 7\n\ts_nop 3"              \
                         : "+a"(acc[I][J])                                                     \
                         : "v"(fb[Q][J][0]), "v"(fa[Q][I][0]), "v"(sc[4 + (J)]), "v"(sc[I]));  \
        else if constexpr(fast_)                                                               \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 "            \
                         "op_sel:[1,1,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4"                      \
                         : "+a"(acc[I][J])                                                     \
                         : "v"(fb[Q][J][1]), "v"(fa[Q][I][1]), "v"(sc[4 + (J)]), "v"(sc[I]));  \
        else                                                                                   \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 "            \
                         "op_sel:[1,1,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4\n\ts_nop 7\n\ts_nop 3" \
                         : "+a"(acc[I][J])                                                     \
                         : "v"(fb[Q][J][1]), "v"(fa[Q][I][1]), "v"(sc[4 + (J)]), "v"(sc[I]));  \
    } while(0)
    // slot N of 32: 0..7 A reads, 8..23 B reads (8..15 when B is K-contiguous), 24..31 loads.
#define OTHER(kt, Q, N)                                                                     \
    do                                                                                      \
    {                                                                                       \
        if constexpr((N) < 8)                                                               \
        {                                                                                   \
            if(fast_ || more_) RA((kt) + 1, 1 - (Q), (N) >> 1, (N) & 1);                   \
        }                                                                                   \
        else if constexpr((N) < 24)                                                         \
        {                                                                                   \
            if(fast_ || more_) RB((kt) + 1, 1 - (Q), ((N) - 8) >> 2, ((N) - 8) & 3);       \
        }                                                                                   \
        else if constexpr((N) < 28)                                                         \
        {                                                                                   \
            if(fast_ || ldb_) issue_b((kt) + 4, (N) - 24);                                  \
        }                                                                                   \
        else                                                                                \
        {                                                                                   \
            if(fast_ || lda_) issue_a(ass_, (1 - (Q)) * 4 + (N) - 28);                      \
        }                                                                                   \
    } while(0)
#define ROW(kt, Q, I)                                                                       \
    do                                                                                      \
    {                                                                                       \
        SB(); MF(Q, I, 0, 0); SB(); OTHER(kt, Q, 8 * (I) + 0);                              \
        SB(); MF(Q, I, 1, 0); SB(); OTHER(kt, Q, 8 * (I) + 1);                              \
        SB(); MF(Q, I, 2, 0); SB(); OTHER(kt, Q, 8 * (I) + 2);                              \
        SB(); MF(Q, I, 3, 0); SB(); OTHER(kt, Q, 8 * (I) + 3);                              \
        SB(); MF(Q, I, 0, 1); SB(); OTHER(kt, Q, 8 * (I) + 4);                              \
        SB(); MF(Q, I, 1, 1); SB(); OTHER(kt, Q, 8 * (I) + 5);                              \
        SB(); MF(Q, I, 2, 1); SB(); OTHER(kt, Q, 8 * (I) + 6);                              \
        SB(); MF(Q, I, 3, 1); SB(); OTHER(kt, Q, 8 * (I) + 7);                              \
    } while(0)
#define WAIT_SLAB(kt)                                                                       \
    do                                                                                      \
    {                                                                                       \
        const int cnt_ = issued_in((kt) - 2) + issued_in((kt) - 1) + 8;                      \
        if(cnt_ >= 24)      wait_vmcnt<24>();                                               \
        else if(cnt_ >= 20) wait_vmcnt<20>();                                               \
        else if(cnt_ >= 16) wait_vmcnt<16>();                                               \
        else if(cnt_ >= 12) wait_vmcnt<12>();                                               \
        else                wait_vmcnt<8>();                                                \
    } while(0)
#define SLAB(kt, Q, FAST)                                                                   \
    do                                                                                      \
    {                                                                                       \
        constexpr bool fast_ = (FAST);                                                      \
        const int kt_     = (kt);                                                           \
        const bool more_  = kt_ + 1 < nk;                                                   \
        const bool ldb_   = issues_b(kt_);                                                  \
        const bool lda_   = issues_a(kt_);                                                  \
        const int ass_    = a_step_of(kt_);                                                 \
        (void)more_; (void)ldb_; (void)lda_;                                                \
        WAIT_FRAGS(Q);                                                                      \
        /* pending, oldest first: this slab's scale words, the loads of slab kt - 2, the next   \
           slab's scale words, the loads of slab kt - 1: all but the first may stay in flight */ \
        if constexpr(fast_)                                                                 \
            wait_vmcnt<24>();                                                               \
        else                                                                                \
            WAIT_SLAB(kt_);                                                                 \
        block_barrier();                                                                    \
        asm volatile("" : "+v"(sin[Q][0]), "+v"(sin[Q][1]), "+v"(sin[Q][2]), "+v"(sin[Q][3]), \
                          "+v"(sin[Q][4]), "+v"(sin[Q][5]), "+v"(sin[Q][6]), "+v"(sin[Q][7])); \
        _Pragma("unroll") for(int t_ = 0; t_ < 8; t_++) sc[t_] = sin[Q][t_] >> sc_shift;     \
        asm volatile("" : "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]),               \
                          "+v"(sc[4]), "+v"(sc[5]), "+v"(sc[6]), "+v"(sc[7]));               \
        LOAD_SCALES(kt_ + 2, Q);                                                            \
        ROW(kt_, Q, 0); ROW(kt_, Q, 1); ROW(kt_, Q, 2); ROW(kt_, Q, 3);                     \
        SB();                                                                               \
    } while(0)

    // ---- the steady state in trips of twelve slabs, as in qgemm_w4_i8_kernel: LDS addresses that
    // are a fixed register plus an immediate, loads (operands and exponent words) from a scalar base
    // plus the lane's fixed offset.  The 16 fragment reads follow the first 16 of a slab's 32 MFMAs,
    // the eight loads the last eight.
    uint32_t a_vaddr[2][2][2]; // [slab parity][chunk][0: stages 0 and 1, 1: stage 2]
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int x = 0; x < 2; x++)
        {
            a_vaddr[h][x][0] = lds0 + a_lane[h][x];
            a_vaddr[h][x][1] = lds0 + a_lane[h][x] + 2 * A2_BYTES;
        }
    const uint32_t b_vaddr[2] = {lds0 + b_lane[0], lds0 + b_lane[1]};
    const uint32_t wave_lds   = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const uint32_t sa_off     = (uint32_t)(m0 + wave_m * 128 + lrow) * 4u;
    const uint32_t sb_off     = (uint32_t)(n0 + wave_n * 128 + lrow) * 4u;
#define RA12(U1, Q, I, X)                                                                       \
    RD128(fa[Q][I][X], a_vaddr[(U1) & 1][X][A_STAGE12(U1) == 2 ? 1 : 0],                        \
          (A_STAGE12(U1) == 2 ? 0 : A_STAGE12(U1) * A2_BYTES) + (I) * 32 * 2 * BK)
#define RB12(U1, Q, J, R)                                                                       \
    RD128(fb[Q][J][R], b_vaddr[R], ((U1) & (STAGES - 1)) * B_BYTES + (J) * 32 * BK)
#define LDS1S(dst, off, base, imm)                                                              \
    asm volatile("global_load_dword %0, %1, %2 offset:%3"                                       \
                 : "=v"(dst)                                                                    \
                 : "v"(off), "s"(base), "n"(imm)                                                \
                 : "memory")
#define LOAD_SCALES12(Q)                                                                        \
    do                                                                                          \
    {                                                                                           \
        LDS1S(sin[Q][0], sa_off, sa_run, 0);   LDS1S(sin[Q][1], sa_off, sa_run, 128);           \
        LDS1S(sin[Q][2], sa_off, sa_run, 256); LDS1S(sin[Q][3], sa_off, sa_run, 384);           \
        LDS1S(sin[Q][4], sb_off, sb_run, 0);   LDS1S(sin[Q][5], sb_off, sb_run, 128);           \
        LDS1S(sin[Q][6], sb_off, sb_run, 256); LDS1S(sin[Q][7], sb_off, sb_run, 384);           \
    } while(0)
#define MF12(Q, I, J, X)                                                                        \
    do                                                                                          \
    {                                                                                           \
        if constexpr((X) == 0)                                                                  \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 "             \
                         "op_sel_hi:[0,0,0] cbsz:4 blgp:4"                                      \
                         : "+a"(acc[I][J])                                                      \
                         : "v"(fb[Q][J][0]), "v"(fa[Q][I][0]), "v"(sc[4 + (J)]), "v"(sc[I]));   \
        else                                                                                    \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 "             \
                         "op_sel:[1,1,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4"                       \
                         : "+a"(acc[I][J])                                                      \
                         : "v"(fb[Q][J][1]), "v"(fa[Q][I][1]), "v"(sc[4 + (J)]), "v"(sc[I]));   \
    } while(0)
    // a row of eight MFMAs, read N0 + t of the next slab behind MFMA t (0..7 A reads, 8..15 B reads)
#define READ12(U, Q, N)                                                                         \
    do                                                                                          \
    {                                                                                           \
        if constexpr((N) < 8)                                                                   \
            RA12((U) + 1, 1 - (Q), (N) >> 1, (N) & 1);                                          \
        else                                                                                    \
            RB12((U) + 1, 1 - (Q), ((N) - 8) >> 1, ((N) - 8) & 1);                              \
    } while(0)
#define ROW12_READS(U, Q, I, N0)                                                                \
    do                                                                                          \
    {                                                                                           \
        SB(); MF12(Q, I, 0, 0); SB(); READ12(U, Q, (N0) + 0);                                   \
        SB(); MF12(Q, I, 1, 0); SB(); READ12(U, Q, (N0) + 1);                                   \
        SB(); MF12(Q, I, 2, 0); SB(); READ12(U, Q, (N0) + 2);                                   \
        SB(); MF12(Q, I, 3, 0); SB(); READ12(U, Q, (N0) + 3);                                   \
        SB(); MF12(Q, I, 0, 1); SB(); READ12(U, Q, (N0) + 4);                                   \
        SB(); MF12(Q, I, 1, 1); SB(); READ12(U, Q, (N0) + 5);                                   \
        SB(); MF12(Q, I, 2, 1); SB(); READ12(U, Q, (N0) + 6);                                   \
        SB(); MF12(Q, I, 3, 1); SB(); READ12(U, Q, (N0) + 7);                                   \
    } while(0)
#define ROW12_PLAIN(Q, I)                                                                       \
    do                                                                                          \
    {                                                                                           \
        SB(); MF12(Q, I, 0, 0); MF12(Q, I, 1, 0); MF12(Q, I, 2, 0); MF12(Q, I, 3, 0);           \
        MF12(Q, I, 0, 1); MF12(Q, I, 1, 1); MF12(Q, I, 2, 1); MF12(Q, I, 3, 1); SB();           \
    } while(0)
    // four MFMAs (chunk X of the lane's bytes) with a load behind each; M0 (the load's LDS
    // destination) is written ahead of the MFMA, which is the wait state between the two
#define MF4_LOAD4(Q, I, X, SEL, LDS_CONST, OFF0, OFF1, OFF2, OFF3, BASE)                        \
    asm volatile("s_add_i32 m0, %[wl], %[lc0]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c0], %[b0], %[a], %[c0], %[s0], %[sa] " SEL "\n\t" \
                 "global_load_lds_dwordx4 %[o0], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc1]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c1], %[b1], %[a], %[c1], %[s1], %[sa] " SEL "\n\t" \
                 "global_load_lds_dwordx4 %[o1], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc2]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c2], %[b2], %[a], %[c2], %[s2], %[sa] " SEL "\n\t" \
                 "global_load_lds_dwordx4 %[o2], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc3]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c3], %[b3], %[a], %[c3], %[s3], %[sa] " SEL "\n\t" \
                 "global_load_lds_dwordx4 %[o3], %[base]"                                       \
                 : [c0] "+a"(acc[I][0]), [c1] "+a"(acc[I][1]), [c2] "+a"(acc[I][2]),            \
                   [c3] "+a"(acc[I][3])                                                         \
                 : [b0] "v"(fb[Q][0][X]), [b1] "v"(fb[Q][1][X]), [b2] "v"(fb[Q][2][X]),         \
                   [b3] "v"(fb[Q][3][X]), [a] "v"(fa[Q][I][X]), [s0] "v"(sc[4]), [s1] "v"(sc[5]), \
                   [s2] "v"(sc[6]), [s3] "v"(sc[7]), [sa] "v"(sc[I]), [wl] "s"(wave_lds),       \
                   [lc0] "n"((LDS_CONST) + 0 * 4096), [lc1] "n"((LDS_CONST) + 1 * 4096),        \
                   [lc2] "n"((LDS_CONST) + 2 * 4096), [lc3] "n"((LDS_CONST) + 3 * 4096),        \
                   [o0] "v"(OFF0), [o1] "v"(OFF1), [o2] "v"(OFF2), [o3] "v"(OFF3),              \
                   [base] "s"(BASE)                                                             \
                 : "memory", "scc")
#define SLAB12(U)                                                                               \
    do                                                                                          \
    {                                                                                           \
        constexpr int q_ = (U) & 1;                                                             \
        /* may stay in flight: the loads of the last two slabs and the next slab's scale words */ \
        asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)"                                           \
                 : "+v"(fa[q_][0][0]), "+v"(fa[q_][1][0]), "+v"(fa[q_][2][0]), "+v"(fa[q_][3][0]),  \
                   "+v"(fa[q_][0][1]), "+v"(fa[q_][1][1]), "+v"(fa[q_][2][1]), "+v"(fa[q_][3][1]),  \
                   "+v"(fb[q_][0][0]), "+v"(fb[q_][1][0]), "+v"(fb[q_][2][0]), "+v"(fb[q_][3][0]),  \
                   "+v"(fb[q_][0][1]), "+v"(fb[q_][1][1]), "+v"(fb[q_][2][1]), "+v"(fb[q_][3][1])::"memory"); \
        block_barrier();                                                                        \
        asm volatile("" : "+v"(sin[q_][0]), "+v"(sin[q_][1]), "+v"(sin[q_][2]), "+v"(sin[q_][3]), \
                          "+v"(sin[q_][4]), "+v"(sin[q_][5]), "+v"(sin[q_][6]), "+v"(sin[q_][7])); \
        _Pragma("unroll") for(int t_ = 0; t_ < 8; t_++) sc[t_] = sin[q_][t_] >> sc_shift;        \
        asm volatile("" : "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]),                   \
                          "+v"(sc[4]), "+v"(sc[5]), "+v"(sc[6]), "+v"(sc[7]));                   \
        LOAD_SCALES12(q_);                                                                      \
        ROW12_READS(U, q_, 0, 0);                                                               \
        ROW12_READS(U, q_, 1, 8);                                                               \
        ROW12_PLAIN(q_, 2);                                                                     \
        MF4_LOAD4(q_, 3, 0, "op_sel_hi:[0,0,0] cbsz:4 blgp:4",                                  \
                  W4_B_BASE + (((U) + 4) & (STAGES - 1)) * B_BYTES,                             \
                  b_off[0], b_off[1], b_off[2], b_off[3], b_ptr);                               \
        MF4_LOAD4(q_, 3, 1, "op_sel:[1,1,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4",                   \
                  A_LOAD_STAGE12(U) * A2_BYTES + A_LOAD_BLOCK12(U) * 4096,                      \
                  a_off[A_LOAD_BLOCK12(U) + 0], a_off[A_LOAD_BLOCK12(U) + 1],                   \
                  a_off[A_LOAD_BLOCK12(U) + 2], a_off[A_LOAD_BLOCK12(U) + 3], a_ptr);           \
        SB();                                                                                   \
        b_ptr += b_step;                                                                        \
        sa_run += sa_step;                                                                      \
        sb_run += sb_step;                                                                      \
        if constexpr(((U) & 1) == 0)                                                            \
            a_ptr += 2 * BK;                                                                    \
    } while(0)

    // ---- main loop: the schedule of qgemm_w4_i8_kernel ------------------------------------------
#pragma unroll
    for(int h = 0; h < 8; h++)
        issue_a(0, h);
#pragma unroll
    for(int kt = -4; kt < 0; kt++)
    {
        if(kt == -2)
            LOAD_SCALES(0, 0);
        if(kt == -1)
            LOAD_SCALES(1, 1);
        if(issues_b(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_b(kt + 4, h);
        }
        if(issues_a(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_a(a_step_of(kt), ((kt & 1) != 0 ? 0 : 4) + h);
        }
    }
    // slab 0 and its scale words are complete when only what came behind those is in flight
    {
        const int cnt = issued_in(-2) + 8 + issued_in(-1);
        if(cnt >= 24)      wait_vmcnt<24>();
        else if(cnt == 20) wait_vmcnt<20>();
        else if(cnt == 16) wait_vmcnt<16>();
        else if(cnt == 12) wait_vmcnt<12>();
        else               wait_vmcnt<8>();
    }
    block_barrier();
#pragma unroll
    for(int i = 0; i < 4; i++)
    {
        RA(0, 0, i, 0);
        RA(0, 0, i, 1);
    }
#pragma unroll
    for(int j = 0; j < 4; j++)
    {
        RB(0, 0, j, 0);
        RB(0, 0, j, 1);
        RB(0, 0, j, 2);
        RB(0, 0, j, 3);
    }
    int kt = 0;
    if(nk > 17)
    {
        // b_ptr: slab kt + 4 of B; a_ptr: K step a_step_of(kt) of A; sa_run / sb_run: the exponent
        // words of slab kt + 2; all for the slab about to run
        const int64_t b_step = BK;
        const uint8_t* b_ptr = gb + 4 * b_step;
        const uint8_t* a_ptr = ga + 2 * (2 * BK);
        const uint8_t* sa_run = p.mx_ea + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_a * 4 + 2 * sa_step;
        const uint8_t* sb_run = p.mx_eb + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_b * 4 + 2 * sb_step;
        uint32_t m0_saved;
        asm volatile("s_mov_b32 %0, m0" : "=s"(m0_saved));
        W4_TRIPS_OF_TWELVE(kt, nk, SLAB12);
        asm volatile("s_mov_b32 m0, %0" ::"s"(m0_saved));
    }
    for(; kt + 6 < nk; kt += 2)
    {
        SLAB(kt, 0, true);
        SLAB(kt + 1, 1, true);
    }
    // The second half of the accumulators was written last: it passes through a statement that
    // holds the wait states before anything the compiler places here can read it.  The first half
    // is at least eight MFMAs old.
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3"
                 : "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]),
                   "+a"(acc[3][0]), "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3]));
    for(; kt + 1 < nk; kt += 2)
    {
        SLAB(kt, 0, false);
        SLAB(kt + 1, 1, false);
    }
    if(kt < nk)
        SLAB(kt, 0, false);
    // the scale words requested for slabs past the end are still on their way to registers
    wait_vmcnt<0>();
    asm volatile("" : "+v"(sin[0][0]), "+v"(sin[0][1]), "+v"(sin[0][2]), "+v"(sin[0][3]), "+v"(sin[0][4]),
                      "+v"(sin[0][5]), "+v"(sin[0][6]), "+v"(sin[0][7]), "+v"(sin[1][0]), "+v"(sin[1][1]),
                      "+v"(sin[1][2]), "+v"(sin[1][3]), "+v"(sin[1][4]), "+v"(sin[1][5]), "+v"(sin[1][6]),
                      "+v"(sin[1][7]));
#undef SLAB12
#undef MF4_LOAD4
#undef ROW12_PLAIN
#undef ROW12_READS
#undef READ12
#undef MF12
#undef LOAD_SCALES12
#undef LDS1S
#undef RB12
#undef RA12
#undef SLAB
#undef WAIT_SLAB
#undef ROW
#undef OTHER
#undef MF
#undef WAIT_FRAGS
#undef RB
#undef RA
#undef LOAD_SCALES
#undef LDS1
#undef SB
#undef RDTR8
#undef RD128

    // ---- epilogue: the fp8 part of qgemm_dma_kernel's, 4 x 4 tiles per wave ---------------------
    // Element e of lane l belongs to row l % 32 of the A tile and column 8*(e/4) + 4*(l/32) + e%4
    // of the B tile: four groups of 4 consecutive columns, each written with one store.  One block
    // of 32 columns at a time; its scales and biases are loaded ahead of the stores of the block
    // before it (a load issued behind a store waits for it), and no more than two blocks' worth is
    // held in registers.
    if constexpr(!DEQ)
    {
        {
            // The bare result through the LDS, as in qgemm_w4_i8_kernel: straight from the
            // accumulators a store instruction writes 32 bytes of each of 32 rows, from a row-major
            // copy in the LDS the 512 bytes of two whole rows of the wave's quadrant.
            block_barrier();
            constexpr int PITCH = 512 + 16;
            uint8_t* mine       = lds + wave * 40960;
            const int out_col   = n0 + wave_n * 128 + 4 * (lane & 31);
            float* out_base     = static_cast<float*>(p.c) + (int64_t)blockIdx.y * p.stride_c + out_col;
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                uint8_t* buf = mine + (i & 1) * (32 * PITCH);
#pragma unroll
                for(int j = 0; j < 4; j++)
#pragma unroll
                    for(int g = 0; g < 4; g++)
                        *reinterpret_cast<v4f*>(buf + lrow * PITCH + (32 * j + 8 * g + 4 * lgrp) * 4) =
                            v4f{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
                // (every read before the first store, see qgemm_w4_i8_kernel)
                v4f val[16];
#pragma unroll
                for(int t = 0; t < 16; t++)
                    val[t] = *reinterpret_cast<const v4f*>(buf + (2 * t + (lane >> 5)) * PITCH + (lane & 31) * 16);
#pragma unroll
                for(int t = 0; t < 16; t++)
                    asm volatile("" : "+v"(val[t]));
#pragma unroll
                for(int t = 0; t < 16; t++)
                {
                    const int row = m0 + wave_m * 128 + 32 * i + 2 * t + (lane >> 5);
                    if(row < p.m && out_col < p.n)
                        store_rows(reinterpret_cast<v4f*>(out_base + (int64_t)row * p.ldc), val[t], p.stream_c);
                }
            }
            return;
        }
    }
}

// The same for fp8 x fp8 (a slab row is 64 codes in two blocks): the fragments, slots and MFMA count
// of qgemm_w4_f8_kernel, one scaled MFMA per tile pair; lane group g holds chunks g and 2 + g of a
// slab row (the instruction scales K [32 g, 32 g + 32) by group g's exponent), byte g of the row's
// exponent word is its scale.
__global__ __launch_bounds__(W4_THREADS) void qgemm_w4_mx8_kernel(dma_params p)
{
    constexpr bool TRANS_B = true;
    constexpr bool DEQ     = false;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    if(*p.mx_flag == p.mx_ticket)
        return;

    const int tid    = threadIdx.x;
    const int lane   = tid & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 1; // 0..1
    const int wave_n = wave & 1;  // 0..1

    int tm, tn;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    const uint8_t* __restrict__ ga = p.a + (int64_t)blockIdx.y * p.stride_a;
    const uint8_t* __restrict__ gb = p.b + (int64_t)blockIdx.y * p.stride_b;
    const int nk = p.k / BK;

    // ---- global -> LDS: exactly as in qgemm_w4_i8_kernel -------------------------------------
    uint32_t a_off[8], b_off[4];
    const int a_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
#pragma unroll
    for(int h = 0; h < 8; h++)
    {
        const int r   = 8 * (wave + 4 * h) + (lane >> 3);
        const int row = min(m0 + r, p.m - 1);
        a_off[h]      = (uint32_t)row * (uint32_t)p.lda + a_chunk * 16;
    }
    const uint32_t a_tail_back = a_chunk >= 4 ? 64u : 0u;
#pragma unroll
    for(int h = 0; h < 4; h++)
    {
        const int blk = wave + 4 * h;
        if constexpr(TRANS_B)
        {
            const int r     = 16 * blk + (lane >> 2);
            const int chunk = (lane & 3) ^ ((r >> 2) & 3);
            const int col   = min(n0 + r, p.n - 1);
            b_off[h]        = (uint32_t)col * (uint32_t)p.ldb + chunk * 16;
        }
        else
        {
            const int k     = 4 * blk + (lane >> 4);
            const int chunk = (lane & 15) ^ (k & 7);
            const int col   = min(n0 + chunk * 16, p.n - 16);
            b_off[h]        = (uint32_t)k * (uint32_t)p.ldb + col;
        }
    }
    auto issue_a = [&](int ss, int h) {
        uint8_t* st           = lds + (ss % W4_A_STAGES) * A2_BYTES;
        const uint8_t* a_base = ga + (int64_t)ss * (2 * BK);
        const uint32_t back   = 2 * ss + 1 < nk ? 0u : a_tail_back;
        load_to_lds(a_base + (a_off[h] - back), st + (wave + 4 * h) * 1024);
    };
    auto issue_b = [&](int kt, int h) {
        uint8_t* st           = lds + W4_B_BASE + (kt & (STAGES - 1)) * B_BYTES;
        const uint8_t* b_base = TRANS_B ? gb + (int64_t)kt * BK : gb + (int64_t)kt * BK * p.ldb;
        load_to_lds(b_base + b_off[h], st + (wave + 4 * h) * 1024);
    };
    auto a_step_of   = [](int kt) { return (kt & 1) != 0 ? (kt + 5) / 2 : (kt + 4) / 2; };
    auto issues_b    = [&](int kt) { return kt + 4 >= 0 && kt + 4 < nk; };
    auto issues_a    = [&](int kt) { const int ss = a_step_of(kt); return ss >= 1 && 2 * ss < nk; };
    auto issued_in   = [&](int kt) { return (issues_b(kt) ? 4 : 0) + (issues_a(kt) ? 4 : 0); };

    // ---- LDS -> operand fragments -------------------------------------------------------------
    const int lrow      = lane & 31;
    const int lgrp      = lane >> 5;
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    // A: rows of 128 bytes (two slabs); slab parity h, chunk x of this lane's 32 bytes is logical
    // chunk 4h + 2*lgrp + x at position c ^ ((row >> 1) & 7)
    uint32_t a_lane[2][2];
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int x = 0; x < 2; x++)
            a_lane[h][x] = (wave_m * 128 + lrow) * (2 * BK) + (((4 * h + 2 * x + lgrp) ^ ((lrow >> 1) & 7)) << 4);
    uint32_t b_lane[2];
    {
        const int sw = (lrow >> 2) & 3;
#pragma unroll
        for(int x = 0; x < 2; x++)
            b_lane[x] = W4_B_BASE + (wave_n * 128 + lrow) * BK + (((2 * x + lgrp) ^ sw) << 4);
    }

    v8i fa[2][4];
    v8i fb[2][4];
    // exponent bytes of the lane's rows (0..3: A tiles, 4..7: B tiles): in flight, one set per slab
    // parity, and the current slab's, shifted so that byte 0 is the lane group's block
    int sin[2][8] = {{0, 0, 0, 0, 0, 0, 0, 0}, {0, 0, 0, 0, 0, 0, 0, 0}};
    int sc[8]     = {0, 0, 0, 0, 0, 0, 0, 0};
    const int sc_shift = 8 * lgrp;
    const uint8_t* sa_ptr = p.mx_ea + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_a * 4 +
                            (int64_t)(m0 + wave_m * 128 + lrow) * 4;
    const uint8_t* sb_ptr = p.mx_eb + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_b * 4 +
                            (int64_t)(n0 + wave_n * 128 + lrow) * 4;
    const int64_t sa_step = (int64_t)p.mx_rows_a * 4, sb_step = (int64_t)p.mx_rows_b * 4;
    v16f acc[4][4];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
#pragma unroll
            for(int e = 0; e < 16; e++)
                acc[i][j][e] = 0.f;

#define RD128(dst, addr, imm) \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define RDTR8(dst, addr, imm) \
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(imm) : "memory")
#define SB() __builtin_amdgcn_sched_barrier(0)
#define LDS1(dst, ptr, imm) \
    asm volatile("global_load_dword %0, %1, off offset:%2" : "=v"(dst) : "v"(ptr), "n"(imm) : "memory")
#define LOAD_SCALES(s, Q)                                                   \
    do                                                                      \
    {                                                                       \
        const int s_          = min((s), nk - 1);                           \
        const uint8_t* pa_    = sa_ptr + (int64_t)s_ * sa_step;             \
        const uint8_t* pb_    = sb_ptr + (int64_t)s_ * sb_step;             \
        LDS1(sin[Q][0], pa_, 0);   LDS1(sin[Q][1], pa_, 128);               \
        LDS1(sin[Q][2], pa_, 256); LDS1(sin[Q][3], pa_, 384);               \
        LDS1(sin[Q][4], pb_, 0);   LDS1(sin[Q][5], pb_, 128);               \
        LDS1(sin[Q][6], pb_, 256); LDS1(sin[Q][7], pb_, 384);               \
    } while(0)
#define PUT4(frag, X, t)                \
    do                                  \
    {                                   \
        frag[4 * (X) + 0] = t.x;        \
        frag[4 * (X) + 1] = t.y;        \
        frag[4 * (X) + 2] = t.z;        \
        frag[4 * (X) + 3] = t.w;        \
    } while(0)
    // half X of A tile I of slab kt -> fa[Q][I]
#define RA(kt, Q, I, X)                                                                         \
    do                                                                                          \
    {                                                                                           \
        v4i t_;                                                                                 \
        RD128(t_, lds0 + (((kt) >> 1) % W4_A_STAGES) * A2_BYTES + a_lane[(kt) & 1][X],          \
              (I) * 32 * 2 * BK);                                                               \
        PUT4(fa[Q][I], X, t_);                                                                  \
    } while(0)
    // part R of B tile J of slab kt: row-major B four transposing reads, K-contiguous B two
#define RB(kt, Q, J, R)                                                                         \
    do                                                                                          \
    {                                                                                           \
        const uint32_t s_ = lds0 + ((kt) & (STAGES - 1)) * B_BYTES;                             \
        if constexpr(TRANS_B)                                                                   \
        {                                                                                       \
            if((R) < 2)                                                                         \
            {                                                                                   \
                v4i t_;                                                                         \
                RD128(t_, s_ + b_lane[(R) & 1], (J) * 32 * BK);                                 \
                PUT4(fb[Q][J], (R) & 1, t_);                                                    \
            }                                                                                   \
        }                                                                                       \
        else                                                                                    \
        {                                                                                       \
            (void)s_;                                                                           \
        }                                                                                       \
    } while(0)
#define WAIT_FRAGS(Q)                                                                           \
    asm volatile("s_waitcnt lgkmcnt(0)"                                                         \
                 : "+v"(fa[Q][0]), "+v"(fa[Q][1]), "+v"(fa[Q][2]), "+v"(fa[Q][3]),              \
                   "+v"(fb[Q][0]), "+v"(fb[Q][1]), "+v"(fb[Q][2]), "+v"(fb[Q][3])::"memory")
    // The B tile goes in first: the accumulator then holds the tile transposed and a lane owns runs
    // of four consecutive columns of C (see the epilogue).  Assembly for the reason given in
    // qgemm_w4_i8_kernel.  The compiler does not know that the statement is an MFMA and adds none
    // of the wait states a 16-pass MFMA needs before its result may be read.  In the steady-state
    // loop nothing reads an accumulator.  In the last slabs, whose loads and reads are conditional,
    // the compiler keeps copies of the accumulators in scratch memory and stores them right behind
    // the MFMA, so there the statement carries the wait states itself.
#define MF(Q, I, J)                                                                        \
    do                                                                                     \
    {                                                                                      \
        if constexpr(fast_)                                                                \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]" \
                         : "+a"(acc[I][J])                                                 \
                         : "v"(fb[Q][J]), "v"(fa[Q][I]), "v"(sc[4 + (J)]), "v"(sc[I]));    \
        else                                                                               \
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]\n\t" \
                         "s_nop 7\n\ts_nop 7\n\ts_nop 3"                                   \
                         : "+a"(acc[I][J])                                                 \
                         : "v"(fb[Q][J]), "v"(fa[Q][I]), "v"(sc[4 + (J)]), "v"(sc[I]));    \
    } while(0)
    // slot N of 32: 0..7 A reads, 8..23 B reads (8..15 when B is K-contiguous), 24..31 loads.
#define OTHER(kt, Q, N)                                                                     \
    do                                                                                      \
    {                                                                                       \
        if constexpr((N) < 8)                                                               \
        {                                                                                   \
            if(fast_ || more_) RA((kt) + 1, 1 - (Q), (N) >> 1, (N) & 1);                   \
        }                                                                                   \
        else if constexpr((N) < 24)                                                         \
        {                                                                                   \
            if(fast_ || more_) RB((kt) + 1, 1 - (Q), ((N) - 8) >> 2, ((N) - 8) & 3);       \
        }                                                                                   \
        else if constexpr((N) < 28)                                                         \
        {                                                                                   \
            if(fast_ || ldb_) issue_b((kt) + 4, (N) - 24);                                  \
        }                                                                                   \
        else                                                                                \
        {                                                                                   \
            if(fast_ || lda_) issue_a(ass_, (1 - (Q)) * 4 + (N) - 28);                      \
        }                                                                                   \
    } while(0)
#define ROW(kt, Q, I)                                                                       \
    do                                                                                      \
    {                                                                                       \
        SB(); MF(Q, I, 0); SB(); OTHER(kt, Q, 8 * (I) + 0); SB(); OTHER(kt, Q, 8 * (I) + 1);  \
        SB(); MF(Q, I, 1); SB(); OTHER(kt, Q, 8 * (I) + 2); SB(); OTHER(kt, Q, 8 * (I) + 3);  \
        SB(); MF(Q, I, 2); SB(); OTHER(kt, Q, 8 * (I) + 4); SB(); OTHER(kt, Q, 8 * (I) + 5);  \
        SB(); MF(Q, I, 3); SB(); OTHER(kt, Q, 8 * (I) + 6); SB(); OTHER(kt, Q, 8 * (I) + 7);  \
    } while(0)
#define WAIT_SLAB(kt)                                                                       \
    do                                                                                      \
    {                                                                                       \
        const int cnt_ = issued_in((kt) - 2) + issued_in((kt) - 1) + 8;                      \
        if(cnt_ >= 24)      wait_vmcnt<24>();                                               \
        else if(cnt_ >= 20) wait_vmcnt<20>();                                               \
        else if(cnt_ >= 16) wait_vmcnt<16>();                                               \
        else if(cnt_ >= 12) wait_vmcnt<12>();                                               \
        else                wait_vmcnt<8>();                                                \
    } while(0)
#define SLAB(kt, Q, FAST)                                                                   \
    do                                                                                      \
    {                                                                                       \
        constexpr bool fast_ = (FAST);                                                      \
        const int kt_     = (kt);                                                           \
        const bool more_  = kt_ + 1 < nk;                                                   \
        const bool ldb_   = issues_b(kt_);                                                  \
        const bool lda_   = issues_a(kt_);                                                  \
        const int ass_    = a_step_of(kt_);                                                 \
        (void)more_; (void)ldb_; (void)lda_;                                                \
        WAIT_FRAGS(Q);                                                                      \
        if constexpr(fast_)                                                                 \
            wait_vmcnt<24>();                                                               \
        else                                                                                \
            WAIT_SLAB(kt_);                                                                 \
        block_barrier();                                                                    \
        asm volatile("" : "+v"(sin[Q][0]), "+v"(sin[Q][1]), "+v"(sin[Q][2]), "+v"(sin[Q][3]), \
                          "+v"(sin[Q][4]), "+v"(sin[Q][5]), "+v"(sin[Q][6]), "+v"(sin[Q][7])); \
        _Pragma("unroll") for(int t_ = 0; t_ < 8; t_++) sc[t_] = sin[Q][t_] >> sc_shift;     \
        asm volatile("" : "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]),               \
                          "+v"(sc[4]), "+v"(sc[5]), "+v"(sc[6]), "+v"(sc[7]));               \
        LOAD_SCALES(kt_ + 2, Q);                                                            \
        ROW(kt_, Q, 0); ROW(kt_, Q, 1); ROW(kt_, Q, 2); ROW(kt_, Q, 3);                     \
        SB();                                                                               \
    } while(0)

    // ---- the steady state in trips of twelve slabs, as in qgemm_w4_mx4_kernel: the 16 fragment
    // reads follow the first eight of a slab's 16 MFMAs (two each), the eight loads the last eight.
    uint32_t a_vaddr[2][2][2]; // [slab parity][chunk][0: stages 0 and 1, 1: stage 2]
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int x = 0; x < 2; x++)
        {
            a_vaddr[h][x][0] = lds0 + a_lane[h][x];
            a_vaddr[h][x][1] = lds0 + a_lane[h][x] + 2 * A2_BYTES;
        }
    const uint32_t b_vaddr[2] = {lds0 + b_lane[0], lds0 + b_lane[1]};
    const uint32_t wave_lds   = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const uint32_t sa_off     = (uint32_t)(m0 + wave_m * 128 + lrow) * 4u;
    const uint32_t sb_off     = (uint32_t)(n0 + wave_n * 128 + lrow) * 4u;
#define RA12(U1, Q, I, X)                                                                       \
    do                                                                                          \
    {                                                                                           \
        v4i t_;                                                                                 \
        RD128(t_, a_vaddr[(U1) & 1][X][A_STAGE12(U1) == 2 ? 1 : 0],                             \
              (A_STAGE12(U1) == 2 ? 0 : A_STAGE12(U1) * A2_BYTES) + (I) * 32 * 2 * BK);         \
        PUT4(fa[Q][I], X, t_);                                                                  \
    } while(0)
#define RB12(U1, Q, J, R)                                                                       \
    do                                                                                          \
    {                                                                                           \
        v4i t_;                                                                                 \
        RD128(t_, b_vaddr[R], ((U1) & (STAGES - 1)) * B_BYTES + (J) * 32 * BK);                 \
        PUT4(fb[Q][J], R, t_);                                                                  \
    } while(0)
#define LDS1S(dst, off, base, imm)                                                              \
    asm volatile("global_load_dword %0, %1, %2 offset:%3"                                       \
                 : "=v"(dst)                                                                    \
                 : "v"(off), "s"(base), "n"(imm)                                                \
                 : "memory")
#define LOAD_SCALES12(Q)                                                                        \
    do                                                                                          \
    {                                                                                           \
        LDS1S(sin[Q][0], sa_off, sa_run, 0);   LDS1S(sin[Q][1], sa_off, sa_run, 128);           \
        LDS1S(sin[Q][2], sa_off, sa_run, 256); LDS1S(sin[Q][3], sa_off, sa_run, 384);           \
        LDS1S(sin[Q][4], sb_off, sb_run, 0);   LDS1S(sin[Q][5], sb_off, sb_run, 128);           \
        LDS1S(sin[Q][6], sb_off, sb_run, 256); LDS1S(sin[Q][7], sb_off, sb_run, 384);           \
    } while(0)
#define MF12(Q, I, J)                                                                           \
    asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]"    \
                 : "+a"(acc[I][J])                                                              \
                 : "v"(fb[Q][J]), "v"(fa[Q][I]), "v"(sc[4 + (J)]), "v"(sc[I]))
#define READ12(U, Q, N)                                                                         \
    do                                                                                          \
    {                                                                                           \
        if constexpr((N) < 8)                                                                   \
            RA12((U) + 1, 1 - (Q), (N) >> 1, (N) & 1);                                          \
        else                                                                                    \
            RB12((U) + 1, 1 - (Q), ((N) - 8) >> 1, ((N) - 8) & 1);                              \
    } while(0)
#define ROW12_READS(U, Q, I, N0)                                                                \
    do                                                                                          \
    {                                                                                           \
        SB(); MF12(Q, I, 0); SB(); READ12(U, Q, (N0) + 0); READ12(U, Q, (N0) + 1);              \
        SB(); MF12(Q, I, 1); SB(); READ12(U, Q, (N0) + 2); READ12(U, Q, (N0) + 3);              \
        SB(); MF12(Q, I, 2); SB(); READ12(U, Q, (N0) + 4); READ12(U, Q, (N0) + 5);              \
        SB(); MF12(Q, I, 3); SB(); READ12(U, Q, (N0) + 6); READ12(U, Q, (N0) + 7);              \
    } while(0)
#define MF4_LOAD4(Q, I, LDS_CONST, OFF0, OFF1, OFF2, OFF3, BASE)                                \
    asm volatile("s_add_i32 m0, %[wl], %[lc0]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c0], %[b0], %[a], %[c0], %[s0], %[sa] op_sel_hi:[0,0,0]\n\t" \
                 "global_load_lds_dwordx4 %[o0], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc1]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c1], %[b1], %[a], %[c1], %[s1], %[sa] op_sel_hi:[0,0,0]\n\t" \
                 "global_load_lds_dwordx4 %[o1], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc2]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c2], %[b2], %[a], %[c2], %[s2], %[sa] op_sel_hi:[0,0,0]\n\t" \
                 "global_load_lds_dwordx4 %[o2], %[base]\n\t"                                   \
                 "s_nop 0\n\t"                                                                  \
                 "s_add_i32 m0, %[wl], %[lc3]\n\t"                                              \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %[c3], %[b3], %[a], %[c3], %[s3], %[sa] op_sel_hi:[0,0,0]\n\t" \
                 "global_load_lds_dwordx4 %[o3], %[base]"                                       \
                 : [c0] "+a"(acc[I][0]), [c1] "+a"(acc[I][1]), [c2] "+a"(acc[I][2]),            \
                   [c3] "+a"(acc[I][3])                                                         \
                 : [b0] "v"(fb[Q][0]), [b1] "v"(fb[Q][1]), [b2] "v"(fb[Q][2]),                  \
                   [b3] "v"(fb[Q][3]), [a] "v"(fa[Q][I]), [s0] "v"(sc[4]), [s1] "v"(sc[5]),     \
                   [s2] "v"(sc[6]), [s3] "v"(sc[7]), [sa] "v"(sc[I]), [wl] "s"(wave_lds),       \
                   [lc0] "n"((LDS_CONST) + 0 * 4096), [lc1] "n"((LDS_CONST) + 1 * 4096),        \
                   [lc2] "n"((LDS_CONST) + 2 * 4096), [lc3] "n"((LDS_CONST) + 3 * 4096),        \
                   [o0] "v"(OFF0), [o1] "v"(OFF1), [o2] "v"(OFF2), [o3] "v"(OFF3),              \
                   [base] "s"(BASE)                                                             \
                 : "memory", "scc")
#define SLAB12(U)                                                                               \
    do                                                                                          \
    {                                                                                           \
        constexpr int q_ = (U) & 1;                                                             \
        /* may stay in flight: the loads of the last two slabs and the next slab's scale words */ \
        asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)"                                           \
                     : "+v"(fa[q_][0]), "+v"(fa[q_][1]), "+v"(fa[q_][2]), "+v"(fa[q_][3]),      \
                       "+v"(fb[q_][0]), "+v"(fb[q_][1]), "+v"(fb[q_][2]), "+v"(fb[q_][3])::"memory"); \
        block_barrier();                                                                        \
        asm volatile("" : "+v"(sin[q_][0]), "+v"(sin[q_][1]), "+v"(sin[q_][2]), "+v"(sin[q_][3]), \
                          "+v"(sin[q_][4]), "+v"(sin[q_][5]), "+v"(sin[q_][6]), "+v"(sin[q_][7])); \
        _Pragma("unroll") for(int t_ = 0; t_ < 8; t_++) sc[t_] = sin[q_][t_] >> sc_shift;        \
        asm volatile("" : "+v"(sc[0]), "+v"(sc[1]), "+v"(sc[2]), "+v"(sc[3]),                   \
                          "+v"(sc[4]), "+v"(sc[5]), "+v"(sc[6]), "+v"(sc[7]));                   \
        LOAD_SCALES12(q_);                                                                      \
        ROW12_READS(U, q_, 0, 0);                                                               \
        ROW12_READS(U, q_, 1, 8);                                                               \
        SB();                                                                                   \
        MF4_LOAD4(q_, 2, W4_B_BASE + (((U) + 4) & (STAGES - 1)) * B_BYTES,                      \
                  b_off[0], b_off[1], b_off[2], b_off[3], b_ptr);                               \
        MF4_LOAD4(q_, 3, A_LOAD_STAGE12(U) * A2_BYTES + A_LOAD_BLOCK12(U) * 4096,               \
                  a_off[A_LOAD_BLOCK12(U) + 0], a_off[A_LOAD_BLOCK12(U) + 1],                   \
                  a_off[A_LOAD_BLOCK12(U) + 2], a_off[A_LOAD_BLOCK12(U) + 3], a_ptr);           \
        SB();                                                                                   \
        b_ptr += b_step;                                                                        \
        sa_run += sa_step;                                                                      \
        sb_run += sb_step;                                                                      \
        if constexpr(((U) & 1) == 0)                                                            \
            a_ptr += 2 * BK;                                                                    \
    } while(0)

    // ---- main loop: the schedule of qgemm_w4_i8_kernel ------------------------------------------
#pragma unroll
    for(int h = 0; h < 8; h++)
        issue_a(0, h);
#pragma unroll
    for(int kt = -4; kt < 0; kt++)
    {
        if(kt == -2)
            LOAD_SCALES(0, 0);
        if(kt == -1)
            LOAD_SCALES(1, 1);
        if(issues_b(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_b(kt + 4, h);
        }
        if(issues_a(kt))
        {
#pragma unroll
            for(int h = 0; h < 4; h++)
                issue_a(a_step_of(kt), ((kt & 1) != 0 ? 0 : 4) + h);
        }
    }
    {
        const int cnt = issued_in(-2) + 8 + issued_in(-1);
        if(cnt >= 24)      wait_vmcnt<24>();
        else if(cnt == 20) wait_vmcnt<20>();
        else if(cnt == 16) wait_vmcnt<16>();
        else if(cnt == 12) wait_vmcnt<12>();
        else               wait_vmcnt<8>();
    }
    block_barrier();
#pragma unroll
    for(int i = 0; i < 4; i++)
    {
        RA(0, 0, i, 0);
        RA(0, 0, i, 1);
    }
#pragma unroll
    for(int j = 0; j < 4; j++)
    {
        RB(0, 0, j, 0);
        RB(0, 0, j, 1);
        RB(0, 0, j, 2);
        RB(0, 0, j, 3);
    }
    int kt = 0;
    if(nk > 17)
    {
        // b_ptr: slab kt + 4 of B; a_ptr: K step a_step_of(kt) of A; sa_run / sb_run: the exponent
        // words of slab kt + 2; all for the slab about to run
        const int64_t b_step = BK;
        const uint8_t* b_ptr = gb + 4 * b_step;
        const uint8_t* a_ptr = ga + 2 * (2 * BK);
        const uint8_t* sa_run = p.mx_ea + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_a * 4 + 2 * sa_step;
        const uint8_t* sb_run = p.mx_eb + (int64_t)blockIdx.y * (int64_t)nk * p.mx_rows_b * 4 + 2 * sb_step;
        uint32_t m0_saved;
        asm volatile("s_mov_b32 %0, m0" : "=s"(m0_saved));
        W4_TRIPS_OF_TWELVE(kt, nk, SLAB12);
        asm volatile("s_mov_b32 m0, %0" ::"s"(m0_saved));
    }
    for(; kt + 6 < nk; kt += 2)
    {
        SLAB(kt, 0, true);
        SLAB(kt + 1, 1, true);
    }
    // The second half of the accumulators was written last: it passes through a statement that
    // holds the wait states before anything the compiler places here can read it.  The first half
    // is at least eight MFMAs old.
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3"
                 : "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]),
                   "+a"(acc[3][0]), "+a"(acc[3][1]), "+a"(acc[3][2]), "+a"(acc[3][3]));
    for(; kt + 1 < nk; kt += 2)
    {
        SLAB(kt, 0, false);
        SLAB(kt + 1, 1, false);
    }
    if(kt < nk)
        SLAB(kt, 0, false);
    wait_vmcnt<0>();
    asm volatile("" : "+v"(sin[0][0]), "+v"(sin[0][1]), "+v"(sin[0][2]), "+v"(sin[0][3]), "+v"(sin[0][4]),
                      "+v"(sin[0][5]), "+v"(sin[0][6]), "+v"(sin[0][7]), "+v"(sin[1][0]), "+v"(sin[1][1]),
                      "+v"(sin[1][2]), "+v"(sin[1][3]), "+v"(sin[1][4]), "+v"(sin[1][5]), "+v"(sin[1][6]),
                      "+v"(sin[1][7]));
#undef SLAB12
#undef MF4_LOAD4
#undef ROW12_READS
#undef READ12
#undef MF12
#undef LOAD_SCALES12
#undef LDS1S
#undef RB12
#undef RA12
#undef SLAB
#undef WAIT_SLAB
#undef ROW
#undef OTHER
#undef MF
#undef WAIT_FRAGS
#undef RB
#undef RA
#undef PUT4
#undef LOAD_SCALES
#undef LDS1
#undef SB
#undef RDTR8
#undef RD128

    // ---- epilogue: the fp8 part of qgemm_dma_kernel's, 4 x 4 tiles per wave ---------------------
    // Element e of lane l belongs to row l % 32 of the A tile and column 8*(e/4) + 4*(l/32) + e%4
    // of the B tile: four groups of 4 consecutive columns, each written with one store.  One block
    // of 32 columns at a time; its scales and biases are loaded ahead of the stores of the block
    // before it (a load issued behind a store waits for it), and no more than two blocks' worth is
    // held in registers.
    if constexpr(!DEQ)
    {
        {
            // The bare result through the LDS, as in qgemm_w4_i8_kernel: straight from the
            // accumulators a store instruction writes 32 bytes of each of 32 rows, from a row-major
            // copy in the LDS the 512 bytes of two whole rows of the wave's quadrant.
            block_barrier();
            constexpr int PITCH = 512 + 16;
            uint8_t* mine       = lds + wave * 40960;
            const int out_col   = n0 + wave_n * 128 + 4 * (lane & 31);
            float* out_base     = static_cast<float*>(p.c) + (int64_t)blockIdx.y * p.stride_c + out_col;
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                uint8_t* buf = mine + (i & 1) * (32 * PITCH);
#pragma unroll
                for(int j = 0; j < 4; j++)
#pragma unroll
                    for(int g = 0; g < 4; g++)
                        *reinterpret_cast<v4f*>(buf + lrow * PITCH + (32 * j + 8 * g + 4 * lgrp) * 4) =
                            v4f{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
                // (every read before the first store, see qgemm_w4_i8_kernel)
                v4f val[16];
#pragma unroll
                for(int t = 0; t < 16; t++)
                    val[t] = *reinterpret_cast<const v4f*>(buf + (2 * t + (lane >> 5)) * PITCH + (lane & 31) * 16);
#pragma unroll
                for(int t = 0; t < 16; t++)
                    asm volatile("" : "+v"(val[t]));
#pragma unroll
                for(int t = 0; t < 16; t++)
                {
                    const int row = m0 + wave_m * 128 + 32 * i + 2 * t + (lane >> 5);
                    if(row < p.m && out_col < p.n)
                        store_rows(reinterpret_cast<v4f*>(out_base + (int64_t)row * p.ldc), val[t], p.stream_c);
                }
            }
            return;
        }
    }
}

template <bool FP8, bool TRANS_B, bool DEQ, int OUT>
int launch_one(const dma_params& p, int batch, hipStream_t stream)
{
    if constexpr(FP8)
    {
        // as for int8 (launch_i8_one): the four-wave kernel from K = 3072 on, where C takes whole
        // groups of 4 outputs
        if(p.k >= 3072 && p.vec_store && p.n % 4 == 0)
        {
            constexpr bool half_out = DEQ && (OUT == MI355_F16 || OUT == MI355_BF16);
            auto kern4 = qgemm_w4_f8_kernel<TRANS_B, DEQ, OUT, false>;
            if constexpr(half_out)
            {
                if(p.vec8_store)
                    kern4 = qgemm_w4_f8_kernel<TRANS_B, DEQ, OUT, true>;
            }
            // once per kernel: above the 64 KiB default
            static const hipError_t attr4 = hipFuncSetAttribute(
                reinterpret_cast<const void*>(qgemm_w4_f8_kernel<TRANS_B, DEQ, OUT, false>),
                hipFuncAttributeMaxDynamicSharedMemorySize, W4_LDS_BYTES);
            static const hipError_t attr8 =
                half_out ? hipFuncSetAttribute(reinterpret_cast<const void*>(qgemm_w4_f8_kernel<TRANS_B, DEQ, OUT, half_out>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, W4_LDS_BYTES)
                         : hipSuccess;
            if(attr4 != hipSuccess || attr8 != hipSuccess)
                return MI355_ERR_LAUNCH;
            dim3 grid4(p.tiles_m * p.tiles_n, batch);
            hipLaunchKernelGGL(kern4, grid4, dim3(W4_THREADS), W4_LDS_BYTES, stream, p);
            return mi355_launch_status();
        }
    }
    auto kern = qgemm_dma_kernel<FP8, TRANS_B, DEQ, OUT>;
    // above the 64 KiB default: opt in once per kernel instantiation
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if(attr != hipSuccess)
        return MI355_ERR_LAUNCH;
    dim3 grid(p.tiles_m * p.tiles_n, batch);
    hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), LDS_BYTES, stream, p);
    return mi355_launch_status();
}

template <bool FP8, bool TRANS_B>
int launch_out(const dma_params& p, int batch, bool deq, int out, hipStream_t s)
{
    if(!deq)
        return launch_one<FP8, TRANS_B, false, MI355_F32>(p, batch, s);
    switch(out)
    {
    case MI355_F32: return launch_one<FP8, TRANS_B, true, MI355_F32>(p, batch, s);
    case MI355_F16: return launch_one<FP8, TRANS_B, true, MI355_F16>(p, batch, s);
    case MI355_BF16: return launch_one<FP8, TRANS_B, true, MI355_BF16>(p, batch, s);
    default: return MI355_ERR_UNSUPPORTED;
    }
}

} // namespace

// Block-scaled fp4 x fp4 or fp8 x fp8 (see qgemm_dma_kernel<.., MX>): kbytes = bytes per row of A
// [M, kbytes] and of B [N, kbytes] (K / 2 or K), a multiple of the 64-byte slab; bits = 4 or 8;
// ea / eb as described at dma_params::mx_ea.
bool mi355_dma_mx_supported(int64_t m, int64_t n, int64_t kbytes, int64_t lda, int64_t ldb, int64_t ldc,
                            int64_t stride_a, int64_t stride_b, const void* a, const void* b)
{
    (void)ldc;
    if(m <= 0 || n <= 0 || kbytes < BK || kbytes % BK != 0)
        return false;
    if(lda % 16 != 0 || ldb % 16 != 0 || stride_a % 16 != 0 || stride_b % 16 != 0 ||
       reinterpret_cast<uintptr_t>(a) % 16 != 0 || reinterpret_cast<uintptr_t>(b) % 16 != 0)
        return false;
    const int64_t lim = (int64_t)1 << 31;
    return m * lda < lim && n * ldb < lim && m < (1 << 30) && n < (1 << 30);
}

int mi355_dma_mx_launch(const void* a, const void* b, float* c, int64_t m, int64_t n, int64_t kbytes,
                        int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b,
                        int64_t stride_c, int64_t batch, const uint8_t* ea, const uint8_t* eb,
                        const uint32_t* flag, uint32_t ticket, int bits, hipStream_t stream)
{
    dma_params p{};
    p.a          = static_cast<const uint8_t*>(a);
    p.b          = static_cast<const uint8_t*>(b);
    p.c          = c;
    p.m          = (int)m;
    p.n          = (int)n;
    p.k          = (int)kbytes;
    p.lda        = lda;
    p.ldb        = ldb;
    p.ldc        = ldc;
    p.stride_a   = stride_a;
    p.stride_b   = stride_b;
    p.stride_c   = stride_c;
    p.tiles_m    = (p.m + BM - 1) / BM;
    p.tiles_n    = (p.n + BN - 1) / BN;
    p.ksplit     = 1;
    p.partial_ld = (int)((n + 3) / 4 * 4);
    p.vec_store  = ldc % 4 == 0 && stride_c % 4 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0;
    p.stream_c   = (double)batch * (double)m * (double)n * 4.0 >= 128.0 * 1048576.0;
    p.mx_ea      = ea;
    p.mx_eb      = eb;
    p.mx_flag    = flag;
    p.mx_ticket  = ticket;
    p.mx_rows_a  = p.tiles_m * BM;
    p.mx_rows_b  = p.tiles_n * BN;
    constexpr int lds_bytes = STAGES * (STAGE_BYTES + 2048);
    using kernel_t = void (*)(dma_params);
    static const kernel_t kerns[4] = {qgemm_dma_kernel<true, true, false, MI355_F32, 4, false>,
                                      qgemm_dma_kernel<true, true, false, MI355_F32, 8, false>,
                                      qgemm_dma_kernel<true, true, false, MI355_F32, 4, true>,
                                      qgemm_dma_kernel<true, true, false, MI355_F32, 8, true>};
    static const bool attrs_ok = [] {
        bool ok = true;
        for(kernel_t k : kerns)
            ok = ok && hipFuncSetAttribute(reinterpret_cast<const void*>(k),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) == hipSuccess;
        return ok;
    }();
    if(!attrs_ok || (bits != 4 && bits != 8))
        return MI355_ERR_LAUNCH;
    dim3 grid(p.tiles_m * p.tiles_n, (unsigned)batch);
    // rows of 2048 bytes and more (4096 fp4 codes, 2048 fp8 codes): the four-wave kernels (as for int8
    // and fp8: they pay more per tile and less per slab)
    if(kbytes >= 2048 && p.vec_store && p.n % 4 == 0)
    {
        static const hipError_t attr4 =
            hipFuncSetAttribute(reinterpret_cast<const void*>(qgemm_w4_mx4_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, W4_LDS_BYTES);
        static const hipError_t attr8 =
            hipFuncSetAttribute(reinterpret_cast<const void*>(qgemm_w4_mx8_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, W4_LDS_BYTES);
        if(attr4 != hipSuccess || attr8 != hipSuccess)
            return MI355_ERR_LAUNCH;
        hipLaunchKernelGGL(bits == 4 ? qgemm_w4_mx4_kernel : qgemm_w4_mx8_kernel, grid, dim3(W4_THREADS),
                           W4_LDS_BYTES, stream, p);
        return mi355_launch_status();
    }
    // a result that stays in the caches leaves through the LDS copy (whole groups of 4 outputs)
    const bool via_lds = !p.stream_c && p.vec_store && p.n % 4 == 0;
    hipLaunchKernelGGL(kerns[(bits == 8 ? 1 : 0) + (via_lds ? 2 : 0)], grid, dim3(NTHREADS), lds_bytes, stream, p);
    return mi355_launch_status();
}

// The direct-to-LDS kernel moves whole 16-byte chunks and cannot zero-fill a
// partial one: K must be a multiple of the 64-byte slab, row-major B needs N a
// multiple of 16, and every chunk must be 16-byte aligned in memory.
bool mi355_dma_gemm_supported(const mi355_quant_dot_desc* d, const void* a, const void* b)
{
    if(d->trans_a)
        return false;
    if(d->k % BK != 0 || d->k < BK)
        return false;
    if(d->lda % 16 != 0 || d->stride_a % 16 != 0 || reinterpret_cast<uintptr_t>(a) % 16 != 0)
        return false;
    if(d->ldb % 16 != 0 || d->stride_b % 16 != 0 || reinterpret_cast<uintptr_t>(b) % 16 != 0)
        return false;
    if(!d->trans_b && (d->n % 16 != 0 || d->n < 16))
        return false;
    if(d->m > (1 << 30) || d->n > (1 << 30) || d->k > (1 << 30))
        return false;
    // per-lane byte offsets inside one matrix are kept in 32 bits
    const int64_t lim = (int64_t)1 << 31;
    if(d->m * d->lda >= lim || (d->trans_b ? d->n * d->ldb : d->k * d->ldb) >= lim)
        return false;
    return true;
}

// fp8: the shares are equal slices of K (the split goes through the kernel's batch index), so the
// count from the model is lowered to the next divisor of the number of slabs; one batch only
static int fp8_shares(const mi355_quant_dot_desc* d)
{
    if(d->batch != 1 || d->k % BK != 0 || d->m <= 0 || d->n <= 0)
        return 1;
    const int nk    = (int)(d->k / BK);
    const int tiles = (int)(((d->m + BM - 1) / BM) * ((d->n + BN - 1) / BN));
    int s           = choose_ksplit_ws(tiles, 1, nk, d->m, d->n, d->k);
    while(s > 1 && nk % s != 0)
        s--;
    return s;
}

// bytes of workspace that would let a quant_dot of this description (bare or dequantizing) split K
// without atomics (0: no use for one)
size_t mi355_dma_gemm_workspace(const mi355_quant_dot_desc* d)
{
    if(d->in_type == MI355_FP8)
    {
        if(d->trans_a || d->n % 4 != 0 || d->ldc % 4 != 0 || (!d->trans_b && d->n % 16 != 0))
            return 0;
        const int s = fp8_shares(d);
        return s > 1 ? (size_t)s * d->m * d->n * 4 : 0;
    }
    if(d->in_type != MI355_I8 || d->trans_a || d->k % BK != 0 || d->k < BK || d->m <= 0 || d->n <= 0 ||
       d->batch <= 0 || (!d->trans_b && d->n % 16 != 0))
        return 0;
    const int tiles = (int)(((d->m + BM - 1) / BM) * ((d->n + BN - 1) / BN));
    const int s     = choose_ksplit_ws(tiles, (int)d->batch, (int)(d->k / BK), d->m, d->n, d->k);
    return s > 1 ? (size_t)s * d->batch * d->m * ((d->n + 3) / 4 * 4) * 4 : 0;
}

int mi355_dma_gemm_launch(const mi355_quant_dot_desc* d,
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
                          hipStream_t stream)
{
    dma_params p;
    p.bias         = bias;
    p.partial      = nullptr;
    p.partial_ld   = (int)((d->n + 3) / 4 * 4);
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
    const bool fp8 = d->in_type == MI355_FP8;
    const bool deq = d->dequant != 0;
    // column scales and a bias per batch entry: the dense int8 kernels with the epilogue
    const bool cols_per_batch = d->scale_b_mode == MI355_QP_PER_COL_BATCH;
    if(cols_per_batch)
    {
        if(fp8 || !deq || d->n % 4 != 0)
            return MI355_ERR_UNSUPPORTED;
        p.scale_b_mode = MI355_QP_PER_COL;
        p.stride_cols  = d->n;
    }
    {
        const size_t esz = deq ? mi355_dtype_size(d->out_type) : 4;
        p.vec_store = d->ldc % 4 == 0 && d->stride_c % 4 == 0 &&
                      reinterpret_cast<uintptr_t>(c) % (4 * esz) == 0;
        p.vec8_store = esz == 2 && d->n % 8 == 0 && d->ldc % 8 == 0 && d->stride_c % 8 == 0 &&
                       reinterpret_cast<uintptr_t>(c) % 16 == 0;
        // half of the 256 MB last-level cache and more: the result streams past it
        p.stream_c = (double)d->batch * (double)d->m * (double)d->n * (double)esz >= 128.0 * 1048576.0;
        auto aligned16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
        p.vec_cols = d->n % 4 == 0 && (p.scale_b_mode != MI355_QP_PER_COL || aligned16(scale_b)) &&
                     (d->zp_a == 0 || aligned16(colsum_b)) && (bias == nullptr || aligned16(bias));
    }
    p.ksplit = 1;
    if(fp8 && workspace != nullptr && reinterpret_cast<uintptr_t>(workspace) % 16 == 0 && p.vec_store &&
       d->n % 4 == 0)
    {
        // Split K through the batch index: share z is the bare product of A[:, z*kz : (z+1)*kz]
        // and the matching rows of B, written to partial[z] (the kernel itself is unchanged);
        // the second kernel adds the shares and applies the epilogue.
        const int s = fp8_shares(d);
        if(s > 1 && (size_t)s * d->m * d->n * 4 <= workspace_bytes)
        {
            dma_params q = p;
            q.k          = p.k / s;
            q.c          = workspace;
            q.ldc        = d->n;
            q.stride_c   = d->m * d->n;
            q.stride_a   = q.k;
            q.stride_b   = d->trans_b ? (int64_t)q.k : (int64_t)q.k * d->ldb;
            q.vec_store  = 1;
            q.vec8_store = 0;
            q.bias       = nullptr;
            const int st = d->trans_b ? launch_out<true, true>(q, s, false, MI355_F32, stream)
                                      : launch_out<true, false>(q, s, false, MI355_F32, stream);
            if(st != MI355_OK)
                return st;
            p.ksplit  = s;
            p.partial = static_cast<int32_t*>(workspace);
            return launch_reduce<true>(p, 1, s, deq, d->out_type, stream);
        }
    }
    if(fp8)
        return d->trans_b ? launch_out<true, true>(p, (int)d->batch, deq, d->out_type, stream)
                          : launch_out<true, false>(p, (int)d->batch, deq, d->out_type, stream);
    // int8: 4 consecutive outputs of a row go out in one store when every row of
    // C keeps them aligned (N % 4 == 0 holds whenever this path is taken for
    // row-major B; for [N, K] B it is checked here)
    const size_t osz = deq ? mi355_dtype_size(d->out_type) : 4;
    const bool vec   = d->n % 4 == 0 && d->ldc % 4 == 0 && d->stride_c % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(c) % (4 * osz) == 0;
    if(workspace != nullptr && reinterpret_cast<uintptr_t>(workspace) % 16 == 0 && !cols_per_batch &&
       (!deq || d->out_type == MI355_F32 || d->out_type == MI355_F16 || d->out_type == MI355_BF16))
    {
        const int s = choose_ksplit_ws(p.tiles_m * p.tiles_n, (int)d->batch, p.k / BK, d->m, d->n, d->k);
        if(s > 1 && (size_t)s * d->batch * d->m * p.partial_ld * 4 <= workspace_bytes)
        {
            p.ksplit  = s;
            p.partial = static_cast<int32_t*>(workspace);
            return d->trans_b ? launch_i8_splitk<true>(p, (int)d->batch, stream, deq, d->out_type)
                              : launch_i8_splitk<false>(p, (int)d->batch, stream, deq, d->out_type);
        }
    }
    if(d->n % 4 != 0)
        // the 16 x 16 kernel drops or keeps 4 columns together
        return d->trans_b ? launch_out<false, true>(p, (int)d->batch, deq, d->out_type, stream)
                          : launch_out<false, false>(p, (int)d->batch, deq, d->out_type, stream);
    p.ksplit = 1;
    if(vec && !deq)
    {
        p.ksplit = choose_ksplit(p.tiles_m * p.tiles_n, (int)d->batch, p.k / BK, d->m, d->n, d->k);
        if(p.ksplit > 1)
            return d->trans_b ? launch_i8_splitk<true>(p, (int)d->batch, stream)
                              : launch_i8_splitk<false>(p, (int)d->batch, stream);
    }
    if(vec)
        return d->trans_b ? launch_i8_out<true, true>(p, (int)d->batch, deq, d->out_type, stream)
                          : launch_i8_out<false, true>(p, (int)d->batch, deq, d->out_type, stream);
    return d->trans_b ? launch_i8_out<true, false>(p, (int)d->batch, deq, d->out_type, stream)
                      : launch_i8_out<false, false>(p, (int)d->batch, deq, d->out_type, stream);
}
