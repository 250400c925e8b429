// quant_convolution over one, two or three spatial axes (a missing leading axis is a depth of one),
// in four forms that mi355_quant_convolution3d chooses between:
//   - a window of one element with unit strides and no padding: the batched quantized GEMM on the
//     tensors as they lie (the input is its row-major second operand);
//   - many groups of a few channels: one or four outputs per thread on the vector ALU; depthwise
//     layers over images from input rows staged in LDS (conv_depthwise_rows_kernel);
//   - one group, or groups of a multiple of 16 channels: the direct kernel (an implicit GEMM over a
//     padded channels-last copy of the input, see conv_direct_kernel; pixels of 4 channels for a
//     first layer's 1 to 4 channels, see direct_narrow);
//   - everything else, im2col + GEMM: the windows of the input are gathered into a
//     [N, group, OD*OH*OW, Kp] matrix (Kp = C/group * KD * KH * KW rounded up to the GEMM's K step,
//     zero filled), the weights are copied to rows of the same pitch, and for every image the result
//     plane [O, OD*OH*OW] = W [O, Kp] . col^T is one batched mi355_quant_dot with the col matrix as
//     the transposed operand: the GEMM writes NC(D)HW directly and its dequantize epilogue applies
//     the per-output-channel scale as a per-row scale.
// Zero padding adds exact zeros to every sum (int8: 0 * w; fp8: the code 0 is +0.0 and the padded
// weights are +0.0 too), so every form gives the direct convolution's result.
#include "common.h"

namespace {

constexpr int64_t K_STEP = 64;

struct im2col_params
{
    const uint8_t* x;
    uint8_t* col;
    int64_t rows;         // N * OD * OH * OW
    int64_t c, d, h, w;   // input channels (all groups), depth, height, width
    int64_t cg;           // channels per group
    int64_t kd, kh, kw, od, oh, ow;
    int64_t pad_d, pad_h, pad_w, stride_d, stride_h, stride_w, dil_d, dil_h, dil_w;
    int64_t group;
    int64_t kg, kp;    // window elements per group, padded row length
};

// A wave covers 64 consecutive output positions (lane = position) and one 16-byte piece of their
// rows at a time: every byte load then reads neighbouring input bytes across the lanes (one or two
// cache lines per instruction), and the (channel, window plane, row, column) of a piece is the
// same for the whole wave.  The four waves of a workgroup write four neighbouring pieces of the
// same rows, which the L2 merges into whole lines.  blockIdx.y is the group, blockIdx.z the set of
// four pieces.
__global__ __launch_bounds__(256) void im2col_kernel(im2col_params p)
{
    const int lane      = threadIdx.x & 63;
    const int wave      = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int chunks    = (int)(p.kp / 16);
    const int g         = blockIdx.y;
    const int64_t plane = p.od * p.oh * p.ow;
    const int kw = (int)p.kw, kh = (int)p.kh, kd = (int)p.kd, kg = (int)p.kg;
    const int d = (int)p.d, h = (int)p.h, w = (int)p.w;
    const int dil_d = (int)p.dil_d, dil_h = (int)p.dil_h, dil_w = (int)p.dil_w;
    for(int64_t base = (int64_t)blockIdx.x * 64; base < p.rows; base += (int64_t)gridDim.x * 64)
    {
        const int64_t row = base + lane;
        const bool live   = row < p.rows;
        const int64_t rr  = live ? row : p.rows - 1;
        const int64_t n   = rr / plane;
        const int64_t pos = rr % plane;
        const int oz      = (int)(pos / (p.oh * p.ow));
        const int oy      = (int)(pos / p.ow % p.oh);
        const int ox      = (int)(pos % p.ow);
        const int z0      = oz * (int)p.stride_d - (int)p.pad_d;
        const int y0      = oy * (int)p.stride_h - (int)p.pad_h;
        const int x0      = ox * (int)p.stride_w - (int)p.pad_w;
        const uint8_t* img = p.x + (n * p.c + g * p.cg) * d * h * w;
        uint8_t* dst_row   = p.col + ((n * p.group + g) * plane + pos) * p.kp;
        const int chunk = blockIdx.z * 4 + wave;
        if(chunk < chunks)
        {
            int k  = chunk * 16;
            int q  = k % kw;
            int r  = (k / kw) % kh;
            int t  = (k / (kw * kh)) % kd;
            int ch = k / (kw * kh * kd);
            uint32_t packed[4] = {0, 0, 0, 0};
#pragma unroll
            for(int e = 0; e < 16; e++, k++)
            {
                // always load (from a clamped address) and select afterwards: the 16 loads are then
                // independent and in flight together
                const int iz     = z0 + t * dil_d;
                const int iy     = y0 + r * dil_h;
                const int ix     = x0 + q * dil_w;
                const bool valid = k < kg && iz >= 0 && iz < d && iy >= 0 && iy < h && ix >= 0 && ix < w;
                const int64_t at = valid ? (((int64_t)ch * d + iz) * h + iy) * w + ix : 0;
                const uint32_t v = valid ? img[at] : (uint32_t)(img[at] & 0);
                packed[e / 4] |= v << (8 * (e % 4));
                if(++q == kw)
                {
                    q = 0;
                    if(++r == kh)
                    {
                        r = 0;
                        if(++t == kd)
                        {
                            t = 0;
                            ch++;
                        }
                    }
                }
            }
            if(live)
                *reinterpret_cast<uint4*>(dst_row + chunk * 16) =
                    make_uint4(packed[0], packed[1], packed[2], packed[3]);
        }
    }
}

// The same matrix from a channels-last copy of the input (xt[n][z][y][x][c]) when every group has a
// multiple of 16 channels: the window elements are ordered (window plane, row, column, channel),
// so a 16-byte piece of a row is 16 consecutive channels of one input position -- one aligned
// 16-byte load and one 16-byte store per thread, neighbouring threads on neighbouring pieces.
// I: the type of the index arithmetic (32-bit when every count fits, which the launcher checks;
// the byte offsets themselves are always 64-bit)
template <class I>
__global__ __launch_bounds__(256) void im2col_cl_kernel(im2col_params p)
{
    const I pieces = (I)(p.kp / 16);
    const I plane  = (I)(p.od * p.oh * p.ow);
    const I ow = (I)p.ow, oh = (I)p.oh, group = (I)p.group, cg = (I)p.cg, kw = (I)p.kw, kh = (I)p.kh;
    const I total = (I)p.rows * group * pieces;
    const I step  = (I)gridDim.x * 256;
    for(I t = (I)blockIdx.x * 256 + threadIdx.x; t < total; t += step)
    {
        const I piece = t % pieces;
        const I rg    = t / pieces;
        const I g     = rg % group;
        const I row   = rg / group;
        const I pos   = row % plane;
        const I n     = row / plane;
        const I k     = piece * 16;
        uint4 v       = make_uint4(0, 0, 0, 0);
        if(k < (I)p.kg)
        {
            const I rq = k / cg;
            const I c0 = k % cg;
            const int64_t iz = (int64_t)(pos / (ow * oh)) * p.stride_d - p.pad_d + (int64_t)(rq / (kw * kh)) * p.dil_d;
            const int64_t iy = (int64_t)(pos / ow % oh) * p.stride_h - p.pad_h + (int64_t)(rq / kw % kh) * p.dil_h;
            const int64_t ix = (int64_t)(pos % ow) * p.stride_w - p.pad_w + (int64_t)(rq % kw) * p.dil_w;
            if(iz >= 0 && iz < p.d && iy >= 0 && iy < p.h && ix >= 0 && ix < p.w)
                v = *reinterpret_cast<const uint4*>(p.x + ((((int64_t)n * p.d + iz) * p.h + iy) * p.w + ix) * p.c +
                                                    (int64_t)g * p.cg + c0);
        }
        *reinterpret_cast<uint4*>(p.col + (((int64_t)n * p.group + g) * plane + pos) * p.kp + k) = v;
    }
}

// weights [O][Cg][KD*KH*KW] -> rows of kp bytes in (window position, channel) order, zero filled
__global__ __launch_bounds__(256) void weights_cl_kernel(
    const uint8_t* w, uint8_t* out, int64_t o, int64_t cg, int64_t win, int64_t kp)
{
    const int64_t total = o * kp;
    const int64_t step  = (int64_t)gridDim.x * 256;
    for(int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += step)
    {
        const int64_t k  = t % kp;
        const int64_t oc = t / kp;
        uint8_t v        = 0;
        if(k < cg * win)
            v = w[(oc * cg + k % cg) * win + k / cg];
        out[t] = v;
    }
}

// ---------------------------------------------------------------------------------------------
// Direct (implicit-GEMM) int8 convolution for groups with a multiple of 16 channels.
//
// The input is first copied channels-last WITH its zero padding (xt[n][z][y][x][c], the padded
// volume), so a 16-byte piece of a window row -- 16 consecutive channels of one window element
// -- is one aligned 16-byte load at (position of the output element) + (offset of the window
// element), with no bounds to check.  The main kernel is a GEMM whose rows are output positions
// (all images flattened), whose columns are a group's output channels and whose K is
// (window element, channel); its row operand is never materialised: every direct-to-LDS load
// forms its address from the row's base and the K piece's offset (a table in LDS).
//
// Workgroup: 4 waves, 128 rows x 64 output channels, K in steps of 128 bytes through a ring of
// LDS stages (16 KiB of rows + 8 KiB of weights each).  A load instruction fetches 8 rows x 128
// bytes: whole cache lines when a group has 128 channels or more (64-byte pieces of 16 rows, as a
// 64-byte K step would fetch, cost the CU's cache two line slots for one line of payload); the
// weights are stored [group][K step][channel][128 bytes] by the kernel in front, so their loads
// are 1 KiB contiguous.  A wave multiplies 32 rows by the 64 channels (2 x 4
// v_mfma_i32_16x16x64_i8 per half step, rows as the first operand, so a lane ends up with four
// consecutive output positions of one channel: 16 contiguous bytes of an NC(D)HW float result).
// LDS rows are 128 bytes as eight 16-byte chunks, logical chunk c at position c ^ ((r >> 1) & 7);
// a direct-to-LDS load writes lane l at base + 16 l, so the swizzle goes into the address a lane
// fetches.
// ---------------------------------------------------------------------------------------------
constexpr int DC_ROWS    = 128;
constexpr int DC_COLS    = 64;
constexpr int DC_KSTEP   = 128;
constexpr int DC_A_BYTES = DC_ROWS * DC_KSTEP;
constexpr int DC_STAGE   = (DC_ROWS + DC_COLS) * DC_KSTEP;
constexpr int DC_MAX_PIECES = 1024; // K pieces of 16 bytes a layer may have (the table is LDS)
constexpr int DC_PITCH   = DC_ROWS * 4 + 16; // bytes of one channel's 128 results in the LDS copy

struct direct_params
{
    const uint8_t* xt;  // padded channels-last input
    const uint8_t* wp;  // weights [group][nk][ogp][128], (window element, channel) order, zero filled
    void* out;
    const float* scale_x;
    const float* scale_w;
    int64_t rows;       // N * plane
    int plane, oh, ow;  // output positions per image; od = plane / (oh * ow)
    int o, og, ogp, c, cg;
    int kh, kw;         // kd is not needed: window element index / (kh * kw)
    int dp, hp, wp_;    // padded input volume
    int stride_d, stride_h, stride_w, dil_d, dil_h, dil_w;
    int kg, nk;         // K bytes of a group's window, K steps
    int col_tiles;      // 64-channel tiles per group
    int dequant, scale_x_mode, scale_w_mode;
    int narrow;         // pixels of 4 channels; a K piece is 4 neighbouring window columns of one window row
};

MI355_DEVINL void dc_load_to_lds(const uint8_t* g, uint8_t* l)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g),
                                     (__attribute__((address_space(3))) void*)(l), 16, 0, 0);
}

// 8 of a fragment's 16 bytes
MI355_DEVINL long dc_half(v4i f, int hi)
{
    const v2i h = hi ? v2i{f[2], f[3]} : v2i{f[0], f[1]};
    return __builtin_bit_cast(long, h);
}

template <int N>
MI355_DEVINL void dc_wait_vmcnt()
{
    __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// at most `steps` K steps of six loads may stay in flight
MI355_DEVINL void dc_wait_steps(int steps)
{
    switch(steps)
    {
    case 0: dc_wait_vmcnt<0>(); break;
    case 1: dc_wait_vmcnt<6>(); break;
    case 2: dc_wait_vmcnt<12>(); break;
    case 3: dc_wait_vmcnt<18>(); break;
    default: dc_wait_vmcnt<24>(); break;
    }
}

// one dequantized value as the GEMM's epilogue forms it: int8 through a double product, fp8 (the
// accumulator's bits are a float) as a float product
template <bool FP8>
MI355_DEVINL float dc_scaled(int32_t a, float s)
{
    if constexpr(FP8)
        return __builtin_bit_cast(float, a) * s;
    else
        return (float)((double)a * (double)s);
}

// OUT == MI355_I32 stands for the bare accumulators (int32, or the float sums of fp8 operands).
// Nontemporal stores: the workgroup's stores cover whole lines of the result, which nothing on
// this CU reads again.
template <bool FP8, int OUT>
MI355_DEVINL void dc_store4(void* out, int64_t idx, v4i a, float s)
{
    if constexpr(OUT == MI355_I32)
        __builtin_nontemporal_store(a, reinterpret_cast<v4i*>(static_cast<int32_t*>(out) + idx));
    else
    {
        float v[4];
#pragma unroll
        for(int e = 0; e < 4; e++)
            v[e] = dc_scaled<FP8>(a[e], s);
        if constexpr(OUT == MI355_F32)
            __builtin_nontemporal_store(v4f{v[0], v[1], v[2], v[3]},
                                        reinterpret_cast<v4f*>(static_cast<float*>(out) + idx));
        else if constexpr(OUT == MI355_F16)
            __builtin_nontemporal_store(
                v2i{(int)(convert_f32_to_half(v[0]) | ((uint32_t)convert_f32_to_half(v[1]) << 16)),
                    (int)(convert_f32_to_half(v[2]) | ((uint32_t)convert_f32_to_half(v[3]) << 16))},
                reinterpret_cast<v2i*>(static_cast<uint16_t*>(out) + idx));
        else
            __builtin_nontemporal_store(
                v2i{(int)convert_f32_to_bf16x2(v[0], v[1]), (int)convert_f32_to_bf16x2(v[2], v[3])},
                reinterpret_cast<v2i*>(static_cast<uint16_t*>(out) + idx));
    }
}

// FP8: e4m3fn operands on v_mfma_f32_16x16x32_fp8_fp8 (two per 64 K bytes; the lanes' K bytes are
// assigned as for int8, the same for both operands, so the sum runs over the same products in another
// order).  OUT: MI355_I32 (bare sums), MI355_F32 / F16 / BF16 (dequantized); VEC: the plane is a
// multiple of 4 positions, so a lane's four rows are one image's and their store is one aligned
// vector.  STAGES: LDS ring; the loads of K step s + STAGES go out when step s has been read.
template <bool FP8, int OUT, bool VEC, int STAGES>
__global__ __launch_bounds__(256) void conv_direct_kernel(direct_params p)
{
    static_assert(STAGES * DC_STAGE >= DC_COLS * DC_PITCH, "the result copy reuses the ring");
    static_assert(STAGES >= 2 && STAGES <= 6);
    constexpr int AHEAD = STAGES - 1;
    extern __shared__ __align__(1024) uint8_t lds[];
    int32_t* table  = reinterpret_cast<int32_t*>(lds + STAGES * DC_STAGE);
    const int lane  = threadIdx.x & 63;
    const int wave  = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g     = blockIdx.y / p.col_tiles;
    const int o0    = (blockIdx.y % p.col_tiles) * DC_COLS; // first output channel, within the group
    const int64_t row0 = (int64_t)blockIdx.x * DC_ROWS;
    const int nk    = p.nk;
    const int pieces = nk * 8;

    // byte offset of every K piece from a row's base: (window element, first channel)
    for(int q = threadIdx.x; q < pieces; q += 256)
    {
        // past the window (the zero-filled tail of the last K step): the row's first piece again,
        // times zero weights.  (An fp8 NaN there is in the true sum as well: it is the row's first
        // window element.)
        int off = 0;
        if(p.narrow)
        {
            const int kwq = (p.kw + 3) / 4;
            if(q * 16 < p.kg)
            {
                const int kxq = q % kwq;
                const int ky  = q / kwq % p.kh;
                const int kz  = q / (kwq * p.kh);
                off = ((kz * p.dil_d * p.hp + ky * p.dil_h) * p.wp_ + 4 * kxq) * 4;
            }
        }
        else if(q * 16 < p.kg)
        {
            const int tap = q * 16 / p.cg;
            const int c0  = q * 16 % p.cg;
            const int kx  = tap % p.kw;
            const int ky  = tap / p.kw % p.kh;
            const int kz  = tap / (p.kw * p.kh);
            off = ((kz * p.dil_d * p.hp + ky * p.dil_h) * p.wp_ + kx * p.dil_w) * p.c + c0;
        }
        table[q] = off;
    }
    __syncthreads();

    // ---- global -> LDS: a wave issues row blocks {wave + 4 h} (8 rows each) and weight blocks
    // {wave, wave + 4} of a K step; (r >> 1) & 7 of a lane's row only depends on the block's parity
    const int chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7); // logical chunk of this lane's position
    const uint8_t* row_base[4];
#pragma unroll
    for(int h = 0; h < 4; h++)
    {
        int64_t r = row0 + 8 * (wave + 4 * h) + (lane >> 3);
        r         = r < p.rows ? r : p.rows - 1;
        int n, pos;
        if(p.rows < ((int64_t)1 << 31))
        {
            n   = (int)((uint32_t)r / (uint32_t)p.plane);
            pos = (int)((uint32_t)r - (uint32_t)n * (uint32_t)p.plane);
        }
        else
        {
            n   = (int)(r / p.plane);
            pos = (int)(r - (int64_t)n * p.plane);
        }
        const int ox = pos % p.ow;
        const int oy = pos / p.ow % p.oh;
        const int oz = pos / (p.ow * p.oh);
        row_base[h] = p.xt + (((((int64_t)n * p.dp + oz * p.stride_d) * p.hp + oy * p.stride_h) * (int64_t)p.wp_ +
                               ox * p.stride_w) * p.c + g * p.cg);
    }
    uint32_t w_off[2];
#pragma unroll
    for(int h = 0; h < 2; h++)
        w_off[h] = (uint32_t)((o0 + 8 * (wave + 4 * h) + (lane >> 3)) * DC_KSTEP + chunk * 16);
    const uint8_t* w_base  = p.wp + (int64_t)g * nk * p.ogp * DC_KSTEP;
    const uint32_t w_step  = (uint32_t)p.ogp * DC_KSTEP;
    const uint32_t lds0    = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
    const uint32_t tab0    = lds0 + STAGES * DC_STAGE;

    auto read_offset = [&](int s, int& dst) {
        const int q = min(8 * s + chunk, pieces - 1);
        asm volatile("ds_read_b32 %0, %1" : "=v"(dst) : "v"(tab0 + 4 * q) : "memory");
    };
    auto issue = [&](int s, int off) {
        uint8_t* st        = lds + (s % STAGES) * DC_STAGE;
        const uint8_t* wgt = w_base + (int64_t)s * w_step;
#pragma unroll
        for(int h = 0; h < 4; h++)
            dc_load_to_lds(row_base[h] + off, st + (wave + 4 * h) * 1024);
#pragma unroll
        for(int h = 0; h < 2; h++)
            dc_load_to_lds(wgt + w_off[h], st + DC_A_BYTES + (wave + 4 * h) * 1024);
    };

    // ---- LDS -> operand fragments: lane l supplies row l % 16 and K bytes 16 (l / 16) .. of a half step
    const int lrow = lane & 15, lgrp = lane >> 4;
    uint32_t a_lane[2], b_lane[2];
#pragma unroll
    for(int hf = 0; hf < 2; hf++)
    {
        const uint32_t f = (uint32_t)(lrow * DC_KSTEP + (((4 * hf + lgrp) ^ ((lrow >> 1) & 7)) << 4));
        a_lane[hf]       = (uint32_t)(wave * 32 * DC_KSTEP) + f;
        b_lane[hf]       = (uint32_t)DC_A_BYTES + f;
    }

    v4i acc[2][4];
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
            acc[i][j] = v4i{0, 0, 0, 0};
    v4i fa[2][2], fb[2][4]; // [register set][tile]: set 0 holds first halves, set 1 second halves
    int off_next = 0;

    // half HF of K step s_ -> register set HF
#define DC_READ(s_, HF)                                                                                  \
    do                                                                                                   \
    {                                                                                                    \
        const uint32_t st_ = lds0 + ((s_) % STAGES) * DC_STAGE;                                          \
        asm volatile("ds_read_b128 %0, %1" : "=v"(fa[HF][0]) : "v"(st_ + a_lane[HF]) : "memory");        \
        asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(fa[HF][1]) : "v"(st_ + a_lane[HF]) : "memory"); \
        asm volatile("ds_read_b128 %0, %1" : "=v"(fb[HF][0]) : "v"(st_ + b_lane[HF]) : "memory");        \
        asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(fb[HF][1]) : "v"(st_ + b_lane[HF]) : "memory"); \
        asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fb[HF][2]) : "v"(st_ + b_lane[HF]) : "memory"); \
        asm volatile("ds_read_b128 %0, %1 offset:6144" : "=v"(fb[HF][3]) : "v"(st_ + b_lane[HF]) : "memory"); \
    } while(0)
#define DC_WAIT(HF)                                                                                      \
    asm volatile("s_waitcnt lgkmcnt(0)"                                                                  \
                 : "+v"(fa[HF][0]), "+v"(fa[HF][1]), "+v"(fb[HF][0]), "+v"(fb[HF][1]), "+v"(fb[HF][2]),  \
                   "+v"(fb[HF][3]), "+v"(off_next)                                                       \
                 :                                                                                       \
                 : "memory")
    // Inline assembly pins each accumulator to its registers (the builtin lets the compiler rename
    // them per instruction and shuffle them back at the loop head) and keeps the order reads ->
    // MFMAs -> wait.  Inside the loop an accumulator is next touched eight MFMAs later; behind the
    // loop the results are read after the wait states below.
    // fp8 goes through the builtin (its operands are halves of a fragment; every fragment is tied
    // into the wait in front, so the compiler takes them behind it).
#define DC_MFMA(HF)                                                                                      \
    _Pragma("unroll") for(int i = 0; i < 2; i++)                                                         \
        _Pragma("unroll") for(int j = 0; j < 4; j++)                                                     \
        {                                                                                                \
            if constexpr(FP8)                                                                            \
            {                                                                                            \
                v4f c_ = __builtin_bit_cast(v4f, acc[i][j]);                                             \
                c_ = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(dc_half(fa[HF][i], 0), dc_half(fb[HF][j], 0), c_, 0, 0, 0); \
                c_ = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(dc_half(fa[HF][i], 1), dc_half(fb[HF][j], 1), c_, 0, 0, 0); \
                acc[i][j] = __builtin_bit_cast(v4i, c_);                                                 \
            }                                                                                            \
            else                                                                                         \
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0"                                     \
                             : "+v"(acc[i][j])                                                           \
                             : "v"(fa[HF][i]), "v"(fb[HF][j]));                                          \
        }

    for(int t = 0; t <= AHEAD && t < nk; t++)
    {
        int off;
        read_offset(t, off);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(off)::"memory");
        issue(t, off);
    }
    read_offset(AHEAD + 1, off_next);
    dc_wait_steps(min(nk - 1, AHEAD));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    DC_READ(0, 0);
    DC_WAIT(0);
    // From a read to the wait that covers it the code is one straight line: across a branch the
    // compiler may copy a fragment to other registers, and it would do so before the data has
    // arrived (it cannot see that the read is asynchronous).  The last step therefore reads a
    // "next" first half too (the stage after it, which nothing is written to any more) and drops it.
    for(int s = 0; s < nk; s++)
    {
        DC_READ(s, 1);
        DC_MFMA(0);
        DC_WAIT(1);
        // every wave has read step s: its stage is free for step s + STAGES, once step s + 1 has landed
        dc_wait_steps(max(0, min(nk - 1, s + AHEAD) - (s + 1)));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if(s + 1 + AHEAD < nk)
            issue(s + 1 + AHEAD, off_next);
        DC_READ(s + 1, 0);
        read_offset(s + 2 + AHEAD, off_next);
        DC_MFMA(1);
        DC_WAIT(0);
    }
#undef DC_MFMA
#undef DC_WAIT
#undef DC_READ
    // a 4-pass MFMA's result may be read 7 wait states after it issued at the earliest
    asm volatile("s_nop 7\n\ts_nop 7"
                 : "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[0][2]), "+v"(acc[0][3]), "+v"(acc[1][0]),
                   "+v"(acc[1][1]), "+v"(acc[1][2]), "+v"(acc[1][3]));

    // ---- result: lane holds rows 4 (l / 16) .. + 3 of its 16-row block for channel l % 16
    const float sx = (p.dequant && p.scale_x_mode != MI355_QP_NONE) ? p.scale_x[0] : 1.f;
    auto scale_of = [&](int och) {
        float sw = 1.f;
        if(p.scale_w_mode == MI355_QP_PER_TENSOR)
            sw = p.scale_w[0];
        else if(p.scale_w_mode == MI355_QP_PER_ROW)
            sw = p.scale_w[och];
        return sw * sx;
    };
    if constexpr(VEC)
    {
        // Through LDS as [channel][128 rows]: a store instruction then writes 512 contiguous bytes
        // (float) of each of two channels instead of 64-byte pieces of sixteen.
        __syncthreads(); // every wave has read its last fragments
#pragma unroll
        for(int j = 0; j < 4; j++)
#pragma unroll
            for(int i = 0; i < 2; i++)
                *reinterpret_cast<v4i*>(lds + (16 * j + lrow) * DC_PITCH + (wave * 32 + 16 * i + 4 * lgrp) * 4) =
                    acc[i][j];
        __syncthreads();
            const int quad  = threadIdx.x & 31;
        const int64_t r = row0 + 4 * quad;
        if(r < p.rows)
        {
            const int64_t n   = r / p.plane;
            const int64_t at  = (n * p.o + (int64_t)g * p.og + o0) * p.plane + (r - n * p.plane);
            const int osub    = threadIdx.x >> 5;
            // all scales first: a load between two stores would wait for the store in front of it
            float sc[8];
#pragma unroll
            for(int it = 0; it < 8; it++)
            {
                sc[it] = 1.f;
                if constexpr(OUT != MI355_I32)
                    sc[it] = scale_of(g * p.og + min(o0 + 8 * it + osub, p.og - 1));
            }
#pragma unroll
            for(int it = 0; it < 8; it++)
            {
                const int oc = 8 * it + osub;
                if(o0 + oc < p.og)
                {
                    const v4i a = *reinterpret_cast<const v4i*>(lds + oc * DC_PITCH + quad * 16);
                    dc_store4<FP8, OUT>(p.out, at + (int64_t)oc * p.plane, a, sc[it]);
                }
            }
        }
    }
    else
    {
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            const int oc = o0 + 16 * j + lrow; // within the group
            if(oc >= p.og)
                continue;
            const int och = g * p.og + oc;
            float s       = 1.f;
            if constexpr(OUT != MI355_I32)
                s = scale_of(och);
#pragma unroll
            for(int i = 0; i < 2; i++)
            {
                const int64_t r = row0 + wave * 32 + 16 * i + 4 * lgrp;
#pragma unroll
                for(int e = 0; e < 4; e++)
                {
                    const int64_t re = r + e;
                    if(re >= p.rows)
                        break;
                    const int64_t idx = (re / p.plane * p.o + och) * p.plane + re % p.plane;
                    if constexpr(OUT == MI355_I32)
                        static_cast<int32_t*>(p.out)[idx] = acc[i][j][e];
                    else
                    {
                        const float v = dc_scaled<FP8>(acc[i][j][e], s);
                        if constexpr(OUT == MI355_F32)
                            static_cast<float*>(p.out)[idx] = v;
                        else if constexpr(OUT == MI355_F16)
                            static_cast<uint16_t*>(p.out)[idx] = convert_f32_to_half(v);
                        else
                            static_cast<uint16_t*>(p.out)[idx] = convert_f32_to_bf16(v);
                    }
                }
            }
        }
    }
}

// What runs in front of it, as one launch.  Blocks [0, tiles): the channels-last copy, 64 channels
// x 64 or 256 input positions per block through LDS (loads along the positions, which are
// contiguous per channel; 16-byte stores of 16 channels per position).  Blocks [tiles, tiles +
// border_rows): the zero borders, one row (n, z, y) of the padded volume each.  The blocks behind
// them share the reordered weights ([O][Cg][window] -> [group][K step][channel, padded to 64][128
// bytes] in (window element, channel) order, zero filled).  All counts fit 32 bits (the launcher
// checks).
struct prep_params
{
    const uint8_t* x;
    const uint8_t* w;
    uint8_t* xt;
    uint8_t* wp;
    int n, c, d, h, w_;    // input
    int cp;                // channels of the copy: c, or c rounded up to 16 (one group) with zeros behind
    int dp, hp, wp_;       // padded volume
    int pad_d, pad_h, pad_w;
    int group, og, ogp, cg, window, nk;
    int tiles_s, tiles_c;  // tiles along the positions and the channels of one image
    int tiles;             // n * tiles_c * tiles_s
    int border_rows;       // n * dp * hp, or 0 when nothing is padded
    int narrow, kh, kw;    // pixels of 4 channels (cp = 4): a K piece of the weights is 4 window columns x 4 channels
};

// PW: input positions per load, 1 (bytes) or 4 (dwords, when the volume is a multiple of 4
// positions); a tile is 64 channels x 64 PW positions
template <int PW>
__global__ __launch_bounds__(256) void conv_prep_kernel(prep_params p)
{
    constexpr int TILE_S = 64 * PW;
    __shared__ __align__(16) uint8_t tile[64][TILE_S + 4];
    const int space = p.d * p.h * p.w_;
    if(p.narrow && (int)blockIdx.x < p.tiles)
    {
        // pixels of 4 channels (at most 4 channel planes): a thread forms 4 pixels of the padded copy, zero border
        // included, from one byte per channel; a tile is 1024 pixels
        const int64_t total = (int64_t)p.n * p.dp * p.hp * p.wp_;
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            const int64_t px = ((int64_t)blockIdx.x * 4 + j) * 256 + threadIdx.x;
            if(px >= total)
                break;
            const int ix = (int)(px % p.wp_) - p.pad_w;
            int64_t r    = px / p.wp_;
            const int iy = (int)(r % p.hp) - p.pad_h;
            r /= p.hp;
            const int iz = (int)(r % p.dp) - p.pad_d;
            const int n  = (int)(r / p.dp);
            uint32_t v   = 0;
            if(ix >= 0 && ix < p.w_ && iy >= 0 && iy < p.h && iz >= 0 && iz < p.d)
            {
                const uint8_t* src = p.x + (int64_t)n * p.c * space + (iz * p.h + iy) * p.w_ + ix;
#pragma unroll
                for(int e = 0; e < 4; e++)
                    if(e < p.c)
                        v |= (uint32_t)src[(int64_t)e * space] << (8 * e);
            }
            __builtin_nontemporal_store(v, reinterpret_cast<uint32_t*>(p.xt + px * 4));
        }
        return;
    }
    if((int)blockIdx.x < p.tiles)
    {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int t    = blockIdx.x;
        const int ts   = t % p.tiles_s;
        const int tc   = t / p.tiles_s % p.tiles_c;
        const int n    = t / (p.tiles_s * p.tiles_c);
        const int s    = ts * TILE_S + lane * PW;
        const int c0   = tc * 64;
        // all 16 loads first, so that they are in flight together
        uint32_t v[16];
#pragma unroll
        for(int i = 0; i < 16; i++)
        {
            const int ch = c0 + 16 * wave + i;
            v[i]         = 0;
            if(ch < p.c && s < space)
            {
                const uint8_t* src = p.x + ((int64_t)n * p.c + ch) * space + s;
                if constexpr(PW == 4)
                    v[i] = *reinterpret_cast<const uint32_t*>(src);
                else
                    v[i] = *src;
            }
        }
#pragma unroll
        for(int i = 0; i < 16; i++)
        {
            if constexpr(PW == 4)
                *reinterpret_cast<uint32_t*>(&tile[16 * wave + i][4 * lane]) = v[i];
            else
                tile[16 * wave + i][lane] = (uint8_t)v[i];
        }
        __syncthreads();
        // a thread gathers the 16 channels of one piece at one position; the four pieces of 16
        // neighbouring positions make a wave's store 1 KiB contiguous when C = 64
        const int piece = threadIdx.x & 3;
        if(c0 + 16 * piece >= p.cp)
            return;
#pragma unroll
        for(int q = 0; q < PW; q++)
        {
            const int sl = 64 * q + (threadIdx.x >> 2);
            const int so = ts * TILE_S + sl;
            if(so >= space)
                continue;
            uint32_t packed[4] = {0, 0, 0, 0};
            if constexpr(PW == 4)
            {
                // byte (sl & 3) of 16 dwords; selector bytes 0x0c give zero
                const uint32_t b   = sl & 3;
                const uint32_t sel = 0x0c0c0000u | ((4 + b) << 8) | b;
#pragma unroll
                for(int j = 0; j < 4; j++)
                {
                    const uint32_t r0 = *reinterpret_cast<const uint32_t*>(&tile[16 * piece + 4 * j + 0][sl & ~3]);
                    const uint32_t r1 = *reinterpret_cast<const uint32_t*>(&tile[16 * piece + 4 * j + 1][sl & ~3]);
                    const uint32_t r2 = *reinterpret_cast<const uint32_t*>(&tile[16 * piece + 4 * j + 2][sl & ~3]);
                    const uint32_t r3 = *reinterpret_cast<const uint32_t*>(&tile[16 * piece + 4 * j + 3][sl & ~3]);
                    const uint32_t lo = __builtin_amdgcn_perm(r1, r0, sel);
                    const uint32_t hi = __builtin_amdgcn_perm(r3, r2, sel);
                    packed[j]         = lo | (hi << 16);
                }
            }
            else
            {
#pragma unroll
                for(int e = 0; e < 16; e++)
                    packed[e / 4] |= (uint32_t)tile[16 * piece + e][sl] << (8 * (e % 4));
            }
            const int ix = so % p.w_;
            const int iy = so / p.w_ % p.h;
            const int iz = so / (p.w_ * p.h);
            const int64_t at =
                ((((int64_t)n * p.dp + iz + p.pad_d) * p.hp + iy + p.pad_h) * (int64_t)p.wp_ + ix + p.pad_w) * p.cp + c0 +
                16 * piece;
            __builtin_nontemporal_store(v4u{packed[0], packed[1], packed[2], packed[3]}, reinterpret_cast<v4u*>(p.xt + at));
        }
        return;
    }
    const int cp = p.cp / 16;
    if((int)blockIdx.x < p.tiles + p.border_rows)
    {
        const int row = blockIdx.x - p.tiles;
        const int y   = row % p.hp - p.pad_h;
        const int z   = row / p.hp % p.dp - p.pad_d;
        uint8_t* dst  = p.xt + (int64_t)row * p.wp_ * p.cp;
        const bool whole = y < 0 || y >= p.h || z < 0 || z >= p.d;
        for(int t = threadIdx.x; t < p.wp_ * cp; t += 256)
        {
            const int x = t / cp - p.pad_w;
            if(whole || x < 0 || x >= p.w_)
                __builtin_nontemporal_store(v4u{0, 0, 0, 0}, reinterpret_cast<v4u*>(dst + (int64_t)t * 16));
        }
        return;
    }
    // weights: a thread fills 16 bytes of K for one channel
    const int first    = p.tiles + p.border_rows;
    const int nthreads = ((int)gridDim.x - first) * 256;
    const int total    = p.group * p.nk * p.ogp * (DC_KSTEP / 16);
    const int cgp      = p.group == 1 ? p.cp : p.cg; // a group's channels in the copy
    const int kg       = cgp * p.window;
    for(int t = ((int)blockIdx.x - first) * 256 + threadIdx.x; t < total; t += nthreads)
    {
        const int k0 = t % (DC_KSTEP / 16) * 16;
        const int oc = t / (DC_KSTEP / 16) % p.ogp;
        const int s  = t / (DC_KSTEP / 16) / p.ogp % p.nk;
        const int g  = t / (DC_KSTEP / 16) / p.ogp / p.nk;
        uint32_t packed[4] = {0, 0, 0, 0};
        const int k  = s * DC_KSTEP + k0;
        if(p.narrow)
        {
            const int kwq = (p.kw + 3) / 4;
            const int q   = k / 16;
            if(oc < p.og && q < p.window / p.kw * kwq)
            {
                const int kxq      = q % kwq;
                const int rowk     = q / kwq; // (kz, ky)
                const uint8_t* src = p.w + (int64_t)oc * p.cg * p.window + rowk * p.kw;
#pragma unroll
                for(int e = 0; e < 16; e++)
                {
                    const int kx = 4 * kxq + e / 4, ch = e % 4;
                    if(kx < p.kw && ch < p.cg)
                        packed[e / 4] |= (uint32_t)src[(int64_t)ch * p.window + kx] << (8 * (e % 4));
                }
            }
        }
        else if(oc < p.og && k < kg)
        {
            // the 16 bytes are 16 consecutive channels of one window element (zeros for the channels
            // the copy adds)
            const int tap      = k / cgp;
            const int c0       = k % cgp;
            const uint8_t* src = p.w + (((int64_t)g * p.og + oc) * p.cg + c0) * p.window + tap;
#pragma unroll
            for(int e = 0; e < 16; e++)
                if(c0 + e < p.cg)
                    packed[e / 4] |= (uint32_t)src[(int64_t)e * p.window] << (8 * (e % 4));
        }
        *reinterpret_cast<uint4*>(p.wp + (int64_t)t * 16) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    }
}

// ---------------------------------------------------------------------------------------------
// Many groups of a few channels each (depthwise layers: one channel per group).  A GEMM per group
// would be a launch per group with K of a few bytes; here a thread computes one output element
// from its C/G x window products (the input read along x, coalesced; a group's weights are a few
// bytes that stay in the cache), in int32 / float, and applies the dequantizing epilogue.
// ---------------------------------------------------------------------------------------------
struct small_params
{
    const uint8_t* x;
    const uint8_t* w;
    void* out;
    const float* scale_x;
    const float* scale_w;
    int64_t total; // N * O * plane
    int64_t items; // work items: outputs, or groups of four outputs along x
    int c, d, h, w_;
    int o, og, cg;
    int kd, kh, kw, od, oh, ow;
    int pad_d, pad_h, pad_w, stride_d, stride_h, stride_w, dil_d, dil_h, dil_w;
    int dequant, scale_x_mode, scale_w_mode;
};

// I: the type of the work index (32-bit when every count fits, which the launcher checks).
// ROW4: unit stride and dilation along x and a window of at most 4 columns: a thread computes four
// neighbouring outputs of a row from one segment of 4 + kw - 1 input bytes per window row -- the
// kernel is bound by the number of load instructions, and this needs 7 instead of 18 per output
// for a depthwise 3 x 3.
template <bool FP8, int OUT, class I, bool ROW4>
__global__ __launch_bounds__(256) void conv_small_groups_kernel(small_params p)
{
    constexpr int NQ  = ROW4 ? 4 : 1;
    const I step      = (I)gridDim.x * 256;
    const int owq     = (p.ow + NQ - 1) / NQ;
    const int planeq  = p.od * p.oh * owq;
    const int plane   = p.od * p.oh * p.ow;
    const int space   = p.d * p.h * p.w_; // below 2^30 (checked by the entry point)
    const int window  = p.kd * p.kh * p.kw;
    const float sx    = (p.dequant && p.scale_x_mode != MI355_QP_NONE) ? p.scale_x[0] : 1.f;
    for(I t = (I)blockIdx.x * 256 + threadIdx.x; t < (I)p.items; t += step)
    {
        const int posq = (int)(t % (I)planeq);
        const I r      = t / (I)planeq;
        const int oc   = (int)(r % (I)p.o);
        const int64_t n = (int64_t)(r / (I)p.o);
        const int ox0 = posq % owq * NQ, oy = posq / owq % p.oh, oz = posq / (owq * p.oh);
        const int g   = oc / p.og;
        const uint8_t* xg = p.x + (n * p.c + (int64_t)g * p.cg) * (int64_t)space;
        const uint8_t* wo = p.w + (int64_t)oc * p.cg * window;
        int32_t acc_i[NQ];
        float acc_f[NQ];
#pragma unroll
        for(int q = 0; q < NQ; q++)
        {
            acc_i[q] = 0;
            acc_f[q] = 0.f;
        }
        auto add = [&](int q, uint8_t xv, uint8_t wv, bool valid) {
            if constexpr(FP8)
                acc_f[q] += valid ? __builtin_amdgcn_cvt_f32_fp8(xv, 0) * __builtin_amdgcn_cvt_f32_fp8(wv, 0) : 0.f;
            else
                acc_i[q] += valid ? (int32_t)(int8_t)xv * (int32_t)(int8_t)wv : 0;
        };
        for(int c = 0; c < p.cg; c++)
            for(int kz = 0; kz < p.kd; kz++)
            {
                const int iz = oz * p.stride_d - p.pad_d + kz * p.dil_d;
                if(iz < 0 || iz >= p.d)
                    continue;
                for(int ky = 0; ky < p.kh; ky++)
                {
                    const int iy = oy * p.stride_h - p.pad_h + ky * p.dil_h;
                    if(iy < 0 || iy >= p.h)
                        continue;
                    const uint8_t* row = xg + (int64_t)c * space + (iz * p.h + iy) * p.w_;
                    const uint8_t* wr  = wo + ((c * p.kd + kz) * p.kh + ky) * p.kw;
                    if constexpr(ROW4)
                    {
                        const int ix0 = ox0 - p.pad_w;
                        uint8_t seg[7];
                        bool ok[7];
#pragma unroll
                        for(int j = 0; j < 7; j++)
                        {
                            const int ix = ix0 + j;
                            ok[j]        = j < 3 + p.kw && ix >= 0 && ix < p.w_;
                            seg[j]       = ok[j] ? row[ix] : (uint8_t)0;
                        }
#pragma unroll
                        for(int kx = 0; kx < 4; kx++)
                        {
                            if(kx < p.kw)
                            {
                                const uint8_t wv = wr[kx];
#pragma unroll
                                for(int q = 0; q < 4; q++)
                                    add(q, seg[q + kx], wv, ok[q + kx]);
                            }
                        }
                    }
                    else
                    {
                        for(int kx = 0; kx < p.kw; kx++)
                        {
                            const int ix = ox0 * p.stride_w - p.pad_w + kx * p.dil_w;
                            if(ix >= 0 && ix < p.w_)
                                add(0, row[ix], wr[kx], true);
                        }
                    }
                }
            }
        float s = 1.f;
        if constexpr(OUT != MI355_I32)
        {
            float sw = 1.f;
            if(p.scale_w_mode == MI355_QP_PER_TENSOR)
                sw = p.scale_w[0];
            else if(p.scale_w_mode == MI355_QP_PER_ROW)
                sw = p.scale_w[oc];
            s = sw * sx;
        }
        const int64_t at = ((int64_t)n * p.o + oc) * plane + (oz * p.oh + oy) * p.ow + ox0;
#pragma unroll
        for(int q = 0; q < NQ; q++)
        {
            if(ox0 + q >= p.ow)
                break;
            if constexpr(OUT == MI355_I32)
            {
                // the bare sums: int32, or float for fp8 operands
                if constexpr(FP8)
                    static_cast<float*>(p.out)[at + q] = acc_f[q];
                else
                    static_cast<int32_t*>(p.out)[at + q] = acc_i[q];
            }
            else
            {
                const float v = FP8 ? acc_f[q] * s : (float)((double)acc_i[q] * (double)s);
                if constexpr(OUT == MI355_F32)
                    static_cast<float*>(p.out)[at + q] = v;
                else if constexpr(OUT == MI355_F16)
                    static_cast<uint16_t*>(p.out)[at + q] = convert_f32_to_half(v);
                else
                    static_cast<uint16_t*>(p.out)[at + q] = convert_f32_to_bf16(v);
            }
        }
    }
}

// Depthwise layers over images (one input channel per group, unit stride and dilation along x, at
// most 4 window columns, at most 4 columns of padding on the left): a workgroup stages the input
// rows that `th` output rows of one (image, output channel) need in LDS, zero border included, and
// the window in front of them; a thread then computes four neighbouring outputs of a row from three
// aligned LDS dwords per window row.  The one-output-per-thread form is bound by the number of
// global byte loads (16 cycles of the address unit each); here a plane is fetched once, in dwords
// where the rows are dword aligned (DW).
// LDS: 64 bytes of window, then rows of `pitch` bytes; input column ix lies at byte 4 + ix.
template <bool FP8, int OUT, bool DW>
__global__ __launch_bounds__(256) void conv_depthwise_rows_kernel(small_params p, int th, int chunks, int pitch)
{
    extern __shared__ uint32_t dw_lds[];
    uint8_t* wl        = reinterpret_cast<uint8_t*>(dw_lds);
    uint32_t* tile32   = dw_lds + 16;
    uint8_t* tile      = reinterpret_cast<uint8_t*>(tile32);
    const int tid      = threadIdx.x;
    const int nt       = blockDim.x; // 64, 128 or 256: a small plane takes one wave, and all of a layer's are resident at once
    const int chunk    = blockIdx.x % chunks;
    const int64_t noc  = blockIdx.x / chunks;
    const int oc       = (int)(noc % p.o);
    const int64_t n    = noc / p.o;
    const int c        = oc / p.og;
    const int window   = p.kh * p.kw;
    const int oy0      = chunk * th;
    const int nrows    = p.oh - oy0 < th ? p.oh - oy0 : th;
    const int iy_base  = oy0 * p.stride_h - p.pad_h;
    const int rows_in  = (nrows - 1) * p.stride_h + (p.kh - 1) * p.dil_h + 1;
    const int pitch4   = pitch / 4;
    for(int i = tid; i < rows_in * pitch4; i += nt)
        tile32[i] = 0;
    if(tid < window)
        wl[tid] = p.w[(int64_t)oc * window + tid];
    __syncthreads();
    const uint8_t* xp = p.x + (n * p.c + c) * (int64_t)(p.h * p.w_);
    if constexpr(DW)
    {
        const int wq = p.w_ / 4;
        for(int i = tid; i < rows_in * wq; i += nt)
        {
            const int r = i / wq, q = i - r * wq, iy = iy_base + r;
            if(iy >= 0 && iy < p.h)
                tile32[r * pitch4 + 1 + q] = reinterpret_cast<const uint32_t*>(xp)[iy * wq + q];
        }
    }
    else
    {
        for(int i = tid; i < rows_in * p.w_; i += nt)
        {
            const int r = i / p.w_, ix = i - r * p.w_, iy = iy_base + r;
            if(iy >= 0 && iy < p.h)
                tile[r * pitch + 4 + ix] = xp[iy * p.w_ + ix];
        }
    }
    __syncthreads();

    const int owq     = (p.ow + 3) / 4;
    const int first   = p.pad_w == 0 ? 1 : 0;  // dword of a row that holds column 4 q - pad_w, minus q
    const int shift   = (4 - p.pad_w) & 3;     // and that column's byte in it
    const float sx    = (p.dequant && p.scale_x_mode != MI355_QP_NONE) ? p.scale_x[0] : 1.f;
    float s           = 1.f;
    if constexpr(OUT != MI355_I32)
    {
        float sw = 1.f;
        if(p.scale_w_mode == MI355_QP_PER_TENSOR)
            sw = p.scale_w[0];
        else if(p.scale_w_mode == MI355_QP_PER_ROW)
            sw = p.scale_w[oc];
        s = sw * sx;
    }
    const bool vec = p.ow % 4 == 0 && reinterpret_cast<uintptr_t>(p.out) % 16 == 0;
    for(int it = tid; it < nrows * owq; it += nt)
    {
        const int ry = it / owq, q = it - ry * owq;
        int32_t acc_i[4] = {0, 0, 0, 0};
        float acc_f[4]   = {0.f, 0.f, 0.f, 0.f};
        // columns outside the image hold zeros; an fp8 product with them is left out all the same (a NaN weight)
        bool okx[7];
#pragma unroll
        for(int j = 0; j < 7; j++)
            okx[j] = 4 * q - p.pad_w + j >= 0 && 4 * q - p.pad_w + j < p.w_;
        for(int ky = 0; ky < p.kh; ky++)
        {
            const int r         = ry * p.stride_h + ky * p.dil_h;
            const uint32_t* row = tile32 + r * pitch4 + q + first;
            const uint32_t d0 = row[0], d1 = row[1], d2 = row[2];
            const uint32_t lo = __builtin_amdgcn_alignbyte(d1, d0, shift);
            const uint32_t hi = __builtin_amdgcn_alignbyte(d2, d1, shift);
            const bool oky    = iy_base + r >= 0 && iy_base + r < p.h;
#pragma unroll
            for(int kx = 0; kx < 4; kx++)
            {
                if(kx < p.kw)
                {
                    const uint8_t wv = wl[ky * p.kw + kx];
#pragma unroll
                    for(int o4 = 0; o4 < 4; o4++)
                    {
                        const int j       = o4 + kx;
                        const uint32_t xb = ((j < 4 ? lo : hi) >> (8 * (j & 3))) & 0xffu;
                        if constexpr(FP8)
                            acc_f[o4] += (okx[j] && oky) ? __builtin_amdgcn_cvt_f32_fp8(xb, 0) * __builtin_amdgcn_cvt_f32_fp8(wv, 0) : 0.f;
                        else
                            acc_i[o4] += (int32_t)(int8_t)xb * (int32_t)(int8_t)wv;
                    }
                }
            }
        }
        const int64_t at = (noc * p.oh + oy0 + ry) * (int64_t)p.ow + 4 * q;
        float v[4];
#pragma unroll
        for(int o4 = 0; o4 < 4; o4++)
            v[o4] = FP8 ? (OUT == MI355_I32 ? acc_f[o4] : acc_f[o4] * s) : (float)((double)acc_i[o4] * (double)s);
        if constexpr(OUT == MI355_I32 || OUT == MI355_F32)
        {
            if(vec)
            {
                if constexpr(OUT == MI355_I32 && !FP8)
                    *reinterpret_cast<v4i*>(static_cast<int32_t*>(p.out) + at) = v4i{acc_i[0], acc_i[1], acc_i[2], acc_i[3]};
                else
                    *reinterpret_cast<v4f*>(static_cast<float*>(p.out) + at) = v4f{v[0], v[1], v[2], v[3]};
                continue;
            }
        }
#pragma unroll
        for(int o4 = 0; o4 < 4; o4++)
        {
            if(4 * q + o4 >= p.ow)
                break;
            if constexpr(OUT == MI355_I32 && !FP8)
                static_cast<int32_t*>(p.out)[at + o4] = acc_i[o4];
            else if constexpr(OUT == MI355_I32 || OUT == MI355_F32)
                static_cast<float*>(p.out)[at + o4] = v[o4];
            else if constexpr(OUT == MI355_F16)
                static_cast<uint16_t*>(p.out)[at + o4] = convert_f32_to_half(v[o4]);
            else
                static_cast<uint16_t*>(p.out)[at + o4] = convert_f32_to_bf16(v[o4]);
        }
    }
}

// rows of output per workgroup of the kernel above (0: not its form), and its LDS
int depthwise_rows(const small_params& p, int* chunks, int* pitch, size_t* lds)
{
    if(p.cg != 1 || p.kd != 1 || p.d != 1 || p.od != 1 || p.pad_d != 0 || p.stride_w != 1 || p.dil_w != 1 || p.kw > 4 ||
       p.pad_w > 4 || p.kh * p.kw > 64)
        return 0;
    const int owq = (p.ow + 3) / 4;
    *pitch        = 4 * (owq + 3);
    if(4 + p.w_ > *pitch) // (cannot be with unit stride and dilation; the staging loop relies on it)
        return 0;
    const int64_t halo    = (int64_t)(p.kh - 1) * p.dil_h + 1;
    const int64_t rows_in = (32768 - 64) / *pitch;
    if(rows_in < halo)
        return 0;
    int64_t th = (rows_in - halo) / p.stride_h + 1;
    // about four work items per thread at most, so that large planes give several workgroups
    const int64_t few = (1024 + owq - 1) / owq;
    th                = th > few ? few : th;
    th                = th > p.oh ? p.oh : th;
    *chunks           = (int)((p.oh + th - 1) / th);
    th                = (p.oh + *chunks - 1) / *chunks; // chunks of equal size
    if((int64_t)p.total / p.ow / p.oh * *chunks >= ((int64_t)1 << 31))
        return 0;
    *lds = 64 + (size_t)(((th - 1) * p.stride_h + halo) * *pitch);
    return (int)th;
}

template <bool FP8, int OUT>
bool launch_depthwise_rows(const small_params& p, hipStream_t hs)
{
    int chunks = 0, pitch = 0;
    size_t lds = 0;
    const int th = depthwise_rows(p, &chunks, &pitch, &lds);
    if(th == 0)
        return false;
    const int64_t items = (int64_t)th * ((p.ow + 3) / 4);
    const dim3 grid((unsigned)(p.total / p.ow / p.oh * chunks)), block(items <= 256 ? 64 : items <= 512 ? 128 : 256);
    if(p.w_ % 4 == 0 && reinterpret_cast<uintptr_t>(p.x) % 4 == 0)
        hipLaunchKernelGGL((conv_depthwise_rows_kernel<FP8, OUT, true>), grid, block, lds, hs, p, th, chunks, pitch);
    else
        hipLaunchKernelGGL((conv_depthwise_rows_kernel<FP8, OUT, false>), grid, block, lds, hs, p, th, chunks, pitch);
    return true;
}

template <bool FP8, int OUT>
void launch_small_groups_as(small_params p, hipStream_t hs)
{
    if(launch_depthwise_rows<FP8, OUT>(p, hs))
        return;
    const bool row4 = p.stride_w == 1 && p.dil_w == 1 && p.kw <= 4;
    p.items         = p.total / p.ow * ((p.ow + (row4 ? 3 : 0)) / (row4 ? 4 : 1));
    int64_t blocks  = (p.items + 255) / 256;
    blocks          = blocks > 256 * 64 ? 256 * 64 : blocks;
    const dim3 grid((unsigned)blocks), block(256);
    const bool small = p.items + blocks * 256 < ((int64_t)1 << 32);
    if(row4)
    {
        if(small)
            hipLaunchKernelGGL((conv_small_groups_kernel<FP8, OUT, uint32_t, true>), grid, block, 0, hs, p);
        else
            hipLaunchKernelGGL((conv_small_groups_kernel<FP8, OUT, int64_t, true>), grid, block, 0, hs, p);
    }
    else if(small)
        hipLaunchKernelGGL((conv_small_groups_kernel<FP8, OUT, uint32_t, false>), grid, block, 0, hs, p);
    else
        hipLaunchKernelGGL((conv_small_groups_kernel<FP8, OUT, int64_t, false>), grid, block, 0, hs, p);
}

template <bool FP8>
void launch_small_groups(const small_params& p, bool dequant, int out_type, hipStream_t hs)
{
    if(!dequant)
        launch_small_groups_as<FP8, MI355_I32>(p, hs);
    else if(out_type == MI355_F32)
        launch_small_groups_as<FP8, MI355_F32>(p, hs);
    else if(out_type == MI355_F16)
        launch_small_groups_as<FP8, MI355_F16>(p, hs);
    else
        launch_small_groups_as<FP8, MI355_BF16>(p, hs);
}

// several groups of few channels each (and not the direct kernel's form): the vector-ALU kernel above
bool small_groups_form(const mi355_quant_conv3d_desc* d)
{
    const int64_t cg = d->c / d->group;
    return d->group > 1 && cg % 16 != 0 && cg * d->kd * d->kh * d->kw <= 256;
}

int64_t out_len(int64_t in, int64_t k, int64_t pad_lo, int64_t pad_hi, int64_t stride, int64_t dil)
{
    const int64_t span = in - (1 + dil * (k - 1)) + pad_lo + pad_hi;
    const int64_t v    = span / stride + 1; // truncating division, as the reference's shape rule
    return v < 1 ? 1 : v;
}

bool valid(const mi355_quant_conv3d_desc* d)
{
    if(d == nullptr)
        return false;
    if(d->n < 0 || d->c < 1 || d->d < 1 || d->h < 1 || d->w < 1 || d->o < 1 || d->kd < 1 || d->kh < 1 || d->kw < 1)
        return false;
    for(int i = 0; i < 3; i++)
    {
        if(d->pad[i] < 0 || d->pad_hi[i] < 0 || d->stride[i] < 1 || d->dil[i] < 1)
            return false;
    }
    if(d->group < 1 || d->c % d->group != 0 || d->o % d->group != 0)
        return false;
    return d->in_type == MI355_I8 || d->in_type == MI355_FP8;
}

void launch_im2col(const im2col_params& p, hipStream_t stream)
{
    int64_t blocks = (p.rows + 63) / 64;
    if(blocks > 65535 * 16)
        blocks = 65535 * 16;
    const int64_t chunk_blocks = (p.kp / 16 + 3) / 4;
    hipLaunchKernelGGL(im2col_kernel, dim3((unsigned)blocks, (unsigned)p.group, (unsigned)chunk_blocks), dim3(256),
                       0, stream, p);
}

// [rows][k] -> rows of kp bytes, zero filled: the window kernel with a window of one element
im2col_params copy_rows(const uint8_t* src, uint8_t* dst, int64_t rows, int64_t k, int64_t kp)
{
    im2col_params t{};
    t.x = src;
    t.col = dst;
    t.rows = rows;
    t.c = t.cg = t.kg = k;
    t.d = t.h = t.w = 1;
    t.kd = t.kh = t.kw = 1;
    t.od = t.oh = t.ow = 1;
    t.stride_d = t.stride_h = t.stride_w = 1;
    t.dil_d = t.dil_h = t.dil_w = 1;
    t.group = 1;
    t.kp = kp;
    return t;
}

// the batched GEMM of one group: weights [O/G, Kp] times the group's window matrix [P, Kp]^T per image
mi355_quant_dot_desc gemm_of(const mi355_quant_conv3d_desc* d, int64_t plane, int64_t kp)
{
    mi355_quant_dot_desc g{};
    g.m            = d->o / d->group;
    g.n            = plane;
    g.k            = kp;
    g.lda          = kp;
    g.ldb          = kp;
    g.ldc          = plane;
    g.batch        = d->n;
    g.stride_a     = 0;
    g.stride_b     = d->group * plane * kp;
    g.stride_c     = d->o * plane;
    g.trans_a      = 0;
    g.trans_b      = 1;
    g.in_type      = d->in_type;
    g.out_type     = d->out_type;
    g.dequant      = d->dequant;
    // the weights are the GEMM's first operand: one scale per output channel is one per row
    g.scale_a_mode = d->dequant ? d->scale_w_mode : MI355_QP_NONE;
    g.scale_b_mode = d->dequant ? d->scale_x_mode : MI355_QP_NONE;
    return g;
}

// window matrix + reordered weights + channels-last copy, rounded up so that what follows (room for
// the GEMM's split-K partial sums) is 16-byte aligned
size_t staging_bytes(const mi355_quant_conv3d_desc* d, int64_t plane, int64_t kp)
{
    const size_t b = (size_t)((d->n * d->group * plane + d->o) * kp + d->n * d->c * d->d * d->h * d->w);
    return (b + 15) / 16 * 16;
}

// A group's channels in the direct kernel's copy of the input: with one group, any channel count
// is rounded up to 16 (the copy and the reordered weights hold zeros there)
// One group of at most 4 channels with several window columns (an image network's first layer), int8:
// pixels of 4 channels, and a K piece of 16 bytes is 4 neighbouring window columns of a window row (unit
// dilation along x) -- 16 x kd x kh x ceil(kw / 4) bytes of K per output instead of 16 x kd x kh x kw.
// (Not for fp8: a piece reaches up to 3 pixels past the window, whose zero weights would not silence a NaN.)
bool direct_narrow(const mi355_quant_conv3d_desc* d)
{
    return d->group == 1 && d->c <= 4 && d->kw >= 2 && d->dil[2] == 1 && d->in_type == MI355_I8;
}

int64_t direct_cgp(const mi355_quant_conv3d_desc* d)
{
    const int64_t cg = d->c / d->group;
    if(direct_narrow(d))
        return 4;
    return d->group == 1 ? (cg + 15) / 16 * 16 : cg;
}

// K steps and padded channel count of the direct kernel's weights
int64_t direct_steps(const mi355_quant_conv3d_desc* d)
{
    if(direct_narrow(d))
        return (16 * d->kd * d->kh * ((d->kw + 3) / 4) + DC_KSTEP - 1) / DC_KSTEP;
    return (direct_cgp(d) * d->kd * d->kh * d->kw + DC_KSTEP - 1) / DC_KSTEP;
}
int64_t direct_ogp(const mi355_quant_conv3d_desc* d)
{
    return (d->o / d->group + DC_COLS - 1) / DC_COLS * DC_COLS;
}

// The direct kernel's form of a layer: one group, or every group a multiple of 16 channels; every
// window inside the padded volume, counts that fit the kernels' 32-bit indices.
// fp8 layers with padding are taken like any other.  The kernel multiplies the zero border of the
// padded copy by the weights, where the reference (op/convolution.hpp:84-92) leaves window elements
// outside the image out of the sum: the same number unless a weight is NaN, which then reaches the
// border outputs as well (0 * NaN); the gathered form does the same, the vector-ALU forms mask.
bool direct_form(const mi355_quant_conv3d_desc* d, const int64_t* ol)
{
    const int64_t lim    = (int64_t)1 << 31;
    const int64_t window = d->kd * d->kh * d->kw;
    // a window of one element with unit strides is served better by the GEMM itself (the pointwise
    // form of mi355_quant_convolution3d, or the gathered form for odd sizes); with strides the
    // direct kernel's addressing does the subsampling
    if((direct_cgp(d) % 16 != 0 && !direct_narrow(d)) || (window <= 1 && d->stride[0] == 1 && d->stride[1] == 1 && d->stride[2] == 1))
        return false;
    const int64_t in[3]  = {d->d, d->h, d->w};
    const int64_t win[3] = {d->kd, d->kh, d->kw};
    const int64_t cp     = direct_cgp(d) * d->group;
    int64_t volume       = cp;
    for(int i = 0; i < 3; i++)
    {
        const int64_t padded = in[i] + d->pad[i] + d->pad_hi[i];
        if((ol[i] - 1) * d->stride[i] + d->dil[i] * (win[i] - 1) + 1 > padded)
            return false;
        volume *= padded;
        if(volume >= lim)
            return false;
    }
    if(d->n * (volume / cp) >= lim || d->n * d->c >= lim) // padded positions; channel planes
        return false;
    const int64_t nk = direct_steps(d);
    if(nk * 8 > DC_MAX_PIECES)
        return false;
    if(direct_ogp(d) / DC_COLS * d->group > 65535 || d->group * nk * direct_ogp(d) * (DC_KSTEP / 16) >= lim)
        return false;
    // a handful of workgroups with a long K each (one image of a deep 7x7 layer: 8 workgroups x 36
    // steps) is what the GEMM's split of K over the chip is for
    const int64_t plane      = ol[0] * ol[1] * ol[2];
    const int64_t workgroups = (d->n * plane + DC_ROWS - 1) / DC_ROWS * (direct_ogp(d) / DC_COLS) * d->group;
    return !(workgroups < 32 && nk >= 24);
}

// reordered weights + padded channels-last copy
size_t direct_bytes(const mi355_quant_conv3d_desc* d)
{
    return (size_t)(d->group * direct_steps(d) * direct_ogp(d) * DC_KSTEP +
                    d->n * direct_cgp(d) * d->group * (d->d + d->pad[0] + d->pad_hi[0]) * (d->h + d->pad[1] + d->pad_hi[1]) *
                        (d->w + d->pad[2] + d->pad_hi[2]) +
                    16); // (a narrow layer's last piece reaches up to 3 pixels past the copy's end)
}

template <bool FP8, int OUT, bool VEC, int STAGES>
void launch_direct_as(const direct_params& p, dim3 grid, hipStream_t hs)
{
    // ring + offset table; may be above the 64 KiB default: opt in once per instantiation
    auto kern = conv_direct_kernel<FP8, OUT, VEC, STAGES>;
    static const hipError_t attr =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            STAGES * DC_STAGE + DC_MAX_PIECES * 4);
    (void)attr;
    hipLaunchKernelGGL(kern, grid, dim3(256), STAGES * DC_STAGE + p.nk * 8 * 4, hs, p);
}

// The ring is as deep as the workgroups a CU gets at a time allow (160 KiB of LDS per CU): one
// workgroup has to hide its load latency itself, three hide each other's.
template <bool FP8, int OUT, bool VEC>
void launch_direct_vec(const direct_params& p, dim3 grid, hipStream_t hs)
{
    const int64_t per_cu = ((int64_t)grid.x * grid.y + 255) / 256;
    if(per_cu <= 1)
        launch_direct_as<FP8, OUT, VEC, 6>(p, grid, hs);
    else if(per_cu == 2)
        launch_direct_as<FP8, OUT, VEC, 3>(p, grid, hs);
    else
        launch_direct_as<FP8, OUT, VEC, 2>(p, grid, hs);
}

template <bool FP8>
void launch_direct(const direct_params& p, bool dequant, int out_type, bool vec, dim3 grid, hipStream_t hs)
{
    if(!dequant)
        vec ? launch_direct_vec<FP8, MI355_I32, true>(p, grid, hs) : launch_direct_vec<FP8, MI355_I32, false>(p, grid, hs);
    else if(out_type == MI355_F32)
        vec ? launch_direct_vec<FP8, MI355_F32, true>(p, grid, hs) : launch_direct_vec<FP8, MI355_F32, false>(p, grid, hs);
    else if(out_type == MI355_F16)
        vec ? launch_direct_vec<FP8, MI355_F16, true>(p, grid, hs) : launch_direct_vec<FP8, MI355_F16, false>(p, grid, hs);
    else
        vec ? launch_direct_vec<FP8, MI355_BF16, true>(p, grid, hs) : launch_direct_vec<FP8, MI355_BF16, false>(p, grid, hs);
}

// a depth of one in front of the two-dimensional description
mi355_quant_conv3d_desc with_unit_depth(const mi355_quant_conv_desc* d)
{
    mi355_quant_conv3d_desc v{};
    v.n = d->n, v.c = d->c, v.d = 1, v.h = d->h, v.w = d->w;
    v.o = d->o, v.kd = 1, v.kh = d->kh, v.kw = d->kw;
    v.pad[0] = 0, v.pad[1] = d->pad_h, v.pad[2] = d->pad_w;
    v.pad_hi[0] = 0, v.pad_hi[1] = d->pad_h_hi, v.pad_hi[2] = d->pad_w_hi;
    v.stride[0] = 1, v.stride[1] = d->stride_h, v.stride[2] = d->stride_w;
    v.dil[0] = 1, v.dil[1] = d->dil_h, v.dil[2] = d->dil_w;
    v.group        = d->group;
    v.in_type      = d->in_type;
    v.out_type     = d->out_type;
    v.dequant      = d->dequant;
    v.scale_x_mode = d->scale_x_mode;
    v.scale_w_mode = d->scale_w_mode;
    return v;
}

} // namespace

// ---- float convolution: a correctness path ------------------------------------------------------
// op::convolution::compute (src/include/migraphx/op/convolution.hpp:208-239 -> convolution.hpp:37-100)
// as the reference evaluates it: the float product rounded, added into a double over (channel,
// kd, kh, kw) in that order, one conversion to float at the end.  One thread per output; what the
// integer front ends leave of a layer whose tensors are uint8 (QLinearConv) runs here.
struct convf_params
{
    const float* x;
    const float* w;
    float* out;
    int64_t n, c, d, h, w_, o, kd, kh, kw, od, oh, ow;
    int64_t pad[3], stride[3], dil[3];
    int64_t group;
};

__global__ __launch_bounds__(256) void conv_f32_kernel(convf_params p)
{
#pragma clang fp contract(off)
    const int64_t total = p.n * p.o * p.od * p.oh * p.ow;
    const int64_t step  = (int64_t)gridDim.x * 256;
    const int64_t cg = p.c / p.group, og = p.o / p.group;
    for(int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += step)
    {
        const int64_t ox = idx % p.ow;
        const int64_t oy = (idx / p.ow) % p.oh;
        const int64_t oz = (idx / (p.ow * p.oh)) % p.od;
        const int64_t oc = (idx / (p.ow * p.oh * p.od)) % p.o;
        const int64_t b  = idx / (p.ow * p.oh * p.od * p.o);
        const int64_t g  = oc / og;
        double acc       = 0.0;
        for(int64_t k = 0; k < cg; k++)
        {
            const int64_t ic = g * cg + k;
            for(int64_t t = 0; t < p.kd; t++)
            {
                const int64_t iz = oz * p.stride[0] - p.pad[0] + t * p.dil[0];
                if(iz < 0 || iz >= p.d)
                    continue;
                for(int64_t r = 0; r < p.kh; r++)
                {
                    const int64_t iy = oy * p.stride[1] - p.pad[1] + r * p.dil[1];
                    if(iy < 0 || iy >= p.h)
                        continue;
                    for(int64_t q = 0; q < p.kw; q++)
                    {
                        const int64_t ix = ox * p.stride[2] - p.pad[2] + q * p.dil[2];
                        if(ix < 0 || ix >= p.w_)
                            continue;
                        const float prod = p.x[(((b * p.c + ic) * p.d + iz) * p.h + iy) * p.w_ + ix] *
                                           p.w[(((oc * cg + k) * p.kd + t) * p.kh + r) * p.kw + q];
                        acc += (double)prod;
                    }
                }
            }
        }
        p.out[idx] = (float)acc;
    }
}

extern "C" int mi355_convolution_f32(const mi355_quant_conv3d_desc* d,
                                     const float* x,
                                     const float* w,
                                     float* out,
                                     void* stream)
{
    if(d == nullptr || d->in_type != MI355_F32)
        return MI355_ERR_BAD_ARG;
    mi355_quant_conv3d_desc q = *d;
    q.in_type                 = MI355_I8; // the shape rules are those of the quantized operator
    if(!valid(&q))
        return MI355_ERR_BAD_ARG;
    convf_params p;
    const int64_t in[3]  = {d->d, d->h, d->w};
    const int64_t win[3] = {d->kd, d->kh, d->kw};
    int64_t o[3];
    for(int i = 0; i < 3; i++)
    {
        o[i]        = out_len(in[i], win[i], d->pad[i], d->pad_hi[i], d->stride[i], d->dil[i]);
        p.pad[i]    = d->pad[i];
        p.stride[i] = d->stride[i];
        p.dil[i]    = d->dil[i];
        if(o[i] < 1)
            return MI355_ERR_BAD_ARG;
    }
    const int64_t total = d->n * d->o * o[0] * o[1] * o[2];
    if(total == 0)
        return MI355_OK;
    if(x == nullptr || w == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    p.x = x; p.w = w; p.out = out;
    p.n = d->n; p.c = d->c; p.d = d->d; p.h = d->h; p.w_ = d->w;
    p.o = d->o; p.kd = d->kd; p.kh = d->kh; p.kw = d->kw;
    p.od = o[0]; p.oh = o[1]; p.ow = o[2];
    p.group = d->group;
    int64_t blocks = (total + 255) / 256;
    if(blocks > 256 * 64)
        blocks = 256 * 64;
    hipLaunchKernelGGL(conv_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), p);
    return mi355_launch_status();
}

extern "C" int mi355_quant_convolution3d_dims(const mi355_quant_conv3d_desc* d,
                                              int64_t* out_lens,
                                              size_t* workspace_bytes)
{
    if(!valid(d))
        return MI355_ERR_BAD_ARG;
    const int64_t in[3]  = {d->d, d->h, d->w};
    const int64_t win[3] = {d->kd, d->kh, d->kw};
    int64_t o[3];
    for(int i = 0; i < 3; i++)
        o[i] = out_len(in[i], win[i], d->pad[i], d->pad_hi[i], d->stride[i], d->dil[i]);
    const int64_t kg = d->c / d->group * d->kd * d->kh * d->kw;
    const int64_t kp = (kg + K_STEP - 1) / K_STEP * K_STEP;
    if(out_lens != nullptr)
    {
        for(int i = 0; i < 3; i++)
            out_lens[i] = o[i];
    }
    if(workspace_bytes != nullptr)
    {
        // few output tiles (small images, one image at a time): the GEMM splits K when it has room
        const int64_t plane          = o[0] * o[1] * o[2];
        const mi355_quant_dot_desc g = gemm_of(d, plane, kp);
        *workspace_bytes             = staging_bytes(d, plane, kp) + mi355_quant_dot_workspace_size(&g);
        if(direct_form(d, o) && *workspace_bytes < direct_bytes(d))
            *workspace_bytes = direct_bytes(d);
        // the kernel for many small groups stages nothing (the entry point still wants a pointer)
        if(small_groups_form(d))
            *workspace_bytes = 16;
    }
    return MI355_OK;
}

extern "C" int mi355_quant_convolution3d(const mi355_quant_conv3d_desc* d,
                                         const void* x,
                                         const void* w,
                                         void* out,
                                         const float* scale_x,
                                         const float* scale_w,
                                         void* workspace,
                                         size_t workspace_bytes,
                                         void* stream)
{
    int64_t ol[3] = {0, 0, 0};
    size_t need   = 0;
    const int st  = mi355_quant_convolution3d_dims(d, ol, &need);
    if(st != MI355_OK)
        return st;
    const bool fp8 = d->in_type == MI355_FP8;
    if(d->dequant)
    {
        if(d->out_type != MI355_F32 && d->out_type != MI355_F16 && d->out_type != MI355_BF16)
            return MI355_ERR_BAD_ARG;
        if(d->scale_x_mode != MI355_QP_NONE && d->scale_x_mode != MI355_QP_PER_TENSOR)
            return MI355_ERR_BAD_ARG;
        if(d->scale_w_mode != MI355_QP_NONE && d->scale_w_mode != MI355_QP_PER_TENSOR &&
           d->scale_w_mode != MI355_QP_PER_ROW)
            return MI355_ERR_BAD_ARG;
        if((d->scale_x_mode != MI355_QP_NONE && scale_x == nullptr) ||
           (d->scale_w_mode != MI355_QP_NONE && scale_w == nullptr))
            return MI355_ERR_BAD_ARG;
    }
    else if(d->out_type != (fp8 ? MI355_F32 : MI355_I32))
        return MI355_ERR_BAD_ARG;
    if(d->n == 0)
        return MI355_OK;
    if(x == nullptr || w == nullptr || out == nullptr || workspace == nullptr)
        return MI355_ERR_BAD_ARG;
    if(workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return MI355_ERR_BAD_ARG;
    // batch and group become grid dimensions, the spatial sizes and positions 32-bit indices
    const int64_t lim    = (int64_t)1 << 30;
    const int64_t window = d->kd * d->kh * d->kw;
    if(d->n > 65535 || d->group > 65535 || d->d * d->h * d->w >= lim || window >= lim ||
       ol[0] * ol[1] * ol[2] >= lim || d->c / d->group * window >= 65535 * 64)
        return MI355_ERR_UNSUPPORTED;
    for(int i = 0; i < 3; i++)
    {
        if(d->pad[i] >= lim || d->stride[i] >= lim || d->dil[i] >= lim ||
           d->dil[i] * ((i == 0 ? d->kd : i == 1 ? d->kh : d->kw) - 1) >= lim || ol[i] * d->stride[i] >= lim)
            return MI355_ERR_UNSUPPORTED;
    }

    hipStream_t hs      = static_cast<hipStream_t>(stream);
    const int64_t cg    = d->c / d->group;
    const int64_t og    = d->o / d->group;
    const int64_t kg    = cg * window;
    const int64_t kp    = (kg + K_STEP - 1) / K_STEP * K_STEP;
    const int64_t plane = ol[0] * ol[1] * ol[2];
    uint8_t* col        = static_cast<uint8_t*>(workspace);
    uint8_t* wp         = col + d->n * d->group * plane * kp;

    // A window of one element with unit strides and no padding is a product of matrices as the
    // tensors lie: out[n] [O/G, P] = W [O/G, C/G] . x[n] [C/G, P], the input row-major as the second
    // operand.  Nothing is gathered or copied.
    // (channels in whole K steps and positions in fours: the GEMM's matrix-core kernels; other shapes would fall to
    // its general kernel, which the gathered form below beats)
    bool pointwise = window == 1 && plane % 4 == 0 && cg % K_STEP == 0 &&
                     reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
    for(int i = 0; i < 3; i++)
        pointwise = pointwise && d->stride[i] == 1 && d->pad[i] == 0 && d->pad_hi[i] == 0;
    if(pointwise)
    {
        mi355_quant_dot_desc g = gemm_of(d, plane, cg);
        g.ldb      = plane;
        g.stride_b = d->c * plane;
        g.trans_b  = 0;
        const size_t esz1 = mi355_dtype_size(d->out_type);
        for(int64_t grp = 0; grp < d->group; grp++)
        {
            const float* sw = scale_w;
            if(d->dequant && d->scale_w_mode == MI355_QP_PER_ROW)
                sw = scale_w + grp * og;
            const int r = mi355_quant_dot_ws(&g, static_cast<const uint8_t*>(w) + grp * og * cg,
                                             static_cast<const uint8_t*>(x) + grp * cg * plane,
                                             static_cast<uint8_t*>(out) + (size_t)(grp * og * plane) * esz1, sw,
                                             scale_x, nullptr, nullptr, nullptr, workspace, workspace_bytes, stream);
            if(r != MI355_OK)
                return r;
        }
        return MI355_OK;
    }

    // several groups of few channels: one or four outputs per thread, nothing staged
    if(small_groups_form(d))
    {
        small_params q{};
        q.x = static_cast<const uint8_t*>(x), q.w = static_cast<const uint8_t*>(w), q.out = out;
        q.scale_x = scale_x, q.scale_w = scale_w;
        q.total = d->n * d->o * plane;
        q.c = (int)d->c, q.d = (int)d->d, q.h = (int)d->h, q.w_ = (int)d->w;
        q.o = (int)d->o, q.og = (int)og, q.cg = (int)cg;
        q.kd = (int)d->kd, q.kh = (int)d->kh, q.kw = (int)d->kw;
        q.od = (int)ol[0], q.oh = (int)ol[1], q.ow = (int)ol[2];
        q.pad_d = (int)d->pad[0], q.pad_h = (int)d->pad[1], q.pad_w = (int)d->pad[2];
        q.stride_d = (int)d->stride[0], q.stride_h = (int)d->stride[1], q.stride_w = (int)d->stride[2];
        q.dil_d = (int)d->dil[0], q.dil_h = (int)d->dil[1], q.dil_w = (int)d->dil[2];
        q.dequant = d->dequant, q.scale_x_mode = d->scale_x_mode, q.scale_w_mode = d->scale_w_mode;
        if(fp8)
            launch_small_groups<true>(q, d->dequant != 0, d->out_type, hs);
        else
            launch_small_groups<false>(q, d->dequant != 0, d->out_type, hs);
        return mi355_launch_status();
    }

    if(direct_form(d, ol) && reinterpret_cast<uintptr_t>(x) % 16 == 0)
    {
        uint8_t* ws = static_cast<uint8_t*>(workspace);
        const int64_t nk  = direct_steps(d);
        const int64_t ogp = direct_ogp(d);
        prep_params q{};
        q.x = static_cast<const uint8_t*>(x);
        q.w = static_cast<const uint8_t*>(w);
        q.wp = ws;
        q.xt = ws + d->group * nk * ogp * DC_KSTEP;
        q.n = (int)d->n;
        q.c = (int)d->c, q.d = (int)d->d, q.h = (int)d->h, q.w_ = (int)d->w;
        q.cp = (int)(direct_cgp(d) * d->group);
        q.pad_d = (int)d->pad[0], q.pad_h = (int)d->pad[1], q.pad_w = (int)d->pad[2];
        q.dp = (int)(d->d + d->pad[0] + d->pad_hi[0]);
        q.hp = (int)(d->h + d->pad[1] + d->pad_hi[1]);
        q.wp_ = (int)(d->w + d->pad[2] + d->pad_hi[2]);
        q.group = (int)d->group, q.og = (int)og, q.ogp = (int)ogp;
        q.cg = (int)cg, q.window = (int)window, q.nk = (int)nk;
        q.narrow = direct_narrow(d) ? 1 : 0, q.kh = (int)d->kh, q.kw = (int)d->kw;
        const int64_t space = d->d * d->h * d->w;
        const bool dwords   = space % 4 == 0;
        q.tiles_s = (int)((space + (dwords ? 255 : 63)) / (dwords ? 256 : 64));
        q.tiles_c = (int)((q.cp + 63) / 64);
        int64_t tiles       = d->n * q.tiles_c * q.tiles_s;
        const bool padded   = q.dp != q.d || q.hp != q.h || q.wp_ != q.w_;
        int64_t border_rows = padded ? d->n * q.dp * q.hp : 0;
        if(q.narrow)
        {
            // the narrow copy writes every pixel of the padded volume, the border among them
            tiles       = (d->n * q.dp * q.hp * q.wp_ + 1023) / 1024;
            border_rows = 0;
        }
        // blocks behind them: the weights, one piece of 16 bytes per thread up to 1024 blocks
        int64_t extra = d->group * nk * ogp * (DC_KSTEP / 16) / 256 + 1;
        extra         = extra > 1024 ? 1024 : extra;
        if(tiles + border_rows + extra >= ((int64_t)1 << 31))
            return MI355_ERR_UNSUPPORTED;
        q.tiles       = (int)tiles;
        q.border_rows = (int)border_rows;
        const dim3 prep_grid((unsigned)(tiles + border_rows + extra));
        if(dwords)
            hipLaunchKernelGGL(conv_prep_kernel<4>, prep_grid, dim3(256), 0, hs, q);
        else
            hipLaunchKernelGGL(conv_prep_kernel<1>, prep_grid, dim3(256), 0, hs, q);
        if(mi355_launch_status() != MI355_OK)
            return MI355_ERR_LAUNCH;

        direct_params p{};
        p.xt = q.xt, p.wp = q.wp, p.out = out;
        p.scale_x = scale_x, p.scale_w = scale_w;
        p.rows = d->n * plane;
        p.plane = (int)plane, p.oh = (int)ol[1], p.ow = (int)ol[2];
        p.o = (int)d->o, p.og = (int)og, p.ogp = (int)ogp, p.c = q.cp, p.cg = (int)direct_cgp(d);
        p.kh = (int)d->kh, p.kw = (int)d->kw;
        p.dp = q.dp, p.hp = q.hp, p.wp_ = q.wp_;
        p.stride_d = (int)d->stride[0], p.stride_h = (int)d->stride[1], p.stride_w = (int)d->stride[2];
        p.dil_d = (int)d->dil[0], p.dil_h = (int)d->dil[1], p.dil_w = (int)d->dil[2];
        p.kg = (int)(direct_cgp(d) * window), p.nk = (int)nk;
        p.narrow = q.narrow;
        if(p.narrow)
            p.kg = (int)(16 * d->kd * d->kh * ((d->kw + 3) / 4));
        p.col_tiles = (int)(ogp / DC_COLS);
        p.dequant = d->dequant, p.scale_x_mode = d->scale_x_mode, p.scale_w_mode = d->scale_w_mode;
        const int64_t row_tiles = (p.rows + DC_ROWS - 1) / DC_ROWS;
        if(row_tiles >= ((int64_t)1 << 31))
            return MI355_ERR_UNSUPPORTED;
        const dim3 grid((unsigned)row_tiles, (unsigned)(p.col_tiles * d->group));
        const bool vec = plane % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
        if(fp8)
            launch_direct<true>(p, d->dequant != 0, d->out_type, vec, grid, hs);
        else
            launch_direct<false>(p, d->dequant != 0, d->out_type, vec, grid, hs);
        return mi355_launch_status();
    }

    uint8_t* xt         = wp + d->o * kp; // channels-last copy of the input, when that form is used
    // every group a multiple of 16 channels and a real window: gather through a channels-last copy
    const bool channels_last = cg % 16 == 0 && window > 1 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
    if(channels_last)
    {
        // [N][C][D*H*W] -> [N][D*H*W][C]: the window kernel with a window of one element, K = C, the
        // volume flattened to one axis
        im2col_params t{};
        t.x = static_cast<const uint8_t*>(x);
        t.col = xt;
        t.rows = d->n * d->d * d->h * d->w;
        t.c = t.cg = t.kg = t.kp = d->c;
        t.d = t.h = 1;
        t.w = d->d * d->h * d->w;
        t.kd = t.kh = t.kw = 1;
        t.od = t.oh = 1;
        t.ow = t.w;
        t.stride_d = t.stride_h = t.stride_w = 1;
        t.dil_d = t.dil_h = t.dil_w = 1;
        t.group = 1;
        launch_im2col(t, hs);
        if(mi355_launch_status() != MI355_OK)
            return MI355_ERR_LAUNCH;
    }

    im2col_params p{};
    p.x        = channels_last ? xt : static_cast<const uint8_t*>(x);
    p.col      = col;
    p.rows     = d->n * plane;
    p.c        = d->c;
    p.d        = d->d;
    p.h        = d->h;
    p.w        = d->w;
    p.cg       = cg;
    p.kd       = d->kd;
    p.kh       = d->kh;
    p.kw       = d->kw;
    p.od       = ol[0];
    p.oh       = ol[1];
    p.ow       = ol[2];
    p.pad_d    = d->pad[0];
    p.pad_h    = d->pad[1];
    p.pad_w    = d->pad[2];
    p.stride_d = d->stride[0];
    p.stride_h = d->stride[1];
    p.stride_w = d->stride[2];
    p.dil_d    = d->dil[0];
    p.dil_h    = d->dil[1];
    p.dil_w    = d->dil[2];
    p.group    = d->group;
    p.kg       = kg;
    p.kp       = kp;
    if(channels_last)
    {
        const int64_t total = p.rows * p.group * (kp / 16);
        int64_t blocks      = (total + 255) / 256;
        if(blocks > 256 * 64)
            blocks = 256 * 64;
        if(total + blocks * 256 < ((int64_t)1 << 31))
            hipLaunchKernelGGL(im2col_cl_kernel<uint32_t>, dim3((unsigned)blocks), dim3(256), 0, hs, p);
        else
            hipLaunchKernelGGL(im2col_cl_kernel<int64_t>, dim3((unsigned)blocks), dim3(256), 0, hs, p);
    }
    else
        launch_im2col(p, hs);
    if(mi355_launch_status() != MI355_OK)
        return MI355_ERR_LAUNCH;

    // the weights as O rows of Kp bytes; rows that already have that length (and a 16-byte aligned
    // start) are used where they are
    const bool pad_weights = !channels_last && (kg != kp || reinterpret_cast<uintptr_t>(w) % 16 != 0);
    const uint8_t* wmat    = (pad_weights || channels_last) ? wp : static_cast<const uint8_t*>(w);
    if(channels_last)
    {
        // the same element order as the window matrix
        const int64_t total = d->o * kp;
        int64_t blocks      = (total + 255) / 256;
        if(blocks > 256 * 16)
            blocks = 256 * 16;
        hipLaunchKernelGGL(weights_cl_kernel, dim3((unsigned)blocks), dim3(256), 0, hs,
                           static_cast<const uint8_t*>(w), wp, d->o, cg, window, kp);
        if(mi355_launch_status() != MI355_OK)
            return MI355_ERR_LAUNCH;
    }
    else if(pad_weights)
    {
        launch_im2col(copy_rows(static_cast<const uint8_t*>(w), wp, d->o, kg, kp), hs);
        if(mi355_launch_status() != MI355_OK)
            return MI355_ERR_LAUNCH;
    }

    const mi355_quant_dot_desc g = gemm_of(d, plane, kp);
    void* room                   = static_cast<uint8_t*>(workspace) + staging_bytes(d, plane, kp);
    const size_t room_bytes      = need - staging_bytes(d, plane, kp);
    const size_t esz = mi355_dtype_size(d->out_type);
    for(int64_t grp = 0; grp < d->group; grp++)
    {
        const float* sw = scale_w;
        if(d->dequant && d->scale_w_mode == MI355_QP_PER_ROW)
            sw = scale_w + grp * og;
        const int r = mi355_quant_dot_ws(&g, wmat + grp * og * kp, col + grp * plane * kp,
                                         static_cast<uint8_t*>(out) + (size_t)(grp * og * plane) * esz, sw, scale_x,
                                         nullptr, nullptr, nullptr, room_bytes > 0 ? room : nullptr, room_bytes,
                                         stream);
        if(r != MI355_OK)
            return r;
    }
    return MI355_OK;
}

extern "C" int mi355_quant_convolution_dims(const mi355_quant_conv_desc* d,
                                            int64_t* oh,
                                            int64_t* ow,
                                            size_t* workspace_bytes)
{
    if(d == nullptr)
        return MI355_ERR_BAD_ARG;
    const mi355_quant_conv3d_desc v = with_unit_depth(d);
    int64_t ol[3]                   = {0, 0, 0};
    const int st                    = mi355_quant_convolution3d_dims(&v, ol, workspace_bytes);
    if(st != MI355_OK)
        return st;
    if(oh != nullptr)
        *oh = ol[1];
    if(ow != nullptr)
        *ow = ol[2];
    return MI355_OK;
}

extern "C" int mi355_quant_convolution(const mi355_quant_conv_desc* d,
                                       const void* x,
                                       const void* w,
                                       void* out,
                                       const float* scale_x,
                                       const float* scale_w,
                                       void* workspace,
                                       size_t workspace_bytes,
                                       void* stream)
{
    if(d == nullptr)
        return MI355_ERR_BAD_ARG;
    const mi355_quant_conv3d_desc v = with_unit_depth(d);
    return mi355_quant_convolution3d(&v, x, w, out, scale_x, scale_w, workspace, workspace_bytes, stream);
}
