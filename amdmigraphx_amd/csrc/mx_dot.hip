// quant_dot with block scales (the MX formats): fp8 e4m3fn or packed fp4 e2m1 operands, one scale
// per 32 elements along K for each row of A and each column of B, on the block-scaled matrix-core
// instruction v_mfma_scale_f32_16x16x128_f8f6f4.
//
// The instruction takes, per lane, 32 consecutive K elements of one row (A) or column (B) and one
// e8m0 scale (a power of two, the biased exponent byte of a float) for exactly those 32 elements:
// a lane's fragment is one scale block.  The operator (ref_quant_gemm::compute, four inputs,
// src/targets/ref/lowering.cpp:221-242) is more general: its scales are float tensors of the
// operands' own shape, any value per element.  Three kernels keep every input right without a
// host-side decision:
//   mx_prepare_kernel   walks the scale tensors once: a block whose 32 scales are one normal power
//                       of two becomes its exponent byte in a compact [rows, K/32] array; anything
//                       else raises a flag in device memory (by writing the call's number there:
//                       the word needs no clearing, see next_ticket);
//   mx_gemm_kernel      the matrix-core product from the compact scales; returns at once when the
//                       flag is up;
//   mx_exact_kernel     the operator's arithmetic one output per thread -- float(a) * scale in
//                       float, products and sum in double, one rounding to float -- and returns at
//                       once when the flag is down.
// With power-of-two block scales every float(a) * scale is exact, so the first path computes the
// same sum as the second up to the fp32 accumulation of the instruction (the tolerance of the fp8
// quant_dot); small sums are exact.
#include "common.h"

#include <atomic>

// the LDS-staged kernel for packed fp4 x packed fp4 and fp8 x fp8 (qgemm_dma.hip)
bool mi355_dma_mx_supported(int64_t m, int64_t n, int64_t kbytes, int64_t lda, int64_t ldb, int64_t ldc,
                            int64_t stride_a, int64_t stride_b, const void* a, const void* b);
int mi355_dma_mx_launch(const void* a, const void* b, float* c, int64_t m, int64_t n, int64_t kbytes,
                        int64_t lda, int64_t ldb, int64_t ldc, int64_t stride_a, int64_t stride_b,
                        int64_t stride_c, int64_t batch, const uint8_t* ea, const uint8_t* eb,
                        const uint32_t* flag, uint32_t ticket, int bits, hipStream_t stream);

namespace {

typedef float v4f32 __attribute__((ext_vector_type(4)));

struct mx_params
{
    const uint8_t* a;
    const uint8_t* b;
    float* c;
    const float* scale_a;
    const float* scale_b;
    int m, n, k, nblk;
    int64_t lda, ldb, ldc; // lda / ldb in bytes of the stored operand
    int64_t stride_a, stride_b, stride_c;
    int64_t sa_batch, sa_row, sa_block, sa_elem;
    int64_t sb_batch, sb_row, sb_block, sb_elem;
    int a4, b4; // operand stored as packed fp4 (two codes per byte, low nibble = even k)
    uint32_t* flag;   // holds `ticket` when this call's scales are not what the matrix-core path takes
    uint32_t ticket; // this call's number, never 0
    uint8_t* ea; // [batch][m][nblk] exponent bytes
    uint8_t* eb; // [batch][n][nblk]
    // staged: the layout the LDS-staged kernel loads, [batch][slab][rows rounded up to 256][4]: the
    // blocks of a 64-byte slab of one row side by side (4 of packed fp4, 2 of fp8 and two bytes
    // unused); rows past the end are not written and their products are dropped
    int staged;
    int group; // blocks per thread of mx_prepare_kernel: 4, or the slab's 2 when staged fp8
    int rows_a, rows_b; // m and n rounded up to 256
};


// one thread per (operand, batch, row, group of p.group blocks): the exponent bytes of a group leave
// as one word where the layout keeps them together
__global__ __launch_bounds__(256) void mx_prepare_kernel(mx_params p, int batch)
{
    const bool is_b     = blockIdx.y != 0;
    const int rows      = is_b ? p.n : p.m;
    const int groups    = (p.nblk + p.group - 1) / p.group;
    const int64_t total = (int64_t)batch * rows * groups;
    const int64_t i     = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(i >= total)
        return;
    const int grp  = (int)(i % groups);
    const int row  = (int)((i / groups) % rows);
    const int bt   = (int)(i / ((int64_t)groups * rows));
    const float* s = is_b ? p.scale_b + bt * p.sb_batch + row * p.sb_row : p.scale_a + bt * p.sa_batch + row * p.sa_row;
    const int64_t sblock = is_b ? p.sb_block : p.sa_block;
    const int64_t e      = is_b ? p.sb_elem : p.sa_elem;
    bool ok        = true;
    uint32_t word  = 0;
    const int nb   = min(p.group, p.nblk - p.group * grp);
    for(int c = 0; c < nb; c++)
    {
        const int blk        = p.group * grp + c;
        const float* sp      = s + blk * sblock;
        const uint32_t first = __builtin_bit_cast(uint32_t, sp[0]);
        const uint32_t field = (first >> 23) & 0xffu;
        // a positive normal power of two: no sign, no mantissa, exponent field 1..254
        ok = ok && (first & 0x807fffffu) == 0 && field >= 1 && field <= 254;
        if(e != 0)
        {
            const int last = min(32, p.k - blk * 32);
            for(int j = 1; j < last; j++)
                ok = ok && __builtin_bit_cast(uint32_t, sp[j * e]) == first;
        }
        word |= field << (8 * c);
    }
    uint8_t* out = is_b ? p.eb : p.ea;
    if(p.staged)
    {
        // whole slabs only, one word each
        const int padded = is_b ? p.rows_b : p.rows_a;
        *reinterpret_cast<uint32_t*>(out + (((int64_t)bt * groups + grp) * padded + row) * 4) = word;
    }
    else
    {
        uint8_t* o = out + ((int64_t)bt * rows + row) * p.nblk + p.group * grp;
        for(int c = 0; c < nb; c++)
            o[c] = (uint8_t)(word >> (8 * c));
    }
    if(!ok)
        *p.flag = p.ticket;
}

MI355_DEVINL float fp4_value(uint32_t code)
{
    // e2m1: sign, two exponent bits, one mantissa bit
    const float mag[8] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
    const float v      = mag[code & 7];
    return (code & 8) ? -v : v;
}

MI355_DEVINL float operand_value(const uint8_t* base, int k, int packed)
{
    if(packed)
    {
        const uint8_t byte = base[k >> 1];
        return fp4_value((k & 1) ? (byte >> 4) : (byte & 0xf));
    }
    return fp8_to_f32(base[k]);
}

// the operator's own arithmetic, for scales the matrix-core path cannot take
// (a fixed, modest number of workgroups walks the 16 x 16 tiles: when the flag is down -- the usual
// case -- the launch is over after that many reads of it, whatever the size of C)
__global__ __launch_bounds__(256) void mx_exact_kernel(mx_params p, int batch)
{
    if(*p.flag != p.ticket)
        return;
    const int tiles_n   = (p.n + 15) / 16;
    const int tiles_m   = (p.m + 15) / 16;
    const int64_t tiles = (int64_t)batch * tiles_m * tiles_n;
    for(int64_t t = blockIdx.x; t < tiles; t += gridDim.x)
    {
    const int col = (int)(t % tiles_n) * 16 + (threadIdx.x & 15);
    const int row = (int)((t / tiles_n) % tiles_m) * 16 + (threadIdx.x >> 4);
    const int bt  = (int)(t / ((int64_t)tiles_n * tiles_m));
    if(row >= p.m || col >= p.n)
        continue;
    const uint8_t* a = p.a + bt * p.stride_a + row * p.lda;
    const uint8_t* b = p.b + bt * p.stride_b + col * p.ldb;
    const float* sa  = p.scale_a + bt * p.sa_batch + row * p.sa_row;
    const float* sb  = p.scale_b + bt * p.sb_batch + col * p.sb_row;
    double sum       = 0;
    for(int k = 0; k < p.k; k++)
    {
#pragma clang fp contract(off)
        const float x = operand_value(a, k, p.a4) * sa[(k >> 5) * p.sa_block + (k & 31) * p.sa_elem];
        const float w = operand_value(b, k, p.b4) * sb[(k >> 5) * p.sb_block + (k & 31) * p.sb_elem];
        sum += (double)x * (double)w;
    }
    p.c[bt * p.stride_c + (int64_t)row * p.ldc + col] = (float)sum;
    }
}

// 128 x 128 of C per workgroup of 4 waves (2 x 2), 64 x 64 per wave as 4 x 4 tiles of 16 x 16;
// K in steps of 128.  A lane's fragment of a tile is the 32 K elements [32 g, 32 g + 32) of row
// (or column) r, g = lane / 16, r = lane % 16: contiguous bytes of a K-contiguous operand, loaded
// straight from memory (rows of one tile are read by the two waves beside each other; the
// operands of block-scaled layers are a quarter to a half of an int8 layer's bytes).
template <bool A4, bool B4>
__global__ __launch_bounds__(256) void mx_gemm_kernel(mx_params p)
{
    if(*p.flag == p.ticket)
        return;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wm   = wave >> 1, wn = wave & 1;
    const int r    = lane & 15, g = lane >> 4;
    const int bt   = blockIdx.z;
    const int m0   = blockIdx.y * 128 + wm * 64;
    const int n0   = blockIdx.x * 128 + wn * 64;
    const uint8_t* a  = p.a + bt * p.stride_a;
    const uint8_t* b  = p.b + bt * p.stride_b;
    const uint8_t* ea = p.ea + (int64_t)bt * p.m * p.nblk;
    const uint8_t* eb = p.eb + (int64_t)bt * p.n * p.nblk;

    const uint8_t* arow[4];
    const uint8_t* brow[4];
    const uint8_t* earow[4];
    const uint8_t* ebrow[4];
#pragma unroll
    for(int i = 0; i < 4; i++)
    {
        const int row = min(m0 + i * 16 + r, p.m - 1);
        const int col = min(n0 + i * 16 + r, p.n - 1);
        arow[i]       = a + row * p.lda;
        brow[i]       = b + col * p.ldb;
        earow[i]      = ea + (int64_t)row * p.nblk;
        ebrow[i]      = eb + (int64_t)col * p.nblk;
    }
    v4f32 acc[4][4];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 4; j++)
            acc[i][j] = v4f32{0.f, 0.f, 0.f, 0.f};

    // Operand registers of the instruction.  4-bit codes: lane group g holds K elements
    // [32 g, 32 g + 32) of the step in four registers -- one scale block.  8-bit codes: the
    // 128-deep instruction is laid out as two 64-deep halves, lane group g holding
    // [16 g, 16 g + 16) in registers 0-3 and [64 + 16 g, 64 + 16 g + 16) in registers 4-7, while
    // the scale a lane supplies is still that of block g, i.e. of K [32 g, 32 g + 32).
    // Past the end of K: zeros, which add nothing whatever their scale.
    auto fragment = [&](const uint8_t* row, int k0, auto packed) -> v8i {
        v8i f = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr(decltype(packed)::value)
        {
            const int k = k0 + 32 * g;
            if(k < p.k)
            {
                const v4i lo = *reinterpret_cast<const v4i*>(row + (k >> 1));
                f            = v8i{lo.x, lo.y, lo.z, lo.w, 0, 0, 0, 0};
            }
        }
        else
        {
            const int k = k0 + 16 * g;
            v4i lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
            if(k < p.k)
                lo = *reinterpret_cast<const v4i*>(row + k);
            if(k + 64 < p.k)
                hi = *reinterpret_cast<const v4i*>(row + k + 64);
            f = v8i{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        }
        return f;
    };

    for(int k0 = 0; k0 < p.k; k0 += 128)
    {
        const int k   = k0 + 32 * g;
        const int blk = min(k >> 5, p.nblk - 1);
        v8i fa[4], fb[4];
        int sa[4], sb[4];
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            fa[i] = fragment(arow[i], k0, std::integral_constant<bool, A4>{});
            fb[i] = fragment(brow[i], k0, std::integral_constant<bool, B4>{});
            sa[i] = earow[i][blk];
            sb[i] = ebrow[i][blk];
        }
#pragma unroll
        for(int i = 0; i < 4; i++)
#pragma unroll
            for(int j = 0; j < 4; j++)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    fa[i], fb[j], acc[i][j], A4 ? 4 : 0, B4 ? 4 : 0, 0, sa[i], 0, sb[j]);
    }
    // element e of lane (r, g) of tile (i, j): row 16 i + 4 g + e, column 16 j + r
    float* c = p.c + bt * p.stride_c;
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int e = 0; e < 4; e++)
        {
            const int row = m0 + i * 16 + 4 * g + e;
            if(row >= p.m)
                continue;
#pragma unroll
            for(int j = 0; j < 4; j++)
            {
                const int col = n0 + j * 16 + r;
                if(col < p.n)
                    c[(int64_t)row * p.ldc + col] = acc[i][j][e];
            }
        }
}

size_t align16(size_t x) { return (x + 15) / 16 * 16; }

// The flag word of the workspace is never cleared: a call raises it by writing its own number, and
// only that number counts.  Whatever the word held before -- an earlier call's number, or anything
// at all in a fresh workspace -- reads as "not raised", except the one value in 2^32 that happens
// to be this call's number; then (as after a replay of a captured call whose earlier run raised it)
// the exact path computes the result, which is right for every input, only slower.
uint32_t next_ticket()
{
    static std::atomic<uint32_t> counter{0};
    uint32_t t = counter.fetch_add(1, std::memory_order_relaxed) + 1;
    return t != 0 ? t : counter.fetch_add(1, std::memory_order_relaxed) + 1;
}

} // namespace

extern "C" size_t mi355_quant_dot_mx_workspace_size(const mi355_mx_dot_desc* d)
{
    if(d == nullptr || d->m <= 0 || d->n <= 0 || d->k <= 0 || d->batch <= 0)
        return 0;
    // rows rounded up to the 256 of the staged layout (mx_params::staged), which spends four bytes
    // on the two blocks of an fp8 slab
    const size_t nblk = (size_t)(d->k + 31) / 32 * (d->a_type == MI355_FP8 && d->b_type == MI355_FP8 ? 2 : 1);
    const size_t ra = (size_t)(d->m + 255) / 256 * 256, rb = (size_t)(d->n + 255) / 256 * 256;
    return 16 + align16((size_t)d->batch * ra * nblk) + align16((size_t)d->batch * rb * nblk);
}

extern "C" int mi355_quant_dot_mx(const mi355_mx_dot_desc* d,
                                  const void* a,
                                  const void* b,
                                  float* c,
                                  const float* scale_a,
                                  const float* scale_b,
                                  void* workspace,
                                  size_t workspace_bytes,
                                  void* stream)
{
    if(d == nullptr)
        return MI355_ERR_BAD_ARG;
    if(d->m < 0 || d->n < 0 || d->k < 0 || d->batch < 0)
        return MI355_ERR_BAD_ARG;
    if((d->a_type != MI355_FP8 && d->a_type != MI355_FP4X2) || (d->b_type != MI355_FP8 && d->b_type != MI355_FP4X2))
        return MI355_ERR_UNSUPPORTED;
    if(d->m == 0 || d->n == 0 || d->batch == 0)
        return MI355_OK;
    if(a == nullptr || b == nullptr || c == nullptr || scale_a == nullptr || scale_b == nullptr || workspace == nullptr)
        return MI355_ERR_BAD_ARG;
    if(d->k == 0 || d->k % 32 != 0)
        return MI355_ERR_UNSUPPORTED; // whole scale blocks only
    const bool a4 = d->a_type == MI355_FP4X2, b4 = d->b_type == MI355_FP4X2;
    const int64_t a_row = a4 ? d->k / 2 : d->k, b_row = b4 ? d->k / 2 : d->k;
    if(d->lda < a_row || d->ldb < b_row || d->ldc < d->n)
        return MI355_ERR_BAD_ARG;
    // fragments are 16-byte loads
    if(d->lda % 16 != 0 || d->ldb % 16 != 0 || d->stride_a % 16 != 0 || d->stride_b % 16 != 0 ||
       reinterpret_cast<uintptr_t>(a) % 16 != 0 || reinterpret_cast<uintptr_t>(b) % 16 != 0 ||
       reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return MI355_ERR_UNSUPPORTED;
    if(d->m > (1 << 30) || d->n > (1 << 30) || d->k > (1 << 30) || d->batch > 65535 || (d->m + 15) / 16 > 65535)
        return MI355_ERR_UNSUPPORTED;
    if(workspace_bytes < mi355_quant_dot_mx_workspace_size(d))
        return MI355_ERR_BAD_ARG;
    mx_params p{};
    p.a        = static_cast<const uint8_t*>(a);
    p.b        = static_cast<const uint8_t*>(b);
    p.c        = c;
    p.scale_a  = scale_a;
    p.scale_b  = scale_b;
    p.m        = (int)d->m;
    p.n        = (int)d->n;
    p.k        = (int)d->k;
    p.nblk     = (int)(d->k / 32);
    p.lda      = d->lda;
    p.ldb      = d->ldb;
    p.ldc      = d->ldc;
    p.stride_a = d->stride_a;
    p.stride_b = d->stride_b;
    p.stride_c = d->stride_c;
    p.sa_batch = d->sa_batch;
    p.sa_row   = d->sa_row;
    p.sa_block = d->sa_block;
    p.sa_elem  = d->sa_elem;
    p.sb_batch = d->sb_batch;
    p.sb_row   = d->sb_row;
    p.sb_block = d->sb_block;
    p.sb_elem  = d->sb_elem;
    p.a4       = a4;
    p.b4       = b4;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    p.flag      = reinterpret_cast<uint32_t*>(ws);
    p.ticket    = next_ticket();
    p.ea        = ws + 16;
    p.rows_a    = (int)((d->m + 255) / 256 * 256);
    p.rows_b    = (int)((d->n + 255) / 256 * 256);
    p.eb        = p.ea + align16((size_t)d->batch * p.rows_a * p.nblk * (!a4 && !b4 ? 2 : 1));
    // both operands packed fp4 or both fp8, whole 64-byte slabs: the LDS-staged kernel
    p.staged = a4 == b4 && d->k % (a4 ? 128 : 64) == 0 &&
               mi355_dma_mx_supported(d->m, d->n, a_row, d->lda, d->ldb, d->ldc, d->stride_a, d->stride_b, a, b);
    p.group = p.staged && !a4 ? 2 : 4;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t most = (int64_t)d->batch * (d->m > d->n ? d->m : d->n) * ((p.nblk + p.group - 1) / p.group);
    hipLaunchKernelGGL(mx_prepare_kernel, dim3((unsigned)((most + 255) / 256), 2), dim3(256), 0, s, p, (int)d->batch);
    const dim3 grid((unsigned)((d->n + 127) / 128), (unsigned)((d->m + 127) / 128), (unsigned)d->batch);
    if(p.staged)
    {
        const int st = mi355_dma_mx_launch(a, b, c, d->m, d->n, a_row, d->lda, d->ldb, d->ldc, d->stride_a,
                                           d->stride_b, d->stride_c, d->batch, p.ea, p.eb, p.flag, p.ticket, a4 ? 4 : 8, s);
        if(st != MI355_OK)
            return st;
    }
    else if(a4 && b4)
        hipLaunchKernelGGL((mx_gemm_kernel<true, true>), grid, dim3(256), 0, s, p);
    else if(a4)
        hipLaunchKernelGGL((mx_gemm_kernel<true, false>), grid, dim3(256), 0, s, p);
    else if(b4)
        hipLaunchKernelGGL((mx_gemm_kernel<false, true>), grid, dim3(256), 0, s, p);
    else
        hipLaunchKernelGGL((mx_gemm_kernel<false, false>), grid, dim3(256), 0, s, p);
    const int64_t etiles = (int64_t)d->batch * ((d->n + 15) / 16) * ((d->m + 15) / 16);
    hipLaunchKernelGGL(mx_exact_kernel, dim3((unsigned)(etiles < 2048 ? etiles : 2048)), dim3(256), 0, s, p,
                       (int)d->batch);
    return mi355_launch_status();
}
