// quant_convolution as im2col + the quantized GEMM, over one, two or three spatial axes (a missing
// leading axis is a depth of one).  The windows of the input are gathered into a
// [N, group, OD*OH*OW, Kp] matrix (Kp = C/group * KD * KH * KW rounded up to the GEMM's K step, zero
// filled), the weights are copied to rows of the same pitch, and for every image the result
// plane [O, OD*OH*OW] = W [O, Kp] . col^T is one batched mi355_quant_dot with the col matrix as the
// transposed operand: the GEMM writes NC(D)HW directly and its dequantize epilogue applies the
// per-output-channel scale as a per-row scale.  Zero padding adds exact zeros to every sum
// (int8: 0 * w; fp8: the code 0 is +0.0 and the padded weights are +0.0 too), so the result is the
// direct convolution's.
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
