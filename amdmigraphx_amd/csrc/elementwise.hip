// Float operators around the quantized GEMMs of an encoder graph: broadcasting binary operators,
// unary functions, reduce_mean and softmax over the last axis, gather along axis 0.  They follow
// the ref target's arithmetic (plain IEEE float operations; reductions accumulate in double as
// accumulator_type<float> does, src/include/migraphx/type_traits.hpp:78-81) and are written for
// correctness and coalesced access, not tuned: the GEMMs dominate the graph.
#include "common.h"

namespace {

struct bcast_params
{
    const float* a;
    const float* b;
    float* out;
    int64_t lens[MI355_MAX_DIMS];
    int64_t a_strides[MI355_MAX_DIMS];
    int64_t b_strides[MI355_MAX_DIMS];
    int64_t total;
    int ndim;
    int op;
};

MI355_DEVINL float binary_apply(int op, float x, float y);

__global__ __launch_bounds__(256) void binary_kernel(bcast_params p)
{
    const int64_t step = (int64_t)gridDim.x * 256;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += step)
    {
        int64_t rem = i, ao = 0, bo = 0;
        for(int d = p.ndim - 1; d >= 0; d--)
        {
            const int64_t c = rem % p.lens[d];
            rem /= p.lens[d];
            ao += c * p.a_strides[d];
            bo += c * p.b_strides[d];
        }
        p.out[i] = binary_apply(p.op, p.a[ao], p.b[bo]);
    }
}

MI355_DEVINL float binary_apply(int op, float x, float y)
{
    switch(op)
    {
    case MI355_BIN_ADD: return x + y;
    case MI355_BIN_SUB: return x - y;
    case MI355_BIN_MUL: return x * y;
    case MI355_BIN_MAX: return x < y ? y : x; // std::max(x, y) (op/max.hpp)
    case MI355_BIN_MIN: return y < x ? y : x; // std::min(x, y) (op/min.hpp)
    default: return x / y; // correctly rounded IEEE division
    }
}

// int32 add / sub / mul with the same addressing: the zero-point terms simplify_qdq adds up in
// front of a dequantizelinear (src/simplify_qdq.cpp:196-222).  Wrapping arithmetic, as int32 in
// the reference wraps on every target it is built for.
struct bcast_params_i32
{
    const int32_t* a;
    const int32_t* b;
    int32_t* out;
    int64_t lens[MI355_MAX_DIMS];
    int64_t a_strides[MI355_MAX_DIMS];
    int64_t b_strides[MI355_MAX_DIMS];
    int64_t total;
    int ndim;
    int op;
};

__global__ __launch_bounds__(256) void binary_i32_kernel(bcast_params_i32 p)
{
    const int64_t step = (int64_t)gridDim.x * 256;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += step)
    {
        int64_t rem = i, ao = 0, bo = 0;
        for(int d = p.ndim - 1; d >= 0; d--)
        {
            const int64_t c = rem % p.lens[d];
            rem /= p.lens[d];
            ao += c * p.a_strides[d];
            bo += c * p.b_strides[d];
        }
        const uint32_t x = (uint32_t)p.a[ao], y = (uint32_t)p.b[bo];
        const uint32_t r = p.op == MI355_BIN_ADD ? x + y : (p.op == MI355_BIN_SUB ? x - y : x * y);
        p.out[i]         = (int32_t)r;
    }
}

// The same for the narrow types that the integer-MatMul front end leaves in a graph: int8 / uint8
// (the operands promote to int and the result converts back, wrapping; division is not offered)
// and half / bf16 (op/binary.hpp with generic_float.hpp:303-326: the operator works on floats and
// the result converts back, toward zero).
struct bcast_params_typed
{
    const void* a;
    const void* b;
    void* out;
    int64_t lens[MI355_MAX_DIMS];
    int64_t a_strides[MI355_MAX_DIMS];
    int64_t b_strides[MI355_MAX_DIMS];
    int64_t total;
    int ndim;
    int op;
    int type;
};

__global__ __launch_bounds__(256) void binary_typed_kernel(bcast_params_typed p)
{
    const int64_t step = (int64_t)gridDim.x * 256;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < p.total; i += step)
    {
        int64_t rem = i, ao = 0, bo = 0;
        for(int d = p.ndim - 1; d >= 0; d--)
        {
            const int64_t c = rem % p.lens[d];
            rem /= p.lens[d];
            ao += c * p.a_strides[d];
            bo += c * p.b_strides[d];
        }
        if(p.type == MI355_I8 || p.type == MI355_U8)
        {
            const int x = p.type == MI355_I8 ? (int)static_cast<const int8_t*>(p.a)[ao]
                                             : (int)static_cast<const uint8_t*>(p.a)[ao];
            const int y = p.type == MI355_I8 ? (int)static_cast<const int8_t*>(p.b)[bo]
                                             : (int)static_cast<const uint8_t*>(p.b)[bo];
            const int r = p.op == MI355_BIN_ADD ? x + y : (p.op == MI355_BIN_SUB ? x - y : x * y);
            static_cast<uint8_t*>(p.out)[i] = (uint8_t)(unsigned)r;
        }
        else
        {
            const uint16_t xb = static_cast<const uint16_t*>(p.a)[ao], yb = static_cast<const uint16_t*>(p.b)[bo];
            const float x = p.type == MI355_F16 ? half_to_f32(xb) : bf16_to_f32(xb);
            const float y = p.type == MI355_F16 ? half_to_f32(yb) : bf16_to_f32(yb);
            const float r = binary_apply(p.op, x, y);
            static_cast<uint16_t*>(p.out)[i] = p.type == MI355_F16 ? f32_to_half_rtz(r) : f32_to_bf16_rtz(r);
        }
    }
}

// The shapes that matter collapse to [rows, cols] with each operand either running along the
// columns (column stride 1) or constant along them (column stride 0: a per-row value or a scalar):
// activations against a bias row, a per-row statistic, another activation.  Four columns per
// thread as one 16-byte access, rows by grid stride; no index division at all.
struct binary2d_params
{
    const float* a;
    const float* b;
    float* out;
    int64_t rows, cols;
    int64_t a_sr, b_sr;
    int a_sc, b_sc; // 0 or 1
    int op;
};

__global__ __launch_bounds__(256) void binary2d_kernel(binary2d_params p)
{
    const int64_t c4 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if(c4 >= p.cols)
        return;
    for(int64_t r = blockIdx.y; r < p.rows; r += gridDim.y)
    {
        v4f x, y;
        if(p.a_sc)
            x = *reinterpret_cast<const v4f*>(p.a + r * p.a_sr + c4);
        else
        {
            const float s = p.a[r * p.a_sr];
            x             = v4f{s, s, s, s};
        }
        if(p.b_sc)
            y = *reinterpret_cast<const v4f*>(p.b + r * p.b_sr + c4);
        else
        {
            const float s = p.b[r * p.b_sr];
            y             = v4f{s, s, s, s};
        }
        v4f o;
#pragma unroll
        for(int e = 0; e < 4; e++)
            o[e] = binary_apply(p.op, x[e], y[e]);
        *reinterpret_cast<v4f*>(p.out + r * p.cols + c4) = o;
    }
}

MI355_DEVINL float unary_apply(int op, float x)
{
    switch(op)
    {
    case MI355_UN_ERF: return erff(x);
    case MI355_UN_SQRT: return sqrtf(x); // correctly rounded (hipcc default)
    case MI355_UN_RSQRT: return 1.0f / sqrtf(x); // 1 / std::sqrt(x), two IEEE operations
    case MI355_UN_EXP: return expf(x);
    case MI355_UN_TANH: return tanhf(x);
    case MI355_UN_NEARBYINT: return rintf(x); // std::nearbyint under round-to-nearest-even
    default: return -x;
    }
}

// One operator over the N values a thread holds, the operator chosen once for all of them (the
// code is the same for every lane, so the choice costs scalar branches and each case is N
// straight-line operations).  value = value (op) operand, or operand (op) value when reversed.
template <int N>
MI355_DEVINL void binary_block(int op, bool reversed, float* value, const float* operand)
{
#pragma clang fp contract(off)
#define MI355_BLOCK_OF(EXPR)                                   \
    _Pragma("unroll") for(int i = 0; i < N; i++)               \
    {                                                          \
        const float x = reversed ? operand[i] : value[i];      \
        const float y = reversed ? value[i] : operand[i];      \
        value[i]      = EXPR;                                  \
    }
    if(reversed)
    {
        switch(op)
        {
        case MI355_BIN_ADD: MI355_BLOCK_OF(x + y) break;
        case MI355_BIN_SUB: MI355_BLOCK_OF(x - y) break;
        case MI355_BIN_MUL: MI355_BLOCK_OF(x * y) break;
        case MI355_BIN_MAX: MI355_BLOCK_OF(x < y ? y : x) break;
        case MI355_BIN_MIN: MI355_BLOCK_OF(y < x ? y : x) break;
        default: MI355_BLOCK_OF(x / y) break;
        }
    }
    else
    {
        switch(op)
        {
        case MI355_BIN_ADD: MI355_BLOCK_OF(x + y) break;
        case MI355_BIN_SUB: MI355_BLOCK_OF(x - y) break;
        case MI355_BIN_MUL: MI355_BLOCK_OF(x * y) break;
        case MI355_BIN_MAX: MI355_BLOCK_OF(x < y ? y : x) break;
        case MI355_BIN_MIN: MI355_BLOCK_OF(y < x ? y : x) break;
        default: MI355_BLOCK_OF(x / y) break;
        }
    }
#undef MI355_BLOCK_OF
}

template <int N>
MI355_DEVINL void unary_block(int op, float* value)
{
#define MI355_BLOCK_OF(EXPR)                                   \
    _Pragma("unroll") for(int i = 0; i < N; i++)               \
    {                                                          \
        const float x = value[i];                              \
        value[i]      = EXPR;                                  \
    }
    switch(op)
    {
    case MI355_UN_ERF: MI355_BLOCK_OF(erff(x)) break;
    case MI355_UN_SQRT: MI355_BLOCK_OF(sqrtf(x)) break;
    case MI355_UN_RSQRT: MI355_BLOCK_OF(1.0f / sqrtf(x)) break;
    case MI355_UN_EXP: MI355_BLOCK_OF(expf(x)) break;
    case MI355_UN_TANH: MI355_BLOCK_OF(tanhf(x)) break;
    case MI355_UN_NEARBYINT: MI355_BLOCK_OF(rintf(x)) break;
    default: MI355_BLOCK_OF(-x) break;
    }
#undef MI355_BLOCK_OF
}

__global__ __launch_bounds__(256) void unary_kernel(const float* in, float* out, int64_t n, int op)
{
    const int64_t step = (int64_t)gridDim.x * 256;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step)
        out[i] = unary_apply(op, in[i]);
}

// n a multiple of 4, both pointers 16-byte aligned
__global__ __launch_bounds__(256) void unary4_kernel(const v4f* in, v4f* out, int64_t n4, int op)
{
    const int64_t step = (int64_t)gridDim.x * 256;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += step)
    {
        const v4f x = in[i];
        v4f r;
#pragma unroll
        for(int e = 0; e < 4; e++)
            r[e] = unary_apply(op, x[e]);
        out[i] = r;
    }
}

// A chain of binary and unary operators over [rows, cols] in one pass.  W columns per thread
// (4 as one 16-byte access, or 1), rows by grid stride.  The step list is uniform over the grid,
// so the switch costs scalar branches only; every operation is the one the single-operator
// kernels perform, and separate steps are never contracted into a fused multiply-add.
struct chain_params
{
    const float* in[MI355_CHAIN_MAX_INPUTS];
    int64_t sr[MI355_CHAIN_MAX_INPUTS];
    int sc[MI355_CHAIN_MAX_INPUTS];
    mi355_chain_step steps[MI355_CHAIN_MAX_STEPS];
    float* out;
    int64_t rows, cols;
    int n_steps;
    // Q: the chain's last value leaves as int8, quantized with one scale and one zero point for the
    // whole tensor (quantizelinear's arithmetic: rintf(v / scale) + zp, clamped), instead of as float
    int8_t* qout;
    const float* qscale;
    const int8_t* qzp;
};

template <int W, int R, bool Q = false>
__global__ __launch_bounds__(256) void chain_kernel(chain_params p)
{
#pragma clang fp contract(off)
    const int64_t c0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * W;
    if(c0 >= p.cols)
        return;
    // R rows at a time: their loads are in flight together and the step list is walked once for
    // all of them.  Rows past the end repeat the last one and are not stored.
    for(int64_t r0 = (int64_t)blockIdx.y * R; r0 < p.rows; r0 += (int64_t)gridDim.y * R)
    {
        float acc[R][W], saved[R][W], operand[R][W];
#pragma unroll
        for(int i = 0; i < R; i++)
#pragma unroll
            for(int e = 0; e < W; e++)
                acc[i][e] = saved[i][e] = 0.0f;
        auto fetch = [&](int in, float(&dst)[R][W]) __attribute__((always_inline)) {
            const float* base = p.in[in];
            const int64_t sr  = p.sr[in];
            if(p.sc[in] == 0)
            {
#pragma unroll
                for(int i = 0; i < R; i++)
                {
                    const int64_t r = min(r0 + i, p.rows - 1);
                    const float s   = base[r * sr];
#pragma unroll
                    for(int e = 0; e < W; e++)
                        dst[i][e] = s;
                }
            }
            else
            {
#pragma unroll
                for(int i = 0; i < R; i++)
                {
                    const int64_t r = min(r0 + i, p.rows - 1);
                    if constexpr(W == 4)
                    {
                        const v4f v = *reinterpret_cast<const v4f*>(base + r * sr + c0);
#pragma unroll
                        for(int e = 0; e < W; e++)
                            dst[i][e] = v[e];
                    }
                    else
                    {
                        dst[i][0] = base[r * sr + c0];
                    }
                }
            }
        };
        for(int s = 0; s < p.n_steps; s++)
        {
            const mi355_chain_step st = p.steps[s];
            switch(st.kind)
            {
            case MI355_CH_LOAD: fetch(st.src, acc); break;
            case MI355_CH_BINARY: {
                if(st.src >= 0)
                {
                    fetch(st.src, operand);
                    binary_block<R * W>(st.op, st.reversed != 0, &acc[0][0], &operand[0][0]);
                }
                else if(st.src == MI355_CH_SAVED)
                    binary_block<R * W>(st.op, st.reversed != 0, &acc[0][0], &saved[0][0]);
                else
                    binary_block<R * W>(st.op, st.reversed != 0, &acc[0][0], &acc[0][0]);
                break;
            }
            case MI355_CH_UNARY: unary_block<R * W>(st.op, &acc[0][0]); break;
            default:
#pragma unroll
                for(int i = 0; i < R; i++)
#pragma unroll
                    for(int e = 0; e < W; e++)
                        saved[i][e] = acc[i][e];
                break;
            }
        }
#pragma unroll
        for(int i = 0; i < R; i++)
        {
            const int64_t r = r0 + i;
            if(r >= p.rows)
                break;
            if constexpr(Q)
            {
                const float sv = p.qscale[0];
                const double z = p.qzp != nullptr ? (double)p.qzp[0] : 0.0;
                uint32_t w     = 0;
#pragma unroll
                for(int e = 0; e < W; e++)
                {
                    const double qv = clamp_like_ref((double)rintf(acc[i][e] / sv) + z, -128.0, 127.0);
                    w |= (uint32_t)(uint8_t)(int8_t)(int)qv << (8 * e);
                }
                if constexpr(W == 4)
                    *reinterpret_cast<uint32_t*>(p.qout + r * p.cols + c0) = w;
                else
                    p.qout[r * p.cols + c0] = (int8_t)w;
            }
            else if constexpr(W == 4)
                *reinterpret_cast<v4f*>(p.out + r * p.cols + c0) = v4f{acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
            else
                p.out[r * p.cols + c0] = acc[i][0];
        }
    }
}

// sum of 64 doubles across a wave, every lane receives it; fixed pairing, so deterministic
MI355_DEVINL double wave_sum_f64(double v)
{
#pragma unroll
    for(int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}

MI355_DEVINL double wave_max_f64(double v)
{
#pragma unroll
    for(int off = 32; off > 0; off >>= 1)
        v = fmax(v, __shfl_xor(v, off, 64));
    return v;
}

// The chain machine with the whole row in the registers of one wave (lane l holds columns l, l + 64,
// ...: up to 64 * NV of them) and one more step, MI355_CH_ROW_MEAN: the running value becomes the
// mean of its row -- reduce_mean over the last axis and the broadcast back in one -- summed as
// reduce_mean_kernel below sums it (a lane's columns in ascending order in a double, then the fixed
// pairing across the wave, one rounding to float), so a layer normalisation written as reduce_mean /
// sub / mul / reduce_mean / add / rsqrt / mul ... gives the bits of its separate operators while x
// is read once and only the result is written.  Columns past the end hold values nobody reads.
template <int NV>
__global__ __launch_bounds__(256) void chain_rows_kernel(chain_params p)
{
#pragma clang fp contract(off)
    const int lane    = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if(row >= p.rows)
        return;
    float acc[NV], saved[NV], operand[NV];
#pragma unroll
    for(int i = 0; i < NV; i++)
        acc[i] = saved[i] = 0.0f;
    auto fetch = [&](int in, float(&dst)[NV]) __attribute__((always_inline)) {
        // one form for both column strides and no branch, so that the loads of several inputs are in
        // flight together; a column past the end reads the last one
        const float* base = p.in[in] + row * p.sr[in];
        const int sc      = p.sc[in];
#pragma unroll
        for(int i = 0; i < NV; i++)
        {
            const int64_t c = lane + 64 * i;
            dst[i]          = base[(c < p.cols ? c : p.cols - 1) * sc];
        }
    };
    for(int s = 0; s < p.n_steps; s++)
    {
        const mi355_chain_step st = p.steps[s];
        switch(st.kind)
        {
        case MI355_CH_LOAD: fetch(st.src, acc); break;
        case MI355_CH_BINARY: {
            if(st.src >= 0)
            {
                fetch(st.src, operand);
                binary_block<NV>(st.op, st.reversed != 0, acc, operand);
            }
            else if(st.src == MI355_CH_SAVED)
                binary_block<NV>(st.op, st.reversed != 0, acc, saved);
            else
                binary_block<NV>(st.op, st.reversed != 0, acc, acc);
            break;
        }
        case MI355_CH_UNARY: unary_block<NV>(st.op, acc); break;
        case MI355_CH_ROW_MEAN: {
            double sum = 0.0;
#pragma unroll
            for(int i = 0; i < NV; i++)
                if(lane + 64 * i < p.cols)
                    sum += (double)acc[i];
            sum              = wave_sum_f64(sum);
            const float mean = (float)(sum / (double)p.cols);
#pragma unroll
            for(int i = 0; i < NV; i++)
                acc[i] = mean;
            break;
        }
        default:
#pragma unroll
            for(int i = 0; i < NV; i++)
                saved[i] = acc[i];
            break;
        }
    }
    float* y = p.out + row * p.cols;
#pragma unroll
    for(int i = 0; i < NV; i++)
    {
        const int64_t c = lane + 64 * i;
        if(c < p.cols)
            y[c] = acc[i];
    }
}

// The step list of a layer normalisation as the lowering writes it -- [x | a (op) b], save, row mean,
// saved - mean, save, square, row mean, + eps, rsqrt | sqrt, saved * | / root, then up to two more
// operators with an input each (the scale and the shift) -- has this kernel of its own: the same
// operations in the same order as the step machine above performs them (the same bits), written out,
// so that every input row is requested before the first one is waited for, and the operators on
// the row's statistics run once per row instead of once per column.
struct layer_norm_plan
{
    int x, pre_src, pre_op; // pre_op < 0: the row is input x itself
    int eps;
    int recip; // rsqrt and a product, else sqrt and a quotient
    int n_tail;
    int tail_op[2], tail_src[2];
};

template <int NV>
__global__ __launch_bounds__(256) void layer_norm_rows_kernel(chain_params p, layer_norm_plan q)
{
#pragma clang fp contract(off)
    const int lane    = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if(row >= p.rows)
        return;
    auto fetch = [&](int in, float(&dst)[NV]) __attribute__((always_inline)) {
        // one form for both column strides and no branch, so that the loads of several inputs are in
        // flight together; a column past the end reads the last one
        const float* base = p.in[in] + row * p.sr[in];
        const int sc      = p.sc[in];
#pragma unroll
        for(int i = 0; i < NV; i++)
        {
            const int64_t c = lane + 64 * i;
            dst[i]          = base[(c < p.cols ? c : p.cols - 1) * sc];
        }
    };
    auto row_mean = [&](const float(&v)[NV]) __attribute__((always_inline)) {
        double sum = 0.0;
#pragma unroll
        for(int i = 0; i < NV; i++)
            if(lane + 64 * i < p.cols)
                sum += (double)v[i];
        sum = wave_sum_f64(sum);
        return (float)(sum / (double)p.cols);
    };
    float acc[NV], other[NV], tail0[NV], tail1[NV];
    fetch(q.x, acc);
    if(q.pre_op >= 0)
        fetch(q.pre_src, other);
    if(q.n_tail > 0)
        fetch(q.tail_src[0], tail0);
    if(q.n_tail > 1)
        fetch(q.tail_src[1], tail1);
    const float eps = p.in[q.eps][row * p.sr[q.eps]];
    if(q.pre_op >= 0)
        binary_block<NV>(q.pre_op, false, acc, other);
    const float mean = row_mean(acc);
#pragma unroll
    for(int i = 0; i < NV; i++)
    {
        acc[i]   = acc[i] - mean;
        other[i] = acc[i] * acc[i];
    }
    const float var  = row_mean(other);
    const float root = unary_apply(q.recip ? MI355_UN_RSQRT : MI355_UN_SQRT, var + eps);
#pragma unroll
    for(int i = 0; i < NV; i++)
        acc[i] = q.recip ? acc[i] * root : acc[i] / root;
    if(q.n_tail > 0)
        binary_block<NV>(q.tail_op[0], false, acc, tail0);
    if(q.n_tail > 1)
        binary_block<NV>(q.tail_op[1], false, acc, tail1);
    float* y = p.out + row * p.cols;
#pragma unroll
    for(int i = 0; i < NV; i++)
    {
        const int64_t c = lane + 64 * i;
        if(c < p.cols)
            y[c] = acc[i];
    }
}

// one wave per row; double accumulation (the order differs from the reference's sequential sum,
// which moves the float result by at most its last bit)
__global__ __launch_bounds__(256) void reduce_mean_kernel(const float* in, float* out, int64_t rows, int64_t cols)
{
    const int lane    = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if(row >= rows)
        return;
    const float* x = in + row * cols;
    double s       = 0.0;
    for(int64_t c = lane; c < cols; c += 64)
        s += (double)x[c];
    s = wave_sum_f64(s);
    if(lane == 0)
        out[row] = (float)(s / (double)cols);
}

// Is the double q within `units` units in its last place of the midpoint between two neighbouring
// floats (q in the range of the normal floats)?  A value that is not rounds to the same float as
// every double that close to it.
MI355_DEVINL bool near_float_midpoint(double q, int units)
{
    const int low = (int)((uint32_t)__double_as_longlong(q) & 0x1fffffffu); // the 29 bits a float drops
    const int d   = low - 0x10000000;
    return (d < 0 ? -d : d) <= units;
}

// float(exp(d)), d <= 0 (softmax: a value minus its row's maximum), the float that the exact
// exponential rounds to.  Eleven Taylor terms behind the usual reduction to |r| <= ln(2) / 2 are
// within 2^-46 of it (r^12 / 12! < 2^-47, the rounding of the steps a few times 2^-53), i.e. within 90
// units in the last place of a double; unless that reaches a midpoint between two floats, the
// float is settled.  The few values where it might (one in a million), and the arguments whose
// results are float denormals, take the library's exp as before.
MI355_DEVINL float exp_to_float(double d)
{
    const double n = rint(d * 1.4426950408889634074);
    double r       = fma(-n, 6.93147180369123816490e-01, d);
    r              = fma(-n, 1.90821492927058770002e-10, r);
    double p       = 2.50521083854417187751e-08; // 1 / 11!
    p              = fma(p, r, 2.75573192239858906526e-07);
    p              = fma(p, r, 2.75573192239858906526e-06);
    p              = fma(p, r, 2.48015873015873015873e-05);
    p              = fma(p, r, 1.98412698412698412698e-04);
    p              = fma(p, r, 1.38888888888888888889e-03);
    p              = fma(p, r, 8.33333333333333333333e-03);
    p              = fma(p, r, 4.16666666666666666667e-02);
    p              = fma(p, r, 1.66666666666666666667e-01);
    p              = fma(p, r, 0.5);
    p              = fma(p, r, 1.0);
    p              = fma(p, r, 1.0);
    const double q = ldexp(p, (int)n);
    float e        = (float)q;
    // one branch for everything the short way does not settle (its value above is then not used):
    // arguments below the normal floats' exponentials, -inf, NaN, and the midpoints
    if(!(d >= -87.0) || near_float_midpoint(q, 256))
        e = d < -104.0 ? 0.0f : (float)exp(d); // exp(-104) < 2^-150 rounds to 0
    return e;
}

// float(double(e) / s) given rs = 1 / s: e * rs is within 3 units in the last place of the quotient's
// double, so unless it comes that close to a midpoint between two floats (or the result is a float
// denormal) it rounds to the same float, and the division is left to those rare values.
MI355_DEVINL float quotient_to_float(float e, double s, double rs)
{
    const double q = (double)e * rs;
    if(q != 0.0 && (!(q >= 2.4e-38) || near_float_midpoint(q, 8)))
        return (float)((double)e / s);
    return (float)q;
}

// ref_softmax (src/targets/ref/lowering.cpp:281-312): e = float(exp(double(x) - max)),
// sum of e in double, out = float(double(e) / sum)
__global__ __launch_bounds__(256) void softmax_kernel(const float* in, float* out, int64_t rows, int64_t cols)
{
    const int lane    = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if(row >= rows)
        return;
    const float* x = in + row * cols;
    float* y       = out + row * cols;
    double m       = -1.7976931348623157e308;
    for(int64_t c = lane; c < cols; c += 64)
        m = fmax(m, (double)x[c]);
    m        = wave_max_f64(m);
    double s = 0.0;
    for(int64_t c = lane; c < cols; c += 64)
    {
        const float e = exp_to_float((double)x[c] - m);
        y[c]          = e;
        s += (double)e;
    }
    s               = wave_sum_f64(s);
    const double rs = 1.0 / s;
    for(int64_t c = lane; c < cols; c += 64)
        y[c] = quotient_to_float(y[c], s, rs);
}

// The same arithmetic with the row held in registers (up to 64*NV columns): one read and one write
// of the tensor instead of three and two.  A lane's elements are summed in the same order as above,
// so the results are the same bits.  FULL: the row has exactly 64*NV columns.  Otherwise the
// columns past the end enter as -inf, which leaves the maximum alone and adds an exact zero to the
// sum, so that no step needs a branch of its own.
template <int NV, bool FULL>
__global__ __launch_bounds__(256) void softmax_rows_kernel(const float* in, float* out, int64_t rows, int cols)
{
    const int lane    = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if(row >= rows)
        return;
    const float* x = in + row * cols;
    float* y       = out + row * cols;
    float v[NV];
    // every load before the first use, none behind a branch
#pragma unroll
    for(int i = 0; i < NV; i++)
    {
        const int c = lane + 64 * i;
        v[i]        = x[FULL ? c : min(c, cols - 1)];
    }
    if constexpr(!FULL)
    {
#pragma unroll
        for(int i = 0; i < NV; i++)
            v[i] = lane + 64 * i < cols ? v[i] : -__builtin_huge_valf();
    }
    double m = -1.7976931348623157e308;
#pragma unroll
    for(int i = 0; i < NV; i++)
        m = fmax(m, (double)v[i]);
    m        = wave_max_f64(m);
    double s = 0.0;
#pragma unroll
    for(int i = 0; i < NV; i++)
    {
        v[i] = exp_to_float((double)v[i] - m);
        s += (double)v[i];
    }
    s               = wave_sum_f64(s);
    const double rs = 1.0 / s;
#pragma unroll
    for(int i = 0; i < NV; i++)
    {
        const int c = lane + 64 * i;
        if(FULL || c < cols)
            y[c] = quotient_to_float(v[i], s, rs);
    }
}

// out[i, :] = table[ids[i], :]; negative indices count from the end (op/gather.hpp:100-118)
template <class I>
__global__ __launch_bounds__(256) void gather_rows_kernel(
    const uint32_t* table, const I* ids, uint32_t* out, int64_t n_ids, int64_t table_rows, int64_t row_words)
{
    const int64_t total = n_ids * row_words;
    const int64_t step  = (int64_t)gridDim.x * 256;
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step)
    {
        const int64_t r = i / row_words;
        int64_t id      = (int64_t)ids[r];
        if(id < 0)
            id += table_rows;
        // an index outside the table reads row 0 rather than memory out of bounds
        if(id < 0 || id >= table_rows)
            id = 0;
        out[i] = table[id * row_words + (i - r * row_words)];
    }
}

unsigned blocks_for_n(int64_t n)
{
    int64_t b = (n + 255) / 256;
    return (unsigned)(b > 256 * 16 ? 256 * 16 : (b < 1 ? 1 : b));
}

} // namespace

extern "C" int mi355_binary_f32(int32_t op,
                                const float* a,
                                const int64_t* a_strides,
                                const float* b,
                                const int64_t* b_strides,
                                float* out,
                                int32_t ndim,
                                const int64_t* lens,
                                void* stream)
{
    if(op < MI355_BIN_ADD || op > MI355_BIN_MIN || ndim < 1 || ndim > MI355_MAX_DIMS ||
       lens == nullptr || a_strides == nullptr || b_strides == nullptr)
        return MI355_ERR_BAD_ARG;
    bcast_params p{};
    p.total = 1;
    for(int d = 0; d < ndim; d++)
    {
        if(lens[d] < 0 || a_strides[d] < 0 || b_strides[d] < 0)
            return MI355_ERR_BAD_ARG;
        p.lens[d]      = lens[d];
        p.a_strides[d] = a_strides[d];
        p.b_strides[d] = b_strides[d];
        p.total *= lens[d];
    }
    if(p.total == 0)
        return MI355_OK;
    if(a == nullptr || b == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    p.a    = a;
    p.b    = b;
    p.out  = out;
    p.ndim = ndim;
    p.op   = op;
    // collapse to [rows, cols]: leading dimensions merge into one row index when, for both
    // operands, each stride continues the next one (or both are broadcast there)
    {
        int last = ndim - 1;
        while(last > 0 && lens[last] == 1)
            last--;
        const int64_t cols = lens[last];
        int64_t rows       = 1;
        int64_t a_sr = 0, b_sr = 0;
        bool ok      = true;
        bool first   = true;
        for(int d = last - 1; d >= 0 && ok; d--)
        {
            if(lens[d] == 1)
                continue;
            if(first)
            {
                a_sr  = a_strides[d];
                b_sr  = b_strides[d];
                first = false;
            }
            else
            {
                ok = a_strides[d] == a_sr * rows && b_strides[d] == b_sr * rows;
            }
            rows *= lens[d];
        }
        const int64_t a_sc = cols == 1 ? 0 : a_strides[last];
        const int64_t b_sc = cols == 1 ? 0 : b_strides[last];
        auto vec_ok        = [&](const float* q, int64_t sr, int64_t sc) {
            if(sc == 0)
                return true;
            return sc == 1 && sr % 4 == 0 && reinterpret_cast<uintptr_t>(q) % 16 == 0;
        };
        if(ok && cols % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 && vec_ok(a, a_sr, a_sc) &&
           vec_ok(b, b_sr, b_sc))
        {
            binary2d_params q{a, b, out, rows, cols, a_sr, b_sr, (int)a_sc, (int)b_sc, op};
            const int64_t gx = (cols / 4 + 255) / 256;
            const int64_t gy = rows < 65535 ? rows : 65535;
            hipLaunchKernelGGL(binary2d_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0,
                               static_cast<hipStream_t>(stream), q);
            return mi355_launch_status();
        }
    }
    hipLaunchKernelGGL(binary_kernel, dim3(blocks_for_n(p.total)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
    return mi355_launch_status();
}

namespace {
// Is the (validated) step list the layer normalisation layer_norm_rows_kernel evaluates?
bool layer_norm_steps(const chain_params& p, layer_norm_plan& q)
{
    const mi355_chain_step* st = p.steps;
    auto kind_at = [&](int at, int kind) { return at < p.n_steps && st[at].kind == kind; };
    auto binary  = [&](int at, int op, int src, int reversed) {
        return kind_at(at, MI355_CH_BINARY) && st[at].op == op && st[at].src == src && st[at].reversed == reversed;
    };
    auto unary = [&](int at, int op) { return kind_at(at, MI355_CH_UNARY) && st[at].op == op; };
    // an operator with an input as its second operand
    auto binary_with_input = [&](int at) {
        return kind_at(at, MI355_CH_BINARY) && st[at].src >= 0 && st[at].reversed == 0;
    };
    q.x      = st[0].src; // the first step is a LOAD
    q.pre_op = -1;
    int s    = 1;
    if(binary_with_input(1))
    {
        q.pre_op  = st[1].op;
        q.pre_src = st[1].src;
        s         = 2;
    }
    if(!(kind_at(s, MI355_CH_SAVE) && kind_at(s + 1, MI355_CH_ROW_MEAN) &&
         binary(s + 2, MI355_BIN_SUB, MI355_CH_SAVED, 1) && kind_at(s + 3, MI355_CH_SAVE) &&
         binary(s + 4, MI355_BIN_MUL, MI355_CH_SELF, 0) && kind_at(s + 5, MI355_CH_ROW_MEAN) &&
         binary_with_input(s + 6) && st[s + 6].op == MI355_BIN_ADD && p.sc[st[s + 6].src] == 0))
        return false;
    q.eps = st[s + 6].src;
    if(unary(s + 7, MI355_UN_RSQRT) && binary(s + 8, MI355_BIN_MUL, MI355_CH_SAVED, 1))
        q.recip = 1;
    else if(unary(s + 7, MI355_UN_SQRT) && binary(s + 8, MI355_BIN_DIV, MI355_CH_SAVED, 1))
        q.recip = 0;
    else
        return false;
    s += 9;
    q.n_tail = p.n_steps - s;
    if(q.n_tail < 0 || q.n_tail > 2)
        return false;
    for(int t = 0; t < q.n_tail; t++)
    {
        if(!binary_with_input(s + t))
            return false;
        q.tail_op[t]  = st[s + t].op;
        q.tail_src[t] = st[s + t].src;
    }
    return true;
}

int chain_launch(const mi355_chain_step* steps,
                 int32_t n_steps,
                 const float* const* inputs,
                 const int64_t* row_strides,
                 const int32_t* col_strides,
                 int32_t n_inputs,
                 float* out,
                 int8_t* qout,
                 const float* qscale,
                 const int8_t* qzp,
                 int64_t rows,
                 int64_t cols,
                 void* stream,
                 bool whole_rows = false)
{
    if(steps == nullptr || n_steps < 1 || n_steps > MI355_CHAIN_MAX_STEPS || n_inputs < 1 ||
       n_inputs > MI355_CHAIN_MAX_INPUTS || inputs == nullptr || row_strides == nullptr ||
       col_strides == nullptr || rows < 0 || cols < 0)
        return MI355_ERR_BAD_ARG;
    if(steps[0].kind != MI355_CH_LOAD)
        return MI355_ERR_BAD_ARG;
    chain_params p{};
    for(int s = 0; s < n_steps; s++)
    {
        const mi355_chain_step& st = steps[s];
        switch(st.kind)
        {
        case MI355_CH_LOAD:
            if(st.src < 0 || st.src >= n_inputs)
                return MI355_ERR_BAD_ARG;
            break;
        case MI355_CH_BINARY:
            if(st.op < MI355_BIN_ADD || st.op > MI355_BIN_DIV || st.src >= n_inputs || st.src < MI355_CH_SELF)
                return MI355_ERR_BAD_ARG;
            break;
        case MI355_CH_UNARY:
            if(st.op < MI355_UN_ERF || st.op > MI355_UN_NEG)
                return MI355_ERR_BAD_ARG;
            break;
        case MI355_CH_SAVE: break;
        case MI355_CH_ROW_MEAN:
            if(!whole_rows)
                return MI355_ERR_BAD_ARG;
            break;
        default: return MI355_ERR_BAD_ARG;
        }
        p.steps[s] = st;
    }
    if(rows == 0 || cols == 0)
        return MI355_OK;
    const bool quant = qout != nullptr;
    if(out == nullptr && !quant)
        return MI355_ERR_BAD_ARG;
    bool vec = cols % 4 == 0 && (quant ? reinterpret_cast<uintptr_t>(qout) % 4 == 0
                                       : reinterpret_cast<uintptr_t>(out) % 16 == 0);
    for(int i = 0; i < n_inputs; i++)
    {
        if(inputs[i] == nullptr || row_strides[i] < 0 || (col_strides[i] != 0 && col_strides[i] != 1))
            return MI355_ERR_BAD_ARG;
        p.in[i] = inputs[i];
        p.sr[i] = row_strides[i];
        p.sc[i] = cols == 1 ? 0 : col_strides[i];
        if(p.sc[i] == 1 && (row_strides[i] % 4 != 0 || reinterpret_cast<uintptr_t>(inputs[i]) % 16 != 0))
            vec = false;
    }
    p.out     = out;
    p.qout    = qout;
    p.qscale  = qscale;
    p.qzp     = qzp;
    p.rows    = rows;
    p.cols    = cols;
    p.n_steps = n_steps;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    if(whole_rows)
    {
        // one wave per row, four rows per workgroup
        const int64_t blocks = (rows + 3) / 4;
        if(quant || cols > MI355_CHAIN_ROWS_MAX_COLS || blocks > 0x7fffffff)
            return MI355_ERR_UNSUPPORTED;
        const dim3 grid((unsigned)blocks);
        layer_norm_plan plan{};
        if(cols <= 1024 && layer_norm_steps(p, plan))
        {
            if(cols <= 256)
                hipLaunchKernelGGL(layer_norm_rows_kernel<4>, grid, dim3(256), 0, hs, p, plan);
            else if(cols <= 768)
                hipLaunchKernelGGL(layer_norm_rows_kernel<12>, grid, dim3(256), 0, hs, p, plan);
            else
                hipLaunchKernelGGL(layer_norm_rows_kernel<16>, grid, dim3(256), 0, hs, p, plan);
            return mi355_launch_status();
        }
        if(cols <= 256)
            hipLaunchKernelGGL(chain_rows_kernel<4>, grid, dim3(256), 0, hs, p);
        else if(cols <= 768)
            hipLaunchKernelGGL(chain_rows_kernel<12>, grid, dim3(256), 0, hs, p);
        else if(cols <= 1024)
            hipLaunchKernelGGL(chain_rows_kernel<16>, grid, dim3(256), 0, hs, p);
        else if(cols <= 2048)
            hipLaunchKernelGGL(chain_rows_kernel<32>, grid, dim3(256), 0, hs, p);
        else
            hipLaunchKernelGGL(chain_rows_kernel<64>, grid, dim3(256), 0, hs, p);
        return mi355_launch_status();
    }
    // four rows per pass when there are enough rows to keep every CU busy that way
    const int64_t col_blocks = ((vec ? cols / 4 : cols) + 255) / 256;
    const bool rows4         = rows * col_blocks >= 4 * 2048;
    const int64_t row_groups = rows4 ? (rows + 3) / 4 : rows;
    const dim3 grid((unsigned)col_blocks, (unsigned)(row_groups < 65535 ? row_groups : 65535));
    if(quant)
    {
        if(vec && rows4)
            hipLaunchKernelGGL((chain_kernel<4, 4, true>), grid, dim3(256), 0, hs, p);
        else if(vec)
            hipLaunchKernelGGL((chain_kernel<4, 1, true>), grid, dim3(256), 0, hs, p);
        else if(rows4)
            hipLaunchKernelGGL((chain_kernel<1, 4, true>), grid, dim3(256), 0, hs, p);
        else
            hipLaunchKernelGGL((chain_kernel<1, 1, true>), grid, dim3(256), 0, hs, p);
    }
    else if(vec && rows4)
        hipLaunchKernelGGL((chain_kernel<4, 4>), grid, dim3(256), 0, hs, p);
    else if(vec)
        hipLaunchKernelGGL((chain_kernel<4, 1>), grid, dim3(256), 0, hs, p);
    else if(rows4)
        hipLaunchKernelGGL((chain_kernel<1, 4>), grid, dim3(256), 0, hs, p);
    else
        hipLaunchKernelGGL((chain_kernel<1, 1>), grid, dim3(256), 0, hs, p);
    return mi355_launch_status();
}
} // namespace

extern "C" int mi355_chain_f32(const mi355_chain_step* steps,
                               int32_t n_steps,
                               const float* const* inputs,
                               const int64_t* row_strides,
                               const int32_t* col_strides,
                               int32_t n_inputs,
                               float* out,
                               int64_t rows,
                               int64_t cols,
                               void* stream)
{
    return chain_launch(steps, n_steps, inputs, row_strides, col_strides, n_inputs, out, nullptr, nullptr, nullptr,
                        rows, cols, stream);
}

extern "C" int mi355_chain_rows_f32(const mi355_chain_step* steps,
                                    int32_t n_steps,
                                    const float* const* inputs,
                                    const int64_t* row_strides,
                                    const int32_t* col_strides,
                                    int32_t n_inputs,
                                    float* out,
                                    int64_t rows,
                                    int64_t cols,
                                    void* stream)
{
    return chain_launch(steps, n_steps, inputs, row_strides, col_strides, n_inputs, out, nullptr, nullptr, nullptr,
                        rows, cols, stream, true);
}

extern "C" int mi355_chain_f32_q8(const mi355_chain_step* steps,
                                  int32_t n_steps,
                                  const float* const* inputs,
                                  const int64_t* row_strides,
                                  const int32_t* col_strides,
                                  int32_t n_inputs,
                                  const float* scale,
                                  const int8_t* zero_point,
                                  int8_t* out,
                                  int64_t rows,
                                  int64_t cols,
                                  void* stream)
{
    if(scale == nullptr || (out == nullptr && rows > 0 && cols > 0))
        return MI355_ERR_BAD_ARG;
    return chain_launch(steps, n_steps, inputs, row_strides, col_strides, n_inputs, nullptr, out, scale, zero_point,
                        rows, cols, stream);
}

extern "C" int mi355_binary_i32(int32_t op,
                                const int32_t* a,
                                const int64_t* a_strides,
                                const int32_t* b,
                                const int64_t* b_strides,
                                int32_t* out,
                                int32_t ndim,
                                const int64_t* lens,
                                void* stream)
{
    if(op < MI355_BIN_ADD || op > MI355_BIN_MUL || ndim < 1 || ndim > MI355_MAX_DIMS || lens == nullptr ||
       a_strides == nullptr || b_strides == nullptr)
        return MI355_ERR_BAD_ARG;
    bcast_params_i32 p{};
    p.total = 1;
    for(int d = 0; d < ndim; d++)
    {
        if(lens[d] < 0 || a_strides[d] < 0 || b_strides[d] < 0)
            return MI355_ERR_BAD_ARG;
        p.lens[d]      = lens[d];
        p.a_strides[d] = a_strides[d];
        p.b_strides[d] = b_strides[d];
        p.total *= lens[d];
    }
    if(p.total == 0)
        return MI355_OK;
    if(a == nullptr || b == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    p.a    = a;
    p.b    = b;
    p.out  = out;
    p.ndim = ndim;
    p.op   = op;
    hipLaunchKernelGGL(binary_i32_kernel, dim3(blocks_for_n(p.total)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
    return mi355_launch_status();
}

// reduce_max / reduce_min over every element (op/reduce_max.hpp, reduce_min.hpp with all axes: what
// DynamicQuantizeLinear asks for): one workgroup, a correctness path.  op 0: max, 1: min.
__global__ __launch_bounds__(1024) void reduce_all_kernel(const float* in, float* out, int64_t n, int op)
{
    __shared__ float part[1024];
    float v = in[0];
    for(int64_t i = threadIdx.x; i < n; i += 1024)
    {
        const float x = in[i];
        v             = op == 0 ? (v < x ? x : v) : (x < v ? x : v);
    }
    part[threadIdx.x] = v;
    __syncthreads();
    for(int s = 512; s > 0; s >>= 1)
    {
        if((int)threadIdx.x < s)
        {
            const float a = part[threadIdx.x], b = part[threadIdx.x + s];
            part[threadIdx.x] = op == 0 ? (a < b ? b : a) : (b < a ? b : a);
        }
        __syncthreads();
    }
    if(threadIdx.x == 0)
        out[0] = part[0];
}

extern "C" int mi355_reduce_all_f32(int32_t op, const float* in, float* out, int64_t n, void* stream)
{
    if((op != 0 && op != 1) || n <= 0 || in == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    hipLaunchKernelGGL(reduce_all_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream), in, out, n, op);
    return mi355_launch_status();
}

extern "C" int mi355_binary_typed(int32_t op,
                                  int32_t type,
                                  const void* a,
                                  const int64_t* a_strides,
                                  const void* b,
                                  const int64_t* b_strides,
                                  void* out,
                                  int32_t ndim,
                                  const int64_t* lens,
                                  void* stream)
{
    if(op < MI355_BIN_ADD || op > MI355_BIN_DIV || ndim < 1 || ndim > MI355_MAX_DIMS || lens == nullptr ||
       a_strides == nullptr || b_strides == nullptr)
        return MI355_ERR_BAD_ARG;
    const bool integer = type == MI355_I8 || type == MI355_U8;
    if(!integer && type != MI355_F16 && type != MI355_BF16)
        return MI355_ERR_UNSUPPORTED;
    if(integer && op == MI355_BIN_DIV)
        return MI355_ERR_UNSUPPORTED;
    bcast_params_typed p{};
    p.total = 1;
    for(int d = 0; d < ndim; d++)
    {
        if(lens[d] < 0 || a_strides[d] < 0 || b_strides[d] < 0)
            return MI355_ERR_BAD_ARG;
        p.lens[d]      = lens[d];
        p.a_strides[d] = a_strides[d];
        p.b_strides[d] = b_strides[d];
        p.total *= lens[d];
    }
    if(p.total == 0)
        return MI355_OK;
    if(a == nullptr || b == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    p.a    = a;
    p.b    = b;
    p.out  = out;
    p.ndim = ndim;
    p.op   = op;
    p.type = type;
    hipLaunchKernelGGL(binary_typed_kernel, dim3(blocks_for_n(p.total)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
    return mi355_launch_status();
}

extern "C" int mi355_unary_f32(int32_t op, const float* in, float* out, int64_t n, void* stream)
{
    if(op < MI355_UN_ERF || op > MI355_UN_NEARBYINT || n < 0)
        return MI355_ERR_BAD_ARG;
    if(n == 0)
        return MI355_OK;
    if(in == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    if(n % 4 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0)
        hipLaunchKernelGGL(unary4_kernel, dim3(blocks_for_n(n / 4)), dim3(256), 0, static_cast<hipStream_t>(stream),
                           reinterpret_cast<const v4f*>(in), reinterpret_cast<v4f*>(out), n / 4, op);
    else
        hipLaunchKernelGGL(unary_kernel, dim3(blocks_for_n(n)), dim3(256), 0,
                           static_cast<hipStream_t>(stream), in, out, n, op);
    return mi355_launch_status();
}

extern "C" int mi355_reduce_mean_f32(const float* in, float* out, int64_t rows, int64_t cols, void* stream)
{
    if(rows < 0 || cols <= 0)
        return MI355_ERR_BAD_ARG;
    if(rows == 0)
        return MI355_OK;
    if(in == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    if((rows + 3) / 4 > 0x7fffffff)
        return MI355_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(reduce_mean_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), in, out, rows, cols);
    return mi355_launch_status();
}

extern "C" int mi355_softmax_f32(const float* in, float* out, int64_t rows, int64_t cols, void* stream)
{
    if(rows < 0 || cols <= 0)
        return MI355_ERR_BAD_ARG;
    if(rows == 0)
        return MI355_OK;
    if(in == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    if((rows + 3) / 4 > 0x7fffffff)
        return MI355_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)((rows + 3) / 4));
    hipStream_t s = static_cast<hipStream_t>(stream);
    // rows of up to 1024 columns stay in registers: 2, 6, 8 or 16 values per lane
    const int nc = (int)(cols <= 1024 ? cols : 0);
#define MI355_SOFTMAX_ROWS(NV)                                                                              \
    if(nc == 64 * NV)                                                                                       \
        hipLaunchKernelGGL((softmax_rows_kernel<NV, true>), grid, dim3(256), 0, s, in, out, rows, nc);      \
    else                                                                                                    \
        hipLaunchKernelGGL((softmax_rows_kernel<NV, false>), grid, dim3(256), 0, s, in, out, rows, nc)
    if(cols <= 64 * 2)
    {
        MI355_SOFTMAX_ROWS(2);
    }
    else if(cols <= 64 * 6)
    {
        MI355_SOFTMAX_ROWS(6);
    }
    else if(cols <= 64 * 8)
    {
        MI355_SOFTMAX_ROWS(8);
    }
    else if(cols <= 64 * 16)
    {
        MI355_SOFTMAX_ROWS(16);
    }
    else
        hipLaunchKernelGGL(softmax_kernel, grid, dim3(256), 0, s, in, out, rows, cols);
#undef MI355_SOFTMAX_ROWS
    return mi355_launch_status();
}

extern "C" int mi355_gather_rows(const void* table,
                                 const void* ids,
                                 int32_t ids_are_int64,
                                 void* out,
                                 int64_t n_ids,
                                 int64_t table_rows,
                                 int64_t row_bytes,
                                 void* stream)
{
    if(n_ids < 0 || table_rows <= 0 || row_bytes <= 0 || row_bytes % 4 != 0)
        return MI355_ERR_BAD_ARG;
    if(n_ids == 0)
        return MI355_OK;
    if(table == nullptr || ids == nullptr || out == nullptr)
        return MI355_ERR_BAD_ARG;
    const int64_t words = row_bytes / 4;
    const dim3 grid(blocks_for_n(n_ids * words));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if(ids_are_int64)
        hipLaunchKernelGGL(gather_rows_kernel<int64_t>, grid, dim3(256), 0, s,
                           static_cast<const uint32_t*>(table), static_cast<const int64_t*>(ids),
                           static_cast<uint32_t*>(out), n_ids, table_rows, words);
    else
        hipLaunchKernelGGL(gather_rows_kernel<int32_t>, grid, dim3(256), 0, s,
                           static_cast<const uint32_t*>(table), static_cast<const int32_t*>(ids),
                           static_cast<uint32_t*>(out), n_ids, table_rows, words);
    return mi355_launch_status();
}
