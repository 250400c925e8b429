// Operators of the mi355 target.  Each compute() fills the C-ABI arguments from the shapes of the
// arguments it was handed, launches on the context's stream and returns its output buffer (the
// last argument), following the device-operator convention of
// src/targets/gpu/include/migraphx/gpu/gemm.hpp:109-128.
#ifndef MIGRAPHX_GUARD_MI355_DEVICE_OPS_HPP
#define MIGRAPHX_GUARD_MI355_DEVICE_OPS_HPP

#include <migraphx/mi355/target.hpp>
#include <migraphx/operation.hpp>
#include <mi355_qgemm.h>

namespace migraphx {
namespace mi355 {

int to_mi355_type(shape::type_t t); // throws for a type the kernels do not take

// How a [..., R, C] tensor maps onto the (pointer, leading dimension, transpose flag, batch
// stride) form the GEMM entry points take.
struct matrix_view
{
    bool ok           = false;
    bool trans        = false; // element (r, c) at c*ld + r instead of r*ld + c
    int64_t rows      = 0;
    int64_t cols      = 0;
    int64_t ld        = 0;
    int64_t batch     = 1;
    int64_t batch_stride = 0;
    int64_t stride_r  = 0; // plain element strides, for entry points that take them
    int64_t stride_c  = 0;
};
matrix_view view_as_matrix(const shape& s);

// strides (row, column) of a tensor seen as [prod(leading dims), last dim]; false when the
// leading dimensions do not collapse into one stride
bool collapse_2d(const shape& s, int64_t& stride_r, int64_t& stride_c);
// true when the dimensions in front of the last two can be walked with one stride
bool batch_collapses(const shape& s);

struct allocate
{
    shape s;
    argument buffer; // set by finalize
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.s, "shape");
    }
    std::string name() const { return "mi355::allocate"; }
    shape compute_shape(const std::vector<shape>&) const { return s; }
    void finalize(migraphx::context&, const shape&, const std::vector<shape>&)
    {
        if(buffer.empty())
            buffer = allocate_device(s);
    }
    argument compute(migraphx::context&, const shape&, const std::vector<argument>&) const;
};

// One block of device memory that holds the program's intermediate buffers (memory_coloring).
struct arena
{
    std::size_t bytes = 0;
    argument buffer; // set by finalize
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.bytes, "bytes");
    }
    std::string name() const { return "mi355::arena"; }
    shape compute_shape(const std::vector<shape>&) const { return shape{shape::uint8_type, {bytes}}; }
    void finalize(migraphx::context&, const shape&, const std::vector<shape>&)
    {
        if(buffer.empty())
            buffer = allocate_device(shape{shape::uint8_type, {bytes}});
    }
    argument compute(migraphx::context&, const shape&, const std::vector<argument>&) const;
};

// A buffer at a fixed place of the arena.  inputs: the arena
struct load
{
    shape s;
    std::size_t offset = 0;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.s, "shape");
        f(self.offset, "offset");
    }
    std::string name() const { return "mi355::load"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context&, const shape&, const std::vector<argument>& args) const
    {
        return args.front().offset(offset, s);
    }
};

// Buffer reuse (the counterpart of src/memory_coloring.cpp with "mi355::allocate" as the allocation
// operator): every mi355::allocate of the lowered program lives from the instruction that writes
// it to the last instruction that reads it or a view of it; allocations whose lives do not overlap
// share memory.  All of them become mi355::load at fixed offsets of one mi355::arena, allocated
// once when the program is finalized.
struct memory_coloring
{
    std::string name() const { return "mi355::memory_coloring"; }
    void apply(module& m) const;
};

struct device_literal
{
    argument data;
    // saved as host bytes: written from a copy of the device buffer, read straight into a new one
    value to_value() const;
    void from_value(const value& v);
    std::string name() const { return "mi355::literal"; }
    shape compute_shape(const std::vector<shape>&) const { return data.get_shape(); }
    argument compute(migraphx::context&, const shape&, const std::vector<argument>&) const
    {
        return data;
    }
};

struct copy_to_device
{
    std::string name() const { return "mi355::copy_to_device"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

struct copy_from_device
{
    std::string name() const { return "mi355::copy_from_device"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape& out, const std::vector<argument>& args) const;
};

// inputs: a, b, [scale_a, scale_b] (dequant), [colsum_b] (zp_a != 0), [rowsum_a] (zp_b != 0),
// [bias: float [N]] (has_bias), out
struct quant_dot
{
    bool dequant           = false;
    bool has_bias          = false;
    bool workspace         = false; // a uint8 buffer before `out` (mi355_quant_dot_workspace_size)
    int64_t zp_a           = 0;
    int64_t zp_b           = 0;
    int64_t scale_a_mode   = MI355_QP_NONE;
    int64_t scale_b_mode   = MI355_QP_NONE;
    shape::type_t out_type = shape::int32_type;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.dequant, "dequant");
        f(self.has_bias, "has_bias");
        f(self.workspace, "workspace");
        f(self.zp_a, "zp_a");
        f(self.zp_b, "zp_b");
        f(self.scale_a_mode, "scale_a_mode");
        f(self.scale_b_mode, "scale_b_mode");
        f(self.out_type, "out_type");
    }
    std::string name() const { return "mi355::quant_dot"; }
    std::size_t expected_inputs() const
    {
        return 3 + (dequant ? 2 : 0) + (zp_a != 0 ? 1 : 0) + (zp_b != 0 ? 1 : 0) + (has_bias ? 1 : 0) +
               (workspace ? 1 : 0);
    }
    mi355_quant_dot_desc describe(const shape& a, const shape& b) const;
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// A constant B of a quant_dot reordered once into the matrix-core operand tiles
// (mi355_quant_dot_prepack).  inputs: b [K, N] (any matrix view), out uint8 [N * K]
struct quant_dot_prepack
{
    template <class Self, class F>
    static void reflect(Self&, F)
    {
    }
    std::string name() const { return "mi355::quant_dot_prepack"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// mi355::quant_dot of at most 16 rows against a reordered B (mi355_quant_dot_prepacked): the
// attributes and inputs of mi355::quant_dot without the workspace, the second input being the
// uint8 buffer mi355::quant_dot_prepack wrote.
struct quant_dot_prepacked
{
    bool dequant           = false;
    bool has_bias          = false;
    int64_t zp_a           = 0;
    int64_t zp_b           = 0;
    int64_t scale_a_mode   = MI355_QP_NONE;
    int64_t scale_b_mode   = MI355_QP_NONE;
    shape::type_t out_type = shape::int32_type;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.dequant, "dequant");
        f(self.has_bias, "has_bias");
        f(self.zp_a, "zp_a");
        f(self.zp_b, "zp_b");
        f(self.scale_a_mode, "scale_a_mode");
        f(self.scale_b_mode, "scale_b_mode");
        f(self.out_type, "out_type");
    }
    std::string name() const { return "mi355::quant_dot_prepacked"; }
    std::size_t expected_inputs() const
    {
        return 3 + (dequant ? 2 : 0) + (zp_a != 0 ? 1 : 0) + (zp_b != 0 ? 1 : 0) + (has_bias ? 1 : 0);
    }
    mi355_quant_dot_desc describe(const shape& a, const shape& out) const;
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: x [N, C, D, H, W], [N, C, H, W] or [N, C, W], weights [O, C / group, window...] (both dense),
// [scale_x (one float), scale_w (one float or one per output channel)] (dequant),
// workspace (uint8, the size mi355_quant_convolution3d_dims reports), out
struct quant_convolution
{
    std::vector<int64_t> padding  = {0, 0};
    std::vector<int64_t> stride   = {1, 1};
    std::vector<int64_t> dilation = {1, 1};
    int64_t group                 = 1;
    bool dequant                  = false;
    int64_t scale_w_mode          = MI355_QP_NONE;
    shape::type_t out_type        = shape::int32_type;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.padding, "padding");
        f(self.stride, "stride");
        f(self.dilation, "dilation");
        f(self.group, "group");
        f(self.dequant, "dequant");
        f(self.scale_w_mode, "scale_w_mode");
        f(self.out_type, "out_type");
    }
    std::string name() const { return "mi355::quant_convolution"; }
    mi355_quant_conv3d_desc describe(const shape& x, const shape& w) const;
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// Float convolution (mi355_convolution_f32, a correctness path).  inputs: x, weights (dense float), out
struct convolution
{
    std::vector<int64_t> padding  = {0, 0};
    std::vector<int64_t> stride   = {1, 1};
    std::vector<int64_t> dilation = {1, 1};
    int64_t group                 = 1;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.padding, "padding");
        f(self.stride, "stride");
        f(self.dilation, "dilation");
        f(self.group, "group");
    }
    std::string name() const { return "mi355::convolution"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: int8 matrix, out (int32 [cols] or [rows])
struct colsum
{
    std::string name() const { return "mi355::colsum"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};
struct rowsum
{
    std::string name() const { return "mi355::rowsum"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: a, b, out
// (with `scaled`: a, b, scale (one float), out -- the result times that value, fp32 only)
struct dot
{
    bool scaled  = false;
    bool fp32acc = false; // fp32 matrix cores: faster, within fp32 accumulation error of the exact sum
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.scaled, "scaled");
        f(self.fp32acc, "fp32acc");
    }
    std::string name() const { return "mi355::dot"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// The four-input quant_dot of block-scaled operands on the block-scaled matrix-core instruction.
// inputs: a [.., M, K] fp8 codes or [.., M, K/2] fp4x2 (standard), b stored as [.., N, K] likewise,
// scale_a, scale_b (float), workspace (uint8, mi355_quant_dot_mx_workspace_size), out float [.., M, N].
// A scale is either a view with the operand's logical shape (scale_a [.., M, K], scale_b [.., K, N],
// any strides: what the operator itself takes) or, with *_compact, a standard [.., rows, K/32] tensor
// of one scale per block.
struct quant_dot_mx
{
    bool a_fp4      = false;
    bool b_fp4      = false;
    bool sa_compact = false;
    bool sb_compact = false;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.a_fp4, "a_fp4");
        f(self.b_fp4, "b_fp4");
        f(self.sa_compact, "sa_compact");
        f(self.sb_compact, "sb_compact");
    }
    std::string name() const { return "mi355::quant_dot_mx"; }
    mi355_mx_dot_desc describe(const std::vector<shape>& inputs) const;
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: a fp16 [M, K], packed weights uint8 [N, K/2], scales fp16 [N, K/group], [zero points], out
struct w4a16_gemm
{
    int64_t group     = 128;
    int64_t zp_mode   = MI355_W4_ZP_SCALAR;
    int64_t zp_scalar = 8;
    bool workspace    = false; // a uint8 buffer before `out` (mi355_w4a16_gemm_workspace_size)
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.group, "group");
        f(self.zp_mode, "zp_mode");
        f(self.zp_scalar, "zp_scalar");
        f(self.workspace, "workspace");
    }
    std::string name() const { return "mi355::w4a16_gemm"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// Constant int4 weights reordered once for the one-row product (mi355_w4a16_prepack).
// inputs: packed weights uint8 [N, K/2], scales fp16 [N, K/128], out uint8 [mi355_w4a16_prepacked_size]
struct w4a16_prepack
{
    int64_t zp_scalar = 8;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.zp_scalar, "zp_scalar");
    }
    std::string name() const { return "mi355::w4a16_prepack"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: a fp16 [M, K] (M <= mi355_w4a16_prepacked_max_rows), reordered weights uint8 [bytes], out fp16 [M, N]
struct w4a16_gemm_prepacked
{
    template <class Self, class F>
    static void reflect(Self&, F)
    {
    }
    std::string name() const { return "mi355::w4a16_gemm_prepacked"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: x, scale view, [zero point view], out
struct quantizelinear
{
    shape::type_t out_type = shape::uint8_type;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.out_type, "out_type");
    }
    std::string name() const { return "mi355::quantizelinear"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

struct dequantizelinear
{
    std::string name() const { return "mi355::dequantizelinear"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: x, out.  The packed axis is the last one.
struct unpack_int4
{
    int64_t axis = -1; // the packed axis; any strided (also broadcast) input view is taken as it is
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "mi355::unpack_int4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};
struct pack_int4
{
    int64_t axis = -1; // the packed axis; any strided (also broadcast) input view is taken as it is
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.axis, "axis");
    }
    std::string name() const { return "mi355::pack_int4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: x (fp4x2), out (fp8e4m3fn) / x (float), out (fp4x2).  The packed axis is the last one.
struct unpack_fp4
{
    std::string name() const { return "mi355::unpack_fp4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};
struct pack_fp4
{
    std::string name() const { return "mi355::pack_fp4"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

struct convert
{
    shape::type_t target_type = shape::half_type;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.target_type, "target_type");
    }
    std::string name() const { return "mi355::convert"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: a, b (views with any strides, broadcast included), out
struct binary
{
    int64_t op = MI355_BIN_ADD;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.op, "op");
    }
    std::string name() const { return "mi355::binary"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: x, out
struct unary
{
    int64_t op = MI355_UN_ERF;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.op, "op");
    }
    std::string name() const { return "mi355::unary"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// A chain of binary and unary float operators evaluated element by element in one kernel.
// inputs: x0 .. x(n-1) (views of the output's dimensions whose strides collapse to a row stride
// and a column stride of 0 or 1), out.  `steps` holds kind, op, src, reversed for every step of
// the register machine mi355_chain_f32 describes.
struct chain
{
    std::vector<int64_t> steps;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.steps, "steps");
    }
    std::string name() const { return "mi355::chain"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// The same chain with a per-tensor quantizelinear to int8 as its last operation (the float value is
// not stored).  inputs: the chain's inputs, scale (float, every element the same: any broadcast of one
// value), zero point (int8, likewise) when has_zero_point, out (dense int8)
struct chain_q8
{
    std::vector<int64_t> steps;
    bool has_zero_point = false;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.steps, "steps");
        f(self.has_zero_point, "has_zero_point");
    }
    std::string name() const { return "mi355::chain_q8"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// The chain with MI355_CH_ROW_MEAN steps (the mean over the last axis, in every column of the row):
// a layer normalisation in one kernel, a whole row in the registers of one wave.  inputs: tensors of
// the result's dimensions or with one value per row (last dimension 1), then out (dense float, rows
// of at most MI355_CHAIN_ROWS_MAX_COLS elements)
struct chain_rows
{
    std::vector<int64_t> steps;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.steps, "steps");
    }
    std::string name() const { return "mi355::chain_rows"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: x (standard), out; over the last axis
struct reduce_mean
{
    std::string name() const { return "mi355::reduce_mean"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};
// reduce_max (op 0) / reduce_min (op 1) over every element.  inputs: x (dense float), out (one element)
struct reduce_all
{
    int64_t op = 0;
    template <class Self, class F>
    static void reflect(Self& self, F f)
    {
        f(self.op, "op");
    }
    std::string name() const { return "mi355::reduce_all"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};
struct softmax
{
    std::string name() const { return "mi355::softmax"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

// inputs: table (standard), indices (standard int32 / int64), out; along axis 0
struct gather
{
    std::string name() const { return "mi355::gather"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

struct contiguous
{
    std::string name() const { return "mi355::contiguous"; }
    shape compute_shape(const std::vector<shape>& inputs) const;
    argument compute(migraphx::context& ctx, const shape&, const std::vector<argument>& args) const;
    std::ptrdiff_t output_alias(const std::vector<shape>& s) const { return s.size() - 1; }
};

} // namespace mi355
} // namespace migraphx
#endif
