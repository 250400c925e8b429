#ifndef MIGRAPHX_GUARD_MAKE_OP_HPP
#define MIGRAPHX_GUARD_MAKE_OP_HPP
#include <migraphx/register_op.hpp>
#endif
