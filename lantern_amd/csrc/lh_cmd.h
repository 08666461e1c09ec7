// The command of the command list and the operations it can stand for: plain C++ (no device headers), so that the host-side
// analysis of a recorded buffer (lh_cmdlist_levels.h) can be built and checked on its own.
#pragma once
#include <stdint.h>
namespace lh {
enum {
  CL_ZERO16 = 0, CL_FILL, CL_COPY, CL_GEAM, CL_SCALAR, CL_BIN, CL_ACC, CL_ACCNEG, CL_ACCMUL, CL_UNARY, CL_UNARY_GRAD,
  CL_GEMV_N, CL_GEMV_T, CL_GER, CL_DOT, CL_AXPY_DEV, CL_SOFTMAX, CL_SOFTMAX_GRAD, CL_NLL, CL_NLL_GRAD, CL_ADAGRAD, CL_SGD
};
struct LhCmd { int32_t op, i0, i1, i2; float f0, f1, f2, f3; void* p0; void* p1; void* p2; void* p3; };   // 64 bytes
constexpr int64_t REC_MAX_ELEMS = 1 << 16;        // element-wise operands up to this many elements are recorded
constexpr int64_t REC_MAX_MATRIX = 1 << 17;       // matrix-vector operands up to this many matrix elements
constexpr int CL_BUF_CMDS = 2048;                 // commands per host buffer: a full buffer is launched while the host records the next
}  // namespace lh
