// The 2:4 matmul kernels of spmm_kernels.hpp instantiated for f16_t operands.
#include "spmm_kernels.hpp"

namespace tf24 {
int spmm_f16(TF24_SPMM_ENTRY_ARGS) { return dispatch_out<f16_t>(TF24_SPMM_ENTRY_PASS); }
}  // namespace tf24
