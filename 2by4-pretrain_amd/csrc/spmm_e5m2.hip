// The 2:4 matmul kernels of spmm_kernels.hpp instantiated for e5m2_t operands.
#include "spmm_kernels.hpp"

namespace tf24 {
int spmm_e5m2(TF24_SPMM_ENTRY_ARGS) { return dispatch_out<e5m2_t>(TF24_SPMM_ENTRY_PASS); }
}  // namespace tf24
