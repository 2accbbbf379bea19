// The 2:4 matmul kernels of spmm_kernels.hpp instantiated for e4m3_t operands.
#include "spmm_kernels.hpp"

namespace tf24 {
int spmm_e4m3(TF24_SPMM_ENTRY_ARGS) { return dispatch_out<e4m3_t>(TF24_SPMM_ENTRY_PASS); }
}  // namespace tf24
