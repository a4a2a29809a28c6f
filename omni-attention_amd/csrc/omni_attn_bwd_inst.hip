// One translation unit per (element type, head_dim) of the backward: compiled several times
// with -DOMNI_INST_BF16={0,1} -DOMNI_INST_D={32,64,128}; each object defines the four
// (QB, KB) instances of both backward kernels for that pair behind one C++ symbol.
#include "omni_attn_bwd_kernel.hpp"

#ifndef OMNI_INST_BF16
#error "compile with -DOMNI_INST_BF16=0|1"
#endif
#ifndef OMNI_INST_D
#error "compile with -DOMNI_INST_D=32|64|128"
#endif

namespace omni_attn {

template <bool BF16, int D>
int launch_bwd_blocks(const BwdParams& p, int QB, int KB, hipStream_t stream);

template <>
int launch_bwd_blocks<OMNI_INST_BF16 != 0, OMNI_INST_D>(const BwdParams& p, int QB, int KB,
                                                        hipStream_t stream) {
  constexpr bool BF = OMNI_INST_BF16 != 0;
  constexpr int D = OMNI_INST_D;
  if (QB == 128 && KB == 128) return launch_bwd<BF, D, 128, 128>(p, stream);
  if (QB == 128 && KB == 64) return launch_bwd<BF, D, 128, 64>(p, stream);
  if (QB == 64 && KB == 128) return launch_bwd<BF, D, 64, 128>(p, stream);
  if (QB == 64 && KB == 64) return launch_bwd<BF, D, 64, 64>(p, stream);
  return int(hipErrorInvalidValue);
}

}  // namespace omni_attn
