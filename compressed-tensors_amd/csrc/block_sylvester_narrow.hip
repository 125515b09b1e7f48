// block (x) Sylvester transforms: the kernels for bfloat16 tensors, Sylvester factors of 4, 8 and 16.
#include "block_sylvester_impl.h"

namespace ctmi {

CTMI_BS_ENTRY(bs_narrow_bf16) { return bs_narrow<false>(tab, inner, ma_t, k, sign_in, sign_out, scale, st); }

}  // namespace ctmi
