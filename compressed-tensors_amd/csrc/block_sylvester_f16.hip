// block (x) Sylvester transforms: the kernels for float16 tensors, Sylvester factors of 32, 64 and 128.
#include "block_sylvester_impl.h"

namespace ctmi {

CTMI_BS_ENTRY(bs_wide_f16) { return bs_wide<true>(tab, inner, ma_t, k, sign_in, sign_out, scale, st); }

}  // namespace ctmi
