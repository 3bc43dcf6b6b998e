// MFMA tile kernel for block-sparse attention (placeholder until the tile kernel lands).
#include "bsa.hpp"

namespace hipattn {
int bsa_mfma_launch(const BsaParams &, int, int, hipStream_t) { return HIPATTN_E_UNSUPPORTED; }
}  // namespace hipattn
