// Large aligned int8 Gemm: software-pipelined MFMA kernel (placeholder dispatcher for now).
#include "epilogues.h"
#include "mfma_tile.h"

namespace ncnnhip {

int launch_gemm_int8_pipelined(const int8_t*, size_t, const int8_t*, size_t, int, int, int, const GemmEpilogue&, hipStream_t, bool* handled)
{
    *handled = false;
    return NCNNHIP_OK;
}

} // namespace ncnnhip
