// placeholder until the MFMA kernel lands
#include "common.h"
namespace mi355 {
bool mfma_supported(int, int, int, int, int, int, int, float) { return false; }
int mfma_num_parts(int, int, int) { return 0; }
size_t mfma_workspace_bytes(int, int, int, int) { return 0; }
const char* launch_mfma(const DecodeParams&, int, int, hipStream_t) { return "MFMA kernel not built"; }
}  // namespace mi355
