// bf16 MFMA backward kernels (placeholder until the two-pass kernels land).
#include "sba_mfma.h"
bool sba_mfma_bwd_available() { return false; }
int sba_launch_mfma_bwd(const sba::KParams&, hipStream_t) { return SBA_ERR_LAUNCH; }
