#include "launch.hpp"
namespace tri {
bool mfma_supported(int, const KParams&) { return false; }
int launch_mfma_fwd(int, const KParams&, hipStream_t) { return TRI_ATTN_ESHAPE; }
int launch_mfma_dq(int, const KParams&, hipStream_t) { return TRI_ATTN_ESHAPE; }
int launch_mfma_dkdv(int, const KParams&, hipStream_t) { return TRI_ATTN_ESHAPE; }
int launch_delta(int dtype, const KParams& p, hipStream_t s) { return launch_generic_any(kGenericDelta, dtype, p, s); }
}
