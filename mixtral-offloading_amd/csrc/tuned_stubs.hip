// placeholders until the tuned kernel families land
#include "hqq_common.hpp"
namespace hqq {
bool vec3_supported(const hqq_linear *, int64_t) { return false; }
size_t vec3_workspace_bytes(const hqq_linear *, int64_t) { return 0; }
int launch_vec3_matmul(const hqq_linear *, const f16 *, int64_t, f16 *, void *, size_t, hipStream_t) { return HQQ_E_UNSUPPORTED; }
}
