// Block-prefill full attention for gfx950.  Operators registered here, with the
// reference kernels whose argument tables they accept
// (src/backend/metal/kernels/prefill_attention.metal): attn_qk_rope_blk (:1).
#include "../tt_internal.h"

namespace tt {

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side tables of launchers
const KernelDesc kAttentionPrefillKernels[] = {
    {"attn_qk_rope_blk", op_attn_qk_rope_blk},
};
const uint32_t kAttentionPrefillKernelCount =
    sizeof(kAttentionPrefillKernels) / sizeof(kAttentionPrefillKernels[0]);

#endif

}  // namespace tt
