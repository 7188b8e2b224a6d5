// Entry points that one source file of the library offers another; not part of the C ABI.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "../../include/fp8gmm.h"

namespace fp8gmm {

// fp8gmm_multi_quantize / fp8gmm_multi_cast_dgelu without their second launch, the one that merges the tensors'
// running maxima into the callers' amax slots: the caller hands the table to the GEMM launch that follows
// (launch_gemm_merging), whose first workgroup does the merge before it starts on its tiles.  Two small launches
// fewer per pass of a module.
int launch_cast_unmerged(fp8gmm_tensor_desc* descs_dev, int n, int total_blocks, int out_fmt, bool dgelu, void* stream);

// fp8gmm_grouped_gemm, with the amax merge of the `merge_n` cast descriptors at `merge_descs` in front.
int launch_gemm_merging(const fp8gmm_gemm_problem* probs_dev, int n, const fp8gmm_gemm_item* items_dev,
                        const fp8gmm_gemm_fixup_desc* fixups_dev, const fp8gmm_gemm_plan* plan, int a_fmt, int b_fmt,
                        int out_kind, int epilogue, void* workspace, size_t workspace_bytes,
                        const fp8gmm_tensor_desc* merge_descs, int merge_n, void* stream);

}  // namespace fp8gmm
