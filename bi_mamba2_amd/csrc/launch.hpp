// Host-side declarations shared by the kernel files and the C ABI.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/bimamba2.h"

namespace bm2 {

static inline int check_launch() { return hipGetLastError() == hipSuccess ? BIMAMBA2_OK : BIMAMBA2_ELAUNCH; }

// Width of the headdim column tile of the chunk-scan kernels (64 columns for 16-bit types, 32 for float32, less for narrow
// heads), and with it the number of planes of ddt_direct: every column tile of the dx kernel writes the row sums of its own
// columns to its own (batch, nheads, nchunks, chunk_size) plane, and the reader adds the planes in order (no atomics).
__host__ __device__ inline int scan_col_tile_of(int headdim, int dtype) {
    return headdim <= 16 ? 16 : (headdim <= 32 || dtype == BIMAMBA2_F32) ? 32 : 64;
}
__host__ __device__ inline int ddt_direct_planes(const bimamba2_params &p) {
    const int pw = scan_col_tile_of(p.headdim, p.dtype);
    return (p.headdim + pw - 1) / pw;
}

int launch_chunk_cumsum_fwd(const bimamba2_params *p);
int launch_bmm_chunk_fwd(const bimamba2_params *p);
int launch_chunk_state(const bimamba2_params *p, bool dstates, bool cumsum = false);   // cumsum: also does the chunk cumsum
bool chunk_state_does_cumsum(const bimamba2_params *p);
// the forward pass may keep its per-chunk states in states16_f/b only (16-bit type, no float32 state tensors)
bool chunk_states_in_16bit(const bimamba2_params *p);
// the chunk-state kernel whose workgroups walk through several heads of one (batch, chunk): where it is used, and its launch
bool chunk_state_uses_heads_kernel(const bimamba2_params *p);
int launch_chunk_state_heads(const bimamba2_params *p);
int launch_state_passing_fwd(const bimamba2_params *p);
int launch_chunk_scan(const bimamba2_params *p, bool bwd);
// the 16-bit kernel of kernels_scan16.hip (launch_chunk_scan picks it where it applies)
int launch_chunk_scan16(const bimamba2_params *p, bool bwd);
// heads of one group that a workgroup of that kernel walks through (they share one C.B^T product)
int chunk_scan16_heads_per_workgroup(const bimamba2_params *p);
// whether launch_chunk_scan() would pick that kernel for this problem (the 16-bit copies of the entering states given)
bool chunk_scan_uses_scan16(const bimamba2_params *p, bool bwd);
// true when that launch recomputes CB (bwd: CB^T) from the C and B rows instead of reading it
bool scan_recomputes_cb(const bimamba2_params *p, bool bwd);
// true when the dCB launch can rebuild its CB tiles from the C and B rows (then CB may be NULL)
bool dcb_recomputes_cb(const bimamba2_params *p);

int launch_bwd_dz(const bimamba2_params *p);
bool bwd_dz_dstates_fused(const bimamba2_params *p);   // dz and dstates as one launch
int launch_bwd_dz_dstates(const bimamba2_params *p);
int launch_state_passing_bwd(const bimamba2_params *p);
int launch_bwd_dbdc(const bimamba2_params *p, bool is_db);
int launch_bwd_dcb(const bimamba2_params *p);
int dcb_slices(const bimamba2_params *p);   // head slices whose dCB partial sums the kernel keeps apart
int launch_bmm_chunk_bwd(const bimamba2_params *p);
// out[j] = sum_i sum_k in[(i*nj + j)*nk + k]
struct ReduceJob { const float *in; float *out; int ni, nj, nk; };
struct ReduceJobs { ReduceJob job[4]; int n = 0; };
int launch_reduce_jobs(const ReduceJobs &jobs, hipStream_t stream);
// defer != NULL: the final reductions of dA and ddt_bias are appended to *defer instead of being launched
int launch_chunk_cumsum_bwd(const bimamba2_params *p, ReduceJobs *defer = nullptr);
// bmm_chunk_bwd and chunk_cumsum_bwd as one launch, where bwd_tail_merged() says it exists
// the dCB kernel and the backward state passing as one launch, where bwd_dcb_sp_merged() says it exists
bool bwd_dcb_sp_merged(const bimamba2_params *p);
// out16 / in16: dCB and dCBT in the element type of the inputs between the two launches (one head slice: the reader rounds
// them to that type anyway)
int launch_bwd_dcb_sp(const bimamba2_params *p, bool out16 = false);
bool bwd_tail_merged(const bimamba2_params *p);
int launch_bwd_tail(const bimamba2_params *p, ReduceJobs *defer, bool in16 = false);
int launch_fill(float *ptr, size_t n, float value, hipStream_t stream);
// out[j] = sum_{i<ni} sum_{k<nk} in[(i*nj + j)*nk + k]
int launch_reduce(const float *in, float *out, int ni, int nj, int nk, hipStream_t stream);

// gated RMSNorm (kernels_norm.hip)
int launch_rmsnorm_gated(const bimamba2_norm_params *p, bool bwd);
size_t norm_workspace_bytes(const bimamba2_norm_params *p);
// out[j] = sum_i in[i * nj + j], fixed order
int launch_colsum(const float *in, float *out, int ni, int nj, hipStream_t stream);

// depthwise conv1d + SiLU (kernels_conv.hip)
int launch_conv1d_silu(const bimamba2_conv_params *p, bool bwd);
size_t conv_workspace_bytes(const bimamba2_conv_params *p);
// several small element-wise conversions in one launch (kernels_conv.hip)
int launch_cast_many(const bimamba2_cast_params *p);

}  // namespace bm2
