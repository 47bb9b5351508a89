/* C ABI of libbimamba2_hip.so: the bidirectional SSD operator of Bi-Mamba2 for AMD MI355X (gfx950).
 *
 *   y = SS(x) + flip(SS(flip(x))) + D*x   [* silu(z)]          forward and backward
 *
 * Every entry point takes one `const bimamba2_params*`, enqueues its kernels on `stream` and returns
 * immediately (no host synchronisation, no device allocation, no global state).  Return value: 0 on
 * success, a negative BIMAMBA2_E* code otherwise (bimamba2_strerror() gives the text).  All pointers are
 * device pointers; the caller owns every buffer, including the intermediates and the workspace.
 *
 * Each declaration cites the function of the reference project (Hprairie/Bi-Mamba2, paths relative to its
 * root) that it replaces.
 *
 * Layouts (row-major, sizes in elements; B=batch L=seqlen H=nheads P=headdim G=ngroups N=dstate
 * Q=chunk_size nc=ceil(L/Q)):
 *   x, z, out, out_x, dout, dx, dz   (B, L, H, P)   element type `dtype`; last-dim stride 1, the other three
 *                                                   strides given for the inputs x, z, dout; outputs contiguous
 *   Bm, Cm, dB, dC                   (B, L, G, N)   element type `dtype`; input strides given; outputs contiguous
 *   dt, ddt                          (B, L, H)      element type `dt_dtype`; strides given for dt; ddt contiguous
 *   A, D, dt_bias, dA, dD, ddt_bias  (H,) [D, dD may be (H, P)]   float32, contiguous
 *   dt_out, cs_f, cs_b, u_f, u_b, v_f, v_b   (B, H, nc, Q)   float32; ddt_direct: bimamba2_ddt_direct_planes() such planes
 *   CB, CBT, dCB                     (B, nc, G, Q, Q)   float32, CB[.., l, s] = C_l . B_s, CBT its transpose
 *   states_f/b, dstates_f/b          (B, nc, H, P, N)   float32 (states16_*, dstates16_*: the same shape in `dtype`)
 *   final_f, final_b                 (B, H, P, N)       float32
 */
#ifndef BIMAMBA2_H
#define BIMAMBA2_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { BIMAMBA2_F32 = 0, BIMAMBA2_BF16 = 1, BIMAMBA2_F16 = 2 };

enum {
    BIMAMBA2_OK = 0,
    BIMAMBA2_EINVAL = -1,      /* null pointer / inconsistent dimensions */
    BIMAMBA2_EUNSUPPORTED = -2,/* shape or dtype outside what the kernels are built for */
    BIMAMBA2_EWORKSPACE = -3,  /* workspace missing or too small */
    BIMAMBA2_ELAUNCH = -4,     /* HIP reported a launch error */
    BIMAMBA2_ESCRATCH = -5     /* bimamba2_fwd_static: the problem needs more than BIMAMBA2_STATIC_SCRATCH_BYTES */
};

/* limits of the compiled kernels */
#define BIMAMBA2_MAX_CHUNK 256
#define BIMAMBA2_MIN_CHUNK 32   /* same lower bound as the reference (src/ssd/bi/ssd_combined.py:306) */
#define BIMAMBA2_MAX_HEADDIM 128
#define BIMAMBA2_MAX_DSTATE 256

/* Added to the decay exponent across a change of seq_idx: every factor across a boundary carries e^-20 = 2e-9, below
 * float32 resolution next to the terms it is added to.  The cumulative sums of a chunk grow by this much per boundary
 * inside it, and their float32 resolution with them: relative accuracy of the in-sequence decays about 1.2e-6 per boundary
 * in the chunk, so a float32 contract of 1e-4 holds up to about 40 boundaries per chunk.  The library does not count
 * boundaries: a caller whose sequences can be shorter than chunk_size / 32 positions on average picks a smaller chunk_size
 * (the result does not depend on it); the Python host does so for at most 32 boundaries per chunk. */
#define BIMAMBA2_SEQ_CUT (-20.0f)

typedef struct bimamba2_params {
    /* problem */
    int32_t batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size;
    int32_t dtype;          /* BIMAMBA2_* : x, z, Bm, Cm, out, out_x, dout and their gradients */
    int32_t dt_dtype;       /* BIMAMBA2_* : dt and ddt */
    int32_t has_D, D_has_hdim, has_z, has_dt_bias, dt_softplus;
    int32_t fwd_saved;      /* bimamba2_bwd only: dt_out, cs_f, cs_b, states_f, states_b hold what bimamba2_fwd left in
                               them, so the backward pass does not recompute them (CB is always recomputed) */
    int32_t causal;         /* 0: the bidirectional operator.  1: the single-direction (causal) operator built from the same
                               kernels with the reverse direction left out - the comparator the bidirectional pass is
                               timed against.  Every entry point follows it, but only for the shapes whose scan
                               kernels rebuild CB (bimamba2_chunk_scan_reads_cb() == 0): BIMAMBA2_EUNSUPPORTED otherwise.
                               The reverse direction's buffers (states_b, dstates_b, u_b, v_b, ddA_chunk_b) are neither
                               written nor used; final_b must be NULL. */
    float dt_min, dt_max;
    /* element strides of the strided inputs (last dim contiguous) */
    int64_t x_sb, x_sl, x_sh;
    int64_t z_sb, z_sl, z_sh;
    int64_t dout_sb, dout_sl, dout_sh;
    int64_t B_sb, B_sl, B_sg;
    int64_t C_sb, C_sl, C_sg;
    int64_t dt_sb, dt_sl, dt_sh;
    /* inputs */
    const void *x, *dt, *Bm, *Cm, *z, *dout;
    const float *A, *D, *dt_bias;
    /* forward outputs */
    void *out, *out_x;
    float *final_f, *final_b;   /* optional */
    /* backward outputs */
    void *dx, *ddt, *dB, *dC, *dz;
    float *dA, *dD, *ddt_bias;
    /* intermediates (caller-owned; the composite entry points carve them from `workspace` when NULL) */
    float *dt_out, *cs_f, *cs_b;
    float *CB;
    float *dCB;                     /* room for min(4, max(1, H/G/32)) copies: head-slice partial sums, added up in place */
    float *CBT;                     /* optional: CB transposed per chunk, CBT[.., s, l] = CB[.., l, s] */
    float *dCBT;                    /* dCB transposed per chunk (same number of copies as dCB) */
    float *states_f, *states_b;     /* chunk states, overwritten in place by the inter-chunk scan */
    float *dstates_f, *dstates_b;
    void *dout_x;                   /* dout * silu(z), element type `dtype` */
    float *ddt_direct, *u_f, *u_b, *v_f, *v_b;     /* ddt_direct: bimamba2_ddt_direct_planes() planes of (B, H, nc, Q) */
    float *da_intra;                    /* (B, H, nc, T*T, 2, 64), T = ceil(Q/64): per-tile column / row sums */
    float *ddA_chunk_f, *ddA_chunk_b;   /* (B, H, nc, ceil(P*N/1024)) partial sums */
    float *dBs, *dCs;                   /* (S, B, L, G, N) float32 partial gradients, S = ceil(H/G/8) head slices */
    float *red;                         /* scratch for two-stage reductions: max(B*nc*H*P, 2*B*nc*H) floats for the single
                                           stages, B*nc*H*P + 2*B*nc*H for bimamba2_bwd */
    /* States at the ends of the sequence, all (B, H, P, N) float32, all optional (NULL = absent).  The reference's
       bidirectional path has neither initial states nor a backward pass through its final states
       (README.md:66, src/ssd/bi/ssd_combined.py:571 there); they are what chunked / streaming use and a split of the
       sequence over devices need.
       initial_f: state of the forward recurrence in front of position 0 (instead of 0);
       initial_b: state of the reverse recurrence behind position L-1.
       dfinal_f, dfinal_b (backward): gradients with respect to final_f, final_b.
       dinitial_f, dinitial_b (backward, outputs): gradients with respect to initial_f, initial_b. */
    const float *initial_f, *initial_b;
    const float *dfinal_f, *dfinal_b;
    float *dinitial_f, *dinitial_b;
    /* Packed sequences (optional): seq_idx (B, L) int32, constant over each of the sequences packed one behind the other
       along L.  Positions with different seq_idx do not interact: neither recurrence carries state across a change.
       The bidirectional reference has no such argument (its causal sibling has, src/ssd/uni/ssd_combined.py there).
       It is applied where the decay exponents are formed (bimamba2_chunk_cumsum_fwd, or bimamba2_fwd / bimamba2_bwd):
       the forward cumulative sum gets BIMAMBA2_SEQ_CUT added at the first position of a sequence, the reverse one at
       the last, so that every decay factor across a change underflows to zero and no other kernel needs to know. */
    const int32_t *seq_idx;
    /* Optional 16-bit copies of the states that enter the chunks (element type `dtype`, which must be a 16-bit one;
       same shape as states_* / dstates_*).  Every kernel that reads entering states rounds them to `dtype` for its MFMA
       anyway; kept in that type they cost half the memory traffic.  When states16_f / states16_b are given,
       bimamba2_state_passing_fwd writes the entering states there and leaves the per-chunk states in states_f / states_b
       as they were, and bimamba2_chunk_scan_fwd, bimamba2_chunk_scan_bwd_dc and bimamba2_state_passing_bwd read them
       from there.  dstates16_f / dstates16_b likewise: written by bimamba2_state_passing_bwd (dstates_f / dstates_b keep
       the per-chunk gradients), read by bimamba2_chunk_scan_bwd_dx and bimamba2_chunk_state_bwd_db.  Only the kernels for
       16-bit dtype, dstate 64, headdim % 64 == 0, chunk_size % 64 == 0 and 16-byte aligned operands know them
       (bimamba2_state_copies() == 1); the others return BIMAMBA2_EUNSUPPORTED when they are set - except the two
       forward stages: bimamba2_state_passing_fwd writes, and bimamba2_chunk_scan_fwd reads, states16_* for every 16-bit
       problem with headdim * dstate % 4 == 0 and 16-byte aligned state tensors.
       bimamba2_fwd / bimamba2_bwd use such copies on their own, from the workspace, where the caller leaves states_f
       resp. dstates_f NULL (does not ask for the float32 entering states); a caller that keeps the forward's intermediates
       for the backward pass (fwd_saved) then passes states16_f / states16_b to both instead of states_f / states_b.
       bimamba2_fwd does so for every 16-bit problem (a forward pass without kept states has the scan stage as the only
       reader), bimamba2_bwd where bimamba2_state_copies() == 1.
       Without the float32 tensors: with states_f = states_b = NULL and states16_* given (16-bit dtype, headdim and dstate
       multiples of 64, chunk_size % 32 == 0, aligned operands, not causal), bimamba2_chunk_state_fwd writes the per-chunk
       states to states16_* in `dtype` and bimamba2_state_passing_fwd turns them into the entering states in place; with
       dstates_f = dstates_b = NULL and dstates16_* given (bimamba2_state_copies() == 1), bimamba2_chunk_scan_bwd_dstates /
       _dz_dstates write the per-chunk gradients to dstates16_* and bimamba2_state_passing_bwd (which then needs states16_*
       as well) replaces them in place.  The values are rounded to `dtype` once more than with the float32 tensors (the
       per-chunk value before the inter-chunk scan adds it up in float32).  bimamba2_fwd and bimamba2_bwd work this way
       whenever they own the state tensors: no float32 state tensor is written or read in a 16-bit pass.
       The reference keeps its entering states in the input dtype as well (out_dtype=C.dtype, src/ssd/bi/ssd_combined.py:324-327). */
    void *states16_f, *states16_b;
    void *dstates16_f, *dstates16_b;
    void *workspace;
    size_t workspace_bytes;
    void *stream;                   /* hipStream_t */
    /* Element strides (batch, position) of the gradients dx (batch, seqlen, nheads, headdim), dB and dC (batch, seqlen,
       ngroups, dstate); the inner dimensions are always contiguous.  A position stride of 0 (the default) means the
       contiguous tensor.  With strides the three can be slices of one (batch, seqlen, channels) buffer, as x, B and C are
       slices of the convolution's output in the BiMamba2 layer: no concatenation of the gradients afterwards.  Multiples of
       8 elements (16 bytes) where the vector kernels are to run. */
    int64_t dx_sb, dx_sl, dB_sb, dB_sl, dC_sb, dC_sl;
} bimamba2_params;

/* text of an error code */
const char *bimamba2_strerror(int code);
/* library version (major*10000 + minor*100 + patch) */
int bimamba2_version(void);
/* sizeof(bimamba2_params) as compiled into the library, for bindings to check their mirror of the struct */
size_t bimamba2_params_size(void);

/* bytes of workspace the composite entry points need (is_bwd = 0: forward, 1: backward) */
size_t bimamba2_workspace_bytes(const bimamba2_params *p, int is_bwd);

/* 1 if the kernels of this problem can keep the entering states in 16-bit copies (see states16_f), else 0 */
int bimamba2_state_copies(const bimamba2_params *p);

/* Whether a kernel of this problem reads CB (1) or rebuilds the CB tiles it needs from the C and B rows with MFMAs (0):
 *   which = 0: bimamba2_chunk_scan_fwd reads CB      (0 for 16-bit dtype, dstate 64, headdim % 64 == 0, chunk_size % 32 == 0;
 *              also 0 at dstate 128 when states16_* are set, i.e. when the persistent scan kernel runs)
 *   which = 1: bimamba2_chunk_scan_bwd_dx reads CBT  (0 for 16-bit dtype, dstate 64, headdim % 64 == 0, chunk_size % 32 == 0)
 *   which = 2: bimamba2_chunk_scan_bwd_dcb reads CB  (0 for 16-bit dtype, dstate % 32 == 0, headdim % 64 == 0, chunk_size % 64 == 0)
 *   which = 3: (not about CB) 1 when bimamba2_fwd launches bimamba2_chunk_cumsum_fwd on its own, 0 when its chunk-state
 *              launch does the cumsum as well (16-bit dtype, headdim and dstate multiples of 64, chunk_size % 32 == 0)
 * always with 16-byte aligned operands.  When it is 0 a caller of the single stages may pass that pointer as NULL; when
 * the first three are 0, bimamba2_bmm_chunk_fwd is not needed at all.  Fuses _bmm_chunk_fwd (src/ssd/bi/ssd_bmm.py:163-208)
 * into its consumers for those shapes. */
int bimamba2_chunk_scan_reads_cb(const bimamba2_params *p, int which);

/* Planes of ddt_direct: the dx kernel works on headdim column tiles (64 columns for 16-bit types, 32 for float32) and
 * every tile writes the row sums of its own columns into its own (B, H, nc, Q) plane, plane k at ddt_direct + k*B*H*nc*Q;
 * bimamba2_chunk_cumsum_bwd called with the same headdim adds them in order.  1 for headdim <= 64 (16-bit) / 32 (float32).
 * (The reference adds the tiles with atomics, src/ssd/bi/ssd_combined.py:232.) */
int bimamba2_ddt_direct_planes(const bimamba2_params *p);

/* Heads of one group that one workgroup of bimamba2_chunk_scan_fwd (bwd = 0) or bimamba2_chunk_scan_bwd_dx (bwd = 1)
 * works through when it rebuilds C.B^T itself: the product is formed once per workgroup and shared by these heads, so the
 * flops a launch executes for it are (batch * nchunks * nheads / this) * 2 * Q * Q * N.  1 for the kernels that read CB or
 * rebuild it per head.  A measurement aid (the reference has no counterpart: its _bmm_chunk_fwd computes CB once per group,
 * src/ssd/bi/ssd_bmm.py:163-208). */
int bimamba2_chunk_scan_heads_per_workgroup(const bimamba2_params *p, int bwd);

/* Whole forward; replaces _mamba_chunk_scan_combined_fwd (src/ssd/bi/ssd_combined.py:297-331).
 * Needs: x dt A Bm Cm [D z dt_bias] out [out_x when has_z] [final_f final_b] workspace.  Intermediates given as
 * non-NULL pointers (dt_out cs_f cs_b CB CBT states_f states_b) are filled in place of workspace memory, so a
 * caller can keep them for the backward pass (CB and CBT are only computed when given or when the scan kernel
 * reads them). */
int bimamba2_fwd(const bimamba2_params *p);

/* bimamba2_fwd for callers that cannot allocate device memory or bring a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its wrappers allocate every
 * intermediate with torch.empty).  Same arguments, same kernels and bit for bit the same results as bimamba2_fwd, but
 * `workspace` / `workspace_bytes` are ignored: the intermediates that the caller does not bring live in a buffer of
 * BIMAMBA2_STATIC_SCRATCH_BYTES that is part of the library's device image (each GPU the library runs on holds one until
 * the process ends).  Calls no hipMalloc / hipFree or any other allocating routine.  Returns BIMAMBA2_ESCRATCH when
 * bimamba2_workspace_bytes(p, 0) exceeds the buffer.  All calls on one GPU share that GPU's buffer: calls that overlap
 * on one GPU (two streams, two host threads) race; calls on one stream, one after the other, are safe. */
#define BIMAMBA2_STATIC_SCRATCH_BYTES (64u << 20)
int bimamba2_fwd_static(const bimamba2_params *p);

/* Whole backward; replaces _mamba_chunk_scan_combined_bwd (src/ssd/bi/ssd_combined.py:334-475).
 * Needs: the forward inputs, dout, out_x (pre-gate output, when has_z), dx ddt dA dB dC [dD dz ddt_bias],
 * workspace.  With fwd_saved = 0 it recomputes the forward intermediates as the reference does; with
 * fwd_saved = 1 it reads them from the five pointers named at that flag. */
int bimamba2_bwd(const bimamba2_params *p);

/* ---- single stages (each is also what the composites run) ------------------------------------------ */

/* dt -> dt_out, cs_f, cs_b.  Replaces _chunk_cumsum_fwd (src/ssd/bi/ssd_chunk_state.py:699-724). */
int bimamba2_chunk_cumsum_fwd(const bimamba2_params *p);
/* Cm, Bm -> CB (and CBT when that pointer is set).  Replaces _bmm_chunk_fwd (src/ssd/bi/ssd_bmm.py:163-208). */
int bimamba2_bmm_chunk_fwd(const bimamba2_params *p);
/* x, Bm, dt_out, cs_f, cs_b -> states_f, states_b (or states16_f/b, see there).  Replaces _chunk_state_fwd
 * (src/ssd/bi/ssd_chunk_state.py:764-798). */
int bimamba2_chunk_state_fwd(const bimamba2_params *p);
/* states_f/b (chunk states) -> states_f/b (state entering each chunk), in place, both directions in one
 * launch; optional final_f/final_b and initial_f/initial_b.  Replaces the two _state_passing_fwd calls
 * (src/ssd/bi/ssd_state_passing.py:190-207; src/ssd/bi/ssd_combined.py:324-327). */
int bimamba2_state_passing_fwd(const bimamba2_params *p);
/* CB, x, z, dt_out, cs_f, cs_b, Cm, Bm, states_f/b, D -> out, out_x.  Replaces _chunk_scan_fwd
 * (src/ssd/bi/ssd_chunk_scan.py:1638-1686).  With CB = NULL, allowed when bimamba2_chunk_scan_reads_cb(p, 0) is 0,
 * the kernel rebuilds the CB tiles from Cm and Bm; a CB that is given is read. */
int bimamba2_chunk_scan_fwd(const bimamba2_params *p);

/* z, out_x, dout -> dz, dout_x.  Replaces _chunk_scan_bwd_dz (src/ssd/bi/ssd_chunk_scan.py:1741-1798);
 * dD is produced by bimamba2_chunk_scan_bwd_dx. */
int bimamba2_chunk_scan_bwd_dz(const bimamba2_params *p);
/* dout (dout_x when has_z), Cm, cs_f, cs_b -> dstates_f/b.  Replaces _chunk_scan_bwd_dstates
 * (src/ssd/bi/ssd_chunk_scan.py:1801-1826). */
int bimamba2_chunk_scan_bwd_dstates(const bimamba2_params *p);
/* The two above as one launch: z, out_x, dout, Cm, cs_f, cs_b -> dz, dout_x, dstates_f/b, with the same results.  A
 * workgroup forms dout_x for its (batch, chunk, head) and multiplies it with C without reading it back.  Exists for
 * 16-bit types with a z gate, dstate 64, headdim % 64 == 0, chunk_size % 32 == 0 and 16-byte aligned operands with
 * strides that are multiples of 8 elements; BIMAMBA2_EUNSUPPORTED otherwise (bimamba2_bwd then runs the two).  Replaces
 * _chunk_scan_bwd_dz and _chunk_scan_bwd_dstates (src/ssd/bi/ssd_combined.py:381-392). */
int bimamba2_chunk_scan_bwd_dz_dstates(const bimamba2_params *p);
/* states_f/b, dstates_f/b (in place), cs [dfinal_f/b] -> dstates_f/b (gradient of each chunk state), ddA_chunk_f/b
 * [dinitial_f/b].  Replaces the two _state_passing_bwd calls (src/ssd/bi/ssd_state_passing.py:210-248). */
int bimamba2_state_passing_bwd(const bimamba2_params *p);
/* -> dx, ddt_direct, dD partials (reduced into dD).  Replaces _chunk_scan_chunk_state_bwd_dx
 * (src/ssd/bi/ssd_combined.py:235-294).  With CBT = NULL, allowed when bimamba2_chunk_scan_reads_cb(p, 1) is 0,
 * the kernel rebuilds the tiles from Cm and Bm; a CBT that is given is read. */
int bimamba2_chunk_scan_bwd_dx(const bimamba2_params *p);
/* x, dstates_f/b, dt_out, cs, Bm -> dBs, v_f, v_b.  Replaces _chunk_state_bwd_db
 * (src/ssd/bi/ssd_chunk_state.py:836-894); v_* are its ddA_next terms before the scan. */
int bimamba2_chunk_state_bwd_db(const bimamba2_params *p);
/* dout, states_f/b, cs, Cm -> dCs, u_f, u_b.  Replaces _chunk_scan_bwd_dC
 * (src/ssd/bi/ssd_chunk_scan.py:1829-1877); u_* are its ddA_cumsum_prev terms. */
int bimamba2_chunk_scan_bwd_dc(const bimamba2_params *p);
/* x, dout, dt_out, cs, CB -> dCB, dCBT, da_intra.  Replaces _chunk_scan_bwd_dcb (src/ssd/bi/ssd_chunk_scan.py:1880-1909)
 * and _chunk_scan_bwd_ddAcs_stable_fwd/_bwd (src/ssd/bi/ssd_chunk_scan.py:2036-2098) in one pass.  With CB = NULL,
 * allowed when bimamba2_chunk_scan_reads_cb(p, 2) is 0, the kernel rebuilds its CB tiles from Cm and Bm. */
int bimamba2_chunk_scan_bwd_dcb(const bimamba2_params *p);
/* dCB, dCBT, Cm, Bm, dBs, dCs -> dB, dC.  Replaces the two _bmm_chunk_bwd calls (src/ssd/bi/ssd_bmm.py:211-262). */
int bimamba2_bmm_chunk_bwd(const bimamba2_params *p);
/* da_intra, u, v, ddA_chunk, ddt_direct, dt, A, dt_bias -> ddt, dA, ddt_bias.  Replaces the host-side
 * scans (src/ssd/bi/ssd_combined.py:456-466) and _chunk_cumsum_bwd (src/ssd/bi/ssd_chunk_state.py:727-761). */
int bimamba2_chunk_cumsum_bwd(const bimamba2_params *p);

/* ---- gated RMSNorm (the step after the operator in the BiMamba2 layer) -------------------------------------
 *   xg = x (norm_before_gate) or x * silu(z);  y = xg * rstd * weight (+ bias), rstd = 1/sqrt(mean_group(xg^2) + eps);
 *   out = y * silu(z) (norm_before_gate) or y.
 * Rows of `cols` elements (last dim contiguous, row strides in elements), groups of `group_size` consecutive columns
 * (group_size divides cols, <= 32768: 64 KB of a 16-bit row, the reference kernel's limit; beyond 8192 columns a workgroup
 * instead of a wave works on a (row, group)).  Replaces rmsnorm_fn / RMSNorm of the reference, i.e. _layer_norm_fwd
 * (src/ssd/bi/layernorm_gated.py:108-152, kernel :45-105) and _layer_norm_bwd (:271-330, kernel :155-268) with
 * is_rms_norm = True; math of rms_norm_ref (:18-39). */
typedef struct bimamba2_norm_params {
    int64_t rows;
    int32_t cols, group_size;
    int32_t dtype;              /* BIMAMBA2_*: x, z, out, dout, dx, dz */
    int32_t has_z, has_bias, norm_before_gate;
    float eps;
    int32_t layer_norm;         /* 0: RMS norm (the BiMamba2 layer's);  1: LayerNorm - the group's mean is subtracted first
                                   (is_rms_norm = False of the reference, same kernels there) and kept in `mean` */
    int64_t x_rs, z_rs, out_rs, dout_rs, dx_rs, dz_rs;
    const void *x, *z;
    const float *weight, *bias; /* (cols,) float32 */
    void *out;                  /* forward */
    float *rstd;                /* (rows, cols / group_size) float32: written by the forward (optional there), read by the backward */
    const void *dout;           /* backward */
    void *dx, *dz;
    float *dweight, *dbias;     /* (cols,) float32 */
    void *workspace;            /* backward only: bimamba2_rmsnorm_gated_workspace_bytes() */
    size_t workspace_bytes;
    void *stream;               /* hipStream_t */
    float *mean;                /* layer_norm only: (rows, cols / group_size) float32, written by the forward (optional
                                   there), read by the backward */
} bimamba2_norm_params;

size_t bimamba2_norm_params_size(void);
size_t bimamba2_rmsnorm_gated_workspace_bytes(const bimamba2_norm_params *p);
/* x [z] weight [bias] -> out, rstd */
int bimamba2_rmsnorm_gated_fwd(const bimamba2_norm_params *p);
/* x [z] weight [bias] rstd dout -> dx [dz] dweight [dbias] */
int bimamba2_rmsnorm_gated_bwd(const bimamba2_norm_params *p);

/* ---------------------------------------------------------------------------------------------------------
 * Non-causal depthwise conv1d + SiLU on channels-last activations: the step in front of the operator in the
 * BiMamba2 layer.  Replaces  act(conv1d(xBC.transpose(1, 2)).transpose(1, 2))  of the reference
 * (src/ssd/modules.py:162-164; the convolution is constructed at :68-75 with groups = channels and
 * padding = d_conv // 2) without the two transposes:
 *   out[b, l, c] = silu(bias[c] + sum_k weight[c, k] * x[b, l + k - width / 2, c]),   zero padding.
 * width is odd, 1..9.  x and dout may be strided views (batch and position strides in elements, channels contiguous);
 * out and dx are written contiguous as (batch, seqlen, channels).  weight (channels, width), bias, dweight, dbias are
 * float32.  The backward pass recomputes the pre-activation from x, and needs
 * bimamba2_conv1d_silu_workspace_bytes() bytes of workspace for its fixed-order partial sums.
 * --------------------------------------------------------------------------------------------------------- */
typedef struct bimamba2_conv_params {
    int64_t batch, seqlen;
    int32_t channels, width;
    int32_t dtype;              /* BIMAMBA2_* : x, out, dout, dx */
    int32_t has_bias;
    int64_t x_sb, x_sl;         /* element strides of x: batch, position */
    int64_t dout_sb, dout_sl;   /* of dout (backward) */
    const void *x;
    const float *weight;        /* (channels, width) */
    const float *bias;          /* (channels) or NULL */
    void *out;                  /* forward: (batch, seqlen, channels) */
    const void *dout;           /* backward */
    void *dx;                   /* backward: (batch, seqlen, channels) */
    float *dweight;             /* backward: (channels, width) */
    float *dbias;               /* backward: (channels) when has_bias */
    void *workspace;
    size_t workspace_bytes;
    void *stream;               /* hipStream_t */
    int64_t dx_sb, dx_sl;       /* element strides of dx: batch, position; both 0 = contiguous (seqlen * channels, channels).
                                   Lets the gradient land in a slice of a wider buffer (the layer's projection gradient). */
} bimamba2_conv_params;

size_t bimamba2_conv_params_size(void);
size_t bimamba2_conv1d_silu_workspace_bytes(const bimamba2_conv_params *p);
/* x weight [bias] -> out */
int bimamba2_conv1d_silu_fwd(const bimamba2_conv_params *p);
/* x weight [bias] dout -> dx dweight [dbias] */
int bimamba2_conv1d_silu_bwd(const bimamba2_conv_params *p);

/* ---------------------------------------------------------------------------------------------------------
 * Several small element-wise conversions in ONE launch: the parameter maps in front of and behind the layer's kernels
 * (A = -exp(A_log), and dt_bias, D, the convolution's filter and bias and the norm's weight as float32 when the module
 * holds them in a 16-bit type; on the way back the float32 gradients into the parameters' types, dA_log = dA * A).  The
 * reference does them as separate torch ops (src/ssd/modules.py:156, the .float() calls in its kernels' wrappers);
 * captured in a graph each of those is a launch of a few microseconds.
 * ------------------------------------------------------------------------------------------------------- */
#define BIMAMBA2_CAST_MAX 8
enum { BIMAMBA2_CAST_COPY = 0,      /* dst = src */
       BIMAMBA2_CAST_NEG_EXP = 1,   /* dst = -exp(src) */
       BIMAMBA2_CAST_MUL = 2 };     /* dst = src * aux (aux: float32, same length) */
typedef struct bimamba2_cast_item {
    const void *src;
    void *dst;
    const float *aux;
    int64_t n;                  /* elements (contiguous) */
    int32_t src_dtype, dst_dtype, op, reserved;
} bimamba2_cast_item;
typedef struct bimamba2_cast_params {
    int32_t count, reserved;    /* items in use, at most BIMAMBA2_CAST_MAX */
    bimamba2_cast_item item[BIMAMBA2_CAST_MAX];
    void *stream;               /* hipStream_t */
} bimamba2_cast_params;
size_t bimamba2_cast_params_size(void);
int bimamba2_cast_many(const bimamba2_cast_params *p);

#ifdef __cplusplus
}
#endif
#endif /* BIMAMBA2_H */
