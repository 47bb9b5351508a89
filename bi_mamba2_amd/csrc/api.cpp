// C ABI of libbimamba2_hip.so: argument checks, workspace carving and the forward / backward pipelines.
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>

#include "../../include/bimamba2.h"
#include "launch.hpp"

using namespace bm2;

namespace {

inline int nchunks(const bimamba2_params *p) { return (p->seqlen + p->chunk_size - 1) / p->chunk_size; }
inline hipStream_t stream_of(const bimamba2_params *p) { return reinterpret_cast<hipStream_t>(p->stream); }
inline size_t elem_size(int dtype) { return dtype == BIMAMBA2_F32 ? 4 : 2; }
inline int sp_nsplit(const bimamba2_params *p) { return (p->headdim * p->dstate + 1023) / 1024; }

// the forward scan kernel that rebuilds C.B^T from the 16-bit copies' side: it exists beyond state dimension 64 (128) and
// runs where the entering states are given as copies
inline bool fwd_scan_rebuilds_cb(const bimamba2_params *p) {
    return chunk_scan_uses_scan16(p, false) && p->states16_f && (p->causal || p->states16_b);
}

int check_problem(const bimamba2_params *p) {
    if (!p) return BIMAMBA2_EINVAL;
    if (p->batch <= 0 || p->seqlen <= 0 || p->nheads <= 0 || p->headdim <= 0 || p->ngroups <= 0 || p->dstate <= 0)
        return BIMAMBA2_EINVAL;
    if (p->nheads % p->ngroups) return BIMAMBA2_EINVAL;
    if (p->dtype < BIMAMBA2_F32 || p->dtype > BIMAMBA2_F16) return BIMAMBA2_EUNSUPPORTED;
    if (p->dt_dtype < BIMAMBA2_F32 || p->dt_dtype > BIMAMBA2_F16) return BIMAMBA2_EUNSUPPORTED;
    if (p->chunk_size < BIMAMBA2_MIN_CHUNK || p->chunk_size > BIMAMBA2_MAX_CHUNK) return BIMAMBA2_EUNSUPPORTED;
    if (p->headdim > BIMAMBA2_MAX_HEADDIM || p->dstate > BIMAMBA2_MAX_DSTATE) return BIMAMBA2_EUNSUPPORTED;
    // grid.z = batch * nchunks * nheads must fit the launch limits
    const int64_t z = (int64_t)p->batch * nchunks(p) * p->nheads;
    if (z > 2147483647LL / 2) return BIMAMBA2_EUNSUPPORTED;
    return BIMAMBA2_OK;
}

#define REQUIRE(ptr)                        \
    do {                                    \
        if (!(ptr)) return BIMAMBA2_EINVAL; \
    } while (0)
#define TRY(expr)              \
    do {                       \
        int rc_ = (expr);      \
        if (rc_) return rc_;   \
    } while (0)

struct Carver {
    char *base;
    size_t off = 0;
    explicit Carver(void *b) : base(static_cast<char *>(b)) {}
    template <typename T> T *take(size_t n) {
        off = (off + 255) & ~size_t(255);
        T *r = base ? reinterpret_cast<T *>(base + off) : nullptr;
        off += n * sizeof(T);
        return r;
    }
};

// Assigns every intermediate that is NULL in `q` from the workspace; returns the bytes used.
size_t carve(bimamba2_params *q, int is_bwd, void *ws) {
    Carver cv(ws);
    const size_t nc = nchunks(q), Q = q->chunk_size;
    const size_t bhcq = (size_t)q->batch * q->nheads * nc * Q;
    const size_t cbn = (size_t)q->batch * nc * q->ngroups * Q * Q;
    const size_t stn = (size_t)q->batch * nc * q->nheads * q->headdim * q->dstate;
    auto need_f = [&](float *&ptr, size_t n) { if (!ptr) ptr = cv.take<float>(n); };
    need_f(q->dt_out, bhcq);
    need_f(q->cs_f, bhcq);
    need_f(q->cs_b, bhcq);
    // 16-bit copies of the entering states (see states16_f in the header): used where the kernels know them and the
    // caller does not ask for the float32 entering states; a backward pass that got the copies from the forward pass
    // needs no float32 states at all
    const bool copies = bimamba2_state_copies(q) != 0;
    const bool saved_copies = is_bwd && q->fwd_saved && q->states16_f;
    // a forward pass whose caller keeps no states (no pointer given for them) has one reader of the entering states, the scan
    // kernel, and every 16-bit scan kernel reads the copies: the state passing then writes half the bytes, the scan reads half
    // (under the conditions of the state-passing kernel that writes them)
    auto al16 = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    const bool fwd_only_copies = !is_bwd && !q->causal && (q->dtype == BIMAMBA2_BF16 || q->dtype == BIMAMBA2_F16) &&
                                 (q->headdim * q->dstate) % 4 == 0 && al16(q->final_f) && al16(q->final_b) &&
                                 al16(q->initial_f) && al16(q->initial_b) && !q->states_b && !q->states16_b;
    const bool carve16 = (copies || fwd_only_copies) && !q->states_f && !q->states16_f;
    // CB: read by the forward scan and by the dCB kernel unless they rebuild it; CB^T: by the dx kernel, likewise.  (The
    // forward scan kernel for state dimension 128 rebuilds it as well, and runs where the entering states travel as copies.)
    const bool fwd_scan16 = !is_bwd && chunk_scan_uses_scan16(q, false) && (carve16 || q->states16_f) && (q->causal || carve16 || q->states16_b);
    if (is_bwd ? !(scan_recomputes_cb(q, true) && dcb_recomputes_cb(q)) : !(scan_recomputes_cb(q, false) || fwd_scan16)) need_f(q->CB, cbn);
    if (carve16) {
        q->states16_f = cv.take<char>(stn * 2);
        q->states16_b = cv.take<char>(stn * 2);
    }
    // a forward pass whose caller asks for no float32 states at all keeps the per-chunk states in the 16-bit copies' place
    // too (the chunk-state kernel writes them there, the inter-chunk scan replaces them by the entering states)
    const bool states16_only = !is_bwd && !q->states_f && !q->states_b && (carve16 || (q->states16_f && q->states16_b)) &&
                               chunk_states_in_16bit(q);
    if (!saved_copies && !states16_only) {
        need_f(q->states_f, stn);
        need_f(q->states_b, stn);
    }
    if (is_bwd && copies && !q->dstates_f && !q->dstates16_f) {
        q->dstates16_f = cv.take<char>(stn * 2);
        q->dstates16_b = cv.take<char>(stn * 2);
    }
    if (is_bwd) {
        const size_t nqt = (Q + 63) / 64;
        need_f(q->dCB, cbn * dcb_slices(q));
        need_f(q->dCBT, cbn * dcb_slices(q));
        if (!scan_recomputes_cb(q, true)) need_f(q->CBT, cbn);
        // where the 16-bit copies of the gradients exist and the caller asks for no float32 tensors, the per-chunk gradients
        // live in the copies' place as well (written there by the dstates kernels, replaced in place by the backward
        // inter-chunk scan): no float32 tensors at all
        // (the in-place kernel of the backward inter-chunk scan reads the entering states from their copies as well)
        const bool dstates16_only = copies && !q->dstates_f && !q->dstates_b && (carve16 || q->states16_f);
        if (!dstates16_only) {
            need_f(q->dstates_f, stn);
            need_f(q->dstates_b, stn);
        }
        if (q->has_z && !q->dout_x)
            q->dout_x = cv.take<char>((size_t)q->batch * q->seqlen * q->nheads * q->headdim * elem_size(q->dtype));
        need_f(q->ddt_direct, bhcq * ddt_direct_planes(*q));
        need_f(q->u_f, bhcq);
        need_f(q->u_b, bhcq);
        need_f(q->v_f, bhcq);
        need_f(q->v_b, bhcq);
        need_f(q->da_intra, (size_t)q->batch * q->nheads * nc * nqt * nqt * 128);
        need_f(q->ddA_chunk_f, (size_t)q->batch * q->nheads * nc * sp_nsplit(q));
        need_f(q->ddA_chunk_b, (size_t)q->batch * q->nheads * nc * sp_nsplit(q));
        const size_t slices = (q->nheads / q->ngroups + 7) / 8;   // head slices of the dB / dC partial sums
        const size_t bn = slices * q->batch * q->seqlen * q->ngroups * q->dstate;
        need_f(q->dBs, bn);
        need_f(q->dCs, bn);
        // partial sums of dD, then those of dA and ddt_bias (the composite reduces all three in one launch at the end)
        need_f(q->red, (size_t)q->batch * nc * q->nheads * q->headdim + (size_t)2 * q->batch * nc * q->nheads);
    }
    return (cv.off + 255) & ~size_t(255);
}

// Device memory that lives as long as the process: the workspace of bimamba2_fwd_static.  Every GPU the library runs on
// holds its own copy at its own address; in host code the array's name is not a device address, so the address is asked
// for once per device (hipGetSymbolAddress, with that device current) and kept.
static __device__ __align__(256) unsigned char scratch[BIMAMBA2_STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::atomic<void *> scratch_of_device[MAX_DEVICES];

int static_scratch(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return BIMAMBA2_ELAUNCH;
    void *ptr = scratch_of_device[dev].load(std::memory_order_acquire);
    if (!ptr) {
        // two host threads may both get here: they are given the same address
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return BIMAMBA2_ELAUNCH;
        scratch_of_device[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return BIMAMBA2_OK;
}

}  // namespace

extern "C" {

const char *bimamba2_strerror(int code) {
    switch (code) {
        case BIMAMBA2_OK: return "ok";
        case BIMAMBA2_EINVAL: return "invalid argument (null pointer or inconsistent dimensions)";
        case BIMAMBA2_EUNSUPPORTED:
            return "unsupported problem (need 32 <= chunk_size <= 256, headdim <= 128, dstate <= 256, dtype f32/bf16/f16)";
        case BIMAMBA2_EWORKSPACE: return "workspace missing or too small";
        case BIMAMBA2_ELAUNCH: return "HIP kernel launch failed";
        case BIMAMBA2_ESCRATCH: return "the problem needs more intermediate memory than the static scratch buffer holds";
        default: return "unknown error";
    }
}

int bimamba2_version(void) { return 100; }
size_t bimamba2_params_size(void) { return sizeof(bimamba2_params); }

size_t bimamba2_workspace_bytes(const bimamba2_params *p, int is_bwd) {
    if (check_problem(p)) return 0;
    bimamba2_params q = *p;
    return carve(&q, is_bwd, nullptr);
}

int bimamba2_state_copies(const bimamba2_params *p) {
    if (check_problem(p)) return 0;
    if (p->dtype != BIMAMBA2_BF16 && p->dtype != BIMAMBA2_F16) return 0;
    if (p->dstate != 64 || p->headdim % 64 || p->chunk_size % 64) return 0;
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    // the vector kernels of the two state-passing stages, the scan kernels that rebuild CB, the dB / dC kernels with the
    // ring of state tiles: every one of them must be the one that runs
    if (!(al(p->states_f) && al(p->states_b) && al(p->dstates_f) && al(p->dstates_b) && al(p->final_f) && al(p->final_b) &&
          al(p->initial_f) && al(p->initial_b) && al(p->dfinal_f) && al(p->dfinal_b) && al(p->dinitial_f) && al(p->dinitial_b)))
        return 0;
    if (!al(p->states16_f) || !al(p->states16_b) || !al(p->dstates16_f) || !al(p->dstates16_b)) return 0;
    return scan_recomputes_cb(p, false) && scan_recomputes_cb(p, true) && dcb_recomputes_cb(p) ? 1 : 0;
}

int bimamba2_chunk_scan_reads_cb(const bimamba2_params *p, int which) {
    if (check_problem(p)) return 1;
    if (which == 2) return dcb_recomputes_cb(p) ? 0 : 1;
    if (which == 3) return chunk_state_does_cumsum(p) ? 0 : 1;
    if (which == 0 && fwd_scan_rebuilds_cb(p)) return 0;
    return scan_recomputes_cb(p, which != 0) ? 0 : 1;
}

int bimamba2_chunk_scan_heads_per_workgroup(const bimamba2_params *p, int bwd) {
    if (check_problem(p)) return 1;
    return chunk_scan_uses_scan16(p, bwd != 0) ? chunk_scan16_heads_per_workgroup(p) : 1;
}

int bimamba2_ddt_direct_planes(const bimamba2_params *p) {
    if (check_problem(p)) return 1;
    return ddt_direct_planes(*p);
}

int bimamba2_chunk_cumsum_fwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->dt); REQUIRE(p->A); REQUIRE(p->dt_out); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (p->has_dt_bias) REQUIRE(p->dt_bias);
    return launch_chunk_cumsum_fwd(p);
}

int bimamba2_bmm_chunk_fwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->Bm); REQUIRE(p->Cm); REQUIRE(p->CB);
    return launch_bmm_chunk_fwd(p);
}

int bimamba2_chunk_state_fwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->x); REQUIRE(p->Bm); REQUIRE(p->dt_out); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (p->states_f || !p->states16_f) { REQUIRE(p->states_f); REQUIRE(p->states_b); }   // (else: 16-bit per-chunk states in states16_*)
    return launch_chunk_state(p, false);
}

int bimamba2_state_passing_fwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (p->states_f || !p->states16_f) { REQUIRE(p->states_f); REQUIRE(p->states_b); }
    return launch_state_passing_fwd(p);
}

int bimamba2_chunk_scan_fwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->x); REQUIRE(p->Cm); REQUIRE(p->dt_out); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (!p->CB && !(p->Bm && (scan_recomputes_cb(p, false) || fwd_scan_rebuilds_cb(p)))) return BIMAMBA2_EINVAL;   // without CB the kernel rebuilds it from Cm, Bm
    if (!p->states16_f) { REQUIRE(p->states_f); REQUIRE(p->states_b); }
    REQUIRE(p->out);
    if (p->has_D) REQUIRE(p->D);
    if (p->has_z) REQUIRE(p->z);
    return launch_chunk_scan(p, false);
}

int bimamba2_chunk_scan_bwd_dz(const bimamba2_params *p) {
    TRY(check_problem(p));
    if (!p->has_z) return BIMAMBA2_EINVAL;
    REQUIRE(p->z); REQUIRE(p->dout); REQUIRE(p->out_x); REQUIRE(p->dz); REQUIRE(p->dout_x);
    return launch_bwd_dz(p);
}

int bimamba2_chunk_scan_bwd_dstates(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->Cm); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (p->dstates_f || !p->dstates16_f) { REQUIRE(p->dstates_f); REQUIRE(p->dstates_b); }   // (else: 16-bit per-chunk gradients in dstates16_*)
    if (p->has_z) REQUIRE(p->dout_x); else REQUIRE(p->dout);
    return launch_chunk_state(p, true);
}

int bimamba2_chunk_scan_bwd_dz_dstates(const bimamba2_params *p) {
    TRY(check_problem(p));
    if (!p->has_z) return BIMAMBA2_EINVAL;
    REQUIRE(p->z); REQUIRE(p->dout); REQUIRE(p->out_x); REQUIRE(p->dz); REQUIRE(p->dout_x);
    REQUIRE(p->Cm); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (p->dstates_f || !p->dstates16_f) { REQUIRE(p->dstates_f); REQUIRE(p->dstates_b); }
    return launch_bwd_dz_dstates(p);       // BIMAMBA2_EUNSUPPORTED where only the two separate kernels exist
}

int bimamba2_state_passing_bwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (!p->states16_f) { REQUIRE(p->states_f); REQUIRE(p->states_b); }
    if (p->dstates_f || !p->dstates16_f) { REQUIRE(p->dstates_f); REQUIRE(p->dstates_b); }
    REQUIRE(p->ddA_chunk_f); REQUIRE(p->ddA_chunk_b);
    return launch_state_passing_bwd(p);
}

int bimamba2_chunk_scan_bwd_dx(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->x); REQUIRE(p->Bm); REQUIRE(p->dt_out); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (!p->CBT && !(p->Cm && scan_recomputes_cb(p, true))) return BIMAMBA2_EINVAL;   // without CBT the kernel rebuilds it from Cm, Bm
    if (!p->dstates16_f) { REQUIRE(p->dstates_f); REQUIRE(p->dstates_b); }
    REQUIRE(p->dx); REQUIRE(p->ddt_direct);
    if (p->has_z) REQUIRE(p->dout_x); else REQUIRE(p->dout);
    if (p->has_D) { REQUIRE(p->D); REQUIRE(p->dD); REQUIRE(p->red); }
    const int nc = nchunks(p);
    TRY(launch_chunk_scan(p, true));
    if (p->has_D) {
        if (p->D_has_hdim) return launch_reduce(p->red, p->dD, p->batch * nc, p->nheads * p->headdim, 1, stream_of(p));
        return launch_reduce(p->red, p->dD, p->batch * nc, p->nheads, p->headdim, stream_of(p));
    }
    return BIMAMBA2_OK;
}

int bimamba2_chunk_state_bwd_db(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->x); REQUIRE(p->Bm); REQUIRE(p->dt_out); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (!p->dstates16_f) { REQUIRE(p->dstates_f); REQUIRE(p->dstates_b); }
    REQUIRE(p->dBs); REQUIRE(p->v_f); REQUIRE(p->v_b);
    return launch_bwd_dbdc(p, true);
}

int bimamba2_chunk_scan_bwd_dc(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->Cm); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (!p->states16_f) { REQUIRE(p->states_f); REQUIRE(p->states_b); }
    REQUIRE(p->dCs); REQUIRE(p->u_f); REQUIRE(p->u_b);
    if (p->has_z) REQUIRE(p->dout_x); else REQUIRE(p->dout);
    return launch_bwd_dbdc(p, false);
}

int bimamba2_chunk_scan_bwd_dcb(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->x); REQUIRE(p->dt_out); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
    if (!p->CB && !(p->Cm && p->Bm && dcb_recomputes_cb(p))) return BIMAMBA2_EINVAL;   // without CB the kernel rebuilds it from Cm, Bm
    REQUIRE(p->dCB); REQUIRE(p->dCBT); REQUIRE(p->da_intra);
    if (p->has_z) REQUIRE(p->dout_x); else REQUIRE(p->dout);
    return launch_bwd_dcb(p);
}

int bimamba2_bmm_chunk_bwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->Bm); REQUIRE(p->Cm); REQUIRE(p->dCB); REQUIRE(p->dCBT); REQUIRE(p->dBs); REQUIRE(p->dCs); REQUIRE(p->dB); REQUIRE(p->dC);
    return launch_bmm_chunk_bwd(p);
}

int bimamba2_chunk_cumsum_bwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    REQUIRE(p->dt); REQUIRE(p->A); REQUIRE(p->da_intra); REQUIRE(p->u_f); REQUIRE(p->u_b); REQUIRE(p->v_f); REQUIRE(p->v_b);
    REQUIRE(p->ddA_chunk_f); REQUIRE(p->ddA_chunk_b); REQUIRE(p->ddt_direct); REQUIRE(p->ddt); REQUIRE(p->dA); REQUIRE(p->red);
    if (p->has_dt_bias) REQUIRE(p->dt_bias);
    return launch_chunk_cumsum_bwd(p);
}

// chunk cumsum + chunk states: one launch where the chunk-state kernel does both, else the two stages
static int forward_cumsum_and_states(const bimamba2_params *q) {
    if (chunk_state_does_cumsum(q)) {
        REQUIRE(q->dt); REQUIRE(q->A); REQUIRE(q->x); REQUIRE(q->Bm);
        if (q->has_dt_bias) REQUIRE(q->dt_bias);
        return launch_chunk_state(q, false, true);
    }
    TRY(bimamba2_chunk_cumsum_fwd(q));
    return bimamba2_chunk_state_fwd(q);
}

int bimamba2_fwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    if (p->causal && p->final_b) return BIMAMBA2_EINVAL;
    bimamba2_params q = *p;
    const size_t need = carve(&q, 0, p->workspace);
    if (need > 256 && (!p->workspace || p->workspace_bytes < need)) return BIMAMBA2_EWORKSPACE;
    TRY(forward_cumsum_and_states(&q));
    if (q.CB) TRY(bimamba2_bmm_chunk_fwd(&q));     // given by the caller, or carved because the scan kernel reads it
    TRY(bimamba2_state_passing_fwd(&q));
    if (scan_recomputes_cb(&q, false) || fwd_scan_rebuilds_cb(&q)) q.CB = nullptr;
    TRY(bimamba2_chunk_scan_fwd(&q));
    return BIMAMBA2_OK;
}

int bimamba2_fwd_static(const bimamba2_params *p) {
    TRY(check_problem(p));
    bimamba2_params q = *p;
    q.workspace = nullptr;
    q.workspace_bytes = 0;
    {
        bimamba2_params sized = q;
        if (carve(&sized, 0, nullptr) > BIMAMBA2_STATIC_SCRATCH_BYTES) return BIMAMBA2_ESCRATCH;
    }
    // nothing in the forward pipeline accumulates into its intermediates: every one is written in full before it is
    // read, so what the last call left in the buffer does not matter
    TRY(static_scratch(&q.workspace));
    q.workspace_bytes = BIMAMBA2_STATIC_SCRATCH_BYTES;
    return bimamba2_fwd(&q);
}

int bimamba2_bwd(const bimamba2_params *p) {
    TRY(check_problem(p));
    bimamba2_params q = *p;
    q.final_f = q.final_b = nullptr;
    const size_t need = carve(&q, 1, p->workspace);
    if (need > 256 && (!p->workspace || p->workspace_bytes < need)) return BIMAMBA2_EWORKSPACE;
    if (p->fwd_saved) {
        REQUIRE(p->dt_out); REQUIRE(p->cs_f); REQUIRE(p->cs_b);
        if (!p->states16_f) { REQUIRE(p->states_f); REQUIRE(p->states_b); }
    } else {
        // recompute the forward intermediates (the reference does the same, src/ssd/bi/ssd_combined.py:373-380)
        TRY(forward_cumsum_and_states(&q));
        TRY(bimamba2_state_passing_fwd(&q));
    }
    // dCB / dCBT in the 16-bit element type where this call owns them and the two launches that write and read them are the
    // merged ones (their reader rounds them to that type for its MFMA anyway)
    const bool dcb16 = !p->dCB && !p->dCBT && bwd_dcb_sp_merged(&q) && bwd_tail_merged(&q);
    const bool need_cbt = !scan_recomputes_cb(&q, true), need_cb = need_cbt || !dcb_recomputes_cb(&q);
    if (need_cb) TRY(bimamba2_bmm_chunk_fwd(&q));  // CB for the dCB kernel, CB^T for the dx kernel, unless they rebuild it
    else q.CB = nullptr;
    // dz and dstates as one launch where the kernel for it exists (dout_x goes from the first to the second inside the workgroup)
    const bool dz_dstates = q.has_z && bwd_dz_dstates_fused(&q);
    if (dz_dstates) TRY(bimamba2_chunk_scan_bwd_dz_dstates(&q));
    else if (q.has_z) TRY(bimamba2_chunk_scan_bwd_dz(&q));
    // the dCB kernel is bound by instruction issue and moves little data: right behind dz it runs while the memory system
    // still writes back dz's output, which the memory-bound kernels after it would otherwise wait behind
    if (bwd_dcb_sp_merged(&q)) {
        // the backward state passing (streams, few instructions) rides along with the dCB kernel in one launch
        TRY(bimamba2_chunk_scan_bwd_dc(&q));
        if (!dz_dstates) TRY(bimamba2_chunk_scan_bwd_dstates(&q));
        REQUIRE(q.x); REQUIRE(q.dt_out); REQUIRE(q.cs_f); REQUIRE(q.cs_b); REQUIRE(q.dCB); REQUIRE(q.dCBT); REQUIRE(q.da_intra);
        if (!q.dstates16_f) REQUIRE(q.dstates_f);
        REQUIRE(q.ddA_chunk_f); REQUIRE(q.ddA_chunk_b);
        if (q.has_z) REQUIRE(q.dout_x); else REQUIRE(q.dout);
        TRY(launch_bwd_dcb_sp(&q, dcb16));
    } else {
        TRY(bimamba2_chunk_scan_bwd_dcb(&q));
        if (!dz_dstates) TRY(bimamba2_chunk_scan_bwd_dstates(&q));
        TRY(bimamba2_chunk_scan_bwd_dc(&q));           // (between the two memory-bound state kernels: measured best)
        TRY(bimamba2_state_passing_bwd(&q));
    }
    TRY(bimamba2_chunk_state_bwd_db(&q));
    ReduceJobs jobs;
    {
        // as bimamba2_chunk_scan_bwd_dx, with the reduction of the dD partial sums left for the end
        bimamba2_params qx = q;
        if (scan_recomputes_cb(&q, true)) qx.CBT = nullptr;
        REQUIRE(qx.dx); REQUIRE(qx.ddt_direct);
        if (qx.has_D) { REQUIRE(qx.D); REQUIRE(qx.dD); }
        const int nc = nchunks(&q);
        TRY(launch_chunk_scan(&qx, true));
        if (q.has_D) {
            if (q.D_has_hdim) jobs.job[jobs.n++] = ReduceJob{q.red, q.dD, q.batch * nc, q.nheads * q.headdim, 1};
            else jobs.job[jobs.n++] = ReduceJob{q.red, q.dD, q.batch * nc, q.nheads, q.headdim};
        }
    }
    {
        // as bimamba2_bmm_chunk_bwd and bimamba2_chunk_cumsum_bwd (its partial sums behind those of dD): one launch for
        // both where the kernel for it exists
        bimamba2_params qc = q;
        qc.red = q.red + (size_t)q.batch * nchunks(&q) * q.nheads * q.headdim;
        REQUIRE(q.ddt); REQUIRE(q.dA); REQUIRE(q.dB); REQUIRE(q.dC);
        if (bwd_tail_merged(&q)) {
            TRY(launch_bwd_tail(&qc, &jobs, dcb16));
        } else {
            TRY(bimamba2_bmm_chunk_bwd(&q));
            TRY(launch_chunk_cumsum_bwd(&qc, &jobs));
        }
    }
    TRY(launch_reduce_jobs(jobs, stream_of(&q)));
    return BIMAMBA2_OK;
}

size_t bimamba2_norm_params_size(void) { return sizeof(bimamba2_norm_params); }

static int check_norm(const bimamba2_norm_params *p) {
    if (!p) return BIMAMBA2_EINVAL;
    if (p->rows < 0 || p->cols <= 0 || p->group_size <= 0 || p->cols % p->group_size) return BIMAMBA2_EINVAL;
    if (p->dtype != BIMAMBA2_F32 && p->dtype != BIMAMBA2_BF16 && p->dtype != BIMAMBA2_F16) return BIMAMBA2_EUNSUPPORTED;
    if (p->group_size > 32768) return BIMAMBA2_EUNSUPPORTED;
    if (!p->x || !p->weight || (p->has_z && !p->z) || (p->has_bias && !p->bias)) return BIMAMBA2_EINVAL;
    return BIMAMBA2_OK;
}

size_t bimamba2_rmsnorm_gated_workspace_bytes(const bimamba2_norm_params *p) {
    if (check_norm(p)) return 0;
    return norm_workspace_bytes(p);
}

int bimamba2_rmsnorm_gated_fwd(const bimamba2_norm_params *p) {
    TRY(check_norm(p));
    REQUIRE(p->out);
    if (p->rows == 0) return BIMAMBA2_OK;
    return launch_rmsnorm_gated(p, false);
}

int bimamba2_rmsnorm_gated_bwd(const bimamba2_norm_params *p) {
    TRY(check_norm(p));
    REQUIRE(p->dout); REQUIRE(p->rstd); REQUIRE(p->dx); REQUIRE(p->dweight);
    if (p->layer_norm) REQUIRE(p->mean);
    if (p->has_z) REQUIRE(p->dz);
    if (p->has_bias) REQUIRE(p->dbias);
    if (!p->workspace || p->workspace_bytes < norm_workspace_bytes(p)) return BIMAMBA2_EWORKSPACE;
    return launch_rmsnorm_gated(p, true);
}

size_t bimamba2_conv_params_size(void) { return sizeof(bimamba2_conv_params); }

size_t bimamba2_cast_params_size(void) { return sizeof(bimamba2_cast_params); }

int bimamba2_cast_many(const bimamba2_cast_params *p) {
    if (!p || p->count < 0 || p->count > BIMAMBA2_CAST_MAX) return BIMAMBA2_EINVAL;
    auto known = [](int d) { return d == BIMAMBA2_F32 || d == BIMAMBA2_BF16 || d == BIMAMBA2_F16; };
    for (int k = 0; k < p->count; ++k) {
        const bimamba2_cast_item &it = p->item[k];
        if (it.n < 0 || (it.n > 0 && (!it.src || !it.dst))) return BIMAMBA2_EINVAL;
        if (!known(it.src_dtype) || !known(it.dst_dtype)) return BIMAMBA2_EUNSUPPORTED;
        if (it.op < BIMAMBA2_CAST_COPY || it.op > BIMAMBA2_CAST_MUL) return BIMAMBA2_EINVAL;
        if (it.op == BIMAMBA2_CAST_MUL && it.n > 0 && !it.aux) return BIMAMBA2_EINVAL;
    }
    return launch_cast_many(p);
}

static int check_conv(const bimamba2_conv_params *p) {
    if (!p) return BIMAMBA2_EINVAL;
    if (p->batch < 0 || p->seqlen < 0 || p->channels <= 0) return BIMAMBA2_EINVAL;
    if (p->dtype != BIMAMBA2_F32 && p->dtype != BIMAMBA2_BF16 && p->dtype != BIMAMBA2_F16) return BIMAMBA2_EUNSUPPORTED;
    if (p->width < 1 || p->width > 9 || p->width % 2 == 0) return BIMAMBA2_EUNSUPPORTED;
    if (p->seqlen > (1 << 30)) return BIMAMBA2_EUNSUPPORTED;
    if (!p->x || !p->weight || (p->has_bias && !p->bias)) return BIMAMBA2_EINVAL;
    return BIMAMBA2_OK;
}

size_t bimamba2_conv1d_silu_workspace_bytes(const bimamba2_conv_params *p) {
    if (check_conv(p)) return 0;
    return conv_workspace_bytes(p);
}

int bimamba2_conv1d_silu_fwd(const bimamba2_conv_params *p) {
    TRY(check_conv(p));
    REQUIRE(p->out);
    if (p->batch == 0 || p->seqlen == 0) return BIMAMBA2_OK;
    return launch_conv1d_silu(p, false);
}

int bimamba2_conv1d_silu_bwd(const bimamba2_conv_params *p) {
    TRY(check_conv(p));
    REQUIRE(p->dout); REQUIRE(p->dx); REQUIRE(p->dweight);
    if (p->has_bias) REQUIRE(p->dbias);
    if (!p->workspace || p->workspace_bytes < conv_workspace_bytes(p)) return BIMAMBA2_EWORKSPACE;
    if (p->batch == 0 || p->seqlen == 0) {
        TRY(launch_fill(p->dweight, (size_t)p->channels * p->width, 0.f, reinterpret_cast<hipStream_t>(p->stream)));
        if (p->has_bias) TRY(launch_fill(p->dbias, (size_t)p->channels, 0.f, reinterpret_cast<hipStream_t>(p->stream)));
        return BIMAMBA2_OK;
    }
    return launch_conv1d_silu(p, true);
}

}  // extern "C"
