// Forward kernels of the bidirectional SSD operator for gfx950.
//   chunk_cumsum_fwd   dt -> dt', forward and reverse within-chunk cumulative sums of dt'*A
//   bmm_chunk_fwd      CB = C . B^T per chunk and group
//   chunk_state        per chunk and head: x^T . (B * decay * dt) for both directions (also used, with other
//                      operands and weights, for the gradient of the chunk-entry states)
//   state_passing_fwd  forward and reverse inter-chunk recurrences in one launch, in place
// (the chunk-scan kernel itself lives in kernels_scan.hip)
#include "common.hpp"
#include "launch.hpp"

namespace bm2 {

// =========================================================================================================
// chunk cumsum: one wave per (b, c, h); lane i owns positions 4i..4i+3 of the chunk (Q <= 256)
// =========================================================================================================
template <typename DT>
__global__ __launch_bounds__(NTHREADS) void chunk_cumsum_fwd_kernel(const bimamba2_params p, int nc) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = blockIdx.x * 4 + wave, c = blockIdx.y, b = blockIdx.z;
    if (h >= p.nheads) return;
    const int Q = p.chunk_size;
    const int limit = min(Q, p.seqlen - c * Q);
    const DT *dt = reinterpret_cast<const DT *>(p.dt) + b * p.dt_sb + (int64_t)c * Q * p.dt_sl + h * p.dt_sh;
    const float A = p.A[h];
    const float bias = p.has_dt_bias ? p.dt_bias[h] : 0.f;
    float v[4], a[4], ar[4];                          // ar: exponents of the reverse direction (differ with seq_idx only)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int q = lane * 4 + e;
        float d = 0.f;
        if (q < limit) {
            d = to_f(dt[(int64_t)q * p.dt_sl]) + bias;
            if (p.dt_softplus) d = d > 20.f ? d : log1pf(expf(d));
            d = fminf(fmaxf(d, p.dt_min), p.dt_max);
        }
        v[e] = d;
        a[e] = ar[e] = d * A;
        if (p.seq_idx && q < limit) {
            // packed sequences: cut the forward recurrence in front of a sequence's first position, the reverse one
            // behind its last
            const int l = c * Q + q;
            const int32_t *si = p.seq_idx + (int64_t)b * p.seqlen + l;
            const int32_t cur = si[0];
            if (l > 0 && si[-1] != cur) a[e] += BIMAMBA2_SEQ_CUT;
            if (l + 1 < p.seqlen && si[1] != cur) ar[e] += BIMAMBA2_SEQ_CUT;
        }
    }
    // forward inclusive scan, reverse inclusive scan
    float pf[4], sb[4];
    pf[0] = a[0]; pf[1] = pf[0] + a[1]; pf[2] = pf[1] + a[2]; pf[3] = pf[2] + a[3];
    sb[3] = ar[3]; sb[2] = sb[3] + ar[2]; sb[1] = sb[2] + ar[1]; sb[0] = sb[1] + ar[0];
    const float tot = pf[3], tot_r = sb[0];
    const float incl = wave_incl_prefix(tot, lane);
    const float before = incl - tot;
    const float incl_s = wave_incl_suffix(tot_r, lane);
    const float after = incl_s - tot_r;
    const int64_t o = (((int64_t)b * p.nheads + h) * nc + c) * Q;
    if (Q % 4 == 0) {
        // a lane's four positions are contiguous: 16-byte stores (the three tensors are contiguous and Q * 4 bytes per row)
        if (lane * 4 < Q) {
            *reinterpret_cast<f32x4 *>(p.dt_out + o + lane * 4) = f32x4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f32x4 *>(p.cs_f + o + lane * 4) = f32x4{before + pf[0], before + pf[1], before + pf[2], before + pf[3]};
            *reinterpret_cast<f32x4 *>(p.cs_b + o + lane * 4) = f32x4{after + sb[0], after + sb[1], after + sb[2], after + sb[3]};
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int q = lane * 4 + e;
        if (q < Q) {
            p.dt_out[o + q] = v[e];
            p.cs_f[o + q] = before + pf[e];
            p.cs_b[o + q] = after + sb[e];
        }
    }
}

// =========================================================================================================
// CB[t, s] = sum_n C[t, n] B[s, n]
// =========================================================================================================
template <typename T>
__global__ __launch_bounds__(NTHREADS) void bmm_chunk_fwd_kernel(const bimamba2_params p, int nc) {
    constexpr int LD = Mma<T>::LD;
    __shared__ __attribute__((aligned(16))) T As[64 * LD];
    __shared__ __attribute__((aligned(16))) T Bs[64 * LD];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int st = blockIdx.x, tt = blockIdx.y;
    const int g = blockIdx.z % p.ngroups, bc = blockIdx.z / p.ngroups, c = bc % nc, b = bc / nc;
    const int Q = p.chunk_size, N = p.dstate;
    const int limit = min(Q, p.seqlen - c * Q);
    const T *Cp = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + ((int64_t)c * Q + tt * 64) * p.C_sl + g * p.C_sg;
    const T *Bp = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + ((int64_t)c * Q + st * 64) * p.B_sl + g * p.B_sg;
    f32x4 acc[4] = {};
    for (int k0 = 0; k0 < N; k0 += BK) {
        __syncthreads();
        tile_load_kcontig<T, T, 64>(As, Cp + k0, p.C_sl, limit - tt * 64, N - k0, Ident());
        tile_load_kcontig<T, T, 64>(Bs, Bp + k0, p.B_sl, limit - st * 64, N - k0, Ident());
        __syncthreads();
        mma_tile<T, 4>(acc, As + wave * 16 * LD, Bs, lane);
    }
    float *out = p.CB + (int64_t)blockIdx.z * Q * Q;
    float *outT = p.CBT ? p.CBT + (int64_t)blockIdx.z * Q * Q : nullptr;   // CBT[s, t] = CB[t, s], read by the dx kernel
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = tt * 64 + wave * 16 + (lane >> 4) * 4 + i, s = st * 64 + j * 16 + (lane & 15);
            if (t < Q && s < Q) {
                out[(int64_t)t * Q + s] = acc[j][i];
                if (outT) outT[(int64_t)s * Q + t] = acc[j][i];
            }
        }
}

// =========================================================================================================
// chunk state (DSTATES = false):  S_f[p,n] = sum_k x[k,p] B[k,n] e^{cs_f[Q-1]-cs_f[k]} dt[k],  S_b with
//                                 e^{cs_b[0]-cs_b[k]}
// gradient of the chunk-entry states (DSTATES = true):  dprev_f[p,n] = sum_k dy[k,p] C[k,n] e^{cs_f[k]},
//                                 dprev_b with e^{cs_b[k]}
// =========================================================================================================
// Both operands have K = chunk position as their slow dimension, so both are staged transposed (8x8 in-register
// transposes) into LDS, KH positions at a time; the decay weights are applied to the B-side image while staging.
template <typename T, bool DSTATES, bool FAST>
__global__ __launch_bounds__(NTHREADS) void chunk_state_kernel(const bimamba2_params p, int nc) {
    typedef Mma<T> M;
    constexpr int KPL = M::KPL, KSTEP = M::KSTEP;
    constexpr int KH = sizeof(T) == 2 ? 128 : 64;          // chunk positions staged per round
    constexpr int LDX = KH + 16 / (int)sizeof(T);
    __shared__ __attribute__((aligned(16))) T xT[64 * LDX];
    __shared__ __attribute__((aligned(16))) T Bf[64 * LDX];
    __shared__ __attribute__((aligned(16))) T Bb[64 * LDX];
    __shared__ float wf[BIMAMBA2_MAX_CHUNK], wb[BIMAMBA2_MAX_CHUNK];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int nt = blockIdx.x, pt = blockIdx.y;
    const int h = blockIdx.z % p.nheads, bc = blockIdx.z / p.nheads, c = bc % nc, b = bc / nc;
    const int g = h / (p.nheads / p.ngroups);
    const int Q = p.chunk_size, N = p.dstate, P = p.headdim;
    const int limit = min(Q, p.seqlen - c * Q);
    const int64_t o = (((int64_t)b * p.nheads + h) * nc + c) * Q;
    for (int q = threadIdx.x; q < Q; q += NTHREADS) {
        float f = 0.f, r = 0.f;
        if (q < limit) {
            if (DSTATES) {
                f = __expf(p.cs_f[o + q]);
                r = __expf(p.cs_b[o + q]);
            } else {
                const float d = p.dt_out[o + q];
                f = __expf(p.cs_f[o + Q - 1] - p.cs_f[o + q]) * d;
                r = __expf(p.cs_b[o] - p.cs_b[o + q]) * d;
            }
        }
        wf[q] = f;
        wb[q] = r;
    }
    const T *xp;
    int64_t xs;
    if (DSTATES) {
        const T *src = reinterpret_cast<const T *>(p.has_z ? p.dout_x : p.dout);
        if (p.has_z) { xs = (int64_t)p.nheads * P; xp = src + ((int64_t)b * p.seqlen + (int64_t)c * Q) * xs + (int64_t)h * P; }
        else { xs = p.dout_sl; xp = src + b * p.dout_sb + (int64_t)c * Q * xs + h * p.dout_sh; }
    } else {
        xs = p.x_sl;
        xp = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * xs + h * p.x_sh;
    }
    xp += pt * 64;
    const T *bp;
    int64_t bs;
    if (DSTATES) { bs = p.C_sl; bp = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * bs + g * p.C_sg; }
    else { bs = p.B_sl; bp = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * bs + g * p.B_sg; }
    bp += nt * 64;
    f32x4 accf[4] = {}, accb[4] = {};
    for (int k0 = 0; k0 < limit; k0 += KH) {
        __syncthreads();       // weights written / previous round consumed
        const int kv = limit - k0;
        stage_transposed<T, KH, 64, LDX, FAST>(xT, xp + (int64_t)k0 * xs, xs, kv, P - pt * 64,
                                               [&](int k) { return k < kv ? 1.f : 0.f; });
        stage_transposed2<T, KH, 64, LDX, FAST>(Bf, Bb, bp + (int64_t)k0 * bs, bs, kv, N - nt * 64,
                                                [&](int k) { return k < kv ? wf[k0 + k] : 0.f; },
                                                [&](int k) { return k < kv ? wb[k0 + k] : 0.f; });
        __syncthreads();
        const int kend = min(KH, (kv + KSTEP - 1) / KSTEP * KSTEP);
        for (int ks = 0; ks < kend; ks += KSTEP) {
            const int kq = ks + lg * KPL;
            const typename M::Frag a = M::load(xT + xt_index<T, LDX>(wave * 16 + lr, kq));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                accf[j] = M::mma(a, M::load(Bf + xt_index<T, LDX>(j * 16 + lr, kq)), accf[j]);
                accb[j] = M::mma(a, M::load(Bb + xt_index<T, LDX>(j * 16 + lr, kq)), accb[j]);
            }
        }
    }
    float *of = (DSTATES ? p.dstates_f : p.states_f) + (int64_t)blockIdx.z * P * N;
    float *ob = (DSTATES ? p.dstates_b : p.states_b) + (int64_t)blockIdx.z * P * N;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pp = pt * 64 + wave * 16 + lg * 4 + i, n = nt * 64 + j * 16 + lr;
            if (pp < P && n < N) {
                of[(int64_t)pp * N + n] = accf[j][i];
                ob[(int64_t)pp * N + n] = accb[j][i];
            }
        }
}

// ---------------------------------------------------------------------------------------------------------
// The same for 16-bit types with headdim % 64 == 0, dstate % 64 == 0, chunk_size % 32 == 0 and aligned operands: both
// tiles travel as they are from global memory into LDS (direct loads: no registers, nothing to wait for until all of
// the chunk is under way), and the MFMA operands are read from the row-major images with LDS transpose reads.  The
// weights go onto the x-side fragment, one scaled copy per direction; the B-side fragments serve both directions.
// ---------------------------------------------------------------------------------------------------------
// CUMSUM (states only): the workgroup also does the work of chunk_cumsum_fwd_kernel for its (b, c, h) - wave 0 transforms
// dt and scans it while the tiles are under way - and the first tile's workgroup writes dt_out, cs_f, cs_b for the later
// kernels: one launch less in front of the forward pass.
// UNI: forward direction only (single-direction comparator).
// OUT16 (chunk states of the forward pass only): the per-chunk states leave in the inputs' 16-bit type, into states16_f/b
// (where the inter-chunk scan turns them into the entering states in place) - half the bytes of the float32 tensors; the
// tile passes through LDS so that it is written as 16-byte vectors, a whole 128-byte row piece per eight lanes.
template <typename T, bool DSTATES, bool CUMSUM, bool UNI = false, bool OUT16 = false>
__global__ __launch_bounds__(NTHREADS) void chunk_state_direct_kernel(const bimamba2_params p, int nc) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    static_assert(sizeof(T) == 2, "16-bit operands");
    constexpr int KR = 4;                                  // ring of K steps (32 positions each): requests run KR - 1 steps ahead
    __shared__ __attribute__((aligned(16))) T xt[KR * 32 * 64];
    __shared__ __attribute__((aligned(16))) T bt[KR * 32 * 64];
    __shared__ __attribute__((aligned(16))) float wf[BIMAMBA2_MAX_CHUNK], wb[BIMAMBA2_MAX_CHUNK];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    // Workgroups are dealt to the chip's eight dies in launch order, one after the other, and each die has its own L2.
    // Workgroups that read the same rows are therefore put eight launch positions apart, i.e. on one die.  With small
    // groups (at most 8 heads) that is all the workgroups of one (b, c) - the tiles of a head share its x rows, the heads of
    // a group the B (C) rows: eight (b, c) at a time, one per die, go through their heads and tiles (in plain launch order
    // the 4 heads of a group of the 8-group benchmark shape sat on 4 dies and each fetched the B rows: 151 -> 100 MB read).
    // With large groups only the tiles of one (b, c, h) are kept together: the heads of a (b, c) spread over the dies,
    // a few per die, and the B rows are a small part of the traffic (all 32 heads of a one-group (b, c) on one die, asking
    // for the same B tile at the same time, made the launch slower: 16.3 -> 18.7 us).
    int nt = blockIdx.x, pt = blockIdx.y, bch = blockIdx.z;
    {
        const int tiles = gridDim.x * gridDim.y;
        const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        if (p.nheads <= 8 * p.ngroups) {
            int inner, bc_;
            xcd_order(lin, tiles * p.nheads, (int)gridDim.z / p.nheads, inner, bc_);
            const int tile = inner % tiles;
            bch = bc_ * p.nheads + inner / tiles;
            nt = tile % (int)gridDim.x;
            pt = tile / (int)gridDim.x;
        } else if (tiles > 1) {
            int tile;
            xcd_order(lin, tiles, (int)gridDim.z, tile, bch);
            nt = tile % (int)gridDim.x;
            pt = tile / (int)gridDim.x;
        }
    }
    const int h = bch % p.nheads, bc = bch / p.nheads, c = bc % nc, b = bc / nc;
    const int g = h / (p.nheads / p.ngroups);
    const int Q = p.chunk_size, N = p.dstate, P = p.headdim;
    const int limit = min(Q, p.seqlen - c * Q);
    const T *xp;
    int64_t xs;
    if (DSTATES) {
        const T *src = reinterpret_cast<const T *>(p.has_z ? p.dout_x : p.dout);
        if (p.has_z) { xs = (int64_t)p.nheads * P; xp = src + ((int64_t)b * p.seqlen + (int64_t)c * Q) * xs + (int64_t)h * P; }
        else { xs = p.dout_sl; xp = src + b * p.dout_sb + (int64_t)c * Q * xs + h * p.dout_sh; }
    } else {
        xs = p.x_sl;
        xp = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * xs + h * p.x_sh;
    }
    const T *bp;
    int64_t bs;
    if (DSTATES) { bs = p.C_sl; bp = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * bs + g * p.C_sg; }
    else { bs = p.B_sl; bp = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * bs + g * p.B_sg; }
    const int rows = (limit + 31) & ~31, nsteps = rows / 32;     // K steps of 32 positions
    const int64_t o = (((int64_t)b * p.nheads + h) * nc + c) * Q;
    constexpr bool DO_CUMSUM = CUMSUM && !DSTATES;
    // Order of this wave's vector memory operations: first the few register loads the weight tables need, then, K step by
    // K step, one request for 8 rows of the x tile and one for 8 rows of the B tile (4 waves x 8 rows = the 32 rows of a
    // step).  Loads complete in order, so "at most 2 (nsteps - 1 - s) outstanding" means that the register loads and this
    // wave's part of steps 0..s have landed; a barrier then covers the other waves' parts.  The products of step s run
    // while the later steps are still under way.  Until the last step every LDS access is a raw one (the compiler would
    // make an access it knows of wait for all outstanding requests).
    float r_cf = 0.f, r_cb = 0.f, r_dt = 0.f, e_f = 0.f, e_b = 0.f, A_h = 0.f, bias_h = 0.f;
    unsigned dt_raw[4] = {0u, 0u, 0u, 0u};                   // DO_CUMSUM, wave 0: bits of dt at this lane's four positions
    if constexpr (DO_CUMSUM) {
        if (wave == 0) {
            const int64_t dto = b * p.dt_sb + (int64_t)c * Q * p.dt_sl + h * p.dt_sh;
            int64_t at[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) at[e] = dto + (int64_t)min(lane * 4 + e, limit - 1) * p.dt_sl;
            if (p.dt_dtype == BIMAMBA2_F32) {
#pragma unroll
                for (int e = 0; e < 4; ++e) dt_raw[e] = __float_as_uint(raw_global_load_f32(reinterpret_cast<const float *>(p.dt) + at[e]));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) dt_raw[e] = raw_global_load_u16(reinterpret_cast<const uint16_t *>(p.dt) + at[e]);
            }
            A_h = raw_global_load_f32(p.A + h);
            bias_h = raw_global_load_f32(p.has_dt_bias ? p.dt_bias + h : p.A + h);
        }
    } else {
        const int q = min((int)threadIdx.x, limit - 1);      // chunk_size <= 256 = NTHREADS: one position per thread
        r_cf = raw_global_load_f32(p.cs_f + o + q);
        r_cb = raw_global_load_f32(p.cs_b + o + q);
        if (!DSTATES) {
            r_dt = raw_global_load_f32(p.dt_out + o + q);
            e_f = raw_global_load_f32(p.cs_f + o + Q - 1);
            e_b = raw_global_load_f32(p.cs_b + o);
        }
    }
    // step s: this wave's 8 rows of the x tile and of the B tile, into slot s % KR (the swizzle of a row does not depend on s)
    auto issue = [&](int s) {
        const int row = 32 * s + 8 * wave + (lane >> 3);
        const int col = ((lane & 7) ^ tile64_swz(row)) << 3;
        const int at = ((s % KR) * 4 + wave) * 512;
        load16_to_lds(xp + pt * 64 + (int64_t)min(row, limit - 1) * xs + col, xt + at);
        load16_to_lds(bp + nt * 64 + (int64_t)min(row, limit - 1) * bs + col, bt + at);
    };
    const int nahead = min(KR - 1, nsteps);
    for (int s = 0; s < nahead; ++s) issue(s);
    auto wait_steps = [&](int newer) {       // at most 2 * newer requests outstanding (newer is wave-uniform, 0..7)
        switch (newer) {
            case 0: wait_vmcnt<0>(); break;
            case 1: wait_vmcnt<2>(); break;
            case 2: wait_vmcnt<4>(); break;
            case 3: wait_vmcnt<6>(); break;
            case 4: wait_vmcnt<8>(); break;
            case 5: wait_vmcnt<10>(); break;
            case 6: wait_vmcnt<12>(); break;
            case 7: wait_vmcnt<14>(); break;
            default: wait_vmcnt<16>(); break;
        }
    };
    const unsigned wf_a = lds_addr(wf), wb_a = lds_addr(wb);
    float keep_dt[4], keep_f[4], keep_b[4];                  // DO_CUMSUM, wave 0: what the first tile's workgroup writes out at the end
    if constexpr (DO_CUMSUM) {
        __shared__ float dts[BIMAMBA2_MAX_CHUNK], csfs[BIMAMBA2_MAX_CHUNK], csbs[BIMAMBA2_MAX_CHUNK];
        const unsigned dts_a = lds_addr(dts), csf_a = lds_addr(csfs), csb_a = lds_addr(csbs);
        if (wave == 0) {
            wait_steps(nahead);
            raw_lds_use(A_h); raw_lds_use(bias_h);
#pragma unroll
            for (int e = 0; e < 4; ++e) raw_lds_use(dt_raw[e]);
            const float A = A_h;
            const float bias = p.has_dt_bias ? bias_h : 0.f;
            float a[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int q = lane * 4 + e;
                const float dtv = p.dt_dtype == BIMAMBA2_F32 ? __uint_as_float(dt_raw[e])
                                  : p.dt_dtype == BIMAMBA2_BF16 ? __uint_as_float(dt_raw[e] << 16)
                                                                : to_f(__builtin_bit_cast(f16_t, (unsigned short)dt_raw[e]));
                float d = dtv + bias;
                if (p.dt_softplus) d = d > 20.f ? d : log1pf(expf(d));
                d = fminf(fmaxf(d, p.dt_min), p.dt_max);
                if (q >= limit) d = 0.f;
                keep_dt[e] = d;
                a[e] = d * A;
            }
            float pf[4], sb[4];
            pf[0] = a[0]; pf[1] = pf[0] + a[1]; pf[2] = pf[1] + a[2]; pf[3] = pf[2] + a[3];
            sb[3] = a[3]; sb[2] = sb[3] + a[2]; sb[1] = sb[2] + a[1]; sb[0] = sb[1] + a[0];
            const float tot = pf[3];
            const float before = wave_incl_prefix(tot, lane) - tot, after = wave_incl_suffix(tot, lane) - tot;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                keep_f[e] = before + pf[e];
                keep_b[e] = after + sb[e];
            }
            raw_lds_write128_at<0>(dts_a + lane * 16, f32x4{keep_dt[0], keep_dt[1], keep_dt[2], keep_dt[3]});
            raw_lds_write128_at<0>(csf_a + lane * 16, f32x4{keep_f[0], keep_f[1], keep_f[2], keep_f[3]});
            raw_lds_write128_at<0>(csb_a + lane * 16, f32x4{keep_b[0], keep_b[1], keep_b[2], keep_b[3]});
            raw_lds_wait();
        }
        raw_lds_barrier();
        {
            const int q = threadIdx.x;
            float d = raw_lds_read_at<float, 0>(dts_a + q * 4), cf = raw_lds_read_at<float, 0>(csf_a + q * 4);
            float cb = raw_lds_read_at<float, 0>(csb_a + q * 4);
            float ef = raw_lds_read_at<float, 0>(csf_a + (Q - 1) * 4), eb = raw_lds_read_at<float, 0>(csb_a);
            raw_lds_wait();
            raw_lds_use(d); raw_lds_use(cf); raw_lds_use(cb); raw_lds_use(ef); raw_lds_use(eb);
            const bool in = q < limit;
            raw_lds_write_at<0>(wf_a + q * 4, in ? __expf(ef - cf) * d : 0.f);
            raw_lds_write_at<0>(wb_a + q * 4, in ? __expf(eb - cb) * d : 0.f);
            raw_lds_wait();
        }
    } else {
        wait_steps(nahead);
        raw_lds_use(r_cf); raw_lds_use(r_cb); raw_lds_use(r_dt); raw_lds_use(e_f); raw_lds_use(e_b);
        const int q = threadIdx.x;
        float f = 0.f, r = 0.f;
        if (q < limit) {
            if (DSTATES) { f = __expf(r_cf); r = __expf(r_cb); }
            else { f = __expf(e_f - r_cf) * r_dt; r = __expf(e_b - r_cb) * r_dt; }
        }
        raw_lds_write_at<0>(wf_a + q * 4, f);
        raw_lds_write_at<0>(wb_a + q * 4, r);
        raw_lds_wait();
    }
    // lane parts of the fragment addresses (see tile64_tr_frag): rows kk and kk + 4 of a step, 4 columns from nn on
    const int kk = 8 * lg + (lr >> 2), nn = 4 * (lr & 3);
    const unsigned xa_lo = lds_addr(xt) + tile64_tr_offset(kk, wave * 16 + nn), xa_hi = lds_addr(xt) + tile64_tr_offset(kk + 4, wave * 16 + nn);
    unsigned ba_lo[4], ba_hi[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        ba_lo[j] = lds_addr(bt) + tile64_tr_offset(kk, j * 16 + nn);
        ba_hi[j] = lds_addr(bt) + tile64_tr_offset(kk + 4, j * 16 + nn);
    }
    const unsigned wfl = wf_a + 32 * lg, wbl = wb_a + 32 * lg;
    f32x4 accf[4] = {}, accb[4] = {};
    auto kstep = [&](auto S) {
        constexpr int s = decltype(S)::value;
        constexpr int TO = (s % KR) * 32 * 128, WO = s * 32 * 4;   // byte offsets of the step's slot / in the weight tables
        wait_steps(min(KR - 2, nsteps - 1 - s));           // this wave's part of step s has landed ...
        raw_lds_barrier();                                  // ... and everybody's; the slot of step s - 1 is free again
        if (s + KR - 1 < nsteps) issue(s + KR - 1);
        i16x4 alo = raw_lds_tr16_read_at<TO>(xa_lo), ahi = raw_lds_tr16_read_at<TO>(xa_hi);
        f32x4 f0 = raw_lds_read_at<f32x4, WO>(wfl), f1 = raw_lds_read_at<f32x4, WO + 16>(wfl);
        f32x4 r0 = raw_lds_read_at<f32x4, WO>(wbl), r1 = raw_lds_read_at<f32x4, WO + 16>(wbl);
        i16x4 blo[4], bhi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) { blo[j] = raw_lds_tr16_read_at<TO>(ba_lo[j]); bhi[j] = raw_lds_tr16_read_at<TO>(ba_hi[j]); }
        raw_lds_wait();
        raw_lds_use(alo); raw_lds_use(ahi); raw_lds_use(f0); raw_lds_use(f1); raw_lds_use(r0); raw_lds_use(r1);
        const Frag a = __builtin_bit_cast(Frag, __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7));
        float vf[8], vb[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float v = to_f(a[i]);
            vf[i] = v * (i < 4 ? f0[i & 3] : f1[i & 3]);
            vb[i] = v * (i < 4 ? r0[i & 3] : r1[i & 3]);
        }
        const Frag af = M::pack(vf), ab = M::pack(vb);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            raw_lds_use(blo[j]); raw_lds_use(bhi[j]);
            const Frag bfr = __builtin_bit_cast(Frag, __builtin_shufflevector(blo[j], bhi[j], 0, 1, 2, 3, 4, 5, 6, 7));
            accf[j] = M::mma(af, bfr, accf[j]);
            if (!UNI) accb[j] = M::mma(ab, bfr, accb[j]);
        }
    };
    static_assert(BIMAMBA2_MAX_CHUNK == 256, "eight K steps of 32 positions");
    kstep(std::integral_constant<int, 0>());
    if (nsteps > 1) kstep(std::integral_constant<int, 1>());
    if (nsteps > 2) kstep(std::integral_constant<int, 2>());
    if (nsteps > 3) kstep(std::integral_constant<int, 3>());
    if (nsteps > 4) kstep(std::integral_constant<int, 4>());
    if (nsteps > 5) kstep(std::integral_constant<int, 5>());
    if (nsteps > 6) kstep(std::integral_constant<int, 6>());
    if (nsteps > 7) kstep(std::integral_constant<int, 7>());
    if constexpr (OUT16) {
        // the two 64 x 64 tiles as 16-bit values into the rings' LDS (everybody is done reading them behind the barrier): row
        // r at r * 128 bytes, 16-byte chunk ch at position ch ^ ((r / 4) % 4), which keeps the four lane groups (rows 4 apart)
        // off each other's banks; then every thread takes 32 contiguous bytes of a row of each tile to memory
        __syncthreads();
        unsigned char *stf = reinterpret_cast<unsigned char *>(xt), *stb = reinterpret_cast<unsigned char *>(bt);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = wave * 16 + lg * 4 + i, col = j * 16 + lr;
                const int at = r * 128 + ((((col >> 3) ^ lg) << 4) | ((col & 7) << 1));
                *reinterpret_cast<T *>(stf + at) = from_f<T>(accf[j][i]);
                if (!UNI) *reinterpret_cast<T *>(stb + at) = from_f<T>(accb[j][i]);
            }
        __syncthreads();
        const int r = threadIdx.x >> 2, c2 = (threadIdx.x & 3) * 2, sw = (r >> 2) & 3;
        T *of = reinterpret_cast<T *>(DSTATES ? p.dstates16_f : p.states16_f) + (int64_t)bch * P * N + (int64_t)(pt * 64 + r) * N + nt * 64 + c2 * 8;
        T *ob = reinterpret_cast<T *>(DSTATES ? p.dstates16_b : p.states16_b) + (int64_t)bch * P * N + (int64_t)(pt * 64 + r) * N + nt * 64 + c2 * 8;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int at = r * 128 + (((c2 + k) ^ sw) << 4);
            *reinterpret_cast<f32x4 *>(of + k * 8) = *reinterpret_cast<const f32x4 *>(stf + at);
            if (!UNI) *reinterpret_cast<f32x4 *>(ob + k * 8) = *reinterpret_cast<const f32x4 *>(stb + at);
        }
    } else {
    float *of = (DSTATES ? p.dstates_f : p.states_f) + (int64_t)bch * P * N;
    float *ob = (DSTATES ? p.dstates_b : p.states_b) + (int64_t)bch * P * N;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pp = pt * 64 + wave * 16 + lg * 4 + i, n = nt * 64 + j * 16 + lr;
            of[(int64_t)pp * N + n] = accf[j][i];
            if (!UNI) ob[(int64_t)pp * N + n] = accb[j][i];
        }
    }
    if constexpr (DO_CUMSUM) {
        if (wave == 0 && nt == 0 && pt == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int q = lane * 4 + e;
                if (q < Q) {
                    p.dt_out[o + q] = keep_dt[e];
                    p.cs_f[o + q] = keep_f[e];
                    p.cs_b[o + q] = keep_b[e];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// dz and dstates in one pass (16-bit types, z gate, dstate 64, headdim % 64 == 0, chunk_size % 32 == 0): the workgroup of
// (b, c, h, 64 channels) takes dout, z and the ungated forward output through registers, 32 positions at a time and two
// steps ahead, writes dz and dout_x = dout silu(z) for the later kernels and puts dout_x into LDS where the other kernel
// requests it from memory: dstates is then the chunk-state product of dout_x with C as above.  dout_x is not read back
// by this kernel and the launch of the dz kernel goes away.
// Order of a wave's vector memory operations: two loads for the weight tables, then per step dout, z, out_x (registers)
// and its 8 rows of the C tile (direct to LDS); the stores of a step follow its loads by two steps.  Loads complete in
// order among themselves, stores do not keep that order, so a wait counts the younger loads only.
// UNI: forward direction only (single-direction comparator).
// ---------------------------------------------------------------------------------------------------------
template <typename T, bool UNI = false>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void bwd_dz_dstates_kernel(const bimamba2_params p, int nc) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    static_assert(sizeof(T) == 2, "16-bit operands");
    constexpr int KX = 2, KB = 3;                          // slots of the dout_x ring (written here) and of the C ring (requests 2 steps ahead)
    __shared__ __attribute__((aligned(16))) T xt[KX * 32 * 64];
    __shared__ __attribute__((aligned(16))) T bt[KB * 32 * 64];
    __shared__ __attribute__((aligned(16))) float wf[BIMAMBA2_MAX_CHUNK], wb[BIMAMBA2_MAX_CHUNK];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    // with small groups the workgroups of one (b, c) run on one die, as in chunk_state_direct_kernel: the heads of a group
    // share the C rows
    int pt = blockIdx.y, bch = blockIdx.z;
    if (p.nheads <= 8 * p.ngroups) {
        const int lin = blockIdx.y + gridDim.y * blockIdx.z;
        int inner, bc_;
        xcd_order(lin, (int)gridDim.y * p.nheads, (int)gridDim.z / p.nheads, inner, bc_);
        pt = inner % (int)gridDim.y;
        bch = bc_ * p.nheads + inner / (int)gridDim.y;
    }
    const int h = bch % p.nheads, bc = bch / p.nheads, c = bc % nc, b = bc / nc;
    const int g = h / (p.nheads / p.ngroups);
    const int Q = p.chunk_size, N = p.dstate, P = p.headdim;
    const int limit = min(Q, p.seqlen - c * Q);
    const int nsteps = ((limit + 31) & ~31) / 32;
    const int64_t o = (((int64_t)b * p.nheads + h) * nc + c) * Q;
    // this lane's 16 bytes of a step: row 8 wave + lane / 8 of the step's 32, the column chunk that the swizzled tile holds
    // at lane % 8 (the swizzle of a row does not depend on the step)
    const int row0 = 8 * wave + (lane >> 3);
    const int col = pt * 64 + (((lane & 7) ^ tile64_swz(row0)) << 3);
    const T *zp = reinterpret_cast<const T *>(p.z) + b * p.z_sb + (int64_t)c * Q * p.z_sl + h * p.z_sh + col;
    const T *dp = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * p.dout_sl + h * p.dout_sh + col;
    const int64_t os = (int64_t)p.nheads * P;               // row stride of out_x, dz, dout_x
    const int64_t ob = ((int64_t)b * p.seqlen + (int64_t)c * Q) * os + (int64_t)h * P + col;
    const T *oxp = reinterpret_cast<const T *>(p.out_x) + ob;
    T *dzp = reinterpret_cast<T *>(p.dz) + ob;
    T *doxp = reinterpret_cast<T *>(p.dout_x) + ob;
    const int64_t bs = p.C_sl;
    const T *bp = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * bs + g * p.C_sg + (((lane & 7) ^ tile64_swz(row0)) << 3);
    float r_cf, r_cb;
    {
        const int q = min((int)threadIdx.x, limit - 1);
        r_cf = raw_global_load_f32(p.cs_f + o + q);
        r_cb = raw_global_load_f32((UNI ? p.cs_f : p.cs_b) + o + q);     // (UNI: a second load all the same, the waits below count two)
    }
    f32x4 rd[2], rz[2], ro[2];                               // two steps in flight
    auto issue = [&](auto S) {
        constexpr int s = decltype(S)::value;
        const int row = min(32 * s + row0, limit - 1);
        rd[s % 2] = raw_global_load_b128<f32x4>(dp + (int64_t)row * p.dout_sl);
        rz[s % 2] = raw_global_load_b128<f32x4>(zp + (int64_t)row * p.z_sl);
        ro[s % 2] = raw_global_load_b128<f32x4>(oxp + (int64_t)row * os);
        load16_to_lds(bp + (int64_t)row * bs, bt + ((s % KB) * 4 + wave) * 512);
    };
    issue(std::integral_constant<int, 0>());
    if (nsteps > 1) issue(std::integral_constant<int, 1>());
    const unsigned wf_a = lds_addr(wf), wb_a = lds_addr(wb);
    if (nsteps > 1) wait_vmcnt<8>(); else wait_vmcnt<4>();
    raw_lds_use(r_cf); raw_lds_use(r_cb);
    {
        const int q = threadIdx.x;
        raw_lds_write_at<0>(wf_a + q * 4, q < limit ? __expf(r_cf) : 0.f);
        if (!UNI) raw_lds_write_at<0>(wb_a + q * 4, q < limit ? __expf(r_cb) : 0.f);
        raw_lds_wait();
    }
    const int kk = 8 * lg + (lr >> 2), nn = 4 * (lr & 3);
    const unsigned xa_lo = lds_addr(xt) + tile64_tr_offset(kk, wave * 16 + nn), xa_hi = lds_addr(xt) + tile64_tr_offset(kk + 4, wave * 16 + nn);
    unsigned ba_lo[4], ba_hi[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        ba_lo[j] = lds_addr(bt) + tile64_tr_offset(kk, j * 16 + nn);
        ba_hi[j] = lds_addr(bt) + tile64_tr_offset(kk + 4, j * 16 + nn);
    }
    const unsigned xw = lds_addr(xt) + wave * 1024 + lane * 16;     // where this lane's 16 bytes of dout_x go (slot 0)
    const unsigned wfl = wf_a + 32 * lg, wbl = wb_a + 32 * lg;
    f32x4 accf[4] = {}, accb[4] = {};
    auto kstep = [&](auto S) {
        constexpr int s = decltype(S)::value;
        constexpr int XO = (s % KX) * 32 * 128, BO = (s % KB) * 32 * 128, WO = s * 32 * 4;
        if (s + 1 < nsteps) wait_vmcnt<4>(); else wait_vmcnt<0>();      // this wave's loads of step s have landed
        raw_lds_use(rd[s % 2]); raw_lds_use(rz[s % 2]); raw_lds_use(ro[s % 2]);
        {
            const Vec16<T> a = __builtin_bit_cast(Vec16<T>, rz[s % 2]), d = __builtin_bit_cast(Vec16<T>, rd[s % 2]),
                           e = __builtin_bit_cast(Vec16<T>, ro[s % 2]);
            Vec16<T> r1, r2;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float zv = to_f(a.v[i]), dv = to_f(d.v[i]), ov = to_f(e.v[i]);
                const float sg = sigmoid_f(zv);
                r1.v[i] = from_f<T>(dv * ov * sg * (1.f + zv * (1.f - sg)));
                r2.v[i] = from_f<T>(dv * zv * sg);
            }
            raw_lds_write128_at<XO>(xw, __builtin_bit_cast(f32x4, r2));
            const int row = 32 * s + row0;
            if (row < limit) {
                __builtin_nontemporal_store(__builtin_bit_cast(f32x4, r1), reinterpret_cast<f32x4 *>(dzp + (int64_t)row * os));
                *reinterpret_cast<f32x4 *>(doxp + (int64_t)row * os) = __builtin_bit_cast(f32x4, r2);
            }
        }
        raw_lds_wait();
        raw_lds_barrier();          // dout_x and everybody's C rows of step s are in LDS; the slots of step s - 1 are free again
        if constexpr (s + 2 < 8) {
            if (s + 2 < nsteps) issue(std::integral_constant<int, s + 2>());
        }
        i16x4 alo = raw_lds_tr16_read_at<XO>(xa_lo), ahi = raw_lds_tr16_read_at<XO>(xa_hi);
        f32x4 f0 = raw_lds_read_at<f32x4, WO>(wfl), f1 = raw_lds_read_at<f32x4, WO + 16>(wfl);
        f32x4 r0 = {0.f, 0.f, 0.f, 0.f}, r1 = {0.f, 0.f, 0.f, 0.f};
        if (!UNI) { r0 = raw_lds_read_at<f32x4, WO>(wbl); r1 = raw_lds_read_at<f32x4, WO + 16>(wbl); }
        i16x4 blo[4], bhi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) { blo[j] = raw_lds_tr16_read_at<BO>(ba_lo[j]); bhi[j] = raw_lds_tr16_read_at<BO>(ba_hi[j]); }
        raw_lds_wait();
        raw_lds_use(alo); raw_lds_use(ahi); raw_lds_use(f0); raw_lds_use(f1);
        if (!UNI) { raw_lds_use(r0); raw_lds_use(r1); }
        const Frag a = __builtin_bit_cast(Frag, __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7));
        float vf[8], vb[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float v = to_f(a[i]);
            vf[i] = v * (i < 4 ? f0[i & 3] : f1[i & 3]);
            vb[i] = v * (i < 4 ? r0[i & 3] : r1[i & 3]);
        }
        const Frag af = M::pack(vf), ab = M::pack(vb);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            raw_lds_use(blo[j]); raw_lds_use(bhi[j]);
            const Frag bfr = __builtin_bit_cast(Frag, __builtin_shufflevector(blo[j], bhi[j], 0, 1, 2, 3, 4, 5, 6, 7));
            accf[j] = M::mma(af, bfr, accf[j]);
            if (!UNI) accb[j] = M::mma(ab, bfr, accb[j]);
        }
    };
    static_assert(BIMAMBA2_MAX_CHUNK == 256, "eight K steps of 32 positions");
    kstep(std::integral_constant<int, 0>());
    if (nsteps > 1) kstep(std::integral_constant<int, 1>());
    if (nsteps > 2) kstep(std::integral_constant<int, 2>());
    if (nsteps > 3) kstep(std::integral_constant<int, 3>());
    if (nsteps > 4) kstep(std::integral_constant<int, 4>());
    if (nsteps > 5) kstep(std::integral_constant<int, 5>());
    if (nsteps > 6) kstep(std::integral_constant<int, 6>());
    if (nsteps > 7) kstep(std::integral_constant<int, 7>());
    if (p.dstates_f == nullptr) {
        // no float32 tensors for the per-chunk gradients: they go to dstates16_f/b in the 16-bit type (where the backward
        // inter-chunk scan replaces them in place), through LDS as 16-byte vectors - see chunk_state_direct_kernel<.., OUT16>
        __syncthreads();
        unsigned char *stf = reinterpret_cast<unsigned char *>(xt), *stb = reinterpret_cast<unsigned char *>(bt);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = wave * 16 + lg * 4 + i, cc = j * 16 + lr;
                const int at = r * 128 + ((((cc >> 3) ^ lg) << 4) | ((cc & 7) << 1));
                *reinterpret_cast<T *>(stf + at) = from_f<T>(accf[j][i]);
                if (!UNI) *reinterpret_cast<T *>(stb + at) = from_f<T>(accb[j][i]);
            }
        __syncthreads();
        const int r = threadIdx.x >> 2, c2 = (threadIdx.x & 3) * 2, sw = (r >> 2) & 3;
        const int64_t so = (int64_t)bch * P * N + (int64_t)(pt * 64 + r) * N + c2 * 8;
        T *of = reinterpret_cast<T *>(p.dstates16_f) + so, *ob16 = reinterpret_cast<T *>(p.dstates16_b) + so;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int at = r * 128 + (((c2 + k) ^ sw) << 4);
            *reinterpret_cast<f32x4 *>(of + k * 8) = *reinterpret_cast<const f32x4 *>(stf + at);
            if (!UNI) *reinterpret_cast<f32x4 *>(ob16 + k * 8) = *reinterpret_cast<const f32x4 *>(stb + at);
        }
        return;
    }
    float *of = p.dstates_f + (int64_t)bch * P * N;
    float *obk = (UNI ? p.dstates_f : p.dstates_b) + (int64_t)bch * P * N;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pp = pt * 64 + wave * 16 + lg * 4 + i, n = j * 16 + lr;
            of[(int64_t)pp * N + n] = accf[j][i];
            if (!UNI) obk[(int64_t)pp * N + n] = accb[j][i];
        }
}

// =========================================================================================================
// inter-chunk recurrences, both directions, in place:
//   forward : prev_f[0] = 0, prev_f[c+1] = e^{tot_c} prev_f[c] + S_f[c]   (final_f = value after the last chunk)
//   reverse : prev_b[nc-1] = 0, prev_b[c-1] = e^{tot_c} prev_b[c] + S_b[c] (final_b = value after chunk 0)
// One thread owns one (b, h, p, n) element; the chunk loop is unrolled by 8 so that 8 loads are in flight.
// =========================================================================================================
__global__ __launch_bounds__(NTHREADS) void state_passing_fwd_kernel(const bimamba2_params p, int nc) {
    const int PN = p.headdim * p.dstate;
    const int e = blockIdx.x * NTHREADS + threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z;
    if (e >= PN) return;
    const int Q = p.chunk_size;
    const float *csf = p.cs_f + ((int64_t)b * p.nheads + h) * nc * Q;
    const float *csb = p.cs_b + ((int64_t)b * p.nheads + h) * nc * Q;
    const int64_t cstride = (int64_t)p.nheads * PN;
    float *sf = p.states_f + ((int64_t)b * nc * p.nheads + h) * PN + e;
    float *sb = p.states_b + ((int64_t)b * nc * p.nheads + h) * PN + e;
    float s = p.initial_f ? p.initial_f[((int64_t)b * p.nheads + h) * PN + e] : 0.f;
    for (int c0 = 0; c0 < nc; c0 += 8) {
        float v[8], d[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (c0 + i < nc) {
                v[i] = sf[(c0 + i) * cstride];
                d[i] = __expf(csf[(int64_t)(c0 + i) * Q + Q - 1]);
            }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (c0 + i < nc) {
                sf[(c0 + i) * cstride] = s;
                s = d[i] * s + v[i];
            }
    }
    if (p.final_f) p.final_f[((int64_t)b * p.nheads + h) * PN + e] = s;
    s = p.initial_b ? p.initial_b[((int64_t)b * p.nheads + h) * PN + e] : 0.f;
    for (int c0 = nc - 1; c0 >= 0; c0 -= 8) {
        float v[8], d[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (c0 - i >= 0) {
                v[i] = sb[(c0 - i) * cstride];
                d[i] = __expf(csb[(int64_t)(c0 - i) * Q]);
            }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (c0 - i >= 0) {
                sb[(c0 - i) * cstride] = s;
                s = d[i] * s + v[i];
            }
    }
    if (p.final_b) p.final_b[((int64_t)b * p.nheads + h) * PN + e] = s;
}

// =========================================================================================================
// launchers
// =========================================================================================================
static inline int nchunks(const bimamba2_params *p) { return (p->seqlen + p->chunk_size - 1) / p->chunk_size; }
static inline hipStream_t stream_of(const bimamba2_params *p) { return reinterpret_cast<hipStream_t>(p->stream); }

int launch_chunk_cumsum_fwd(const bimamba2_params *p) {
    const int nc = nchunks(p);
    dim3 grid((p->nheads + 3) / 4, nc, p->batch);
    switch (p->dt_dtype) {
        case BIMAMBA2_F32: hipLaunchKernelGGL(chunk_cumsum_fwd_kernel<float>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;
        case BIMAMBA2_BF16: hipLaunchKernelGGL(chunk_cumsum_fwd_kernel<bf16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;
        case BIMAMBA2_F16: hipLaunchKernelGGL(chunk_cumsum_fwd_kernel<f16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;
        default: return BIMAMBA2_EUNSUPPORTED;
    }
    return check_launch();
}

#define BM2_DISPATCH_T(p, KERNEL, grid, ...)                                                                          \
    switch ((p)->dtype) {                                                                                             \
        case BIMAMBA2_F32: hipLaunchKernelGGL((KERNEL<float, ##__VA_ARGS__>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;   \
        case BIMAMBA2_BF16: hipLaunchKernelGGL((KERNEL<bf16_t, ##__VA_ARGS__>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break; \
        case BIMAMBA2_F16: hipLaunchKernelGGL((KERNEL<f16_t, ##__VA_ARGS__>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;   \
        default: return BIMAMBA2_EUNSUPPORTED;                                                                        \
    }

int launch_bmm_chunk_fwd(const bimamba2_params *p) {
    const int nc = nchunks(p), qt = (p->chunk_size + 63) / 64;
    dim3 grid(qt, qt, p->batch * nc * p->ngroups);
    switch (p->dtype) {
        case BIMAMBA2_F32: hipLaunchKernelGGL(bmm_chunk_fwd_kernel<float>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;
        case BIMAMBA2_BF16: hipLaunchKernelGGL(bmm_chunk_fwd_kernel<bf16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;
        case BIMAMBA2_F16: hipLaunchKernelGGL(bmm_chunk_fwd_kernel<f16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc); break;
        default: return BIMAMBA2_EUNSUPPORTED;
    }
    return check_launch();
}

// Whether the forward pass of this problem can keep its per-chunk states in the 16-bit type only, in states16_f/b: written
// there by the chunk-state kernel with direct loads, turned into the entering states in place by the vector kernel of the
// inter-chunk scan (bidirectional operator, 16-byte aligned operands; the pointers themselves are checked where they are used).
bool chunk_states_in_16bit(const bimamba2_params *p) {
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % 8 == 0 && b % 8 == 0 && c % 8 == 0; };
    return p->dtype != BIMAMBA2_F32 && !p->causal && p->headdim % 64 == 0 && p->dstate % 64 == 0 && p->chunk_size % 32 == 0 &&
           al(p->Bm) && mult(p->B_sb, p->B_sl, p->B_sg) && al(p->x) && mult(p->x_sb, p->x_sl, p->x_sh) && al(p->states16_f) &&
           al(p->states16_b) && al(p->final_f) && al(p->final_b) && al(p->initial_f) && al(p->initial_b);
}

// ---------------------------------------------------------------------------------------------------------
// The chunk states of several heads of one (batch, chunk) in one workgroup (16-bit inputs, 16-bit per-chunk states out,
// state dimension NH * 64).  With many heads per group and a wide state the kernel above is made of thousands of short
// workgroups, each a chain of waits (weights, first rows, eight barriers, stores), and reaches half the memory rate; here a
// workgroup of 4 * NH waves keeps the B rows of the chunk in LDS (loaded once), walks through its heads with the x tile of
// the next head under way while the current one is multiplied, and stores a head's states while the next one is worked on.
//   wave w: rows 16 (w % 4) .. of the 64 channels, 64-column tile w / 4 of the state dimension.
//   LDS: B tile NH x [256][64] (tile64 swizzle) | two x tiles [256][64] | raw cs_f, cs_b, dt vectors of two heads | wf, wb.
//   The finished head's x tile serves as the staging area of its output (16-byte stores of whole 128-byte row pieces).
// Needs dt_out, cs_f, cs_b from bimamba2_chunk_cumsum_fwd.  Requests complete in order; a wave waits for everything it has
// in flight (vmcnt(0)) once per head, in front of that head's stores, when the next head's operands have long landed.
// ---------------------------------------------------------------------------------------------------------
template <int NH> struct CshMap {
    static constexpr int BT = 0;                               // NH tiles of 32 KB
    static constexpr int XT = BT + NH * 32768;                 // 2 x 32 KB
    static constexpr int RAW = XT + 2 * 32768;                 // 2 x (cs_f, cs_b, dt) x 1 KB
    static constexpr int WT = RAW + 2 * 3 * 1024;              // wf, wb
    static constexpr int LDS = WT + 2 * 1024;
};

template <typename T, int NH>
__global__ __launch_bounds__(NH * NTHREADS) void chunk_state_heads_kernel(const bimamba2_params p, int nc, int hpw) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    typedef CshMap<NH> L;
    static_assert(sizeof(T) == 2, "16-bit operands");
    __shared__ __attribute__((aligned(1024))) unsigned char smem[L::LDS];
    const unsigned sbase = lds_addr(smem);
    constexpr int NW = 4 * NH;
    const int lane = threadIdx.x & 63, wave8 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave = wave8 & 3, nh = wave8 >> 2;
    const int lr = lane & 15, lg = lane >> 4;
    const int pt = blockIdx.x, slice = blockIdx.y, bc = blockIdx.z, c = bc % nc, b = bc / nc;
    const int Q = p.chunk_size, N = p.dstate, P = p.headdim, H = p.nheads;
    const int h0 = slice * hpw, g = h0 / (H / p.ngroups);
    const int limit = min(Q, p.seqlen - c * Q);
    const int nsteps = (limit + 31) >> 5;
    // ---- the B rows of the chunk: tile t (64 columns) row r at t * 32 KB + r * 128, 16-byte chunk ^ tile64_swz(r)
    {
        const T *bp = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * p.B_sl + g * p.B_sg;
        for (int u = wave8; u < NH * 32; u += NW) {                  // units of 8 rows x 128 bytes
            const int t = u >> 5, row = (u & 31) * 8 + (lane >> 3);
            if ((u & 31) * 8 < nsteps * 32)
                load16_to_lds(bp + t * 64 + (int64_t)min(row, limit - 1) * p.B_sl + (((lane & 7) ^ tile64_swz(row)) << 3), smem + L::BT + u * 1024);
        }
    }
    // requests of a head: its x tile (32 units of 8 rows) and its three vectors, into buffer `buf`
    auto request_head = [&](int h, int buf) __attribute__((always_inline)) {
        const T *xp = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * p.x_sl + h * p.x_sh + pt * 64;
        for (int u = wave8; u < 32; u += NW) {
            const int row = u * 8 + (lane >> 3);
            if (u * 8 < nsteps * 32)
                load16_to_lds(xp + (int64_t)min(row, limit - 1) * p.x_sl + (((lane & 7) ^ tile64_swz(row)) << 3), smem + L::XT + buf * 32768 + u * 1024);
        }
        if (wave8 < 3) {
            const float *src = (wave8 == 0 ? p.cs_f : wave8 == 1 ? p.cs_b : p.dt_out) + (((int64_t)b * H + h) * nc + c) * Q;
            load16_to_lds(src + min(lane * 4, Q - 4), smem + L::RAW + (buf * 3 + wave8) * 1024);
        }
    };
    request_head(h0, 0);
    // lane parts of the fragment addresses (see tile64_tr_frag): rows kk and kk + 4 of a step, 4 columns from nn on
    const int kk = 8 * lg + (lr >> 2), nn = 4 * (lr & 3);
    const unsigned xa_lo0 = sbase + L::XT + tile64_tr_offset(kk, wave * 16 + nn), xa_hi0 = sbase + L::XT + tile64_tr_offset(kk + 4, wave * 16 + nn);
    unsigned ba_lo[4], ba_hi[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        ba_lo[j] = sbase + L::BT + nh * 32768 + tile64_tr_offset(kk, j * 16 + nn);
        ba_hi[j] = sbase + L::BT + nh * 32768 + tile64_tr_offset(kk + 4, j * 16 + nn);
    }
    const unsigned wfl = sbase + L::WT + 32 * lg, wbl = sbase + L::WT + 1024 + 32 * lg;
    wait_vmcnt<0>();
    for (int hi = 0; hi < hpw; ++hi) {
        const int h = h0 + hi, cur = hi & 1;
        // #1: this head's x tile and vectors have landed for everybody (each wave waited for its own requests in front of the
        // previous head's stores, or above); everybody is done with the other x buffer (the previous head's staging area)
        raw_lds_barrier();
        if (hi + 1 < hpw) request_head(h + 1, cur ^ 1);
        if (threadIdx.x < NTHREADS) {
            const int q = threadIdx.x, qq = min(q, Q - 1);
            const unsigned ra = sbase + L::RAW + cur * 3072;
            float cf = raw_lds_read_at<float, 0>(ra + qq * 4), cb = raw_lds_read_at<float, 1024>(ra + qq * 4);
            float d = raw_lds_read_at<float, 2048>(ra + qq * 4);
            float ef = raw_lds_read_at<float, 0>(ra + (Q - 1) * 4), eb = raw_lds_read_at<float, 1024>(ra);
            raw_lds_wait();
            raw_lds_use(cf); raw_lds_use(cb); raw_lds_use(d); raw_lds_use(ef); raw_lds_use(eb);
            const bool in = q < limit;
            raw_lds_write_at<0>(sbase + L::WT + q * 4, in ? __expf(ef - cf) * d : 0.f);
            raw_lds_write_at<1024>(sbase + L::WT + q * 4, in ? __expf(eb - cb) * d : 0.f);
            raw_lds_wait();
        }
        raw_lds_barrier();                          // #2: the weights are there
        f32x4 accf[4] = {}, accb[4] = {};
        const unsigned xa_lo = xa_lo0 + cur * 32768, xa_hi = xa_hi0 + cur * 32768;
        auto kstep = [&](auto S) __attribute__((always_inline)) {
            constexpr int s = decltype(S)::value;
            constexpr int TO = s * 32 * 128, WO = s * 32 * 4;
            i16x4 alo = raw_lds_tr16_read_at<TO>(xa_lo), ahi = raw_lds_tr16_read_at<TO>(xa_hi);
            f32x4 f0 = raw_lds_read_at<f32x4, WO>(wfl), f1 = raw_lds_read_at<f32x4, WO + 16>(wfl);
            f32x4 r0 = raw_lds_read_at<f32x4, WO>(wbl), r1 = raw_lds_read_at<f32x4, WO + 16>(wbl);
            i16x4 blo[4], bhi[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) { blo[j] = raw_lds_tr16_read_at<TO>(ba_lo[j]); bhi[j] = raw_lds_tr16_read_at<TO>(ba_hi[j]); }
            raw_lds_wait();
            raw_lds_use(alo); raw_lds_use(ahi); raw_lds_use(f0); raw_lds_use(f1); raw_lds_use(r0); raw_lds_use(r1);
            const Frag a = __builtin_bit_cast(Frag, __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7));
            float vf[8], vb[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float v = to_f(a[i]);
                vf[i] = v * (i < 4 ? f0[i & 3] : f1[i & 3]);
                vb[i] = v * (i < 4 ? r0[i & 3] : r1[i & 3]);
            }
            const Frag af = M::pack(vf), ab = M::pack(vb);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                raw_lds_use(blo[j]); raw_lds_use(bhi[j]);
                const Frag bfr = __builtin_bit_cast(Frag, __builtin_shufflevector(blo[j], bhi[j], 0, 1, 2, 3, 4, 5, 6, 7));
                accf[j] = M::mma(af, bfr, accf[j]);
                accb[j] = M::mma(ab, bfr, accb[j]);
            }
        };
        kstep(std::integral_constant<int, 0>());
        if (nsteps > 1) kstep(std::integral_constant<int, 1>());
        if (nsteps > 2) kstep(std::integral_constant<int, 2>());
        if (nsteps > 3) kstep(std::integral_constant<int, 3>());
        if (nsteps > 4) kstep(std::integral_constant<int, 4>());
        if (nsteps > 5) kstep(std::integral_constant<int, 5>());
        if (nsteps > 6) kstep(std::integral_constant<int, 6>());
        if (nsteps > 7) kstep(std::integral_constant<int, 7>());
        raw_lds_barrier();                          // #3: everybody is done with this head's x tile: it becomes the staging area
        // tile (direction d, column tile nh) at (d * NH + nh) * 8 KB: row r at r * 128, 16-byte chunk ch at ch ^ ((r / 4) % 4)
        const unsigned st = sbase + L::XT + cur * 32768;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = wave * 16 + lg * 4 + i, col = j * 16 + lr;
                const unsigned at = st + nh * 8192 + r * 128 + ((((col >> 3) ^ lg) << 4) | ((col & 7) << 1));
                // (the 16 bits of the value, whatever the type: the accessor takes them as a _Float16)
                raw_lds_write16_at<0>(at, __builtin_bit_cast(_Float16, from_f<T>(accf[j][i])));
                raw_lds_write16_at<NH * 8192>(at, __builtin_bit_cast(_Float16, from_f<T>(accb[j][i])));
            }
        raw_lds_wait();
        raw_lds_barrier();                          // #4
        {
            const int tid = threadIdx.x & 255, r = tid >> 2, c2 = (tid & 3) * 2, sw = (r >> 2) & 3;
            const unsigned at = st + nh * 8192 + r * 128;
            f32x4 vf0 = raw_lds_read_at<f32x4, 0>(at + ((c2 ^ sw) << 4)), vf1 = raw_lds_read_at<f32x4, 0>(at + (((c2 + 1) ^ sw) << 4));
            f32x4 vb0 = raw_lds_read_at<f32x4, NH * 8192>(at + ((c2 ^ sw) << 4)), vb1 = raw_lds_read_at<f32x4, NH * 8192>(at + (((c2 + 1) ^ sw) << 4));
            raw_lds_wait();
            raw_lds_use(vf0); raw_lds_use(vf1); raw_lds_use(vb0); raw_lds_use(vb1);
            // the next head's operands (this wave's share) have landed long ago; waited for here, in front of the stores
            wait_vmcnt<0>();
            const int64_t so = (((int64_t)(b * nc + c) * H + h) * P + pt * 64 + r) * N + nh * 64 + c2 * 8;
            T *of = reinterpret_cast<T *>(p.states16_f) + so, *ob = reinterpret_cast<T *>(p.states16_b) + so;
            *reinterpret_cast<f32x4 *>(of) = vf0;
            *reinterpret_cast<f32x4 *>(of + 8) = vf1;
            *reinterpret_cast<f32x4 *>(ob) = vb0;
            *reinterpret_cast<f32x4 *>(ob + 8) = vb1;
        }
    }
}

// heads per workgroup of the kernel above: the divisor of the heads per group (at most 32) that brings the number of workgroups
// closest to a whole number of rounds of one per CU, the larger on a tie
static int csh_heads_per_block(const bimamba2_params *p, int nc) {
    const int hpg = p->nheads / p->ngroups;
    int cus = 256;
    {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
    }
    const long long units = (long long)p->batch * nc * (p->headdim / 64) * p->nheads;
    int best = 1;
    double best_cost = 0;
    for (int k = 1; k <= std::min(hpg, 32); ++k) {
        if (hpg % k) continue;
        const long long rounds = (units / k + cus - 1) / cus;
        const double cost = rounds * (1.5 + k);          // a workgroup's start (B rows, first head's operands) costs about 1.5 heads
        if (k == 1 || cost <= best_cost) { best = k; best_cost = cost; }
    }
    return best;
}

bool chunk_state_uses_heads_kernel(const bimamba2_params *p) {
    // where it pays: a state of 128 columns and enough heads per group to share the B rows
    return chunk_states_in_16bit(p) && p->dstate == 128 && p->headdim % 64 == 0 && p->nheads / p->ngroups >= 4 &&
           p->x_sl > 0 && p->x_sl <= (1 << 21) && p->B_sl > 0 && p->B_sl <= (1 << 21);
}

template <typename T>
static int launch_chunk_state_heads_t(const bimamba2_params *p) {
    const int nc = nchunks(p), hpw = csh_heads_per_block(p, nc);
    dim3 grid(p->headdim / 64, p->nheads / hpw, p->batch * nc);
    hipLaunchKernelGGL((chunk_state_heads_kernel<T, 2>), grid, dim3(2 * NTHREADS), 0, stream_of(p), *p, nc, hpw);
    return check_launch();
}

int launch_chunk_state_heads(const bimamba2_params *p) {
    if (!p->states16_f || !p->states16_b || !chunk_state_uses_heads_kernel(p)) return BIMAMBA2_EINVAL;
    if (p->dtype == BIMAMBA2_BF16) return launch_chunk_state_heads_t<bf16_t>(p);
    if (p->dtype == BIMAMBA2_F16) return launch_chunk_state_heads_t<f16_t>(p);
    return BIMAMBA2_EUNSUPPORTED;
}


template <typename T>
static int launch_chunk_state_t(const bimamba2_params *p, bool dstates, bool cumsum) {
    const int nc = nchunks(p);
    dim3 grid((p->dstate + 63) / 64, (p->headdim + 63) / 64, p->batch * nc * p->nheads);
    constexpr int VS = 16 / (int)sizeof(T);
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % VS == 0 && b % VS == 0 && c % VS == 0; };
    bool fast = p->headdim % 64 == 0 && p->dstate % 64 == 0;
    if (dstates) {
        fast = fast && al(p->Cm) && mult(p->C_sb, p->C_sl, p->C_sg);
        fast = fast && (p->has_z ? al(p->dout_x) : (al(p->dout) && mult(p->dout_sb, p->dout_sl, p->dout_sh)));
    } else {
        fast = fast && al(p->Bm) && mult(p->B_sb, p->B_sl, p->B_sg) && al(p->x) && mult(p->x_sb, p->x_sl, p->x_sh);
    }
    hipStream_t s = stream_of(p);
    if constexpr (sizeof(T) == 2) {
        if (fast && p->chunk_size % 32 == 0 && dstates && !p->dstates_f) {
            // no float32 tensors for the per-chunk gradients: 16-bit, into dstates16_f/b
            if (!p->dstates16_f || !(p->causal || p->dstates16_b)) return BIMAMBA2_EINVAL;
            if (p->causal) hipLaunchKernelGGL((chunk_state_direct_kernel<T, true, false, true, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else hipLaunchKernelGGL((chunk_state_direct_kernel<T, true, false, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            return check_launch();
        }
        if (fast && p->chunk_size % 32 == 0 && p->causal) {
            if (dstates) hipLaunchKernelGGL((chunk_state_direct_kernel<T, true, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else if (cumsum) hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, true, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            return check_launch();
        }
        if (fast && p->chunk_size % 32 == 0 && !dstates && !p->states_f) {
            // no float32 tensors for the per-chunk states: they go to states16_f/b in the 16-bit type
            if (!p->states16_f || !p->states16_b || !chunk_states_in_16bit(p)) return BIMAMBA2_EINVAL;
            if (!cumsum && chunk_state_uses_heads_kernel(p)) return launch_chunk_state_heads(p);
            if (cumsum) hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, true, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, false, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            return check_launch();
        }
        if (fast && p->chunk_size % 32 == 0) {
            if (dstates) hipLaunchKernelGGL((chunk_state_direct_kernel<T, true, false>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else if (cumsum) hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, false>), grid, dim3(NTHREADS), 0, s, *p, nc);
            return check_launch();
        }
    }
    if (p->causal) return BIMAMBA2_EUNSUPPORTED;
    if (cumsum) return BIMAMBA2_EINVAL;      // the caller checked chunk_state_does_cumsum()
    if (!dstates && !(p->states_f && p->states_b)) return BIMAMBA2_EINVAL;   // (16-bit per-chunk states: the kernel above only)
    if (dstates && !(p->dstates_f && p->dstates_b)) return BIMAMBA2_EINVAL;
    if (dstates) {
        if (fast) hipLaunchKernelGGL((chunk_state_kernel<T, true, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
        else hipLaunchKernelGGL((chunk_state_kernel<T, true, false>), grid, dim3(NTHREADS), 0, s, *p, nc);
    } else {
        if (fast) hipLaunchKernelGGL((chunk_state_kernel<T, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
        else hipLaunchKernelGGL((chunk_state_kernel<T, false, false>), grid, dim3(NTHREADS), 0, s, *p, nc);
    }
    return check_launch();
}

int launch_chunk_state(const bimamba2_params *p, bool dstates, bool cumsum) {
    switch (p->dtype) {
        case BIMAMBA2_F32: return launch_chunk_state_t<float>(p, dstates, cumsum);
        case BIMAMBA2_BF16: return launch_chunk_state_t<bf16_t>(p, dstates, cumsum);
        case BIMAMBA2_F16: return launch_chunk_state_t<f16_t>(p, dstates, cumsum);
        default: return BIMAMBA2_EUNSUPPORTED;
    }
}

// whether launch_chunk_state(p, false, true) exists for this problem: the chunk-state launch that also does the chunk
// cumsum (16-bit dtype, headdim and dstate multiples of 64, chunk_size a multiple of 32, aligned x and B)
bool chunk_state_does_cumsum(const bimamba2_params *p) {
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % 8 == 0 && b % 8 == 0 && c % 8 == 0; };
    if (p->seq_idx) return false;                 // packed sequences: the stand-alone cumsum kernel applies the cuts
    // (the kernel that walks through several heads per workgroup reads the cumulative sums: the stand-alone launch comes first)
    if (!p->states_f && p->states16_f && p->states16_b && chunk_state_uses_heads_kernel(p)) return false;
    return p->dtype != BIMAMBA2_F32 && p->headdim % 64 == 0 && p->dstate % 64 == 0 && p->chunk_size % 32 == 0 && al(p->Bm) &&
           mult(p->B_sb, p->B_sl, p->B_sg) && al(p->x) && mult(p->x_sb, p->x_sl, p->x_sh);
}

// whether launch_bwd_dz_dstates(p) exists for this problem
bool bwd_dz_dstates_fused(const bimamba2_params *p) {
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % 8 == 0 && b % 8 == 0 && c % 8 == 0; };
    return p->has_z && p->dtype != BIMAMBA2_F32 && p->headdim % 64 == 0 && p->dstate == 64 && p->chunk_size % 32 == 0 &&
           al(p->Cm) && mult(p->C_sb, p->C_sl, p->C_sg) && al(p->z) && mult(p->z_sb, p->z_sl, p->z_sh) && al(p->dout) &&
           mult(p->dout_sb, p->dout_sl, p->dout_sh) && al(p->out_x) && al(p->dz) && al(p->dout_x);
}

int launch_bwd_dz_dstates(const bimamba2_params *p) {
    if (!bwd_dz_dstates_fused(p)) return BIMAMBA2_EUNSUPPORTED;
    const int nc = nchunks(p);
    dim3 grid(1, p->headdim / 64, p->batch * nc * p->nheads);
    if (p->causal) {
        if (p->dtype == BIMAMBA2_BF16) hipLaunchKernelGGL((bwd_dz_dstates_kernel<bf16_t, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
        else hipLaunchKernelGGL((bwd_dz_dstates_kernel<f16_t, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
    } else {
        if (p->dtype == BIMAMBA2_BF16) hipLaunchKernelGGL((bwd_dz_dstates_kernel<bf16_t>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
        else hipLaunchKernelGGL((bwd_dz_dstates_kernel<f16_t>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
    }
    return check_launch();
}

// The same with 16-byte accesses and one direction per workgroup (blockIdx.z = 2 b + dir); the loads of 8 chunks go out
// together, unconditionally (past the last chunk a valid chunk is read again and not used).  Needs P*N % 4 == 0 and
// 16-byte aligned tensors.
// ndir = 1: the forward recurrence only (blockIdx.z = b).
// T16 != void: the entering states go to the 16-bit copies (states16_*) and the per-chunk states stay as they are.
template <typename T16>
__global__ __launch_bounds__(NTHREADS) void state_passing_fwd_vec_kernel(const bimamba2_params p, int nc, int ndir) {
    const int PN = p.headdim * p.dstate;
    const int e = (blockIdx.x * NTHREADS + threadIdx.x) * 4;
    const int h = blockIdx.y, b = blockIdx.z / ndir, dir = blockIdx.z % ndir;
    if (e >= PN) return;
    const int Q = p.chunk_size;
    const float *cs = (dir == 0 ? p.cs_f : p.cs_b) + ((int64_t)b * p.nheads + h) * nc * Q + (dir == 0 ? Q - 1 : 0);
    const int64_t cstride = (int64_t)p.nheads * PN;
    float *st = (dir == 0 ? p.states_f : p.states_b) + ((int64_t)b * nc * p.nheads + h) * PN + e;
    constexpr bool COPY = !std::is_same<T16, void>::value;
    typedef typename std::conditional<COPY, T16, bf16_t>::type TC;
    struct alignas(8) Out4 { TC v[4]; };
    TC *st16 = reinterpret_cast<TC *>(dir == 0 ? p.states16_f : p.states16_b) + ((int64_t)b * nc * p.nheads + h) * PN + e;
    const float *ini = dir == 0 ? p.initial_f : p.initial_b;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    if (ini) s = *reinterpret_cast<const f32x4 *>(ini + ((int64_t)b * p.nheads + h) * PN + e);
    for (int s0 = 0; s0 < nc; s0 += 8) {
        f32x4 v[8];
        float d[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int si = min(s0 + i, nc - 1), c = dir == 0 ? si : nc - 1 - si;
            // (with the 16-bit copies the per-chunk states are read for the last time here: past the caches)
            v[i] = COPY ? __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(st + c * cstride)) : *reinterpret_cast<const f32x4 *>(st + c * cstride);
            d[i] = cs[(int64_t)c * Q];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (s0 + i < nc) {
                const int c = dir == 0 ? s0 + i : nc - 1 - (s0 + i);
                if constexpr (COPY) {
                    Out4 o;
#pragma unroll
                    for (int k = 0; k < 4; ++k) o.v[k] = from_f<TC>(s[k]);
                    *reinterpret_cast<Out4 *>(st16 + c * cstride) = o;
                } else {
                    *reinterpret_cast<f32x4 *>(st + c * cstride) = s;
                }
                s = __expf(d[i]) * s + v[i];
            }
    }
    float *fin = dir == 0 ? p.final_f : p.final_b;
    if (fin) *reinterpret_cast<f32x4 *>(fin + ((int64_t)b * p.nheads + h) * PN + e) = s;
}

// The same recurrences on per-chunk states that lie in states16_f/b in the 16-bit type (chunk_state_direct_kernel<.., OUT16>):
// every state is read once and replaced by the state entering its chunk; the running state stays in float32 registers.
// 8 elements (16 bytes) per thread, the loads of 8 chunks in flight.
template <typename T16>
__global__ __launch_bounds__(NTHREADS) void state_passing_fwd_inplace16_kernel(const bimamba2_params p, int nc) {
    const int PN = p.headdim * p.dstate;
    const int e = (blockIdx.x * NTHREADS + threadIdx.x) * 8;
    const int h = blockIdx.y, b = blockIdx.z >> 1, dir = blockIdx.z & 1;
    if (e >= PN) return;
    const int Q = p.chunk_size;
    const float *cs = (dir == 0 ? p.cs_f : p.cs_b) + ((int64_t)b * p.nheads + h) * nc * Q + (dir == 0 ? Q - 1 : 0);
    const int64_t cstride = (int64_t)p.nheads * PN;
    T16 *st = reinterpret_cast<T16 *>(dir == 0 ? p.states16_f : p.states16_b) + ((int64_t)b * nc * p.nheads + h) * PN + e;
    const float *ini = dir == 0 ? p.initial_f : p.initial_b;
    float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (ini) {
        const f32x4 a = *reinterpret_cast<const f32x4 *>(ini + ((int64_t)b * p.nheads + h) * PN + e);
        const f32x4 c4 = *reinterpret_cast<const f32x4 *>(ini + ((int64_t)b * p.nheads + h) * PN + e + 4);
#pragma unroll
        for (int k = 0; k < 4; ++k) { s[k] = a[k]; s[4 + k] = c4[k]; }
    }
    for (int s0 = 0; s0 < nc; s0 += 8) {
        Vec16<T16> v[8];
        float d[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int si = min(s0 + i, nc - 1), c = dir == 0 ? si : nc - 1 - si;
            v[i] = *reinterpret_cast<const Vec16<T16> *>(st + c * cstride);
            d[i] = cs[(int64_t)c * Q];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (s0 + i < nc) {
                const int c = dir == 0 ? s0 + i : nc - 1 - (s0 + i);
                Vec16<T16> o;
#pragma unroll
                for (int k = 0; k < 8; ++k) o.v[k] = from_f<T16>(s[k]);
                *reinterpret_cast<Vec16<T16> *>(st + c * cstride) = o;
                const float dec = __expf(d[i]);
#pragma unroll
                for (int k = 0; k < 8; ++k) s[k] = dec * s[k] + to_f(v[i].v[k]);
            }
    }
    float *fin = dir == 0 ? p.final_f : p.final_b;
    if (fin) {
        *reinterpret_cast<f32x4 *>(fin + ((int64_t)b * p.nheads + h) * PN + e) = f32x4{s[0], s[1], s[2], s[3]};
        *reinterpret_cast<f32x4 *>(fin + ((int64_t)b * p.nheads + h) * PN + e + 4) = f32x4{s[4], s[5], s[6], s[7]};
    }
}

int launch_state_passing_fwd(const bimamba2_params *p) {
    const int nc = nchunks(p), PN = p->headdim * p->dstate;
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    const int ndir = p->causal ? 1 : 2;
    if (!p->states_f) {
        // the per-chunk states lie in states16_f/b (16-bit): in place
        if (!p->states16_f || !p->states16_b || !chunk_states_in_16bit(p)) return BIMAMBA2_EINVAL;
        dim3 grid((PN / 8 + NTHREADS - 1) / NTHREADS, p->nheads, p->batch * 2);
        if (p->dtype == BIMAMBA2_BF16) hipLaunchKernelGGL(state_passing_fwd_inplace16_kernel<bf16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
        else hipLaunchKernelGGL(state_passing_fwd_inplace16_kernel<f16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
        return check_launch();
    }
    if (PN % 4 == 0 && al(p->states_f) && al(p->states_b) && al(p->final_f) && al(p->final_b) && al(p->initial_f) && al(p->initial_b)) {
        dim3 grid((PN / 4 + NTHREADS - 1) / NTHREADS, p->nheads, p->batch * ndir);
        if (p->states16_f) {
            if (!(p->causal || p->states16_b) || !al(p->states16_f) || !al(p->states16_b)) return BIMAMBA2_EINVAL;
            if (p->dtype == BIMAMBA2_BF16) hipLaunchKernelGGL(state_passing_fwd_vec_kernel<bf16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, ndir);
            else if (p->dtype == BIMAMBA2_F16) hipLaunchKernelGGL(state_passing_fwd_vec_kernel<f16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, ndir);
            else return BIMAMBA2_EUNSUPPORTED;
        } else {
            hipLaunchKernelGGL(state_passing_fwd_vec_kernel<void>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, ndir);
        }
        return check_launch();
    }
    if (p->states16_f) return BIMAMBA2_EUNSUPPORTED;
    if (p->causal) return BIMAMBA2_EUNSUPPORTED;
    dim3 grid((PN + NTHREADS - 1) / NTHREADS, p->nheads, p->batch);
    hipLaunchKernelGGL(state_passing_fwd_kernel, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
    return check_launch();
}

}  // namespace bm2
