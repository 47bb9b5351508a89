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
    float v[4], a[4];
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
        a[e] = d * A;
    }
    // forward inclusive scan
    float pf[4], sb[4];
    pf[0] = a[0]; pf[1] = pf[0] + a[1]; pf[2] = pf[1] + a[2]; pf[3] = pf[2] + a[3];
    sb[3] = a[3]; sb[2] = sb[3] + a[2]; sb[1] = sb[2] + a[1]; sb[0] = sb[1] + a[0];
    const float tot = pf[3];
    const float incl = wave_incl_prefix(tot, lane);
    const float before = incl - tot;
    const float incl_s = wave_incl_suffix(tot, lane);
    const float after = incl_s - tot;
    const int64_t o = (((int64_t)b * p.nheads + h) * nc + c) * Q;
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
template <typename T, bool DSTATES, bool CUMSUM, bool UNI = false>
__global__ __launch_bounds__(NTHREADS) void chunk_state_direct_kernel(const bimamba2_params p, int nc) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    static_assert(sizeof(T) == 2, "16-bit operands");
    __shared__ __attribute__((aligned(16))) T xt[BIMAMBA2_MAX_CHUNK * 64];
    __shared__ __attribute__((aligned(16))) T bt[BIMAMBA2_MAX_CHUNK * 64];
    __shared__ __attribute__((aligned(16))) float wf[BIMAMBA2_MAX_CHUNK], wb[BIMAMBA2_MAX_CHUNK];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    const int nt = blockIdx.x, pt = blockIdx.y;
    const int h = blockIdx.z % p.nheads, bc = blockIdx.z / p.nheads, c = bc % nc, b = bc / nc;
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
    const int rows = (limit + 31) & ~31;                   // K steps of 32 positions
    tile64_request(xt, xp + pt * 64, xs, rows, limit, wave, NTHREADS / 64, lane);
    tile64_request(bt, bp + nt * 64, bs, rows, limit, wave, NTHREADS / 64, lane);
    const int64_t o = (((int64_t)b * p.nheads + h) * nc + c) * Q;
    if constexpr (CUMSUM && !DSTATES) {
        __shared__ float dts[BIMAMBA2_MAX_CHUNK], csfs[BIMAMBA2_MAX_CHUNK], csbs[BIMAMBA2_MAX_CHUNK];
        if (wave == 0) {
            const float A = p.A[h];
            const float bias = p.has_dt_bias ? p.dt_bias[h] : 0.f;
            const int64_t dto = b * p.dt_sb + (int64_t)c * Q * p.dt_sl + h * p.dt_sh;
            float v[4], a[4], raw[4];
            int64_t at[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) at[e] = dto + (int64_t)min(lane * 4 + e, limit - 1) * p.dt_sl;
            // one branch on the type around all four loads, so that they go out together
            if (p.dt_dtype == BIMAMBA2_F32) {
#pragma unroll
                for (int e = 0; e < 4; ++e) raw[e] = reinterpret_cast<const float *>(p.dt)[at[e]];
            } else if (p.dt_dtype == BIMAMBA2_BF16) {
#pragma unroll
                for (int e = 0; e < 4; ++e) raw[e] = to_f(reinterpret_cast<const bf16_t *>(p.dt)[at[e]]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) raw[e] = to_f(reinterpret_cast<const f16_t *>(p.dt)[at[e]]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int q = lane * 4 + e;
                float d = raw[e] + bias;
                if (p.dt_softplus) d = d > 20.f ? d : log1pf(expf(d));
                d = fminf(fmaxf(d, p.dt_min), p.dt_max);
                if (q >= limit) d = 0.f;
                v[e] = d;
                a[e] = d * A;
            }
            float pf[4], sb[4];
            pf[0] = a[0]; pf[1] = pf[0] + a[1]; pf[2] = pf[1] + a[2]; pf[3] = pf[2] + a[3];
            sb[3] = a[3]; sb[2] = sb[3] + a[2]; sb[1] = sb[2] + a[1]; sb[0] = sb[1] + a[0];
            const float tot = pf[3];
            const float before = wave_incl_prefix(tot, lane) - tot, after = wave_incl_suffix(tot, lane) - tot;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int q = lane * 4 + e;
                dts[q] = v[e];
                csfs[q] = before + pf[e];
                csbs[q] = after + sb[e];
                if (q < Q && nt == 0 && pt == 0) {
                    p.dt_out[o + q] = v[e];
                    p.cs_f[o + q] = before + pf[e];
                    p.cs_b[o + q] = after + sb[e];
                }
            }
        }
        __syncthreads();
        for (int q = threadIdx.x; q < rows; q += NTHREADS) {
            wf[q] = q < limit ? __expf(csfs[Q - 1] - csfs[q]) * dts[q] : 0.f;
            wb[q] = q < limit ? __expf(csbs[0] - csbs[q]) * dts[q] : 0.f;
        }
    } else
    for (int q = threadIdx.x; q < rows; q += NTHREADS) {
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
    __syncthreads();       // (the compiler drains this wave's requests before its first LDS access; the barrier covers the rest)
    f32x4 accf[4] = {}, accb[4] = {};
    for (int k0 = 0; k0 < rows; k0 += 32) {
        const Frag a = tile64_tr_frag<Frag>(xt, k0, wave * 16, lr, lg);
        const f32x4 f0 = *reinterpret_cast<const f32x4 *>(wf + k0 + 8 * lg), f1 = *reinterpret_cast<const f32x4 *>(wf + k0 + 8 * lg + 4);
        const f32x4 r0 = *reinterpret_cast<const f32x4 *>(wb + k0 + 8 * lg), r1 = *reinterpret_cast<const f32x4 *>(wb + k0 + 8 * lg + 4);
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
            const Frag bfr = tile64_tr_frag<Frag>(bt, k0, j * 16, lr, lg);
            accf[j] = M::mma(af, bfr, accf[j]);
            if (!UNI) accb[j] = M::mma(ab, bfr, accb[j]);
        }
    }
    float *of = (DSTATES ? p.dstates_f : p.states_f) + (int64_t)blockIdx.z * P * N;
    float *ob = (DSTATES ? p.dstates_b : p.states_b) + (int64_t)blockIdx.z * P * N;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pp = pt * 64 + wave * 16 + lg * 4 + i, n = nt * 64 + j * 16 + lr;
            of[(int64_t)pp * N + n] = accf[j][i];
            if (!UNI) ob[(int64_t)pp * N + n] = accb[j][i];
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
    float s = 0.f;
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
    s = 0.f;
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
        if (fast && p->chunk_size % 32 == 0 && p->causal) {
            if (dstates) hipLaunchKernelGGL((chunk_state_direct_kernel<T, true, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else if (cumsum) hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, true, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
            else hipLaunchKernelGGL((chunk_state_direct_kernel<T, false, false, true>), grid, dim3(NTHREADS), 0, s, *p, nc);
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
    return p->dtype != BIMAMBA2_F32 && p->headdim % 64 == 0 && p->dstate % 64 == 0 && p->chunk_size % 32 == 0 && al(p->Bm) &&
           mult(p->B_sb, p->B_sl, p->B_sg) && al(p->x) && mult(p->x_sb, p->x_sl, p->x_sh);
}

// The same with 16-byte accesses and one direction per workgroup (blockIdx.z = 2 b + dir); the loads of 8 chunks go out
// together, unconditionally (past the last chunk a valid chunk is read again and not used).  Needs P*N % 4 == 0 and
// 16-byte aligned tensors.
// ndir = 1: the forward recurrence only (blockIdx.z = b).
__global__ __launch_bounds__(NTHREADS) void state_passing_fwd_vec_kernel(const bimamba2_params p, int nc, int ndir) {
    const int PN = p.headdim * p.dstate;
    const int e = (blockIdx.x * NTHREADS + threadIdx.x) * 4;
    const int h = blockIdx.y, b = blockIdx.z / ndir, dir = blockIdx.z % ndir;
    if (e >= PN) return;
    const int Q = p.chunk_size;
    const float *cs = (dir == 0 ? p.cs_f : p.cs_b) + ((int64_t)b * p.nheads + h) * nc * Q + (dir == 0 ? Q - 1 : 0);
    const int64_t cstride = (int64_t)p.nheads * PN;
    float *st = (dir == 0 ? p.states_f : p.states_b) + ((int64_t)b * nc * p.nheads + h) * PN + e;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < nc; s0 += 8) {
        f32x4 v[8];
        float d[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int si = min(s0 + i, nc - 1), c = dir == 0 ? si : nc - 1 - si;
            v[i] = *reinterpret_cast<const f32x4 *>(st + c * cstride);
            d[i] = cs[(int64_t)c * Q];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (s0 + i < nc) {
                const int c = dir == 0 ? s0 + i : nc - 1 - (s0 + i);
                *reinterpret_cast<f32x4 *>(st + c * cstride) = s;
                s = __expf(d[i]) * s + v[i];
            }
    }
    float *fin = dir == 0 ? p.final_f : p.final_b;
    if (fin) *reinterpret_cast<f32x4 *>(fin + ((int64_t)b * p.nheads + h) * PN + e) = s;
}

int launch_state_passing_fwd(const bimamba2_params *p) {
    const int nc = nchunks(p), PN = p->headdim * p->dstate;
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    const int ndir = p->causal ? 1 : 2;
    if (PN % 4 == 0 && al(p->states_f) && al(p->states_b) && al(p->final_f) && al(p->final_b)) {
        dim3 grid((PN / 4 + NTHREADS - 1) / NTHREADS, p->nheads, p->batch * ndir);
        hipLaunchKernelGGL(state_passing_fwd_vec_kernel, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, ndir);
        return check_launch();
    }
    if (p->causal) return BIMAMBA2_EUNSUPPORTED;
    dim3 grid((PN + NTHREADS - 1) / NTHREADS, p->nheads, p->batch);
    hipLaunchKernelGGL(state_passing_fwd_kernel, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc);
    return check_launch();
}

}  // namespace bm2
