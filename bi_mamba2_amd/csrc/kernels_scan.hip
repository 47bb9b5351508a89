// The chunk-scan kernel (forward output) and its mirror (dx in the backward pass) for gfx950.
//
// One workgroup (8 waves) owns one (batch, chunk, head) and a tile of up to 64 headdim columns; wave w owns the
// rows [w*16*QT, (w+1)*16*QT) of the chunk.  The K operand of the big product (x * dt, resp. dy) is staged ONCE,
// transposed, into LDS; the A operand (CB times the decay factors) is built directly in registers in the MFMA
// operand layout from float32 CB rows, so the main loop has no barrier and no LDS round trip for A.
//
//   forward (BWD = false), rows r = output positions t, k = source positions s:
//     acc[r,p] = e^{cs_f[r]} C_r.prev_f[p,:] + e^{cs_b[r]} C_r.prev_b[p,:]
//              + sum_k CB[r,k] m(r,k) dt[k] x[k,p],    m = e^{cs_f[r]-cs_f[k]} (k<r), e^{cs_b[r]-cs_b[k]} (k>r), 2 (k=r)
//     out_x = acc + D x[r,p];  out = out_x * silu(z)
//   mirror (BWD = true), rows r = input positions s, k = output positions t, CBT[r,k] = CB[k,r]:
//     acc[r,p] = e^{cs_f[Q-1]-cs_f[r]} B_r.dS_f[p,:] + e^{cs_b[0]-cs_b[r]} B_r.dS_b[p,:]
//              + sum_k CBT[r,k] m'(r,k) dy[k,p],       m' = e^{cs_f[k]-cs_f[r]} (k>r), e^{cs_b[k]-cs_b[r]} (k<r), 2 (k=r)
//     dx = acc dt[r] + D dy[r,p];  ddt_direct[r] = sum_p acc x[r,p];  dD partial = sum_r dy x
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace bm2 {

static inline int nchunks(const bimamba2_params *p) { return (p->seqlen + p->chunk_size - 1) / p->chunk_size; }
static inline hipStream_t stream_of(const bimamba2_params *p) { return reinterpret_cast<hipStream_t>(p->stream); }


constexpr int SCAN_WAVES = 8, SCAN_THREADS = 64 * SCAN_WAVES;

// FAST = true is chosen by the launcher when chunk_size % 32 == 0, headdim is a multiple of the column tile,
// dstate % 64 == 0 and every operand is 16-byte aligned with strides that keep rows aligned: all guarded scalar
// fallbacks compile away and loads become unconditional (rows past the end of the sequence are read from a valid
// row and never stored).
//
// NF > 0 (16-bit types, FAST, dstate = 32 * NF): CB is not read at all.  The 16 x 32 piece of CB (resp. CB^T) a wave needs
// for a K step is recomputed with MFMAs from the C and B rows, arranged so that the product comes out in the A operand
// layout: D[m][n] = sum_d Krow[k(m)][d] * Ownrow[n][d] with k(m) = k0 + 8*(m/4) + m%4 (+4 for the second product) leaves
// lane (l%16 = row, l/16 = g) with columns k0 + 8g + 0..3 (resp. +4..7) of its row.  All waves of a workgroup read the
// same 32 K rows per step, so they come from L1, where the CB rows were 256 KB of L2 traffic per workgroup.  The state
// products use the raw rows as well and scale the accumulator instead of the operand.
// UNI (with NF > 0 only): the single-direction (causal) operator - the reverse direction's state product, the K steps on
// the far side of the diagonal and the far half of the diagonal step are left out.
template <typename T, int QT, int NJ, bool BWD, bool FAST, int NF, bool UNI = false>
__global__ __launch_bounds__(SCAN_THREADS, 4) void chunk_scan_kernel(const bimamba2_params p, int nc, int npt) {
    typedef Mma<T> M;
    constexpr int KPL = M::KPL, KSTEP = M::KSTEP;
    constexpr int VS = 16 / (int)sizeof(T);
    constexpr int QP = SCAN_WAVES * 16 * QT;      // rows the workgroup covers (>= chunk_size); QT row tiles per wave
    constexpr int PW = 16 * NJ;                   // headdim columns the workgroup covers
    constexpr int LDX = QP + VS;
    constexpr int NW = 64;                        // dstate columns of the state tiles held in LDS at a time
    constexpr int LDS_ = M::LD - BK + NW;         // their leading dimension
    constexpr int SLD = PW + 4;                   // float32 row of the epilogue staging patches
    constexpr int XT_BYTES = PW * LDX * (int)sizeof(T), ST_BYTES = 2 * PW * LDS_ * (int)sizeof(T);
    constexpr int STG_BYTES = SCAN_WAVES * 16 * SLD * 4;
    // the operand images (xT and the two state tiles) and the per-wave epilogue staging patches are never live together
    __shared__ __attribute__((aligned(16))) char shared_u[XT_BYTES + ST_BYTES > STG_BYTES ? XT_BYTES + ST_BYTES : STG_BYTES];
    __shared__ float lo[QP], up[QP];              // decay exponents (times log2 e), see below
    __shared__ float glo[QP], gup[QP];            // their column factors relative to the edge of the 16-block, see below
    __shared__ float dtl[BWD ? 4 : QP];           // forward: dt of the columns, for the step across the diagonal
    __shared__ float red[SCAN_WAVES][PW];
    T *xT = reinterpret_cast<T *>(shared_u);
    T *sF = reinterpret_cast<T *>(shared_u + XT_BYTES), *sB = sF + PW * LDS_;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    // linear block id -> (pt, h, bc) with bc fastest: all heads of one (batch, chunk) share CB and C, and
    // consecutive ids are dealt round-robin to the 8 XCDs, so equal bc % 8 keeps them on one XCD's L2
    const int nbc = p.batch * nc;
    const int bc = blockIdx.x % nbc, hp = blockIdx.x / nbc, pt = hp % npt, h = hp / npt;
    const int c = bc % nc, b = bc / nc;
    const int g = h / (p.nheads / p.ngroups);
    const int Q = p.chunk_size, N = p.dstate, P = p.headdim, H = p.nheads;
    const int limit = min(Q, p.seqlen - c * Q);
    const int p0 = pt * PW;
    const int64_t o = (((int64_t)b * H + h) * nc + c) * Q;
    const float *csf = p.cs_f + o, *csb = p.cs_b + o, *dto = p.dt_out + o;
    const float d_head = (p.has_D && !p.D_has_hdim) ? p.D[h] : 0.f;   // read here: in the epilogue its latency would be exposed
    // NF > 0: the K rows of part 2 (forward: B rows, mirror: C rows) travel straight into a ring of LDS slots, KRING - 1
    // K steps (of 32 rows) ahead of their use: a global access takes microseconds when the memory system is busy.  Wave w brings rows 4w..4w+3 of the step: unit u = 32*w + lane (lane < 32) is row
    // u/8, chunk position u%8, which holds the row's 16-byte chunk (u%8) ^ (row % 8).
    constexpr int KRING = 4;                       // slots of the K-row image: requests run KRING - 1 steps ahead
    __shared__ __attribute__((aligned(16))) T krl[NF > 0 ? KRING * 32 * 64 : 8];
    const char *krbase = nullptr;                  // uniform: row 0 of the chunk in the K-row matrix
    unsigned krs_bytes = 0;                        // its row stride (the launcher checks that 256 rows fit 32 bits)
    if constexpr (NF > 0) {
        if (BWD) { krs_bytes = (unsigned)p.C_sl * sizeof(T); krbase = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * p.C_sl + g * p.C_sg); }
        else { krs_bytes = (unsigned)p.B_sl * sizeof(T); krbase = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * p.B_sl + g * p.B_sg); }
    }
    if constexpr (NF > 0) {
        // keep the base in scalar registers (it is uniform, but that is not visible through the 64-bit arithmetic)
        const uint64_t kb64 = reinterpret_cast<uint64_t>(krbase);
        const uint32_t klo = __builtin_amdgcn_readfirstlane((uint32_t)kb64), khi = __builtin_amdgcn_readfirstlane((uint32_t)(kb64 >> 32));
        krbase = reinterpret_cast<const char *>(((uint64_t)khi << 32) | klo);
    }
    auto kr_issue = [&](int step) {
        if (lane < 32) {
            int ln = lane;
            asm volatile("" : "+v"(ln));           // recompute the few lane terms per call rather than keep them in registers
            const int rowl = wave * 4 + (ln >> 3);
            const unsigned off = (unsigned)min(step * 32 + rowl, limit - 1) * krs_bytes + (((ln & 7) ^ (rowl & 7)) * 16);
            load16_to_lds(krbase + off, krl + (step % KRING) * (32 * 64) + wave * 256);
        }
    };
    if constexpr (NF > 0) {
#pragma unroll
        for (int st = 0; st < KRING - 1; ++st)
            if (st * 32 < limit) kr_issue(st);
    }
    int rowi[QT];                                  // this lane's A-operand row in each row tile
#pragma unroll
    for (int rt = 0; rt < QT; ++rt) rowi[rt] = (wave * QT + rt) * 16 + lr;

    // A operand of part 1: C rows (forward) or B rows (mirror), straight from global memory in operand layout
    const T *ap;
    int64_t as;
    if (BWD) { as = p.B_sl; ap = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * as + g * p.B_sg; }
    else { as = p.C_sl; ap = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * as + g * p.C_sg; }
    const bool avec = aligned16(ap, as) && (N % VS == 0);
    float arow[QT][NW / KSTEP][KPL];               // rows of the first NW dstate columns, requested up front
    auto load_arows = [&](int n0) {
#pragma unroll
        for (int rt = 0; rt < QT; ++rt)
#pragma unroll
            for (int s = 0; s < NW / KSTEP; ++s) {
                const int r = rowi[rt], kb = n0 + s * KSTEP + lg * KPL;
                if (FAST && KPL == 1) {
                    arow[rt][s][0] = to_f(ap[(int64_t)min(r, limit - 1) * as + kb]);
                } else if (KPL > 1 && (FAST || (r < limit && avec && kb + KPL <= N))) {
                    Vec16<T> raw = *reinterpret_cast<const Vec16<T> *>(ap + (int64_t)(FAST ? min(r, limit - 1) : r) * as + kb);
#pragma unroll
                    for (int i = 0; i < KPL; ++i) arow[rt][s][i] = to_f(raw.v[i % Vec16<T>::N]);
                } else {
#pragma unroll
                    for (int i = 0; i < KPL; ++i) arow[rt][s][i] = (r < limit && kb + i < N) ? to_f(ap[(int64_t)r * as + kb + i]) : 0.f;
                }
            }
    };

    // forward: k<r uses lo[r]-lo[k] with lo = cs_f, k>r uses up[r]-up[k] with up = cs_b
    // mirror : k<r uses e^{cs_b[k]-cs_b[r]} -> lo = -cs_b;  k>r uses e^{cs_f[k]-cs_f[r]} -> up = -cs_f
    // Away from the diagonal the factor separates: with m = lo at the last position of k's block of 16 (which lies
    // between k and r), 2^{lo[r]-lo[k]} = 2^{lo[r]-m} * glo[k], glo[k] = 2^{m-lo[k]}, both factors <= 1 for A <= 0;
    // likewise gup[k] = 2^{up[first of k's block] - up[k]}.  One exponential per lane and K step instead of one per element.
    for (int q = threadIdx.x; q < QP; q += SCAN_THREADS) {
        const int qq = min(q, Q - 1), qe = min(q | 15, Q - 1), qs = min(q & ~15, Q - 1);
        const float f = csf[qq] * LOG2E, r = csb[qq] * LOG2E;
        const float l = BWD ? -r : f, u = BWD ? -f : r;
        lo[q] = l;
        up[q] = u;
        // forward: dt[k] of the source position rides on the column factors (and on the diagonal step through dtl), so
        // that the operand image holds x as it is and the D term can take x from there
        const float dtq = BWD ? 1.f : dto[qq];
        glo[q] = __builtin_amdgcn_exp2f((BWD ? -csb[qe] : csf[qe]) * LOG2E - l) * dtq;
        gup[q] = __builtin_amdgcn_exp2f((BWD ? -csf[qs] : csb[qs]) * LOG2E - u) * dtq;
        if (!BWD) dtl[q] = dtq;
    }
    // K operand of part 2, transposed into LDS
    const T *kp;
    int64_t ks;
    if (!BWD) { ks = p.x_sl; kp = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * ks + h * p.x_sh; }
    else if (p.has_z) { ks = (int64_t)H * P; kp = reinterpret_cast<const T *>(p.dout_x) + ((int64_t)b * p.seqlen + (int64_t)c * Q) * ks + (int64_t)h * P; }
    else { ks = p.dout_sl; kp = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * ks + h * p.dout_sh; }
    stage_transposed<T, QP, PW, LDX, FAST>(xT, kp + p0, ks, limit, P - p0, [&](int k) { return k < limit ? 1.f : 0.f; });

    typename M::Frag own[QT][NF > 0 ? NF : 1];     // NF > 0: this lane's rows, 32 dstate columns per fragment
    if constexpr (NF > 0) {
#pragma unroll
        for (int rt = 0; rt < QT; ++rt)
#pragma unroll
            for (int f = 0; f < NF; ++f) own[rt][f] = M::load(ap + (int64_t)min(rowi[rt], limit - 1) * as + f * KSTEP + lg * KPL);
    } else {
        load_arows(0);
    }
    f32x4 acc[QT][NJ] = {};

    // ---- part 1: states.  A = (C or B rows) * row scale, K = dstate; B operand = state tiles [p][n] in LDS ----
    {
        const int64_t so = ((int64_t)(b * nc + c) * H + h) * P * N + (int64_t)p0 * N;
        const float *stf = (BWD ? p.dstates_f : p.states_f) + so, *stb = (BWD ? p.dstates_b : p.states_b) + so;
        float rsf[QT], rsb[QT];
#pragma unroll
        for (int rt = 0; rt < QT; ++rt) {
            const int r = rowi[rt];
            float ef = 0.f, eb = 0.f;
            if (r < limit) {
                ef = BWD ? __expf(csf[Q - 1] - csf[r]) : __expf(csf[r]);
                eb = BWD ? __expf(csb[0] - csb[r]) : __expf(csb[r]);
            }
            rsf[rt] = ef;
            rsb[rt] = eb;
        }
        if constexpr (NF > 0) {
            // raw rows as the A operand; the row factors go onto the accumulators (rows 4*(l/16)+i of each tile).
            // One direction after the other, to keep one set of temporaries.
            static_assert(NF == 0 || NF * KSTEP == NW, "one round of state tiles");
            // full 64 x 64 float tiles (the launcher checked it): every 16-byte load of both tiles goes out
            // before the first one is converted
            const T *s16f = reinterpret_cast<const T *>(BWD ? p.dstates16_f : p.states16_f);
            if (s16f) {
                // the 16-bit copies of the entering states: 64 x 64 elements per direction, 16 bytes per thread
                static_assert(PW * NW * (int)sizeof(T) == SCAN_THREADS * 16, "one 16-byte unit per thread and direction");
                const T *s16b = reinterpret_cast<const T *>(BWD ? p.dstates16_b : p.states16_b);
                const f32x4 rf = *reinterpret_cast<const f32x4 *>(s16f + so + threadIdx.x * VS);
                const f32x4 rb = UNI ? rf : *reinterpret_cast<const f32x4 *>(s16b + so + threadIdx.x * VS);
                const int r = threadIdx.x / (NW / VS), k0 = (threadIdx.x % (NW / VS)) * VS;
                *reinterpret_cast<f32x4 *>(sF + r * LDS_ + k0) = rf;
                *reinterpret_cast<f32x4 *>(sB + r * LDS_ + k0) = rb;
            } else {
                constexpr int PER = PW * NW / 4 / SCAN_THREADS;
                float4 rawf[PER], rawb[PER];
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    const int idx = threadIdx.x + i * SCAN_THREADS;
                    rawf[i] = *reinterpret_cast<const float4 *>(stf + idx * 4);
                    rawb[i] = UNI ? rawf[i] : *reinterpret_cast<const float4 *>(stb + idx * 4);
                }
                struct alignas(sizeof(T) * 4) Out { T v[4]; };
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    const int idx = threadIdx.x + i * SCAN_THREADS, r = idx / (NW / 4), k0 = (idx % (NW / 4)) * 4;
                    Out of, ob;
                    of.v[0] = from_f<T>(rawf[i].x); of.v[1] = from_f<T>(rawf[i].y); of.v[2] = from_f<T>(rawf[i].z); of.v[3] = from_f<T>(rawf[i].w);
                    ob.v[0] = from_f<T>(rawb[i].x); ob.v[1] = from_f<T>(rawb[i].y); ob.v[2] = from_f<T>(rawb[i].z); ob.v[3] = from_f<T>(rawb[i].w);
                    *reinterpret_cast<Out *>(sF + r * LDS_ + k0) = of;
                    *reinterpret_cast<Out *>(sB + r * LDS_ + k0) = ob;
                }
            }
            __syncthreads();
#pragma unroll
            for (int dir = 0; dir < (UNI ? 1 : 2); ++dir) {
                const T *st = dir ? sB : sF;
                f32x4 tmp[QT][NJ] = {};
#pragma unroll
                for (int s = 0; s < NW / KSTEP; ++s) {
                    typename M::Frag bfs[NJ];
#pragma unroll
                    for (int j = 0; j < NJ; ++j) bfs[j] = M::load(st + (j * 16 + lr) * LDS_ + s * KSTEP + lg * KPL);
#pragma unroll
                    for (int rt = 0; rt < QT; ++rt)
#pragma unroll
                        for (int j = 0; j < NJ; ++j) tmp[rt][j] = M::mma(own[rt][s], bfs[j], tmp[rt][j]);
                }
#pragma unroll
                for (int rt = 0; rt < QT; ++rt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int r = (wave * QT + rt) * 16 + lg * 4 + i, rc = min(r, limit - 1);
                        const float *cs = dir ? csb : csf;
                        float e = BWD ? __expf(cs[dir ? 0 : Q - 1] - cs[rc]) : __expf(cs[rc]);
                        if (r >= limit) e = 0.f;
#pragma unroll
                        for (int j = 0; j < NJ; ++j) acc[rt][j][i] = dir ? __builtin_fmaf(tmp[rt][j][i], e, acc[rt][j][i]) : tmp[rt][j][i] * e;
                    }
            }
        } else
        for (int n0 = 0; n0 < N; n0 += NW) {
            if (n0) {
                __syncthreads();
                load_arows(n0);
            }
            if (sizeof(T) == 2 && !BWD && p.states16_f) {
                // the 16-bit copies of the entering states (a forward pass whose caller keeps no states: half the bytes)
                tile_load_kcontig<T, T, PW, NW>(sF, reinterpret_cast<const T *>(p.states16_f) + so + n0, N, P - p0, N - n0, Ident());
                tile_load_kcontig<T, T, PW, NW>(sB, reinterpret_cast<const T *>(p.states16_b) + so + n0, N, P - p0, N - n0, Ident());
            } else {
                tile_load_kcontig<T, float, PW, NW>(sF, stf + n0, N, P - p0, N - n0, Ident());
                tile_load_kcontig<T, float, PW, NW>(sB, stb + n0, N, P - p0, N - n0, Ident());
            }
            __syncthreads();
#pragma unroll
            for (int s = 0; s < NW / KSTEP; ++s) {
                if (n0 + s * KSTEP >= N) break;
                const int kq = s * KSTEP + lg * KPL;
                typename M::Frag bff[NJ], bfb[NJ];
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    bff[j] = M::load(sF + (j * 16 + lr) * LDS_ + kq);
                    bfb[j] = M::load(sB + (j * 16 + lr) * LDS_ + kq);
                }
#pragma unroll
                for (int rt = 0; rt < QT; ++rt) {
                    float vf[KPL], vb[KPL];
#pragma unroll
                    for (int i = 0; i < KPL; ++i) { vf[i] = arow[rt][s][i] * rsf[rt]; vb[i] = arow[rt][s][i] * rsb[rt]; }
                    const typename M::Frag aff = M::pack(vf), afb = M::pack(vb);
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        acc[rt][j] = M::mma(aff, bff[j], acc[rt][j]);
                        acc[rt][j] = M::mma(afb, bfb[j], acc[rt][j]);
                    }
                }
            }
        }
    }

    // ---- epilogue operands (x and z, resp. x and dy) are requested one row tile ahead of their use ----
    constexpr int CPR = PW / VS;                   // 16-byte chunks per row
    constexpr int NPASS = (16 * CPR + 63) / 64;    // chunks per lane and row tile
    const T *xrow = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * p.x_sl + h * p.x_sh;
    const T *zrow = (!BWD && p.has_z) ? reinterpret_cast<const T *>(p.z) + b * p.z_sb + (int64_t)c * Q * p.z_sl + h * p.z_sh : nullptr;
    const bool need2 = BWD ? (bool)p.has_D : (bool)p.has_z;      // second operand: dy (for D) resp. z
    const T *row2 = BWD ? kp : zrow;
    const int64_t s2 = BWD ? ks : p.z_sl;
    const bool xvec = aligned16(xrow + p0, p.x_sl) && (P % VS == 0);
    const bool vec2 = need2 && aligned16(row2 + p0, s2) && (P % VS == 0);
    const bool ovec = (P % VS == 0);
    Vec16<T> ex[QT][NPASS], e2[QT][NPASS];         // kept as loaded; converted where they are used
    auto load_vec = [&](const T *ptr, bool vec, int ncol, Vec16<T> &v) {
        if (FAST || (vec && ncol >= VS)) {
            v = *reinterpret_cast<const Vec16<T> *>(ptr);
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i) v.v[i] = i < ncol ? ptr[i] : from_f<T>(0.f);
        }
    };
    // past_caches: a result that no kernel of the pass reads again (out, dx) leaves the caches to what is read again
    auto store_vec = [&](T *ptr, bool vec, int ncol, const float (&v)[VS], bool past_caches = false) {
        if (FAST || (vec && ncol >= VS)) {
            Vec16<T> ov;
#pragma unroll
            for (int i = 0; i < VS; ++i) ov.v[i] = from_f<T>(v[i]);
            if (past_caches) __builtin_nontemporal_store(__builtin_bit_cast(f32x4, ov), reinterpret_cast<f32x4 *>(ptr));
            else *reinterpret_cast<Vec16<T> *>(ptr) = ov;
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i)
                if (i < ncol) ptr[i] = from_f<T>(v[i]);
        }
    };
    auto epi_issue = [&](int rt) {
        const int B_ = rt;
        const int r0 = (wave * QT + rt) * 16;
#pragma unroll
        for (int ps = 0; ps < NPASS; ++ps) {
            const int id = lane + ps * 64;
            const int r = r0 + id / CPR, col = p0 + (id % CPR) * VS;
            const int ncol = (id < 16 * CPR && r < limit) ? P - col : 0;
            if (FAST && id >= 16 * CPR) continue;
            const int rc = min(r, limit - 1);
            if (BWD) load_vec(xrow + (int64_t)rc * p.x_sl + col, xvec, ncol, ex[B_][ps]);
            if (need2 && !BWD) load_vec(row2 + (int64_t)rc * s2 + col, vec2, ncol, e2[B_][ps]);
        }
    };
    typedef std::integral_constant<int, 0> B0;
    typedef std::integral_constant<int, 1> B1;
    // ---- part 2: inside the chunk.  A built in registers from CB (forward) or CB^T (mirror); the CB rows of
    // the next K step are requested before the current step is consumed (two register buffers) ----
    {
        const float *cb = (BWD ? p.CBT : p.CB) + ((int64_t)(b * nc + c) * p.ngroups + g) * Q * Q;
        const bool cvec = (Q % 4 == 0);
        float lor[QT], upr[QT];
        const float *rowp[QT];
#pragma unroll
        for (int rt = 0; rt < QT; ++rt) {
            lor[rt] = lo[rowi[rt]];
            upr[rt] = up[rowi[rt]];
            rowp[rt] = cb + (int64_t)min(rowi[rt], Q - 1) * Q;
        }
        float cbv[1][QT][KPL];
        auto issue = [&](auto BUF, int k0) {
            constexpr int B_ = decltype(BUF)::value;
            const int kb = k0 + lg * KPL;
#pragma unroll
            for (int rt = 0; rt < QT; ++rt) {
                if (FAST || (cvec && kb + KPL <= Q)) {
                    if (KPL >= 4) {
#pragma unroll
                        for (int i = 0; i < KPL; i += 4) {
                            const float4 t4 = *reinterpret_cast<const float4 *>(rowp[rt] + kb + i);
                            cbv[B_][rt][i] = t4.x; cbv[B_][rt][(i + 1) % KPL] = t4.y;
                            cbv[B_][rt][(i + 2) % KPL] = t4.z; cbv[B_][rt][(i + 3) % KPL] = t4.w;
                        }
                    } else {
                        cbv[B_][rt][0] = rowp[rt][kb];
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < KPL; ++i) cbv[B_][rt][i] = (kb + i < Q) ? rowp[rt][kb + i] : 0.f;
                }
            }
        };
        auto process = [&](auto BUF, int k0) {
            constexpr int B_ = decltype(BUF)::value;
            const int kb = k0 + lg * KPL;
            typename M::Frag bf[NJ];
#pragma unroll
            for (int j = 0; j < NJ; ++j) bf[j] = M::load(xT + xt_index<T, LDX>(j * 16 + lr, kb));
            // this lane's KPL columns lie in one block of 16
#pragma unroll
            for (int rt = 0; rt < QT; ++rt) {
                const int r = rowi[rt], r0 = (wave * QT + rt) * 16;
                float v[KPL];
                if (k0 + KSTEP - 1 < r0) {            // every k of this step is below every row of the tile
                    const float rf = __builtin_amdgcn_exp2f(lor[rt] - lo[kb | 15]);
#pragma unroll
                    for (int i = 0; i < KPL; ++i) v[i] = cbv[B_][rt][i] * rf * glo[kb + i];
                } else if (k0 > r0 + 15) {            // every k above every row
                    const float rf = __builtin_amdgcn_exp2f(upr[rt] - up[kb & ~15]);
#pragma unroll
                    for (int i = 0; i < KPL; ++i) v[i] = cbv[B_][rt][i] * rf * gup[kb + i];
                } else {
#pragma unroll
                    for (int i = 0; i < KPL; ++i) {
                        const int k = kb + i;
                        const float e = k < r ? lor[rt] - lo[k] : upr[rt] - up[k];
                        v[i] = cbv[B_][rt][i] * ((k == r) ? 2.f : __builtin_amdgcn_exp2f(e));
                        if (!BWD) v[i] *= dtl[min(k, QP - 1)];
                    }
                }
                const typename M::Frag af = M::pack(v);
#pragma unroll
                for (int j = 0; j < NJ; ++j) acc[rt][j] = M::mma(af, bf[j], acc[rt][j]);
            }
        };
        if constexpr (NF > 0) {
            static_assert(NF == 0 || (NF == 2 && KPL == 8 && KSTEP == 32), "K-row image: 32 rows of 64 elements per step");
            // fragment (hh, f): K row krow + 4*hh of the step, 16-byte chunk lg + 4*f, stored at chunk ^ (row % 8); with
            // krow % 8 = lr % 4 that is element kfb + 256*hh + 32*(f ^ hh) of the slot
            const int kfb = (8 * (lr >> 2) + (lr & 3)) * 64 + (lg ^ (lr & 3)) * 8;
            // x^T fragment j of step s (xt_index(16j + lr, 32s + 8lg)): lane part by the parity of j, the rest is uniform
            static_assert(NF == 0 || NJ == 4, "fragment addresses below are written out for four column tiles");
            const int xl0 = lr * LDX + 8 * (lg ^ (lr >> 3)), xl1 = lr * LDX + 8 * (lg ^ ((lr >> 3) + 2));
            // While requests are in flight every LDS access goes through the raw accessors (the compiler would make an
            // access it knows of wait for all of them), and the barrier is the bare instruction.
            const unsigned krl_a = lds_addr(krl) + kfb * 2, xt_a = lds_addr(xT);
            const unsigned lg32 = lg * 32;             // this lane's 8 columns inside a step of the float tables
            const int nsteps = (limit + KSTEP - 1) / KSTEP;
            typedef typename M::Frag Frag;
            for (int step = 0; step < nsteps; ++step) {
                const int k0 = step * KSTEP;
                // this wave's request for the step has landed: one request per step, up to KRING - 2 newer ones
                const int newer = min(KRING - 2, nsteps - 1 - step);
                if (newer >= 2) wait_vmcnt<2>();
                else if (newer == 1) wait_vmcnt<1>();
                else wait_vmcnt<0>();
                raw_lds_barrier();                     // ... and everybody else's; the slot of step - 1 is free again
                if (step + KRING - 1 < nsteps) kr_issue(step + KRING - 1);
                if (UNI && (BWD ? k0 + KSTEP - 1 < wave * QT * 16 : k0 > wave * QT * 16 + QT * 16 - 1)) continue;   // far side of the diagonal
                const unsigned slot = krl_a + (step % KRING) * (32 * 64 * 2);
                // the CB tiles of both row tiles first; the K fragments are dead after that
                f32x4 cb1[QT], cb2[QT];
                {
                    Frag kf00 = raw_lds_read_at<Frag, 0>(slot), kf01 = raw_lds_read_at<Frag, 64>(slot);
                    Frag kf10 = raw_lds_read_at<Frag, 512 + 64>(slot), kf11 = raw_lds_read_at<Frag, 512>(slot);
                    raw_lds_wait();
                    raw_lds_use(kf00); raw_lds_use(kf01); raw_lds_use(kf10); raw_lds_use(kf11);
#pragma unroll
                    for (int rt = 0; rt < QT; ++rt) {
                        cb1[rt] = M::mma(kf00, own[rt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                        cb2[rt] = M::mma(kf10, own[rt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                        cb1[rt] = M::mma(kf01, own[rt][1], cb1[rt]);
                        cb2[rt] = M::mma(kf11, own[rt][1], cb2[rt]);
                    }
                }
                // the wave's rows [wr0, wr0 + 16*QT) meet the step's columns [k0, k0 + 32) in one step only
                const int wr0 = wave * QT * 16;
                const int cls = (k0 + KSTEP - 1 < wr0) ? 0 : (k0 > wr0 + QT * 16 - 1) ? 1 : 2;   // below, above, across the diagonal
                const int kb = k0 + lg * KPL;
                // ---- A operands of both row tiles: CB times the decay factors
                Frag af[QT];
                if (cls != 2) {
                    const unsigned ta = lds_addr(cls == 0 ? glo : gup) + k0 * 4 + lg32;
                    f32x4 ga0 = raw_lds_read_at<f32x4, 0>(ta), ga1 = raw_lds_read_at<f32x4, 16>(ta);
                    float mref = raw_lds_read_at<float, 0>(cls == 0 ? lds_addr(lo) + (kb | 15) * 4 : lds_addr(up) + (kb & ~15) * 4);
                    raw_lds_wait();
                    raw_lds_use(ga0); raw_lds_use(ga1); raw_lds_use(mref);
#pragma unroll
                    for (int rt = 0; rt < QT; ++rt) {
                        const float rf = __builtin_amdgcn_exp2f((cls == 0 ? lor[rt] : upr[rt]) - mref);
                        float v[KPL];
#pragma unroll
                        for (int i = 0; i < 4; ++i) { v[i] = cb1[rt][i] * rf * ga0[i]; v[i + 4] = cb2[rt][i] * rf * ga1[i]; }
                        af[rt] = M::pack(v);
                    }
                } else {
                    // the one step across the diagonal: element by element
                    const unsigned la = lds_addr(lo) + k0 * 4 + lg32, ua = lds_addr(up) + k0 * 4 + lg32;
                    f32x4 l0 = raw_lds_read_at<f32x4, 0>(la), l1 = raw_lds_read_at<f32x4, 16>(la);
                    f32x4 u0 = raw_lds_read_at<f32x4, 0>(ua), u1 = raw_lds_read_at<f32x4, 16>(ua);
                    f32x4 d0 = {1.f, 1.f, 1.f, 1.f}, d1 = d0;
                    if (!BWD) {
                        const unsigned da = lds_addr(dtl) + k0 * 4 + lg32;
                        d0 = raw_lds_read_at<f32x4, 0>(da);
                        d1 = raw_lds_read_at<f32x4, 16>(da);
                    }
                    raw_lds_wait();
                    raw_lds_use(l0); raw_lds_use(l1); raw_lds_use(u0); raw_lds_use(u1);
                    if (!BWD) { raw_lds_use(d0); raw_lds_use(d1); }
#pragma unroll
                    for (int rt = 0; rt < QT; ++rt) {
                        const int r = (wave * QT + rt) * 16 + lr;
                        float v[KPL];
#pragma unroll
                        for (int i = 0; i < KPL; ++i) {
                            const int k = kb + i;
                            const float lk = i < 4 ? l0[i & 3] : l1[i & 3], uk = i < 4 ? u0[i & 3] : u1[i & 3];
                            const float e = k < r ? lor[rt] - lk : upr[rt] - uk;
                            float w = (k == r) ? (UNI ? 1.f : 2.f) : __builtin_amdgcn_exp2f(e);
                            if (UNI && (BWD ? k < r : k > r)) w = 0.f;
                            if (!BWD) w *= i < 4 ? d0[i & 3] : d1[i & 3];
                            v[i] = (i < 4 ? cb1[rt][i & 3] : cb2[rt][i & 3]) * w;
                        }
                        af[rt] = M::pack(v);
                    }
                }
                // ---- the x product, two column tiles at a time
                const unsigned xa = xt_a + 64 * step, xb = xt_a + 64 * (step ^ 1);
                {
                    Frag b0 = raw_lds_read_at<Frag, 0>(xa + 2 * xl0), b1 = raw_lds_read_at<Frag, 32 * LDX>(xa + 2 * xl1);
                    raw_lds_wait();
                    raw_lds_use(b0); raw_lds_use(b1);
#pragma unroll
                    for (int rt = 0; rt < QT; ++rt) {
                        acc[rt][0] = M::mma(af[rt], b0, acc[rt][0]);
                        acc[rt][1] = M::mma(af[rt], b1, acc[rt][1]);
                    }
                }
                {
                    Frag b2 = raw_lds_read_at<Frag, 64 * LDX>(xb + 2 * xl0), b3 = raw_lds_read_at<Frag, 96 * LDX>(xb + 2 * xl1);
                    raw_lds_wait();
                    raw_lds_use(b2); raw_lds_use(b3);
#pragma unroll
                    for (int rt = 0; rt < QT; ++rt) {
                        acc[rt][2] = M::mma(af[rt], b2, acc[rt][2]);
                        acc[rt][3] = M::mma(af[rt], b3, acc[rt][3]);
                    }
                }
            }
            wait_vmcnt<0>();
            __syncthreads();
        } else {
            for (int k0 = 0; k0 < limit; k0 += KSTEP) {
                issue(B0(), k0);
                process(B0(), k0);
            }
        }
    }

    // ---- epilogue.  Each wave passes its 16-row accumulator tiles through a private LDS patch so that out, out_x,
    // dx are written (and x, z, dy were read) as 16-byte vectors along headdim ----
    // the rows that the D term needs (forward: x, mirror: dy) lie in the operand image (transposed, unscaled; zero past the
    // end of the sequence and of headdim): they are read from there, elements a row of the image apart, before the image
    // becomes the staging area - and before the global requests below, which an LDS access known to the compiler would
    // wait for
    if (BWD ? need2 : (bool)p.has_D) {
#pragma unroll
        for (int rt = 0; rt < QT; ++rt) {
            if ((wave * QT + rt) * 16 < limit) {
#pragma unroll
                for (int ps = 0; ps < NPASS; ++ps) {
                    const int id = lane + ps * 64;
                    if (FAST && id >= 16 * CPR) continue;
                    const int r = (wave * QT + rt) * 16 + min(id / CPR, 15), cc = (id % CPR) * VS;
#pragma unroll
                    for (int i = 0; i < VS; ++i) (BWD ? e2 : ex)[rt][ps].v[i] = xT[xt_index<T, LDX>(cc + i, r)];
                }
            }
        }
    }
    // the epilogue operands of all row tiles are requested before the barrier
#pragma unroll
    for (int rt = 0; rt < QT; ++rt) {
        if ((wave * QT + rt) * 16 < limit) epi_issue(rt);
    }
    __syncthreads();   // every wave is done with xT: the operand images become the staging area
    float *stg = reinterpret_cast<float *>(shared_u) + wave * 16 * SLD;
    float dsum[VS];
#pragma unroll
    for (int i = 0; i < VS; ++i) dsum[i] = 0.f;
    auto epi_consume = [&](int rt) {
        const int B_ = rt;
        const int r0 = (wave * QT + rt) * 16;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) stg[(lg * 4 + i) * SLD + j * 16 + lr] = acc[rt][j][i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int ps = 0; ps < NPASS; ++ps) {
            const int id = lane + ps * 64;
            const int rl = id / CPR, cc = (id % CPR) * VS;
            const int r = r0 + rl, col = p0 + cc;
            const int ncol = P - col;              // valid columns from col on
            const bool ok = id < 16 * CPR && r < limit && ncol > 0;
            float a[VS];
#pragma unroll
            for (int i = 0; i < VS; i += 4) {
                const float4 t4 = *reinterpret_cast<const float4 *>(stg + (rl & 15) * SLD + cc + i);
                a[i] = t4.x; a[i + 1] = t4.y; a[i + 2] = t4.z; a[i + 3] = t4.w;
            }
            const int64_t orow = (((int64_t)b * p.seqlen + (int64_t)c * Q + r) * H + h) * P + col;
            float rsum = 0.f;
            if (ok) {
                if (!BWD) {
                    if (p.has_D) {
#pragma unroll
                        for (int i = 0; i < VS; ++i)
                            a[i] += (p.D_has_hdim ? (i < ncol ? p.D[h * P + col + i] : 0.f) : d_head) * to_f(ex[B_][ps].v[i]);
                    }
                    if (p.has_z) {
                        if (p.out_x) store_vec(reinterpret_cast<T *>(p.out_x) + orow, ovec, ncol, a);
#pragma unroll
                        for (int i = 0; i < VS; ++i) a[i] *= silu_f(to_f(e2[B_][ps].v[i]));
                    }
                    store_vec(reinterpret_cast<T *>(p.out) + orow, ovec, ncol, a, true);
                } else {
                    const float dtr = dto[r];
                    float dxv[VS];
#pragma unroll
                    for (int i = 0; i < VS; ++i) { rsum += a[i] * to_f(ex[B_][ps].v[i]); dxv[i] = a[i] * dtr; }
                    if (p.has_D) {
#pragma unroll
                        for (int i = 0; i < VS; ++i) {
                            dxv[i] += (p.D_has_hdim ? (i < ncol ? p.D[h * P + col + i] : 0.f) : d_head) * to_f(e2[B_][ps].v[i]);
                            dsum[i] += to_f(e2[B_][ps].v[i]) * to_f(ex[B_][ps].v[i]);
                        }
                    }
                    // (dx may be a slice of a wider buffer: its own position and batch strides)
                    const int64_t dxo = p.dx_sl ? b * p.dx_sb + ((int64_t)c * Q + r) * p.dx_sl + (int64_t)h * P + col : orow;
                    store_vec(reinterpret_cast<T *>(p.dx) + dxo, ovec && (p.dx_sl % VS == 0) && (p.dx_sb % VS == 0), ncol, dxv, true);
                }
            }
            if (BWD) {
                // the CPR lanes of a row sit next to each other: butterfly over them
#pragma unroll
                for (int d = 1; d < CPR; d <<= 1) rsum += __shfl_xor(rsum, d, 64);
                if (id < 16 * CPR && r < limit && (id % CPR) == 0) {
                    // (several headdim tiles share a row: each writes the plane of its tile, the reader adds them)
                    p.ddt_direct[(int64_t)pt * ((int64_t)p.batch * H * nc * Q) + o + r] = rsum;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
#pragma unroll
    for (int rt = 0; rt < QT; ++rt) {
        if ((wave * QT + rt) * 16 < limit) epi_consume(rt);
    }
    if (BWD && p.has_D) {
        // dsum[i]: this lane's share of column (lane % CPR)*VS + i; add the lanes that hold other rows
#pragma unroll
        for (int i = 0; i < VS; ++i) {
            float v = dsum[i];
#pragma unroll
            for (int d = CPR; d < 64; d <<= 1) v += __shfl_xor(v, d, 64);
            dsum[i] = v;
        }
        if (lane < CPR) {
#pragma unroll
            for (int i = 0; i < VS; ++i) red[wave][lane * VS + i] = dsum[i];
        }
        __syncthreads();
        if (threadIdx.x < PW && p0 + (int)threadIdx.x < P) {
            float v = 0.f;
#pragma unroll
            for (int wv = 0; wv < SCAN_WAVES; ++wv) v += red[wv][threadIdx.x];
            p.red[((int64_t)(b * nc + c) * H + h) * P + p0 + threadIdx.x] = v;   // partials [(b, c)][h][P]
        }
    }
}

static inline bool al16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

static inline int scan_col_tile(const bimamba2_params *p) {
    // headdim tile: the widest the LDS image allows (64 columns for 16-bit types, 32 for float32)
    return scan_col_tile_of(p->headdim, p->dtype);
}

// whether the kernels without guarded fallbacks apply (vs = elements per 16 bytes)
static bool scan_fast(const bimamba2_params *p, bool bwd, int pw, int vs) {
    auto mult = [vs](int64_t a, int64_t b, int64_t c) { return a % vs == 0 && b % vs == 0 && c % vs == 0; };
    bool fast = p->chunk_size % 32 == 0 && p->headdim % pw == 0 && p->dstate % 64 == 0 && al16(p->x) && mult(p->x_sb, p->x_sl, p->x_sh);
    if (bwd) {
        fast = fast && al16(p->Bm) && mult(p->B_sb, p->B_sl, p->B_sg) && al16(p->dx) && mult(p->dx_sb, p->dx_sl, 0);
        fast = fast && (p->has_z ? al16(p->dout_x) : (al16(p->dout) && mult(p->dout_sb, p->dout_sl, p->dout_sh)));
    } else {
        fast = fast && al16(p->Cm) && mult(p->C_sb, p->C_sl, p->C_sg) && al16(p->out);
        if (p->has_z) fast = fast && al16(p->z) && mult(p->z_sb, p->z_sl, p->z_sh) && (!p->out_x || al16(p->out_x));
    }
    return fast;
}

// the conditions of the kernels that rebuild C.B^T, apart from the state dimension
static bool scan_rebuild_shape(const bimamba2_params *p, bool bwd) {
    if (p->dtype == BIMAMBA2_F32 || scan_col_tile(p) != 64) return false;
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % 8 == 0 && b % 8 == 0 && c % 8 == 0; };
    if (p->B_sl <= 0 || p->C_sl <= 0 || p->B_sl > (1 << 21) || p->C_sl > (1 << 21)) return false;   // 256 rows in 32-bit byte offsets
    if (!(bwd ? al16(p->dstates_f) && al16(p->dstates_b) : al16(p->states_f) && al16(p->states_b))) return false;
    return scan_fast(p, bwd, 64, 8) && al16(p->Bm) && mult(p->B_sb, p->B_sl, p->B_sg) && al16(p->Cm) && mult(p->C_sb, p->C_sl, p->C_sg);
}

bool scan_recomputes_cb(const bimamba2_params *p, bool bwd) { return p->dstate == 64 && scan_rebuild_shape(p, bwd); }

bool chunk_scan_uses_scan16(const bimamba2_params *p, bool bwd) {
    // state dimension 64, or 128 in the forward kernel
    return scan_rebuild_shape(p, bwd) && (p->headdim == 64 || p->headdim == 128) && (p->dstate == 64 || (p->dstate == 128 && !bwd));
}

template <typename T, int NJMAX, bool BWD>
static int launch_scan_t(const bimamba2_params *p) {
    const int nc = nchunks(p);
    const int P = p->headdim, Q = p->chunk_size, N = p->dstate;
    constexpr int VS = 16 / (int)sizeof(T);
    const int pw = scan_col_tile(p);
    const int npt = (P + pw - 1) / pw;
    dim3 grid(p->batch * nc * p->nheads * npt);
    hipStream_t s = reinterpret_cast<hipStream_t>(p->stream);
    const bool fast = scan_fast(p, BWD, pw, VS);
#define BM2_SCAN(QTV, NJV)                                                                                                        \
    do {                                                                                                                          \
        if (fast) hipLaunchKernelGGL((chunk_scan_kernel<T, QTV, NJV, BWD, true, 0>), grid, dim3(SCAN_THREADS), 0, s, *p, nc, npt); \
        else hipLaunchKernelGGL((chunk_scan_kernel<T, QTV, NJV, BWD, false, 0>), grid, dim3(SCAN_THREADS), 0, s, *p, nc, npt);     \
    } while (0)
    const int qt = Q <= 128 ? 1 : 2;             // 16-row tiles per wave (8 waves)
    // 16-bit copies of the entering states: known to the kernels that rebuild CB only
    const void *c16f = BWD ? p->dstates16_f : p->states16_f, *c16b = BWD ? p->dstates16_b : p->states16_b;
    if (c16f && (!al16(c16f) || !al16(c16b) || !(p->causal || c16b))) return BIMAMBA2_EINVAL;
    if constexpr (sizeof(T) == 2 && NJMAX == 4) {
        // the shapes of the 16-bit kernel with transposed products and a raw operand tile: it needs the 16-bit copies of the
        // entering states (the composites keep them at these shapes) and no CB
        if (c16f && (BWD ? p->CBT : p->CB) == nullptr && chunk_scan_uses_scan16(p, BWD) && (p->causal || c16b))
            return launch_chunk_scan16(p, BWD);
        if (p->causal) {                                // single-direction comparator: the fused kernels only
            if (!scan_recomputes_cb(p, BWD)) return BIMAMBA2_EUNSUPPORTED;
            if (qt == 1) hipLaunchKernelGGL((chunk_scan_kernel<T, 1, 4, BWD, true, 2, true>), grid, dim3(SCAN_THREADS), 0, s, *p, nc, npt);
            else hipLaunchKernelGGL((chunk_scan_kernel<T, 2, 4, BWD, true, 2, true>), grid, dim3(SCAN_THREADS), 0, s, *p, nc, npt);
            return check_launch();
        }
        if ((BWD ? p->CBT : p->CB) == nullptr) {
            if (!scan_recomputes_cb(p, BWD)) return BIMAMBA2_EINVAL;   // (the kernels below rebuild C.B^T at state dimension 64 only)
            if (qt == 1) hipLaunchKernelGGL((chunk_scan_kernel<T, 1, 4, BWD, true, 2>), grid, dim3(SCAN_THREADS), 0, s, *p, nc, npt);
            else hipLaunchKernelGGL((chunk_scan_kernel<T, 2, 4, BWD, true, 2>), grid, dim3(SCAN_THREADS), 0, s, *p, nc, npt);
            return check_launch();
        }
    }
    // (the kernels below read the forward pass's 16-bit copies of the entering states too, but not the mirror's)
    if (p->causal || (c16f && (BWD || sizeof(T) != 2))) return BIMAMBA2_EUNSUPPORTED;
    if ((BWD ? p->CBT : p->CB) == nullptr) return BIMAMBA2_EINVAL;
    if (pw == 16) { if (qt == 1) BM2_SCAN(1, 1); else BM2_SCAN(2, 1); }
    else if (pw == 32) { if (qt == 1) BM2_SCAN(1, 2); else BM2_SCAN(2, 2); }
    else { if (qt == 1) BM2_SCAN(1, NJMAX); else BM2_SCAN(2, NJMAX); }
#undef BM2_SCAN
    return check_launch();
}

int launch_chunk_scan(const bimamba2_params *p, bool bwd) {
    switch (p->dtype) {
        case BIMAMBA2_F32: return bwd ? launch_scan_t<float, 2, true>(p) : launch_scan_t<float, 2, false>(p);
        case BIMAMBA2_BF16: return bwd ? launch_scan_t<bf16_t, 4, true>(p) : launch_scan_t<bf16_t, 4, false>(p);
        case BIMAMBA2_F16: return bwd ? launch_scan_t<f16_t, 4, true>(p) : launch_scan_t<f16_t, 4, false>(p);
        default: return BIMAMBA2_EUNSUPPORTED;
    }
}

}  // namespace bm2
