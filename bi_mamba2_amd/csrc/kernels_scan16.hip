// The chunk-scan kernel (forward output) and its mirror (dx in the backward pass) for 16-bit inputs on gfx950, for the
// shapes every BASELINE configuration with dstate 64 has: headdim a multiple of 64, dstate 64, chunk_size a multiple of 32,
// 16-byte aligned operands, the states entering the chunks kept in their 16-bit copies.
//
// The math is that of chunk_scan_kernel (kernels_scan.hip); what differs is how little of the work is vector ALU work,
// which is what bounds that kernel (counters: VALU busy 53 % of its duration, MFMA 19 %, LDS 29 %):
//  * the K operand of the big product (x, resp. dy: 256 x 64 elements) goes from global memory straight into LDS as it
//    lies in memory (direct loads, no registers, no staging code) and its MFMA fragments are LDS transpose reads;
//  * the products are computed transposed, D[p][r] = sum_k X[k][p] A[r][k]: operand fragments are the same registers as
//    for D[r][p] with the two MFMA operands swapped, but a lane then holds four consecutive headdim columns of ONE row
//    per 16-column tile.  Which headdim column an MFMA row stands for is free (it is decided where the operand
//    fragments are read), and is chosen so that the tiles 2t and 2t + 1 together give a lane EIGHT consecutive columns,
//    32 t + 8 (lane / 16) ..: out / out_x / dx leave as 16-byte stores and x / z / dy arrive as 16-byte loads without the
//    accumulators passing through LDS, and the per-row factors are one value per lane;
//  * the D term's rows are 16-byte LDS reads of the raw tile;
//  * the state tiles arrive by direct loads as well; one barrier in front of the K loop, none behind it (waves leave the
//    loop and write their rows independently);
//  * the K loop is unrolled over its (at most 8) steps, so ring slots, table offsets and fragment offsets are immediates.
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

namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr int S16_WAVES = 8, S16_THREADS = 64 * S16_WAVES;
constexpr int S16_KRING = 4;                       // slots of the K-row ring: requests run three K steps ahead

// byte offset of the four elements (r, n .. n + 3), n a multiple of 4, in a raw [rows][64] 16-bit tile whose 16-byte chunks
// are swizzled by tile64_swz (the layout tile64_request leaves)
__device__ __forceinline__ int tile64_row_offset(int r, int n) {
    return r * 128 + ((((n >> 3) ^ tile64_swz(r)) << 4) | ((n & 4) << 1));
}

// headdim column (inside the workgroup's 64) that row m of the 16-row MFMA tile j stands for: 32 (j/2) + 8 (m/4) + 4 (j%2) + m%4.
// Output rows m = 4 g + i of lane group g are then the columns 32 t + 8 g + i (tile 2t) and 32 t + 8 g + 4 + i (tile 2t + 1).
__device__ __forceinline__ int s16_col(int j, int m) { return 32 * (j >> 1) + 8 * (m >> 2) + 4 * (j & 1) + (m & 3); }

// f(integral_constant<int, I>) for I = 0 .. N - 1, until it returns false: a loop whose index is a constant expression inside
// the body (LDS offsets become immediates)
template <int I, int N, class F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        if (f(std::integral_constant<int, I>())) static_for<I + 1, N>(f);
    }
}

}  // namespace

// QT: 16-row tiles per wave (8 waves: the workgroup covers 128 * QT rows >= chunk_size).  UNI: the single-direction
// (causal) operator: the reverse direction's state product, the K steps on the far side of the diagonal and the far half of
// the diagonal step are left out.
template <typename T, int QT, bool BWD, bool UNI>
__global__ __launch_bounds__(S16_THREADS, 4) void chunk_scan16_kernel(const bimamba2_params p, int nc, int npt) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    static_assert(sizeof(T) == 2, "16-bit operands");
    constexpr int KSTEP = 32;
    constexpr int QP = S16_WAVES * 16 * QT;        // rows the workgroup covers
    constexpr int NSTEP = QP / KSTEP;              // K steps at most
    __shared__ __attribute__((aligned(16))) T xr[QP * 64];                     // raw K-operand tile (x, resp. dy), swizzled
    __shared__ __attribute__((aligned(16))) T krl[S16_KRING * 32 * 64];        // ring of K rows (B, resp. C) for the CB tiles
    __shared__ __attribute__((aligned(16))) T sF[64 * 64], sB[UNI ? 8 : 64 * 64];   // state tiles [p][n], 16-byte chunks ^ (p % 8)
    __shared__ float lo[QP], up[QP];               // decay exponents (times log2 e), see below
    __shared__ float glo[QP], gup[QP];             // their column factors relative to the edge of the 16-block
    __shared__ float dtl[QP];                      // forward: dt of the columns; mirror: 1 inside the sequence, 0 behind it
    __shared__ float red[BWD ? S16_WAVES : 1][64];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    // linear block id -> (pt, h, bc) with bc fastest: consecutive ids are dealt round-robin to the 8 XCDs, so all heads of
    // one (batch, chunk), which share the B and C rows, stay on one XCD's L2
    const int nbc = p.batch * nc;
    const int bc = blockIdx.x % nbc, hp = blockIdx.x / nbc, pt = hp % npt, h = hp / npt;
    const int c = bc % nc, b = bc / nc;
    const int g = h / (p.nheads / p.ngroups);
    const int Q = p.chunk_size, P = p.headdim, H = p.nheads;
    const int limit = min(Q, p.seqlen - c * Q);
    const int nsteps = (limit + KSTEP - 1) / KSTEP;
    const int p0 = pt * 64;
    const int64_t o = (((int64_t)b * H + h) * nc + c) * Q;
    const float *csf = p.cs_f + o, *csb = p.cs_b + o, *dto = p.dt_out + o;
    const float d_head = (p.has_D && !p.D_has_hdim) ? p.D[h] : 0.f;

    // ---- every request of the prologue goes out before anything is waited for ----
    // K rows of the first ring slots: wave w brings rows 4w..4w+3 of a step; unit u = 32*w + lane (lane < 32) is row u/8,
    // chunk position u%8, which holds the row's 16-byte chunk (u%8) ^ (row % 8)
    const char *krbase;
    unsigned krs_bytes;
    if (BWD) { krs_bytes = (unsigned)p.C_sl * sizeof(T); krbase = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * p.C_sl + g * p.C_sg); }
    else { krs_bytes = (unsigned)p.B_sl * sizeof(T); krbase = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * p.B_sl + g * p.B_sg); }
    {
        const uint64_t kb64 = reinterpret_cast<uint64_t>(krbase);
        const uint32_t klo = __builtin_amdgcn_readfirstlane((uint32_t)kb64), khi = __builtin_amdgcn_readfirstlane((uint32_t)(kb64 >> 32));
        krbase = reinterpret_cast<const char *>(((uint64_t)khi << 32) | klo);
    }
    const int kr_row = wave * 4 + ((lane & 31) >> 3);                           // this lane's row inside a step
    const unsigned kr_col = (((lane & 7) ^ (kr_row & 7)) * 16);
    auto kr_issue = [&](int step) {
        if (lane < 32) {
            const unsigned off = (unsigned)min(step * 32 + kr_row, limit - 1) * krs_bytes + kr_col;
            load16_to_lds(krbase + off, krl + (step % S16_KRING) * (32 * 64) + wave * 256);
        }
    };
#pragma unroll
    for (int st = 0; st < S16_KRING - 1; ++st)
        if (st < nsteps) kr_issue(st);
    // the K operand of the big product, as it lies in memory
    const T *kp;
    int64_t ks;
    if (!BWD) { ks = p.x_sl; kp = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * ks + h * p.x_sh; }
    else if (p.has_z) { ks = (int64_t)H * P; kp = reinterpret_cast<const T *>(p.dout_x) + ((int64_t)b * p.seqlen + (int64_t)c * Q) * ks + (int64_t)h * P; }
    else { ks = p.dout_sl; kp = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * ks + h * p.dout_sh; }
    tile64_request(xr, kp + p0, ks, nsteps * KSTEP, limit, wave, S16_WAVES, lane);
    // the two state tiles: thread t brings row t/8, chunk position t%8 <- chunk (t%8) ^ (row%8)
    {
        const int64_t so = ((int64_t)(b * nc + c) * H + h) * P * 64 + (int64_t)p0 * 64;
        const int row = threadIdx.x >> 3, ch = (threadIdx.x & 7) ^ (row & 7);
        const T *s16f = reinterpret_cast<const T *>(BWD ? p.dstates16_f : p.states16_f) + so + row * 64 + ch * 8;
        load16_to_lds(s16f, sF + wave * 512);
        if (!UNI) {
            const T *s16b = reinterpret_cast<const T *>(BWD ? p.dstates16_b : p.states16_b) + so + row * 64 + ch * 8;
            load16_to_lds(s16b, sB + wave * 512);
        }
    }
    // this lane's rows of the other matrix (forward: C, mirror: B) in operand layout: rows wr0 + 16 rt + lr
    const int wr0 = wave * 16 * QT;
    const T *ap;
    int64_t as;
    if (BWD) { as = p.B_sl; ap = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * as + g * p.B_sg; }
    else { as = p.C_sl; ap = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * as + g * p.C_sg; }
    Frag own[QT][2];
#pragma unroll
    for (int rt = 0; rt < QT; ++rt)
#pragma unroll
        for (int f = 0; f < 2; ++f) own[rt][f] = M::load(ap + (int64_t)min(wr0 + rt * 16 + lr, limit - 1) * as + f * KSTEP + lg * 8);
    // forward: k<r uses lo[r]-lo[k] with lo = cs_f, k>r uses up[r]-up[k] with up = cs_b
    // mirror : k<r uses e^{cs_b[k]-cs_b[r]} -> lo = -cs_b;  k>r uses e^{cs_f[k]-cs_f[r]} -> up = -cs_f
    // Away from the diagonal the factor separates: with m = lo at the last position of k's block of 16 (which lies
    // between k and r), 2^{lo[r]-lo[k]} = 2^{lo[r]-m} * glo[k], glo[k] = 2^{m-lo[k]}, both factors <= 1 for A <= 0;
    // likewise gup[k] = 2^{up[first of k's block] - up[k]}.  The column factors also carry dt[k] (forward) and the zero
    // of the rows behind the end of the sequence, which the raw tile holds as copies of its last row.
    for (int q = threadIdx.x; q < QP; q += S16_THREADS) {
        const int qq = min(q, Q - 1), qe = min(q | 15, Q - 1), qs = min(q & ~15, Q - 1);
        const float f = csf[qq] * LOG2E, r = csb[qq] * LOG2E;
        const float fe = (BWD ? -csb[qe] : csf[qe]) * LOG2E, rs = (BWD ? -csf[qs] : csb[qs]) * LOG2E;
        const float dtq = q < limit ? (BWD ? 1.f : dto[qq]) : 0.f;
        const float l = BWD ? -r : f, u = BWD ? -f : r;
        lo[q] = l;
        up[q] = u;
        glo[q] = __builtin_amdgcn_exp2f(fe - l) * dtq;
        gup[q] = __builtin_amdgcn_exp2f(rs - u) * dtq;
        dtl[q] = dtq;
    }
    const float e_f = BWD ? csf[Q - 1] * LOG2E : 0.f, e_b = BWD ? csb[0] * LOG2E : 0.f;   // mirror: the far ends of the chunk
    wait_vmcnt<0>();
    __syncthreads();

    // ---- part 1: states.  D[p][r] = sum_n S[p][n] Own[r][n], scaled by this lane's row factor, one direction after the other
    f32x4 acc[QT][4];
    float lor[QT], upr[QT];
#pragma unroll
    for (int rt = 0; rt < QT; ++rt) {
        lor[rt] = lo[wr0 + rt * 16 + lr];
        upr[rt] = up[wr0 + rt * 16 + lr];
    }
#pragma unroll
    for (int dir = 0; dir < (UNI ? 1 : 2); ++dir) {
        const T *st = dir ? sB : sF;
        f32x4 tmp[QT][4] = {};
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            Frag sf[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int pr = s16_col(j, lr);     // the state row (headdim column) this lane's MFMA row stands for
                sf[j] = M::load(st + pr * 64 + (((s * 4 + lg) ^ (pr & 7)) << 3));
            }
#pragma unroll
            for (int rt = 0; rt < QT; ++rt)
#pragma unroll
                for (int j = 0; j < 4; ++j) tmp[rt][j] = M::mma(sf[j], own[rt][s], tmp[rt][j]);
        }
#pragma unroll
        for (int rt = 0; rt < QT; ++rt) {
            // forward: e^{cs_f[r]} = 2^{lo[r]}, e^{cs_b[r]} = 2^{up[r]}; mirror: e^{cs_f[Q-1]-cs_f[r]} = 2^{e_f+up[r]}, e^{cs_b[0]-cs_b[r]} = 2^{e_b+lo[r]}
            const float e = __builtin_amdgcn_exp2f(BWD ? (dir ? e_b + lor[rt] : e_f + upr[rt]) : (dir ? upr[rt] : lor[rt]));
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[rt][j] = dir ? tmp[rt][j] * e + acc[rt][j] : tmp[rt][j] * e;
        }
    }

    // ---- part 2: inside the chunk.  Per K step of 32 columns: the CB (resp. CB^T) tiles of this wave's rows from its own
    // rows and the step's K rows (arranged so that the product comes out in operand layout: D[m][n] = sum_d Krow[k(m)][d]
    // Own[n][d] with k(m) = k0 + 8*(m/4) + m%4 leaves lane (l%16 = row, l/16 = g) with columns k0 + 8g + 0..3, the second
    // product with +4), times the decay factors, times the K operand.
    {
        // fragment (hh, f): K row krow + 4*hh of the step, 16-byte chunk lg + 4*f, stored at chunk ^ (row % 8); with
        // krow % 8 = lr % 4 that is element kfb + 256*hh + 32*(f ^ hh) of the slot
        const int kfb = (8 * (lr >> 2) + (lr & 3)) * 64 + (lg ^ (lr & 3)) * 8;
        const unsigned krl_a = lds_addr(krl) + kfb * 2;
        // K-operand fragments: LDS transpose reads of the raw tile, rows k0 + 8 lg + lr/4 (+4); source lane s of a 16-lane group
        // supplies the four columns s16_col(j, 4 (s%4)) .., which lanes 4 (s%4) .. + 3 of the group receive
        // (rows k + 4: the swizzle flips bit 2 of the chunk position, i.e. byte bit 6, and the row adds 512 bytes)
        unsigned xo_lo[4];
        {
            const int kk = 8 * lg + (lr >> 2);
#pragma unroll
            for (int j = 0; j < 4; ++j) xo_lo[j] = lds_addr(xr) + tile64_tr_offset(kk, s16_col(j, 4 * (lr & 3)));
        }
        const unsigned lg32 = lg * 32;             // this lane's 8 columns inside a step of the float tables
        const unsigned glo_a = lds_addr(glo) + lg32, gup_a = lds_addr(gup) + lg32, lo_a = lds_addr(lo) + lg32, up_a = lds_addr(up) + lg32;
        const unsigned dtl_a = lds_addr(dtl) + lg32;
        // reference points of the column factors: lo at the last, up at the first position of this lane's block of 16
        const unsigned mlo_a = lds_addr(lo) + ((lg * 8) | 15) * 4, mup_a = lds_addr(up) + ((lg * 8) & ~15) * 4;
        auto k_step = [&](auto STEP) __attribute__((always_inline)) -> bool {
            constexpr int step = decltype(STEP)::value;
            if (step >= nsteps) return false;
            constexpr int k0 = step * KSTEP;
            // this wave's request for the step has landed: one request per step, up to KRING - 2 newer ones
            const int newer = min(S16_KRING - 2, nsteps - 1 - step);
            if (newer >= 2) wait_vmcnt<2>();
            else if (newer == 1) wait_vmcnt<1>();
            else wait_vmcnt<0>();
            raw_lds_barrier();                     // ... and everybody else's; the slot of step - 1 is free again
            if (step + S16_KRING - 1 < nsteps) kr_issue(step + S16_KRING - 1);
            // the wave's rows [wr0, wr0 + 16*QT) meet the step's columns [k0, k0 + 32) in one step only
            const int cls = (k0 + KSTEP - 1 < wr0) ? 0 : (k0 > wr0 + QT * 16 - 1) ? 1 : 2;   // below, above, across the diagonal
            if (UNI && cls == (BWD ? 0 : 1)) return true;                                      // far side of the diagonal
            constexpr int SLOT = (step % S16_KRING) * (32 * 64 * 2);
            f32x4 cb1[QT], cb2[QT];
            {
                Frag kf00 = raw_lds_read_at<Frag, SLOT>(krl_a), kf01 = raw_lds_read_at<Frag, SLOT + 64>(krl_a);
                Frag kf10 = raw_lds_read_at<Frag, SLOT + 512 + 64>(krl_a), kf11 = raw_lds_read_at<Frag, SLOT + 512>(krl_a);
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
            const int kb = k0 + lg * 8;
            constexpr int TB = step * (KSTEP * 4);     // byte offset of the step inside the float tables
            Frag af[QT];
            if (cls != 2) {
                const unsigned ta = cls == 0 ? glo_a : gup_a;
                f32x4 ga0 = raw_lds_read_at<f32x4, TB>(ta), ga1 = raw_lds_read_at<f32x4, TB + 16>(ta);
                float mref = raw_lds_read_at<float, TB>(cls == 0 ? mlo_a : mup_a);
                raw_lds_wait();
                raw_lds_use(ga0); raw_lds_use(ga1); raw_lds_use(mref);
#pragma unroll
                for (int rt = 0; rt < QT; ++rt) {
                    const float rf = __builtin_amdgcn_exp2f((cls == 0 ? lor[rt] : upr[rt]) - mref);
                    float v[8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) { v[i] = cb1[rt][i] * rf * ga0[i]; v[i + 4] = cb2[rt][i] * rf * ga1[i]; }
                    af[rt] = M::pack(v);
                }
            } else {
                // the one step across the diagonal: element by element
                f32x4 l0 = raw_lds_read_at<f32x4, TB>(lo_a), l1 = raw_lds_read_at<f32x4, TB + 16>(lo_a);
                f32x4 u0 = raw_lds_read_at<f32x4, TB>(up_a), u1 = raw_lds_read_at<f32x4, TB + 16>(up_a);
                f32x4 d0 = raw_lds_read_at<f32x4, TB>(dtl_a), d1 = raw_lds_read_at<f32x4, TB + 16>(dtl_a);
                raw_lds_wait();
                raw_lds_use(l0); raw_lds_use(l1); raw_lds_use(u0); raw_lds_use(u1); raw_lds_use(d0); raw_lds_use(d1);
#pragma unroll
                for (int rt = 0; rt < QT; ++rt) {
                    const int r = wr0 + rt * 16 + lr;
                    float v[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int k = kb + i;
                        const float lk = i < 4 ? l0[i & 3] : l1[i & 3], uk = i < 4 ? u0[i & 3] : u1[i & 3];
                        const float e = k < r ? lor[rt] - lk : upr[rt] - uk;
                        float w = (k == r) ? (UNI ? 1.f : 2.f) : __builtin_amdgcn_exp2f(e);
                        if (UNI && (BWD ? k < r : k > r)) w = 0.f;
                        w *= i < 4 ? d0[i & 3] : d1[i & 3];
                        v[i] = (i < 4 ? cb1[rt][i & 3] : cb2[rt][i & 3]) * w;
                    }
                    af[rt] = M::pack(v);
                }
            }
            // ---- the product with the K operand, transposed: D[p][r] += X[k][p] A[r][k]; two column tiles at a time
            constexpr int XS = step * (KSTEP * 128);
#pragma unroll
            for (int jj = 0; jj < 4; jj += 2) {
                const i16x4 a0 = raw_lds_tr16_read_at<XS>(xo_lo[jj]), a1 = raw_lds_tr16_read_at<XS + 512>(xo_lo[jj] ^ 64u);
                const i16x4 b0 = raw_lds_tr16_read_at<XS>(xo_lo[jj + 1]), b1 = raw_lds_tr16_read_at<XS + 512>(xo_lo[jj + 1] ^ 64u);
                raw_lds_wait();
                i16x8 fa = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7), fb = __builtin_shufflevector(b0, b1, 0, 1, 2, 3, 4, 5, 6, 7);
                raw_lds_use(fa); raw_lds_use(fb);
                const Frag xa = __builtin_bit_cast(Frag, fa), xb = __builtin_bit_cast(Frag, fb);
#pragma unroll
                for (int rt = 0; rt < QT; ++rt) {
                    acc[rt][jj] = M::mma(xa, af[rt], acc[rt][jj]);
                    acc[rt][jj + 1] = M::mma(xb, af[rt], acc[rt][jj + 1]);
                }
            }
            return true;
        };
        static_for<0, NSTEP>(k_step);
        wait_vmcnt<0>();
    }

    // ---- epilogue.  acc[rt][2t][i], acc[rt][2t+1][i] = row wr0 + 16 rt + lr, headdim columns p0 + 32 t + 8 lg + i, + 4 + i ----
    const int cq = 8 * lg;                         // first of this lane's eight columns inside a 32-column half
    const bool need_d = p.has_D;
    // operands of all row tiles first (the D term's rows - forward: x, mirror: dy - from the raw tile; z resp. x from memory)
    Vec16<T> kx[QT][2], g2[QT][2];
    const bool want2 = BWD || p.has_z;
#pragma unroll
    for (int rt = 0; rt < QT; ++rt) {
        if (wr0 + rt * 16 >= limit) break;         // (uniform) the whole row tile lies behind the end of the sequence
        const int rc = min(wr0 + rt * 16 + lr, limit - 1);
        if (need_d || BWD) {
#pragma unroll
            for (int t = 0; t < 2; ++t) kx[rt][t] = *reinterpret_cast<const Vec16<T> *>(reinterpret_cast<const char *>(xr) + tile64_row_offset(rc, t * 32 + cq));
        }
        if (want2) {
            const T *row2 = BWD ? reinterpret_cast<const T *>(p.x) + b * p.x_sb + ((int64_t)c * Q + rc) * p.x_sl + h * p.x_sh
                                : reinterpret_cast<const T *>(p.z) + b * p.z_sb + ((int64_t)c * Q + rc) * p.z_sl + h * p.z_sh;
#pragma unroll
            for (int t = 0; t < 2; ++t) g2[rt][t] = *reinterpret_cast<const Vec16<T> *>(row2 + p0 + cq + t * 32);
        }
    }
    float dtr[QT];                                 // mirror: dt of this lane's rows
    if (BWD) {
#pragma unroll
        for (int rt = 0; rt < QT; ++rt) dtr[rt] = dto[min(wr0 + rt * 16 + lr, Q - 1)];
    }
    float dcol[2][8];                              // D of this lane's columns
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int e = 0; e < 8; ++e) dcol[t][e] = d_head;
        if (p.has_D && p.D_has_hdim) {
            const float4 d0 = *reinterpret_cast<const float4 *>(p.D + h * P + p0 + t * 32 + cq), d1 = *reinterpret_cast<const float4 *>(p.D + h * P + p0 + t * 32 + cq + 4);
            dcol[t][0] = d0.x; dcol[t][1] = d0.y; dcol[t][2] = d0.z; dcol[t][3] = d0.w;
            dcol[t][4] = d1.x; dcol[t][5] = d1.y; dcol[t][6] = d1.z; dcol[t][7] = d1.w;
        }
    }
#pragma unroll
    for (int rt = 0; rt < QT; ++rt) {
        if (wr0 + rt * 16 >= limit) break;
        const int r = wr0 + rt * 16 + lr, rc = min(r, limit - 1);
        const bool live = r < limit;
        const int64_t orow = (((int64_t)b * p.seqlen + (int64_t)c * Q + rc) * H + h) * P + p0 + cq;
        float rsum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            float a[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = acc[rt][2 * t + (e >> 2)][e & 3];
            if (!BWD) {
                if (need_d) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) a[e] = __builtin_fmaf(dcol[t][e], to_f(kx[rt][t].v[e]), a[e]);
                }
                if (p.has_z) {
                    if (p.out_x && live) {
                        Vec16<T> ox;
#pragma unroll
                        for (int e = 0; e < 8; ++e) ox.v[e] = from_f<T>(a[e]);
                        *reinterpret_cast<Vec16<T> *>(reinterpret_cast<T *>(p.out_x) + orow + t * 32) = ox;
                    }
#pragma unroll
                    for (int e = 0; e < 8; ++e) a[e] *= silu_f(to_f(g2[rt][t].v[e]));
                }
                if (live) {
                    Vec16<T> ov;
#pragma unroll
                    for (int e = 0; e < 8; ++e) ov.v[e] = from_f<T>(a[e]);
                    // out is not read again by any kernel of the pass: past the caches
                    __builtin_nontemporal_store(__builtin_bit_cast(f32x4, ov), reinterpret_cast<f32x4 *>(reinterpret_cast<T *>(p.out) + orow + t * 32));
                }
            } else {
                Vec16<T> ov;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float xv = to_f(g2[rt][t].v[e]), yv = to_f(kx[rt][t].v[e]);
                    rsum = __builtin_fmaf(a[e], xv, rsum);
                    float dxv = a[e] * dtr[rt];
                    if (need_d) dxv = __builtin_fmaf(dcol[t][e], yv, dxv);
                    ov.v[e] = from_f<T>(dxv);
                    // dD: kept in the accumulator's place (it is dead from here on); rows behind the end count nothing
                    acc[rt][2 * t + (e >> 2)][e & 3] = live ? yv * xv : 0.f;
                }
                if (live) __builtin_nontemporal_store(__builtin_bit_cast(f32x4, ov), reinterpret_cast<f32x4 *>(reinterpret_cast<T *>(p.dx) + orow + t * 32));
            }
        }
        if (BWD) {
            // the four lanes lr, lr + 16, lr + 32, lr + 48 hold the four column groups of a row
            rsum += __shfl_xor(rsum, 16, 64);
            rsum += __shfl_xor(rsum, 32, 64);
            if (lg == 0 && live) {
                if (npt == 1) p.ddt_direct[o + r] = rsum;
                else atomicAdd(p.ddt_direct + o + r, rsum);   // several headdim tiles share a row
            }
        }
    }
    if (BWD && p.has_D) {
        // dD partial of this (b, c, h): column sums of dy * x over the rows; a lane holds columns s16_col(j, 4 lg + i) of the
        // rows lr (+16): add the row tiles, then the 16 lanes of a row group, then the waves
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = 0.f;
#pragma unroll
                for (int rt = 0; rt < QT; ++rt)
                    if (wr0 + rt * 16 < limit) v += acc[rt][j][i];
                v = row16_sum(v);
                if (lr == 0) red[wave][s16_col(j, 4 * lg + i)] = v;
            }
        __syncthreads();
        if (threadIdx.x < 64) {
            float v = 0.f;
#pragma unroll
            for (int wv = 0; wv < S16_WAVES; ++wv) v += red[wv][threadIdx.x];
            p.red[((int64_t)(b * nc + c) * H + h) * P + p0 + threadIdx.x] = v;   // partials [(b, c)][h][P]
        }
    }
}

// Launches the kernel above; the caller (launch_chunk_scan) has checked that the problem is one of its shapes:
// scan_recomputes_cb(), 16-bit copies of the entering states present and 16-byte aligned.
template <typename T, bool BWD>
static int launch_scan16_t(const bimamba2_params *p, int nc) {
    const int npt = p->headdim / 64;
    dim3 grid(p->batch * nc * p->nheads * npt);
    hipStream_t s = reinterpret_cast<hipStream_t>(p->stream);
    const bool one = p->chunk_size <= 128;
#define BM2_S16(QTV, UNIV) hipLaunchKernelGGL((chunk_scan16_kernel<T, QTV, BWD, UNIV>), grid, dim3(S16_THREADS), 0, s, *p, nc, npt)
    if (p->causal) { if (one) BM2_S16(1, true); else BM2_S16(2, true); }
    else { if (one) BM2_S16(1, false); else BM2_S16(2, false); }
#undef BM2_S16
    return check_launch();
}

int launch_chunk_scan16(const bimamba2_params *p, bool bwd) {
    const int nc = (p->seqlen + p->chunk_size - 1) / p->chunk_size;
    if (p->dtype == BIMAMBA2_BF16) return bwd ? launch_scan16_t<bf16_t, true>(p, nc) : launch_scan16_t<bf16_t, false>(p, nc);
    if (p->dtype == BIMAMBA2_F16) return bwd ? launch_scan16_t<f16_t, true>(p, nc) : launch_scan16_t<f16_t, false>(p, nc);
    return BIMAMBA2_EUNSUPPORTED;
}

}  // namespace bm2
