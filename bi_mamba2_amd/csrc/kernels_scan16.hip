// The chunk-scan kernel (forward output) and its mirror (dx in the backward pass) for 16-bit inputs on gfx950, for the
// shapes the benchmark configurations with dstate 64 have: headdim a multiple of 64, dstate 64, chunk_size a multiple of 32,
// 16-byte aligned operands, the states entering the chunks kept in their 16-bit copies.
//
// The math is that of chunk_scan_kernel (kernels_scan.hip).  That kernel runs one workgroup per (batch, chunk, head): it
// asks for its operands, waits, computes, asks for its epilogue operands, waits, stores - with two workgroups per CU the
// memory system idles while they compute and the ALUs idle while they wait (counters: VALU busy 53 %, MFMA 19 %, 60 % of
// the copy bandwidth).  Here ONE workgroup of 16 waves owns a CU and walks through several heads of one (batch, chunk):
//  * everything a head needs - its x (resp. dy) tile, its two state tiles, its decay vectors, its z (resp. x) rows - travels
//    from global memory straight into LDS (direct loads: no registers, no staging code) one head ahead of its use
//    (double-buffered; the z / x rows of the head in hand arrive while its K loop runs), so nothing but the first head's
//    operands is ever waited for.  The requests for the next head go out a part at a time during the K loop (issued in one
//    go behind the previous head's stores they fill the memory pipeline's queue and the wave stalls at the issue), and
//    between the requests and the wait in front of the epilogue there is no vector memory operation and no LDS access the
//    compiler knows of: it would make either wait for everything in flight (hence the raw_lds_* accessors);
//  * the heads of a group share C.B^T: each wave computes the CB (resp. CB^T) entries of its 16 rows x 256 columns once and
//    keeps them in 32 registers as float16 pairs, scaled by a power of two that is common to the workgroup so that the
//    largest entry sits at 2^14 (float16 keeps 11 bits of mantissa, three more than the bf16 the masked entries are
//    rounded to for the MFMA anyway; the scale rules out overflow); the K loop has neither a ring of K rows nor a barrier
//    nor CB MFMAs;
//  * away from the diagonal the decay factor of (row r, column k) separates into a factor of the row and the column's
//    16-block and a factor of the column; the column factors are kept as float16 as well (scaled per block into [0.5, 1),
//    the exponent going to the row factor), so a K step multiplies them onto the CB entries two at a time and then
//    applies the row factor with the conversion to float32 in the same instruction: 2 instructions per entry instead of 3.5
//    (the kernel is bound by VALU issue: 63 % busy against 16 % for the MFMA pipe);
//  * the K operand lies in LDS as it lies in memory and its MFMA fragments are LDS transpose reads;
//  * the products are computed transposed, D[p][r] = sum_k X[k][p] A[r][k]: operand fragments are the same registers as
//    for D[r][p] with the two MFMA operands swapped, but a lane then holds four consecutive headdim columns of ONE row
//    per 16-column tile.  Which headdim column an MFMA row stands for is free (it is decided where the operand
//    fragments are read), and is chosen so that the tiles 2t and 2t + 1 together give a lane EIGHT consecutive columns,
//    32 t + 8 (lane / 16) ..: out / out_x / dx leave as 16-byte stores and z / x / dy arrive as 16-byte LDS reads without
//    the accumulators passing through LDS, and the per-row factors are one value per lane;
//  * the K loop is unrolled over its (at most 8) steps: table and fragment offsets are immediates.
//
//   forward (BWD = false), rows r = output positions t, k = source positions s:
//     acc[r,p] = e^{cs_f[r]} C_r.prev_f[p,:] + e^{cs_b[r]} C_r.prev_b[p,:]
//              + sum_k CB[r,k] m(r,k) dt[k] x[k,p],    m = e^{cs_f[r]-cs_f[k]} (k<r), e^{cs_b[r]-cs_b[k]} (k>r), 2 (k=r)
//     out_x = acc + D x[r,p];  out = out_x * silu(z)
//   mirror (BWD = true), rows r = input positions s, k = output positions t, CBT[r,k] = CB[k,r]:
//     acc[r,p] = e^{cs_f[Q-1]-cs_f[r]} B_r.dS_f[p,:] + e^{cs_b[0]-cs_b[r]} B_r.dS_b[p,:]
//              + sum_k CBT[r,k] m'(r,k) dy[k,p],       m' = e^{cs_f[k]-cs_f[r]} (k>r), e^{cs_b[k]-cs_b[r]} (k<r), 2 (k=r)
//     dx = acc dt[r] + D dy[r,p];  ddt_direct[r] = sum_p acc x[r,p];  dD partial = sum_r dy x
#include <atomic>
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace bm2 {

namespace {

constexpr int S16_WAVES = 16, S16_THREADS = 64 * S16_WAVES;
constexpr int S16_ROWS = 16 * S16_WAVES;          // rows the workgroup covers (>= chunk_size)
constexpr int S16_NSTEP = S16_ROWS / 32;          // K steps at most
constexpr int S16_MAX_HEADS = 12;                 // heads a workgroup walks through at most

// LDS map (bytes), by the state dimension DS (64 or 128).
// DS = 64: two buffers of x (dy) tiles, two buffers of state tiles, the K rows (32 KB) whose place takes the z (x) rows later.
// DS = 128: the K rows take 64 KB and a pair of state tiles 32 KB, so the map holds one pair of state tiles; the K rows, needed
// only in front of the first head, lie over the second x-tile buffer and the z-row area, which are filled later.  With a z
// gate the state tiles are single-buffered (the requests for the next head's pair go out behind a barrier that follows
// this head's state products); without one the z-row area holds the second pair.
template <int DS> struct S16Map {
    static constexpr int ROWB = DS * 2;                                   // bytes of a K row / of a state-tile row
    static constexpr int ST_TILE = 64 * ROWB;                             // one state tile [p][n], 16-byte chunks ^ (p % 8)
    static constexpr int ST_BUFS = DS == 64 ? 2 : 1;
    static constexpr int XR0 = 0;                                         // raw K-operand tile (x, resp. dy) of buffer 0: [256][64] 16-bit, tile64 swizzle
    static constexpr int ST = XR0 + 32768;                                // ST_BUFS x 2 state tiles
    static constexpr int XR1 = ST + ST_BUFS * 2 * ST_TILE;                // K-operand tile of buffer 1
    static constexpr int XR_STRIDE = XR1 - XR0;
    static constexpr int ZR = XR1 + 32768;                                // z (resp. x) rows of the head in hand, tile64 swizzle
    static constexpr int KT = DS == 64 ? ZR : XR1;                        // K rows (B, resp. C) of the chunk, chunks ^ (row % 8)
    static constexpr int RAW = ZR + 32768;                                // 2 x (cs_f, cs_b, dt) of a head as they lie in memory
    static constexpr int TAB = RAW + 2 * 3 * 1024;                        // lo, up, glo, gup, dtl of the head in hand
    static constexpr int RED = TAB + 5 * 1024;                            // mirror: per-wave column sums of dy * x
    static constexpr int DT = RED + S16_WAVES * 64 * 4;                   // D of the workgroup's heads, one value per headdim column
    static constexpr int LDS = DT + S16_MAX_HEADS * 64 * 4;
    static_assert(KT + 256 * ROWB <= RAW, "the K rows must end in front of the tables");
    static_assert(LDS <= 160 * 1024, "LDS of a CU");
};

// byte offset of the elements (r, n ..), n a multiple of 4, in a raw [rows][64] 16-bit tile whose 16-byte chunks are swizzled
// by tile64_swz (the layout tile64_request leaves)
__device__ __forceinline__ int tile64_row_offset(int r, int n) {
    return r * 128 + ((((n >> 3) ^ tile64_swz(r)) << 4) | ((n & 4) << 1));
}

// headdim column (inside the workgroup's 64) that row m of the 16-row MFMA tile j stands for: 32 (j/2) + 8 (m/4) + 4 (j%2) + m%4.
// Output rows m = 4 g + i of lane group g are then the columns 32 t + 8 g + i (tile 2t) and 32 t + 8 g + 4 + i (tile 2t + 1).
__device__ __forceinline__ constexpr int s16_col(int j, int m) { return 32 * (j >> 1) + 8 * (m >> 2) + 4 * (j & 1) + (m & 3); }

// f(integral_constant<int, I>) for I = 0 .. N - 1, until it returns false: a loop whose index is a constant expression inside
// the body (LDS offsets become immediates)
template <int I, int N, class F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        if (f(std::integral_constant<int, I>())) static_for<I + 1, N>(f);
    }
}

}  // namespace

// UNI: the single-direction (causal) operator: the reverse direction's state product, the K steps on the far side of the
// diagonal and the far half of the diagonal step are left out.
// hpw: heads per workgroup (divides nheads / ngroups, <= S16_MAX_HEADS); blockIdx.x = ((pt * nslices + slice) * nbc + bc).
// DCOLS (mirror): dD per (head, headdim column); else one value per head.
// DS: the state dimension, 64 or 128 (128: forward only).
template <typename T, bool BWD, bool UNI, bool DCOLS = false, int DS = 64>
__global__ __launch_bounds__(S16_THREADS) void chunk_scan16_kernel(const bimamba2_params p, int nc, int npt, int hpw) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    typedef S16Map<DS> L;
    static_assert(sizeof(T) == 2, "16-bit operands");
    static_assert(DS == 64 || (DS == 128 && !BWD), "state dimension 64, or 128 in the forward kernel");
    constexpr int KSTEP = 32, NSTEP = S16_NSTEP;
    constexpr int NF = DS / 32;                    // MFMA K steps over the state dimension
    constexpr int ROWB = L::ROWB;
    // One pair of state tiles where the map has room for one only (DS = 128) and the z-row area is in use; without a z gate
    // that area (32 KB, free once the K rows are done with) holds the second pair.
    const bool st_single = L::ST_BUFS == 1 && (BWD || p.has_z);
    auto st_buf_off = [&](int buf) __attribute__((always_inline)) {
        return L::ST_BUFS == 2 ? buf * 2 * L::ST_TILE : st_single ? 0 : buf * (L::ZR - L::ST);
    };
    // (aligned: the fragment addresses below flip bit 6 of an absolute LDS address)
    __shared__ __attribute__((aligned(1024))) unsigned char smem[L::LDS];
    const unsigned sbase = lds_addr(smem);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    // consecutive block ids are dealt round-robin to the 8 XCDs: bc fastest keeps the workgroups of one (batch, chunk), which
    // share the B and C rows, on one XCD's L2
    const int nbc = p.batch * nc;
    const int bc = blockIdx.x % nbc, sp = blockIdx.x / nbc, nslices = p.nheads / hpw, slice = sp % nslices, pt = sp / nslices;
    const int c = bc % nc, b = bc / nc;
    const int h0 = slice * hpw;
    const int g = h0 / (p.nheads / p.ngroups);
    const int Q = p.chunk_size, P = p.headdim, H = p.nheads;
    const int limit = min(Q, p.seqlen - c * Q);
    const int nsteps = (limit + KSTEP - 1) / KSTEP;
    const int p0 = pt * 64;
    const int wr0 = wave * 16;                     // this wave's rows wr0 .. wr0 + 15
    const bool active = wr0 < limit;               // (uniform) waves whose rows lie behind the end only help with the loads
    const int r_own = wr0 + lr, rc_own = min(r_own, limit - 1);

    // Every global address below is a wave-uniform 64-bit base (scalar registers) plus a 32-bit byte offset of the lane (the
    // launcher checks that 256 rows of every row stride fit 32 bits): lane parts are few and cheap to keep.
    // rows u*8 + lane/8 (u = 2 wave, 2 wave + 1) of a 256-row tile, 16-byte chunk (lane%8) ^ swizzle(row) at chunk position lane%8
    // The lane parts are recomputed from the lane number wherever they are needed (`ln` is made opaque there: kept across
    // the head loop they would be spilled, and a reload from scratch memory between two requests waits for the first one).
    const unsigned ks_bytes = (unsigned)((!BWD ? p.x_sl : p.has_z ? (int64_t)H * P : p.dout_sl) * (int64_t)sizeof(T));
    const unsigned s2_bytes = (unsigned)((BWD ? p.x_sl : p.z_sl) * (int64_t)sizeof(T));
    // rows wave*16 + ln/8 (+8) of a 256-row tile with row stride `rs` bytes: 16-byte chunk (ln%8) ^ swizzle(row) at position ln%8
    auto tile_off = [&](int ln, int half, unsigned rs) __attribute__((always_inline)) {
        const int row = wave * 16 + half * 8 + (ln >> 3);
        return (unsigned)min(row, limit - 1) * rs + (unsigned)(((ln & 7) ^ tile64_swz(row)) << 4);
    };

    // ---- requests of a head: its K-operand tile (parts 0, 1), its two state tiles (2), its decay vectors (3) -> buffer `buf`.
    // In parts, so that the K loop can hand them to the memory pipeline one at a time: issued in one go behind the previous
    // head's output stores they fill its queue, and a wave whose request does not fit waits there instead of computing.
    auto request_part = [&](int h, int buf, int part) __attribute__((always_inline)) {
        int ln = lane;
        asm volatile("" : "+v"(ln));
        if (part < 2) {
            const char *kp;
            if (!BWD) kp = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * p.x_sl + h * p.x_sh + p0);
            else if (p.has_z) kp = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.dout_x) + ((int64_t)b * p.seqlen + (int64_t)c * Q) * H * P + (int64_t)h * P + p0);
            else kp = reinterpret_cast<const char *>(reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * p.dout_sl + h * p.dout_sh + p0);
            kp = uniform_ptr(kp);
            // (rows behind the last K step are never read; their requests go to the clamped, valid row all the same)
            // (the mirror is the last kernel of the pass that reads dout_x and the gradients of the entering states)
            load16_to_lds_at<BWD>(kp, tile_off(ln, part, ks_bytes), smem + L::XR0 + buf * L::XR_STRIDE + wave * 2048 + part * 1024);
        } else if (part == 2) {
            const int dir = wave >> 3;
            if (!(UNI && dir)) {
                const int64_t so = ((int64_t)(b * nc + c) * H + h) * P * DS + (int64_t)p0 * DS;
                const T *src = reinterpret_cast<const T *>(BWD ? (dir ? p.dstates16_b : p.dstates16_f) : (dir ? p.states16_b : p.states16_f));
                const int sboff = st_buf_off(buf);
                if constexpr (DS == 64) {
                    // thread t of a half brings row t/8, chunk position t%8 <- chunk (t%8) ^ (row%8)
                    const int row = (wave & 7) * 8 + (ln >> 3);
                    const unsigned soff = (unsigned)((row * 64 + (((ln & 7) ^ (row & 7)) << 3)) * sizeof(T));
                    load16_to_lds_at<BWD>(uniform_ptr(src + so), soff, smem + L::ST + sboff + dir * L::ST_TILE + (wave & 7) * 1024);
                } else {
                    // rows of 256 bytes: a wave of a half brings 8 rows in two loads of 4, chunk position l%16 <- chunk (l%16) ^ (row%8)
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const int row = ((wave & 7) * 2 + u) * 4 + (ln >> 4);
                        const unsigned soff = (unsigned)(row * ROWB + (((ln & 15) ^ (row & 7)) << 4));
                        load16_to_lds_at<BWD>(uniform_ptr(src + so), soff, smem + L::ST + sboff + dir * L::ST_TILE + ((wave & 7) * 2 + u) * 1024);
                    }
                }
            }
        } else if (wave < 3) {
            // cs_f, cs_b, dt (waves 0, 1, 2): 256 floats each (entries past chunk_size are never used: clamped to stay inside)
            const float *src = (wave == 0 ? p.cs_f : wave == 1 ? p.cs_b : p.dt_out) + (((int64_t)b * H + h) * nc + c) * Q;
            load16_to_lds_at(uniform_ptr(src), (unsigned)min(ln * 4, Q - 4) * 4u, smem + L::RAW + (buf * 3 + wave) * 1024);
        }
    };
    auto request_head = [&](int h, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int part = 0; part < 4; ++part) request_part(h, buf, part);
    };
    // requests of a head this wave issues (the vmcnt a wait for something older has to leave outstanding)
    const int head_requests = 2 + ((UNI && wave >= 8) ? 0 : (DS == 64 ? 1 : 2)) + (wave < 3 ? 1 : 0);

    // ---- prologue: the K rows of the chunk (B, resp. C), this lane's own rows (C, resp. B), the first head's operands.  The
    // products below wait for the first two only; the head's operands land meanwhile.  (LDS accesses are raw from here on.)
    {
        const T *kr;
        int64_t krs;
        if (BWD) { krs = p.C_sl; kr = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * krs + g * p.C_sg; }
        else { krs = p.B_sl; kr = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * krs + g * p.B_sg; }
        // units of 1 KB: 8 rows of 128 bytes (DS = 64) or 4 rows of 256 bytes (DS = 128), 16-byte chunk ^ (row % 8)
        constexpr int UR = 1024 / ROWB, UC = ROWB / 16, NU = 256 / UR / S16_WAVES;
#pragma unroll
        for (int uu = 0; uu < NU; ++uu) {
            const int u = wave * NU + uu, row = u * UR + lane / UC;
            if (u * UR < nsteps * KSTEP)
                load16_to_lds_at(uniform_ptr(kr), (unsigned)min(row, limit - 1) * (unsigned)(krs * sizeof(T)) + (((lane & (UC - 1)) ^ (row & 7)) << 4), smem + L::KT + u * 1024);
        }
    }
    Frag own[NF];
    {
        const T *ap;
        int64_t as;
        if (BWD) { as = p.B_sl; ap = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * as + g * p.B_sg; }
        else { as = p.C_sl; ap = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * as + g * p.C_sg; }
#pragma unroll
        for (int f = 0; f < NF; ++f) own[f] = M::load(ap + (int64_t)rc_own * as + f * KSTEP + lg * 8);
    }
    float d_val = 0.f;                             // D of head h0 + tid / 64, headdim column tid % 64
    if ((int)threadIdx.x < hpw * 64 && p.has_D) {
        const int hh = h0 + ((int)threadIdx.x >> 6), col = threadIdx.x & 63;
        d_val = p.D_has_hdim ? p.D[hh * P + p0 + col] : p.D[hh];
    }
    request_head(h0, 0);
    // everything older than this wave's last two requests has landed (a wave issues at least two per head): the K rows it
    // brought, its own rows, its D values
    wait_vmcnt<2>();
    if ((int)threadIdx.x < hpw * 64) raw_lds_write_at<0>(sbase + L::DT + threadIdx.x * 4, d_val);
    raw_lds_wait();
    raw_lds_barrier();
    // CB (resp. CB^T) of this wave's rows against every column of the chunk, in operand layout: D[m][n] = sum_d Krow[k(m)][d]
    // Own[n][d] with k(m) = k0 + 8*(m/4) + m%4 leaves lane (l%16 = row, l/16 = g) with columns k0 + 8g + 0..3, the second
    // product (k(m) + 4) with columns k0 + 8g + 4..7.  Fragment (hh, f): K row krow + 4*hh of the step, 16-byte chunk lg + 4*f,
    // stored at chunk ^ (row % 8); with krow % 8 = lr % 4 that is element kfb + 256*hh + 32*(f ^ hh) of the step's 32 rows.
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    unsigned cbh[NSTEP][4];                        // step s: columns k0 + 8 lg + {0,1}, {2,3}, {4,5}, {6,7} of row wr0 + lr (float16 pairs)
    float cb_unscale;                              // 1 / (the power of two the entries were scaled by)
    {
        f32x4 cb1[NSTEP], cb2[NSTEP];
        // (in bytes, rows of ROWB: fragment (hh, f) of step s sits at s*32*ROWB + hh*4*ROWB + 64*((f&1)^hh) + 128*(f>>1) from here)
        const unsigned kt = sbase + L::KT + (8 * (lr >> 2) + (lr & 3)) * ROWB + (lg ^ (lr & 3)) * 16;
        static_for<0, NSTEP>([&](auto S) __attribute__((always_inline)) {
            constexpr int s = decltype(S)::value;
            cb1[s] = cb2[s] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (active && s < nsteps) {
                static_for<0, NF / 2>([&](auto F2) __attribute__((always_inline)) {
                    constexpr int f2 = decltype(F2)::value, O = s * 32 * ROWB + 128 * f2;
                    Frag kf00 = raw_lds_read_at<Frag, O>(kt), kf01 = raw_lds_read_at<Frag, O + 64>(kt);
                    Frag kf10 = raw_lds_read_at<Frag, O + 4 * ROWB + 64>(kt), kf11 = raw_lds_read_at<Frag, O + 4 * ROWB>(kt);
                    raw_lds_wait();
                    raw_lds_use(kf00); raw_lds_use(kf01); raw_lds_use(kf10); raw_lds_use(kf11);
                    cb1[s] = M::mma(kf00, own[2 * f2], cb1[s]);
                    cb2[s] = M::mma(kf10, own[2 * f2], cb2[s]);
                    cb1[s] = M::mma(kf01, own[2 * f2 + 1], cb1[s]);
                    cb2[s] = M::mma(kf11, own[2 * f2 + 1], cb2[s]);
                    return true;
                });
            }
            return true;
        });
        // the largest entry of the workgroup decides the scale
        float mx = 0.f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) mx = fmaxf(mx, fmaxf(fabsf(cb1[s][i]), fabsf(cb2[s][i])));
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
        if (lane == 0) raw_lds_write_at<0>(sbase + L::RED + wave * 4, mx);
        raw_lds_wait();
        wait_vmcnt<0>();                           // the first head's operands (this wave's share; the barrier makes it everybody's)
        raw_lds_barrier();                         // (everybody is done with the K rows as well: their place takes the z / x rows)
        {
            float wm = raw_lds_read_at<float, 0>(sbase + L::RED + (lane & (S16_WAVES - 1)) * 4);
            raw_lds_wait();
            raw_lds_use(wm);
            mx = wm;
#pragma unroll
            for (int d = S16_WAVES / 2; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
        }
        // scale = 2^(14 - e), e the exponent of the maximum (1 for an all-zero or non-finite block)
        const int ex = (int)((__float_as_uint(mx) >> 23) & 255u);
        const bool ok = ex > 0 && ex < 255;
        const float scale = ok ? __uint_as_float((unsigned)min(254, 127 + 14 + 127 - ex) << 23) : 1.f;
        cb_unscale = ok ? __uint_as_float((unsigned)max(1, 127 - 14 - 127 + ex) << 23) : 1.f;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            cbh[s][0] = __builtin_bit_cast(unsigned, half2_t{(_Float16)(cb1[s][0] * scale), (_Float16)(cb1[s][1] * scale)});
            cbh[s][1] = __builtin_bit_cast(unsigned, half2_t{(_Float16)(cb1[s][2] * scale), (_Float16)(cb1[s][3] * scale)});
            cbh[s][2] = __builtin_bit_cast(unsigned, half2_t{(_Float16)(cb2[s][0] * scale), (_Float16)(cb2[s][1] * scale)});
            cbh[s][3] = __builtin_bit_cast(unsigned, half2_t{(_Float16)(cb2[s][2] * scale), (_Float16)(cb2[s][3] * scale)});
        }
    }

    // per-lane LDS addresses
    const unsigned tab = sbase + L::TAB;          // lo +0, up +1024, glo +2048 (mlo +2560), gup +3072 (mup +3584), dtl +4096
    const unsigned lg32 = lg * 32;                 // this lane's 8 columns inside a step of the float tables
    // column factors of this lane's 8 columns (8 float16 = 16 bytes) and the reference exponent of their block of 16
    unsigned g_l = tab + 2048 + lg * 16, m_l = tab + 2048 + 512 + (lg >> 1) * 4;
    unsigned tab_l = tab + lg32;                   // lo of this lane's columns; up +1024, glo +2048, gup +3072, dtl +4096
    // K-operand fragments: LDS transpose reads of the raw tile, rows k0 + 8 lg + lr/4 (+4); source lane s of a 16-lane group
    // supplies the four columns s16_col(j, 4 (s%4)) .., which lanes 4 (s%4) .. + 3 of the group receive
    // (rows k + 4: the swizzle flips bit 2 of the chunk position, i.e. byte bit 6, and the row adds 512 bytes).
    // The addresses follow the buffer of the head in hand.
    // Tile j reads the columns s16_col(j, 4 (lr%4)) = 32 (j/2) + 4 (j%2) + 8 (lr%4) ..: against tile 0 that is 8 bytes further
    // for j%2 (bit 3 of the offset, clear in tile 0's) and bit 6 flipped for j/2 (chunk position bit 2), so tile 0's address and
    // its bit-6 twin serve all four tiles and both row halves, everything else being immediates.
    unsigned xo0 = sbase + L::XR0 + tile64_tr_offset(8 * lg + (lr >> 2), s16_col(0, 4 * (lr & 3)));
    const int cq = 8 * lg;                         // first of this lane's eight columns inside a 32-column half

    auto cb_at = [&](int s, int col) __attribute__((always_inline)) { return (float)__builtin_bit_cast(half2_t, cbh[s][col >> 1])[col & 1]; };
    int r_lane = r_own;
    for (int hi = 0; hi < hpw; ++hi) {
        int h = h0 + hi;
        // (opaque: seen as a function of the loop counter, the head's base addresses become per-lane running pointers)
        asm volatile("" : "+s"(h));
        const int cur = hi & 1;
        // What does not change from head to head (the packed CB entries, the lane's row) is made opaque here: hoisted out of
        // the loop, the unpacked entries and the diagonal steps' comparison masks would take a few hundred registers.
#pragma unroll
        for (int s = 0; s < NSTEP; ++s)
#pragma unroll
            for (int k = 0; k < 4; ++k) asm volatile("" : "+v"(cbh[s][k]));
        asm volatile("" : "+v"(r_lane));
        asm volatile("" : "+v"(tab_l));
        asm volatile("" : "+v"(g_l));
        asm volatile("" : "+v"(m_l));
        int wr0_l = wr0;
        asm volatile("" : "+s"(wr0_l));
        unsigned sb = sbase;                       // (addresses used once per head are rebuilt from this, not kept across the loop)
        asm volatile("" : "+s"(sb));
        // From here to the end of the loop every LDS access is a raw one (the compiler makes an LDS access it knows of, and a
        // register it believes a load still owes, wait for EVERY vector memory operation in flight: the requests below and
        // the previous head's output stores, which are meant to drain while this head is worked on), and there is no global
        // load besides the requests.
        // ---- requests: this head's z (resp. x) rows, each wave its own 16; the next head's operands go out during the K
        // loop, four parts at the first four steps (waves without rows in the chunk have no K loop: theirs go out here)
        const bool more = hi + 1 < hpw;
        int hn = h + 1;
        asm volatile("" : "+s"(hn));
        // (single-buffered state tiles: theirs go out behind the barrier that follows the state products)
        if (!st_single && more && !active) request_head(hn, cur ^ 1);
        if (BWD || p.has_z) {
            const char *row2 = uniform_ptr(
                BWD ? reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * p.x_sl + h * p.x_sh + p0
                    : reinterpret_cast<const T *>(p.z) + b * p.z_sb + (int64_t)c * Q * p.z_sl + h * p.z_sh + p0);
            if (active) {
                int ln = lane;
                asm volatile("" : "+v"(ln));
                load16_to_lds_at(row2, tile_off(ln, 0, s2_bytes), smem + L::ZR + wave * 2048);
                load16_to_lds_at(row2, tile_off(ln, 1, s2_bytes), smem + L::ZR + wave * 2048 + 1024);
            }
        }
        // ---- tables of this head
        // forward: k<r uses lo[r]-lo[k] with lo = cs_f, k>r uses up[r]-up[k] with up = cs_b
        // mirror : k<r uses e^{cs_b[k]-cs_b[r]} -> lo = -cs_b;  k>r uses e^{cs_f[k]-cs_f[r]} -> up = -cs_f
        // Away from the diagonal the factor separates: with m = lo at the last position of k's block of 16 (which lies
        // between k and r), 2^{lo[r]-lo[k]} = 2^{lo[r]-m} * glo[k], glo[k] = 2^{m-lo[k]}, both factors <= 1 for A <= 0;
        // likewise gup[k] = 2^{up[first of k's block] - up[k]}.  The column factors also carry dt[k] (forward) and the zero
        // of the rows behind the end of the sequence, which the raw tile holds as copies of its last row.
        const unsigned raw_a = sb + L::RAW + cur * 3072;        // cs_f +0, cs_b +1024, dt +2048
        if (threadIdx.x < S16_ROWS) {
            int q = threadIdx.x;
            asm volatile("" : "+v"(q));             // (the addresses below are rebuilt per head, not kept across the loop)
            const int qq = min(q, Q - 1), qe = min(q | 15, Q - 1), qs = min(q & ~15, Q - 1);
            float f = raw_lds_read_at<float, 0>(raw_a + qq * 4), r = raw_lds_read_at<float, 1024>(raw_a + qq * 4);
            float fe = BWD ? raw_lds_read_at<float, 1024>(raw_a + qe * 4) : raw_lds_read_at<float, 0>(raw_a + qe * 4);
            float rs = BWD ? raw_lds_read_at<float, 0>(raw_a + qs * 4) : raw_lds_read_at<float, 1024>(raw_a + qs * 4);
            float dtq = BWD ? 1.f : raw_lds_read_at<float, 2048>(raw_a + qq * 4);
            raw_lds_wait();
            raw_lds_use(f); raw_lds_use(r); raw_lds_use(fe); raw_lds_use(rs); raw_lds_use(dtq);
            f *= LOG2E; r *= LOG2E;
            fe *= BWD ? -LOG2E : LOG2E; rs *= BWD ? -LOG2E : LOG2E;
            if (q >= limit) dtq = 0.f;
            const float l = BWD ? -r : f, u = BWD ? -f : r;
            const unsigned ta = sb + L::TAB + q * 4;
            raw_lds_write_at<0>(ta, l);
            raw_lds_write_at<1024>(ta, u);
            raw_lds_write_at<4096>(ta, dtq);
            // the column factors as float16, scaled by a power of two per block of 16 (this thread's 16-lane row) that brings
            // the block's largest one into [0.5, 1) (the scaled CB entries stay below 2^15, so the products stay finite): the K loop multiplies them onto the float16 CB entries two at a time.
            // The block's exponent goes into its reference point, i.e. into the row factor.
            const float gl = __builtin_amdgcn_exp2f(fe - l) * dtq, gu = __builtin_amdgcn_exp2f(rs - u) * dtq;
            const unsigned exl = (__float_as_uint(row16_max(gl)) >> 23) & 255u, exu = (__float_as_uint(row16_max(gu)) >> 23) & 255u;
            const bool okl = exl > 0 && exl < 254, oku = exu > 0 && exu < 254;       // (zero or denormal maximum: left as it is)
            const _Float16 hl = (_Float16)(okl ? gl * __uint_as_float((253u - exl) << 23) : gl);
            const _Float16 hu = (_Float16)(oku ? gu * __uint_as_float((253u - exu) << 23) : gu);
            const unsigned tg = sb + L::TAB + q * 2;
            raw_lds_write16_at<2048>(tg, hl);
            raw_lds_write16_at<3072>(tg, hu);
            if ((q & 15) == 0) {
                const unsigned tm = sb + L::TAB + (q >> 4) * 4;
                raw_lds_write_at<2048 + 512>(tm, fe - (okl ? (float)((int)exl - 126) : 0.f));
                raw_lds_write_at<3072 + 512>(tm, rs - (oku ? (float)((int)exu - 126) : 0.f));
            }
        }
        // mirror: the far ends of the chunk and dt of this lane's row
        float e_f = 0.f, e_b = 0.f;
        if (BWD) {
            e_f = raw_lds_read_at<float, 0>(raw_a + (Q - 1) * 4);
            e_b = raw_lds_read_at<float, 1024>(raw_a);
            raw_lds_wait();
            raw_lds_use(e_f); raw_lds_use(e_b);
            e_f *= LOG2E; e_b *= LOG2E;
        }
        raw_lds_wait();
        raw_lds_barrier();                         // #1: the tables are there (everybody's requests for this head landed before #2)

        f32x4 acc[4];
        float lor = 0.f, upr = 0.f;
        if (active) {
            lor = raw_lds_read_at<float, 0>(tab + r_own * 4);
            upr = raw_lds_read_at<float, 1024>(tab + r_own * 4);
            // ---- part 1: states.  D[p][r] = sum_n S[p][n] Own[r][n], scaled by this lane's row factor, one direction after the other
            // Fragment (tile j, state step s) of a state tile lies at row s16_col(j, lr), 16-byte chunk (4 s + lg) ^ (row % 8).  With
            // row = [32 (j/2) + 4 (j%2)] + [8 (lr/4) + lr%4] the lane's part is one address and everything else a constant:
            // (row % 8) = lr%4 + 4 (j%2), so the chunk is (lg ^ lr%4) + 4 ((s%2) ^ (j%2)) + 8 (s/2).
            const unsigned st_lane = sb + L::ST + st_buf_off(cur) + (8 * (lr >> 2) + (lr & 3)) * ROWB + ((lg ^ (lr & 3)) << 4);
            static_for<0, (UNI ? 1 : 2)>([&](auto DIR) __attribute__((always_inline)) {
                constexpr int dir = decltype(DIR)::value;
                f32x4 tmp[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) tmp[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                static_for<0, 2 * (NF / 2)>([&](auto JS) __attribute__((always_inline)) {
                    constexpr int jj = 2 * (decltype(JS)::value / (NF / 2)), s0 = 2 * (decltype(JS)::value % (NF / 2));
                    constexpr int O0 = dir * L::ST_TILE + (32 * (jj >> 1)) * ROWB + 128 * (s0 >> 1);      // tile jj (even): j%2 = 0
                    constexpr int O1 = O0 + 4 * ROWB;                                                     // tile jj + 1
                    Frag a0 = raw_lds_read_at<Frag, O0>(st_lane), a1 = raw_lds_read_at<Frag, O0 + 64>(st_lane);
                    Frag b0 = raw_lds_read_at<Frag, O1 + 64>(st_lane), b1 = raw_lds_read_at<Frag, O1>(st_lane);
                    raw_lds_wait();
                    raw_lds_use(a0); raw_lds_use(a1); raw_lds_use(b0); raw_lds_use(b1);
                    tmp[jj] = M::mma(a0, own[s0], tmp[jj]);
                    tmp[jj] = M::mma(a1, own[s0 + 1], tmp[jj]);
                    tmp[jj + 1] = M::mma(b0, own[s0], tmp[jj + 1]);
                    tmp[jj + 1] = M::mma(b1, own[s0 + 1], tmp[jj + 1]);
                    return true;
                });
                raw_lds_use(lor); raw_lds_use(upr);
                // forward: e^{cs_f[r]} = 2^{lo[r]}, e^{cs_b[r]} = 2^{up[r]}; mirror: e^{cs_f[Q-1]-cs_f[r]} = 2^{e_f+up[r]}, e^{cs_b[0]-cs_b[r]} = 2^{e_b+lo[r]}
                const float e = __builtin_amdgcn_exp2f(BWD ? (dir ? e_b + lor : e_f + upr) : (dir ? upr : lor));
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = dir ? tmp[j] * e + acc[j] : tmp[j] * e;
                return true;
            });
        }
        if (st_single) {
            // the one pair of state tiles: every wave is done with it here, so the next head's pair may be requested (the
            // active waves do that at their third K step)
            raw_lds_wait();
            raw_lds_barrier();
            if (more && !active) request_head(hn, cur ^ 1);
        }
        if (active) {
            // ---- part 2: inside the chunk.  Per K step of 32 columns: CB (resp. CB^T) times the decay factors, times the K operand
            const unsigned xo1 = xo0 ^ 64u;
            auto k_step = [&](auto STEP) __attribute__((always_inline)) -> bool {
                constexpr int step = decltype(STEP)::value;
                if (step < 4 && more) request_part(hn, cur ^ 1, step);
                if (step >= nsteps) return true;
                constexpr int k0 = step * KSTEP;
                // the wave's rows [wr0, wr0 + 16) meet the step's columns [k0, k0 + 32) in one step only
                const int cls = (k0 + KSTEP - 1 < wr0_l) ? 0 : (k0 > wr0_l + 15) ? 1 : 2;   // below, above, across the diagonal
                if (UNI && cls == (BWD ? 0 : 1)) return true;                              // far side of the diagonal
                constexpr int TB = step * (KSTEP * 4);     // byte offset of the step inside the float tables
                constexpr int XS = step * (KSTEP * 128);
                Frag af;
                // the K-operand fragments of the first two column tiles are asked for behind the step's table values and
                // arrive while the decay factors are worked out
                // (all of them in straight-line code in front of the branch: a value read from inline assembly must not pass
                // through a merge of two definitions, whose copy could be placed in front of the wait; the step across the
                // diagonal reads the column factors without using them)
                const unsigned sel = cls == 1 ? 1024u : 0u;
                typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
                u32x4 gq = raw_lds_read_at<u32x4, step * 64>(g_l + sel);
                float mref = raw_lds_read_at<float, step * 8>(m_l + sel);
                i16x4 xa0 = raw_lds_tr16_read_at<XS>(xo0), xa1 = raw_lds_tr16_read_at<XS + 512>(xo1);
                i16x4 xb0 = raw_lds_tr16_read_at<XS + 8>(xo0), xb1 = raw_lds_tr16_read_at<XS + 512 + 8>(xo1);
                raw_lds_wait_n<4>();
                raw_lds_use(gq); raw_lds_use(mref);
                if (cls != 2) {
                    const float rf = __builtin_amdgcn_exp2f((cls == 0 ? lor : upr) - mref) * cb_unscale;
                    float v[8];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        // two entries times their column factors in float16, then each times the row factor in float32
                        // (vector element copied to a scalar first: __builtin_bit_cast applied to the element itself reads element 0)
                        const unsigned gk = gq[k];
                        const half2_t t = __builtin_bit_cast(half2_t, cbh[step][k]) * __builtin_bit_cast(half2_t, gk);
                        v[2 * k] = __builtin_fmaf((float)t[0], rf, 0.f);
                        v[2 * k + 1] = __builtin_fmaf((float)t[1], rf, 0.f);
                    }
                    af = M::pack(v);
                } else {
                    // the one step across the diagonal: element by element, four columns at a time
                    const unsigned la = tab_l;
                    const int kb = k0 + lg * 8;
                    float v[8];
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        f32x4 l0 = hh ? raw_lds_read_at<f32x4, TB + 16>(la) : raw_lds_read_at<f32x4, TB>(la);
                        f32x4 u0 = hh ? raw_lds_read_at<f32x4, TB + 1024 + 16>(la) : raw_lds_read_at<f32x4, TB + 1024>(la);
                        f32x4 d0 = hh ? raw_lds_read_at<f32x4, TB + 4096 + 16>(la) : raw_lds_read_at<f32x4, TB + 4096>(la);
                        raw_lds_wait();
                        raw_lds_use(l0); raw_lds_use(u0); raw_lds_use(d0);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int k = kb + hh * 4 + i;
                            const float e = k < r_lane ? lor - l0[i] : upr - u0[i];
                            float w = (k == r_lane) ? (UNI ? 1.f : 2.f) : __builtin_amdgcn_exp2f(e);
                            if (UNI && (BWD ? k < r_lane : k > r_lane)) w = 0.f;
                            v[hh * 4 + i] = cb_at(step, hh * 4 + i) * (w * d0[i] * cb_unscale);
                        }
                    }
                    af = M::pack(v);
                }
                // ---- the product with the K operand, transposed: D[p][r] += X[k][p] A[r][k]; two column tiles at a time
                {
                    // tiles 2, 3 (the bit-6 twins of the addresses) are asked for before tiles 0, 1 are multiplied
                    const i16x4 c0 = raw_lds_tr16_read_at<XS>(xo1), c1 = raw_lds_tr16_read_at<XS + 512>(xo0);
                    const i16x4 d0 = raw_lds_tr16_read_at<XS + 8>(xo1), d1 = raw_lds_tr16_read_at<XS + 512 + 8>(xo0);
                    raw_lds_wait_n<4>();
                    raw_lds_use(xa0); raw_lds_use(xa1); raw_lds_use(xb0); raw_lds_use(xb1);
                    i16x8 fa = __builtin_shufflevector(xa0, xa1, 0, 1, 2, 3, 4, 5, 6, 7), fb = __builtin_shufflevector(xb0, xb1, 0, 1, 2, 3, 4, 5, 6, 7);
                    acc[0] = M::mma(__builtin_bit_cast(Frag, fa), af, acc[0]);
                    acc[1] = M::mma(__builtin_bit_cast(Frag, fb), af, acc[1]);
                    raw_lds_wait();
                    i16x8 fc = __builtin_shufflevector(c0, c1, 0, 1, 2, 3, 4, 5, 6, 7), fd = __builtin_shufflevector(d0, d1, 0, 1, 2, 3, 4, 5, 6, 7);
                    raw_lds_use(fc); raw_lds_use(fd);
                    acc[2] = M::mma(__builtin_bit_cast(Frag, fc), af, acc[2]);
                    acc[3] = M::mma(__builtin_bit_cast(Frag, fd), af, acc[3]);
                }
                return true;
            };
            static_for<0, NSTEP>(k_step);
        }
        // this wave's z (resp. x) rows have landed: everything but the requests for the next head, which are younger
        if (!more) wait_vmcnt<0>();
        else if (head_requests == 2) wait_vmcnt<2>();
        else if (head_requests == 3) wait_vmcnt<3>();
        else if (head_requests == 4) wait_vmcnt<4>();
        else wait_vmcnt<5>();
        // ---- epilogue.  acc[2t][i], acc[2t+1][i] = row wr0 + lr, headdim columns p0 + 32 t + 8 lg + i, + 4 + i ----
        f32x4 res_a[2], res_b[2];                  // packed results of the two column halves: out / dx, and out_x
        float rsum = 0.f, dsum = 0.f;
        constexpr bool d_cols = DCOLS;             // mirror: dD per (head, column), else one value per head
        const bool live = r_own < limit;
        if (active) {
            const bool need_d = p.has_D;
            const unsigned d_a = sb + L::DT + hi * 256 + cq * 4;
            float dtr = 0.f;                       // mirror: dt of this lane's row
            if (BWD) dtr = raw_lds_read_at<float, 2048>(raw_a + min(r_lane, Q - 1) * 4);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                // the D term's row (forward: x, mirror: dy) from the raw tile, z (resp. x) from the rows this wave brought
                const unsigned eo = sb + tile64_row_offset(min(r_lane, limit - 1), t * 32 + cq);
                // (read whether used or not: the addresses are valid, and a conditional read needs its registers cleared first)
                f32x4 kx4 = raw_lds_read_at<f32x4, 0>(eo + (L::XR0 + cur * L::XR_STRIDE));
                f32x4 g24 = raw_lds_read_at<f32x4, 0>(eo + L::ZR);
                f32x4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
                if (!BWD || need_d) {                  // (the mirror is out of registers: there the read stays conditional)
                    d0 = t ? raw_lds_read_at<f32x4, 128>(d_a) : raw_lds_read_at<f32x4, 0>(d_a);
                    d1 = t ? raw_lds_read_at<f32x4, 144>(d_a) : raw_lds_read_at<f32x4, 16>(d_a);
                }
                raw_lds_wait();
                raw_lds_use(kx4); raw_lds_use(g24); raw_lds_use(d0); raw_lds_use(d1);
                const Vec16<T> kx = __builtin_bit_cast(Vec16<T>, kx4), g2 = __builtin_bit_cast(Vec16<T>, g24);
                const float dcol[8] = {d0[0], d0[1], d0[2], d0[3], d1[0], d1[1], d1[2], d1[3]};
                float a[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) a[e] = acc[2 * t + (e >> 2)][e & 3];
                if (!BWD) {
                    if (need_d) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) a[e] = __builtin_fmaf(dcol[e], to_f(kx.v[e]), a[e]);
                    }
                    if (p.has_z) {
                        if (p.out_x) {
                            Vec16<T> ox;
#pragma unroll
                            for (int e = 0; e < 8; ++e) ox.v[e] = from_f<T>(a[e]);
                            res_b[t] = __builtin_bit_cast(f32x4, ox);
                        }
#pragma unroll
                        for (int e = 0; e < 8; ++e) a[e] *= silu_f(to_f(g2.v[e]));
                    }
                    Vec16<T> ov;
#pragma unroll
                    for (int e = 0; e < 8; ++e) ov.v[e] = from_f<T>(a[e]);
                    res_a[t] = __builtin_bit_cast(f32x4, ov);
                } else {
                    Vec16<T> ov;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float xv = to_f(g2.v[e]), yv = to_f(kx.v[e]);
                        rsum = __builtin_fmaf(a[e], xv, rsum);
                        float dxv = a[e] * dtr;
                        if (need_d) dxv = __builtin_fmaf(dcol[e], yv, dxv);
                        ov.v[e] = from_f<T>(dxv);
                        // dD: per headdim column kept in the accumulator's place (it is dead from here on; rows behind the end
                        // count nothing); one value per head: a running sum
                        if (d_cols) acc[2 * t + (e >> 2)][e & 3] = live ? yv * xv : 0.f;
                        else dsum = __builtin_fmaf(yv, xv, dsum);
                    }
                    res_a[t] = __builtin_bit_cast(f32x4, ov);
                }
            }
        }
        // The next head's operands (this wave's share) have landed; waited for here, in front of this head's stores: a wait
        // behind them would be for the stores as well.
        wait_vmcnt<0>();
        if (active) {
            // output rows: uniform base of the (chunk, head) + this lane's row and column group
            int hh = h;
            asm volatile("" : "+s"(hh));            // (addresses are built here, not kept from the top of the loop)
            // (dx may be a slice of a wider buffer: its own position and batch strides)
            const bool own = BWD && p.dx_sl != 0;
            const unsigned osl = own ? (unsigned)p.dx_sl : (unsigned)(H * P);
            const int64_t obase = (own ? b * p.dx_sb + (int64_t)c * Q * p.dx_sl : ((int64_t)b * p.seqlen + (int64_t)c * Q) * (H * P)) + (int64_t)hh * P + p0;
            const unsigned orow = (unsigned)min(r_lane, limit - 1) * osl + cq;
            if (live) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    if (!BWD && p.has_z && p.out_x) *reinterpret_cast<f32x4 *>(reinterpret_cast<T *>(p.out_x) + obase + (orow + t * 32)) = res_b[t];
                    // out (resp. dx) is not read again by any kernel of the pass: past the caches
                    __builtin_nontemporal_store(res_a[t], reinterpret_cast<f32x4 *>(reinterpret_cast<T *>(BWD ? p.dx : p.out) + obase + (orow + t * 32)));
                }
            }
            if (BWD) {
                // the four lanes lr, lr + 16, lr + 32, lr + 48 hold the four column groups of a row
                // (lane indices rebuilt here: kept from the prologue's shuffles they would be spilled)
                int ln = lane;
                asm volatile("" : "+v"(ln));
                rsum += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((ln ^ 16) << 2, __builtin_bit_cast(int, rsum)));
                rsum += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((ln ^ 32) << 2, __builtin_bit_cast(int, rsum)));
                if (lg == 0 && live) {
                    // (several headdim tiles share a row: each writes the plane of its tile, the reader adds them)
                    p.ddt_direct[(int64_t)pt * ((int64_t)p.batch * H * nc * Q) + ((((int64_t)b * H + hh) * nc + c) * Q + r_lane)] = rsum;
                }
            }
        }
        if (BWD && p.has_D) {
            if (d_cols) {
                // dD partial of this (b, c, h): column sums of dy * x over the rows; a lane holds columns s16_col(j, 4 lg + i) of
                // row lr: add the 16 lanes of a row group, then the waves
                const unsigned red_a = sb + L::RED + (wave * 64 + 8 * lg) * 4;
                static_for<0, 16>([&](auto JI) __attribute__((always_inline)) {
                    constexpr int j = decltype(JI)::value >> 2, i = decltype(JI)::value & 3;
                    const float v = row16_sum(active ? acc[j][i] : 0.f);
                    if (lr == 0) raw_lds_write_at<s16_col(j, i) * 4>(red_a, v);   // s16_col(j, 4 lg + i) = s16_col(j, i) + 8 lg
                    return true;
                });
            } else {
                // one value per head: the wave's sum of dy * x over its live rows
                int ln = lane;
                asm volatile("" : "+v"(ln));
                float v = row16_sum((active && live) ? dsum : 0.f);
                v += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((ln ^ 16) << 2, __builtin_bit_cast(int, v)));
                v += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((ln ^ 32) << 2, __builtin_bit_cast(int, v)));
                if (ln == 0) raw_lds_write_at<0>(sb + L::RED + wave * 4, v);
            }
        }
        // #2: everybody is done with this head's tiles, tables and z rows (a bare barrier: the stores just issued need not
        // have completed)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        raw_lds_barrier();
        if (BWD && p.has_D && threadIdx.x < 64) {
            float pv[S16_WAVES];
            // per column: the waves' sums of this thread's column; per head: the waves' sums, kept by thread 0 (the partial sums
            // have the same layout either way, [(b, c)][h][P]: the other columns of the head then hold zeros)
            const unsigned red_a = sb + L::RED + (d_cols ? threadIdx.x * 4 : 0u);
            if (d_cols) {
                static_for<0, S16_WAVES>([&](auto WV) __attribute__((always_inline)) {
                    pv[decltype(WV)::value] = raw_lds_read_at<float, decltype(WV)::value * 256>(red_a);
                    return true;
                });
            } else {
                static_for<0, S16_WAVES>([&](auto WV) __attribute__((always_inline)) {
                    pv[decltype(WV)::value] = raw_lds_read_at<float, decltype(WV)::value * 4>(red_a);
                    return true;
                });
            }
            raw_lds_wait();
            float v = 0.f;
#pragma unroll
            for (int wv = 0; wv < S16_WAVES; ++wv) { raw_lds_use(pv[wv]); v += pv[wv]; }
            if (!d_cols && threadIdx.x != 0) v = 0.f;
            p.red[((int64_t)(b * nc + c) * H + h) * P + p0 + threadIdx.x] = v;   // partials [(b, c)][h][P]
        }
        // the fragment addresses move on to the other buffer
        xo0 = cur ? xo0 - (unsigned)L::XR_STRIDE : xo0 + (unsigned)L::XR_STRIDE;
    }
}

// CUs of the current device (one workgroup of the kernel above fills a CU), asked for once per device
static int cu_count() {
    constexpr int MAXD = 64;
    static std::atomic<int> cached[MAXD];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAXD) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Heads a workgroup of the kernel above walks through: a divisor k <= S16_MAX_HEADS of the heads per group, chosen for the
// shortest launch.  The grid runs in rounds of one workgroup per CU, and a workgroup takes a fixed start (launch, first
// loads, CB: about 0.8 of a head's time) plus k heads: rounds(k) * (0.8 + k) is what is compared, the larger k on a tie.
static int scan16_heads_per_block(const bimamba2_params *p, int nc) {
    const int hpg = p->nheads / p->ngroups, cus = cu_count();
    const long long units = (long long)p->batch * nc * (p->headdim / 64) * p->nheads;
    int best = 1;
    double best_cost = 0;
    for (int k = 1; k <= S16_MAX_HEADS; ++k) {
        if (hpg % k) continue;
        const long long rounds = (units / k + cus - 1) / cus;
        const double cost = rounds * (0.8 + k);
        if (k == 1 || cost <= best_cost) { best = k; best_cost = cost; }
    }
    return best;
}

int chunk_scan16_heads_per_workgroup(const bimamba2_params *p) {
    return scan16_heads_per_block(p, (p->seqlen + p->chunk_size - 1) / p->chunk_size);
}

// Launches the kernel above; the caller (launch_chunk_scan) has checked that the problem is one of its shapes:
// scan_recomputes_cb(), 16-bit copies of the entering states present and 16-byte aligned.
template <typename T, bool BWD>
static int launch_scan16_t(const bimamba2_params *p, int nc) {
    const int npt = p->headdim / 64, hpw = scan16_heads_per_block(p, nc);
    dim3 grid(p->batch * nc * (p->nheads / hpw) * npt);
    hipStream_t s = reinterpret_cast<hipStream_t>(p->stream);
    if (p->dstate == 128) {
        // the forward kernel only (launch_chunk_scan sends the mirror of this shape elsewhere)
        if constexpr (!BWD) {
            if (p->causal) hipLaunchKernelGGL((chunk_scan16_kernel<T, false, true, false, 128>), grid, dim3(S16_THREADS), 0, s, *p, nc, npt, hpw);
            else hipLaunchKernelGGL((chunk_scan16_kernel<T, false, false, false, 128>), grid, dim3(S16_THREADS), 0, s, *p, nc, npt, hpw);
        } else {
            return BIMAMBA2_EUNSUPPORTED;
        }
    } else if (BWD && p->has_D && p->D_has_hdim) {
        if (p->causal) hipLaunchKernelGGL((chunk_scan16_kernel<T, BWD, true, BWD>), grid, dim3(S16_THREADS), 0, s, *p, nc, npt, hpw);
        else hipLaunchKernelGGL((chunk_scan16_kernel<T, BWD, false, BWD>), grid, dim3(S16_THREADS), 0, s, *p, nc, npt, hpw);
    } else {
        if (p->causal) hipLaunchKernelGGL((chunk_scan16_kernel<T, BWD, true>), grid, dim3(S16_THREADS), 0, s, *p, nc, npt, hpw);
        else hipLaunchKernelGGL((chunk_scan16_kernel<T, BWD, false>), grid, dim3(S16_THREADS), 0, s, *p, nc, npt, hpw);
    }
    return check_launch();
}

int launch_chunk_scan16(const bimamba2_params *p, bool bwd) {
    const int nc = (p->seqlen + p->chunk_size - 1) / p->chunk_size;
    if (p->dtype == BIMAMBA2_BF16) return bwd ? launch_scan16_t<bf16_t, true>(p, nc) : launch_scan16_t<bf16_t, false>(p, nc);
    if (p->dtype == BIMAMBA2_F16) return bwd ? launch_scan16_t<f16_t, true>(p, nc) : launch_scan16_t<f16_t, false>(p, nc);
    return BIMAMBA2_EUNSUPPORTED;
}

}  // namespace bm2

