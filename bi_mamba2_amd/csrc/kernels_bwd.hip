// Backward kernels of the bidirectional SSD operator for gfx950 (the gradient of the chunk-entry states and dx
// reuse chunk_state_kernel / chunk_scan_kernel from kernels_fwd.hip).
//   bwd_dz             dz and dout*silu(z)
//   state_passing_bwd  both inter-chunk adjoint recurrences in one launch + the chunk-total decay gradients
//   bwd_dbdc           state part of dB (or dC) summed over the heads of a group + per-position decay terms
//   bwd_dcb            G = dy.x^T once per head -> dCB (summed over heads) and the within-chunk decay gradient
//   bmm_chunk_bwd      dB = dBs + dCB^T.C ; dC = dCs + dCB.B
//   chunk_cumsum_bwd   assembles d(dt*A) from its pieces with wavefront scans; ddt, dA, ddt_bias
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace bm2 {

static inline int nchunks(const bimamba2_params *p) { return (p->seqlen + p->chunk_size - 1) / p->chunk_size; }
static inline hipStream_t stream_of(const bimamba2_params *p) { return reinterpret_cast<hipStream_t>(p->stream); }

// block index of a kernel body that may run as one of several roles of a launch
struct BlockId { int x, y, z; };

// =========================================================================================================
__global__ void fill_kernel(float *ptr, size_t n, float value) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) ptr[i] = value;
}
int launch_fill(float *ptr, size_t n, float value, hipStream_t stream) {
    if (n == 0) return BIMAMBA2_OK;
    const int blocks = (int)std::min<size_t>((n + 255) / 256, 2048);
    hipLaunchKernelGGL(fill_kernel, dim3(blocks), dim3(256), 0, stream, ptr, n, value);
    return check_launch();
}

// out[j] = sum_i sum_k in[(i*nj + j)*nk + k]; one workgroup per j
__global__ __launch_bounds__(NTHREADS) void reduce_kernel(const float *in, float *out, int ni, int nj, int nk) {
    __shared__ float red[4];
    const int j = blockIdx.x;
    float s = 0.f;
    const int total = ni * nk;
    for (int t = threadIdx.x; t < total; t += NTHREADS) {
        const int i = t / nk, k = t - i * nk;
        s += in[((int64_t)i * nj + j) * nk + k];
    }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) out[j] = red[0] + red[1] + red[2] + red[3];
}
int launch_reduce(const float *in, float *out, int ni, int nj, int nk, hipStream_t stream) {
    hipLaunchKernelGGL(reduce_kernel, dim3(nj), dim3(NTHREADS), 0, stream, in, out, ni, nj, nk);
    return check_launch();
}

// several such reductions in one launch (the backward pass ends with three small ones)
__global__ __launch_bounds__(NTHREADS) void reduce_jobs_kernel(ReduceJobs jobs) {
    __shared__ float red[4];
    int j = blockIdx.x, k = 0;
    while (k + 1 < jobs.n && j >= jobs.job[k].nj) { j -= jobs.job[k].nj; ++k; }
    const ReduceJob jb = jobs.job[k];
    float s = 0.f;
    const int total = jb.ni * jb.nk;
    // eight loads go out before the first is added: a load that is waited for costs microseconds here
    for (int t0 = threadIdx.x; t0 < total; t0 += 8 * NTHREADS) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = min(t0 + u * NTHREADS, total - 1), i = t / jb.nk, kk = t - i * jb.nk;
            v[u] = jb.in[((int64_t)i * jb.nj + j) * jb.nk + kk];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (t0 + u * NTHREADS < total) s += v[u];
    }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) jb.out[j] = red[0] + red[1] + red[2] + red[3];
}
int launch_reduce_jobs(const ReduceJobs &jobs, hipStream_t stream) {
    int blocks = 0;
    for (int k = 0; k < jobs.n; ++k) blocks += jobs.job[k].nj;
    if (blocks == 0) return BIMAMBA2_OK;
    hipLaunchKernelGGL(reduce_jobs_kernel, dim3(blocks), dim3(NTHREADS), 0, stream, jobs);
    return check_launch();
}

// =========================================================================================================
// dz = dout * out_x * sigmoid(z) (1 + z (1 - sigmoid(z)));  dout_x = dout * z * sigmoid(z)
// =========================================================================================================
template <typename T>
__global__ __launch_bounds__(NTHREADS) void bwd_dz_kernel(const bimamba2_params p) {
    constexpr int VS = 16 / sizeof(T);
    const int P = p.headdim;
    const int pv = (P + VS - 1) / VS;
    const int64_t nrows = (int64_t)p.batch * p.seqlen * p.nheads;
    const T *zb = reinterpret_cast<const T *>(p.z);
    const T *db = reinterpret_cast<const T *>(p.dout);
    const T *ox = reinterpret_cast<const T *>(p.out_x);
    T *dz = reinterpret_cast<T *>(p.dz);
    T *dox = reinterpret_cast<T *>(p.dout_x);
    // z and dout laid out like out_x (rows of headdim one behind the other, headdim a multiple of the vector): a vector
    // unit's offset is the same in all of them and no index has to be taken apart (three 64-bit divisions per unit, most of
    // the kernel's instructions otherwise)
    const bool packed = P % VS == 0 && p.z_sh == P && p.z_sl == (int64_t)p.nheads * P && p.z_sb == (int64_t)p.seqlen * p.nheads * P &&
                        p.dout_sh == P && p.dout_sl == p.z_sl && p.dout_sb == p.z_sb;
    for (int64_t idx = blockIdx.x * (int64_t)NTHREADS + threadIdx.x; idx < nrows * pv; idx += (int64_t)gridDim.x * NTHREADS) {
        const T *zp, *dp;
        int64_t o;
        int c0;
        if (packed) {
            o = idx * VS;
            c0 = 0;                               // (only its distance from the row's end matters below: a whole vector fits)
            zp = zb + o;
            dp = db + o;
        } else {
            const int64_t row = idx / pv;
            c0 = (int)(idx - row * pv) * VS;
            const int h = (int)(row % p.nheads);
            const int64_t bl = row / p.nheads;
            const int l = (int)(bl % p.seqlen), b = (int)(bl / p.seqlen);
            zp = zb + b * p.z_sb + l * p.z_sl + h * p.z_sh + c0;
            dp = db + b * p.dout_sb + l * p.dout_sl + h * p.dout_sh + c0;
            o = row * P + c0;
        }
        const bool vec = (c0 + VS <= P) && aligned16(zp, 0) && aligned16(dp, 0) && aligned16(ox + o, 0);
        float zv[VS], dv[VS], ov[VS];
        if (vec) {
            // all three are read for the last time in this pass
            const Vec16<T> a = __builtin_bit_cast(Vec16<T>, __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(zp))),
                           d = __builtin_bit_cast(Vec16<T>, __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(dp))),
                           e = __builtin_bit_cast(Vec16<T>, __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(ox + o)));
#pragma unroll
            for (int i = 0; i < VS; ++i) { zv[i] = to_f(a.v[i]); dv[i] = to_f(d.v[i]); ov[i] = to_f(e.v[i]); }
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i) {
                const bool ok = c0 + i < P;
                zv[i] = ok ? to_f(zp[i]) : 0.f; dv[i] = ok ? to_f(dp[i]) : 0.f; ov[i] = ok ? to_f(ox[o + i]) : 0.f;
            }
        }
        Vec16<T> r1, r2;
#pragma unroll
        for (int i = 0; i < VS; ++i) {
            const float sg = sigmoid_f(zv[i]);
            r1.v[i] = from_f<T>(dv[i] * ov[i] * sg * (1.f + zv[i] * (1.f - sg)));
            r2.v[i] = from_f<T>(dv[i] * zv[i] * sg);
        }
        if (vec) {
            // dz is not read again inside the pass, dout_x by four kernels: the first goes past the caches
            __builtin_nontemporal_store(__builtin_bit_cast(f32x4, r1), reinterpret_cast<f32x4 *>(dz + o));
            *reinterpret_cast<Vec16<T> *>(dox + o) = r2;
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i)
                if (c0 + i < P) { dz[o + i] = r1.v[i]; dox[o + i] = r2.v[i]; }
        }
    }
}

int launch_bwd_dz(const bimamba2_params *p) {
    const int64_t n = (int64_t)p->batch * p->seqlen * p->nheads * ((p->headdim + 3) / 4);
    const int blocks = (int)std::min<int64_t>((n + NTHREADS - 1) / NTHREADS, 8192);
    switch (p->dtype) {
        case BIMAMBA2_F32: hipLaunchKernelGGL(bwd_dz_kernel<float>, dim3(blocks), dim3(NTHREADS), 0, stream_of(p), *p); break;
        case BIMAMBA2_BF16: hipLaunchKernelGGL(bwd_dz_kernel<bf16_t>, dim3(blocks), dim3(NTHREADS), 0, stream_of(p), *p); break;
        case BIMAMBA2_F16: hipLaunchKernelGGL(bwd_dz_kernel<f16_t>, dim3(blocks), dim3(NTHREADS), 0, stream_of(p), *p); break;
        default: return BIMAMBA2_EUNSUPPORTED;
    }
    return check_launch();
}

// =========================================================================================================
// adjoint of the inter-chunk recurrences.  On entry dstates_* hold the gradient w.r.t. the state entering
// each chunk (dprev); on exit they hold the gradient w.r.t. each chunk's own state S[c]:
//   forward dir : g = dfinal_f (or 0); for c = nc-1..0 : dS_f[c] = g; ddA_chunk_f[c] = e^{tot_c} <g, prev_f[c]>; g = dprev_f[c] + e^{tot_c} g
//   reverse dir : g = dfinal_b (or 0); for c = 0..nc-1 : dS_b[c] = g; ddA_chunk_b[c] = e^{tot_c} <g, prev_b[c]>; g = dprev_b[c] + e^{tot_c} g
// What g holds at the end is the gradient with respect to the initial state (written to dinitial_* when given).
// A workgroup owns SP_EPT*256 of the P*N elements of one (b, h); its partial inner products go to
// ddA_chunk_*[b, h, c, split].
// =========================================================================================================
constexpr int SP_EPT = 4;
__global__ __launch_bounds__(NTHREADS) void state_passing_bwd_kernel(const bimamba2_params p, int nc, int nsplit) {
    __shared__ float red[2][4];
    const int PN = p.headdim * p.dstate;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int Q = p.chunk_size;
    const float *csf = p.cs_f + ((int64_t)b * p.nheads + h) * nc * Q;
    const float *csb = p.cs_b + ((int64_t)b * p.nheads + h) * nc * Q;
    const int64_t cstride = (int64_t)p.nheads * PN;
    const int64_t base = ((int64_t)b * nc * p.nheads + h) * PN;
    const int e0 = split * SP_EPT * NTHREADS + threadIdx.x;
    for (int dir = 0; dir < 2; ++dir) {
        const float *prev = (dir == 0 ? p.states_f : p.states_b) + base;
        float *ds = (dir == 0 ? p.dstates_f : p.dstates_b) + base;
        float *dda = (dir == 0 ? p.ddA_chunk_f : p.ddA_chunk_b) + ((int64_t)b * p.nheads + h) * nc * nsplit + split;
        const float *dfin = dir == 0 ? p.dfinal_f : p.dfinal_b;
        float *dini = dir == 0 ? p.dinitial_f : p.dinitial_b;
        const int64_t bh = ((int64_t)b * p.nheads + h) * PN;
        float g[SP_EPT];
#pragma unroll
        for (int i = 0; i < SP_EPT; ++i) {
            const int e = e0 + i * NTHREADS;
            g[i] = (dfin && e < PN) ? dfin[bh + e] : 0.f;
        }
        for (int step = 0; step < nc; ++step) {
            const int c = dir == 0 ? nc - 1 - step : step;
            const float dec = __expf(dir == 0 ? csf[(int64_t)c * Q + Q - 1] : csb[(int64_t)c * Q]);
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < SP_EPT; ++i) {
                const int e = e0 + i * NTHREADS;
                if (e < PN) {
                    const int64_t a = c * cstride + e;
                    const float dp = ds[a];
                    dot += g[i] * prev[a];
                    ds[a] = g[i];
                    g[i] = dp + dec * g[i];
                }
            }
            dot = wave_sum(dot);
            if (lane == 0) red[step & 1][wave] = dot;
            __syncthreads();
            if (threadIdx.x == 0) dda[(int64_t)c * nsplit] = dec * (red[step & 1][0] + red[step & 1][1] + red[step & 1][2] + red[step & 1][3]);
        }
        if (dini) {
#pragma unroll
            for (int i = 0; i < SP_EPT; ++i) {
                const int e = e0 + i * NTHREADS;
                if (e < PN) dini[bh + e] = g[i];
            }
        }
        __syncthreads();
    }
}

// The same with 16-byte accesses, one direction per workgroup (blockIdx.z = 2 b + dir) and the loads of SP_CH chunks in
// flight before the first of them is used: the recurrence is a chain over the chunks, and a global access that has to be
// waited for at every link costs microseconds.  Needs P*N % 4 == 0 and 16-byte aligned tensors.
// PREV16: the entering states are read from their 16-bit copies (states16_*); DS16: the gradients with respect to the
// entering states go to dstates16_* and the per-chunk gradients in dstates_* stay as they are.
// DP16 (with DS16): the per-chunk gradients lie in dstates16_* in the 16-bit type as well (no float32 tensors): every one is
// read once and replaced in place by the gradient with respect to the state entering its chunk.
constexpr int SP_CH = 8;
template <typename T16, bool PREV16, bool DS16, bool DP16 = false>
__device__ __forceinline__ void state_passing_bwd_vec_body(const bimamba2_params &p, int nc, int nsplit, int ndir, BlockId bid) {
    struct alignas(8) V4 { T16 v[4]; };
    __shared__ float red[SP_CH][4];
    const int PN = p.headdim * p.dstate;
    const int split = bid.x, h = bid.y, b = bid.z / ndir, dir = bid.z % ndir;   // ndir = 1: forward direction only
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int Q = p.chunk_size;
    const float *cs = (dir == 0 ? p.cs_f : p.cs_b) + ((int64_t)b * p.nheads + h) * nc * Q + (dir == 0 ? Q - 1 : 0);
    const int64_t cstride = (int64_t)p.nheads * PN;
    const int64_t base = ((int64_t)b * nc * p.nheads + h) * PN;
    const int e_own = (split * NTHREADS + threadIdx.x) * SP_EPT;
    const bool live = e_own < PN;
    const int e = live ? e_own : PN - SP_EPT;              // loads are unconditional (so that they all go out together)
    const float *prev = (dir == 0 ? p.states_f : p.states_b) + base + e;
    const T16 *prev16 = reinterpret_cast<const T16 *>(dir == 0 ? p.states16_f : p.states16_b) + base + e;
    float *ds = (dir == 0 ? p.dstates_f : p.dstates_b) + base + e;
    T16 *ds16 = reinterpret_cast<T16 *>(dir == 0 ? p.dstates16_f : p.dstates16_b) + base + e;
    float *dda = (dir == 0 ? p.ddA_chunk_f : p.ddA_chunk_b) + ((int64_t)b * p.nheads + h) * nc * nsplit + split;
    const float *dfin = dir == 0 ? p.dfinal_f : p.dfinal_b;
    float *dini = dir == 0 ? p.dinitial_f : p.dinitial_b;
    const int64_t bh = ((int64_t)b * p.nheads + h) * PN + e;
    f32x4 g = {0.f, 0.f, 0.f, 0.f};
    if (dfin) g = *reinterpret_cast<const f32x4 *>(dfin + bh);
    for (int s0 = 0; s0 < nc; s0 += SP_CH) {
        const int nb = min(SP_CH, nc - s0);
        f32x4 dp[SP_CH], pv[SP_CH];
        float dec[SP_CH];
#pragma unroll
        for (int j = 0; j < SP_CH; ++j) {
            const int sj = min(s0 + j, nc - 1);            // past the last chunk: a valid chunk again, never used
            const int c = dir == 0 ? nc - 1 - sj : sj;
            dec[j] = cs[(int64_t)c * Q];
            // (both are read for the last time in the pass: past the caches)
            if constexpr (DP16) {
                const V4 t = *reinterpret_cast<const V4 *>(ds16 + c * cstride);
#pragma unroll
                for (int k = 0; k < 4; ++k) dp[j][k] = to_f(t.v[k]);
            } else {
                dp[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(ds + c * cstride));
            }
            if constexpr (PREV16) {
                typedef float f32x2 __attribute__((ext_vector_type(2)));
                const V4 t = __builtin_bit_cast(V4, __builtin_nontemporal_load(reinterpret_cast<const f32x2 *>(prev16 + c * cstride)));
#pragma unroll
                for (int k = 0; k < 4; ++k) pv[j][k] = to_f(t.v[k]);
            } else {
                pv[j] = *reinterpret_cast<const f32x4 *>(prev + c * cstride);
            }
        }
#pragma unroll
        for (int j = 0; j < SP_CH; ++j) {
            if (j < nb) {
                const int c = dir == 0 ? nc - 1 - (s0 + j) : s0 + j;
                const float d = __expf(dec[j]);
                float dot = 0.f;
                if (live) {
                    dot = g[0] * pv[j][0] + g[1] * pv[j][1] + g[2] * pv[j][2] + g[3] * pv[j][3];
                    if constexpr (DS16) {
                        V4 t;
#pragma unroll
                        for (int k = 0; k < 4; ++k) t.v[k] = from_f<T16>(g[k]);
                        *reinterpret_cast<V4 *>(ds16 + c * cstride) = t;
                    } else {
                        *reinterpret_cast<f32x4 *>(ds + c * cstride) = g;
                    }
                    g = dp[j] + d * g;
                }
                dot = wave_sum(dot) * d;
                if (lane == 0) red[j][wave] = dot;
            }
        }
        __syncthreads();
        if ((int)threadIdx.x < nb) {
            const int c = dir == 0 ? nc - 1 - (s0 + (int)threadIdx.x) : s0 + (int)threadIdx.x;
            dda[(int64_t)c * nsplit] = red[threadIdx.x][0] + red[threadIdx.x][1] + red[threadIdx.x][2] + red[threadIdx.x][3];
        }
        __syncthreads();
    }
    if (dini && live) *reinterpret_cast<f32x4 *>(dini + bh) = g;
}
template <typename T16, bool PREV16, bool DS16, bool DP16 = false>
__global__ __launch_bounds__(NTHREADS) void state_passing_bwd_vec_kernel(const bimamba2_params p, int nc, int nsplit, int ndir) {
    state_passing_bwd_vec_body<T16, PREV16, DS16, DP16>(p, nc, nsplit, ndir, BlockId{(int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z});
}

int launch_state_passing_bwd(const bimamba2_params *p) {
    const int nc = nchunks(p), PN = p->headdim * p->dstate;
    const int nsplit = (PN + SP_EPT * NTHREADS - 1) / (SP_EPT * NTHREADS);
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    const int ndir = p->causal ? 1 : 2;
    if (PN % 4 == 0 && al(p->states_f) && al(p->states_b) && al(p->dstates_f) && al(p->dstates_b) && al(p->dfinal_f) && al(p->dfinal_b) &&
        al(p->dinitial_f) && al(p->dinitial_b)) {
        dim3 grid(nsplit, p->nheads, p->batch * ndir);
        const bool prev16 = p->states16_f != nullptr, ds16 = p->dstates16_f != nullptr;
        if (prev16 && (!(p->causal || p->states16_b) || !al(p->states16_f) || !al(p->states16_b))) return BIMAMBA2_EINVAL;
        if (ds16 && (!(p->causal || p->dstates16_b) || !al(p->dstates16_f) || !al(p->dstates16_b))) return BIMAMBA2_EINVAL;
        if ((prev16 || ds16) && p->dtype != BIMAMBA2_BF16 && p->dtype != BIMAMBA2_F16) return BIMAMBA2_EUNSUPPORTED;
        if (!p->dstates_f) {
            // the per-chunk gradients lie in dstates16_* (16-bit): in place; known with the 16-bit copies on both sides only
            if (!(prev16 && ds16)) return BIMAMBA2_EINVAL;
            if (p->dtype == BIMAMBA2_F16) hipLaunchKernelGGL((state_passing_bwd_vec_kernel<f16_t, true, true, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsplit, ndir);
            else hipLaunchKernelGGL((state_passing_bwd_vec_kernel<bf16_t, true, true, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsplit, ndir);
            return check_launch();
        }
#define BM2_SPB(TT, A, B) hipLaunchKernelGGL((state_passing_bwd_vec_kernel<TT, A, B>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsplit, ndir)
        if (p->dtype == BIMAMBA2_F16) {
            if (prev16 && ds16) BM2_SPB(f16_t, true, true); else if (prev16) BM2_SPB(f16_t, true, false);
            else if (ds16) BM2_SPB(f16_t, false, true); else BM2_SPB(f16_t, false, false);
        } else {
            if (prev16 && ds16) BM2_SPB(bf16_t, true, true); else if (prev16) BM2_SPB(bf16_t, true, false);
            else if (ds16) BM2_SPB(bf16_t, false, true); else BM2_SPB(bf16_t, false, false);
        }
#undef BM2_SPB
        return check_launch();
    }
    if (p->states16_f || p->dstates16_f) return BIMAMBA2_EUNSUPPORTED;
    if (p->causal) return BIMAMBA2_EUNSUPPORTED;
    if (!p->dstates_f || !p->dstates_b) return BIMAMBA2_EINVAL;
    dim3 grid(nsplit, p->nheads, p->batch);
    hipLaunchKernelGGL(state_passing_bwd_kernel, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsplit);
    return check_launch();
}

// =========================================================================================================
// state part of dC (IS_DB = false), rows r = positions t of a 64-row tile, summed over the heads of a group:
//   tmp_f = dy_h[r,:] . prev_f[h]  (K = headdim),  dCs[r,n] += e^{cs_f[r]} tmp_f + e^{cs_b[r]} tmp_b
//   u_f[h,r] = e^{cs_f[r]} sum_n tmp_f[r,n] C[r,n]      (same for b)
// state part of dB (IS_DB = true), rows r = positions s:
//   tmp_f = x_h[r,:] . dS_f[h],  dBs[r,n] += dt[r] (e^{cs_f[Q-1]-cs_f[r]} tmp_f + e^{cs_b[0]-cs_b[r]} tmp_b)
//   v_f[h,r] = dt[r] e^{cs_f[Q-1]-cs_f[r]} sum_n tmp_f[r,n] B[r,n]
// =========================================================================================================
constexpr int DBDC_HEADS = 8;         // heads per slice (measured against 4 with 256-row tiles: dB / dC / tail 0.323 -> 0.316 ms per step)
static inline int dbdc_slices(const bimamba2_params *p) { return (p->nheads / p->ngroups + DBDC_HEADS - 1) / DBDC_HEADS; }

// The A operand (x or dout rows, K = headdim contiguous) is read from global memory straight into MFMA operand
// registers; the states, stored [p][n], are staged transposed ([n][p], 64 x 64 at a time) in LDS, double-buffered for
// 16-bit types so that one barrier per step suffices.
constexpr int DBDC_WAVES = 8, DBDC_THREADS = 64 * DBDC_WAVES;

// 8 waves; wave w owns QT 16-row tiles: the workgroup covers 128*QT rows, so that with QT = 2 a 256-row chunk reads
// each state once.  Global memory latency is hidden by software pipelining over "steps" (head, dstate tile, headdim
// chunk): the state blocks and A fragments of step s+1 are requested into registers before step s is multiplied, and
// only then written to the LDS image.
// UNI: the forward direction's state only (single-direction comparator).
template <typename T, int NT, int QT, bool IS_DB, bool FAST, bool UNI = false>
__global__ __launch_bounds__(DBDC_THREADS) void bwd_dbdc_kernel(const bimamba2_params p, int nc) {
    typedef Mma<T> M;
    constexpr int KPL = M::KPL, KSTEP = M::KSTEP, KC = 64, NKS = KC / KSTEP;
    constexpr int VK = 16 / (int)sizeof(T);                                // image rows (k) per staged block; 4 columns (n)
    constexpr int LDX = KC + VK;
    constexpr int NBUF = sizeof(T) == 2 ? 2 : 1;
    constexpr int ROWS = DBDC_WAVES * 16 * QT;
    constexpr int NBLK = (KC / VK) * (64 / 4);                             // staged blocks per 64 x 64 state tile
    static_assert(2 * NBLK <= DBDC_THREADS, "one staged block per thread");
    __shared__ __attribute__((aligned(16))) T sF[NBUF][64 * LDX];
    __shared__ __attribute__((aligned(16))) T sB[NBUF][64 * LDX];
    __shared__ float sfs[DBDC_HEADS][ROWS], sbs[DBDC_HEADS][ROWS];         // row scales of the heads of this slice
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    // blockIdx.x = (b, c, g) varies fastest: consecutive workgroups are dealt round-robin to the 8 XCDs, so the row
    // tiles of one (b, c, g), which read the same states, land on the same XCD and share its L2
    const int rt = blockIdx.y;
    const int g = blockIdx.x % p.ngroups, bc = blockIdx.x / p.ngroups, c = bc % nc, b = bc / nc;
    const int Q = p.chunk_size, N = p.dstate, P = p.headdim, H = p.nheads, hpg = H / p.ngroups;
    const int limit = min(Q, p.seqlen - c * Q);
    const int r0 = rt * ROWS;
    // blockIdx.z selects a slice of DBDC_HEADS heads of the group; its partial sum goes to slice blockIdx.z of the
    // output, and bmm_chunk_bwd adds the slices up
    const int hh0 = blockIdx.z * DBDC_HEADS, hh_end = min(hpg, hh0 + DBDC_HEADS);
    const int nkc = (P + KC - 1) / KC, nnt = (N + 63) / 64;
    const int per_head = nnt * nkc, nsteps = (hh_end - hh0) * per_head;

    // ---- software pipeline, stage 1: requests for a step (state blocks of two tiles, A fragments) ----
    Vec16<float> sreg[VK];                                                 // one VK x 4 block of a state tile
    typename M::Frag af[QT][NKS];
    int arow[QT];                                                          // this lane's A-operand rows
#pragma unroll
    for (int q = 0; q < QT; ++q) arow[q] = min(r0 + (wave * QT + q) * 16 + lr, limit - 1);
    const int sblk = threadIdx.x % NBLK, stile = threadIdx.x / NBLK;       // stile 0: forward state, 1: reverse state
    const int s_rb = sblk % 16, s_kb = sblk / 16;
    auto request = [&](int step) __attribute__((always_inline)) {
        const int hh = hh0 + step / per_head, rem = step % per_head, nt = rem / nkc, kc = rem % nkc;
        const int h = g * hpg + hh;
        if (stile < (UNI ? 1 : 2)) {
            const int64_t so = ((int64_t)(b * nc + c) * H + h) * P * N;
            const float *st = (IS_DB ? (stile ? p.dstates_b : p.dstates_f) : (stile ? p.states_b : p.states_f)) + so;
#pragma unroll
            for (int kk = 0; kk < VK; ++kk) {
                const int pp = kc * KC + s_kb * VK + kk, n = nt * 64 + s_rb * 4;
                if (FAST) sreg[kk] = *reinterpret_cast<const Vec16<float> *>(st + (int64_t)pp * N + n);
                else
#pragma unroll
                    for (int i = 0; i < 4; ++i) sreg[kk].v[i] = (pp < P && n + i < N) ? st[(int64_t)pp * N + n + i] : 0.f;
            }
        }
        const T *ap;
        int64_t as;
        if (IS_DB) { as = p.x_sl; ap = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * as + h * p.x_sh; }
        else if (p.has_z) { as = (int64_t)H * P; ap = reinterpret_cast<const T *>(p.dout_x) + ((int64_t)b * p.seqlen + (int64_t)c * Q) * as + (int64_t)h * P; }
        else { as = p.dout_sl; ap = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * as + h * p.dout_sh; }
#pragma unroll
        for (int q = 0; q < QT; ++q)
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const int kb = kc * KC + ks * KSTEP + lg * KPL;
                const T *row = ap + (int64_t)arow[q] * as;
                if (FAST) af[q][ks] = M::load(row + kb);
                else {
                    float v[KPL];
#pragma unroll
                    for (int i = 0; i < KPL; ++i) v[i] = kb + i < P ? to_f(row[kb + i]) : 0.f;
                    af[q][ks] = M::pack(v);
                }
            }
    };
    // stage 2: the requested state block goes, transposed, into the LDS image (r = n, k = p)
    auto commit = [&](int buf) __attribute__((always_inline)) {
        if (stile < (UNI ? 1 : 2)) {
            T *dst = stile ? sB[buf] : sF[buf];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                Vec16<T> o;
#pragma unroll
                for (int kk = 0; kk < VK; ++kk) o.v[kk] = from_f<T>(sreg[kk].v[rr]);
                *reinterpret_cast<Vec16<T> *>(dst + xt_index<T, LDX>(s_rb * 4 + rr, s_kb * VK)) = o;
            }
        }
    };
    request(0);

    int tl[QT][4];                                                         // rows of this lane's accumulator elements
#pragma unroll
    for (int q = 0; q < QT; ++q)
#pragma unroll
        for (int i = 0; i < 4; ++i) tl[q][i] = (wave * QT + q) * 16 + lg * 4 + i;
    // row scales of every head of the slice
    for (int idx = threadIdx.x; idx < (hh_end - hh0) * ROWS; idx += DBDC_THREADS) {
        const int hh = idx / ROWS, rl = idx % ROWS, r = r0 + rl;
        const int64_t o = (((int64_t)b * H + g * hpg + hh0 + hh) * nc + c) * Q;
        float f = 0.f, rv = 0.f;
        if (r < limit) {
            if (IS_DB) {
                const float d = p.dt_out[o + r];
                f = d * __expf(p.cs_f[o + Q - 1] - p.cs_f[o + r]);
                rv = UNI ? 0.f : d * __expf(p.cs_b[o] - p.cs_b[o + r]);
            } else {
                f = __expf(p.cs_f[o + r]);
                rv = UNI ? 0.f : __expf(p.cs_b[o + r]);
            }
        }
        sfs[hh][rl] = f;
        sbs[hh][rl] = rv;
    }
    // B or C values of this lane's output elements
    const T *cbp;
    int64_t cbs;
    if (IS_DB) { cbs = p.B_sl; cbp = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + ((int64_t)c * Q + r0) * cbs + g * p.B_sg; }
    else { cbs = p.C_sl; cbp = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + ((int64_t)c * Q + r0) * cbs + g * p.C_sg; }
    float creg[NT][QT][4][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int q = 0; q < QT; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // unconditional loads from clamped addresses (conditional ones are waited for one by one), masked after
                    const int n = nt * 64 + j * 16 + lr;
                    const float v = to_f(cbp[(int64_t)min(tl[q][i], limit - 1 - r0) * cbs + min(n, N - 1)]);
                    creg[nt][q][j][i] = (r0 + tl[q][i] < limit && n < N) ? v : 0.f;
                }
    f32x4 tot[NT][QT][4] = {};

    int step = 0;
    for (int hh = hh0; hh < hh_end; ++hh) {
        const int h = g * hpg + hh;
        const int64_t o = (((int64_t)b * H + h) * nc + c) * Q;
        float uf[QT][4], ub[QT][4];
#pragma unroll
        for (int q = 0; q < QT; ++q)
#pragma unroll
            for (int i = 0; i < 4; ++i) { uf[q][i] = 0.f; ub[q][i] = 0.f; }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            if (nt >= nnt) break;
            f32x4 tf[QT][4] = {}, tb[QT][4] = {};
            for (int kc = 0; kc < nkc; ++kc, ++step) {
                const int buf = NBUF == 2 ? (step & 1) : 0;
                if (NBUF == 1) __syncthreads();            // the single image is still being read by slower waves
                commit(buf);
                typename M::Frag afc[QT][NKS];
#pragma unroll
                for (int q = 0; q < QT; ++q)
#pragma unroll
                    for (int ks = 0; ks < NKS; ++ks) afc[q][ks] = af[q][ks];
                __syncthreads();
                if (step + 1 < nsteps) request(step + 1);  // in flight while this step is multiplied
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    const int kq = ks * KSTEP + lg * KPL;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const typename M::Frag bff = M::load(sF[buf] + xt_index<T, LDX>(j * 16 + lr, kq));
                        const typename M::Frag bfb = UNI ? bff : M::load(sB[buf] + xt_index<T, LDX>(j * 16 + lr, kq));
#pragma unroll
                        for (int q = 0; q < QT; ++q) {
                            tf[q][j] = M::mma(afc[q][ks], bff, tf[q][j]);
                            if (!UNI) tb[q][j] = M::mma(afc[q][ks], bfb, tb[q][j]);
                        }
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < QT; ++q)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float sf = sfs[hh - hh0][tl[q][i]], sb = sbs[hh - hh0][tl[q][i]];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        uf[q][i] += tf[q][j][i] * creg[nt][q][j][i];
                        ub[q][i] += tb[q][j][i] * creg[nt][q][j][i];
                        tot[nt][q][j][i] += sf * tf[q][j][i] + sb * tb[q][j][i];
                    }
                }
        }
        float *of = IS_DB ? p.v_f : p.u_f, *ob = IS_DB ? p.v_b : p.u_b;
#pragma unroll
        for (int q = 0; q < QT; ++q)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float a = row16_sum(uf[q][i]) * sfs[hh - hh0][tl[q][i]], bb = row16_sum(ub[q][i]) * sbs[hh - hh0][tl[q][i]];
                if (lr == 0 && r0 + tl[q][i] < Q) {
                    of[o + r0 + tl[q][i]] = a;
                    if (!UNI) ob[o + r0 + tl[q][i]] = bb;
                }
            }
    }
    float *out = (IS_DB ? p.dBs : p.dCs) + (int64_t)blockIdx.z * p.batch * p.seqlen * p.ngroups * N;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int q = 0; q < QT; ++q)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int n = nt * 64 + j * 16 + lr, r = r0 + tl[q][i];
                    if (r < limit && n < N)
                        out[(((int64_t)b * p.seqlen + (int64_t)c * Q + r) * p.ngroups + g) * N + n] = tot[nt][q][j][i];
                }
}

// ---------------------------------------------------------------------------------------------------------
// The same for 16-bit types with dstate 64 and headdim % 64 == 0, with every load of the head loop taken out of the
// compiler's hands.  The workgroup is alone on its CU (register-bound), so nothing hides a load it waits for; here the
// float32 state tiles of a step travel straight into a 3-slot LDS ring (no registers), two steps ahead of their use, and
// the x / dout fragments into registers, likewise two steps ahead, from inline assembly.  A step then reads its tiles
// from the ring, transposes them in registers into the 16-bit operand image as before, and multiplies.  All LDS traffic
// of the loop goes through the raw accessors (an access the compiler knows of would wait for every request in flight).
// Order of a wave's vector memory operations per step: NDIR * 2 ring requests, then QT * 2 fragment loads; "at most one
// step's worth outstanding" therefore means that the step in hand has landed.
// ---------------------------------------------------------------------------------------------------------
// S16: the state tiles come from their 16-bit copies (states16_* / dstates16_*).  They lie in the ring as they lie in
// memory ([p][n], 16-byte chunks swizzled as tile64_request does), and the operand fragments are LDS transpose reads
// straight from the ring slot: no operand image, one barrier per step, a third of the LDS.
template <typename T, int QT, bool IS_DB, bool UNI, bool S16>
__global__ __launch_bounds__(DBDC_THREADS) void bwd_dbdc_dma_kernel(const bimamba2_params p, int nc) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    static_assert(sizeof(T) == 2, "16-bit operands");
    constexpr int KSTEP = 32, KC = 64, NKS = 2, VK = 8, LDX = KC + VK;
    constexpr int ROWS = DBDC_WAVES * 16 * QT;
    constexpr int NBLK = (KC / VK) * 16;                       // 8 x 4 blocks of a 64 x 64 tile
    constexpr int RING = 3, NDIR = UNI ? 1 : 2;
    constexpr int TILE_B = 64 * 64 * (S16 ? 2 : 4);            // bytes of a state tile
    constexpr int IMG_B = 64 * LDX * 2;                        // bytes of a 16-bit operand image
    constexpr int PER_STEP = NDIR * (S16 ? 1 : 2) + QT * NKS;  // vector memory operations of a wave per step
    static_assert(NDIR * NBLK <= DBDC_THREADS, "one block per thread");
    static_assert(DBDC_WAVES == 8, "a wave brings 8 (16-bit) resp. 2 x 4 (float32) rows of each tile");
    __shared__ __attribute__((aligned(16))) unsigned char ring[RING * NDIR * TILE_B];
    __shared__ __attribute__((aligned(16))) unsigned char img[S16 ? 16 : 2 * NDIR * IMG_B];
    __shared__ __attribute__((aligned(16))) float sfs[DBDC_HEADS][ROWS], sbs[DBDC_HEADS][ROWS];
    // the per-head decay gradients wait here for the end of the kernel: a global store inside the loop would sit in the
    // same counter as the requests and be waited for with them
    __shared__ __attribute__((aligned(16))) float uvs[DBDC_HEADS][NDIR][ROWS];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    const int rt = blockIdx.y;
    const int g = blockIdx.x % p.ngroups, bc = blockIdx.x / p.ngroups, c = bc % nc, b = bc / nc;
    const int Q = p.chunk_size, N = p.dstate, P = p.headdim, H = p.nheads, hpg = H / p.ngroups;
    const int limit = min(Q, p.seqlen - c * Q);
    const int r0 = rt * ROWS;
    const int hh0 = blockIdx.z * DBDC_HEADS, hh_end = min(hpg, hh0 + DBDC_HEADS);
    const int nkc = P / KC, nsteps = (hh_end - hh0) * nkc;
    int arow[QT];
#pragma unroll
    for (int q = 0; q < QT; ++q) arow[q] = min(r0 + (wave * QT + q) * 16 + lr, limit - 1);

    // requests of a step: this wave's two 4-row units of each state tile, then its fragments
    auto issue_states = [&](int step) {
        const int hh = hh0 + step / nkc, kc = step % nkc, h = g * hpg + hh;
        const int64_t so = ((int64_t)(b * nc + c) * H + h) * P * N + (int64_t)kc * KC * N;
#pragma unroll
        for (int d = 0; d < NDIR; ++d) {
            if constexpr (S16) {
                // rows 8 wave .. 8 wave + 7, 16-byte chunk (lane % 8) ^ swizzle(row) at chunk position lane % 8
                const T *st = reinterpret_cast<const T *>(IS_DB ? (d ? p.dstates16_b : p.dstates16_f) : (d ? p.states16_b : p.states16_f)) + so;
                const int row = wave * 8 + (lane >> 3);
                load16_to_lds(st + row * 64 + (((lane & 7) ^ tile64_swz(row)) << 3), ring + ((step % RING) * NDIR + d) * TILE_B + wave * 1024);
            } else {
                const float *st = (IS_DB ? (d ? p.dstates_b : p.dstates_f) : (d ? p.states_b : p.states_f)) + so;
#pragma unroll
                for (int uu = 0; uu < 2; ++uu) {
                    const int u = wave * 2 + uu;
                    load16_to_lds(st + (4 * u + (lane >> 4)) * 64 + (lane & 15) * 4, ring + ((step % RING) * NDIR + d) * TILE_B + u * 1024);
                }
            }
        }
    };
    auto issue_frags = [&](int step, Frag (&af)[QT][NKS]) {
        const int hh = hh0 + step / nkc, kc = step % nkc, h = g * hpg + hh;
        const T *ap;
        int64_t as;
        if (IS_DB) { as = p.x_sl; ap = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * as + h * p.x_sh; }
        else if (p.has_z) { as = (int64_t)H * P; ap = reinterpret_cast<const T *>(p.dout_x) + ((int64_t)b * p.seqlen + (int64_t)c * Q) * as + (int64_t)h * P; }
        else { as = p.dout_sl; ap = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * as + h * p.dout_sh; }
#pragma unroll
        for (int q = 0; q < QT; ++q)
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) af[q][ks] = raw_global_load_b128<Frag>(ap + (int64_t)arow[q] * as + kc * KC + ks * KSTEP + lg * 8);
    };
    Frag afA[QT][NKS], afB[QT][NKS];                           // fragments of the even / odd steps
    issue_states(0);
    issue_frags(0, afA);
    if (nsteps > 1) { issue_states(1); issue_frags(1, afB); }

    // ---- everything below up to the loop is ordinary code; its waits drain the requests above, which costs nothing here ----
    int tl[QT][4];
#pragma unroll
    for (int q = 0; q < QT; ++q)
#pragma unroll
        for (int i = 0; i < 4; ++i) tl[q][i] = (wave * QT + q) * 16 + lg * 4 + i;
    // one round trip for everything the loop needs besides its requests: the decay vectors of the slice's heads and the
    // B / C values of this lane's output elements, all loaded unconditionally from clamped addresses before the first use
    constexpr int NTAB = DBDC_HEADS * ROWS / DBDC_THREADS;
    static_assert(NTAB * DBDC_THREADS == DBDC_HEADS * ROWS, "table entries per thread");
    float t_dt[NTAB], t_cf[NTAB], t_cb[NTAB], t_ef[NTAB], t_eb[NTAB];
#pragma unroll
    for (int it = 0; it < NTAB; ++it) {
        const int idx = threadIdx.x + it * DBDC_THREADS;
        const int hh = min(idx / ROWS, hh_end - hh0 - 1), r = min(r0 + idx % ROWS, limit - 1);
        const int64_t o = (((int64_t)b * H + g * hpg + hh0 + hh) * nc + c) * Q;
        t_cf[it] = p.cs_f[o + r];
        t_cb[it] = UNI ? 0.f : p.cs_b[o + r];
        t_dt[it] = IS_DB ? p.dt_out[o + r] : 0.f;
        t_ef[it] = IS_DB ? p.cs_f[o + Q - 1] : 0.f;
        t_eb[it] = (IS_DB && !UNI) ? p.cs_b[o] : 0.f;
    }
    const T *cbp;
    int64_t cbs;
    if (IS_DB) { cbs = p.B_sl; cbp = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + ((int64_t)c * Q + r0) * cbs + g * p.B_sg; }
    else { cbs = p.C_sl; cbp = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + ((int64_t)c * Q + r0) * cbs + g * p.C_sg; }
    float creg[QT][4][4];
#pragma unroll
    for (int q = 0; q < QT; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) creg[q][j][i] = to_f(cbp[(int64_t)min(tl[q][i], limit - 1 - r0) * cbs + j * 16 + lr]);
#pragma unroll
    for (int q = 0; q < QT; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (r0 + tl[q][i] >= limit) creg[q][j][i] = 0.f;
#pragma unroll
    for (int it = 0; it < NTAB; ++it) {
        const int idx = threadIdx.x + it * DBDC_THREADS;
        const int hh = idx / ROWS, rl = idx % ROWS;
        if (hh < hh_end - hh0) {
            float f = 0.f, rv = 0.f;
            if (r0 + rl < limit) {
                if (IS_DB) {
                    f = t_dt[it] * __expf(t_ef[it] - t_cf[it]);
                    rv = UNI ? 0.f : t_dt[it] * __expf(t_eb[it] - t_cb[it]);
                } else {
                    f = __expf(t_cf[it]);
                    rv = UNI ? 0.f : __expf(t_cb[it]);
                }
            }
            sfs[hh][rl] = f;
            sbs[hh][rl] = rv;
        }
    }
    f32x4 tot[QT][4] = {};
    __syncthreads();

    // ---- the head loop: raw LDS accesses and counted waits only ----
    const int sblk = threadIdx.x % NBLK, stile = threadIdx.x / NBLK;       // staging: tile stile, block (s_kb, s_rb)
    const int s_rb = sblk % 16, s_kb = sblk / 16;
    const unsigned ring_a = lds_addr(ring) + stile * TILE_B + (s_kb * VK) * 256 + s_rb * 16;
    const unsigned img_w = lds_addr(img) + stile * IMG_B;
    unsigned img_wo[4];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) img_wo[rr] = img_w + xt_index<T, LDX>(s_rb * 4 + rr, s_kb * VK) * 2;
    unsigned img_r[NKS][4];                                    // operand fragments of this lane (the swizzle depends on the row block)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
        for (int j = 0; j < 4; ++j) img_r[ks][j] = lds_addr(img) + xt_index<T, LDX>(j * 16 + lr, ks * KSTEP + lg * 8) * 2;
    const unsigned sfs_a = lds_addr(sfs) + ((wave * QT) * 16 + lg * 4) * 4, sbs_a = lds_addr(sbs) + ((wave * QT) * 16 + lg * 4) * 4;
    const unsigned uvs_a = lds_addr(uvs) + ((wave * QT) * 16 + lg * 4) * 4;
    // S16: lane parts of the transpose reads (see tile64_tr_frag): rows kk .. kk + 3 and kk + 4 .. kk + 7 of a K step,
    // 4 columns from 16 j + nn on; the K step adds 32 rows = 4096 bytes (the swizzle repeats every 16 rows)
    unsigned tr_lo[4], tr_hi[4];
    {
        const int kk = 8 * lg + (lr >> 2), nn = 4 * (lr & 3);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            tr_lo[j] = lds_addr(ring) + tile64_tr_offset(kk, j * 16 + nn);
            tr_hi[j] = lds_addr(ring) + tile64_tr_offset(kk + 4, j * 16 + nn);
        }
    }
    f32x4 tf[QT][4], tb[QT][4];
    // SLOT = step % RING as a compile-time value: the slot's offset goes into the offset field of the LDS reads
    auto step_body = [&](int step, Frag (&af)[QT][NKS], auto SLOT) {
        constexpr int RB = decltype(SLOT)::value * NDIR * TILE_B;
        const int hh = hh0 + step / nkc, kc = step % nkc;
        // this wave's requests of the step have landed (those of the next step may be outstanding) ...
        if (step + 1 < nsteps) wait_vmcnt<PER_STEP>();
        else wait_vmcnt<0>();
        raw_lds_barrier();                                     // ... and everybody's; ring slot and image of step - 1 are free
        if (step + 2 < nsteps) issue_states(step + 2);
        const int buf = step & 1;
        if constexpr (!S16) {
        if (stile < NDIR) {
            // 8 rows (k = p) x 4 columns (n) of the tile from the ring, transposed into the image
            const unsigned ra = ring_a + ((step % RING) * NDIR) * TILE_B;
            f32x4 v[VK];
            v[0] = raw_lds_read_at<f32x4, 0>(ra); v[1] = raw_lds_read_at<f32x4, 256>(ra);
            v[2] = raw_lds_read_at<f32x4, 512>(ra); v[3] = raw_lds_read_at<f32x4, 768>(ra);
            v[4] = raw_lds_read_at<f32x4, 1024>(ra); v[5] = raw_lds_read_at<f32x4, 1280>(ra);
            v[6] = raw_lds_read_at<f32x4, 1536>(ra); v[7] = raw_lds_read_at<f32x4, 1792>(ra);
            raw_lds_wait();
#pragma unroll
            for (int kk = 0; kk < VK; ++kk) raw_lds_use(v[kk]);
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                Vec16<T> o;
#pragma unroll
                for (int kk = 0; kk < VK; ++kk) o.v[kk] = from_f<T>(v[kk][rr]);
                raw_lds_write128_at<0>(img_wo[rr] + buf * NDIR * IMG_B, __builtin_bit_cast(f32x4, o));
            }
        }
        raw_lds_wait();
        raw_lds_barrier();
        }
        // (the first products of a head start from a literal zero: no registers to clear between heads)
        const bool first = kc == 0;
#pragma unroll
        for (int q = 0; q < QT; ++q)
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) raw_lds_use(af[q][ks]);
        const unsigned ib = buf * NDIR * IMG_B;
        if constexpr (S16) {
            // both K halves' fragments are asked for at once; the products of the first half run while the second half's
            // reads are still under way (LDS reads return in order: "at most NR outstanding" = the first half is there)
            static_assert(NKS == 2, "two K halves");
            constexpr int NR = UNI ? 8 : 16;                   // LDS reads per K half
            i16x4 flo[NKS][4], fhi[NKS][4], blo[NKS][4], bhi[NKS][4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                flo[0][j] = raw_lds_tr16_read_at<RB>(tr_lo[j]); fhi[0][j] = raw_lds_tr16_read_at<RB>(tr_hi[j]);
                if (!UNI) { blo[0][j] = raw_lds_tr16_read_at<RB + TILE_B>(tr_lo[j]); bhi[0][j] = raw_lds_tr16_read_at<RB + TILE_B>(tr_hi[j]); }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                flo[1][j] = raw_lds_tr16_read_at<RB + 4096>(tr_lo[j]); fhi[1][j] = raw_lds_tr16_read_at<RB + 4096>(tr_hi[j]);
                if (!UNI) { blo[1][j] = raw_lds_tr16_read_at<RB + TILE_B + 4096>(tr_lo[j]); bhi[1][j] = raw_lds_tr16_read_at<RB + TILE_B + 4096>(tr_hi[j]); }
            }
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                // lgkmcnt(min(NR, 15)), vmcnt and expcnt left alone (the counter has four bits: 15 is its largest value)
                if (ks == 0) __builtin_amdgcn_s_waitcnt(0xC07F | ((NR < 15 ? NR : 15) << 8));
                else raw_lds_wait();
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    raw_lds_use(flo[ks][j]); raw_lds_use(fhi[ks][j]);
                    const Frag bff = __builtin_bit_cast(Frag, __builtin_shufflevector(flo[ks][j], fhi[ks][j], 0, 1, 2, 3, 4, 5, 6, 7));
                    Frag bfb = bff;
                    if (!UNI) {
                        raw_lds_use(blo[ks][j]); raw_lds_use(bhi[ks][j]);
                        bfb = __builtin_bit_cast(Frag, __builtin_shufflevector(blo[ks][j], bhi[ks][j], 0, 1, 2, 3, 4, 5, 6, 7));
                    }
#pragma unroll
                    for (int q = 0; q < QT; ++q) {
                        if (ks == 0 && first) {
                            tf[q][j] = M::mma(af[q][ks], bff, f32x4{0.f, 0.f, 0.f, 0.f});
                            if (!UNI) tb[q][j] = M::mma(af[q][ks], bfb, f32x4{0.f, 0.f, 0.f, 0.f});
                        } else {
                            tf[q][j] = M::mma(af[q][ks], bff, tf[q][j]);
                            if (!UNI) tb[q][j] = M::mma(af[q][ks], bfb, tb[q][j]);
                        }
                    }
                }
            }
        } else {
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            Frag bff[4], bfb[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bff[j] = raw_lds_read_at<Frag, 0>(img_r[ks][j] + ib);
                if (!UNI) bfb[j] = raw_lds_read_at<Frag, IMG_B>(img_r[ks][j] + ib);
            }
            raw_lds_wait();
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                raw_lds_use(bff[j]);
                if (!UNI) raw_lds_use(bfb[j]);
#pragma unroll
                for (int q = 0; q < QT; ++q) {
                    if (ks == 0 && first) {
                        tf[q][j] = M::mma(af[q][ks], bff[j], f32x4{0.f, 0.f, 0.f, 0.f});
                        if (!UNI) tb[q][j] = M::mma(af[q][ks], bfb[j], f32x4{0.f, 0.f, 0.f, 0.f});
                    } else {
                        tf[q][j] = M::mma(af[q][ks], bff[j], tf[q][j]);
                        if (!UNI) tb[q][j] = M::mma(af[q][ks], bfb[j], tb[q][j]);
                    }
                }
            }
        }
        }
        // the fragments of step + 2 take the place of the ones just used
        if (step + 2 < nsteps) issue_frags(step + 2, af);
        if (kc == nkc - 1) {
            // ---- end of a head: its share of dB / dC and of the decay gradients
#pragma unroll
            for (int q = 0; q < QT; ++q) {
                f32x4 sf4 = raw_lds_read_at<f32x4, 0>(sfs_a + ((hh - hh0) * ROWS + q * 16) * 4);
                f32x4 sb4 = raw_lds_read_at<f32x4, 0>(sbs_a + ((hh - hh0) * ROWS + q * 16) * 4);
                raw_lds_wait();
                raw_lds_use(sf4); raw_lds_use(sb4);
                f32x4 av, bv;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float uf = 0.f, ub = 0.f;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        uf += tf[q][j][i] * creg[q][j][i];
                        if (!UNI) ub += tb[q][j][i] * creg[q][j][i];
                        tot[q][j][i] += UNI ? sf4[i] * tf[q][j][i] : sf4[i] * tf[q][j][i] + sb4[i] * tb[q][j][i];
                    }
                    av[i] = row16_sum(uf) * sf4[i];
                    bv[i] = UNI ? 0.f : row16_sum(ub) * sb4[i];
                }
                if (lr == 0) {
                    const unsigned ua = uvs_a + (((hh - hh0) * NDIR) * ROWS + q * 16) * 4;
                    raw_lds_write128_at<0>(ua, av);
                    if (!UNI) raw_lds_write128_at<ROWS * 4>(ua, bv);
                }
            }
        }
    };
    static_assert(RING == 3, "six steps = one round of ring slots and of the two fragment sets");
    for (int step = 0; step < nsteps; step += 6) {
        step_body(step, afA, std::integral_constant<int, 0>());
        if (step + 1 < nsteps) step_body(step + 1, afB, std::integral_constant<int, 1>());
        if (step + 2 < nsteps) step_body(step + 2, afA, std::integral_constant<int, 2>());
        if (step + 3 < nsteps) step_body(step + 3, afB, std::integral_constant<int, 0>());
        if (step + 4 < nsteps) step_body(step + 4, afA, std::integral_constant<int, 1>());
        if (step + 5 < nsteps) step_body(step + 5, afB, std::integral_constant<int, 2>());
    }
    raw_lds_wait();
    __syncthreads();                                           // nothing is in flight any more: ordinary code again
    for (int idx = threadIdx.x; idx < (hh_end - hh0) * NDIR * ROWS; idx += DBDC_THREADS) {
        const int hh = idx / (NDIR * ROWS), d = (idx / ROWS) % NDIR, rl = idx % ROWS;
        if (r0 + rl < Q) {
            float *dst = IS_DB ? (d ? p.v_b : p.v_f) : (d ? p.u_b : p.u_f);
            dst[(((int64_t)b * H + g * hpg + hh0 + hh) * nc + c) * Q + r0 + rl] = uvs[hh][d][rl];
        }
    }
    float *out = (IS_DB ? p.dBs : p.dCs) + (int64_t)blockIdx.z * p.batch * p.seqlen * p.ngroups * N;
#pragma unroll
    for (int q = 0; q < QT; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = j * 16 + lr, r = r0 + tl[q][i];
                if (r < limit) out[(((int64_t)b * p.seqlen + (int64_t)c * Q + r) * p.ngroups + g) * N + n] = tot[q][j][i];
            }
}

template <typename T, bool IS_DB>
static int launch_dbdc_t(const bimamba2_params *p) {
    const int nc = nchunks(p);
    const int nt = (p->dstate + 63) / 64;
    int qt = (p->chunk_size > 128 && nt == 1) ? 2 : 1;                // 16-row tiles per wave
    const int rows = DBDC_WAVES * 16 * qt;
    dim3 grid(p->batch * nc * p->ngroups, (p->chunk_size + rows - 1) / rows, dbdc_slices(p));
    constexpr int VS = 16 / (int)sizeof(T);
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    bool fast = p->headdim % 64 == 0 && p->dstate % 64 == 0;
    if (IS_DB) fast = fast && al(p->x) && p->x_sb % VS == 0 && p->x_sl % VS == 0 && p->x_sh % VS == 0;
    else fast = fast && (p->has_z ? al(p->dout_x) : (al(p->dout) && p->dout_sb % VS == 0 && p->dout_sl % VS == 0 && p->dout_sh % VS == 0));
#define BM2_DBDC(NTV, QTV)                                                                                                    \
    do {                                                                                                                  \
        if (fast) hipLaunchKernelGGL((bwd_dbdc_kernel<T, NTV, QTV, IS_DB, true>), grid, dim3(DBDC_THREADS), 0, stream_of(p), *p, nc); \
        else hipLaunchKernelGGL((bwd_dbdc_kernel<T, NTV, QTV, IS_DB, false>), grid, dim3(DBDC_THREADS), 0, stream_of(p), *p, nc);     \
    } while (0)
    if constexpr (sizeof(T) == 2) {
        // dstate 64: the variant with the ring of state tiles (16-byte aligned state tensors)
        const void *c16f = IS_DB ? p->dstates16_f : p->states16_f, *c16b = IS_DB ? p->dstates16_b : p->states16_b;
        const bool st_al = c16f ? al(c16f) && al(c16b) && (p->causal || c16b)
                                : (IS_DB ? al(p->dstates_f) && al(p->dstates_b) : al(p->states_f) && al(p->states_b));
        if (fast && p->dstate == 64 && st_al) {
            // 128-row tiles here: with eight heads per slice that is still one workgroup per CU at the usual sizes, and
            // the partial sums the slices leave behind (and bmm_chunk_bwd reads again) are half of what four heads give
            qt = 1;
            grid.y = (p->chunk_size + DBDC_WAVES * 16 - 1) / (DBDC_WAVES * 16);
#define BM2_DMA(QTV, UNIV)                                                                                                                  \
    do {                                                                                                                                    \
        if (c16f) hipLaunchKernelGGL((bwd_dbdc_dma_kernel<T, QTV, IS_DB, UNIV, true>), grid, dim3(DBDC_THREADS), 0, stream_of(p), *p, nc);   \
        else hipLaunchKernelGGL((bwd_dbdc_dma_kernel<T, QTV, IS_DB, UNIV, false>), grid, dim3(DBDC_THREADS), 0, stream_of(p), *p, nc);       \
    } while (0)
            if (p->causal) { BM2_DMA(1, true); }
            else { BM2_DMA(1, false); }
#undef BM2_DMA
            return check_launch();
        }
    }
    if (IS_DB ? p->dstates16_f : p->states16_f) return BIMAMBA2_EUNSUPPORTED;   // only the kernel above knows the 16-bit copies
    if (p->causal) {
        if constexpr (sizeof(T) == 2) {
            if (fast && nt == 1) {
                if (qt == 2) hipLaunchKernelGGL((bwd_dbdc_kernel<T, 1, 2, IS_DB, true, true>), grid, dim3(DBDC_THREADS), 0, stream_of(p), *p, nc);
                else hipLaunchKernelGGL((bwd_dbdc_kernel<T, 1, 1, IS_DB, true, true>), grid, dim3(DBDC_THREADS), 0, stream_of(p), *p, nc);
                return check_launch();
            }
        }
        return BIMAMBA2_EUNSUPPORTED;
    }
    if (nt == 1 && qt == 2) BM2_DBDC(1, 2);
    else if (nt == 1) BM2_DBDC(1, 1);
    else if (nt == 2) BM2_DBDC(2, 1);
    else if (nt <= 4) BM2_DBDC(4, 1);
    else return BIMAMBA2_EUNSUPPORTED;
#undef BM2_DBDC
    return check_launch();
}

int launch_bwd_dbdc(const bimamba2_params *p, bool is_db) {
    switch (p->dtype) {
        case BIMAMBA2_F32: return is_db ? launch_dbdc_t<float, true>(p) : launch_dbdc_t<float, false>(p);
        case BIMAMBA2_BF16: return is_db ? launch_dbdc_t<bf16_t, true>(p) : launch_dbdc_t<bf16_t, false>(p);
        case BIMAMBA2_F16: return is_db ? launch_dbdc_t<f16_t, true>(p) : launch_dbdc_t<f16_t, false>(p);
        default: return BIMAMBA2_EUNSUPPORTED;
    }
}

// =========================================================================================================
// One workgroup owns one 64x64 tile (tt, st) of the chunk's (t, s) plane for one (b, c, g) and loops over the
// heads of the group; wave w owns rows 16w..16w+15 of the tile.  Per head, G[t,s] = dy_h[t,:] . x_h[s,:]
// (K = headdim; both operands are read from global memory straight into MFMA operand registers, the next
// K chunk being requested while the current one is multiplied), then
//   f[t,s] = 1[s<=t] G dt[s] e^{cs_f[t]-cs_f[s]},  b[t,s] = 1[s>=t] G dt[s] e^{cs_b[t]-cs_b[s]}
//   dCB[t,s] = sum_{h in group} (f + b)                       (kept in registers across the head loop)
//   W_f = 1[s<t] f CB,  W_b = 1[s>t] b CB                     (what the within-chunk gradient of dt*A is made of)
// The within-chunk gradient  da[i] = sum_{t>=i>s} W_f[t,s] + sum_{t<=i<s} W_b[t,s]  is assembled by the consumer
// (chunk_cumsum_bwd) from per-tile vectors written here to da_intra[b, h, c, tile, 2, 64]:
//   off-diagonal tile: [0] = column sums cw[s] = sum_t W,  [1] = row sums rw[t] = sum_s W
//   diagonal tile    : [0] = cw_f - rw_f, [1] = cw_b - rw_b of the tile's own W_f, W_b; the tile's contribution
//                      to da[i] is the exclusive prefix sum of [0] plus the exclusive suffix sum of [1]
//                      (da[i+1] - da[i] = cw_f[i] - rw_f[i] inside a tile; at most 64 terms, so the cancellation
//                      stays at float32 rounding level)
// One barrier per head (to combine the four waves' column sums); the decay vectors of up to DCB_HEADS heads are
// put into LDS beforehand.
// =========================================================================================================
constexpr int DCB_HEADS = 32;
constexpr int DCB_SLICE_HEADS = 32;     // heads per slice
constexpr int DCB_SLICES_MAX = 4;
constexpr int DCB_VEC = 2 * 64;      // floats per tile and head in da_intra

// Per head: turns the G tile (acc) into this head's share of dCB (added to dcb) and into the column / row sums of W that
// chunk_cumsum_bwd assembles.  cs = {cs_f[t], cs_b[t], cs_f[s], cs_b[s], dt[s]} of the tile (LDS), pb = exchange buffer
// of the four waves (LDS), tv = the (tile, head) slot of da_intra.  Contains one workgroup barrier.
template <typename T>
__device__ __forceinline__ void dcb_finish_head(f32x4 (&acc)[4], f32x4 (&dcb)[4], const f32x4 (&cbr)[4], const float (*cs)[64],
                                                float (*pb)[64], float *tv, const int (&tl)[4], int st, int tt) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lr = lane & 15;
    float cft[4], cbt[4], dtv[4], cfs[4], cbs[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        cft[i] = cs[0][tl[i]];
        cbt[i] = cs[1][tl[i]];
        cfs[i] = cs[2][i * 16 + lr];
        cbs[i] = cs[3][i * 16 + lr];
        dtv[i] = cs[4][i * 16 + lr];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
    }
    // column sums (this wave's 16 rows) and row sums of W; on the diagonal tile one pair per direction
    float cwa[4], cwb[4], rwa[4] = {0.f, 0.f, 0.f, 0.f}, rwb[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int sl = j * 16 + lr;
        float ca = 0.f, cb2 = 0.f;
        if (st != tt) {
            // one direction only: forward below the diagonal, reverse above it
            const float csv = st < tt ? cfs[j] : cbs[j];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float v = acc[j][i] * dtv[j] * __expf((st < tt ? cft[i] : cbt[i]) - csv);
                dcb[j][i] += v;
                const float w = v * cbr[j][i];
                ca += w;
                rwa[i] += w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float gv = acc[j][i] * dtv[j];
                const float f = (sl <= tl[i]) ? gv * __expf(cft[i] - cfs[j]) : 0.f;
                const float r = (sl >= tl[i]) ? gv * __expf(cbt[i] - cbs[j]) : 0.f;
                dcb[j][i] += f + r;
                const float wf = (sl < tl[i]) ? f * cbr[j][i] : 0.f;
                const float wb = (sl > tl[i]) ? r * cbr[j][i] : 0.f;
                ca += wf; rwa[i] += wf;
                cb2 += wb; rwb[i] += wb;
            }
        }
        cwa[j] = ca;
        cwb[j] = cb2;
    }
    // hand the sums to the other waves through LDS (double-buffered by head parity)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float v = cwa[j];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (lane < 16) pb[wave][j * 16 + lane] = v;
        if (st == tt) {
            float u = cwb[j];
            u += __shfl_xor(u, 16, 64);
            u += __shfl_xor(u, 32, 64);
            if (lane < 16) pb[4 + wave][j * 16 + lane] = u;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float r = row16_sum(rwa[i]);
        if (lr == 0) pb[8][tl[i]] = r;
        if (st == tt) {
            const float u = row16_sum(rwb[i]);
            if (lr == 0) pb[9][tl[i]] = u;
        }
    }
    __syncthreads();
    // off-diagonal: [0] = column sums, [1] = row sums.  diagonal: [0] = cw_f - rw_f, [1] = cw_b - rw_b
    // (the consumer turns them into the tile's own contribution with a prefix resp. suffix sum)
    if (threadIdx.x < 128) {
        const int q = threadIdx.x & 63, which = threadIdx.x >> 6;
        const int base = (st != tt || which == 0) ? 0 : 4;
        float a0 = pb[base][q], a1 = pb[base + 1][q];
        float a2 = pb[base + 2][q], a3 = pb[base + 3][q];
        float r8 = pb[st != tt ? 8 : 8 + which][q];
            float v;
        if (st != tt) v = which == 0 ? a0 + a1 + a2 + a3 : r8;
        else v = a0 + a1 + a2 + a3 - r8;
        tv[which * 64 + q] = v;
    }
}

template <typename T, bool FAST>
__global__ __launch_bounds__(NTHREADS) void bwd_dcb_kernel(const bimamba2_params p, int nc, int nqt) {
    typedef Mma<T> M;
    constexpr int KPL = M::KPL, KSTEP = M::KSTEP;
    constexpr int KC = sizeof(T) == 2 ? 64 : 16;          // K chunk held in registers
    constexpr int NKS = KC / KSTEP;
    __shared__ float cst[DCB_HEADS][5][64];               // cs_f[t], cs_b[t], cs_f[s], cs_b[s], dt[s] per head
    __shared__ float part[2][10][64];                     // per-wave column sums (f: 0-3, b: 4-7), row sums (f: 8, b: 9)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    // blockIdx.x = (b, c, g) varies fastest so that the tiles of one (b, c, g), which share x and dout rows, run on
    // the same XCD (workgroups are dealt round-robin to the 8 XCDs) and hit its L2
    const int tile = blockIdx.y;
    const int tt = tile / nqt, st = tile % nqt;
    const int g = blockIdx.x % p.ngroups, bc = blockIdx.x / p.ngroups, c = bc % nc, b = bc / nc;
    const int Q = p.chunk_size, P = p.headdim, H = p.nheads, hpg = H / p.ngroups;
    const int limit = min(Q, p.seqlen - c * Q);
    const int t0 = tt * 64, s0 = st * 64;
    const bool live = t0 < limit && s0 < limit;
    const float *cbg = p.CB + ((int64_t)(b * nc + c) * p.ngroups + g) * Q * Q;
    int tl[4];     // local row of this lane's accumulator elements
#pragma unroll
    for (int i = 0; i < 4; ++i) tl[i] = wave * 16 + lg * 4 + i;
    f32x4 cbr[4], dcb[4] = {};
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = t0 + tl[i], s = s0 + j * 16 + lr;
            cbr[j][i] = (t < limit && s < limit) ? cbg[(int64_t)t * Q + s] : 0.f;   // 0 also masks rows / columns past the end
        }
    // operand rows of this lane: A = dy row t0 + 16 wave + lr; B = x rows s0 + 16 j + lr
    const int arow = min(t0 + wave * 16 + lr, limit - 1);
    int brow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) brow[j] = min(s0 + j * 16 + lr, limit - 1);
    const int nkc = (P + KC - 1) / KC;

    // blockIdx.z selects a slice of the group's heads; its dCB partial sum goes to slice blockIdx.z of the output
    const int hps = (hpg + gridDim.z - 1) / gridDim.z;
    const int h_begin = blockIdx.z * hps, h_end = min(hpg, h_begin + hps);
    for (int hbase = h_begin; hbase < h_end; hbase += DCB_HEADS) {
        const int nh = min(DCB_HEADS, h_end - hbase);
        __syncthreads();
        for (int base = 0; base < nh * 5 * 64; base += NTHREADS * 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {                   // eight independent loads in flight per thread
                const int idx = base + u * NTHREADS + threadIdx.x;
                const int hh = idx / 320, which = (idx % 320) / 64, q = idx % 64;
                const int64_t o = (((int64_t)b * H + g * hpg + hbase + min(hh, nh - 1)) * nc + c) * Q;
                const int pos = min((which < 2 ? t0 : s0) + q, Q - 1);
                const float *src = which == 0 || which == 2 ? p.cs_f : (which == 4 ? p.dt_out : p.cs_b);
                v[u] = src[o + pos];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = base + u * NTHREADS + threadIdx.x;
                if (idx < nh * 5 * 64) cst[idx / 320][(idx % 320) / 64][idx % 64] = v[u];
            }
        }
        __syncthreads();
        if (!live) {
            for (int hh = 0; hh < nh; ++hh) {
                const int64_t o = (((int64_t)b * H + g * hpg + hbase + hh) * nc + c);
                float *tv = p.da_intra + (o * nqt * nqt + tile) * DCB_VEC;
                for (int i = threadIdx.x; i < DCB_VEC; i += NTHREADS) tv[i] = 0.f;
            }
            continue;
        }
        // flattened loop over (head, K chunk) with two operand buffers
        typename M::Frag af[1][NKS], bf[1][4][NKS];        // operands in flight (next step)
        typename M::Frag afc[NKS], bfc[4][NKS];            // operands being multiplied
        const int nit = nh * nkc;
        auto issue = [&](int it) __attribute__((always_inline)) {
            constexpr int B_ = 0;
            const int hh = it / nkc, k0 = (it % nkc) * KC;
            const int h = g * hpg + hbase + hh;
            const T *yp;
            int64_t ys;
            if (p.has_z) { ys = (int64_t)H * P; yp = reinterpret_cast<const T *>(p.dout_x) + ((int64_t)b * p.seqlen + (int64_t)c * Q) * ys + (int64_t)h * P; }
            else { ys = p.dout_sl; yp = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * ys + h * p.dout_sh; }
            const T *xp = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * p.x_sl + h * p.x_sh;
            const T *ar = yp + (int64_t)arow * ys;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const int kb = k0 + ks * KSTEP + lg * KPL;
                if (FAST || ((reinterpret_cast<uintptr_t>(ar + kb) & 15) == 0 && kb + KPL <= P)) af[B_][ks] = M::load(ar + kb);
                else {
                    float v[KPL];
#pragma unroll
                    for (int i = 0; i < KPL; ++i) v[i] = kb + i < P ? to_f(ar[kb + i]) : 0.f;
                    af[B_][ks] = M::pack(v);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const T *br = xp + (int64_t)brow[j] * p.x_sl;
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    const int kb = k0 + ks * KSTEP + lg * KPL;
                    if (FAST || ((reinterpret_cast<uintptr_t>(br + kb) & 15) == 0 && kb + KPL <= P)) bf[B_][j][ks] = M::load(br + kb);
                    else {
                        float v[KPL];
#pragma unroll
                        for (int i = 0; i < KPL; ++i) v[i] = kb + i < P ? to_f(br[kb + i]) : 0.f;
                        bf[B_][j][ks] = M::pack(v);
                    }
                }
            }
        };
        f32x4 acc[4] = {};
        auto finish_head = [&](int hh) __attribute__((always_inline)) {
            const int64_t o = (((int64_t)b * H + g * hpg + hbase + hh) * nc + c);
            dcb_finish_head<T>(acc, dcb, cbr, cst[hh], part[hh & 1], p.da_intra + (o * nqt * nqt + tile) * DCB_VEC, tl, st, tt);
        };
        issue(0);
        for (int it = 0; it < nit; ++it) {
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                afc[ks] = af[0][ks];
#pragma unroll
                for (int j = 0; j < 4; ++j) bfc[j][ks] = bf[0][j][ks];
            }
            if (it + 1 < nit) issue(it + 1);                // requested now, needed in the next iteration
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = M::mma(afc[ks], bfc[j][ks], acc[j]);
            if (it % nkc == nkc - 1) {
                // rows past the end of the sequence were read from a valid row: drop them
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (t0 + tl[i] >= limit) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) acc[j][i] = 0.f;
                    }
                finish_head(it / nkc);
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    }
    const int64_t oo = ((int64_t)blockIdx.z * gridDim.x + (int64_t)(b * nc + c) * p.ngroups + g) * Q * Q;
    float *out = p.dCB + oo, *outT = p.dCBT + oo;       // dCBT[s, t] = dCB[t, s], read by the dB product
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int s = s0 + j * 16 + lr;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = t0 + tl[i];
            if (t < Q && s < Q) out[(int64_t)t * Q + s] = dcb[j][i];
        }
        if (s < Q) {
            if (t0 + tl[0] + 3 < Q && Q % 4 == 0) *reinterpret_cast<f32x4 *>(outT + (int64_t)s * Q + t0 + tl[0]) = dcb[j];
            else
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (t0 + tl[i] < Q) outT[(int64_t)s * Q + t0 + tl[i]] = dcb[j][i];
        }
    }
}

// dst[i] += sum_{s=1..nslices-1} dst[s*n + i]
__global__ __launch_bounds__(NTHREADS) void sum_slices_kernel(float *dst, size_t n4, int nslices) {
    float4 *d = reinterpret_cast<float4 *>(dst);
    for (size_t i = blockIdx.x * (size_t)NTHREADS + threadIdx.x; i < n4; i += (size_t)gridDim.x * NTHREADS) {
        float4 v = d[i];
        for (int s = 1; s < nslices; ++s) {
            const float4 u = d[s * n4 + i];
            v.x += u.x; v.y += u.y; v.z += u.z; v.w += u.w;
        }
        d[i] = v;
    }
}

// head slices of the dCB kernel: one per 32 heads of a group (more slices only cost traffic: measured)
int dcb_slices(const bimamba2_params *p) {
    const int hpg = p->nheads / p->ngroups;
    return std::max(1, std::min(DCB_SLICES_MAX, hpg / DCB_SLICE_HEADS));
}

// ---------------------------------------------------------------------------------------------------------
// Variant for 16-bit types with headdim % 64 == 0, chunk_size % 64 == 0 and aligned operands.
//
// The kernel is bound by its instruction count, not by memory, so everything per head is pared down:
//  * the dout tile, the x tile and the decay vectors of each (head, 64-wide headdim chunk) step travel from global memory
//    straight into a ring of LDS slots (global_load_lds, 16 bytes per lane, no registers, no address arithmetic beyond
//    one 64-bit add per request), one step ahead of the one being multiplied; 16-byte units are XOR-swizzled by the row
//    so that the fragment reads spread over the banks;
//  * a wave owns 16 rows t; against a block of 16 columns s that lies wholly below (s < t) or above (s > t) the diagonal
//    the decay factor separates, exp(cs[t] - cs[s]) = exp(cs[t] - m) * exp(m - cs[s]) with m taken at the edge of the
//    wave's rows nearest to the columns, so that both factors are <= 1 for A <= 0: 8 exponentials instead of 16 per
//    block and the factors move out of the row and column sums.  Only the 16x16 block on the diagonal takes the masked
//    two-direction path;
//  * the column sums over the four 16-lane groups come from one MFMA with a matrix of ones per column block.
// ---------------------------------------------------------------------------------------------------------
// sum of v over the four lanes l%16, l%16+16, l%16+32, l%16+48, delivered to all of them: D = ones(16x4) * B where lane l
// supplies B[k = l/16][n = l%16]
__device__ __forceinline__ float lanegroup_sum_mfma(float v) {
    const f32x4 d = __builtin_amdgcn_mfma_f32_16x16x4f32(1.0f, v, f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    return d[0];
}

// Slots of the ring.  Two (the step being multiplied and the one after it, requested right after the barrier that frees
// its slot) measured 60 us against 62 us for three slots requested two steps ahead.
constexpr int DCB_RING = 2;
constexpr int DCB_RESIDENT_BLOCKS = 1024;                 // a dCB grid up to this size is on the chip all at once
constexpr int DCB_TILE_B = 64 * 64 * 2;                    // one 64 x 64 tile of 16-bit elements
constexpr int DCB_CS_OFF = 2 * DCB_TILE_B;                 // cs_f[t], cs_b[t], cs_f[s], cs_b[s], dt[s]: 5 x 64 floats
constexpr int DCB_SLOT_B = DCB_CS_OFF + 5 * 64 * 4;
constexpr int DCB_PART_OFF = DCB_RING * DCB_SLOT_B;        // per-wave column sums (f: 0-3, b: 4-7), row sums (f: 8, b: 9)
constexpr int DCB_PART_B = 10 * 64 * 4;


// UNI: the single-direction operator - tiles above the diagonal are empty, tiles on it keep the forward half.
// bid / gdx / gdz: block index and grid extents (x: batch * chunks * groups, y: tiles, z: head slices)
// Which (batch, chunk, group) and which tile the id-th workgroup of the dCB grid takes.  Workgroups are dealt round-robin to
// the 8 XCDs in id order, and the tiles of one (b, c, g) read the same dout and x rows (each row tile four times at chunk
// 256), so they belong on one XCD, close in time.  A grid that is resident all at once (two or three workgroups per CU)
// has (b, c, g) fastest: equal ids modulo 8 share an XCD, and all diagonal tiles, which cost more, come first and spread
// over the CUs.  A larger grid runs in several rounds, and with that order a row tile's readers are rounds apart and
// each fetches it from memory again (768 MB of reads at 8 groups of 4 heads, batch 4 x 4096; 172 -> 155 us): there
// eight (b, c, g) at a time, one per XCD, go through all their tiles before the next eight start.
__device__ __forceinline__ BlockId dcb_block_of(int id, int gdx, int ntiles, int nblocks) {
    if (nblocks <= DCB_RESIDENT_BLOCKS || gdx % 8) return BlockId{id % gdx, id / gdx, 0};
    const int k = id >> 3;
    return BlockId{(k / ntiles) * 8 + (id & 7), k % ntiles, 0};
}

template <typename T, bool UNI>
__device__ __forceinline__ void bwd_dcb_ring_body(const bimamba2_params &p, int nc, int nqt, BlockId bid, int gdx, int gdz, bool out16 = false) {
    typedef Mma<T> M;
    typedef typename M::Frag Frag;
    static_assert(sizeof(T) == 2, "ring variant is for 16-bit operands");
    constexpr int KC = 64, NKS = 2;                            // 64 headdim columns = 8 units of 16 bytes per row
    __shared__ __attribute__((aligned(16))) unsigned char smem[DCB_PART_OFF + 2 * DCB_PART_B];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    // the tiles on the diagonal cost more: they come first in launch order, which spreads them over the compute units
    int tt, st;
    if (bid.y < nqt) tt = st = bid.y;
    else {
        const int k = bid.y - nqt;
        tt = k / (nqt - 1);
        st = k % (nqt - 1);
        st += st >= tt;
    }
    const int tile = tt * nqt + st;
    const int g = bid.x % p.ngroups, bc = bid.x / p.ngroups, c = bc % nc, b = bc / nc;
    const int Q = p.chunk_size, P = p.headdim, H = p.nheads, hpg = H / p.ngroups;
    const int limit = min(Q, p.seqlen - c * Q);
    const int t0 = tt * 64, s0 = st * 64;
    const bool live = t0 < limit && s0 < limit && !(UNI && st > tt);
    const int trow = wave * 16 + lg * 4;                       // first of this lane's four accumulator rows
    f32x4 cbr[4] = {}, dcb[4] = {};
    const int hps = (hpg + gdz - 1) / gdz;
    const int h_begin = bid.z * hps, h_end = min(hpg, h_begin + hps);
    const int nkc = P / KC, nhs = h_end - h_begin, nit = nhs * nkc;
    const int h0 = g * hpg + h_begin;
    const int64_t tv_head = (int64_t)nc * nqt * nqt * DCB_VEC;
    float *tv0 = p.da_intra + ((((int64_t)b * H + h0) * nc + c) * nqt * nqt + tile) * DCB_VEC;
    if (!live) {
        for (int hh = 0; hh < nhs; ++hh)
            for (int i = threadIdx.x; i < DCB_VEC; i += NTHREADS) tv0[hh * tv_head + i] = 0.f;
    } else {
        const unsigned sbase = lds_addr(smem);
        // ---- requests: unit u = i*256 + thread of a 64 x 64 tile is row r = u / 8, 16-byte chunk (u % 8) ^ (r % 8).
        // Addresses are a wave-uniform base (scalar registers, moved on from head to head) plus this lane's 32-bit byte offset
        // (the launcher checks that the rows of a chunk lie within 32 bits of each other): six vector registers less than
        // four per-lane pointers (126 registers instead of 138: four workgroups fit a CU where the grid has them).
        const char *ybase, *xbase;
        unsigned yoff[2], xoff[2];
        int64_t y_head, y_row;
        {
            const T *yp;
            if (p.has_z) { y_row = (int64_t)H * P; y_head = P; yp = reinterpret_cast<const T *>(p.dout_x) + ((int64_t)b * p.seqlen + (int64_t)c * Q) * y_row + (int64_t)h0 * P; }
            else { y_row = p.dout_sl; y_head = p.dout_sh; yp = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + (int64_t)c * Q * y_row + h0 * p.dout_sh; }
            const T *xp = reinterpret_cast<const T *>(p.x) + b * p.x_sb + (int64_t)c * Q * p.x_sl + h0 * p.x_sh;
            ybase = uniform_ptr(yp);
            xbase = uniform_ptr(xp);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int u = i * NTHREADS + threadIdx.x, r = u >> 3, col = ((u & 7) ^ (r & 7)) * 8;
                yoff[i] = (unsigned)(((int64_t)min(t0 + r, limit - 1) * y_row + col) * (int64_t)sizeof(T));
                xoff[i] = (unsigned)(((int64_t)min(s0 + r, limit - 1) * p.x_sl + col) * (int64_t)sizeof(T));
            }
        }
        const float *csrc;                                     // threads 0..79: 16-byte unit of the five decay vectors
        {
            const int which = min((int)threadIdx.x >> 4, 4), j4 = (threadIdx.x & 15) * 4;
            const int64_t o = (((int64_t)b * H + h0) * nc + c) * Q + (which < 2 ? t0 : s0) + j4;
            csrc = (which == 0 || which == 2 ? p.cs_f : (which == 4 ? p.dt_out : p.cs_b)) + o;
        }
        const int64_t x_head = p.x_sh, cs_head = (int64_t)nc * Q;
        int ikc = 0;
        // requests one step into `slot` and moves the source pointers on to the next step
        auto issue = [&](int slot) __attribute__((always_inline)) {
            unsigned char *sl = smem + slot * DCB_SLOT_B + wave * 1024;
            load16_to_lds_at(ybase, yoff[0], sl);
            load16_to_lds_at(ybase, yoff[1], sl + 4096);
            load16_to_lds_at(xbase, xoff[0], sl + DCB_TILE_B);
            load16_to_lds_at(xbase, xoff[1], sl + DCB_TILE_B + 4096);
            if (threadIdx.x < 80) __builtin_amdgcn_global_load_lds((gbl_ptr_t)csrc, (lds_ptr_t)(sl + DCB_CS_OFF), 16, 0, 0);
            const bool last = ++ikc == nkc;
            if (last) ikc = 0;
            const int64_t dy = last ? y_head - (nkc - 1) * KC : KC, dx = last ? x_head - (nkc - 1) * KC : KC;
            ybase += dy * (int64_t)sizeof(T);
            xbase += dx * (int64_t)sizeof(T);
            if (last) csrc += cs_head;
        };
        // ---- per-lane LDS byte offsets inside a slot
        unsigned a_off[NKS], b_off[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const int ch = (ks * 4 + lg) ^ (lr & 7);
            a_off[ks] = ((wave * 16 + lr) * 8 + ch) * 16;
            b_off[ks] = DCB_TILE_B + (lr * 8 + ch) * 16;       // column block j adds j * 2048
        }
        const unsigned ct_off = DCB_CS_OFF + trow * 4, cc_off = DCB_CS_OFF + lr * 4, cm_off = DCB_CS_OFF + wave * 64;
        const int rows_left = limit - t0 - trow;               // accumulator rows i >= rows_left lie past the sequence end

        f32x4 acc[4] = {};
        issue(0);
        if (DCB_RING > 2 && nit > 1) issue(1);
        if (p.CB) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float *cbg = p.CB + ((int64_t)(b * nc + c) * p.ngroups + g) * Q * Q;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int t = t0 + trow + i, s = s0 + j * 16 + lr;
                    cbr[j][i] = (t < limit && s < limit) ? cbg[(int64_t)t * Q + s] : 0.f;
                }
            }
        } else {
            // no CB given: the tile CB[t, s] = C_t . B_s is rebuilt here, once per workgroup; both operands are read from
            // global memory in MFMA layout (dstate is contiguous) and the product lands in the layout of cbr
            const T *crow = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + ((int64_t)c * Q + min(t0 + wave * 16 + lr, limit - 1)) * p.C_sl + g * p.C_sg + lg * 8;
            const T *brow = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * p.B_sl + g * p.B_sg + lg * 8;
            for (int n0 = 0; n0 < p.dstate; n0 += 32) {
                const Frag cf = M::load(crow + n0);
#pragma unroll
                for (int j = 0; j < 4; ++j) cbr[j] = M::mma(cf, M::load(brow + (int64_t)min(s0 + j * 16 + lr, limit - 1) * p.B_sl + n0), cbr[j]);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (t0 + trow + i >= limit || s0 + j * 16 + lr >= limit) cbr[j][i] = 0.f;
        }
        // settle these register loads here: inside the loop a wait for them would drain the ring's requests as well
        wait_vmcnt<0>();
        int slot = 0, slot2 = (DCB_RING - 1) % DCB_RING, kc = 0, par = 0;
        float *tv = tv0 + (wave & 1) * 64 + lane;
        // the sums of a head are written out one iteration later, after the barrier that the next step needs anyway
        // (waves 0 and 1; off-diagonal: [0] = column sums, [1] = row sums.  diagonal: [0] = cw_f - rw_f, [1] = cw_b - rw_b,
        // which the consumer turns into the tile's own contribution with a prefix resp. suffix sum)
        bool pending = false;
        auto write_out = [&](int pbuf) __attribute__((always_inline)) {
            if (wave < 2) {
                const unsigned pq = sbase + DCB_PART_OFF + pbuf * DCB_PART_B + lane * 4;
                float v;
                if (st != tt && wave == 1) {
                    v = raw_lds_read_at<float, 2048>(pq);
                    raw_lds_wait();
                    raw_lds_use(v);
                } else {
                    float a0, a1, a2, a3, r8 = 0.f;
                    if (wave == 0) {
                        a0 = raw_lds_read_at<float, 0>(pq); a1 = raw_lds_read_at<float, 256>(pq);
                        a2 = raw_lds_read_at<float, 512>(pq); a3 = raw_lds_read_at<float, 768>(pq);
                        if (st == tt) r8 = raw_lds_read_at<float, 2048>(pq);
                    } else {
                        a0 = raw_lds_read_at<float, 1024>(pq); a1 = raw_lds_read_at<float, 1024 + 256>(pq);
                        a2 = raw_lds_read_at<float, 1024 + 512>(pq); a3 = raw_lds_read_at<float, 1024 + 768>(pq);
                        r8 = raw_lds_read_at<float, 2048 + 256>(pq);
                    }
                    raw_lds_wait();
                    raw_lds_use(a0); raw_lds_use(a1); raw_lds_use(a2); raw_lds_use(a3); raw_lds_use(r8);
                    v = a0 + a1 + a2 + a3 - r8;
                }
                *tv = v;
            }
            tv += tv_head;
        };
        // The head loop is compiled once per kind of tile: off the diagonal (KIND = -1), and on it once per wave (KIND = the
        // wave's index, which decides for every column block whether it lies below, on or above the wave's rows), so that
        // none of these decisions is taken, and no register moved to a common place, inside the loop.
        auto run = [&](auto KC) __attribute__((always_inline)) {
            constexpr int KIND = decltype(KC)::value;
            constexpr bool DIAG = KIND >= 0;
            constexpr bool LOWER = KIND == -1;             // off the diagonal: -1 below it (forward direction), -2 above
        for (int it = 0; it < nit; ++it) {
            // with two slots nothing but step `it` is outstanding here; with more, the requests of step `it` went out before
            // those of the step after it (waves 0 and 1 make five requests per step, the others four)
            if (DCB_RING > 2 && it + 1 < nit) {
                if (wave < 2) wait_vmcnt<5>();
                else wait_vmcnt<4>();
            } else {
                wait_vmcnt<0>();
            }
            raw_lds_barrier();     // step `it` has landed for everybody; every wave is done with the slot and the sums of step it - 1
            // (the store of the sums goes out before the requests: the wait at the top of the next step counts on the
            // requests of the step after it being this wave's youngest operations)
            if (pending) {
                write_out(par ^ 1);
                pending = false;
            }
            if (it + DCB_RING - 1 < nit) issue(slot2);
            const unsigned sb = sbase + slot * DCB_SLOT_B;
            Frag af[NKS], bf[4][NKS];
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                af[ks] = raw_lds_read_at<Frag, 0>(sb + a_off[ks]);
                bf[0][ks] = raw_lds_read_at<Frag, 0>(sb + b_off[ks]);
                bf[1][ks] = raw_lds_read_at<Frag, 2048>(sb + b_off[ks]);
                bf[2][ks] = raw_lds_read_at<Frag, 4096>(sb + b_off[ks]);
                bf[3][ks] = raw_lds_read_at<Frag, 6144>(sb + b_off[ks]);
            }
            raw_lds_wait();
            // (the first product of a head starts from a literal zero: no registers to clear between heads)
            const bool first = kc == 0;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                raw_lds_use(af[ks]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    raw_lds_use(bf[j][ks]);
                    if (ks == 0 && first) acc[j] = M::mma(af[ks], bf[j][ks], f32x4{0.f, 0.f, 0.f, 0.f});
                    else acc[j] = M::mma(af[ks], bf[j][ks], acc[j]);
                }
            }
            if (++kc == nkc) {
                kc = 0;
                // ---- decay vectors of this head (off the diagonal only the ones of the tile's direction)
                f32x4 cft_, cbt_;
                float cfs[4], cbs[4], dts[4], mf, mb;
                if constexpr (DIAG || LOWER) {
                    cft_ = raw_lds_read_at<f32x4, 0>(sb + ct_off);
                    cfs[0] = raw_lds_read_at<float, 512>(sb + cc_off); cfs[1] = raw_lds_read_at<float, 512 + 64>(sb + cc_off);
                    cfs[2] = raw_lds_read_at<float, 512 + 128>(sb + cc_off); cfs[3] = raw_lds_read_at<float, 512 + 192>(sb + cc_off);
                    mf = raw_lds_read_at<float, 0>(sb + cm_off);           // reference point: cs_f at the first of the wave's 16 rows
                }
                if constexpr (DIAG || !LOWER) {
                    cbt_ = raw_lds_read_at<f32x4, 256>(sb + ct_off);
                    cbs[0] = raw_lds_read_at<float, 768>(sb + cc_off); cbs[1] = raw_lds_read_at<float, 768 + 64>(sb + cc_off);
                    cbs[2] = raw_lds_read_at<float, 768 + 128>(sb + cc_off); cbs[3] = raw_lds_read_at<float, 768 + 192>(sb + cc_off);
                    mb = raw_lds_read_at<float, 256 + 60>(sb + cm_off);    // cs_b at the last of them
                }
                dts[0] = raw_lds_read_at<float, 1024>(sb + cc_off); dts[1] = raw_lds_read_at<float, 1024 + 64>(sb + cc_off);
                dts[2] = raw_lds_read_at<float, 1024 + 128>(sb + cc_off); dts[3] = raw_lds_read_at<float, 1024 + 192>(sb + cc_off);
                raw_lds_wait();
                if constexpr (DIAG || LOWER) {
                    raw_lds_use(cft_); raw_lds_use(mf);
#pragma unroll
                    for (int j = 0; j < 4; ++j) raw_lds_use(cfs[j]);
                }
                if constexpr (DIAG || !LOWER) {
                    raw_lds_use(cbt_); raw_lds_use(mb);
#pragma unroll
                    for (int j = 0; j < 4; ++j) raw_lds_use(cbs[j]);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) raw_lds_use(dts[j]);
                if (rows_left < 4) {
                    // rows past the end of the sequence were read from a valid row: drop them
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (i >= rows_left) {
#pragma unroll
                            for (int j = 0; j < 4; ++j) acc[j][i] = 0.f;
                        }
                }
                // W = dCB_h * CB; col*[j]: this lane's part of the column sums, row*[i]: of the row sums
                float colF[4], colB[4] = {0.f, 0.f, 0.f, 0.f}, rowF[4], rowB[4] = {0.f, 0.f, 0.f, 0.f};
                // one 16 x 16 block whose columns lie on one side of the wave's rows: factors E (rows) and Fd (columns)
                auto sep_block = [&](int j, const float (&E)[4], float Fd, float &col, float (&rp)[4]) __attribute__((always_inline)) {
                    float cp = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float a = acc[j][i], y = a * cbr[j][i];
                        cp = __builtin_fmaf(y, E[i], cp);
                        rp[i] = __builtin_fmaf(y, Fd, rp[i]);
                        dcb[j][i] = __builtin_fmaf(a * E[i], Fd, dcb[j][i]);
                    }
                    col = cp * Fd;
                };
                if constexpr (!DIAG) {
                    // forward direction below the diagonal, reverse above it
                    float E[4], rp[4] = {0.f, 0.f, 0.f, 0.f};
                    const float ml = (LOWER ? mf : mb) * LOG2E;
#pragma unroll
                    for (int i = 0; i < 4; ++i) E[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(LOWER ? cft_[i] : cbt_[i], LOG2E, -ml));
#pragma unroll
                    for (int j = 0; j < 4; ++j) sep_block(j, E, dts[j] * __builtin_amdgcn_exp2f(__builtin_fmaf(LOWER ? cfs[j] : cbs[j], -LOG2E, ml)), colF[j], rp);
#pragma unroll
                    for (int i = 0; i < 4; ++i) rowF[i] = rp[i] * E[i];
                } else {
                    float Ef[4], Eb[4], rpf[4] = {0.f, 0.f, 0.f, 0.f}, rpb[4] = {0.f, 0.f, 0.f, 0.f};
                    float df[4] = {0.f, 0.f, 0.f, 0.f}, db[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int i = 0; i < 4; ++i) { Ef[i] = __expf(cft_[i] - mf); Eb[i] = __expf(cbt_[i] - mb); }
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (j < KIND) { sep_block(j, Ef, dts[j] * __expf(mf - cfs[j]), colF[j], rpf); }
                        else if (j > KIND) { colF[j] = 0.f; if (!UNI) sep_block(j, Eb, dts[j] * __expf(mb - cbs[j]), colB[j], rpb); }
                        else {
                            // the block on the diagonal: both directions, masked element by element
                            float ca = 0.f, cb2 = 0.f;
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                const int ti = lg * 4 + i;     // row and column (lr) inside the block
                                const float gv = acc[j][i] * dts[j];
                                const float f = (lr <= ti) ? gv * __expf(cft_[i] - cfs[j]) : 0.f;
                                const float r = (!UNI && lr >= ti) ? gv * __expf(cbt_[i] - cbs[j]) : 0.f;
                                dcb[j][i] += f + r;
                                const float wf = (lr < ti) ? f * cbr[j][i] : 0.f;
                                const float wb = (lr > ti) ? r * cbr[j][i] : 0.f;
                                ca += wf; df[i] += wf;
                                cb2 += wb; db[i] += wb;
                            }
                            colF[j] = ca;
                            colB[j] = cb2;
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) { rowF[i] = __builtin_fmaf(rpf[i], Ef[i], df[i]); rowB[i] = __builtin_fmaf(rpb[i], Eb[i], db[i]); }
                }
                // ---- hand the sums to the other waves through LDS (double-buffered by head parity)
                const unsigned pb = sbase + DCB_PART_OFF + par * DCB_PART_B;
                {
                    float cs4[4], cs4b[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) cs4[j] = lanegroup_sum_mfma(colF[j]);
                    if constexpr (DIAG) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) cs4b[j] = lanegroup_sum_mfma(colB[j]);
                    }
                    f32x4 rs, rsb;
#pragma unroll
                    for (int i = 0; i < 4; ++i) rs[i] = row16_sum(rowF[i]);
                    if constexpr (DIAG) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) rsb[i] = row16_sum(rowB[i]);
                    }
                    const unsigned pw = pb + wave * 256 + lr * 4;
                    if (lane < 16) {
                        raw_lds_write_at<0>(pw, cs4[0]); raw_lds_write_at<64>(pw, cs4[1]);
                        raw_lds_write_at<128>(pw, cs4[2]); raw_lds_write_at<192>(pw, cs4[3]);
                        if constexpr (DIAG) {
                            raw_lds_write_at<1024>(pw, cs4b[0]); raw_lds_write_at<1024 + 64>(pw, cs4b[1]);
                            raw_lds_write_at<1024 + 128>(pw, cs4b[2]); raw_lds_write_at<1024 + 192>(pw, cs4b[3]);
                        }
                    }
                    if (lr == 0) {
                        raw_lds_write128_at<2048>(pb + trow * 4, rs);
                        if constexpr (DIAG) raw_lds_write128_at<2048 + 256>(pb + trow * 4, rsb);
                    }
                }
                raw_lds_wait();
                pending = true;            // written out after the next barrier (or after the loop)
                par ^= 1;
            }
            slot = slot + 1 == DCB_RING ? 0 : slot + 1;
            slot2 = slot2 + 1 == DCB_RING ? 0 : slot2 + 1;
        }
        };
        if (st < tt) run(std::integral_constant<int, -1>());
        else if (st > tt) run(std::integral_constant<int, -2>());
        else if (wave == 0) run(std::integral_constant<int, 0>());
        else if (wave == 1) run(std::integral_constant<int, 1>());
        else if (wave == 2) run(std::integral_constant<int, 2>());
        else run(std::integral_constant<int, 3>());
        if (pending) {
            raw_lds_barrier();
            write_out(par ^ 1);
        }
    }
    const int64_t oo = ((int64_t)bid.z * gdx + (int64_t)(b * nc + c) * p.ngroups + g) * Q * Q;
    if (out16) {
        // dCB / dCBT in the element type of the inputs (inside bimamba2_bwd, one head slice: their one reader rounds them to
        // that type for its MFMA anyway, so nothing changes but the bytes moved)
        T *out = reinterpret_cast<T *>(p.dCB) + oo, *outT = reinterpret_cast<T *>(p.dCBT) + oo;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int s = s0 + j * 16 + lr;
            T v4[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v4[i] = from_f<T>(dcb[j][i]);
                out[(int64_t)(t0 + trow + i) * Q + s] = v4[i];
            }
            *reinterpret_cast<uint2 *>(outT + (int64_t)s * Q + t0 + trow) = *reinterpret_cast<const uint2 *>(v4);
        }
        return;
    }
    float *out = p.dCB + oo, *outT = p.dCBT + oo;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int s = s0 + j * 16 + lr;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[(int64_t)(t0 + trow + i) * Q + s] = dcb[j][i];
        *reinterpret_cast<f32x4 *>(outT + (int64_t)s * Q + t0 + trow) = dcb[j];
    }
}

template <typename T, bool UNI = false>
__global__ __launch_bounds__(NTHREADS) void bwd_dcb_ring_kernel(const bimamba2_params p, int nc, int nqt) {
    BlockId bid = dcb_block_of(blockIdx.x + gridDim.x * blockIdx.y, gridDim.x, gridDim.y, gridDim.x * gridDim.y);
    bid.z = blockIdx.z;
    bwd_dcb_ring_body<T, UNI>(p, nc, nqt, bid, gridDim.x, gridDim.z);
}

// The dCB kernel and the backward state passing as roles of one launch (16-bit copies of the entering states on both sides
// of the state passing, one head slice): the first is bound by instruction issue and moves little data, the second streams
// 70 MB and needs few instructions, and the two depend on different kernels before them.  The first ndcb blocks are the
// dCB tiles in the order of their own grid (so they are placed first, two per CU as when alone), the rest are the state
// passing's blocks, which take what is left of each CU.
template <typename T, bool UNI>
__device__ __forceinline__ void bwd_dcb_sp_body(const bimamba2_params &p, int nc, int nqt, int gdx, int ndcb, int nsplit, int ndir, bool out16) {
    const int id = blockIdx.x;
    if (id < ndcb) {
        bwd_dcb_ring_body<T, UNI>(p, nc, nqt, dcb_block_of(id, gdx, nqt * nqt, ndcb), gdx, 1, out16);
    } else {
        const int k = id - ndcb;                  // grid (nsplit, nheads, batch * ndir) of the state passing
        const BlockId sb{k % nsplit, (k / nsplit) % p.nheads, k / (nsplit * p.nheads)};
        if (p.dstates_f == nullptr) state_passing_bwd_vec_body<T, true, true, true>(p, nc, nsplit, ndir, sb);
        else state_passing_bwd_vec_body<T, true, true>(p, nc, nsplit, ndir, sb);
    }
}

template <typename T, bool UNI>
__global__ __launch_bounds__(NTHREADS) void bwd_dcb_sp_kernel(const bimamba2_params p, int nc, int nqt, int gdx, int ndcb, int nsplit, int ndir, bool out16) {
    bwd_dcb_sp_body<T, UNI>(p, nc, nqt, gdx, ndcb, nsplit, ndir, out16);
}
template <typename T> static void launch_dcb_ring(dim3 grid, const bimamba2_params *p, int nc, int nqt) {
    if constexpr (sizeof(T) == 2) {
        if (p->causal) hipLaunchKernelGGL((bwd_dcb_ring_kernel<T, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt);
        else hipLaunchKernelGGL((bwd_dcb_ring_kernel<T>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt);
    }
}

// whether the dCB kernel can do without CB (it rebuilds its tile from the C and B rows): the 16-bit ring variant, dstate a
// multiple of 32, 16-byte aligned row matrices
// the ring variant addresses the rows of a chunk with 32-bit byte offsets from a per-head base
static bool dcb_rows_in_32bit(const bimamba2_params *p) {
    // (a query that comes before dout is known - no pointer, no strides yet - is answered for the contiguous tensor)
    const int64_t ys = (p->has_z || !p->dout) ? (int64_t)p->nheads * p->headdim : p->dout_sl;
    return p->x_sl > 0 && p->x_sl < (1 << 22) && ys > 0 && ys < (1 << 22);
}

bool dcb_recomputes_cb(const bimamba2_params *p) {
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % 8 == 0 && b % 8 == 0 && c % 8 == 0; };
    if (p->dtype == BIMAMBA2_F32 || p->headdim % 64 || p->chunk_size % 64 || p->dstate % 32 || !dcb_rows_in_32bit(p)) return false;
    if (!(al(p->x) && mult(p->x_sb, p->x_sl, p->x_sh))) return false;
    if (!(p->has_z ? al(p->dout_x) : (al(p->dout) && mult(p->dout_sb, p->dout_sl, p->dout_sh)))) return false;
    return al(p->Bm) && mult(p->B_sb, p->B_sl, p->B_sg) && al(p->Cm) && mult(p->C_sb, p->C_sl, p->C_sg);
}

template <typename T>
static int launch_dcb_t(const bimamba2_params *p) {
    const int nc = nchunks(p), nqt = (p->chunk_size + 63) / 64;
    const int slices = dcb_slices(p);
    dim3 grid(p->batch * nc * p->ngroups, nqt * nqt, slices);
    constexpr int VS = 16 / (int)sizeof(T);
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    bool fast = p->headdim % (sizeof(T) == 2 ? 64 : 16) == 0 && al(p->x) && p->x_sb % VS == 0 && p->x_sl % VS == 0 && p->x_sh % VS == 0;
    fast = fast && (p->has_z ? al(p->dout_x) : (al(p->dout) && p->dout_sb % VS == 0 && p->dout_sl % VS == 0 && p->dout_sh % VS == 0));
    if (!p->CB && !dcb_recomputes_cb(p)) return BIMAMBA2_EINVAL;
    const bool ring = fast && sizeof(T) == 2 && p->chunk_size % 64 == 0 && dcb_rows_in_32bit(p);
    if (p->causal && !ring) return BIMAMBA2_EUNSUPPORTED;
    if (ring) launch_dcb_ring<T>(grid, p, nc, nqt);
    else if (fast) hipLaunchKernelGGL((bwd_dcb_kernel<T, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt);
    else hipLaunchKernelGGL((bwd_dcb_kernel<T, false>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt);
    if (slices > 1) {
        // (Q*Q is a multiple of 4 only when Q is even; odd chunk sizes are rejected by the 16-byte requirement below)
        const size_t n = (size_t)p->batch * nc * p->ngroups * p->chunk_size * p->chunk_size;
        if (n % 4) return BIMAMBA2_EUNSUPPORTED;
        const int blocks = (int)std::min<size_t>((n / 4 + NTHREADS - 1) / NTHREADS, 4096);
        hipLaunchKernelGGL(sum_slices_kernel, dim3(blocks), dim3(NTHREADS), 0, stream_of(p), p->dCB, n / 4, slices);
        hipLaunchKernelGGL(sum_slices_kernel, dim3(blocks), dim3(NTHREADS), 0, stream_of(p), p->dCBT, n / 4, slices);
    }
    return check_launch();
}

// whether bwd_dcb_sp_kernel exists for the problem (the ring variant of the dCB kernel with one head slice, the vector
// variant of the state passing, 16-bit copies of the entering states and of their gradients)
bool bwd_dcb_sp_merged(const bimamba2_params *p) {
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    if (p->dtype != BIMAMBA2_BF16 && p->dtype != BIMAMBA2_F16) return false;
    if (!dcb_recomputes_cb(p) || dcb_slices(p) != 1) return false;       // (implies the conditions of the ring variant)
    if (!p->states16_f || !p->dstates16_f || !(p->causal || (p->states16_b && p->dstates16_b))) return false;
    if ((p->headdim * p->dstate) % 4) return false;
    return al(p->states16_f) && al(p->states16_b) && al(p->dstates16_f) && al(p->dstates16_b) && al(p->dstates_f) && al(p->dstates_b) &&
           al(p->dfinal_f) && al(p->dfinal_b) && al(p->dinitial_f) && al(p->dinitial_b);
}

// bimamba2_chunk_scan_bwd_dcb and bimamba2_state_passing_bwd in one launch (the caller checked bwd_dcb_sp_merged())
int launch_bwd_dcb_sp(const bimamba2_params *p, bool out16) {
    const int nc = nchunks(p), nqt = (p->chunk_size + 63) / 64, PN = p->headdim * p->dstate;
    const int nsplit = (PN + SP_EPT * NTHREADS - 1) / (SP_EPT * NTHREADS), ndir = p->causal ? 1 : 2;
    const int gdx = p->batch * nc * p->ngroups, ndcb = gdx * nqt * nqt, nsp = nsplit * p->nheads * p->batch * ndir;
    dim3 grid(ndcb + nsp);
#define BM2_DS(TT)                                                                                                                     \
    do {                                                                                                                               \
        if (p->causal) hipLaunchKernelGGL((bwd_dcb_sp_kernel<TT, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt, gdx, ndcb, nsplit, ndir, out16);  \
        else hipLaunchKernelGGL((bwd_dcb_sp_kernel<TT, false>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt, gdx, ndcb, nsplit, ndir, out16);           \
    } while (0)
    if (p->dtype == BIMAMBA2_BF16) BM2_DS(bf16_t); else BM2_DS(f16_t);
#undef BM2_DS
    return check_launch();
}

int launch_bwd_dcb(const bimamba2_params *p) {
    switch (p->dtype) {
        case BIMAMBA2_F32: return launch_dcb_t<float>(p);
        case BIMAMBA2_BF16: return launch_dcb_t<bf16_t>(p);
        case BIMAMBA2_F16: return launch_dcb_t<f16_t>(p);
        default: return BIMAMBA2_EUNSUPPORTED;
    }
}

// =========================================================================================================
// which = 0 : dB[s,n] = sum_slices dBs[s,n] + sum_t dCBT[s,t] C[t,n]     which = 1 : dC[t,n] = sum dCs + sum_s dCB[t,s] B[s,n]
// One workgroup: 64 rows x 64 dstate columns of one (b, c, g).  The K operand (C or B rows of the chunk) is staged
// transposed in LDS once; the A operand is read from the float32 dCB / dCBT rows straight into MFMA operand layout.
// =========================================================================================================
// FAST (16-bit types, chunk_size == QP, dstate a multiple of 64, aligned operands, at most 8 slices): every global load
// of a thread (its dCB row pieces, the slices it adds, the K operand) is requested before the first one is used.


// SLIM (with FAST): dCB / dCBT hold 16-bit elements (in16) and there are at most two slices to add: a quarter of the
// registers, and the staging tile of the result shares the LDS of the K operand, so that three workgroups fit a CU where
// the general variant fits two (with few heads per group the launch has thousands of workgroups: 83 -> 76 us at 8 groups
// of 4 heads, batch 4 x 4096, where the launch moves 250 MB).
template <typename T, int QP, bool FAST, bool SLIM = false>
__device__ __forceinline__ void bmm_chunk_bwd_body(const bimamba2_params &p, int nc, int nslices, BlockId bid, bool in16 = false) {
    typedef Mma<T> M;
    constexpr int KPL = M::KPL, KSTEP = M::KSTEP;
    constexpr int LDX = QP + 16 / (int)sizeof(T);
    constexpr int SLD = 64 + 4;
    constexpr int KT_BYTES = 64 * LDX * (int)sizeof(T), STG_BYTES = 64 * SLD * 4;
    __shared__ __attribute__((aligned(16))) unsigned char bmm_lds[SLIM ? (KT_BYTES > STG_BYTES ? KT_BYTES : STG_BYTES) : KT_BYTES + STG_BYTES];
    T *kT = reinterpret_cast<T *>(bmm_lds);
    float *stg = reinterpret_cast<float *>(bmm_lds + (SLIM ? 0 : KT_BYTES));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lr = lane & 15, lg = lane >> 4;
    const int nt = bid.x, rt = bid.y;
    const int which = bid.z & 1, bcg = bid.z >> 1;
    const int g = bcg % p.ngroups, bc = bcg / p.ngroups, c = bc % nc, b = bc / nc;
    const int Q = p.chunk_size, N = p.dstate;
    const int limit = min(Q, p.seqlen - c * Q);
    const int r0 = rt * 64;
    const T *op;
    int64_t os;
    if (which == 0) { os = p.C_sl; op = reinterpret_cast<const T *>(p.Cm) + b * p.C_sb + (int64_t)c * Q * os + g * p.C_sg + nt * 64; }
    else { os = p.B_sl; op = reinterpret_cast<const T *>(p.Bm) + b * p.B_sb + (int64_t)c * Q * os + g * p.B_sg + nt * 64; }
    const float *arow = (which == 0 ? p.dCBT : p.dCB) + (int64_t)bcg * Q * Q + (int64_t)min(r0 + wave * 16 + lr, Q - 1) * Q;
    const float *res = which == 0 ? p.dBs : p.dCs;
    T *out = reinterpret_cast<T *>(which == 0 ? p.dB : p.dC);
    // (dB / dC may be slices of a wider buffer: their own position and batch strides; 0 = contiguous)
    const int64_t o_sl = (which == 0 ? p.dB_sl : p.dC_sl) ? (which == 0 ? p.dB_sl : p.dC_sl) : (int64_t)p.ngroups * p.dstate;
    const int64_t o_sb = (which == 0 ? p.dB_sl : p.dC_sl) ? (which == 0 ? p.dB_sb : p.dC_sb) : p.seqlen * o_sl;
    const int64_t slice = (int64_t)p.batch * p.seqlen * p.ngroups * N;
    constexpr int VS = 16 / (int)sizeof(T);
    if constexpr (FAST) {
        constexpr int NS = QP / KSTEP, NIT = 64 * (64 / VS) / NTHREADS, MAXSL = SLIM ? 2 : 8;
        // in16: dCB / dCBT hold elements of type T (written that way by the dCB kernel inside bimamba2_bwd): a row piece is
        // the MFMA operand as it lies in memory
        float4 raw[NS][SLIM ? 1 : 2];
        if (SLIM || in16) {
            const T *arow16 = reinterpret_cast<const T *>(which == 0 ? p.dCBT : p.dCB) + (int64_t)bcg * Q * Q + (int64_t)min(r0 + wave * 16 + lr, Q - 1) * Q;
#pragma unroll
            for (int s = 0; s < NS; ++s) raw[s][0] = *reinterpret_cast<const float4 *>(arow16 + s * KSTEP + lg * KPL);
        } else if constexpr (!SLIM) {
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                raw[s][0] = *reinterpret_cast<const float4 *>(arow + s * KSTEP + lg * KPL);
                raw[s][1] = *reinterpret_cast<const float4 *>(arow + s * KSTEP + lg * KPL + 4);
            }
        }
        // slices: the first half is requested here, the second half after the products, into the registers of the row pieces
        // (keeps the kernel at two workgroups per CU)
        constexpr int HSL = MAXSL / 2;
        float4 sv[NIT][HSL][2];
        int64_t oa[NIT];
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int id = threadIdx.x + it * NTHREADS;
            const int rl = id / (64 / VS), cc = (id % (64 / VS)) * VS;
            const int r = min(r0 + rl, limit - 1);
            oa[it] = (((int64_t)b * p.seqlen + (int64_t)c * Q + r) * p.ngroups + g) * N + nt * 64 + cc;
#pragma unroll
            for (int sl = 0; sl < HSL; ++sl) {
                const float *q = res + oa[it] + (int64_t)min(sl, nslices - 1) * slice;
                sv[it][sl][0] = *reinterpret_cast<const float4 *>(q);
                sv[it][sl][1] = *reinterpret_cast<const float4 *>(q + 4);
            }
        }
        stage_transposed<T, QP, 64, LDX, true>(kT, op, os, limit, 64, [&](int k) { return k < limit ? 1.f : 0.f; });
        __syncthreads();
        f32x4 acc[4] = {};
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (s * KSTEP < limit) {
                typename M::Frag af;
                if constexpr (SLIM) {
                    static_assert(!SLIM || sizeof(typename M::Frag) == 16, "16-bit operands");
                    af = __builtin_bit_cast(typename M::Frag, raw[s][0]);
                } else {
                    float v[KPL] = {raw[s][0].x, raw[s][0].y, raw[s][0].z, raw[s][0].w, raw[s][1].x, raw[s][1].y, raw[s][1].z, raw[s][1].w};
                    if constexpr (sizeof(typename M::Frag) == 16) af = in16 ? __builtin_bit_cast(typename M::Frag, raw[s][0]) : M::pack(v);
                    else af = M::pack(v);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = M::mma(af, M::load(kT + xt_index<T, LDX>(j * 16 + lr, s * KSTEP + lg * KPL)), acc[j]);
            }
        }
        float4 sw[NIT][HSL][2] = {};
        if (nslices > HSL) {                        // (with one half's worth of slices there is nothing more to wait for)
#pragma unroll
            for (int it = 0; it < NIT; ++it)
#pragma unroll
                for (int sl = 0; sl < HSL; ++sl) {
                    const float *q = res + oa[it] + (int64_t)min(HSL + sl, nslices - 1) * slice;
                    sw[it][sl][0] = *reinterpret_cast<const float4 *>(q);
                    sw[it][sl][1] = *reinterpret_cast<const float4 *>(q + 4);
                }
        }
        if constexpr (SLIM) __syncthreads();       // every wave is done with the K operand, whose LDS the staging tile shares
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) stg[(wave * 16 + lg * 4 + i) * SLD + j * 16 + lr] = acc[j][i];
        __syncthreads();
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int id = threadIdx.x + it * NTHREADS;
            const int rl = id / (64 / VS), cc = (id % (64 / VS)) * VS;
            float v[VS];
#pragma unroll
            for (int i = 0; i < VS; ++i) v[i] = stg[rl * SLD + cc + i];
#pragma unroll
            for (int sl = 0; sl < MAXSL; ++sl) {
                if (sl < nslices) {
                    const float4 a0 = sl < HSL ? sv[it][sl % HSL][0] : sw[it][sl % HSL][0], a1 = sl < HSL ? sv[it][sl % HSL][1] : sw[it][sl % HSL][1];
                    v[0] += a0.x; v[1] += a0.y; v[2] += a0.z; v[3] += a0.w;
                    v[4] += a1.x; v[5] += a1.y; v[6] += a1.z; v[7] += a1.w;
                }
            }
            if (r0 + rl < limit) {
                Vec16<T> ov;
#pragma unroll
                for (int i = 0; i < VS; ++i) ov.v[i] = from_f<T>(v[i]);
                *reinterpret_cast<Vec16<T> *>(out + (b * o_sb + ((int64_t)c * Q + r0 + rl) * o_sl + (int64_t)g * N + nt * 64 + cc)) = ov;
            }
        }
        return;
    }
    stage_transposed<T, QP, 64, LDX, false>(kT, op, os, limit, N - nt * 64, [&](int k) { return 1.f; });
    __syncthreads();
    const bool cvec = Q % 4 == 0;
    f32x4 acc[4] = {};
    for (int k0 = 0; k0 < limit; k0 += KSTEP) {
        const int kb = k0 + lg * KPL;
        float v[KPL];
        if (cvec && kb + KPL <= Q) {
            if (KPL >= 4) {
#pragma unroll
                for (int i = 0; i < KPL; i += 4) {
                    const float4 t4 = *reinterpret_cast<const float4 *>(arow + kb + i);
                    v[i] = t4.x; v[(i + 1) % KPL] = t4.y; v[(i + 2) % KPL] = t4.z; v[(i + 3) % KPL] = t4.w;
                }
            } else {
                v[0] = arow[kb];
            }
        } else {
#pragma unroll
            for (int i = 0; i < KPL; ++i) v[i] = kb + i < Q ? arow[kb + i] : 0.f;
        }
        const typename M::Frag af = M::pack(v);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = M::mma(af, M::load(kT + xt_index<T, LDX>(j * 16 + lr, kb)), acc[j]);
    }
    // pass the tile through LDS so that the slices are read and the result is written
    // as 16-byte vectors along dstate
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) stg[(wave * 16 + lg * 4 + i) * SLD + j * 16 + lr] = acc[j][i];
    __syncthreads();
    // (16-byte stores: the strides and the base of the destination slice must both allow them)
    const bool ovec = N % VS == 0 && o_sl % VS == 0 && o_sb % VS == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
    for (int id = threadIdx.x; id < 64 * (64 / VS); id += NTHREADS) {
        const int rl = id / (64 / VS), cc = (id % (64 / VS)) * VS;
        const int r = r0 + rl, n = nt * 64 + cc;
        if (r >= limit || n >= N) continue;
        const int64_t a = (((int64_t)b * p.seqlen + (int64_t)c * Q + r) * p.ngroups + g) * N + n;
        const int64_t ao = b * o_sb + ((int64_t)c * Q + r) * o_sl + (int64_t)g * N + n;
        float v[VS];
#pragma unroll
        for (int i = 0; i < VS; ++i) v[i] = stg[rl * SLD + cc + i];
        if (ovec) {
            for (int sl = 0; sl < nslices; ++sl)
#pragma unroll
                for (int i = 0; i < VS; i += 4) {
                    const float4 t4 = *reinterpret_cast<const float4 *>(res + a + sl * slice + i);
                    v[i] += t4.x; v[i + 1] += t4.y; v[i + 2] += t4.z; v[i + 3] += t4.w;
                }
            Vec16<T> ov;
#pragma unroll
            for (int i = 0; i < VS; ++i) ov.v[i] = from_f<T>(v[i]);
            *reinterpret_cast<Vec16<T> *>(out + ao) = ov;
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i)
                if (n + i < N) {
                    float u = v[i];
                    for (int sl = 0; sl < nslices; ++sl) u += res[a + sl * slice + i];
                    out[ao + i] = from_f<T>(u);
                }
        }
    }
}

template <typename T, int QP, bool FAST>
__global__ __launch_bounds__(NTHREADS) void bmm_chunk_bwd_kernel(const bimamba2_params p, int nc, int nslices) {
    bmm_chunk_bwd_body<T, QP, FAST>(p, nc, nslices, BlockId{(int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z});
}

template <typename T>
static int launch_bmm_bwd_t(const bimamba2_params *p) {
    const int nc = nchunks(p), Q = p->chunk_size, nsl = dbdc_slices(p);
    dim3 grid((p->dstate + 63) / 64, (Q + 63) / 64, p->batch * nc * p->ngroups * 2);
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % 8 == 0 && b % 8 == 0 && c % 8 == 0; };
    const bool fast = sizeof(T) == 2 && (Q == 64 || Q == 128 || Q == 256) && p->dstate % 64 == 0 && nsl <= 8 && al(p->Bm) && al(p->Cm)
                      && mult(p->B_sb, p->B_sl, p->B_sg) && mult(p->C_sb, p->C_sl, p->C_sg) && al(p->dCB) && al(p->dCBT) && al(p->dBs)
                      && al(p->dCs) && al(p->dB) && al(p->dC) && mult(p->dB_sb, p->dB_sl, p->dC_sb) && p->dC_sl % 8 == 0;
#define BM2_BMMB(QPV)                                                                                                              \
    do {                                                                                                                       \
        if constexpr (sizeof(T) == 2) {                                                                                        \
            if (fast) { hipLaunchKernelGGL((bmm_chunk_bwd_kernel<T, QPV, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl); break; } \
        }                                                                                                                      \
        hipLaunchKernelGGL((bmm_chunk_bwd_kernel<T, QPV, false>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl);          \
    } while (0)
    if (Q <= 64) BM2_BMMB(64);
    else if (Q <= 128) BM2_BMMB(128);
    else BM2_BMMB(256);
#undef BM2_BMMB
    return check_launch();
}

int launch_bmm_chunk_bwd(const bimamba2_params *p) {
    switch (p->dtype) {
        case BIMAMBA2_F32: return launch_bmm_bwd_t<float>(p);
        case BIMAMBA2_BF16: return launch_bmm_bwd_t<bf16_t>(p);
        case BIMAMBA2_F16: return launch_bmm_bwd_t<f16_t>(p);
        default: return BIMAMBA2_EUNSUPPORTED;
    }
}

// =========================================================================================================
// one wave per (b, c, h); lane i owns positions 4i..4i+3.
//   da[q] = (within-chunk part from the tile vectors in da_intra) + sum_{s<q} v_f[s] + sum_{s>q} v_b[s] + sum_{t>=q} u_f[t] + sum_{t<=q} u_b[t]
//           + ddA_chunk_f + ddA_chunk_b
//   ddt' = da*A + ddt_direct ; through clamp and softplus -> ddt ; dA += sum da*dt' ; ddt_bias += sum ddt
// Partials per (b, c) go to red[(b*nc + c)*H + h] (dA) and red[B*nc*H + ...] (ddt_bias).
// =========================================================================================================
template <typename DT>
__device__ __forceinline__ void chunk_cumsum_bwd_body(const bimamba2_params &p, int nc, int nqt, int nsplit, BlockId bid) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = bid.x * 4 + wave, c = bid.y, b = bid.z;
    if (h >= p.nheads) return;
    const int Q = p.chunk_size, H = p.nheads;
    const int limit = min(Q, p.seqlen - c * Q);
    const int64_t o = (((int64_t)b * H + h) * nc + c) * Q;
    // Every load of the kernel goes out here, unconditionally and from clamped (valid) addresses, before anything is
    // used: a load that is waited for costs microseconds, and conditional loads get serialised by the compiler.
    float vf[4], vb[4], uf[4], ub[4], di[4], dtr[4], ddr[4];
    const int nplanes = ddt_direct_planes(p);
    const int64_t plane = (int64_t)p.batch * H * nc * Q;
    const DT *dt = reinterpret_cast<const DT *>(p.dt) + b * p.dt_sb + (int64_t)c * Q * p.dt_sl + h * p.dt_sh;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int qc = min(lane * 4 + e, limit - 1);
        vf[e] = p.v_f[o + qc];
        vb[e] = p.v_b[o + qc];
        uf[e] = p.u_f[o + qc];
        ub[e] = p.u_b[o + qc];
        ddr[e] = p.ddt_direct[o + qc];
        for (int pl = 1; pl < nplanes; ++pl) ddr[e] += p.ddt_direct[pl * plane + o + qc];    // one plane per headdim tile of the dx kernel
        dtr[e] = to_f(dt[(int64_t)qc * p.dt_sl]);
    }
    if (p.causal) {                   // single-direction operator: nothing wrote the reverse direction's terms
#pragma unroll
        for (int e = 0; e < 4; ++e) vb[e] = ub[e] = 0.f;
    }
    const float A = p.A[h];
    const float bias = p.has_dt_bias ? p.dt_bias[h] : 0.f;
    float chunk_term = 0.f;
    for (int s = 0; s < nsplit; ++s)
    {
        const float cf = p.ddA_chunk_f[(((int64_t)b * H + h) * nc + c) * nsplit + s], cr = p.ddA_chunk_b[(((int64_t)b * H + h) * nc + c) * nsplit + s];
        chunk_term += cf + (p.causal ? 0.f : cr);
    }
    // within-chunk part from the per-tile vectors of the dCB kernel; tile I = lane / 16 holds this lane's positions.
    // Four tiles per side at most (Q <= 256): tile indices past nqt are clamped for the loads and masked afterwards.
    const int I = lane >> 4, i0 = (lane & 15) * 4, Ic = min(I, nqt - 1);
    const float *tv = p.da_intra + (o / Q) * nqt * nqt * DCB_VEC;
    float4 colv[4], rowv[4], tot[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int ac = min(a, nqt - 1);
        colv[a] = *reinterpret_cast<const float4 *>(tv + (ac * nqt + Ic) * DCB_VEC + i0);          // [0] of tile (a, I)
        rowv[a] = *reinterpret_cast<const float4 *>(tv + (Ic * nqt + ac) * DCB_VEC + 64 + i0);     // [1] of tile (I, a)
#pragma unroll
        for (int bq = 0; bq < 4; ++bq) tot[a][bq] = *reinterpret_cast<const float4 *>(tv + (ac * nqt + min(bq, nqt - 1)) * DCB_VEC + i0);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (lane * 4 + e >= limit) vf[e] = vb[e] = uf[e] = ub[e] = 0.f;
        di[e] = 0.f;
    }
    {
        if (I < nqt) {
            auto add = [](float (&r)[4], const float4 &v) { r[0] += v.x; r[1] += v.y; r[2] += v.z; r[3] += v.w; };
            // the diagonal tile's difference vectors join the exclusive scans: cwf gets cw_f - rw_f, cwb gets cw_b - rw_b
            float cwf[4] = {0.f, 0.f, 0.f, 0.f}, cwb[4] = {0.f, 0.f, 0.f, 0.f}, rwf[4] = {0.f, 0.f, 0.f, 0.f}, rwb[4] = {0.f, 0.f, 0.f, 0.f};
            float between = 0.f;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                if (a < nqt) {
                    if (a == I) { add(cwf, colv[a]); add(cwb, rowv[a]); }
                    if (a > I) { add(cwf, colv[a]); add(rwb, rowv[a]); }
                    if (a < I) { add(rwf, rowv[a]); add(cwb, colv[a]); }
                    // tiles with this tile strictly between their row tile and column tile add their total
#pragma unroll
                    for (int bq = 0; bq < 4; ++bq)
                        if (bq < nqt && ((bq < I && I < a) || (a < I && I < bq))) between += tot[a][bq].x + tot[a][bq].y + tot[a][bq].z + tot[a][bq].w;
                }
            }
            between = row16_sum(between);
            // forward: exclusive prefix of cwf + inclusive suffix of rwf; reverse: inclusive prefix of rwb + exclusive suffix of cwb
            const float t_cwf = cwf[0] + cwf[1] + cwf[2] + cwf[3], t_rwb = rwb[0] + rwb[1] + rwb[2] + rwb[3];
            const float t_rwf = rwf[0] + rwf[1] + rwf[2] + rwf[3], t_cwb = cwb[0] + cwb[1] + cwb[2] + cwb[3];
            float ex = row16_incl_prefix(t_cwf) - t_cwf, in = row16_incl_prefix(t_rwb) - t_rwb;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                in += rwb[e];
                di[e] = between + ex + in;
                ex += cwf[e];
            }
            float exs = row16_incl_suffix(t_cwb) - t_cwb, ins = row16_incl_suffix(t_rwf) - t_rwf;
#pragma unroll
            for (int e = 3; e >= 0; --e) {
                ins += rwf[e];
                di[e] += exs + ins;
                exs += cwb[e];
            }
        }
    }
    // lane totals and cross-lane scans
    const float tvf = vf[0] + vf[1] + vf[2] + vf[3], tvb = vb[0] + vb[1] + vb[2] + vb[3];
    const float tuf = uf[0] + uf[1] + uf[2] + uf[3], tub = ub[0] + ub[1] + ub[2] + ub[3];
    const float vf_before = wave_incl_prefix(tvf, lane) - tvf;     // sum over lower lanes
    const float ub_before = wave_incl_prefix(tub, lane) - tub;
    const float vb_after = wave_incl_suffix(tvb, lane) - tvb;      // sum over higher lanes
    const float uf_after = wave_incl_suffix(tuf, lane) - tuf;
    float da[4];
    {
        float ex_vf = vf_before, in_ub = ub_before;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            in_ub += ub[e];
            da[e] = di[e] + ex_vf + in_ub + chunk_term;
            ex_vf += vf[e];
        }
        float ex_vb = vb_after, in_uf = uf_after;
#pragma unroll
        for (int e = 3; e >= 0; --e) {
            in_uf += uf[e];
            da[e] += ex_vb + in_uf;
            ex_vb += vb[e];
        }
    }
    DT *ddt = reinterpret_cast<DT *>(p.ddt);
    float sA = 0.f, sb = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int q = lane * 4 + e;
        if (q < limit) {
            const float pre = dtr[e] + bias;
            float d = pre;
            if (p.dt_softplus) d = d > 20.f ? d : log1pf(expf(d));
            const bool clamped = d < p.dt_min || d > p.dt_max;
            d = fminf(fmaxf(d, p.dt_min), p.dt_max);
            float g = da[e] * A + ddr[e];
            if (clamped) g = 0.f;
            if (p.dt_softplus && pre <= 20.f) g *= 1.f / (1.f + expf(-pre));
            ddt[((int64_t)b * p.seqlen + (int64_t)c * Q + q) * H + h] = from_f<DT>(g);
            sA += da[e] * d;
            sb += g;
        }
    }
    sA = wave_sum(sA);
    sb = wave_sum(sb);
    if (lane == 0) {
        p.red[(int64_t)(b * nc + c) * H + h] = sA;
        p.red[(int64_t)p.batch * nc * H + (int64_t)(b * nc + c) * H + h] = sb;
    }
}

template <typename DT>
__global__ __launch_bounds__(NTHREADS) void chunk_cumsum_bwd_kernel(const bimamba2_params p, int nc, int nqt, int nsplit) {
    chunk_cumsum_bwd_body<DT>(p, nc, nqt, nsplit, BlockId{(int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z});
}

// The last two kernels of the backward pass in one launch: the first `nbmm` workgroups do the work of
// bmm_chunk_bwd_kernel (16-bit path, chunk_size 256), the others that of chunk_cumsum_bwd_kernel.  Neither depends on the
// other, both are short and latency-bound, and together they fit the machine in one wave of workgroups.
template <typename T, typename DT, bool SLIM = false>
__global__ __launch_bounds__(NTHREADS) void bwd_tail_kernel(const bimamba2_params p, int nc, int nslices, int nqt, int nsplit, int nbmm,
                                                            int bmm_gy, int cs_gx, bool in16) {
    const int id = blockIdx.x;
    if (id < nbmm) {
        // bmm grid (1, bmm_gy, z).  The bmm_gy row tiles of one z = (which, b, c, g) stage the same K operand (the chunk's C or
        // B rows): consecutive ids are dealt round-robin to the 8 XCDs, so eight z at a time, one per XCD, go through their
        // row tiles (with the row tile fastest every XCD fetched every K operand: +100 MB of reads at 8 groups)
        const int nz = nbmm / bmm_gy, k = id >> 3;
        const BlockId bb = nz % 8 == 0 ? BlockId{0, k % bmm_gy, (k / bmm_gy) * 8 + (id & 7)} : BlockId{0, id % bmm_gy, id / bmm_gy};
        bmm_chunk_bwd_body<T, 256, true, SLIM>(p, nc, nslices, bb, in16);
    } else {
        const int k = id - nbmm;                  // cumsum grid (cs_gx, nc, batch)
        chunk_cumsum_bwd_body<DT>(p, nc, nqt, nsplit, BlockId{k % cs_gx, (k / cs_gx) % nc, k / (cs_gx * nc)});
    }
}

static bool bmm_bwd_fast(const bimamba2_params *p) {
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    auto mult = [](int64_t a, int64_t b, int64_t c) { return a % 8 == 0 && b % 8 == 0 && c % 8 == 0; };
    const int Q = p->chunk_size;
    return p->dtype != BIMAMBA2_F32 && (Q == 64 || Q == 128 || Q == 256) && p->dstate % 64 == 0 && dbdc_slices(p) <= 8 && al(p->Bm) &&
           al(p->Cm) && mult(p->B_sb, p->B_sl, p->B_sg) && mult(p->C_sb, p->C_sl, p->C_sg) && al(p->dCB) && al(p->dCBT) && al(p->dBs) &&
           al(p->dCs) && al(p->dB) && al(p->dC) && mult(p->dB_sb, p->dB_sl, p->dC_sb) && p->dC_sl % 8 == 0;
}

// whether launch_bwd_tail() exists for this problem
bool bwd_tail_merged(const bimamba2_params *p) { return bmm_bwd_fast(p) && p->chunk_size == 256 && p->dstate == 64; }

template <typename T>
static int launch_bwd_tail_t(const bimamba2_params *p, int nc, int nqt, int nsplit, bool in16) {
    const int bmm_gy = (p->chunk_size + 63) / 64, nbmm = bmm_gy * p->batch * nc * p->ngroups * 2;
    const int cs_gx = (p->nheads + 3) / 4, ncs = cs_gx * nc * p->batch;
    dim3 grid(nbmm + ncs);
    const int nsl = dbdc_slices(p);
    if (in16 && nsl <= 2) {
        switch (p->dt_dtype) {
            case BIMAMBA2_F32: hipLaunchKernelGGL((bwd_tail_kernel<T, float, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl, nqt, nsplit, nbmm, bmm_gy, cs_gx, in16); break;
            case BIMAMBA2_BF16: hipLaunchKernelGGL((bwd_tail_kernel<T, bf16_t, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl, nqt, nsplit, nbmm, bmm_gy, cs_gx, in16); break;
            case BIMAMBA2_F16: hipLaunchKernelGGL((bwd_tail_kernel<T, f16_t, true>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl, nqt, nsplit, nbmm, bmm_gy, cs_gx, in16); break;
            default: return BIMAMBA2_EUNSUPPORTED;
        }
        return check_launch();
    }
    switch (p->dt_dtype) {
        case BIMAMBA2_F32: hipLaunchKernelGGL((bwd_tail_kernel<T, float>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl, nqt, nsplit, nbmm, bmm_gy, cs_gx, in16); break;
        case BIMAMBA2_BF16: hipLaunchKernelGGL((bwd_tail_kernel<T, bf16_t>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl, nqt, nsplit, nbmm, bmm_gy, cs_gx, in16); break;
        case BIMAMBA2_F16: hipLaunchKernelGGL((bwd_tail_kernel<T, f16_t>), grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nsl, nqt, nsplit, nbmm, bmm_gy, cs_gx, in16); break;
        default: return BIMAMBA2_EUNSUPPORTED;
    }
    return check_launch();
}

// bmm_chunk_bwd + chunk_cumsum_bwd in one launch (the caller checked bwd_tail_merged()); reductions as in
// launch_chunk_cumsum_bwd
int launch_bwd_tail(const bimamba2_params *p, ReduceJobs *defer, bool in16) {
    const int nc = nchunks(p), nqt = (p->chunk_size + 63) / 64;
    const int PN = p->headdim * p->dstate;
    const int nsplit = (PN + SP_EPT * NTHREADS - 1) / (SP_EPT * NTHREADS);
    int rc = p->dtype == BIMAMBA2_BF16 ? launch_bwd_tail_t<bf16_t>(p, nc, nqt, nsplit, in16) : launch_bwd_tail_t<f16_t>(p, nc, nqt, nsplit, in16);
    if (rc) return rc;
    const int ni = p->batch * nc;
    defer->job[defer->n++] = ReduceJob{p->red, p->dA, ni, p->nheads, 1};
    if (p->has_dt_bias && p->ddt_bias) defer->job[defer->n++] = ReduceJob{p->red + (int64_t)ni * p->nheads, p->ddt_bias, ni, p->nheads, 1};
    return BIMAMBA2_OK;
}

int launch_chunk_cumsum_bwd(const bimamba2_params *p, ReduceJobs *defer) {
    const int nc = nchunks(p), nqt = (p->chunk_size + 63) / 64;
    const int PN = p->headdim * p->dstate;
    const int nsplit = (PN + SP_EPT * NTHREADS - 1) / (SP_EPT * NTHREADS);
    dim3 grid((p->nheads + 3) / 4, nc, p->batch);
    switch (p->dt_dtype) {
        case BIMAMBA2_F32: hipLaunchKernelGGL(chunk_cumsum_bwd_kernel<float>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt, nsplit); break;
        case BIMAMBA2_BF16: hipLaunchKernelGGL(chunk_cumsum_bwd_kernel<bf16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt, nsplit); break;
        case BIMAMBA2_F16: hipLaunchKernelGGL(chunk_cumsum_bwd_kernel<f16_t>, grid, dim3(NTHREADS), 0, stream_of(p), *p, nc, nqt, nsplit); break;
        default: return BIMAMBA2_EUNSUPPORTED;
    }
    int rc = check_launch();
    if (rc) return rc;
    const int ni = p->batch * nc;
    if (defer) {
        // the caller runs these together with its other reductions
        defer->job[defer->n++] = ReduceJob{p->red, p->dA, ni, p->nheads, 1};
        if (p->has_dt_bias && p->ddt_bias) defer->job[defer->n++] = ReduceJob{p->red + (int64_t)ni * p->nheads, p->ddt_bias, ni, p->nheads, 1};
        return BIMAMBA2_OK;
    }
    rc = launch_reduce(p->red, p->dA, ni, p->nheads, 1, stream_of(p));
    if (rc) return rc;
    if (p->has_dt_bias && p->ddt_bias) rc = launch_reduce(p->red + (int64_t)ni * p->nheads, p->ddt_bias, ni, p->nheads, 1, stream_of(p));
    return rc;
}

}  // namespace bm2
