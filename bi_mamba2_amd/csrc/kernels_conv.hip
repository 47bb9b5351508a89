// Non-causal depthwise conv1d + SiLU on channels-last activations (the step in front of the SSD operator in the BiMamba2
// layer; reference: src/ssd/modules.py:68-75 constructs nn.Conv1d(groups = channels, padding = d_conv // 2), :162-164
// applies it between two transposes and then the activation):
//
//   pre[b, l, c] = bias[c] + sum_k weight[c, k] * x[b, l + k - W/2, c]      (zero padding, W odd)
//   out          = pre * sigmoid(pre)
//
// The input is read as it lies in the projection's output (a strided (batch, seqlen, channels) view, channels
// contiguous): no transposes, no padded copy.  A thread owns VS consecutive channels and a run of positions; the W
// inputs under the filter sit in a register window that rotates with period W, so with the position loop unrolled by W
// every slot index is a constant; the loads of the next W positions are in flight while the current ones are used.
//
// Backward, one pass:  g = dout * silu'(pre) with pre recomputed from x;  dx[j] = sum_k weight[c, k] * g[j - k + W/2];
// dweight[c, k] = sum_{b, l} g[l] * x[l + k - W/2];  dbias[c] = sum g.  A second rotating window holds g.  Each thread
// leaves its dweight / dbias partial sums (over its own positions) in the workspace, [tile][channel][W + 1], and a
// column-parallel fixed-order sum adds the tiles up (no atomics).
#include "common.hpp"
#include "launch.hpp"

namespace bm2 {

namespace {

template <typename T, int VS> struct alignas(sizeof(T) * VS) ConvVec {
    T v[VS];
};

template <typename T, int VS> __device__ __forceinline__ ConvVec<T, VS> conv_load(const T *p) {
    return *reinterpret_cast<const ConvVec<T, VS> *>(p);
}

}  // namespace

// grid: ceil(batch * ntl * (channels / VS) / 256) workgroups of 256 threads; TL = positions per thread, a multiple of W
template <typename T, int W, int VS>
__global__ __launch_bounds__(NTHREADS) void conv1d_silu_fwd_kernel(const bimamba2_conv_params p, int ntl, int TL) {
    constexpr int H = W / 2;
    const int CV = p.channels / VS;
    const int64_t id = (int64_t)blockIdx.x * NTHREADS + threadIdx.x;
    const int cv = (int)(id % CV);
    const int64_t tile = id / CV;
    if (tile >= p.batch * ntl) return;
    const int lt = (int)(tile % ntl);
    const int64_t b = tile / ntl;
    const int L = (int)p.seqlen, c0 = cv * VS, l0 = lt * TL, l1 = min(l0 + TL, L);
    float w[W][VS], bias[VS];
#pragma unroll
    for (int i = 0; i < VS; ++i) {
        bias[i] = p.has_bias ? p.bias[c0 + i] : 0.f;
#pragma unroll
        for (int k = 0; k < W; ++k) w[k][i] = p.weight[(int64_t)(c0 + i) * W + k];
    }
    const T *xin = reinterpret_cast<const T *>(p.x) + b * p.x_sb + c0;
    T *out = reinterpret_cast<T *>(p.out) + (b * p.seqlen) * p.channels + c0;
    // unconditional load of position l clamped into the sequence; the caller masks what lies outside
    auto ld = [&](int l) { return conv_load<T, VS>(xin + (int64_t)min(max(l, 0), L - 1) * p.x_sl); };
    float win[W][VS];
#pragma unroll
    for (int j = 0; j < W - 1; ++j) {
        const int l = l0 - H + j;
        const ConvVec<T, VS> r = ld(l);
#pragma unroll
        for (int i = 0; i < VS; ++i) win[j][i] = (l >= 0 && l < L) ? to_f(r.v[i]) : 0.f;
    }
    ConvVec<T, VS> nxt[W];
#pragma unroll
    for (int u = 0; u < W; ++u) nxt[u] = ld(l0 + u + H);
    for (int q0 = l0; q0 < l1; q0 += W) {
        ConvVec<T, VS> cur[W];
#pragma unroll
        for (int u = 0; u < W; ++u) cur[u] = nxt[u];
#pragma unroll
        for (int u = 0; u < W; ++u) nxt[u] = ld(q0 + W + u + H);
#pragma unroll
        for (int u = 0; u < W; ++u) {
            const int q = q0 + u;
            if (q < l1) {
                const bool in = q + H < L;            // the newest input of the window: x[q + H]
#pragma unroll
                for (int i = 0; i < VS; ++i) win[(u + W - 1) % W][i] = in ? to_f(cur[u].v[i]) : 0.f;
                ConvVec<T, VS> o;
#pragma unroll
                for (int i = 0; i < VS; ++i) {
                    float a = bias[i];
#pragma unroll
                    for (int k = 0; k < W; ++k) a = __builtin_fmaf(w[k][i], win[(u + k) % W][i], a);
                    o.v[i] = from_f<T>(a * sigmoid_f(a));
                }
                *reinterpret_cast<ConvVec<T, VS> *>(out + (int64_t)q * p.channels) = o;
            }
        }
    }
}

// Tiled forward for 16-bit activations, channels a multiple of 64 and 16-byte aligned rows: a workgroup brings a tile of
// 64 positions (plus the filter's reach on both sides) x 64 channels into LDS with 16-byte loads, every thread walks
// 8 positions of one channel pair through a register window fed from there, and the results leave through LDS as 16-byte
// vectors.  Four times fewer memory instructions than the register kernel above, whose lanes move 4 bytes each.
constexpr int CONV_TP = 64, CONV_TC = 64;
template <typename T, int W>
__global__ __launch_bounds__(NTHREADS) void conv1d_silu_fwd_tiled_kernel(const bimamba2_conv_params p) {
    static_assert(sizeof(T) == 2, "16-bit activations");
    constexpr int H = W / 2, ROWS = CONV_TP + W - 1, SEG = CONV_TP / 8;
    __shared__ __attribute__((aligned(16))) T xs[ROWS * CONV_TC];
    __shared__ __attribute__((aligned(16))) T os[CONV_TP * CONV_TC];
    const int c0 = blockIdx.x * CONV_TC, l0 = blockIdx.y * CONV_TP;
    const int64_t b = blockIdx.z;
    const int L = (int)p.seqlen;
    const T *xin = reinterpret_cast<const T *>(p.x) + b * p.x_sb + c0;
    // this thread's channel pair and run of positions
    const int cp = threadIdx.x % 32, seg = threadIdx.x / 32;
    float w[W][2], bias[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        bias[i] = p.has_bias ? p.bias[c0 + 2 * cp + i] : 0.f;
#pragma unroll
        for (int k = 0; k < W; ++k) w[k][i] = p.weight[(int64_t)(c0 + 2 * cp + i) * W + k];
    }
    for (int u = threadIdx.x; u < ROWS * (CONV_TC / 8); u += NTHREADS) {
        const int r = u / (CONV_TC / 8), ch = (u % (CONV_TC / 8)) * 8, l = l0 - H + r;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (l >= 0 && l < L) v = *reinterpret_cast<const f32x4 *>(xin + (int64_t)l * p.x_sl + ch);
        *reinterpret_cast<f32x4 *>(xs + r * CONV_TC + ch) = v;
    }
    __syncthreads();
    typedef T Pair __attribute__((ext_vector_type(2)));
    const T *col = xs + (seg * SEG) * CONV_TC + 2 * cp;     // row q of the segment: positions l0 + seg*SEG + q - H .. + H
    float win[W][2];
#pragma unroll
    for (int j = 0; j < W - 1; ++j) {
        const Pair v = *reinterpret_cast<const Pair *>(col + j * CONV_TC);
        win[j][0] = to_f(v[0]); win[j][1] = to_f(v[1]);
    }
#pragma unroll
    for (int q = 0; q < SEG; ++q) {
        const Pair v = *reinterpret_cast<const Pair *>(col + (q + W - 1) * CONV_TC);
        win[(q + W - 1) % W][0] = to_f(v[0]); win[(q + W - 1) % W][1] = to_f(v[1]);
        Pair o;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            float a = bias[i];
#pragma unroll
            for (int k = 0; k < W; ++k) a = __builtin_fmaf(w[k][i], win[(q + k) % W][i], a);
            o[i] = from_f<T>(a * sigmoid_f(a));
        }
        *reinterpret_cast<Pair *>(os + (seg * SEG + q) * CONV_TC + 2 * cp) = o;
    }
    __syncthreads();
    T *out = reinterpret_cast<T *>(p.out) + (b * p.seqlen) * p.channels + c0;
    for (int u = threadIdx.x; u < CONV_TP * (CONV_TC / 8); u += NTHREADS) {
        const int r = u / (CONV_TC / 8), ch = (u % (CONV_TC / 8)) * 8, l = l0 + r;
        if (l < L) *reinterpret_cast<f32x4 *>(out + (int64_t)l * p.channels + ch) = *reinterpret_cast<const f32x4 *>(os + r * CONV_TC + ch);
    }
}

// Steps t = 0 .. TL + 2H - 1 visit positions l = l0 - H + t: g[l] is formed (needs x[l - H .. l + H]) and dx[l - H] leaves.
template <typename T, int W, int VS>
__global__ __launch_bounds__(NTHREADS) void conv1d_silu_bwd_kernel(const bimamba2_conv_params p, int ntl, int TL, float *part) {
    constexpr int H = W / 2;
    const int CV = p.channels / VS;
    const int64_t id = (int64_t)blockIdx.x * NTHREADS + threadIdx.x;
    const int cv = (int)(id % CV);
    const int64_t tile = id / CV;
    if (tile >= p.batch * ntl) return;
    const int lt = (int)(tile % ntl);
    const int64_t b = tile / ntl;
    const int L = (int)p.seqlen, c0 = cv * VS, l0 = lt * TL, l1 = min(l0 + TL, L);
    float w[W][VS], bias[VS];
#pragma unroll
    for (int i = 0; i < VS; ++i) {
        bias[i] = p.has_bias ? p.bias[c0 + i] : 0.f;
#pragma unroll
        for (int k = 0; k < W; ++k) w[k][i] = p.weight[(int64_t)(c0 + i) * W + k];
    }
    const T *xin = reinterpret_cast<const T *>(p.x) + b * p.x_sb + c0;
    const T *din = reinterpret_cast<const T *>(p.dout) + b * p.dout_sb + c0;
    const int64_t dx_sl = p.dx_sl ? p.dx_sl : p.channels, dx_sb = p.dx_sl ? p.dx_sb : p.seqlen * p.channels;
    T *dx = reinterpret_cast<T *>(p.dx) + b * dx_sb + c0;
    auto ldx = [&](int l) { return conv_load<T, VS>(xin + (int64_t)min(max(l, 0), L - 1) * p.x_sl); };
    auto ldd = [&](int l) { return conv_load<T, VS>(din + (int64_t)min(max(l, 0), L - 1) * p.dout_sl); };
    float xw[W][VS], gw[W][VS], dw[W][VS], db[VS];
#pragma unroll
    for (int i = 0; i < VS; ++i) {
        db[i] = 0.f;
#pragma unroll
        for (int k = 0; k < W; ++k) { dw[k][i] = 0.f; gw[k][i] = 0.f; }
    }
    const int lb = l0 - H;                            // position of step 0
#pragma unroll
    for (int j = 0; j < W - 1; ++j) {
        const int l = lb - H + j;
        const ConvVec<T, VS> r = ldx(l);
#pragma unroll
        for (int i = 0; i < VS; ++i) xw[j][i] = (l >= 0 && l < L) ? to_f(r.v[i]) : 0.f;
    }
    ConvVec<T, VS> nx[W], nd[W];
#pragma unroll
    for (int u = 0; u < W; ++u) { nx[u] = ldx(lb + u + H); nd[u] = ldd(lb + u); }
    const int lend = l1 + H;                          // one past the last position visited
    for (int s0 = lb; s0 < lend; s0 += W) {
        ConvVec<T, VS> cx[W], cd[W];
#pragma unroll
        for (int u = 0; u < W; ++u) { cx[u] = nx[u]; cd[u] = nd[u]; }
#pragma unroll
        for (int u = 0; u < W; ++u) { nx[u] = ldx(s0 + W + u + H); nd[u] = ldd(s0 + W + u); }
#pragma unroll
        for (int u = 0; u < W; ++u) {
            const int l = s0 + u;
            if (l < lend) {
                const bool xin_ok = l + H >= 0 && l + H < L, lin = l >= 0 && l < L, own = l >= l0 && l < l1;
#pragma unroll
                for (int i = 0; i < VS; ++i) xw[(u + W - 1) % W][i] = xin_ok ? to_f(cx[u].v[i]) : 0.f;
#pragma unroll
                for (int i = 0; i < VS; ++i) {
                    float a = bias[i];
#pragma unroll
                    for (int k = 0; k < W; ++k) a = __builtin_fmaf(w[k][i], xw[(u + k) % W][i], a);
                    const float sg = sigmoid_f(a);
                    const float g = lin ? to_f(cd[u].v[i]) * sg * (1.f + a * (1.f - sg)) : 0.f;
                    gw[u][i] = g;
                    if (own) {
                        db[i] += g;
#pragma unroll
                        for (int k = 0; k < W; ++k) dw[k][i] = __builtin_fmaf(g, xw[(u + k) % W][i], dw[k][i]);
                    }
                }
                const int j = l - H;                  // dx[j] = sum_k w[k] g[l - k]
                if (j >= l0 && j < l1) {
                    ConvVec<T, VS> o;
#pragma unroll
                    for (int i = 0; i < VS; ++i) {
                        float a = 0.f;
#pragma unroll
                        for (int k = 0; k < W; ++k) a = __builtin_fmaf(w[k][i], gw[(u - k + W) % W][i], a);
                        o.v[i] = from_f<T>(a);
                    }
                    *reinterpret_cast<ConvVec<T, VS> *>(dx + (int64_t)j * dx_sl) = o;
                }
            }
        }
    }
    float *pp = part + (tile * p.channels + c0) * (W + 1);
#pragma unroll
    for (int i = 0; i < VS; ++i) {
#pragma unroll
        for (int k = 0; k < W; ++k) pp[i * (W + 1) + k] = dw[k][i];
        pp[i * (W + 1) + W] = db[i];
    }
}

// positions per thread: forward 4 filter widths, backward 8 (fewer, longer runs: fewer partial sums to add up)
static inline int conv_tile_len(const bimamba2_conv_params *p, bool bwd) { return p->width * (bwd ? 8 : 4); }
static inline int conv_ntl(const bimamba2_conv_params *p, bool bwd) {
    const int tl = conv_tile_len(p, bwd);
    return (int)((p->seqlen + tl - 1) / tl);
}

size_t conv_workspace_bytes(const bimamba2_conv_params *p) {
    // backward: [batch * ntl][channels][width + 1] partial sums, then the summed [channels][width + 1]
    return ((size_t)p->batch * conv_ntl(p, true) + 1) * p->channels * (p->width + 1) * sizeof(float);
}

// sums[c][W + 1] -> dweight[c][W], dbias[c]
__global__ void conv_split_kernel(const float *sums, float *dweight, float *dbias, int channels, int W) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= channels * (W + 1)) return;
    const int c = i / (W + 1), k = i % (W + 1);
    if (k < W) dweight[c * W + k] = sums[i];
    else if (dbias) dbias[c] = sums[i];
}

template <typename T, int W, int VS>
static int launch_conv_w(const bimamba2_conv_params *p, bool bwd) {
    const int ntl = conv_ntl(p, bwd), tl = conv_tile_len(p, bwd);
    const int64_t threads = (int64_t)p->batch * ntl * (p->channels / VS);
    const int64_t blocks = (threads + NTHREADS - 1) / NTHREADS;
    if (blocks <= 0 || blocks > 0x7fffffff) return BIMAMBA2_EUNSUPPORTED;
    hipStream_t s = reinterpret_cast<hipStream_t>(p->stream);
    if (!bwd) {
        if constexpr (sizeof(T) == 2 && VS > 1) {
            auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
            if (p->channels % CONV_TC == 0 && al16(p->x) && al16(p->out) && p->x_sb % 8 == 0 && p->x_sl % 8 == 0 && p->batch <= 65535) {
                const dim3 grid(p->channels / CONV_TC, (unsigned)((p->seqlen + CONV_TP - 1) / CONV_TP), (unsigned)p->batch);
                hipLaunchKernelGGL((conv1d_silu_fwd_tiled_kernel<T, W>), grid, dim3(NTHREADS), 0, s, *p);
                return check_launch();
            }
        }
        hipLaunchKernelGGL((conv1d_silu_fwd_kernel<T, W, VS>), dim3((unsigned)blocks), dim3(NTHREADS), 0, s, *p, ntl, tl);
        return check_launch();
    }
    float *part = reinterpret_cast<float *>(p->workspace);
    const int64_t ntiles = (int64_t)p->batch * ntl;
    const int nj = p->channels * (W + 1);
    float *sums = part + ntiles * nj;
    hipLaunchKernelGGL((conv1d_silu_bwd_kernel<T, W, VS>), dim3((unsigned)blocks), dim3(NTHREADS), 0, s, *p, ntl, tl, part);
    int rc = check_launch();
    if (rc) return rc;
    rc = launch_colsum(part, sums, (int)ntiles, nj, s);
    if (rc) return rc;
    hipLaunchKernelGGL(conv_split_kernel, dim3((nj + 255) / 256), dim3(256), 0, s, sums, p->dweight, p->has_bias ? p->dbias : nullptr,
                       p->channels, W);
    return check_launch();
}

template <typename T, int VS>
static int launch_conv_vs(const bimamba2_conv_params *p, bool bwd) {
    auto al = [](const void *q, size_t a) { return (reinterpret_cast<uintptr_t>(q) % a) == 0; };
    const size_t va = sizeof(T) * VS;
    bool vec = p->channels % VS == 0 && al(p->x, va) && p->x_sb % VS == 0 && p->x_sl % VS == 0;
    if (bwd) vec = vec && al(p->dout, va) && p->dout_sb % VS == 0 && p->dout_sl % VS == 0 && al(p->dx, va) && p->dx_sb % VS == 0 && p->dx_sl % VS == 0;
    else vec = vec && al(p->out, va);
#define BM2_CONV(WV)                                                      \
    case WV: return vec ? launch_conv_w<T, WV, VS>(p, bwd) : launch_conv_w<T, WV, 1>(p, bwd)
    switch (p->width) {
        BM2_CONV(1);
        BM2_CONV(3);
        BM2_CONV(5);
        BM2_CONV(7);
        BM2_CONV(9);
        default: return BIMAMBA2_EUNSUPPORTED;
    }
#undef BM2_CONV
}

// two channels per thread when the rows allow it (else one): measured faster than four or eight - the backward pass has
// three register windows plus the filter-gradient sums per channel, and more, narrower threads hide the load latency better
template <typename T>
static int launch_conv_t(const bimamba2_conv_params *p, bool bwd) {
    return launch_conv_vs<T, 2>(p, bwd);
}

// ---- several small element-wise conversions in one launch (bimamba2_cast_many) -------------------------------------
namespace {
__device__ __forceinline__ float cast_load(const void *src, int dtype, int64_t i) {
    if (dtype == BIMAMBA2_F32) return reinterpret_cast<const float *>(src)[i];
    if (dtype == BIMAMBA2_BF16) return to_f(reinterpret_cast<const bf16_t *>(src)[i]);
    return to_f(reinterpret_cast<const f16_t *>(src)[i]);
}
__device__ __forceinline__ void cast_store(void *dst, int dtype, int64_t i, float v) {
    if (dtype == BIMAMBA2_F32) reinterpret_cast<float *>(dst)[i] = v;
    else if (dtype == BIMAMBA2_BF16) reinterpret_cast<bf16_t *>(dst)[i] = from_f<bf16_t>(v);
    else reinterpret_cast<f16_t *>(dst)[i] = from_f<f16_t>(v);
}
}  // namespace

// blocks are dealt to the items in order: item k owns ceil(n_k / 256) of them
__global__ __launch_bounds__(NTHREADS) void cast_many_kernel(const bimamba2_cast_params p) {
    int blk = blockIdx.x, k = 0;
    for (; k < p.count; ++k) {
        const int nb = (int)((p.item[k].n + NTHREADS - 1) / NTHREADS);
        if (blk < nb) break;
        blk -= nb;
    }
    if (k >= p.count) return;
    const bimamba2_cast_item &it = p.item[k];
    const int64_t i = (int64_t)blk * NTHREADS + threadIdx.x;
    if (i >= it.n) return;
    float v = cast_load(it.src, it.src_dtype, i);
    if (it.op == BIMAMBA2_CAST_NEG_EXP) v = -expf(v);
    else if (it.op == BIMAMBA2_CAST_MUL) v *= it.aux[i];
    cast_store(it.dst, it.dst_dtype, i, v);
}

int launch_cast_many(const bimamba2_cast_params *p) {
    int64_t blocks = 0;
    for (int k = 0; k < p->count; ++k) blocks += (p->item[k].n + NTHREADS - 1) / NTHREADS;
    if (blocks == 0) return BIMAMBA2_OK;
    if (blocks > 0x7fffffff) return BIMAMBA2_EUNSUPPORTED;
    hipLaunchKernelGGL(cast_many_kernel, dim3((unsigned)blocks), dim3(NTHREADS), 0, reinterpret_cast<hipStream_t>(p->stream), *p);
    return check_launch();
}

int launch_conv1d_silu(const bimamba2_conv_params *p, bool bwd) {
    switch (p->dtype) {
        case BIMAMBA2_F32: return launch_conv_t<float>(p, bwd);
        case BIMAMBA2_BF16: return launch_conv_t<bf16_t>(p, bwd);
        case BIMAMBA2_F16: return launch_conv_t<f16_t>(p, bwd);
        default: return BIMAMBA2_EUNSUPPORTED;
    }
}

}  // namespace bm2
