// Shared device helpers for the gfx950 kernels: element types, 16x16 MFMA fragments, LDS tile loaders,
// wavefront scans.  Wave size is 64; every kernel here runs 256 threads = 4 waves per workgroup.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "../../include/bimamba2.h"

namespace bm2 {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int NTHREADS = 256;
constexpr int BK = 32;          // K extent of one LDS tile

constexpr float LOG2E = 1.4426950408889634f;       // exponentials are taken as 2^(x * LOG2E): one v_exp_f32

__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(bf16_t v) { return static_cast<float>(v); }
__device__ __forceinline__ float to_f(f16_t v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f(float v) { return static_cast<T>(v); }

// ---- direct global -> LDS loads (global_load_lds): lane l's 16 bytes land at the wave-uniform LDS address + 16*l ----
typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *gbl_ptr_t;
__device__ __forceinline__ void load16_to_lds(const void *src, void *lds_wave_base) {
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)lds_wave_base, 16, 0, 0);
}
// load16_to_lds(base + off) with the address in the scalar-base form: `base` wave-uniform, `off` this lane's 32-bit byte
// offset.  The offset passes through an empty asm right in front of the load, which keeps the 64-bit add next to the load
// (hoisted into another block it could not be folded into the instruction and would cost two registers per address).
// NT: the lines are not kept in the caches (data that no later kernel of the pass reads).
template <bool NT = false>
__device__ __forceinline__ void load16_to_lds_at(const char *base, unsigned off, void *lds_wave_base) {
    asm volatile("" : "+v"(off));
    if constexpr (NT) __builtin_amdgcn_global_load_lds((gbl_ptr_t)(base + off), (lds_ptr_t)lds_wave_base, 16, 0, 2);
    else load16_to_lds(base + off, lds_wave_base);
}

// A wave-uniform pointer, made visibly so (through 64-bit address arithmetic the compiler loses sight of it and would build
// the address per lane): base + 32-bit lane offset then takes the scalar-base form of the memory instructions.
__device__ __forceinline__ const char *uniform_ptr(const void *ptr) {
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const char *>(((uint64_t)hi << 32) | lo);
}

// at most N vector-memory operations of this wave outstanding; lgkmcnt / expcnt fields left at "no wait"
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// Global loads the compiler does not know of: it neither moves them (a load it knows of may be sunk below later requests
// and then be waited for with vmcnt(0), which drains every request in flight) nor waits for them.  The caller waits with
// wait_vmcnt<N>() and then ties each value to that wait with raw_lds_use() before its first use.
__device__ __forceinline__ float raw_global_load_f32(const float *p) {
    float v;
    asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <typename V, bool NT = false> __device__ __forceinline__ V raw_global_load_b128(const void *p) {   // NT: non-temporal
    static_assert(sizeof(V) == 16, "16-byte value");
    V v;
    if constexpr (NT) asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(v) : "v"(p) : "memory");
    else asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ unsigned raw_global_load_u16(const void *p) {      // zero-extended 16 bits
    unsigned v;
    asm volatile("global_load_ushort %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}

// ---- row-major tiles as MFMA operands: LDS transpose reads ------------------------------------------------------
// A tile of 16-bit elements lies in LDS as it lies in global memory, [k][n] with n contiguous (rows of 64 elements,
// 128 bytes), brought there by direct loads.  Its 16-byte chunks are swizzled, chunk c of row k sits at position
// c ^ tile64_swz(k), which keeps the reads below (4 rows x 32 bytes per 16 lanes, rows 8 apart for the next 16 lanes)
// off each other's banks.
// ds_read_b64_tr_b16 works on groups of 16 lanes: lane s supplies the address of 4 consecutive elements and lane j
// receives element j % 4 of the lanes j / 4, j / 4 + 4, j / 4 + 8, j / 4 + 12.  Pointing lane s at row k0 + s / 4,
// columns n0 + 4 * (s % 4) .. + 3 therefore hands lane j the elements [k0 .. k0 + 3][n0 + j]: four consecutive k of
// "its" column, which is what an MFMA operand holds.  Two such reads give the 8 k of one 16x16x32 operand.
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ int tile64_swz(int k) { return (k & 7) ^ ((k >> 1) & 4); }
// byte offset inside a swizzled [rows][64] 16-bit tile of the 4 elements (k, n .. n + 3), n a multiple of 4
__device__ __forceinline__ int tile64_tr_offset(int k, int n) {
    return k * 128 + ((((n >> 3) ^ tile64_swz(k)) << 4) | ((n & 4) << 1));
}
// fragment of lane (lr = lane % 16, lg = lane / 16): k = k0 + 8 * lg .. + 7 of column n0 + lr
template <typename Frag> __device__ __forceinline__ Frag tile64_tr_frag(const void *tile, int k0, int n0, int lr, int lg) {
    typedef __attribute__((address_space(3))) i16x4 *lds_i16x4_ptr;
    const char *t = reinterpret_cast<const char *>(tile);
    const int k = k0 + 8 * lg + (lr >> 2), n = n0 + 4 * (lr & 3);
    const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(t + tile64_tr_offset(k, n)));
    const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_ptr)(t + tile64_tr_offset(k + 4, n)));
    const i16x8 f = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(Frag, f);
}
// Requests rows [0, nrows) x 64 elements of a row-major global tile into such an LDS image: the calling wave brings the
// units wave, wave + nwaves, ... of 64 lanes x 16 bytes (8 rows each); rows >= rvalid read row rvalid - 1.
template <typename T>
__device__ __forceinline__ void tile64_request(T *tile, const T *src, int64_t row_stride, int nrows, int rvalid, int wave, int nwaves,
                                               int lane) {
    static_assert(sizeof(T) == 2, "16-bit tiles");
    for (int u = wave; u < nrows / 8; u += nwaves) {
        const int row = u * 8 + (lane >> 3);
        load16_to_lds(src + (int64_t)min(row, rvalid - 1) * row_stride + (((lane & 7) ^ tile64_swz(row)) << 3), tile + u * 512);
    }
}

// ---- LDS accesses issued from inline assembly ---------------------------------------------------------------
// While a direct global->LDS load (global_load_lds) is in flight, the compiler makes every LDS access it knows of wait for
// ALL outstanding vector memory operations, which defeats prefetching through LDS.  These accessors hide the DS
// instruction from it.  Protocol: raw_lds_read / raw_lds_write any number of times, then raw_lds_wait(), then
// raw_lds_use(v) on every value read before its first use (the empty asm ties the value to the wait, in program order).
// A value read this way must reach its raw_lds_use() under ONE name: a copy (`r = f`) made before the wait is the same
// value to the compiler, the second raw_lds_use() then needs a register copy, and that copy may be placed in front of the
// wait, where the register still holds what was there before the read.
// With RAW = false they are ordinary accesses and the other two are no-ops.
__device__ __forceinline__ unsigned lds_addr(const void *p) {
    return (unsigned)(size_t)(const __attribute__((address_space(3))) void *)p;
}
template <typename V, bool RAW = true> __device__ __forceinline__ V raw_lds_read(const void *p) {
    if constexpr (!RAW) return *reinterpret_cast<const V *>(p);
    else {
        V v;
        static_assert(sizeof(V) == 16 || sizeof(V) == 4, "raw_lds_read: 4 or 16 bytes");
        if constexpr (sizeof(V) == 16) asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(lds_addr(p)) : "memory");
        else asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(lds_addr(p)) : "memory");
        return v;
    }
}
// the same on an LDS byte address with a compile-time offset (goes into the instruction's offset field)
template <typename V, int OFF> __device__ __forceinline__ V raw_lds_read_at(unsigned addr) {
    V v;
    static_assert(sizeof(V) == 16 || sizeof(V) == 4, "raw_lds_read_at: 4 or 16 bytes");
    static_assert(OFF >= 0 && OFF < 65536, "DS offset field is 16 bits");
    if constexpr (sizeof(V) == 16) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    else asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
// LDS transpose read (see tile64_tr_frag) in the same raw form
template <int OFF> __device__ __forceinline__ i16x4 raw_lds_tr16_read_at(unsigned addr) {
    i16x4 v;
    static_assert(OFF >= 0 && OFF < 65536, "DS offset field is 16 bits");
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}
template <int OFF> __device__ __forceinline__ void raw_lds_write_at(unsigned addr, float v) {
    static_assert(OFF >= 0 && OFF < 65536, "DS offset field is 16 bits");
    asm volatile("ds_write_b32 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void raw_lds_write16_at(unsigned addr, _Float16 v) {
    static_assert(OFF >= 0 && OFF < 65536, "DS offset field is 16 bits");
    asm volatile("ds_write_b16 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int OFF> __device__ __forceinline__ void raw_lds_write128_at(unsigned addr, f32x4 v) {
    static_assert(OFF >= 0 && OFF < 65536, "DS offset field is 16 bits");
    asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <bool RAW = true> __device__ __forceinline__ void raw_lds_write(float *p, float v) {
    if constexpr (!RAW) *p = v;
    else asm volatile("ds_write_b32 %0, %1" ::"v"(lds_addr(p)), "v"(v) : "memory");
}
template <bool RAW = true> __device__ __forceinline__ void raw_lds_wait() {
    if constexpr (RAW) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}
// at most N LDS operations of this wave outstanding (they complete in order): the oldest reads can be used while the
// younger ones are still under way
template <int N> __device__ __forceinline__ void raw_lds_wait_n() {
    static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit field");
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}
// Workgroup barrier to go with them: __syncthreads() carries fences that drain every outstanding vector memory operation
// when a direct global->LDS load is in flight; the bare barrier does not.  All LDS traffic around it must be raw and
// settled with raw_lds_wait() (writes) resp. the caller's own vmcnt wait (direct loads) beforehand.
template <bool RAW = true> __device__ __forceinline__ void raw_lds_barrier() {
    if constexpr (RAW) __builtin_amdgcn_s_barrier();
    else __syncthreads();
}
template <bool RAW = true, typename V> __device__ __forceinline__ void raw_lds_use(V &v) {
    if constexpr (RAW) asm volatile("" : "+v"(v));
}

// ---- MFMA 16x16 fragments -----------------------------------------------------------------------------
// Output tile D (16x16, f32): lane l holds rows 4*(l/16)+i (i=0..3) of column l%16.
// A operand: lane l holds KPL consecutive k of row l%16 starting at KPL*(l/16); B operand likewise for
// column l%16.  Both operands use the same k mapping, so any consistent mapping gives the same product.
template <typename T> struct Mma;
template <> struct Mma<float> {
    static constexpr int KPL = 1, KSTEP = 4, LD = BK + 4;
    typedef float Frag;
    static __device__ __forceinline__ Frag load(const float *p) { return *p; }
    static __device__ __forceinline__ Frag pack(const float *a) { return a[0]; }
    static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<bf16_t> {
    static constexpr int KPL = 8, KSTEP = 32, LD = BK + 8;
    typedef bf16x8 Frag;
    static __device__ __forceinline__ Frag load(const bf16_t *p) { return *reinterpret_cast<const bf16x8 *>(p); }
    static __device__ __forceinline__ Frag pack(const float *a) {
        Frag f;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = static_cast<bf16_t>(a[i]);
        return f;
    }
    static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<f16_t> {
    static constexpr int KPL = 8, KSTEP = 32, LD = BK + 8;
    typedef f16x8 Frag;
    static __device__ __forceinline__ Frag load(const f16_t *p) { return *reinterpret_cast<const f16x8 *>(p); }
    static __device__ __forceinline__ Frag pack(const float *a) {
        Frag f;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = static_cast<f16_t>(a[i]);
        return f;
    }
    static __device__ __forceinline__ f32x4 mma(Frag a, Frag b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
};

// acc[j] += A(16 rows at As) * B(16 cols at Bs + 16*j rows)^T over one BK-wide LDS tile.
// As points at the first of the wave's 16 rows ([row][k], leading dimension LD); Bs at the first of NJ*16
// columns stored [col][k].
// KW is the K extent of the LDS tiles (multiple of BK); their leading dimension is KW + (LD - BK).
template <typename T, int NJ, int KW = BK>
__device__ __forceinline__ void mma_tile(f32x4 (&acc)[NJ], const T *As, const T *Bs, int lane) {
    typedef Mma<T> M;
    constexpr int LD = M::LD - BK + KW;
    const int r = lane & 15, kq = (lane >> 4) * M::KPL;
#pragma unroll
    for (int k0 = 0; k0 < KW; k0 += M::KSTEP) {
        typename M::Frag a = M::load(As + r * LD + k0 + kq);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            typename M::Frag b = M::load(Bs + (16 * j + r) * LD + k0 + kq);
            acc[j] = M::mma(a, b, acc[j]);
        }
    }
}

// ---- global -> LDS tile loaders -----------------------------------------------------------------------
template <typename S> struct Vec16 {
    static constexpr int N = 16 / sizeof(S);
    S v[N];
};

template <typename S> __device__ __forceinline__ bool aligned16(const S *p, int64_t stride_elems) {
    return ((reinterpret_cast<uintptr_t>(p) | static_cast<uintptr_t>(stride_elems * sizeof(S))) & 15) == 0;
}

// dst[r][k] = f(r, k, src[r*rs + k]) for r < ROWS, k < KW; elements with r >= rvalid or k >= kvalid are 0
// (f is still applied to the 0).  Source is contiguous along k.
template <typename T, typename S, int ROWS, int KW = BK, class F>
__device__ __forceinline__ void tile_load_kcontig(T *dst, const S *src, int64_t rs, int rvalid, int kvalid, F f) {
    constexpr int VS = 16 / sizeof(S), KV = KW / VS, LD = Mma<T>::LD - BK + KW;
    const bool vec = aligned16(src, rs);
    for (int idx = threadIdx.x; idx < ROWS * KV; idx += blockDim.x) {
        const int r = idx / KV, k0 = (idx % KV) * VS;
        float v[VS];
        if (vec && r < rvalid && k0 + VS <= kvalid) {
            Vec16<S> raw = *reinterpret_cast<const Vec16<S> *>(src + r * rs + k0);
#pragma unroll
            for (int i = 0; i < VS; ++i) v[i] = to_f(raw.v[i]);
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i) v[i] = (r < rvalid && k0 + i < kvalid) ? to_f(src[r * rs + k0 + i]) : 0.f;
        }
        struct alignas(sizeof(T) * VS) Out { T v[VS]; } o;
#pragma unroll
        for (int i = 0; i < VS; ++i) o.v[i] = from_f<T>(f(r, k0 + i, v[i]));
        *reinterpret_cast<Out *>(dst + r * LD + k0) = o;
    }
}

// dst[r][k] = f(r, k, src[k*ks + r]): the source is contiguous along r (transposing load).
template <typename T, typename S, int ROWS, class F>
__device__ __forceinline__ void tile_load_rcontig(T *dst, const S *src, int64_t ks, int rvalid, int kvalid, F f) {
    constexpr int VS = 16 / sizeof(S), RV = ROWS / VS, LD = Mma<T>::LD;
    const bool vec = aligned16(src, ks);
    for (int idx = threadIdx.x; idx < BK * RV; idx += blockDim.x) {
        const int k = idx / RV, r0 = (idx % RV) * VS;
        float v[VS];
        if (vec && k < kvalid && r0 + VS <= rvalid) {
            Vec16<S> raw = *reinterpret_cast<const Vec16<S> *>(src + k * ks + r0);
#pragma unroll
            for (int i = 0; i < VS; ++i) v[i] = to_f(raw.v[i]);
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i) v[i] = (k < kvalid && r0 + i < rvalid) ? to_f(src[k * ks + r0 + i]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < VS; ++i) dst[(r0 + i) * LD + k] = from_f<T>(f(r0 + i, k, v[i]));
    }
}

// same, writing two tiles with two functors from one read of the source
template <typename T, typename S, int ROWS, class F1, class F2>
__device__ __forceinline__ void tile_load_rcontig2(T *dst1, T *dst2, const S *src, int64_t ks, int rvalid,
                                                   int kvalid, F1 f1, F2 f2) {
    constexpr int VS = 16 / sizeof(S), RV = ROWS / VS, LD = Mma<T>::LD;
    const bool vec = aligned16(src, ks);
    for (int idx = threadIdx.x; idx < BK * RV; idx += blockDim.x) {
        const int k = idx / RV, r0 = (idx % RV) * VS;
        float v[VS];
        if (vec && k < kvalid && r0 + VS <= rvalid) {
            Vec16<S> raw = *reinterpret_cast<const Vec16<S> *>(src + k * ks + r0);
#pragma unroll
            for (int i = 0; i < VS; ++i) v[i] = to_f(raw.v[i]);
        } else {
#pragma unroll
            for (int i = 0; i < VS; ++i) v[i] = (k < kvalid && r0 + i < rvalid) ? to_f(src[k * ks + r0 + i]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < VS; ++i) {
            dst1[(r0 + i) * LD + k] = from_f<T>(f1(r0 + i, k, v[i]));
            dst2[(r0 + i) * LD + k] = from_f<T>(f2(r0 + i, k, v[i]));
        }
    }
}

// ---- transposing stage: global [k][r] -> LDS image addressed by (r, k) ----------------------------------
// LDS image of the K operand: element (r, k) of a [R][KTOT] matrix lives at r*LDX + (16-byte chunk of k, XORed
// with (r/VS)&7) so that neither the staging writes (rows VS apart) nor the fragment reads (consecutive rows)
// pile up on the same banks.
template <typename T, int LDX>
__device__ __forceinline__ int xt_index(int r, int k) {
    constexpr int VS = 16 / sizeof(T);
    const int chunk = (k / VS) ^ ((r / VS) & 7);
    return r * LDX + chunk * VS + (k % VS);
}

// Stage src[k][r] (r contiguous, row stride ks) for k < KTOT, r < RTOT into dst as (r, k), scaled by scale(k);
// rows k >= kvalid and columns r >= rvalid read as 0.  Each thread moves VS x VS blocks: VS 16-byte reads along r,
// transposed in registers, VS 16-byte LDS writes along k.
// FAST: every 16-byte read is known to be aligned and inside the column range; rows past kvalid are read from the
// last valid row and zeroed by scale().
// The source element type S may differ from T (float32 states staged as 16-bit operands): a thread moves a block of
// VK = 16/sizeof(T) rows (k) by VR = 16/sizeof(S) columns (r).
template <typename T, int KTOT, int RTOT, int LDX, bool FAST, typename S, class F>
__device__ __forceinline__ void stage_transposed(T *dst, const S *src, int64_t ks, int kvalid, int rvalid, F scale) {
    constexpr int VK = 16 / sizeof(T), VR = 16 / sizeof(S), RB = RTOT / VR, NB = (KTOT / VK) * RB;
    const bool vec = FAST || aligned16(src, ks);
    for (int blk = threadIdx.x; blk < NB; blk += blockDim.x) {
        const int rb = blk % RB, kb = blk / RB;
        float v[VK][VR];
#pragma unroll
        for (int kk = 0; kk < VK; ++kk) {
            const int k = kb * VK + kk;
            const S *row = src + (int64_t)(FAST ? min(k, kvalid - 1) : k) * ks + rb * VR;
            if (FAST || (vec && k < kvalid && rb * VR + VR <= rvalid)) {
                Vec16<S> raw = *reinterpret_cast<const Vec16<S> *>(row);
#pragma unroll
                for (int i = 0; i < VR; ++i) v[kk][i] = to_f(raw.v[i]);
            } else {
#pragma unroll
                for (int i = 0; i < VR; ++i) v[kk][i] = (k < kvalid && rb * VR + i < rvalid) ? to_f(row[i]) : 0.f;
            }
            const float sc = scale(k);
#pragma unroll
            for (int i = 0; i < VR; ++i) v[kk][i] *= sc;
        }
#pragma unroll
        for (int rr = 0; rr < VR; ++rr) {
            Vec16<T> o;
#pragma unroll
            for (int kk = 0; kk < VK; ++kk) o.v[kk] = from_f<T>(v[kk][rr]);
            *reinterpret_cast<Vec16<T> *>(dst + xt_index<T, LDX>(rb * VR + rr, kb * VK)) = o;
        }
    }
}

// same read of the source, two scaled images (used where both directions weight one operand differently)
template <typename T, int KTOT, int RTOT, int LDX, bool FAST, typename S, class F1, class F2>
__device__ __forceinline__ void stage_transposed2(T *dst1, T *dst2, const S *src, int64_t ks, int kvalid, int rvalid,
                                                  F1 scale1, F2 scale2) {
    constexpr int VK = 16 / sizeof(T), VR = 16 / sizeof(S), RB = RTOT / VR, NB = (KTOT / VK) * RB;
    const bool vec = FAST || aligned16(src, ks);
    for (int blk = threadIdx.x; blk < NB; blk += blockDim.x) {
        const int rb = blk % RB, kb = blk / RB;
        float v[VK][VR], s1[VK], s2[VK];
#pragma unroll
        for (int kk = 0; kk < VK; ++kk) {
            const int k = kb * VK + kk;
            const S *row = src + (int64_t)(FAST ? min(k, kvalid - 1) : k) * ks + rb * VR;
            if (FAST || (vec && k < kvalid && rb * VR + VR <= rvalid)) {
                Vec16<S> raw = *reinterpret_cast<const Vec16<S> *>(row);
#pragma unroll
                for (int i = 0; i < VR; ++i) v[kk][i] = to_f(raw.v[i]);
            } else {
#pragma unroll
                for (int i = 0; i < VR; ++i) v[kk][i] = (k < kvalid && rb * VR + i < rvalid) ? to_f(row[i]) : 0.f;
            }
            s1[kk] = scale1(k);
            s2[kk] = scale2(k);
        }
#pragma unroll
        for (int rr = 0; rr < VR; ++rr) {
            Vec16<T> o1, o2;
#pragma unroll
            for (int kk = 0; kk < VK; ++kk) { o1.v[kk] = from_f<T>(v[kk][rr] * s1[kk]); o2.v[kk] = from_f<T>(v[kk][rr] * s2[kk]); }
            const int at = xt_index<T, LDX>(rb * VR + rr, kb * VK);
            *reinterpret_cast<Vec16<T> *>(dst1 + at) = o1;
            *reinterpret_cast<Vec16<T> *>(dst2 + at) = o2;
        }
    }
}


struct Ident {
    __device__ __forceinline__ float operator()(int, int, float v) const { return v; }
};

// ---- wavefront helpers --------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
    return v;
}
// (row rotations only: every lane has a source, and with bound_ctrl set the compiler folds the move into the
// instruction that uses it - v_add_f32_dpp instead of v_mov_b32_dpp + v_add_f32)
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
    static_assert(CTRL >= 0x121 && CTRL <= 0x12f, "row_ror only");
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// sum over the 16 lanes that share l/16 (one row group of an MFMA output tile); every lane gets the sum
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_mov<0x128>(v);  // row_ror:8
    v += dpp_mov<0x124>(v);  // row_ror:4
    v += dpp_mov<0x122>(v);  // row_ror:2
    v += dpp_mov<0x121>(v);  // row_ror:1
    return v;
}
// the largest of the 16 lanes' values, likewise
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_mov<0x128>(v));
    v = fmaxf(v, dpp_mov<0x124>(v));
    v = fmaxf(v, dpp_mov<0x122>(v));
    v = fmaxf(v, dpp_mov<0x121>(v));
    return v;
}
// inclusive prefix / suffix sums over the 64 lanes
__device__ __forceinline__ float wave_incl_prefix(float v, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        float o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}
__device__ __forceinline__ float wave_incl_suffix(float v, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        float o = __shfl_down(v, d, 64);
        if (lane + d < 64) v += o;
    }
    return v;
}

template <int CTRL> __device__ __forceinline__ float dpp_mov0(float v) {
    // lanes whose source lies outside their row of 16 receive 0
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// inclusive prefix (towards higher lanes) / suffix sums inside each row of 16 lanes
__device__ __forceinline__ float row16_incl_prefix(float v) {
    v += dpp_mov0<0x111>(v);  // row_shr:1
    v += dpp_mov0<0x112>(v);  // row_shr:2
    v += dpp_mov0<0x114>(v);  // row_shr:4
    v += dpp_mov0<0x118>(v);  // row_shr:8
    return v;
}
__device__ __forceinline__ float row16_incl_suffix(float v) {
    v += dpp_mov0<0x101>(v);  // row_shl:1
    v += dpp_mov0<0x102>(v);
    v += dpp_mov0<0x104>(v);
    v += dpp_mov0<0x108>(v);
    return v;
}

// reciprocal by the hardware approximation (1 ulp) instead of a full division sequence
__device__ __forceinline__ float sigmoid_f(float z) { return __builtin_amdgcn_rcpf(1.f + __expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z * sigmoid_f(z); }

// chunk bookkeeping shared by all kernels
struct ChunkIdx {
    int b, c, h, g, limit;
};

// Launch position -> (inner, outer) for a grid of nouter x ninner workgroups whose `ninner` workgroups of one outer index
// share data: workgroups are dealt round-robin to the 8 XCDs (each with its own L2) in launch order, so eight outer indices
// at a time, one per XCD, go through their inner indices; what is left when nouter is not a multiple of 8 shares the XCDs.
__device__ __forceinline__ void xcd_order(int lin, int ninner, int nouter, int &inner, int &outer) {
    const int full = nouter / 8, grp = lin / (8 * ninner);
    if (grp < full) {
        const int r = lin - grp * 8 * ninner;
        inner = r >> 3;
        outer = grp * 8 + (r & 7);
    } else {
        const int m = nouter - full * 8, r = lin - full * 8 * ninner;
        inner = r / m;
        outer = full * 8 + r % m;
    }
}

}  // namespace bm2
