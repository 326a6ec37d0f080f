// RESCALE and CLAMP as stand-alone bandwidth kernels.
//
// RESCALE reads 1/2/4/8 bytes and writes 1/2/4 bytes per element and does ~20 integer instructions per
// element, so it is bound by HBM.  Each lane handles VEC consecutive elements of one row with a single
// vector load and a single vector store; the per-channel constants come from the L1/L2-resident
// multiplier and shift arrays.
#include "tmi_kernels.h"

namespace tmi
{

template <typename T, int N>
struct alignas(sizeof(T) * N) Pack
{
    T v[N];
};

// PRECISE: the FP64 forms of INEXACT_ROUND (precise mode), which the other instantiation does not hold.
template <typename InT, typename OutT, int VEC, bool PRECISE>
__global__ __launch_bounds__(256) void rescale_vec_kernel(RescaleParams p, const InT* __restrict__ in,
                                                          OutT* __restrict__ out, int64_t n_vec, int32_t C,
                                                          uint32_t* flag_word)
{
    // C % VEC == 0, so a pack never straddles a row and its channels are c0 .. c0+VEC-1
    uint32_t flags       = 0;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride)
    {
        const Pack<InT, VEC> a = reinterpret_cast<const Pack<InT, VEC>*>(in)[i];
        const int c0           = (int)((i * VEC) % C);
        Pack<OutT, VEC> r;
#pragma unroll
        for (int j = 0; j < VEC; j++)
        {
            const int32_t m = load_multiplier(p, c0 + j);
            const int32_t s = load_shift(p, c0 + j);
            r.v[j]          = (OutT)rescale_value<PRECISE>(p, a.v[j], m, s, flags);
        }
        reinterpret_cast<Pack<OutT, VEC>*>(out)[i] = r;
    }
    raise_flags(flag_word, flags);
}

template <typename InT, typename OutT, bool PRECISE>
__global__ __launch_bounds__(256) void rescale_scalar_kernel(RescaleParams p, const InT* __restrict__ in,
                                                             OutT* __restrict__ out, int64_t n, int32_t C,
                                                             uint32_t* flag_word)
{
    uint32_t flags       = 0;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    {
        const int c     = (int)(i % C);
        const int32_t m = load_multiplier(p, c);
        const int32_t s = load_shift(p, c);
        out[i]          = (OutT)rescale_value<PRECISE>(p, in[i], m, s, flags);
    }
    raise_flags(flag_word, flags);
}

// The common RESCALE -- signed INT32 in (no input zero point), 32-bit multipliers, SINGLE or DOUBLE rounding,
// C a multiple of 4 -- with the per-channel constants in registers: a lane owns 4 consecutive channels and
// walks down the rows, so multiplier, shift and the 64-bit rounding terms (output zero point folded in) are
// derived once.  A workgroup visits `rpi` rows at a time (a unit); its units are blockIdx, blockIdx + grid, ...
// Four units are in flight per lane: the load of unit k + 4 is issued as soon as unit k has been converted, so
// the loads of a wave never drain while it computes.
//
// HW: every channel of the wave has a shift of at least 32 (33 with double rounding) that also lets the output
// zero point ride in the rounding term: the result is the high word of value * multiplier + R shifted by
// shift - 32, with R's sign-dependent part (double rounding) patched into the addend - no 64-bit shift and no
// range test, which cannot fire for such shifts.
typedef int rs_v4i __attribute__((ext_vector_type(4)));

struct RescaleLane
{
    int32_t mul[4], sh[4], zp_post[4], hw_hi[4];
    uint32_t lim[4], hw_lo[4];
    int64_t rnd_pos[4], rnd_neg[4];
    bool check;
};

template <typename OutT, bool HW, bool DR>
__device__ __forceinline__ void rescale_store_row(const RescaleParams& p, const RescaleLane& k, rs_v4i v, OutT* q,
                                                  uint32_t& flags)
{
    int32_t res[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
    {
        const int32_t x = v[c];
        int32_t o;
        if constexpr (HW)
            o = high_word_rescale<DR>(x, k.mul[c], k.hw_hi[c], k.hw_lo[c], k.sh[c]);
        else
        {
            if (k.check && (uint32_t)x + k.lim[c] > 2u * k.lim[c] - 1u)
                flags |= TMI_FLAG_SCALE_VALUE;
            const int64_t pr = (int64_t)x * (int64_t)k.mul[c] + (x >= 0 ? k.rnd_pos[c] : k.rnd_neg[c]);
            o                = (int32_t)(pr >> k.sh[c]) + k.zp_post[c];
        }
        o      = o < p.lo ? p.lo : o;
        res[c] = o > p.hi ? p.hi : o;
    }
    if constexpr (sizeof(OutT) == 1)
        *reinterpret_cast<int*>(q) = (res[0] & 0xff) | ((res[1] & 0xff) << 8) | ((res[2] & 0xff) << 16) | ((res[3] & 0xff) << 24);
    else if constexpr (sizeof(OutT) == 2)
    {
        reinterpret_cast<int*>(q)[0] = (res[0] & 0xffff) | ((res[1] & 0xffff) << 16);
        reinterpret_cast<int*>(q)[1] = (res[2] & 0xffff) | ((res[3] & 0xffff) << 16);
    }
    else
        *reinterpret_cast<rs_v4i*>(q) = rs_v4i{ res[0], res[1], res[2], res[3] };
}

template <typename OutT, bool HW, bool DR>
__device__ __forceinline__ void rescale_walk(const RescaleParams& p, const RescaleLane& k, const int32_t* __restrict__ in,
                                             OutT* __restrict__ out, int64_t rows, int32_t C, int32_t rpi, int slot,
                                             int c0, bool lane_on, uint32_t& flags)
{
    constexpr int U    = 4;
    const int64_t step = (int64_t)gridDim.x * rpi;    // rows between two units of a workgroup
    int64_t r          = (int64_t)blockIdx.x * rpi + slot;
    rs_v4i v[U];
#pragma unroll
    for (int u = 0; u < U; u++)
    {
        const int64_t ru = r + u * step;
        v[u]             = *reinterpret_cast<const rs_v4i*>(in + ((lane_on && ru < rows) ? ru * C + c0 : 0));
    }
    // every lane of the workgroup runs the same number of rounds: the loads of a round are issued by all
    for (int64_t base = (int64_t)blockIdx.x * rpi; base < rows; base += U * step, r += U * step)
    {
#pragma unroll
        for (int u = 0; u < U; u++)
        {
            const int64_t ru  = r + u * step;
            const rs_v4i cur  = v[u];
            const int64_t nxt = ru + U * step;
            v[u]              = *reinterpret_cast<const rs_v4i*>(in + ((lane_on && nxt < rows) ? nxt * C + c0 : 0));
            if (lane_on && ru < rows)
                rescale_store_row<OutT, HW, DR>(p, k, cur, out + ru * C + c0, flags);
        }
    }
}

template <typename OutT>
__global__ __launch_bounds__(256) void rescale_fast_kernel(RescaleParams p, const int32_t* __restrict__ in,
                                                           OutT* __restrict__ out, int64_t rows, int32_t C,
                                                           int32_t cgs, int32_t rpi, FastDiv div_cgs,
                                                           uint32_t* flag_word)
{
    const int tid      = threadIdx.x;
    const int slot     = fdiv(tid, div_cgs);    // row slot of this lane inside a unit
    const bool lane_on = slot < rpi;
    const int c0       = lane_on ? (tid - slot * cgs) * 4 : 0;
    uint32_t flags     = 0;
    RescaleLane k;
    k.check    = false;
    bool hw_ok = true;
    const int max_fold = zp_fold_max_shift(p.out_zp);
#pragma unroll
    for (int c = 0; c < 4; c++)
    {
        const int i = p.per_channel ? c0 + c : 0;
        const ChannelScale cs =
            make_channel_scale(reinterpret_cast<const int32_t*>(p.multiplier)[i], (int32_t)p.shift[i], p.double_round, flags);
        const bool fold       = cs.s <= max_fold;    // else output_zp is added after the shift
        const int64_t zp_term = fold ? ((int64_t)p.out_zp << cs.s) : 0;
        k.zp_post[c]          = fold ? 0 : p.out_zp;
        k.mul[c] = cs.m, k.lim[c] = cs.lim;
        k.rnd_pos[c] = cs.rnd_pos + zp_term, k.rnd_neg[c] = cs.rnd_neg + zp_term;
        k.check |= cs.lim != 0x80000000u;
        hw_ok &= fold && cs.s >= (p.double_round ? 33 : 32) && flags == 0;
        const HighWordScale h = make_high_word_scale(cs, p.out_zp);
        k.hw_hi[c] = h.hi, k.hw_lo[c] = h.lo;
        k.sh[c] = cs.s;
    }
    if (!lane_on)
        flags = 0, hw_ok = true;
    if (__all(hw_ok))
    {
#pragma unroll
        for (int c = 0; c < 4; c++)
            k.sh[c] -= 32;
        if (p.double_round)
            rescale_walk<OutT, true, true>(p, k, in, out, rows, C, rpi, slot, c0, lane_on, flags);
        else
            rescale_walk<OutT, true, false>(p, k, in, out, rows, C, rpi, slot, c0, lane_on, flags);
    }
    else
        rescale_walk<OutT, false, false>(p, k, in, out, rows, C, rpi, slot, c0, lane_on, flags);
    raise_flags(flag_word, flags);
}

template <typename OutT>
static const char* launch_rescale_fast(hipStream_t st, const RescaleParams& p, const void* in, void* out, int64_t n,
                                       int32_t C, uint32_t* flag_word)
{
    const int32_t cgs   = C / 4;
    const int32_t rpi   = 256 / cgs;
    const int64_t rows  = n / C;
    const int64_t units = (rows + rpi - 1) / rpi;
    // Two workgroups per CU, each with four 16-byte loads in flight per lane, stream faster than more workgroups
    // do (measured on [64,56,56,64]: 12.0 us with 2 per CU, 13.4 with 4, 14.8 with 8, 16.2 with 16; the arithmetic
    // is not what limits it: without it the same walk takes 11.5 us); and as many units for one workgroup as for
    // any other where that is possible
    const int64_t visits = (units + 256 * 2 - 1) / (256 * 2);
    int64_t blocks       = (units + visits - 1) / visits;
    if (blocks < 1)
        blocks = 1;
    hipLaunchKernelGGL((rescale_fast_kernel<OutT>), dim3((int)blocks), dim3(256), 0, st, p, (const int32_t*)in,
                       (OutT*)out, rows, C, cgs, rpi, make_fastdiv(cgs), flag_word);
    return "rescale_fast";
}

static int grid_for(int64_t work_items)
{
    // 256 CUs x 8 blocks of 256 lanes keep every SIMD busy; beyond that the loop strides.
    int64_t blocks = (work_items + 255) / 256;
    if (blocks < 1)
        blocks = 1;
    if (blocks > 256 * 8)
        blocks = 256 * 8;
    return (int)blocks;
}

template <typename InT, typename OutT>
static const char* launch_rescale_t(hipStream_t st, const RescaleParams& p, const void* in, void* out, int64_t n,
                                    int32_t C, uint32_t* flag_word)
{
    constexpr int VEC = 16 / (sizeof(InT) > sizeof(OutT) ? sizeof(InT) : sizeof(OutT)) >= 4
                            ? 16 / (sizeof(InT) > sizeof(OutT) ? sizeof(InT) : sizeof(OutT))
                            : 4;
    const bool aligned = ((uintptr_t)in % (sizeof(InT) * VEC) == 0) && ((uintptr_t)out % (sizeof(OutT) * VEC) == 0);
    if (n == 0)
        return "rescale_empty";
    const bool precise = p.inexact_round >= 2;
    if (aligned && C % VEC == 0)
    {
        const int64_t n_vec = n / VEC;
        if (precise)
            hipLaunchKernelGGL((rescale_vec_kernel<InT, OutT, VEC, true>), dim3(grid_for(n_vec)), dim3(256), 0, st, p,
                               (const InT*)in, (OutT*)out, n_vec, C, flag_word);
        else
            hipLaunchKernelGGL((rescale_vec_kernel<InT, OutT, VEC, false>), dim3(grid_for(n_vec)), dim3(256), 0, st, p,
                               (const InT*)in, (OutT*)out, n_vec, C, flag_word);
        return precise ? "rescale_vec_precise" : "rescale_vec";
    }
    if (precise)
        hipLaunchKernelGGL((rescale_scalar_kernel<InT, OutT, true>), dim3(grid_for(n)), dim3(256), 0, st, p,
                           (const InT*)in, (OutT*)out, n, C, flag_word);
    else
        hipLaunchKernelGGL((rescale_scalar_kernel<InT, OutT, false>), dim3(grid_for(n)), dim3(256), 0, st, p,
                           (const InT*)in, (OutT*)out, n, C, flag_word);
    if (precise)
        return "rescale_scalar_precise";
    return "rescale_scalar";
}

const char* launch_rescale(hipStream_t st, const RescaleParams& p, int32_t in_dtype, int32_t out_dtype,
                           const void* in, void* out, int64_t n, int32_t C, uint32_t* flag_word)
{
    if (p.fast && !p.has_clamp && in_dtype == TMI_INT32 && n > 0 && C >= 4 && (C & 3) == 0 && C <= 1024 &&
        (((uintptr_t)in | (uintptr_t)out) & 15) == 0 && (!p.per_channel || ((uintptr_t)p.multiplier & 3) == 0))
    {
        if (out_dtype == TMI_INT8)
            return launch_rescale_fast<int8_t>(st, p, in, out, n, C, flag_word);
        if (out_dtype == TMI_INT16)
            return launch_rescale_fast<int16_t>(st, p, in, out, n, C, flag_word);
        if (out_dtype == TMI_INT32)
            return launch_rescale_fast<int32_t>(st, p, in, out, n, C, flag_word);
    }
#define TMI_RESCALE_CASE(ID, IT, OD, OT)                                                                            \
    if (in_dtype == ID && out_dtype == OD)                                                                          \
        return launch_rescale_t<IT, OT>(st, p, in, out, n, C, flag_word);
    TMI_RESCALE_CASE(TMI_INT8, int8_t, TMI_INT8, int8_t)
    TMI_RESCALE_CASE(TMI_INT8, int8_t, TMI_INT16, int16_t)
    TMI_RESCALE_CASE(TMI_INT8, int8_t, TMI_INT32, int32_t)
    TMI_RESCALE_CASE(TMI_INT16, int16_t, TMI_INT8, int8_t)
    TMI_RESCALE_CASE(TMI_INT16, int16_t, TMI_INT16, int16_t)
    TMI_RESCALE_CASE(TMI_INT16, int16_t, TMI_INT32, int32_t)
    TMI_RESCALE_CASE(TMI_INT32, int32_t, TMI_INT8, int8_t)
    TMI_RESCALE_CASE(TMI_INT32, int32_t, TMI_INT16, int16_t)
    TMI_RESCALE_CASE(TMI_INT32, int32_t, TMI_INT32, int32_t)
    TMI_RESCALE_CASE(TMI_INT48, int64_t, TMI_INT8, int8_t)
    TMI_RESCALE_CASE(TMI_INT48, int64_t, TMI_INT16, int16_t)
    TMI_RESCALE_CASE(TMI_INT48, int64_t, TMI_INT32, int32_t)
#undef TMI_RESCALE_CASE
    return nullptr;
}

// ------------------------------------------------------------------------------------------------
// CLAMP on INT8 / INT16: min(max(x, lo), hi), 16 bytes per lane.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void clamp_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t n,
                                                    int32_t lo, int32_t hi, int vectorised)
{
    constexpr int VEC    = 16 / sizeof(T);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t n_vec  = vectorised ? n / VEC : 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride)
    {
        Pack<T, VEC> a = reinterpret_cast<const Pack<T, VEC>*>(in)[i];
#pragma unroll
        for (int j = 0; j < VEC; j++)
        {
            int32_t v = a.v[j];
            v         = v >= lo ? v : lo;
            v         = v < hi ? v : hi;
            a.v[j]    = (T)v;
        }
        reinterpret_cast<Pack<T, VEC>*>(out)[i] = a;
    }
    for (int64_t i = n_vec * VEC + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    {
        int32_t v = in[i];
        v         = v >= lo ? v : lo;
        v         = v < hi ? v : hi;
        out[i]    = (T)v;
    }
}

const char* launch_clamp(hipStream_t st, int32_t dtype, const void* in, void* out, int64_t n, int32_t lo,
                         int32_t hi)
{
    if (n == 0)
        return "clamp_empty";
    const int vec = ((uintptr_t)in % 16 == 0) && ((uintptr_t)out % 16 == 0);
    if (dtype == TMI_INT8)
        hipLaunchKernelGGL(clamp_kernel<int8_t>, dim3(grid_for((n + 15) / 16)), dim3(256), 0, st, (const int8_t*)in,
                           (int8_t*)out, n, lo, hi, vec);
    else if (dtype == TMI_INT16)
        hipLaunchKernelGGL(clamp_kernel<int16_t>, dim3(grid_for((n + 7) / 8)), dim3(256), 0, st,
                           (const int16_t*)in, (int16_t*)out, n, lo, hi, vec);
    else
        return nullptr;
    return "clamp_vec";
}

// ------------------------------------------------------------------------------------------------
// CLAMP on FP16 / BF16 / FP32 (activation_funcs.cpp:97-106): applyMax(x, min) then applyMin(., max) of
// arith_util.h:341-413 with the attribute's NaN mode (1 = PROPAGATE: a NaN stays a NaN; 2 = IGNORE: the NaN operand is
// dropped, so a NaN input ends at min), evaluated in float and rounded back to the stored type (fpTrunc).
// ------------------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float clampf_load(const T* p, int64_t i);
template <>
__device__ __forceinline__ float clampf_load<float>(const float* p, int64_t i)
{
    return p[i];
}
template <>
__device__ __forceinline__ float clampf_load<_Float16>(const _Float16* p, int64_t i)
{
    return (float)p[i];
}
template <>
__device__ __forceinline__ float clampf_load<bf16_t>(const bf16_t* p, int64_t i)
{
    return bf16_to_float(p[i]);
}
__device__ __forceinline__ void clampf_store(float* p, int64_t i, float v)
{
    p[i] = v;
}
__device__ __forceinline__ void clampf_store(_Float16* p, int64_t i, float v)
{
    p[i] = (_Float16)v;
}
__device__ __forceinline__ void clampf_store(bf16_t* p, int64_t i, float v)
{
    p[i] = float_to_bf16(v);
}

template <typename T>
__global__ __launch_bounds__(256) void clamp_fp_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t n, float lo,
                                                       float hi, int nan_mode)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    {
        float v = clampf_load<T>(in, i);
        if (v != v)
            v = nan_mode == 1 ? v : lo;
        else
        {
            v = v >= lo ? v : lo;
            v = v < hi ? v : hi;
        }
        clampf_store(out, i, v);
    }
}

const char* launch_clamp_fp(hipStream_t st, int32_t dtype, const void* in, void* out, int64_t n, float lo, float hi,
                            int32_t nan_mode)
{
    if (n == 0)
        return "clamp_empty";
    const dim3 grid(grid_for(n)), block(256);
    if (dtype == TMI_FP32)
        hipLaunchKernelGGL(clamp_fp_kernel<float>, grid, block, 0, st, (const float*)in, (float*)out, n, lo, hi, nan_mode);
    else if (dtype == TMI_FP16)
        hipLaunchKernelGGL(clamp_fp_kernel<_Float16>, grid, block, 0, st, (const _Float16*)in, (_Float16*)out, n, lo, hi,
                           nan_mode);
    else if (dtype == TMI_BF16)
        hipLaunchKernelGGL(clamp_fp_kernel<bf16_t>, grid, block, 0, st, (const bf16_t*)in, (bf16_t*)out, n, lo, hi, nan_mode);
    else
        return nullptr;
    return "clamp_fp";
}

// ------------------------------------------------------------------------------------------------
// A kernel that does nothing, for measuring what one launch of a given grid, block and LDS size costs.
// ------------------------------------------------------------------------------------------------
__global__ void empty_kernel(int32_t touch)
{
    extern __shared__ unsigned char empty_lds[];
    if (touch)    // never set: keeps the dynamic LDS allocation part of the kernel
        empty_lds[threadIdx.x] = 0;
}

const char* launch_empty(hipStream_t st, int32_t grid, int32_t block, int32_t lds_bytes)
{
    if (grid < 1 || block < 1 || block > 1024 || lds_bytes < 0 || lds_bytes > 160 * 1024)
        return nullptr;
    if (lds_bytes > 64 * 1024 &&
        hipFuncSetAttribute((const void*)empty_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
        return nullptr;
    hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), lds_bytes, st, 0);
    return "empty_kernel";
}

// ------------------------------------------------------------------------------------------------
// Streaming probes: what the memory system sustains for a plain copy, a read-only and a write-only pass over
// `vecs` 16-byte vectors.  Each workgroup walks the buffer with a grid stride, four vectors per lane and step.
// MODE 0 = copy, 1 = read only (the lanes fold what they read and store it only if it has a value the fold
// cannot take, so the loads stay), 2 = write only.
// ------------------------------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int MODE>
__global__ __launch_bounds__(256) void stream_probe_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                           int64_t vecs, uint32_t fill)
{
    const int64_t stride = (int64_t)gridDim.x * 256 * 4;
    uint32_t fold        = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 * 4 + threadIdx.x; i < vecs; i += stride)
    {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (MODE != 2 && i + u * 256 < vecs)
                v[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < 4; u++)
        {
            if (i + u * 256 >= vecs)
                continue;
            if (MODE == 1)
                fold |= (v[u].x & v[u].y & v[u].z & v[u].w) >> 31 | (v[u].x ^ v[u].y ^ v[u].z ^ v[u].w) << 1;
            else
                __builtin_nontemporal_store(MODE == 0 ? v[u] : u32x4{ fill, fill, fill, fill }, dst + i + u * 256);
        }
    }
    if (MODE == 1 && fold == fill)    // the caller passes a value the fold of its data never takes
        dst[0] = u32x4{ fold, fold, fold, fold };
}

// MODE 3 of the probe: the same read-only pass with loads that go straight into LDS (global_load_lds_dwordx4), which
// is how the convolution kernels fetch their patches
__global__ __launch_bounds__(256) void stream_probe_lds_kernel(const u32x4* __restrict__ src, int64_t vecs)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char probe_lds[];
    const int wave       = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lbase = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)probe_lds) + wave * 8192;
    const int64_t stride = (int64_t)gridDim.x * 256 * 4;
    int slot             = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 * 4 + threadIdx.x; i + 3 * 256 < vecs; i += stride)
    {
#pragma unroll
        for (int u = 0; u < 4; u++)
        {
            const u32x4* p = src + i + u * 256;
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(p), "s"(__builtin_amdgcn_readfirstlane(lbase + slot * 1024)) : "memory");
            slot = (slot + 1) & 7;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

const char* launch_stream_probe(hipStream_t st, int32_t mode, const void* src, void* dst, int64_t bytes)
{
    if (bytes < 16 || (bytes & 15) || (((uintptr_t)src | (uintptr_t)dst) & 15) || !dst || (mode != 2 && !src) || mode < 0 || mode > 3)
        return nullptr;
    const int64_t vecs = bytes / 16;
    const int64_t wgs  = (vecs + 1023) / 1024;
    const int grid     = (int)(wgs < 256 * 16 ? wgs : 256 * 16);
    if (mode == 0)
        hipLaunchKernelGGL(stream_probe_kernel<0>, dim3(grid), dim3(256), 0, st, (const u32x4*)src, (u32x4*)dst, vecs, 0u);
    else if (mode == 1)
        hipLaunchKernelGGL(stream_probe_kernel<1>, dim3(grid), dim3(256), 0, st, (const u32x4*)src, (u32x4*)dst, vecs, 0xFFFFFFFFu);
    else if (mode == 3)
        hipLaunchKernelGGL(stream_probe_lds_kernel, dim3(grid), dim3(256), 32768, st, (const u32x4*)src, vecs);
    else if (mode == 2)
        hipLaunchKernelGGL(stream_probe_kernel<2>, dim3(grid), dim3(256), 0, st, (const u32x4*)src, (u32x4*)dst, vecs, 0x01010101u);
    else
        return nullptr;
    return mode == 0 ? "stream_copy" : (mode == 1 ? "stream_read" : (mode == 2 ? "stream_write" : "stream_read_lds"));
}

// ------------------------------------------------------------------------------------------------
// Batched transpose [N, R, C] -> [N, C, R] through a padded 64x64 LDS tile: rows are read and written as
// contiguous runs along the fastest dimension of their side.
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(int32_t R, int32_t C, const T* __restrict__ in,
                                                        T* __restrict__ out)
{
    __shared__ T tile[64][64 + 4 / sizeof(T)];
    const size_t base = (size_t)blockIdx.z * R * C;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4)
        if (r0 + i < R && c0 + tx < C)
            tile[i][tx] = in[base + (size_t)(r0 + i) * C + c0 + tx];
    __syncthreads();
    for (int i = ty; i < 64; i += 4)
        if (c0 + i < C && r0 + tx < R)
            out[base + (size_t)(c0 + i) * R + r0 + tx] = tile[tx][i];
}

// The same for shapes made of whole, aligned pieces (C*EB a multiple of 4 bytes, R*EB a multiple of 16): dwords in,
// small blocks transposed in registers with byte permutes, 16-byte rows out.  A 64x64-element tile per workgroup.
typedef int tr_v4i __attribute__((ext_vector_type(4)));

template <int EB>
__global__ __launch_bounds__(256) void transpose_vec_kernel(int32_t R, int32_t C, const uint8_t* __restrict__ in,
                                                            uint8_t* __restrict__ out)
{
    constexpr int kRow = 64 * EB + 16;    // LDS row: 64 elements along R, padded
    __shared__ __attribute__((aligned(16))) uint8_t tile[64 * kRow];    // [c][r]
    const size_t base = (size_t)blockIdx.z * R * C * EB;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int tid = threadIdx.x;
    if constexpr (EB == 1)
    {
        // a thread takes a 4x4 block: four dwords (one per row), transposed to four dwords (one per column)
        const int tx = tid & 15, ty = tid >> 4;
        int d[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
        {
            const bool ok = r0 + 4 * ty + j < R && c0 + 4 * tx < C;
            d[j] = *reinterpret_cast<const int*>(in + base + (ok ? (size_t)(r0 + 4 * ty + j) * C + c0 + 4 * tx : 0));
        }
        const int t01_lo = __builtin_amdgcn_perm(d[1], d[0], 0x05010400);
        const int t01_hi = __builtin_amdgcn_perm(d[1], d[0], 0x07030602);
        const int t23_lo = __builtin_amdgcn_perm(d[3], d[2], 0x05010400);
        const int t23_hi = __builtin_amdgcn_perm(d[3], d[2], 0x07030602);
        int e[4];
        e[0] = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x05040100);
        e[1] = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x07060302);
        e[2] = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x05040100);
        e[3] = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x07060302);
#pragma unroll
        for (int j = 0; j < 4; j++)
            *reinterpret_cast<int*>(tile + (4 * tx + j) * kRow + 4 * ty) = e[j];
    }
    else
    {
        // 2-byte elements: 2x2 blocks, four per thread
#pragma unroll
        for (int k = 0; k < 4; k++)
        {
            const int b  = tid + 256 * k;    // block index: 32 x 32 blocks
            const int bx = b & 31, by = b >> 5;
            int d[2];
#pragma unroll
            for (int j = 0; j < 2; j++)
            {
                const bool ok = r0 + 2 * by + j < R && c0 + 2 * bx < C;
                d[j] = *reinterpret_cast<const int*>(
                    in + base + (ok ? ((size_t)(r0 + 2 * by + j) * C + c0 + 2 * bx) * 2 : 0));
            }
            const int lo = __builtin_amdgcn_perm(d[1], d[0], 0x05040100);    // column 2bx: rows 2by, 2by+1
            const int hi = __builtin_amdgcn_perm(d[1], d[0], 0x07060302);
            *reinterpret_cast<int*>(tile + (2 * bx) * kRow + 4 * by)     = lo;
            *reinterpret_cast<int*>(tile + (2 * bx + 1) * kRow + 4 * by) = hi;
        }
    }
    __syncthreads();
    // 16-byte pieces of the transposed rows: 4 * EB pieces per row
    constexpr int kPieces = 4 * EB;
#pragma unroll
    for (int k = 0; k < EB; k++)
    {
        const int idx  = tid + 256 * k;
        const int c    = idx / kPieces;
        const int part = idx % kPieces;
        const int r    = r0 + part * (16 / EB);
        if (c0 + c < C && r < R)
            *reinterpret_cast<tr_v4i*>(out + base + ((size_t)(c0 + c) * R + r) * EB) =
                *reinterpret_cast<const tr_v4i*>(tile + c * kRow + part * 16);
    }
}

const char* launch_transpose(hipStream_t st, int32_t elem_bytes, int32_t N, int32_t R, int32_t C, const void* in,
                             void* out)
{
    if ((int64_t)N * R * C == 0)
        return "transpose_empty";
    const dim3 grid((C + 63) / 64, (R + 63) / 64, N);
    const bool pieces = (elem_bytes == 1 || elem_bytes == 2) && ((int64_t)C * elem_bytes) % 4 == 0 &&
                        ((int64_t)R * elem_bytes) % 16 == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0;
    if (pieces && elem_bytes == 1)
        hipLaunchKernelGGL(transpose_vec_kernel<1>, grid, dim3(256), 0, st, R, C, (const uint8_t*)in, (uint8_t*)out);
    else if (pieces)
        hipLaunchKernelGGL(transpose_vec_kernel<2>, grid, dim3(256), 0, st, R, C, (const uint8_t*)in, (uint8_t*)out);
    else if (elem_bytes == 1)
        hipLaunchKernelGGL(transpose_kernel<uint8_t>, grid, dim3(256), 0, st, R, C, (const uint8_t*)in, (uint8_t*)out);
    else if (elem_bytes == 2)
        hipLaunchKernelGGL(transpose_kernel<uint16_t>, grid, dim3(256), 0, st, R, C, (const uint16_t*)in,
                           (uint16_t*)out);
    else
        return nullptr;
    return "transpose";
}

}    // namespace tmi
