// Device-side building blocks of the packed-state decode step for gfx950 (wave64).
//
// One wavefront owns one (sequence, value head) tile of the stored state: DV rows of DK codes, value-major.  A row is
// split into 16-column pieces, one per lane, so a lane's piece of an int8 row is one 128-bit load (int4: 64 bits) and
// the lanes of a wavefront read whole, consecutive rows.  Everything below is written for that decomposition.
//
// Arithmetic follows the reference's device kernels: fp32 throughout, explicit fma where the reference uses one,
// IEEE division / sqrt, round-half-to-even, payloads rounded against the fp16-rounded scale
// (/root/reference/src/statequant/kernels/_fold_triton.py:38-62).  The translation unit must be compiled with
// -ffp-contract=off so that no other multiply-add is contracted.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sq {

constexpr int WAVE = 64;

// Ordering point for LDS traffic between the lanes of ONE wavefront (the step kernels run one wavefront per tile): the
// LDS executes a wavefront's instructions in issue order, so a read issued after a write sees it; what is needed is
// that the compiler keeps that order.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
constexpr int CPL = 16;                       // state columns per lane
constexpr float FP16_TINY = 5.960464477539063e-08f;   // 2^-24: floor of a stored fp16 scale

enum DType : int { F32 = 0, BF16 = 1, F16 = 2 };

__host__ __device__ constexpr int pow2_ceil(int n) { int p = 1; while (p < n) p <<= 1; return p; }
__host__ __device__ constexpr int round_up(int n, int k) { return (n + k - 1) / k * k; }
__host__ __device__ constexpr int ilog2(int n) { int l = 0; while ((1 << l) < n) ++l; return l; }

// ---------------------------------------------------------------------------------------------------------------
// bit casts and narrow float formats
// ---------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return as_f32(uint32_t(h) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {      // round to nearest even, quiet NaNs (as torch)
    uint32_t u = as_u32(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return uint16_t(u >> 16);
}
__device__ __forceinline__ float f16_to_f32(uint16_t h) { return float(__builtin_bit_cast(_Float16, h)); }
__device__ __forceinline__ uint16_t f32_to_f16(float f) { return __builtin_bit_cast(uint16_t, _Float16(f)); }

// A scalar of a float tensor of run-time dtype (inputs come as fp32, bf16 or fp16), in two steps so that a kernel can
// issue all its loads first and convert later: a conversion right behind a load, inside the dtype branch, makes
// the compiler wait for memory in every branch and serializes the loads.
// `p` carries the wave-uniform part of the address (see `advance`), `i` the lane's 32-bit element index: the load
// then needs no 64-bit vector arithmetic.
__device__ __forceinline__ uint32_t load_raw(const void* p, int dt, uint32_t i) {
    if (dt == F32) return reinterpret_cast<const uint32_t*>(p)[i];
    return reinterpret_cast<const uint16_t*>(p)[i];
}
__device__ __forceinline__ const void* advance(const void* p, int dt, uint64_t elems) {
    return reinterpret_cast<const uint8_t*>(p) + (elems << (dt == F32 ? 2 : 1));
}
__device__ __forceinline__ void* advance(void* p, int dt, uint64_t elems) {
    return reinterpret_cast<uint8_t*>(p) + (elems << (dt == F32 ? 2 : 1));
}
// The same for a wave-uniform address (a per-head scalar).  The offset is laundered through a vector register so
// that the load stays a vector load: as a scalar load its result would have to be moved into a VGPR right away, and
// the wait for that move also waits for every vector load issued before it.
__device__ __forceinline__ uint32_t load_raw_uniform(const void* p, int dt, uint64_t i) {
    uint32_t z = 0;
    asm volatile("" : "+v"(z));
    return load_raw(advance(p, dt, i), dt, z);
}
__device__ __forceinline__ float raw_to_f(uint32_t r, int dt) {
    return dt == F32 ? as_f32(r) : dt == BF16 ? bf16_to_f32(uint16_t(r)) : f16_to_f32(uint16_t(r));
}
__device__ __forceinline__ void store_f(void* p, int dt, uint32_t i, float v) {
    if (dt == F32) reinterpret_cast<float*>(p)[i] = v;
    else reinterpret_cast<uint16_t*>(p)[i] = dt == BF16 ? f32_to_bf16(v) : f32_to_f16(v);
}

// ---------------------------------------------------------------------------------------------------------------
// rounding (reference: _fold_triton.py:52-62, _fused_triton.py:471-501)
// ---------------------------------------------------------------------------------------------------------------
// x / d with the divisor's reciprocal rc = RN(1 / d): q = RN(x rc), the exact remainder r = x - q d (one fma),
// q + r rc rounded once.  With a correctly rounded reciprocal this is the correctly rounded quotient (Markstein's
// division; the exception, a divisor whose significand is all ones, cannot occur: the divisors here are fp16 values
// or the code ranges 3, 7, 31, 127), i.e. the IEEE quotient at a third of its instructions -- and of its latency,
// which is what counts on a wavefront's serial path.  Checked in exact rational arithmetic over every fp16 divisor
// and the four constants in tests/test_gga_division_cpu.py.
__device__ __forceinline__ float div_rc(float x, float d, float rc) {
    const float q = x * rc;
    const float r = __builtin_fmaf(-q, d, x);
    return __builtin_fmaf(r, rc, q);
}
// RN(1 / d) for a divisor that is an fp16 value (2^-24 and up): the hardware estimate (1 ulp) and one Newton step
// with the exact residual.  The step leaves a relative error of 2^-46 before its single rounding, and the reciprocal
// of an 11-bit significand is never closer than 2^-12 ulp to a rounding boundary, so the result is the correctly
// rounded one.
__device__ __forceinline__ float rcp_f16(float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
}
// A scale as a divisor: the scale itself, or -- a scale that overflowed fp16 to infinity (values beyond 65504 qmax)
// -- the largest finite float, which sends every finite value to code 0 as a division by infinity does, without an
// infinity times zero on the way.
struct Divisor {
    float d, rc;
};
__device__ __forceinline__ Divisor scale_divisor(float scale) {
    Divisor v;
    v.d = fminf(scale, 3.0e38f);
    v.rc = rcp_f16(v.d);
    return v;
}
__device__ __forceinline__ float div_by(float x, const Divisor& v) { return div_rc(x, v.d, v.rc); }
// The fp16-valued divisor back from its correctly rounded reciprocal: 1 / rc is within 2^-22 of it, and rounding to
// fp16's grid (11 bits, subnormals included) removes that.  For paths that are rarely taken and would otherwise keep
// the divisor in a register beside its reciprocal.
__device__ __forceinline__ float divisor_of(float rc) {
    return fminf(float(_Float16(__builtin_amdgcn_rcpf(rc))), 3.0e38f);      // (an overflowed scale: as in scale_divisor)
}

// Quantizer scale: max(amax, 1e-8) / qmax -> fp16 (nearest even, subnormals kept) -> fp32, floored at 2^-24.  qmax is
// 7 or 127 at every call (a constant there, so 1 / qmax is folded).
__device__ __forceinline__ float fp16_scale(float amax, float qmax) {
    float s = div_rc(fmaxf(amax, 1e-8f), qmax, 1.0f / qmax);
    // the quotient is rounded to fp32 first and to fp16 second, as the reference's: without this the compiler folds
    // the division's last fma and the conversion into one instruction with a single rounding (v_fma_mixlo_f16)
    asm volatile("" : "+v"(s));
    s = float(_Float16(s));
    return fmaxf(s, FP16_TINY);
}

// Buffer entry: clamp(rint(x / scale), +-127) as a float; `scale` comes from `fp16_scale`.
__device__ __forceinline__ float round_buf(float x, float scale) {
    return fminf(fmaxf(rintf(div_by(x, scale_divisor(scale))), -127.0f), 127.0f);
}

// ---------------------------------------------------------------------------------------------------------------
// cross-lane movement.  DPP controls: quad_perm = 8-bit selector, 0x141 row_half_mirror, 0x140 row_mirror.
// ---------------------------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return as_f32(uint32_t(__builtin_amdgcn_update_dpp(0, int(as_u32(v)), CTRL, 0xF, 0xF, true)));
}
constexpr int DPP_XOR1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int DPP_HMIRROR = 0x141;    // lane i <-> 7 - i within each 8 lanes
constexpr int DPP_MIRROR = 0x140;     // lane i <-> 15 - i within each 16 lanes

// The value of the partner lane at butterfly level LVL (0: xor 1, 1: xor 2, 2: other half of 8, 3: other half of 16).
// Levels 2 and 3 pair lane i with its mirror image, which is a valid butterfly partner once the lower levels have
// made all lanes of the smaller block equal.
template <int LVL>
__device__ __forceinline__ float partner(float v) {
    if constexpr (LVL == 0) return dpp<DPP_XOR1>(v);
    else if constexpr (LVL == 1) return dpp<DPP_XOR2>(v);
    else if constexpr (LVL == 2) return dpp<DPP_HMIRROR>(v);
    else return dpp<DPP_MIRROR>(v);
}

// Sum / max over aligned blocks of N lanes (N a power of two <= 16); every lane of the block gets the result.
template <int N>
__device__ __forceinline__ float block_sum(float v) {
    if constexpr (N >= 2) v = v + partner<0>(v);
    if constexpr (N >= 4) v = v + partner<1>(v);
    if constexpr (N >= 8) v = v + partner<2>(v);
    if constexpr (N >= 16) v = v + partner<3>(v);
    return v;
}
template <int N>
__device__ __forceinline__ float block_max(float v) {
    if constexpr (N >= 2) v = fmaxf(v, partner<0>(v));
    if constexpr (N >= 4) v = fmaxf(v, partner<1>(v));
    if constexpr (N >= 8) v = fmaxf(v, partner<2>(v));
    if constexpr (N >= 16) v = fmaxf(v, partner<3>(v));
    return v;
}
__device__ __forceinline__ float lane_bcast(float v, int lane) {
    return as_f32(uint32_t(__builtin_amdgcn_readlane(int(as_u32(v)), lane)));
}
// Over the whole wavefront; the result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v) {
    v = block_sum<16>(v);
    return (lane_bcast(v, 0) + lane_bcast(v, 16)) + (lane_bcast(v, 32) + lane_bcast(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
    v = block_max<16>(v);
    return fmaxf(fmaxf(lane_bcast(v, 0), lane_bcast(v, 16)), fmaxf(lane_bcast(v, 32), lane_bcast(v, 48)));
}

// ---------------------------------------------------------------------------------------------------------------
// a lane's 16 codes of one row
// ---------------------------------------------------------------------------------------------------------------
template <int BITS> struct RawRow;
template <> struct RawRow<8> { uint4 v; };      // 16 int8
template <> struct RawRow<4> { uint2 v; };      // 16 nibbles: byte j = (c[2j] + 8) | (c[2j+1] + 8) << 4

// Native vector types for values that stay in registers across the load / use distance (the compiler keeps arrays of
// HIP's uint4 / uint2 structs in scratch memory when an asm statement separates their loads from their uses).
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));

// Loads and stores of data that one launch touches once (the state codes, their scales, the buffered keys and
// values): marked non-temporal they stream through the L2 without displacing the few lines the launch writes
// (outputs, buffer appends, counters).  Measured on the 128 x 128 int8 step: 2 to 3 us of 35 per launch.
template <class V>
__device__ __forceinline__ V stream_load(const V* p) { return __builtin_nontemporal_load(p); }
template <class V>
__device__ __forceinline__ void stream_store(V* p, V v) { __builtin_nontemporal_store(v, p); }

// A lane's piece of a state row from global memory, streamed.
template <int BITS>
__device__ __forceinline__ RawRow<BITS> stream_row(const uint8_t* p) {
    RawRow<BITS> r;
    if constexpr (BITS == 8) {
        const v4u x = stream_load(reinterpret_cast<const v4u*>(p));
        r.v = make_uint4(x.x, x.y, x.z, x.w);
    } else {
        const v2u x = stream_load(reinterpret_cast<const v2u*>(p));
        r.v = make_uint2(x.x, x.y);
    }
    return r;
}
template <int BITS>
__device__ __forceinline__ RawRow<BITS> load_row(const uint8_t* p) {
    RawRow<BITS> r;
    if constexpr (BITS == 8) r.v = *reinterpret_cast<const uint4*>(p);
    else r.v = *reinterpret_cast<const uint2*>(p);
    return r;
}
template <int BITS>
__device__ __forceinline__ RawRow<BITS> zero_row() {
    RawRow<BITS> r;
    if constexpr (BITS == 8) r.v = make_uint4(0, 0, 0, 0);
    else r.v = make_uint2(0x88888888u, 0x88888888u);      // nibble 8 = code 0
    return r;
}
__device__ __forceinline__ float s8_to_f(uint32_t w, int byte) { return float(int32_t(w << (24 - 8 * byte)) >> 24); }

// fp32 value of a lane's 16 codes, times `unit`.  int4: a stored nibble is code + 8; with bit 3 flipped and moved to
// the high half of a byte it reads, as a signed byte, 16 x code -- one byte-to-float conversion per code instead of
// extract, subtract, convert -- and DECODE_UNIT = 1/16 (exact) goes into whatever factor the caller applies next.
template <int BITS> constexpr float DECODE_UNIT = BITS == 4 ? 0.0625f : 1.0f;
template <int BITS>
__device__ __forceinline__ void decode_row_scaled(const RawRow<BITS>& r, float (&c)[CPL]) {
    if constexpr (BITS == 8) {
        const uint32_t w[4] = {r.v.x, r.v.y, r.v.z, r.v.w};
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
            for (int b = 0; b < 4; ++b) c[4 * d + b] = s8_to_f(w[d], b);
    } else {
        const uint32_t w[2] = {r.v.x ^ 0x88888888u, r.v.y ^ 0x88888888u};
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            const uint32_t lo = (w[d] << 4) & 0xF0F0F0F0u, hi = w[d] & 0xF0F0F0F0u;     // columns 0,2,4,6 / 1,3,5,7
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                c[8 * d + 2 * b] = s8_to_f(lo, b);
                c[8 * d + 2 * b + 1] = s8_to_f(hi, b);
            }
        }
    }
}
template <int BITS>
__device__ __forceinline__ void decode_row(const RawRow<BITS>& r, float (&c)[CPL]) {
    decode_row_scaled<BITS>(r, c);
    if constexpr (BITS == 4) {
#pragma unroll
        for (int t = 0; t < CPL; ++t) c[t] = c[t] * 0.0625f;
    }
}

// Integral floats in [-qmax, qmax] -> a lane's stored row.
template <int BITS>
__device__ __forceinline__ RawRow<BITS> encode_row(const float (&c)[CPL]) {
    RawRow<BITS> r;
    if constexpr (BITS == 8) {
        uint32_t w[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            w[d] = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) w[d] |= (uint32_t(int32_t(c[4 * d + b])) & 0xFFu) << (8 * b);
        }
        r.v = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
        uint32_t w[2];
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            w[d] = 0;
#pragma unroll
            for (int nb = 0; nb < 8; ++nb) w[d] |= (uint32_t(int32_t(c[8 * d + nb]) + 8) & 0xFu) << (4 * nb);
        }
        r.v = make_uint2(w[0], w[1]);
    }
    return r;
}
// Quantize a lane's 16 values of one row against scale 1/r: codes = clamp(rint(a r), +-qmax), packed as stored.
// a r + 1.5 2^23 (one fma: the exact product, rounded once, half to even, at integer granularity) leaves the code in
// the low mantissa bits in two's complement; int4 adds its +8 storage bias in the same constant.  The clamp acts on
// the biased float, the bytes / nibbles are gathered with byte permutes.
// CLAMP = false leaves the clamp out: for callers that know |a r| < qmax + 1/2 (a scale that is a NORMAL fp16
// number lies within 2^-11 of absmax / qmax, so the largest quotient is qmax (1 + 2^-11) at most).
// a r differs from the quotient a / d by the reciprocal's rounding, 2^-24 of it: where the quotient is within that
// of a half-integer the code can come out one step from rint(a / d).  For values in general position that is one
// code in 10^5; but a state that is a sum of a few products of low-precision numbers (the first fold after an empty
// state: buffered vectors are bf16 or int8 x fp16) has quotients that are EXACTLY half-integers, thousands of them,
// and those would go by the sign of the reciprocal's error instead of to even.  EXACT = true takes the IEEE quotient
// first (div_rc with the divisor d: two more fmas and an addition per value), bit for bit the reference's
// rint(div_rn(a, d)) (_fused_triton.py:472-486 there); the folds use it where the old state contributes nothing.
template <int BITS, bool CLAMP = true, bool EXACT = false>
__device__ __forceinline__ RawRow<BITS> quantize_row(const float (&a)[CPL], float r, float d = 0.0f) {
    constexpr float QMAX = float((1 << (BITS - 1)) - 1);
    constexpr float MAGIC = 12582912.0f + (BITS == 4 ? 8.0f : 0.0f);
    if constexpr (EXACT) {
        // the rarely taken exact path packs word by word, so that it needs fewer registers than the other one (it
        // must not raise the allocation of kernels that run at their limit)
        constexpr int PER = 32 / BITS;                       // codes per 32-bit word
        uint32_t w[CPL / PER];
#pragma unroll
        for (int i = 0; i < CPL / PER; ++i) {
            uint32_t acc = 0;
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                const float f = __builtin_amdgcn_fmed3f(div_rc(a[PER * i + e], d, r) + MAGIC, MAGIC - QMAX, MAGIC + QMAX);
                acc |= (as_u32(f) & (BITS == 8 ? 0xFFu : 0xFu)) << (BITS * e);
            }
            w[i] = acc;
            __builtin_amdgcn_sched_barrier(0);
        }
        RawRow<BITS> o;
        if constexpr (BITS == 8) o.v = make_uint4(w[0], w[1], w[2], w[3]);
        else o.v = make_uint2(w[0], w[1]);
        return o;
    }
    uint32_t u[CPL];
#pragma unroll
    for (int t = 0; t < CPL; ++t) {
        const float f = __builtin_fmaf(a[t], r, MAGIC);
        u[t] = as_u32(CLAMP ? __builtin_amdgcn_fmed3f(f, MAGIC - QMAX, MAGIC + QMAX) : f);
    }
    RawRow<BITS> o;
    if constexpr (BITS == 8) {
        uint32_t w[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t lo = __builtin_amdgcn_perm(u[4 * d + 1], u[4 * d], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm(u[4 * d + 3], u[4 * d + 2], 0x0c0c0400u);
            w[d] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
        o.v = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
        uint32_t w[2];
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            const uint32_t* e = u + 8 * d;                       // nibbles 0..7 of the word; each low byte is 1..15
            const uint32_t ev = __builtin_amdgcn_perm(__builtin_amdgcn_perm(e[6], e[4], 0x0c0c0400u),
                                                      __builtin_amdgcn_perm(e[2], e[0], 0x0c0c0400u), 0x05040100u);
            const uint32_t od = __builtin_amdgcn_perm(__builtin_amdgcn_perm(e[7], e[5], 0x0c0c0400u),
                                                      __builtin_amdgcn_perm(e[3], e[1], 0x0c0c0400u), 0x05040100u);
            w[d] = ev | (od << 4);
        }
        o.v = make_uint2(w[0], w[1]);
    }
    return o;
}
template <int BITS>
__device__ __forceinline__ void store_row(uint8_t* p, const RawRow<BITS>& r) {
    if constexpr (BITS == 8) *reinterpret_cast<uint4*>(p) = r.v;
    else *reinterpret_cast<uint2*>(p) = r.v;
}

}  // namespace sq
