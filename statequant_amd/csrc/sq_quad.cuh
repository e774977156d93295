// The state tile of one (sequence, value head) shared by the wavefronts of one workgroup: every wavefront owns NB of
// the tile's 32-row blocks.  Shared by the Gated DeltaNet and Mamba2 workgroup-per-key-head step kernels (int4 / int8
// codes with key-axis scale groups and a power-of-two row size).
//
// What this buys over one wavefront per tile (sq_tile.cuh, kept for the other formats):
//   * a tile's life is a quarter as long, so the launch's ramp-up and tail shrink and the dispatcher balances the
//     compute units with a finer grain;
//   * a row block stays in LDS from the state pass to the fold, so a folding tile reads its codes from memory once;
//   * the front end (normalisation, digit planes, gates, buffer coefficients) is split across the wavefronts instead
//     of running back to back in one.
//
// Row dot products run on the matrix core as in sq_tile.cuh (codes against three signed 8-bit digit planes of the
// fixed-point read-out vectors, exact int32 sums), with the operands' roles swapped: the digit planes are the first
// operand (result row 8 g + 4 v + d = scale group g, vector v, digit d) and the codes the second (result column =
// state row).  v_mfma_i32_32x32x32_i8 leaves result rows 8 a + 4 kb + b of column n in lane (n, kb), element
// 4 a + b -- so lane (state row n, vector kb) ends up with exactly the three digits of all of its row's groups, and
// the sums never travel through LDS.
//
// LDS image of a row block: the rows as stored, 16-byte chunks XOR-swizzled inside a row so that both the row-shaped
// writes (lanes along a row) and the operand-shaped reads (lanes down a column of chunks) are conflict free without
// padding.
#pragma once
#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

// LDS-only release / acquire around a workgroup barrier: the state codes still in flight from global memory (plain
// register loads) are not waited for.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a compile-time constant in
// the body (a template argument there).
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// The start of a launch.  Every compute unit takes as many workgroups as its LDS admits, all at once, so all of them
// ask for their row blocks together, get them together, and compute together while memory idles until their
// successors have started: the workgroups the launch starts with (blockIdx below the resident number) therefore hold
// their row-block requests back by a ramp of blockIdx x `ramp` / 256 sleeps of 64 clocks, which spreads the first
// round's requests over about the time memory needs to serve them.  Measured on one machine, int8 rows (four
// workgroups per compute unit): 32.65 -> 32.08 us per launch with 32 (a stepped ramp of the same slope alike), 24:
// 32.28, 40 and more: slower than none; the Mamba2 step 31.35 -> 31.15 (30.96 with 24, the slope its launcher
// passes), sequences out of step 35.9 -> 35.5, 512 slots 62.6 -> 61.9, 128 slots 19.1 -> 18.7.  With six smaller
// workgroups per compute unit (int4) no ramp helped, and a launch of less than two rounds has nothing behind the
// first to gain from (64 slots: 11.38 -> 11.45), so those get 0.
constexpr unsigned COMPUTE_UNITS = 256;                    // MI355X
template <class Q, int WPE>
inline uint32_t quad_start_ramp(uint32_t grid, uint32_t slope) {
    constexpr uint32_t per_cu = WPE * 4 / Q::NW;           // resident workgroups per compute unit
    return (per_cu <= 4 && grid >= 2 * COMPUTE_UNITS * per_cu) ? slope : 0u;
}
template <class Q, int WPE>
__device__ __forceinline__ void quad_start_wait(uint32_t ramp) {
    if (ramp != 0 && blockIdx.x < COMPUTE_UNITS * (WPE * 4 / Q::NW))
        for (uint32_t i = (blockIdx.x * ramp) >> 8; i > 0; --i) __builtin_amdgcn_s_sleep(1);
}

// Diagnostic: quad_lds_pad() (declared with the parameters, set through sq_debug_select) is that many bytes of unused
// dynamic LDS added to every launch of the workgroup kernels, so that a compute unit holds fewer workgroups (static +
// dynamic LDS must stay within 64 KB) -- for measuring how the step time depends on the number of resident workgroups.

template <class T, int NB_, int GH_ = 1>
struct Quad {
    static_assert(!T::FLT && !T::AXV && !T::RAGV, "int4 / int8 codes with key-axis groups, whole row blocks");
    static constexpr int NB = NB_;                         // row blocks per wavefront
    static constexpr int GH = GH_;                         // value heads of one key head per workgroup
    static_assert(T::NRB % NB == 0 && (NB == 1 || NB == 2), "one or two row blocks per wavefront");
    static constexpr int NWH = T::NRB / NB;                // wavefronts per head
    static constexpr int NW = GH * NWH;                    // wavefronts per workgroup
    static constexpr int THREADS = NW * WAVE;
    static_assert(THREADS <= 1024, "workgroup size");
    static constexpr int RW = NB * T::MR;                  // rows per wavefront
    static constexpr int RB = T::ROW_BYTES;
    static_assert((RB & (RB - 1)) == 0 && RB >= 32 && RB <= 256, "row size: a power of two in 32..256 bytes");
    static_assert(T::BITS == 8 || T::DK % 64 == 0, "int4: d_k a multiple of 64");
    static constexpr int CPR = RB / 16;                    // 16-byte chunks per row
    static constexpr int BLK = T::MR * RB;                 // bytes of a row block
    static constexpr int HEAD = T::DV * RB;                // bytes of a head's codes
    static constexpr int NLD = BLK / 1024;                 // wavefront loads per row block
    static constexpr int SWM = CPR < 8 ? CPR : 8;          // swizzle: chunk c of row r sits at chunk c ^ ((r / SWD) % SWM)
    static constexpr int SWD = 8 / SWM;
    static_assert(T::NG <= 4, "at most four scale groups per row (result rows 8 g + 4 v + d)");
    // a d_k vector in a wavefront: lane l holds the NE consecutive elements NE l ..
    static constexpr int NE = T::DK / WAVE;
    static_assert(NE * WAVE == T::DK && NE >= 1 && NE <= 4, "d_k: 64, 128 or 256");
    // buffer passes: keys 4 columns per lane (slots dealt over the workgroup's wavefronts), values 4 rows per lane
    static constexpr int LPS = T::DK / 4;                  // lanes per buffered key
    static constexpr int SPP = WAVE / LPS;                 // keys per wavefront and pass
    static constexpr int KT = (T::MMAX + NW * SPP - 1) / (NW * SPP);
    static constexpr int LU = RW / 4;                      // lanes per buffered value piece of this wavefront's rows
    static constexpr int SU = WAVE / LU;
    static constexpr int UT = (T::MMAX + SU - 1) / SU;
};

// Byte offset, inside a row block's LDS image, of chunk c of row r.
template <class Q>
__device__ __forceinline__ int swz(int r, int c) { return r * Q::RB + ((c ^ ((r / Q::SWD) % Q::SWM)) << 4); }

template <class T, int NB, int GH, int NX, int NV>
struct QuadLds {
    using Q = Quad<T, NB, GH>;
    static constexpr int CODES = 0;                                    // [GH][DV] rows, swizzled
    static constexpr int KBR = CODES + GH * Q::HEAD;                   // buffered keys, raw [m][DK]
    static constexpr int UBR = KBR + T::MMAX * T::DK * T::BE;          // buffered values, raw [GH][m][DV]
    static constexpr int XN = UBR + GH * T::MMAX * T::DV * T::BE;      // read-out vectors, fp32 [NX][DK]
    static constexpr int PL = XN + NX * T::DK * 4;                     // digit planes [k-step][half][8][16]
    static constexpr int XS = PL + T::DK * 8;                          // [NV][NG] exponent factors
    static constexpr int DOTS = XS + round_up(NV * T::NG * 4, 16);     // [NV][MMAX] K_i . x
    static constexpr int KBSF = DOTS + NV * T::MMAX * 4;               // [MMAX] key scales as fp32
    static constexpr int UBSF = KBSF + T::MMAX * 4;                    // [GH][MMAX] value scales as fp32
    static constexpr int SCAL = UBSF + GH * T::MMAX * 4;               // [GH][8] scalars of a head + [8] of the group
    static constexpr int RED = SCAL + (GH + 1) * 32;                   // one float per wavefront
    static constexpr int GBF = RED + round_up(Q::NW * 4, 16);          // [GH][MMAX] cumulative decays of the slots
    static constexpr int SC = GBF + GH * T::MMAX * 4;                  // [GH][DV][NG] fp16 scales of the rows
    static constexpr int BYTES = SC + round_up(GH * T::DV * T::NG * 2, 16);
};

// Where column e of a read-out vector goes in the digit-plane region: the (k-step, lane half, byte) at which the
// matrix core meets it with the codes.  int8: k-step ks, half kb carry columns 32 ks + 16 kb + [0, 16).  int4: a lane
// reads whole 16-byte chunks (32 columns) and feeds them as two k-steps, so k-step ks, half kb carry columns
// 32 (2 (ks / 2) + kb) + 16 (ks % 2) + [0, 16), in the nibble-split order of `operand`.
template <class T>
__device__ __forceinline__ int plane_addr(int e, int pl) {
    int ks, kb, pos;
    if constexpr (T::BITS == 8) {
        ks = e / 32; kb = (e / 16) % 2; pos = e % 16;
    } else {
        const int p = e / 32;
        kb = p % 2; ks = 2 * (p / 2) + (e % 32) / 16; pos = operand_pos<4>(e % 16);
    }
    return ((ks * 2 + kb) * 8 + pl) * 16 + pos;
}
template <class T>
__device__ __forceinline__ constexpr int op_colbase(int ks, int kb) {
    return T::BITS == 8 ? 32 * ks + 16 * kb : 32 * (2 * (ks / 2) + kb) + 16 * (ks % 2);
}

// Both values of a lane pair 16 / 32 lanes apart, in both lanes: {lower lane's, upper lane's}.
struct Pair { float lo, hi; };
__device__ __forceinline__ Pair pair32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(as_u32(v), as_u32(v), false, false);
    return Pair{as_f32(r[0]), as_f32(r[1])};
}
__device__ __forceinline__ Pair pair16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(as_u32(v), as_u32(v), false, false);
    return Pair{as_f32(r[0]), as_f32(r[1])};
}
// Sum / maximum over aligned blocks of N lanes, N a power of two up to 64; every lane of a block gets the result.
template <int N>
__device__ __forceinline__ float lanes_sum(float v) {
    v = block_sum<(N < 16 ? N : 16)>(v);
    if constexpr (N >= 32) { const Pair p = pair16(v); v = p.lo + p.hi; }
    if constexpr (N >= 64) { const Pair p = pair32(v); v = p.lo + p.hi; }
    return v;
}
template <int N>
__device__ __forceinline__ float lanes_max(float v) {
    v = block_max<(N < 16 ? N : 16)>(v);
    if constexpr (N >= 32) { const Pair p = pair16(v); v = fmaxf(p.lo, p.hi); }
    if constexpr (N >= 64) { const Pair p = pair32(v); v = fmaxf(p.lo, p.hi); }
    return v;
}

// One read-out vector -> its three digit planes (plane slots 3 v .. 3 v + 2) and its exponent factors; xe[t] =
// element NE lane + t.  Arithmetic as `stage_planes` in sq_tile.cuh: per scale group e = exponent of the largest
// |x|, q = rint(x 2^(22 - e)) cut into three signed 8-bit digits.
template <class T, int NE>
__device__ __forceinline__ void quad_stage_planes(const float (&xe)[NE], int v, int lane, uint8_t* lds_pl,
                                                  float* lds_xs) {
    float mx = 0.0f;
#pragma unroll
    for (int t = 0; t < NE; ++t) mx = fmaxf(mx, fabsf(xe[t]));
    constexpr int GL = T::KGROUP / NE;                       // lanes per scale group
    static_assert(GL >= 1 && GL <= WAVE, "scale group inside a wavefront");
    const float gmax = lanes_max<GL>(mx);
    int ex = __builtin_amdgcn_frexp_expf(gmax);
    ex = ex < -100 ? -100 : ex;
    const float up = __builtin_ldexpf(1.0f, 22 - ex);
    uint32_t d[NE];
#pragma unroll
    for (int t = 0; t < NE; ++t) {
        const float f = __builtin_fmaf(xe[t], up, 12582912.0f);
        d[t] = (as_u32(f) + 0x408080u) ^ 0x808080u;
    }
    const int e0 = NE * lane;
    if constexpr (T::BITS == 8 && NE == 2) {                 // neighbouring columns are neighbouring operand bytes
        uint8_t* at = lds_pl + plane_addr<T>(e0, 3 * v);
        *reinterpret_cast<uint16_t*>(at) = uint16_t((d[0] & 0xFFu) | ((d[1] & 0xFFu) << 8));
        *reinterpret_cast<uint16_t*>(at + 16) = uint16_t(((d[0] >> 8) & 0xFFu) | (d[1] & 0xFF00u));
        *reinterpret_cast<uint16_t*>(at + 32) = uint16_t(((d[0] >> 16) & 0xFFu) | ((d[1] >> 8) & 0xFF00u));
    } else {
#pragma unroll
        for (int t = 0; t < NE; ++t) {
            uint8_t* at = lds_pl + plane_addr<T>(e0 + t, 3 * v);
            at[0] = uint8_t(d[t]);
            at[16] = uint8_t(d[t] >> 8);
            at[32] = uint8_t(d[t] >> 16);
        }
    }
    if (e0 % T::KGROUP == 0) lds_xs[v * T::NG + e0 / T::KGROUP] = __builtin_ldexpf(1.0f, ex - 22 - (T::BITS == 4 ? 4 : 0));
}

// The digit planes as the matrix core's first operand, per k-step: lane (i, kb) carries result row i = 8 g + 4 v + d,
// i.e. digit d of vector v -- on the k-steps whose columns belong to scale group g, zero elsewhere (and zero in the
// unused rows), so that ONE accumulation over all k-steps leaves every group's sums in its own result rows.
template <class T, int NV>
__device__ __forceinline__ void quad_fetch_planes(const uint8_t* lds_pl, int lane, v4i (&aop)[T::NKS]) {
    const int i = lane & 31, kb = lane >> 5;
    const int g = i >> 3, v = (i >> 2) & 1, d = i & 3;
    const bool used = d < 3 && g < T::NG && v < NV;
#pragma unroll
    for (int ks = 0; ks < T::NKS; ++ks) {
        const v4i x = *reinterpret_cast<const v4i*>(lds_pl + ((ks * 2 + kb) * 8 + 3 * v + (d < 3 ? d : 0)) * 16);
        const bool mine = used && (kb == 0 ? op_colbase<T>(ks, 0) : op_colbase<T>(ks, 1)) / T::KGROUP == g;
        aop[ks] = mine ? x : v4i{0, 0, 0, 0};
    }
}

// Row sums of one 32-row block (its LDS image at `blk`): lane (n, kb) returns (S0 x_kb)[row n of the block] with the
// row's scales applied group by group, in order.  xs[g] = the exponent factor of vector kb, group g; sc[g] = the
// row's scales.
template <class Q, class T>
__device__ __forceinline__ float quad_block_pass(const uint8_t* blk, const v4i (&aop)[T::NKS], const float (&xs)[T::NG],
                                                 const float (&sc)[T::NG], int lane) {
    const int n = lane & 31, kb = lane >> 5;
    v16i acc = {0};
    if constexpr (T::BITS == 8) {
#pragma unroll
        for (int ks = 0; ks < T::NKS; ++ks) {
            const RawRow<8> r = load_row<8>(blk + swz<Q>(n, 2 * ks + kb));
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop[ks], operand<8>(r), acc, 0, 0, 0);
        }
    } else {
#pragma unroll
        for (int kp = 0; kp < T::NKS / 2; ++kp) {
            const uint4 c = *reinterpret_cast<const uint4*>(blk + swz<Q>(n, 2 * kp + kb));
            RawRow<4> lo, hi;
            lo.v = make_uint2(c.x, c.y);
            hi.v = make_uint2(c.z, c.w);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop[2 * kp], operand<4>(lo), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop[2 * kp + 1], operand<4>(hi), acc, 0, 0, 0);
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int g = 0; g < T::NG; ++g) {
        const float f = __builtin_fmaf(float(acc[4 * g + 2]), 65536.0f,
                                       __builtin_fmaf(float(acc[4 * g + 1]), 256.0f, float(acc[4 * g])));
        const float term = (f * xs[g]) * sc[g];
        s = g == 0 ? term : s + term;
    }
    return s;
}


// ---------------------------------------------------------------------------------------------------------------
// Row blocks loaded straight into their LDS image (global_load_lds_dwordx4: no pass through registers, no LDS store
// instructions).  Such a load writes lane l's 16 bytes at (uniform LDS base) + 16 l, so the image's swizzle goes into
// the global address instead: lane l fetches the chunk that belongs at position l of the 1 KB piece -- the lanes of a
// row still cover the row's lines, in another order.
//
// The compiler books a load-to-LDS as touching both memories and forces every wait that follows it down to "nothing
// outstanding", which would drain the row blocks before anything requested around them can be used.  So they are
// requested in assembly, invisible to that bookkeeping.  Loads complete in order, so every wait the compiler places
// for a load requested after them covers them as well; `quad_dma_landed` states it where the image is first read.
//
// The slot's fill counter decides which part of the decode buffer is requested, so it sits in front of those
// requests.  It is fetched with a SCALAR load: scalar loads have a counter of their own, so waiting for it does not
// wait for the row blocks requested behind it.  (The scalar cache is invalidated at every kernel start and the counter
// was written by an earlier launch; within a launch a slot's counter is written by its own workgroup only, at the
// end.)  The compiler would use a vector load here, because the same address is stored to later in the kernel.
// Between the load and its wait the compiler believes the register holds the value; build.py reads the device
// assembly of every unit of these kernels and refuses the build if anything touches that register in between
// (lint_counter_loads).
// ---------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ int quad_dma_counter(const int32_t* p) {
    int v;
    asm volatile("s_load_dword %0, %1, 0x0" : "=s"(v) : "s"(p) : "memory");
    return v;
}
__device__ __forceinline__ void quad_dma_counter_wait(int& counter) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(counter) :: "memory");
}
// NBLK row blocks of this wavefront: `src` their first byte in memory, `dst` their LDS image.  Every 1 KB piece gets
// its own address pair and LDS base on purpose: the four pieces of a block behind one address with the instruction's
// immediate offsets (which advance both addresses) issue back to back and measured slower (headline 33.1 against
// 32.7 us per launch, Mamba2 32.1 against 31.1) -- the address arithmetic in between spaces a wavefront's requests.
template <class Q, int NBLK>
__device__ __forceinline__ void quad_dma_blocks(const uint8_t* src, uint8_t* dst, int lane) {
    const int pr = lane / Q::CPR, pc = lane % Q::CPR;
#pragma unroll
    for (int bi = 0; bi < NBLK; ++bi)
#pragma unroll
        for (int t = 0; t < Q::NLD; ++t) {
            const int r = t * (1024 / Q::RB) + pr;
            const int c = pc ^ ((r / Q::SWD) % Q::SWM);
            const uint8_t* g = src + bi * Q::BLK + r * Q::RB + (c << 4);
            const uint32_t at = uint32_t(reinterpret_cast<uintptr_t>(
                (__attribute__((address_space(3))) uint8_t*)(dst + bi * Q::BLK + t * 1024)));
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
                         :: "v"(g), "s"(at) : "memory", "m0");
        }
}
__device__ __forceinline__ void quad_dma_landed() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Raw buffered elements: four per lane.
template <bool QBUF> struct Raw4;
template <> struct Raw4<true> { uint32_t a; };
template <> struct Raw4<false> { v2u a; };
template <bool QBUF>
__device__ __forceinline__ Raw4<QBUF> load_raw4(const uint8_t* p) {
    Raw4<QBUF> r;
    if constexpr (QBUF) r.a = *reinterpret_cast<const uint32_t*>(p);
    else r.a = *reinterpret_cast<const v2u*>(p);
    return r;
}
template <bool QBUF>
__device__ __forceinline__ Raw4<QBUF> stream_raw4(const uint8_t* p) {       // the same through `stream_load`
    Raw4<QBUF> r;
    if constexpr (QBUF) r.a = stream_load(reinterpret_cast<const uint32_t*>(p));
    else r.a = stream_load(reinterpret_cast<const v2u*>(p));
    return r;
}
template <bool QBUF>
__device__ __forceinline__ void store_raw4(uint8_t* p, const Raw4<QBUF>& r) {
    if constexpr (QBUF) *reinterpret_cast<uint32_t*>(p) = r.a;
    else *reinterpret_cast<v2u*>(p) = r.a;
}
template <bool QBUF>
__device__ __forceinline__ void decode_raw4(const Raw4<QBUF>& r, float (&f)[4]) {
    if constexpr (QBUF) {
#pragma unroll
        for (int b = 0; b < 4; ++b) f[b] = s8_to_f(r.a, b);
    } else {
        f[0] = as_f32(r.a.x << 16); f[1] = as_f32(r.a.x & 0xFFFF0000u);
        f[2] = as_f32(r.a.y << 16); f[3] = as_f32(r.a.y & 0xFFFF0000u);
    }
}
// One raw buffered element from LDS as fp32 (unscaled).
template <bool QBUF>
__device__ __forceinline__ float lds_raw(const uint8_t* base, int idx) {
    if constexpr (QBUF) return float(reinterpret_cast<const int8_t*>(base)[idx]);
    else return bf16_to_f32(reinterpret_cast<const uint16_t*>(base)[idx]);
}

// ---------------------------------------------------------------------------------------------------------------
// the fold of one row block held in LDS
// ---------------------------------------------------------------------------------------------------------------
// fp32 value of byte `b` of `w` taken as unsigned, times s, plus o (one conversion + one fma per code; with
// w = codes ^ 0x80.. and o = -128 s this is (code x s) rounded once, bit-identical to convert-then-multiply).
template <int B>
__device__ __forceinline__ float ubyte_fma(uint32_t w, float s, float o) {
    float f;                                                 // one instruction whichever byte (left to the compiler,
    if constexpr (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(w));      // bytes 1 .. 3 of a masked word
    else if constexpr (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(w)); // cost a shift each)
    else if constexpr (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(w));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(w));
    return __builtin_fmaf(f, s, o);
}

// S = cmul S0 + sum_i du_i (x) kx_i over the m buffer slots, four slots per matrix-core issue in slot order
// (v_mfma_f32_16x16x4_f32, fp32), re-quantized into the block's LDS image and its scales (reference:
// _fused_triton.py:278-394 `_fold_head`).  Half a row block at a time: lane (n, q) -- n = lane % 16 the row of the
// half, q = lane / 16 -- owns the quarter q of row n, CL = d_k / 4 consecutive columns, as CL / 4 accumulator tiles
// of 4 columns: the instruction leaves result rows 4 q + b of result column n in lane (n, q), and the keys are fed
// so that result row 4 q' + b of tile ct is state column q' CL + 4 ct + b.  A lane's codes are whole 16-byte (8-byte)
// pieces of the LDS image, a scale group lies in 1, 2 or 4 lanes of a row (lanes 16 or 32 apart), and a 128-column
// row needs 32 accumulator registers.
//   lds_kbr / kbsf   buffered keys, raw, and their scales (slot m - 1: this token's, as stored)
//   bop[t]           the lane's folded values: slot 4 t + q, row n (decay ratio x stored value)
//   cmul             the decay of the old state over the buffer
typedef float v4f __attribute__((ext_vector_type(4)));

// The folded keys as the matrix core's first operand, once per wavefront (they are the same for every half block):
// key(ct, t) = kx_{4 t + q}[column (n / 4) CL + 4 ct + n % 4] for lane (n, q); 0 for slots >= m.  Held as fp32, or --
// int4 states with the int8 buffer, whose kernels run at 80 registers where 16 more long-lived ones made the compiler
// shuffle and spill -- as the raw bytes (biased to unsigned, four per register) with the slot's scale, expanded where
// they are used: (byte - 128) x scale in one conversion and one fma, the same number as the product it replaces.
template <class T>
struct FoldKeys {
    static constexpr int MT4 = (T::MMAX + 3) / 4, NT = T::DK / 16;
    static constexpr bool PACKED = T::BITS == 4 && T::QBUF && NT % 4 == 0;
    float f[PACKED ? 1 : NT][PACKED ? 1 : MT4];
    uint32_t raw[PACKED ? MT4 : 1][PACKED ? NT / 4 : 1];
    float ks[PACKED ? MT4 : 1], off[PACKED ? MT4 : 1];
    template <int CT, int TT>
    __device__ __forceinline__ float get() const {
        if constexpr (PACKED) return ubyte_fma<CT % 4>(raw[TT][CT / 4], ks[TT], off[TT]);
        else return f[CT][TT];
    }
};

template <class T>
__device__ __forceinline__ void quad_fold_keys(const uint8_t* lds_kbr, const float* lds_kbsf, int m, int lane,
                                               FoldKeys<T>& kop) {
    constexpr int MT4 = (T::MMAX + 3) / 4, CL = T::DK / 4, NT = CL / 4;
    const int n = lane & 15, q = lane >> 4;
    const int kcol = (n >> 2) * CL + (n & 3);
#pragma unroll
    for (int t = 0; t < MT4; ++t) {
        const int slot = 4 * t + q;
        const int sl = slot < m ? slot : 0;
        const float ks = T::QBUF ? lds_kbsf[sl] : 1.0f;
        if constexpr (FoldKeys<T>::PACKED) {
#pragma unroll
            for (int c4 = 0; c4 < NT / 4; ++c4) {
                uint32_t w = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) w |= uint32_t(lds_kbr[sl * T::DK + kcol + 4 * (4 * c4 + b)]) << (8 * b);
                kop.raw[t][c4] = w ^ 0x80808080u;
            }
            kop.ks[t] = slot < m ? ks : 0.0f;                 // a slot beyond m contributes nothing
            kop.off[t] = -128.0f * kop.ks[t];
        } else {
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) {
                float kv = lds_raw<T::QBUF>(lds_kbr, sl * T::DK + kcol + 4 * ct);
                if constexpr (T::QBUF) kv = kv * ks;
                kop.f[ct][t] = slot < m ? kv : 0.0f;
            }
        }
    }
}

template <class Q, class T>
__device__ __forceinline__ void quad_fold_half(uint8_t* blk, int hf, const FoldKeys<T>& kop,
                                               const float (&bop)[(T::MMAX + 3) / 4], float cmul, float s_old,
                                               uint16_t* sc_out, int lane) {
    constexpr int MT4 = (T::MMAX + 3) / 4;
    constexpr int CL = T::DK / 4;                            // columns per lane
    constexpr int NT = CL / 4;                               // accumulator tiles per lane
    constexpr int NBY = Q::RB / 4;                           // bytes per lane
    constexpr int NW32 = NBY / 4;                            // 32-bit words per lane
    static_assert(CL % 16 == 0 && T::KGROUP % CL == 0 && T::KGROUP / CL <= 4, "a scale group is 1, 2 or 4 lanes wide");
    constexpr int LPG = T::KGROUP / CL;
    const int n = lane & 15, q = lane >> 4;
    const int row = 16 * hf + n;
    // where the lane's bytes of the row sit in the LDS image
    const int at = NBY >= 16 ? swz<Q>(row, q * (NBY / 16)) : swz<Q>(row, q >> 1) + 8 * (q & 1);
    const int at1 = NBY >= 32 ? swz<Q>(row, q * (NBY / 16) + 1) : at;      // its second chunk (int8, d_k 128)
    static_assert(NBY <= 32, "at most two chunks per lane");

    uint32_t w[NW32];
    if constexpr (NBY >= 16) {
#pragma unroll
        for (int c = 0; c < NBY / 16; ++c) {
            const v4u x = *reinterpret_cast<const v4u*>(blk + (c == 0 ? at : at1));
            w[4 * c] = x.x; w[4 * c + 1] = x.y; w[4 * c + 2] = x.z; w[4 * c + 3] = x.w;
        }
    } else {
        const v2u x = *reinterpret_cast<const v2u*>(blk + at);
        w[0] = x.x; w[1] = x.y;
    }
    // dequantize: (code x scale) x factor, one conversion + one fma per code
    const float s = T::BITS == 8 ? s_old : s_old * 0.0625f;
    const float sm = s * cmul;
    const float off = -128.0f * sm;
    v4f acc[NT];
    // int8 with one scale group per row: the whole half block is folded in units of the row's old scale x decay
    // (S / sm = code + sum_i (du_i / sm) kx_i), so the codes need neither conversion nor multiplication on the vector
    // ALU -- they enter the accumulators through the matrix core: each byte, biased to unsigned, becomes the fp16
    // number 1024 + byte by a byte permute (exponent byte 0x64 on top), and one v_mfma_f32_16x16x16_f16 against the
    // 16 x 16 identity hands every lane its own four numbers back as fp32 on top of the constant -1152 (exact).
    constexpr bool UNITS = T::BITS == 8 && T::NG == 1;
    // An old scale at its floor is an empty group (or one too small to matter), and a decay of exactly 1 leaves the
    // stored codes times their scale as they are: what is quantized then is a sum of a few products of low-precision
    // numbers, whose quotients by the new scale are exact half-integers by the thousand -- the codes are taken as
    // rint of the IEEE quotient there (quantize_row<.., EXACT>), which sends them to even as the reference's do.
    const bool exact = __builtin_amdgcn_ballot_w64(s_old <= FP16_TINY || cmul == 1.0f) != 0;
    float unit = 1.0f;                                       // what one accumulator unit is worth
    if constexpr (UNITS) {
        typedef _Float16 v4h __attribute__((ext_vector_type(4)));
        unit = fmaxf(sm, 1e-30f);                            // a vanished old state: its term is below any scale
        // exact mode: a power of two as the unit, so that scaling by it rounds nothing (the codes then count ratio
        // = sm / unit each instead of 1)
        const float p2 = as_f32(as_u32(unit) & 0x7F800000u);
        const float ratio = exact ? sm * __builtin_amdgcn_rcpf(p2) : 1.0f;     // the reciprocal of a power of two: exact
        if (exact) unit = p2;
        v4h ident;
#pragma unroll
        for (int j = 0; j < 4; ++j) ident[j] = (n == 4 * q + j) ? _Float16(1.0f) : _Float16(0.0f);
        const v4f bias = {-1152.0f, -1152.0f, -1152.0f, -1152.0f};
#pragma unroll
        for (int d = 0; d < NW32; ++d) {
            const uint32_t u = w[d] ^ 0x80808080u;
            v2u h2;
            h2.x = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);      // halves 1024 + byte 0, 1024 + byte 1
            h2.y = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);      // bytes 2, 3
            acc[d] = __builtin_amdgcn_mfma_f32_16x16x16f16(ident, __builtin_bit_cast(v4h, h2), bias, 0, 0, 0);
        }
        if (exact) {
            asm volatile("" ::: "memory");                   // a real branch: not 32 multiplications by 1 otherwise
#pragma unroll
            for (int d = 0; d < NW32; ++d) acc[d] = acc[d] * ratio;
        }
    } else if constexpr (T::BITS == 8) {
#pragma unroll
        for (int d = 0; d < NW32; ++d) {
            const uint32_t u = w[d] ^ 0x80808080u;
            acc[d][0] = ubyte_fma<0>(u, sm, off); acc[d][1] = ubyte_fma<1>(u, sm, off);
            acc[d][2] = ubyte_fma<2>(u, sm, off); acc[d][3] = ubyte_fma<3>(u, sm, off);
        }
    } else {
        // a stored nibble is code + 8: moved to the high half of a byte it reads 16 code + 128 as an unsigned byte
#pragma unroll
        for (int d = 0; d < NW32; ++d) {                     // word d: columns 8 d .. 8 d + 7
            const uint32_t lo = (w[d] << 4) & 0xF0F0F0F0u, hi = w[d] & 0xF0F0F0F0u;
            acc[2 * d][0] = ubyte_fma<0>(lo, sm, off); acc[2 * d][1] = ubyte_fma<0>(hi, sm, off);
            acc[2 * d][2] = ubyte_fma<1>(lo, sm, off); acc[2 * d][3] = ubyte_fma<1>(hi, sm, off);
            acc[2 * d + 1][0] = ubyte_fma<2>(lo, sm, off); acc[2 * d + 1][1] = ubyte_fma<2>(hi, sm, off);
            acc[2 * d + 1][2] = ubyte_fma<3>(lo, sm, off); acc[2 * d + 1][3] = ubyte_fma<3>(hi, sm, off);
        }
    }
    // the m rank-1 updates: first operand = keys (result row i = 4 q' + b <-> column q' CL + 4 ct + b), second = values
    float bv[MT4];
    {
        // units are this kernel's own device (no reference quantity): an estimate plus one Newton step is plenty
        const float r0 = __builtin_amdgcn_rcpf(unit);
        const float runit = UNITS ? __builtin_fmaf(__builtin_fmaf(-unit, r0, 1.0f), r0, r0) : 1.0f;
#pragma unroll
        for (int t = 0; t < MT4; ++t) bv[t] = UNITS ? bop[t] * runit : bop[t];
    }
    static_for<NT>([&](auto ct) {
        static_for<MT4>([&](auto t) {
            acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(kop.template get<decltype(ct)::value, decltype(t)::value>(), bv[t], acc[ct], 0, 0, 0);
        });
    });
    // absmax of the lane's columns (three-operand maxima), then of its scale group
    float mx = 0.0f;
#pragma unroll
    for (int ct = 0; ct < NT; ++ct) {
        mx = fmaxf(fmaxf(mx, fabsf(acc[ct][0])), fabsf(acc[ct][1]));
        mx = fmaxf(fmaxf(mx, fabsf(acc[ct][2])), fabsf(acc[ct][3]));
    }
    if constexpr (LPG >= 2) { const Pair pm = pair16(mx); mx = fmaxf(pm.lo, pm.hi); }
    if constexpr (LPG >= 4) { const Pair pm = pair32(mx); mx = fmaxf(pm.lo, pm.hi); }
    const float sc = fp16_scale(UNITS ? mx * unit : mx, T::QMAX);
    const Divisor dsc = scale_divisor(sc);                   // sc is an fp16 value: the correctly rounded reciprocal
    const float rs = UNITS ? unit * dsc.rc : dsc.rc;         // (exact mode: unit is a power of two, both stay exact)
    const float ds = UNITS ? dsc.d * __builtin_amdgcn_rcpf(unit) : dsc.d;
    if (q % LPG == 0) *sc_out = f32_to_f16(sc);
    // new codes, back into the LDS image.  A scale in fp16's normal range cannot push a quotient past qmax + 1/2, so
    // the clamp is only compiled into the path taken when some lane's scale is subnormal (or at its floor).
    auto requantize = [&](auto clamp, auto exactly) {
        constexpr bool CLAMP = decltype(clamp)::value, EXACT = decltype(exactly)::value;
        if constexpr (NBY >= 16) {
#pragma unroll
            for (int c = 0; c < CL / 16; ++c) {              // 16 columns per call
                float a16[CPL];
#pragma unroll
                for (int e = 0; e < CPL; ++e) a16[e] = acc[4 * c + e / 4][e % 4];
                const RawRow<T::BITS> r = quantize_row<T::BITS, CLAMP, EXACT>(a16, rs, ds);
                if constexpr (T::BITS == 8) *reinterpret_cast<uint4*>(blk + (c == 0 ? at : at1)) = r.v;
                else *reinterpret_cast<uint2*>(blk + at + 8 * c) = r.v;      // 16 columns = half a chunk
            }
        } else {
            float a16[CPL];
#pragma unroll
            for (int e = 0; e < CPL; ++e) a16[e] = acc[e / 4][e % 4];
            const RawRow<T::BITS> r = quantize_row<T::BITS, CLAMP, EXACT>(a16, rs, ds);
            *reinterpret_cast<uint2*>(blk + at) = r.v;
        }
    };
    if (exact) requantize(std::true_type{}, std::true_type{});
    else if (__builtin_amdgcn_ballot_w64(sc < 6.103515625e-05f) != 0) requantize(std::true_type{}, std::false_type{});
    else requantize(std::false_type{}, std::false_type{});
}

}  // namespace sq
