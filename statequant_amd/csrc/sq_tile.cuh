// The state tile of one (sequence, value head) in one wavefront: geometry, the streaming read of the stored codes
// with the row dot products, the decode buffer, and the fold (advance across the full buffer + re-quantize in
// place).  Shared by the Gated DeltaNet, KDA and Mamba2 step kernels.
//
// Row dot products.  S0 x (x = q, k, ...) over int8 / int4 codes is an integer dot product per row and scale group
// once x is in fixed point.  x is cut, per scale group, into three signed 8-bit digits of a 23-bit fixed-point
// number (exponent = that of the group's largest |x|), and the codes meet the digit planes in the matrix core's
// int8 dot-product instruction (v_mfma_i32_32x32x32_i8: 32 rows x 32 columns of codes against up to 32 planes per
// issue, int32 accumulation, exact).  A vector-ALU formulation (convert every code to fp32, one fma per code and
// vector) costs ~50 instructions per 16-code row piece and made the step ALU-bound at under half the HBM rate; the
// matrix core takes the codes as loaded (int8) or after a nibble split (int4) and leaves the vector ALU to the
// per-row work.  The digits' rounding (|x| 2^-23 of the group maximum per element) is of the order of fp32
// accumulation error.
//
// Resource plan (what keeps four wavefronts per SIMD resident): the codes stream through a window of two 32-row
// blocks per wavefront (32 VGPRs for int8), loaded row-shaped (whole rows per instruction) and turned into matrix
// operands through one 4.6 KB LDS block, refilled block by block; the small operands (buffered values, scales) are
// fetched with one coalesced 128-bit load per lane and parked in LDS until needed; the fold reads the codes a second
// time instead of pinning them on chip (16 KB per wavefront, more than registers or LDS can spare at this occupancy)
// and runs its rank-1 updates on the matrix core in fp32; the fold's LDS operands overlay the front end's.
#pragma once
#include "sq_device.cuh"

namespace sq {

// Compile-time geometry.  A row of DK codes is cut into DK/16 pieces of 16 columns; LPRP (that count rounded up to a
// power of two) consecutive lanes hold one row, lanes past DK/16 idle (d_k = 96: 6 of 8).  The wavefront therefore
// covers RG = 64/LPRP rows per load and a lane sees rows rg, rg + RG, rg + 2 RG, ...  (the fold and the buffer passes
// use this shape; the state pass uses the matrix core's, below).
// AXV: the scale groups run along the VALUE axis instead (GROUP consecutive rows share one scale per key column;
// scales [DV / GROUP][DK]); built for GROUP = 32, one row block of the matrix-core passes.
// BITS = 16 / 32: the unquantized control -- the state kept as bf16 / fp32 [DV][DK], no scales (FLT below).  The front
// end (vectors, buffer, append) keeps the geometry above; the state rows have their own: a lane's 16 bytes are SPL =
// 8 / 4 columns, SLPRP lanes hold a row, a wavefront load covers SRG rows, NLD loads the tile.
template <int BITS_, int DK_, int DV_, int GROUP_, bool QBUF_, int MMAX_, bool AXV_ = false>
struct Tile {
    static constexpr int BITS = BITS_, DK = DK_, DV = DV_, GROUP = GROUP_, MMAX = MMAX_;
    static constexpr bool QBUF = QBUF_, AXV = AXV_;
    static_assert(BITS == 4 || BITS == 8 || BITS == 16 || BITS == 32, "int4 / int8 codes, or a bf16 / fp32 state");
    static constexpr bool FLT = BITS >= 16;
    static_assert(!FLT || (!AXV && GROUP == DK), "a float state has no scale groups");
    static_assert(DK % CPL == 0 && DK >= 32 && DK <= 256, "d_k must be a multiple of 16 in 32..256");
    static constexpr int LPR = DK / CPL;                  // live lanes per row
    static constexpr int LPRP = pow2_ceil(LPR);           // lanes per row incl. idle ones
    static constexpr int RG = WAVE / LPRP;                // rows per wavefront load
    static_assert(DV % RG == 0 && DV >= 32, "d_v must be a multiple of the rows one wavefront load covers");
    static constexpr int RPL = DV / RG;                   // rows per lane (fold, buffer passes)
    static constexpr int NOWN = (DV + WAVE - 1) / WAVE;   // rows a lane owns after the state pass: lane + 64 t
    static constexpr int KGROUP = AXV ? pow2_ceil(DK) : GROUP;     // length of a scale group along a row
    static constexpr int NG = (DK + KGROUP - 1) / KGROUP; // stored key groups per row (last may be ragged); AXV: 1
    static_assert(GROUP % CPL == 0 && GROUP >= CPL, "key group must be a multiple of 16");
    static constexpr int LPG = (GROUP / CPL < LPRP) ? GROUP / CPL : LPRP;   // lanes sharing one scale
    static constexpr int ROW_BYTES = DK * BITS / 8;
    static constexpr int LANE_BYTES = BITS == 4 ? CPL / 2 : CPL;
    static constexpr float QMAX = float((1 << ((FLT ? 8 : BITS) - 1)) - 1);   // unused for a float state
    static constexpr int SPL = FLT ? 128 / BITS : CPL;    // float state: columns per 16-byte lane piece
    static constexpr int SLPR = DK / SPL;
    static constexpr int SLPRP = pow2_ceil(SLPR);
    static_assert(SLPRP <= WAVE, "a float-state row must fit one wavefront load");
    static constexpr int SRG = WAVE / SLPRP;
    static constexpr int NLD = DV / SRG;
    static constexpr int NE = (DK + WAVE - 1) / WAVE;     // elements of a d_k vector per lane (element = lane + 64 t)
    static constexpr int BE = QBUF ? 1 : 2;               // bytes per buffer element (int8 / bf16)
    static constexpr int KPAD = CPL + 4;                  // LDS stride of a 16-column piece (spreads the banks)
    static constexpr int KROW = LPRP * KPAD;              // floats per d_k vector in LDS
    static constexpr int UROW = NOWN * WAVE;              // floats per d_v vector in LDS
    // matrix-core pass: blocks of MR rows x MK columns (one lane: one row, 16 columns; lanes 32.. the next 16)
    static constexpr int MR = 32, MK = 32;
    static_assert(DK % MK == 0 && (AXV || GROUP % MK == 0), "d_k / key-axis group must be multiples of 32");
    // d_v need not be a multiple of the block height (Nemotron-3-Nano: head_dim 80): the last row block is then
    // partly empty -- its wavefront loads beyond d_v are skipped (zeros), its stores and scales masked
    static constexpr bool RAGV = DV % MR != 0;
    static_assert(!AXV || ((2 * GROUP == MR || GROUP == MR || GROUP == 2 * MR) && DV % GROUP == 0),
                  "value-axis groups are half a row block, one or two (16, 32 or 64 rows)");
    static constexpr int VB = AXV && GROUP > MR ? GROUP / MR : 1;    // row blocks per value-axis scale group
    static constexpr int VH = AXV && GROUP < MR ? MR / GROUP : 1;    // value-axis scale groups per row block
    static constexpr int PSLOTS = VH > 1 ? 16 : 8;        // digit-plane slots per 16-column piece
    static constexpr int NRB = (DV + MR - 1) / MR;        // row blocks (the last one may be partly empty)
    static constexpr int NKS = DK / MK;                   // column steps
    static constexpr int PLANES = 3;                      // fixed-point digits per read-out vector
    // digit planes: [16-column piece][8 planes][16]; float state: the read-out vectors themselves (at most two)
    static constexpr int B_BYTES = FLT ? 2 * KROW * 4 : (DK / CPL) * PSLOTS * CPL;
    static constexpr int A_PITCH = ROW_BYTES + LANE_BYTES;  // LDS row pitch of a row block on its way to operand shape
    static constexpr int A_BYTES = FLT ? 0 : MR * A_PITCH;
    static constexpr int UB_BYTES = round_up(MMAX * DV * BE, 16);
    static constexpr int SC_ELEMS = FLT ? 0 : AXV ? (DV / GROUP) * DK : DV * NG;      // fp16 scales of one head
    static constexpr int SC_BYTES = FLT ? 16 : round_up(SC_ELEMS * 2, 16);
};

// LDS plan of a step kernel that stages NX d_k vectors and reads the state out against NV of them.  Front end: the
// vectors, the raw buffered values, the raw scales, the digit planes with their exponents, one row block of codes,
// the finished row sums.  Fold: folded keys, folded values, column multipliers.  The two overlay each other.
template <class T, int NX, int NV = 2>
struct LdsPlan {
    static constexpr int X = 0;
    static constexpr int UB = X + NX * T::KROW * 4;
    static constexpr int SC = UB + T::UB_BYTES;
    static constexpr int XS = SC + T::SC_BYTES;
    // one region, two tenants in turn: the digit planes (until the pass has them in registers), then per row block
    // the codes on their way to operand shape
    static constexpr int B = XS + round_up(NV * T::VH * T::NG * 4, 16);
    static constexpr int A = B + (T::AXV ? T::B_BYTES : 0);    // value-axis: planes are rebuilt per row block
    static constexpr int BA = T::A_BYTES > T::B_BYTES ? T::A_BYTES : T::B_BYTES;
    static constexpr int OWN = A + BA;
    static constexpr int FRONT = OWN + NV * T::UROW * 4;
    static constexpr int FK = 0;
    static constexpr int FU = FK + T::MMAX * T::KROW * 4;
    static constexpr int FC = FU + T::MMAX * T::UROW * 4;
    static constexpr int FOLD = FC + T::KROW * 4;
    static constexpr int BYTES = FRONT > FOLD ? FRONT : FOLD;
    static_assert(T::MMAX * T::KROW * 4 >= T::A_BYTES, "the fold reuses the key region as its row-block buffer");
};

// LDS position of element e of a d_k vector stored piecewise.
template <class T>
__device__ __forceinline__ int kpos(int e) { return (e / CPL) * T::KPAD + e % CPL; }

struct LaneId {
    int lane, cg, rg;
};
template <class T>
__device__ __forceinline__ LaneId lane_id() {
    LaneId l;
    l.lane = threadIdx.x;
    l.cg = l.lane % T::LPRP;
    l.rg = l.lane / T::LPRP;
    return l;
}

// Row index (within the head) of a lane's j-th row.
template <class T>
__device__ __forceinline__ int row_of(const LaneId& l, int j) { return j * T::RG + l.rg; }

// Which (batch row, value head) a workgroup works on; the caller adds the key head.  Consecutive workgroup ids are
// dealt round-robin to the 8 XCDs; with `per_xcd` set every XCD walks a contiguous range of tiles, so the heads of one
// sequence (shared key buffer, neighbouring counters) meet in one L2.  `order` (optional) names the batch row that each
// position of this walk works on.
// The arguments are the kernel's leading scalar arguments -- copies of those fields of the parameter struct.
// Separate scalar arguments ahead of the struct are in registers when a wavefront starts, so the slot index load that
// depends on the batch row need not wait for the argument block to be loaded.  SPEC > 0: the serving cases (a
// power-of-two head count).
struct TileId {
    int b, h, hk;
};
template <int SPEC>
__device__ __forceinline__ TileId tile_id_lead(const int32_t* order, int per_xcd, int hv, int hv_shift) {
    const int wg = blockIdx.x;
    const int tile = per_xcd ? (wg & 7) * per_xcd + (wg >> 3) : wg;
    TileId t;
    t.b = (SPEC > 0 || hv_shift >= 0) ? tile >> hv_shift : tile / hv;
    t.h = tile - t.b * hv;
    if (order) t.b = order[t.b];                  // the caller's dispatch order: position -> batch row
    t.hk = t.h;
    return t;
}
// Address of a per-sequence field: base + sequence x stride + offset inside the sequence, in elements of E.
template <class E>
__device__ __forceinline__ E* field(E* base, uint32_t seq, uint32_t stride, uint32_t off) {
    return base + (uint64_t(seq) * stride + off);
}

// The head rows a lane owns after the state pass (epilogue, append, fold staging): lane + 64 t.
template <class T>
__device__ __forceinline__ int owned_row(const LaneId& l, int t) { return l.lane + WAVE * t; }
template <class T>
__device__ __forceinline__ bool owned_valid(const LaneId& l, int t) { return l.lane + WAVE * t < T::DV; }

// ---------------------------------------------------------------------------------------------------------------
// coalesced staging of a small byte range into LDS: lane i carries bytes [16 i + 1024 c, +16) of it
// ---------------------------------------------------------------------------------------------------------------
template <int MAXBYTES>
struct Staged {
    static constexpr int N = (MAXBYTES + 1023) / 1024;
    uint4 v[N];
};
template <int MAXBYTES>
__device__ __forceinline__ void stage_load(const uint8_t* src, int nbytes, int lane, Staged<MAXBYTES>& s) {
#pragma unroll
    for (int c = 0; c < Staged<MAXBYTES>::N; ++c) {
        const int off = lane * 16 + c * 1024;
        s.v[c] = *reinterpret_cast<const uint4*>(src + (off < nbytes ? off : 0));      // clamped, never branched
    }
}
template <int MAXBYTES>
__device__ __forceinline__ void stage_store(uint8_t* lds, int nbytes, int lane, const Staged<MAXBYTES>& s) {
#pragma unroll
    for (int c = 0; c < Staged<MAXBYTES>::N; ++c) {
        const int off = lane * 16 + c * 1024;
        if (off < nbytes) *reinterpret_cast<uint4*>(lds + off) = s.v[c];
    }
}

// ---------------------------------------------------------------------------------------------------------------
// the streaming pass over the stored codes
// ---------------------------------------------------------------------------------------------------------------
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// Byte position, inside a lane's 16-byte matrix operand, of the lane's column c (0..15).  int8: as stored.  int4: the
// operand is {low nibbles of word 0, high nibbles of word 0, low of word 1, high of word 1}, byte k of a word holding
// columns 2k and 2k + 1.
template <int BITS>
__device__ __forceinline__ int operand_pos(int c) {
    if constexpr (BITS == 8) return c;
    else return 4 * (2 * (c / 8) + (c % 2)) + (c % 8) / 2;
}
// A lane's codes of one row piece as a matrix operand of 16 signed bytes.  int4: a stored nibble is code + 8; with
// bit 3 flipped it is the code in 4-bit two's complement, and in the HIGH half of a byte that reads as 16 x code
// (the pass divides the sums by 16 again, exactly).
template <int BITS>
__device__ __forceinline__ v4i operand(const RawRow<BITS>& r) {
    if constexpr (BITS == 8) {
        return v4i{int(r.v.x), int(r.v.y), int(r.v.z), int(r.v.w)};
    } else {
        const uint32_t w0 = r.v.x ^ 0x88888888u, w1 = r.v.y ^ 0x88888888u;
        return v4i{int((w0 << 4) & 0xF0F0F0F0u), int(w0 & 0xF0F0F0F0u), int((w1 << 4) & 0xF0F0F0F0u),
                   int(w1 & 0xF0F0F0F0u)};
    }
}

// Read-out vectors -> digit planes.  xe[v][t] = element lane + 64 t of vector v (0 past d_k).  Per vector and scale
// group: e = exponent of the group's largest |x| (|x| < 2^e), fixed point q = rint(x 2^(22-e)), |q| <= 2^22,
// q = d0 + 2^8 d1 + 2^16 d2 with signed 8-bit digits.  x 2^(22-e) + 1.5 2^23 (one fma) leaves 2^22 + q in the low
// mantissa bits; adding the digit bias 0x808080 - 2^22 and flipping the three sign bits yields the digits as bytes.
// lds_b[piece][plane 3 v + d][operand_pos]: what `state_pass` loads as its second operand;  lds_xs[v][group] =
// 2^(e-22) (int4: / 16), the factor that turns the integer sums back.
template <class T, int NV>
__device__ __forceinline__ void stage_planes(const float (&xe)[NV][T::NE], const LaneId& l, uint8_t* lds_b,
                                             float* lds_xs) {
    constexpr int NBLK = WAVE / 16;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float mb[T::NE][NBLK];                               // max |x| over each run of 16 columns (wave-uniform)
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const float m16 = block_max<16>(fabsf(xe[v][t]));
#pragma unroll
            for (int k = 0; k < NBLK; ++k) mb[t][k] = lane_bcast(m16, 16 * k);
        }
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            float gm[2];                                     // group maximum for the lanes below / from 32
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int g = (WAVE * t + 32 * hf) / T::KGROUP;
                float mx = 0.0f;
#pragma unroll
                for (int t2 = 0; t2 < T::NE; ++t2)
#pragma unroll
                    for (int k = 0; k < NBLK; ++k)
                        if ((WAVE * t2 + 16 * k) / T::KGROUP == g && WAVE * t2 + 16 * k < T::DK)
                            mx = fmaxf(mx, mb[t2][k]);
                gm[hf] = mx;
            }
            const float gmax = l.lane < 32 ? gm[0] : gm[1];
            int ex = __builtin_amdgcn_frexp_expf(gmax);
            ex = ex < -100 ? -100 : ex;
            const float f = __builtin_fmaf(xe[v][t], __builtin_ldexpf(1.0f, 22 - ex), 12582912.0f);
            const uint32_t d = (as_u32(f) + 0x408080u) ^ 0x808080u;
            const int e = l.lane + WAVE * t;
            if (e < T::DK) {
                uint8_t* at = lds_b + ((e / CPL) * T::PSLOTS + T::PLANES * v) * CPL + operand_pos<T::BITS>(e % CPL);
                at[0] = uint8_t(d);
                at[CPL] = uint8_t(d >> 8);
                at[2 * CPL] = uint8_t(d >> 16);
                if (e % T::KGROUP == 0)
                    lds_xs[v * T::NG + e / T::KGROUP] = __builtin_ldexpf(1.0f, ex - 22 - (T::BITS == 4 ? 4 : 0));
            }
        }
    }
}

// A lane's first row piece in the row-shaped layout (LPRP lanes per row).
template <class T>
__device__ __forceinline__ const uint8_t* lane_codes(const uint8_t* head, const LaneId& l) {
    if constexpr (T::FLT) {
        const int scg = l.lane % T::SLPRP, srg = l.lane / T::SLPRP;
        return head + srg * T::ROW_BYTES + (scg < T::SLPR ? scg : T::SLPR - 1) * 16;
    }
    const int cc = l.cg < T::LPR ? l.cg : T::LPR - 1;       // idle lanes shadow a live one (masked later)
    return head + l.rg * T::ROW_BYTES + cc * T::LANE_BYTES;
}

// Two row blocks of codes in flight per wavefront, loaded row-shaped (LPRP lanes per row, so every load instruction
// covers whole, consecutive rows and costs the address unit one cycle per 64 bytes; fetched in operand shape -- 32
// different rows per instruction -- the same bytes cost it 8 x as many cycles and the step became address-bound).
template <class T, bool FLT = T::FLT>
struct Window {
    static constexpr int NL = T::MR / T::RG;              // loads per row block
    RawRow<T::BITS> a[2][NL];
};
// Float state: the next FW wavefront loads (SRG rows each), 32 registers as well.
template <class T>
struct Window<T, true> {
    static constexpr int FW = T::NLD % 8 == 0 ? 8 : T::NLD % 5 == 0 ? 5 : T::NLD % 4 == 0 ? 4 : T::NLD % 3 == 0 ? 3 : 1;
    uint4 a[FW];
};
// One wavefront load of the row-shaped layout: the rows first .. first + RG - 1 (a lane's own: first + rg).  d_v is a
// multiple of RG, so a load lies wholly inside the head or wholly behind it; behind it nothing is read or written.
template <class T>
__device__ __forceinline__ bool rows_inside(int first) { return !T::RAGV || first < T::DV; }
template <class T>
__device__ __forceinline__ RawRow<T::BITS> load_rows(const uint8_t* lane_base, int first) {
    if (!rows_inside<T>(first)) return zero_row<T::BITS>();
    return stream_row<T::BITS>(lane_base + first * T::ROW_BYTES);
}
template <class T>
__device__ __forceinline__ void store_rows(uint8_t* lane_base, int first, const RawRow<T::BITS>& r) {
    if (rows_inside<T>(first)) store_row<T::BITS>(lane_base + first * T::ROW_BYTES, r);
}
template <class T>
__device__ __forceinline__ void window_load(const uint8_t* lane_base, int rb, Window<T>& w) {
#pragma unroll
    for (int j = 0; j < Window<T>::NL; ++j) w.a[rb & 1][j] = load_rows<T>(lane_base, rb * T::MR + j * T::RG);
}
template <class T>
__device__ __forceinline__ void window_init(const uint8_t* lane_base, Window<T>& w) {
    if constexpr (T::FLT) {
#pragma unroll
        for (int i = 0; i < Window<T>::FW; ++i)
            w.a[i] = *reinterpret_cast<const uint4*>(lane_base + i * T::SRG * T::ROW_BYTES);
    } else {
        window_load<T>(lane_base, 0, w);
        if constexpr (T::NRB > 1) window_load<T>(lane_base, 1, w);
    }
}

// A lane's SPL state columns of a float-state row piece as fp32.
template <int BITS>
__device__ __forceinline__ void float_piece(const uint4& r, float (&s)[128 / BITS]) {
    if constexpr (BITS == 16) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            s[2 * d] = as_f32(w[d] << 16);
            s[2 * d + 1] = as_f32(w[d] & 0xFFFF0000u);
        }
    } else {
        s[0] = as_f32(r.x); s[1] = as_f32(r.y); s[2] = as_f32(r.z); s[3] = as_f32(r.w);
    }
}
// A lane's SPL columns of a d_k vector kept piecewise in LDS (kpos layout); zeros in idle lanes.
template <class T>
__device__ __forceinline__ void float_cols(const float* vec, int scg, float (&x)[T::SPL]) {
    const float4* p4 = reinterpret_cast<const float4*>(vec + kpos<T>((scg < T::SLPR ? scg : 0) * T::SPL));
#pragma unroll
    for (int t = 0; t < T::SPL / 4; ++t) {
        const float4 f = p4[t];
        const bool in = scg < T::SLPR;
        x[4 * t] = in ? f.x : 0.0f; x[4 * t + 1] = in ? f.y : 0.0f;
        x[4 * t + 2] = in ? f.z : 0.0f; x[4 * t + 3] = in ? f.w : 0.0f;
    }
}

// The pass over a float state: plain fp32 products on the vector ALU (a row piece decodes with a shift or not at all,
// so there is nothing for the matrix core to save), each row reduced over its SLPRP lanes.
template <class T, int NV>
__device__ __forceinline__ void float_pass(const uint8_t* lane_base, Window<T>& w, uint8_t* lds_b, float* lds_own,
                                           const LaneId& l, const float (&xe)[NV][T::NE], float (&own)[NV][T::NOWN]) {
    constexpr int FW = Window<T>::FW;
    static_assert(T::NLD % FW == 0, "whole windows");
    const int scg = l.lane % T::SLPRP, srg = l.lane / T::SLPRP;
    float* xf = reinterpret_cast<float*>(lds_b);
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const int e = l.lane + WAVE * t;
            if (e < T::LPRP * CPL) xf[v * T::KROW + kpos<T>(e)] = xe[v][t];
        }
    wave_sync();
    float xc[NV][T::SPL];
#pragma unroll
    for (int v = 0; v < NV; ++v) float_cols<T>(xf + v * T::KROW, scg, xc[v]);
#pragma unroll 1
    for (int i0 = 0; i0 < T::NLD; i0 += FW) {
#pragma unroll
        for (int j = 0; j < FW; ++j) {
            const int i = i0 + j;
            float s[T::SPL];
            float_piece<T::BITS>(w.a[j], s);
            if (i + FW < T::NLD)
                w.a[j] = *reinterpret_cast<const uint4*>(lane_base + (i + FW) * T::SRG * T::ROW_BYTES);
            const int row = i * T::SRG + srg;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                float d = s[0] * xc[v][0];
#pragma unroll
                for (int e = 1; e < T::SPL; ++e) d = __builtin_fmaf(s[e], xc[v][e], d);
                d = block_sum<(T::SLPRP < 16 ? T::SLPRP : 16)>(d);
                if constexpr (T::SLPRP >= 32) d += __shfl_xor(d, 16);
                if constexpr (T::SLPRP >= 64) d += __shfl_xor(d, 32);
                if (scg == 0) lds_own[v * T::UROW + row] = d;
            }
        }
    }
    wave_sync();
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int t = 0; t < T::NOWN; ++t)
            own[v][t] = owned_valid<T>(l, t) ? lds_own[v * T::UROW + owned_row<T>(l, t)] : 0.0f;
}

// Row sums of the whole tile against NV read-out vectors: own[v][t] = (S0 x_v)[lane + 64 t], scales applied.
// Per block of 32 rows, one matrix instruction per column step accumulates, per scale group, the (3 NV) x 32 integer
// sums (digit plane x row): the digit planes are the FIRST operand and the codes the second, so the result leaves
// row n's sums in lane n -- operand row 8 a + 4 v + b carries, for vector v, entry q = 4 a + b of the list (scale
// group g, digit d) at q = 3 g + d, and the instruction hands lane (n, kb) rows 8 a + 4 kb + b in element 4 a + b:
// lane (n, v) ends with all of row n's sums against vector v in its own registers and turns them into fp32 --
// (d0 + 2^8 d1 + 2^16 d2) 2^(e-22) is the group's dot product, times the group's scale, groups added in order (the
// reference's "(group sum) x scale, group by group", _fold_triton.py:191-196).  A plane takes part only in the column
// steps of its own scale group (zero elsewhere), so ONE accumulation over all steps keeps the groups apart.  The block
// just consumed is refilled with the block after next.  A block changes from row shape to operand shape through LDS
// (lds_a, row pitch = row + one lane piece: both the row-shaped writes and the operand-shaped reads are conflict
// free): operand lane (n = lane % 32, kb = lane / 32) takes, for column step ks, the 16 codes at row n, columns
// 32 ks + 16 kb.
// Value-axis scales: the scale belongs to (row block, column), so it goes into the read-out vector instead --
// x'_k = x_k s[rb][k] -- and the digit planes are rebuilt from `xe` (element lane + 64 t of each vector) per block;
// scale groups of half a row block take the key groups' place in the list (entry 3 h + d: the read-out against the
// scales of half h), and a row keeps its own half's.
template <class T, int NV>
__device__ __forceinline__ void state_pass(const uint8_t* lane_base, Window<T>& w, uint8_t* lds_b, float* lds_xs,
                                           const uint16_t* lds_sc, uint8_t* lds_a, float* lds_own,
                                           const LaneId& l, const float (&xe)[NV][T::NE], float (&own)[NV][T::NOWN]) {
    if constexpr (T::FLT) {
        float_pass<T, NV>(lane_base, w, lds_b, lds_own, l, xe, own);
        return;
    } else {
    constexpr int NGC = T::NG * T::VH;                       // entries of the list / 3
    // one vector and more groups than a lane's 16 elements hold (d_k 256 in groups of 32): the second half of the
    // operand rows carries groups 5 .. instead of a second vector, and lane (n, 1) continues lane (n, 0)'s sum
    constexpr bool WIDE = NV == 1 && T::PLANES * NGC > 16;
    constexpr int GPL = 5;                                   // groups per lane of a wide list
    static_assert(NV <= 2 && (WIDE ? NGC <= 2 * GPL && T::VH == 1 : T::PLANES * NGC <= 16),
                  "groups x digit planes must fit the 16 result rows of a lane (one vector: of its two lanes)");
    const int j = l.lane % T::MR, kb = l.lane / T::MR;
    // first operand: which (vector, list entry) this lane's operand row stands for
    const int rv = (j >> 2) & 1, rq = 4 * (j >> 3) + (j & 3);
    const int pgl = rq / T::PLANES, rd = rq - pgl * T::PLANES;
    const int pg = WIDE ? GPL * rv + pgl : pgl, pv = WIDE ? 0 : rv;
    const bool rlive = WIDE ? pgl < GPL && pg < NGC : rv < NV && pg < NGC;
    v4i pop[T::NKS];
    float xs[NGC];
    auto fetch_planes = [&] {
        const int slot = rlive ? (T::VH > 1 ? (pg * NV + pv) * T::PLANES + rd : T::PLANES * pv + rd) : 0;
#pragma unroll
        for (int ks = 0; ks < T::NKS; ++ks) {
            const v4i d = *reinterpret_cast<const v4i*>(lds_b + ((2 * ks + kb) * T::PSLOTS + slot) * CPL);
            const bool mine = rlive && (T::VH > 1 ? true : pg == (ks * T::MK) / T::KGROUP);
            pop[ks] = mine ? d : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int g = 0; g < NGC; ++g)
            xs[g] = T::VH > 1 ? lds_xs[g * NV + (kb < NV ? kb : 0)] : lds_xs[(kb < NV ? kb : 0) * T::NG + g];
    };
    if constexpr (!T::AXV) {
        fetch_planes();
        wave_sync();                                     // the planes' region now carries the row blocks
    }

#pragma unroll
    for (int rb = 0; rb < T::NRB; ++rb) {
        if (T::AXV && rb % T::VB == 0) {                     // a new scale group: its planes serve VB row blocks
            float xr[NV * T::VH][T::NE];                     // (half h, vector v) at h NV + v
#pragma unroll
            for (int t = 0; t < T::NE; ++t) {
                const int e = l.lane + WAVE * t;
#pragma unroll
                for (int hf = 0; hf < T::VH; ++hf) {
                    const int grp = T::VH > 1 ? rb * T::VH + hf : rb / T::VB;
                    const float s = e < T::DK ? f16_to_f32(lds_sc[grp * T::DK + (e < T::DK ? e : 0)]) : 0.0f;
#pragma unroll
                    for (int v = 0; v < NV; ++v) xr[hf * NV + v][t] = xe[v][t] * s;
                }
            }
            stage_planes<T, NV * T::VH>(xr, l, lds_b, lds_xs);
            wave_sync();
            fetch_planes();
        }
        if (l.cg < T::LPR) {
#pragma unroll
            for (int t = 0; t < Window<T>::NL; ++t)
                store_row<T::BITS>(lds_a + (t * T::RG + l.rg) * T::A_PITCH + l.cg * T::LANE_BYTES, w.a[rb & 1][t]);
        }
        if (rb + 2 < T::NRB) window_load<T>(lane_base, rb + 2, w);
        wave_sync();
        v16i acc = {0};
#pragma unroll
        for (int ks = 0; ks < T::NKS; ++ks) {
            const RawRow<T::BITS> r = load_row<T::BITS>(lds_a + j * T::A_PITCH + (2 * ks + kb) * T::LANE_BYTES);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(pop[ks], operand<T::BITS>(r), acc, 0, 0, 0);
        }
        if constexpr (WIDE) {
            const int row = rb * T::MR + j;
            float t[GPL];
#pragma unroll
            for (int g = 0; g < GPL; ++g) {
                const int gg = GPL * kb + g;                 // this lane's g-th group
                const float f = __builtin_fmaf(float(acc[3 * g + 2]), 65536.0f,
                                               __builtin_fmaf(float(acc[3 * g + 1]), 256.0f, float(acc[3 * g])));
                const float x = kb ? xs[GPL + g < NGC ? GPL + g : 0] : xs[g];
                t[g] = (f * x) * f16_to_f32(lds_sc[row * T::NG + (gg < NGC ? gg : 0)]);
            }
            float s = t[0];
#pragma unroll
            for (int g = 1; g < GPL; ++g) s = s + t[g];
            const float lo = __shfl(s, j);                   // groups 0 .. 4, from lane (n, 0)
            s = lo;
#pragma unroll
            for (int g = 0; g < GPL; ++g)
                if (GPL + g < NGC) s = s + t[g];
            if (kb == 1) lds_own[row] = s;
        } else if (kb < NV) {
            const int row = rb * T::MR + j;
            float s = 0.0f;
            if constexpr (T::VH > 1) {                       // the entries of the row's own half
                static_assert(T::VH == 2, "two halves per row block");
                const bool up = j >= T::GROUP;
                const float f = __builtin_fmaf(float(up ? acc[5] : acc[2]), 65536.0f,
                                               __builtin_fmaf(float(up ? acc[4] : acc[1]), 256.0f,
                                                              float(up ? acc[3] : acc[0])));
                s = f * (up ? xs[T::VH - 1] : xs[0]);
            } else {
#pragma unroll
                for (int g = 0; g < T::NG; ++g) {
                    const float f = __builtin_fmaf(float(acc[3 * g + 2]), 65536.0f,
                                                   __builtin_fmaf(float(acc[3 * g + 1]), 256.0f, float(acc[3 * g])));
                    const float term = T::AXV ? f * xs[g] : (f * xs[g]) * f16_to_f32(lds_sc[row * T::NG + g]);
                    s = g == 0 ? term : s + term;
                }
            }
            lds_own[kb * T::UROW + row] = s;
        }
        wave_sync();                                     // every lane has its codes: the next block may take their place
    }
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int t = 0; t < T::NOWN; ++t)
            own[v][t] = owned_valid<T>(l, t) ? lds_own[v * T::UROW + owned_row<T>(l, t)] : 0.0f;
    }
}

// A lane's 16-column piece of a d_k vector kept piecewise in LDS.
template <class T>
__device__ __forceinline__ void lds_piece(const float* vec, int cg, float (&x)[CPL]) {
    const float4* p4 = reinterpret_cast<const float4*>(vec + cg * T::KPAD);
#pragma unroll
    for (int t = 0; t < CPL / 4; ++t) {
        const float4 f = p4[t];
        x[4 * t] = f.x; x[4 * t + 1] = f.y; x[4 * t + 2] = f.z; x[4 * t + 3] = f.w;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// the decode buffer.  Loads are unconditional (indices clamped into the live range) so that they can be issued back
// to back ahead of the state tile; dead slots and idle lanes are masked after the fact with selects.
// ---------------------------------------------------------------------------------------------------------------
template <class T>
struct BufAddr {                       // one (sequence, head)'s buffer fields
    uint8_t* KB;                       // [m][DK] int8 or bf16, of the head's KEY head
    uint8_t* UB;                       // [m][DV] int8 or bf16
    uint16_t* KBS;                     // [m] fp16 (int8 buffer)
    uint16_t* UBS;                     // [m] fp16 (int8 buffer)
};

// Buffered value (slot i, head row r) from the raw copy in LDS.
template <class T>
__device__ __forceinline__ float ub_lds(const uint8_t* ub_lds_, int i, int r) {
    if constexpr (T::QBUF) return float(reinterpret_cast<const int8_t*>(ub_lds_)[i * T::DV + r]);
    else return bf16_to_f32(reinterpret_cast<const uint16_t*>(ub_lds_)[i * T::DV + r]);
}

// A lane's 16-column piece of one buffered key, raw.
template <bool QBUF> struct KPiece;
template <> struct KPiece<true> { uint4 a; };
template <> struct KPiece<false> { uint4 a, b; };

template <class T>
__device__ __forceinline__ KPiece<T::QBUF> load_kpiece(const uint8_t* KB, int slot, int m, const LaneId& l) {
    const int ic = slot < m ? slot : m - 1;
    const int cc = l.cg < T::LPR ? l.cg : T::LPR - 1;
    KPiece<T::QBUF> k;
    if constexpr (T::QBUF) {
        k.a = *reinterpret_cast<const uint4*>(KB + ic * T::DK + cc * CPL);
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(KB + (ic * T::DK + cc * CPL) * 2);
        k.a = p[0];
        k.b = p[1];
    }
    return k;
}
// -> fp32, times the slot's scale for an int8 buffer; zeros in idle lanes.
template <class T>
__device__ __forceinline__ void decode_kpiece(const KPiece<T::QBUF>& k, float scale, const LaneId& l,
                                              float (&kb)[CPL]) {
    if constexpr (T::QBUF) {
        RawRow<8> r;
        r.v = k.a;
        decode_row<8>(r, kb);
#pragma unroll
        for (int c = 0; c < CPL; ++c) kb[c] = kb[c] * scale;
    } else {
        const uint32_t w[8] = {k.a.x, k.a.y, k.a.z, k.a.w, k.b.x, k.b.y, k.b.z, k.b.w};
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            kb[2 * c] = as_f32(w[c] << 16);
            kb[2 * c + 1] = as_f32(w[c] & 0xFFFF0000u);
        }
    }
    if (l.cg >= T::LPR) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) kb[c] = 0.0f;
    }
}
template <class T>
__device__ __forceinline__ void stage_kpiece(float* lds_k, int slot, const LaneId& l, const float (&kb)[CPL]) {
    float4* d4 = reinterpret_cast<float4*>(lds_k + slot * T::KROW + l.cg * T::KPAD);
#pragma unroll
    for (int c = 0; c < CPL / 4; ++c) d4[c] = make_float4(kb[4 * c], kb[4 * c + 1], kb[4 * c + 2], kb[4 * c + 3]);
}

// Passes over the key buffer seen as a small tile: slot = row group + RG x pass.
template <class T>
struct KeyBuf {
    static constexpr int KT = (T::MMAX + T::RG - 1) / T::RG;
    KPiece<T::QBUF> piece[KT];
    uint16_t kbs[KT];                  // raw fp16 scale of the lane's slot (int8 buffer)
};
template <class T>
__device__ __forceinline__ void load_keybuf(const BufAddr<T>& a, int m, const LaneId& l, KeyBuf<T>& kb) {
#pragma unroll
    for (int t = 0; t < KeyBuf<T>::KT; ++t) {
        const int i = l.rg + T::RG * t;
        kb.piece[t] = load_kpiece<T>(a.KB, i, m, l);
        if constexpr (T::QBUF) kb.kbs[t] = a.KBS[i < m ? i : m - 1];
        else kb.kbs[t] = 0;
    }
}

// Buffer coefficients for scalar decays (GDN, Mamba2): c[v][i] = exp(gcur - G_i) (K_i . x_v) for slots i < n, else 0
// (reference `_coefs`, _fold_triton.py:260-272).  `gb` = the lane's slots' G (one per pass).
template <class T, int NV>
__device__ __forceinline__ void buffer_coefs(const KeyBuf<T>& kbuf, const float (&gb)[KeyBuf<T>::KT], float gcur,
                                             int n, const float (&x)[NV][CPL], const LaneId& l,
                                             float (&c)[NV][T::MMAX]) {
    constexpr int KT = KeyBuf<T>::KT;
    float cl[NV][KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
        const int i = l.rg + T::RG * t;
        float kb[CPL];
        decode_kpiece<T>(kbuf.piece[t], f16_to_f32(kbuf.kbs[t]), l, kb);
        const float dec = expf(gcur - gb[t]);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            float p = kb[0] * x[v][0];
#pragma unroll
            for (int k = 1; k < CPL; ++k) p = __builtin_fmaf(kb[k], x[v][k], p);
            p = block_sum<T::LPRP>(p);
            cl[v][t] = i < n ? dec * p : 0.0f;               // dead slots may hold anything: select, never multiply
        }
    }
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) c[v][i] = lane_bcast(cl[v][i / T::RG], (i % T::RG) * T::LPRP);
}

// Buffer term of one owned row r: acc[v] += sum_i U_i[r] c[v][i] as an fma chain in slot order (the reference's
// `_acc`, _fold_triton.py:239-257).  c[v][i] is zero for dead slots (i >= n).  int8 buffer: the slot's scale is folded
// into the coefficient once per tile (wave-uniform; zero for a dead slot, whose scale may be anything), so a slot
// costs one conversion and one fma per vector; dead slots hold finite bytes, times zero.  bf16 buffer: dead slots may
// hold NaNs, so their values are discarded first.
template <class T, int NV>
__device__ __forceinline__ void buffer_term(const uint8_t* lds_ub, const float (&ubs)[T::MMAX],
                                            const float (&c)[NV][T::MMAX], int n, int m, int r, float (&acc)[NV]) {
#pragma unroll
    for (int i = 0; i < T::MMAX; ++i) {
        if (i < n) {                                     // wave-uniform: a dead slot would add exactly zero
            const float uv = ub_lds<T>(lds_ub, i, r);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const float cu = !T::QBUF ? c[v][i] : c[v][i] * ubs[i];
                acc[v] = __builtin_fmaf(uv, cu, acc[v]);
            }
        }
    }
}

// Append the current token's value row: int8 with one absmax scale over the whole row (`us`, stored by lane 0), or
// bf16.  ur = the value as stored, dequantized (what the fold must use for slot n).
template <class T>
__device__ __forceinline__ void append_values(const float (&u)[T::NOWN], float us, const BufAddr<T>& a, int n,
                                              const LaneId& l, float (&ur)[T::NOWN]) {
    if (T::QBUF && l.lane == 0) a.UBS[n] = f32_to_f16(us);
#pragma unroll
    for (int b = 0; b < T::NOWN; ++b) {
        const int r = owned_row<T>(l, b);
        const bool valid = owned_valid<T>(l, b);
        if constexpr (T::QBUF) {
            const float c = round_buf(u[b], us);
            ur[b] = c * us;
            if (valid) reinterpret_cast<int8_t*>(a.UB)[n * T::DV + r] = int8_t(int(c));
        } else {
            const uint16_t hb = f32_to_bf16(u[b]);
            ur[b] = bf16_to_f32(hb);
            if (valid) reinterpret_cast<uint16_t*>(a.UB)[n * T::DV + r] = hb;
        }
    }
}
// Append the current token's key (element e = lane + 64 t of it sits in kx[t]); `write` = this head stores it.
template <class T>
__device__ __forceinline__ void append_key(const float (&kx)[T::NE], float ks, const BufAddr<T>& a, int n, bool write,
                                           const LaneId& l, float (&kr)[T::NE]) {
    if (T::QBUF && write && l.lane == 0) a.KBS[n] = f32_to_f16(ks);
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        if constexpr (T::QBUF) {
            const float c = round_buf(kx[t], ks);
            kr[t] = c * ks;
            if (write && e < T::DK) reinterpret_cast<int8_t*>(a.KB)[n * T::DK + e] = int8_t(int(c));
        } else {
            const uint16_t hb = f32_to_bf16(kx[t]);
            kr[t] = bf16_to_f32(hb);
            if (write && e < T::DK) reinterpret_cast<uint16_t*>(a.KB)[n * T::DK + e] = hb;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// the fold
// ---------------------------------------------------------------------------------------------------------------

// Fold operands, step 1 (before the front end's LDS is overwritten): the buffered values of the rows this lane owns,
// dequantized, slot by slot.  uo[b][i] = U_i[row b] (slot m-1: the value just appended, `ur`).
template <class T>
__device__ __forceinline__ void fold_fetch_values(const uint8_t* ub_lds_, const float (&ubs)[T::MMAX],
                                                  const float (&ur)[T::NOWN], int m, const LaneId& l,
                                                  float (&uo)[T::NOWN][T::MMAX]) {
#pragma unroll
    for (int b = 0; b < T::NOWN; ++b) {
        int r = owned_row<T>(l, b);
        r = r < T::DV ? r : T::DV - 1;
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            float uv = ub_lds<T>(ub_lds_, i < m ? i : m - 1, r);
            if constexpr (T::QBUF) uv = uv * ubs[i];
            uo[b][i] = i == m - 1 ? ur[b] : uv;
        }
    }
}
// Step 2: lds_u[i][row] = f[i] x U_i[row] (f = the slot's decay ratio; KDA passes ones).
template <class T>
__device__ __forceinline__ void fold_stage_values(const float (&uo)[T::NOWN][T::MMAX], const float (&f)[T::MMAX],
                                                  int m, const LaneId& l, float* lds_u) {
#pragma unroll
    for (int b = 0; b < T::NOWN; ++b) {
        const int r = owned_row<T>(l, b);
        const bool valid = owned_valid<T>(l, b);
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i)
            if (i < m) lds_u[i * T::UROW + r] = valid ? f[i] * uo[b][i] : 0.0f;
    }
}
template <class T>
__device__ __forceinline__ void fold_stage_key(const float (&kr)[T::NE], int slot, const LaneId& l, float* lds_k) {
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        if (e < T::LPRP * CPL) lds_k[slot * T::KROW + kpos<T>(e)] = e < T::DK ? kr[t] : 0.0f;
    }
}

// The fold proper: S = colmul * S_0 + sum_i du_i (x) kx_i over all m buffer slots in slot order, re-quantized in place
// (reference: _fused_triton.py:278-394 `_fold_head`; KDA _kda_triton.py:217-316; Mamba2 _mamba2_triton.py:213-332).
//   lds_k   [m][KROW]   the folded keys kx_i (GDN / Mamba2: the buffered keys; KDA: keys times their decay ratio)
//   lds_u   [m][UROW]   the folded values du_i (GDN / Mamba2: decay ratio x delta value; KDA: delta value)
//   lds_c   [KROW]      COLVEC: per-column factors on the dequantized old state (KDA);  else the scalar `cmul`
//                       (GDN / Mamba2: exp(G_m))
// The m rank-1 updates run on the matrix core in fp32 (v_mfma_f32_32x32x2_f32: two slots per issue, accumulating on
// the dequantized old state, slot pairs in order), one 32-row x 32-column block of the state at a time.  The block is
// held "rows across lanes": lane (j = lane % 32, kb = lane / 32) owns row j's columns 16 kb .. 16 kb + 15 of the
// block -- accumulator element 4a + b is output row 8a + 4 kb + b of the instruction, and the keys are fed with
// operand row i = 8a + 4 kb' + b carrying column 16 kb' + 4a + b, so element e of a lane IS column e of its piece.
// That is the operand shape of the state pass: the codes are read again from memory row-shaped (coalesced), turned
// into that shape through LDS (the region of lds_k, free once the keys sit in registers), and the new codes go back
// the same way.  A row's scale group lies in one lane pair (j, 0), (j, 1): absmax = per-lane max + one exchange.
// Codes are rint(S x (1/scale)) with the correctly rounded reciprocal: against rint(S / scale) that moves a code by
// one step only where the quotient lies within |q| 2^-24 of a rounding boundary (a few codes per million, the same
// order as the accumulation-order mismatches).
typedef float v16f __attribute__((ext_vector_type(16)));

// The fold of a float state: S = c S0 + sum_i (decayed u_i) k_i^T in slot order on the vector ALU, rounded to the
// state's type and stored in place (_fused_triton.py:376-382: no scales, no absmax).  A lane keeps its SPL columns of
// all m keys in registers; the values come from LDS (one broadcast read per row and slot).
template <class T, bool COLVEC>
__device__ __forceinline__ void float_fold(const float* lds_k, const float* lds_u, const float* lds_c, float cmul,
                                           int m, uint8_t* head, const LaneId& l) {
    constexpr int FW = 4;
    static_assert(T::NLD % FW == 0, "whole windows");
    const int scg = l.lane % T::SLPRP, srg = l.lane / T::SLPRP;
    const bool live = scg < T::SLPR;
    float kk[T::MMAX][T::SPL], cm[T::SPL];
#pragma unroll
    for (int i = 0; i < T::MMAX; ++i) {
        float_cols<T>(lds_k + (i < m ? i : 0) * T::KROW, scg, kk[i]);
        if (i >= m) {
#pragma unroll
            for (int e = 0; e < T::SPL; ++e) kk[i][e] = 0.0f;
        }
    }
    if constexpr (COLVEC) float_cols<T>(lds_c, scg, cm);
    uint8_t* lane_base = const_cast<uint8_t*>(lane_codes<T>(head, l));
    uint4 w[FW];
#pragma unroll
    for (int j = 0; j < FW; ++j) w[j] = *reinterpret_cast<const uint4*>(lane_base + j * T::SRG * T::ROW_BYTES);
#pragma unroll 1
    for (int i0 = 0; i0 < T::NLD; i0 += FW) {
#pragma unroll
        for (int j = 0; j < FW; ++j) {
            const int i = i0 + j;
            float acc[T::SPL];
            float_piece<T::BITS>(w[j], acc);
            if (i + FW < T::NLD) w[j] = *reinterpret_cast<const uint4*>(lane_base + (i + FW) * T::SRG * T::ROW_BYTES);
#pragma unroll
            for (int e = 0; e < T::SPL; ++e) acc[e] = acc[e] * (COLVEC ? cm[e] : cmul);
            const int row = i * T::SRG + srg;
#pragma unroll
            for (int t = 0; t < T::MMAX; ++t) {
                const float uv = lds_u[(t < m ? t : 0) * T::UROW + row];
#pragma unroll
                for (int e = 0; e < T::SPL; ++e) acc[e] = __builtin_fmaf(uv, kk[t][e], acc[e]);   // dead slots: k = 0
            }
            uint4 o;
            if constexpr (T::BITS == 16) {
                uint32_t q[4];
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    q[d] = uint32_t(f32_to_bf16(acc[2 * d])) | (uint32_t(f32_to_bf16(acc[2 * d + 1])) << 16);
                o = make_uint4(q[0], q[1], q[2], q[3]);
            } else {
                o = make_uint4(as_u32(acc[0]), as_u32(acc[1]), as_u32(acc[2]), as_u32(acc[3]));
            }
            if (live) *reinterpret_cast<uint4*>(lane_base + i * T::SRG * T::ROW_BYTES) = o;
        }
    }
}

template <class T, bool COLVEC>
__device__ __forceinline__ void fold_tile(float* lds_k, const float* lds_u, const float* lds_c, float cmul, int m,
                                          uint8_t* head, uint16_t* sc_head, const LaneId& l) {
    if constexpr (T::FLT) {
        float_fold<T, COLVEC>(lds_k, lds_u, lds_c, cmul, m, head, l);
        return;
    } else {
    constexpr int NCS = T::NKS;                              // 32-column steps
    constexpr int MT = (T::MMAX + 1) / 2;                    // slot pairs
    constexpr int NL = Window<T>::NL;
    const int j = l.lane % T::MR, kb = l.lane / T::MR;
    const bool live = l.cg < T::LPR;

    // keys as matrix operands, for the whole tile:
    // aop[cs][t] = kx_{2t + kb}[32 cs + 16 ((j >> 2) & 1) + 4 (j >> 3) + (j & 3)]
    float aop[NCS][MT];
    {
        const int col = 16 * ((j >> 2) & 1) + 4 * (j >> 3) + (j & 3);
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs)
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int slot = 2 * t + kb;
                const float v = lds_k[(slot < m ? slot : 0) * T::KROW + kpos<T>(32 * cs + col)];
                aop[cs][t] = slot < m ? v : 0.0f;
            }
    }
    wave_sync();                                         // lds_k becomes the block buffer
    uint8_t* blk = reinterpret_cast<uint8_t*>(lds_k);
    uint8_t* lane_base = const_cast<uint8_t*>(lane_codes<T>(head, l));

    RawRow<T::BITS> nxt[NL];                                 // the next row block and its scales, a block ahead
    uint16_t scn[T::NG];
#pragma unroll
    for (int t = 0; t < NL; ++t) nxt[t] = load_rows<T>(lane_base, t * T::RG);
#pragma unroll
    for (int g = 0; g < T::NG; ++g) scn[g] = sc_head[j * T::NG + g];

#pragma unroll 1
    for (int rb = 0; rb < T::NRB; ++rb) {
        const int row = rb * T::MR + j;
        uint16_t scr[T::NG];
#pragma unroll
        for (int g = 0; g < T::NG; ++g) scr[g] = scn[g];
        // an old scale at its floor (stored fp16 bits 0 or 1: an empty group) or a decay of exactly 1: what is
        // quantized is a sum of a few low-precision products with exact half-integer quotients by the thousand --
        // there the codes are rint of the IEEE quotient (quantize_row<.., EXACT>).  Decided here, while the old
        // scales are in registers anyway.
        bool cold = !COLVEC && cmul == 1.0f;
#pragma unroll
        for (int g = 0; g < T::NG; ++g) cold = cold || scr[g] <= 1;
        const bool exact = __builtin_amdgcn_ballot_w64(cold) != 0;
        if (live) {
#pragma unroll
            for (int t = 0; t < NL; ++t)
                store_row<T::BITS>(blk + (t * T::RG + l.rg) * T::A_PITCH + l.cg * T::LANE_BYTES, nxt[t]);
        }
        if (rb + 1 < T::NRB) {
#pragma unroll
            for (int t = 0; t < NL; ++t) nxt[t] = load_rows<T>(lane_base, (rb + 1) * T::MR + t * T::RG);
            const int rown = !T::RAGV || row + T::MR < T::DV ? row + T::MR : T::DV - 1;     // rows behind d_v: unused
#pragma unroll
            for (int g = 0; g < T::NG; ++g) scn[g] = sc_head[rown * T::NG + g];
        }
        float bop[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int slot = 2 * t + kb;
            const float v = lds_u[(slot < m ? slot : 0) * T::UROW + row];
            bop[t] = slot < m ? v : 0.0f;
        }
        wave_sync();

        v16f acc[NCS];
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs) {
            const int piece = 2 * cs + kb;
            const RawRow<T::BITS> r = load_row<T::BITS>(blk + j * T::A_PITCH + piece * T::LANE_BYTES);
            float c[CPL];
            decode_row_scaled<T::BITS>(r, c);
            const float s = f16_to_f32(scr[(piece * CPL) / T::GROUP]) * DECODE_UNIT<T::BITS>;     // exact
            if constexpr (COLVEC) {
                float cm[CPL];
                lds_piece<T>(lds_c, piece, cm);
#pragma unroll
                for (int e = 0; e < CPL; ++e) acc[cs][e] = (c[e] * s) * cm[e];
            } else {
                const float sm = s * cmul;                   // one rounding more than (code x scale) x decay
#pragma unroll
                for (int e = 0; e < CPL; ++e) acc[cs][e] = c[e] * sm;
            }
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[cs] = __builtin_amdgcn_mfma_f32_32x32x2f32(aop[cs][t], bop[t], acc[cs], 0, 0, 0);
        }

        // absmax per scale group: the lane's pieces, then the other half of the row
        float gmax[T::NG];
#pragma unroll
        for (int g = 0; g < T::NG; ++g) gmax[g] = 0.0f;
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs) {
            float mx = 0.0f;
#pragma unroll
            for (int e = 0; e < CPL; ++e) mx = fmaxf(mx, fabsf(acc[cs][e]));
            const int g = (cs * T::MK) / T::GROUP;
            gmax[g] = fmaxf(gmax[g], mx);
        }
        float rs[T::NG];
#pragma unroll
        for (int g = 0; g < T::NG; ++g) {
            const float other = __shfl_xor(gmax[g], 32);
            const float sc = fp16_scale(fmaxf(gmax[g], other), T::QMAX);
            rs[g] = scale_divisor(sc).rc;
            if (kb == 0 && (!T::RAGV || row < T::DV)) sc_head[row * T::NG + g] = f32_to_f16(sc);
        }
        auto requantize = [&](auto exactly) {                // two code paths, not a select between two results
#pragma unroll
            for (int cs = 0; cs < NCS; ++cs) {
                float a16[CPL];
#pragma unroll
                for (int e = 0; e < CPL; ++e) a16[e] = acc[cs][e];
                const int g = (cs * T::MK) / T::GROUP;
                const float d = decltype(exactly)::value ? divisor_of(rs[g]) : 0.0f;
                store_row<T::BITS>(blk + j * T::A_PITCH + (2 * cs + kb) * T::LANE_BYTES,
                                   quantize_row<T::BITS, true, decltype(exactly)::value>(a16, rs[g], d));
            }
        };
        if (exact) requantize(std::true_type{});
        else requantize(std::false_type{});
        wave_sync();
        if (live) {
#pragma unroll
            for (int t = 0; t < NL; ++t)
                store_rows<T>(lane_base, rb * T::MR + t * T::RG,
                              load_row<T::BITS>(blk + (t * T::RG + l.rg) * T::A_PITCH + l.cg * T::LANE_BYTES));
        }
        wave_sync();
    }
}
}

// The fold for value-axis scale groups: one scale per (group of 32 or 64 rows, key column); a 32-row block is held "columns
// across lanes" -- lane (j = lane % 32, kb = lane / 32) owns column j of a 32-column step and, in accumulator element
// 4a + b, row 8a + 4 kb + b -- and a column's absmax is again a per-lane maximum plus one lane exchange.  The rank-1
// updates run as above with the operands' roles swapped (values feed the rows, keys the columns).  The codes arrive in
// that shape through the matrix core as well: the row block in operand shape times a 32 x 32 identity
// (v_mfma_i32_32x32x32_i8) is the block itself, one int32 per code, laid out exactly like the accumulators.  The new
// codes go back to the row-major LDS block byte by byte (int4: even / odd columns paired across neighbouring lanes).
template <class T, bool COLVEC>
__device__ __forceinline__ void fold_tile_v(float* lds_k, const float* lds_u, const float* lds_c, float cmul, int m,
                                            uint8_t* head, uint16_t* sc_head, const LaneId& l) {
    constexpr int NCS = T::NKS;
    constexpr int MT = (T::MMAX + 1) / 2;
    constexpr int NL = Window<T>::NL;
    constexpr float MAGIC = 12582912.0f + (T::BITS == 4 ? 8.0f : 0.0f);
    const int j = l.lane % T::MR, kb = l.lane / T::MR;
    const bool live = l.cg < T::LPR;

    float kop[NCS][MT], cm[NCS];
#pragma unroll
    for (int cs = 0; cs < NCS; ++cs) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int slot = 2 * t + kb;
            const float v = lds_k[(slot < m ? slot : 0) * T::KROW + kpos<T>(32 * cs + j)];
            kop[cs][t] = slot < m ? v : 0.0f;
        }
        cm[cs] = COLVEC ? lds_c[kpos<T>(32 * cs + j)] : cmul;
    }
    // lane (n, kb) of the identity: byte t is 1 where operand position (kb, t) carries column n
    v4i ident = {0, 0, 0, 0};
    {
        const int t = operand_pos<T::BITS>(j % CPL);
        const int one = (j / CPL == kb) ? (1 << (8 * (t % 4))) : 0;
        ident[0] = t / 4 == 0 ? one : 0;
        ident[1] = t / 4 == 1 ? one : 0;
        ident[2] = t / 4 == 2 ? one : 0;
        ident[3] = t / 4 == 3 ? one : 0;
    }
    wave_sync();                                         // lds_k becomes the block buffer
    uint8_t* blk = reinterpret_cast<uint8_t*>(lds_k);
    uint8_t* lane_base = const_cast<uint8_t*>(lane_codes<T>(head, l));

    // groups of half a row block (VH = 2): accumulator elements 0..7 (rows 8a + 4 kb + b, a < 2) belong to the first
    // 16 rows of the block, elements 8..15 to the second; each half has its own scale per column
    constexpr int VH = T::VH;
    RawRow<T::BITS> nxt[NL];
    uint16_t scn[NCS][VH];
#pragma unroll
    for (int t = 0; t < NL; ++t) nxt[t] = load_rows<T>(lane_base, t * T::RG);
#pragma unroll
    for (int cs = 0; cs < NCS; ++cs)
#pragma unroll
        for (int hf = 0; hf < VH; ++hf) scn[cs][hf] = sc_head[hf * T::DK + 32 * cs + j];
    constexpr int NGRP = T::DV / T::GROUP;                   // scale groups of the head (a ragged last block has fewer)

    // A scale group of two row blocks (VB = 2) is visited twice: first for the column maxima over its 64 rows, then
    // -- the folded values computed again from the still untouched codes -- for the codes.  Visit v: group
    // v / (VB PH), phase (v / VB) % PH, block v % VB of the group.
    constexpr int VB = T::VB, PH = VB > 1 ? 2 : 1, VISITS = T::NRB * PH;
    auto block_of = [](int v) { return (v / (VB * PH)) * VB + v % VB; };
    float gmx[NCS];
#pragma unroll 1
    for (int v = 0; v < VISITS; ++v) {
        const int rb = block_of(v), grp = rb / VB;
        const bool last_phase = (v / VB) % PH == PH - 1;
        uint16_t scr[NCS][VH];
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs)
#pragma unroll
            for (int hf = 0; hf < VH; ++hf) scr[cs][hf] = scn[cs][hf];
        bool cold = !COLVEC && cmul == 1.0f;     // as in the key-axis fold: exact quotients where the old state is empty
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs)
#pragma unroll
            for (int hf = 0; hf < VH; ++hf) cold = cold || scr[cs][hf] <= 1;
        const bool exact = __builtin_amdgcn_ballot_w64(cold) != 0;
        if (live) {
#pragma unroll
            for (int t = 0; t < NL; ++t)
                store_row<T::BITS>(blk + (t * T::RG + l.rg) * T::A_PITCH + l.cg * T::LANE_BYTES, nxt[t]);
        }
        if (v + 1 < VISITS) {
            const int rn = block_of(v + 1);
#pragma unroll
            for (int t = 0; t < NL; ++t) nxt[t] = load_rows<T>(lane_base, rn * T::MR + t * T::RG);
#pragma unroll
            for (int cs = 0; cs < NCS; ++cs)
#pragma unroll
                for (int hf = 0; hf < VH; ++hf) {
                    const int gi = (rn / VB) * VH + hf;
                    scn[cs][hf] = sc_head[(gi < NGRP ? gi : NGRP - 1) * T::DK + 32 * cs + j];
                }
        }
        float dop[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int slot = 2 * t + kb;
            const float v = lds_u[(slot < m ? slot : 0) * T::UROW + rb * T::MR + j];
            dop[t] = slot < m ? v : 0.0f;
        }
        wave_sync();

        v16f acc[NCS];
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs) {
            const RawRow<T::BITS> r = load_row<T::BITS>(blk + j * T::A_PITCH + (2 * cs + kb) * T::LANE_BYTES);
            const v16i ci = __builtin_amdgcn_mfma_i32_32x32x32_i8(operand<T::BITS>(r), ident, v16i{0}, 0, 0, 0);
            float s[VH];
#pragma unroll
            for (int hf = 0; hf < VH; ++hf)
                s[hf] = f16_to_f32(scr[cs][hf]) * DECODE_UNIT<T::BITS>;          // exact (int4 operands are 16 x code)
#pragma unroll
            for (int e = 0; e < CPL; ++e) {
                const float se = s[VH > 1 ? e / 8 : 0];
                acc[cs][e] = COLVEC ? (float(ci[e]) * se) * cm[cs] : float(ci[e]) * (se * cm[cs]);
            }
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[cs] = __builtin_amdgcn_mfma_f32_32x32x2f32(dop[t], kop[cs][t], acc[cs], 0, 0, 0);
        }
        float rs[NCS][VH];
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs) {
#pragma unroll
            for (int hf = 0; hf < VH; ++hf) {
                float mx = 0.0f;
#pragma unroll
                for (int e = hf * (CPL / VH); e < (hf + 1) * (CPL / VH); ++e) mx = fmaxf(mx, fabsf(acc[cs][e]));
                mx = fmaxf(mx, __shfl_xor(mx, 32));
                if constexpr (VB > 1) {
                    if (!last_phase) gmx[cs] = v % VB == 0 ? mx : fmaxf(gmx[cs], mx);
                    mx = gmx[cs];
                }
                const float sc = fp16_scale(mx, T::QMAX);
                rs[cs][hf] = scale_divisor(sc).rc;
                // the group's last block writes the scale: the earlier ones' codes were decoded with the old one by then
                if (kb == 0 && last_phase && v % VB == VB - 1 && grp * VH + hf < NGRP)
                    sc_head[(grp * VH + hf) * T::DK + 32 * cs + j] = f32_to_f16(sc);
            }
        }
        wave_sync();                                     // every lane has its codes: the block takes the new ones
        if (!last_phase) continue;
        auto requantize = [&](auto exactly) {                // two code paths, not a select between two results
#pragma unroll
        for (int cs = 0; cs < NCS; ++cs) {
#pragma unroll
            for (int e = 0; e < CPL; ++e) {
                const int hs = VH > 1 ? e / 8 : 0;
                float f;
                if constexpr (decltype(exactly)::value) {
                    float d = divisor_of(rs[cs][hs]);        // anew for every element: the rare path must not hold
                    asm volatile("" : "+v"(d));              // a second table of divisors in registers
                    f = div_rc(acc[cs][e], d, rs[cs][hs]) + MAGIC;
                } else {
                    f = __builtin_fmaf(acc[cs][e], rs[cs][hs], MAGIC);
                }
                const uint32_t u = as_u32(__builtin_amdgcn_fmed3f(f, MAGIC - T::QMAX, MAGIC + T::QMAX));
                const int row = 8 * (e / 4) + 4 * kb + (e % 4);
                if constexpr (T::BITS == 8) {
                    blk[row * T::A_PITCH + 32 * cs + j] = uint8_t(u);
                } else {
                    const uint32_t nib = u & 0xFu;                       // code + 8
                    const uint32_t other = as_u32(partner<0>(as_f32(nib)));
                    if ((j & 1) == 0) blk[row * T::A_PITCH + (32 * cs + j) / 2] = uint8_t(nib | (other << 4));
                }
            }
        }
        };
        if (exact) requantize(std::true_type{});
        else requantize(std::false_type{});
        wave_sync();
        if (live) {
#pragma unroll
            for (int t = 0; t < NL; ++t)
                store_rows<T>(lane_base, rb * T::MR + t * T::RG,
                              load_row<T::BITS>(blk + (t * T::RG + l.rg) * T::A_PITCH + l.cg * T::LANE_BYTES));
        }
        wave_sync();
    }
}

}  // namespace sq
