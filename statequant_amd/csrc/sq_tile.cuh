// The state tile of one (sequence, value head) in one wavefront: geometry, the single read of the stored codes, the
// row dot products with cross-lane reduction, and the fold (advance across the full buffer + re-quantize in place).
// Shared by the Gated DeltaNet, KDA and Mamba2 step kernels.
#pragma once
#include "sq_device.cuh"

namespace sq {

// Compile-time geometry.  A row of DK codes is cut into DK/16 pieces of 16 columns; LPRP (that count rounded up to a
// power of two) consecutive lanes hold one row, lanes past DK/16 idle (d_k = 96: 6 of 8).  The wavefront therefore
// covers RG = 64/LPRP rows per load and a lane sees rows rg, rg + RG, rg + 2 RG, ...
template <int BITS_, int DK_, int DV_, int GROUP_, bool QBUF_, int MMAX_>
struct Tile {
    static constexpr int BITS = BITS_, DK = DK_, DV = DV_, GROUP = GROUP_, MMAX = MMAX_;
    static constexpr bool QBUF = QBUF_;
    static_assert(BITS == 4 || BITS == 8, "stored codes are int4 or int8");
    static_assert(DK % CPL == 0 && DK >= 32 && DK <= 256, "d_k must be a multiple of 16 in 32..256");
    static constexpr int LPR = DK / CPL;                  // live lanes per row
    static constexpr int LPRP = pow2_ceil(LPR);           // lanes per row incl. idle ones
    static constexpr int RG = WAVE / LPRP;                // rows per wavefront load
    static_assert(DV % (4 * RG) == 0, "d_v must be a multiple of 4 x the rows one wavefront load covers");
    static constexpr int RPL = DV / RG;                   // rows per lane
    static constexpr int RPLP = round_up(RPL, LPRP);      // padded so the reduce-scatter divides evenly
    static constexpr int NOWN = RPLP / LPRP;              // rows a lane owns after the reduction
    static constexpr int NG = (DK + GROUP - 1) / GROUP;   // stored key groups per row (last may be ragged)
    static_assert(GROUP % CPL == 0 && GROUP >= CPL, "key group must be a multiple of 16");
    static constexpr int LPG = (GROUP / CPL < LPRP) ? GROUP / CPL : LPRP;   // lanes sharing one scale
    static constexpr int LVL_ROW = ilog2(LPRP);           // butterfly levels across a row
    static constexpr int LVL_GRP = ilog2(LPG);            // ... of which inside one scale group
    static constexpr int ROW_BYTES = BITS == 4 ? DK / 2 : DK;
    static constexpr int LANE_BYTES = BITS == 4 ? CPL / 2 : CPL;
    static constexpr float QMAX = float((1 << (BITS - 1)) - 1);
    static constexpr int NE = (DK + WAVE - 1) / WAVE;     // elements of a d_k vector per lane (element = lane + 64 t)
    static constexpr int KPAD = CPL + 4;                  // LDS stride of a 16-column piece (spreads the banks)
    static constexpr int KROW = LPRP * KPAD;              // floats per d_k vector in LDS
    static constexpr int UROW = RPLP * RG;                // floats per d_v vector in LDS
    static constexpr int LDS_FLOATS = MMAX * KROW + MMAX * UROW + 2 * KROW;
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

// Which of its RPLP rows a lane owns after reduce_rows: own_first(l) + t, t < NOWN.  Every butterfly level halves
// the candidate range; the lane whose bit is set takes the upper half.
template <class T>
__device__ __forceinline__ int own_first(const LaneId& l) {
    int off = 0, n = T::RPLP;
#pragma unroll
    for (int lv = T::LVL_ROW - 1; lv >= 0; --lv) {
        n >>= 1;
        if ((l.cg >> lv) & 1) off += n;
    }
    return off;
}

// The only read of the stored state: a lane's piece of each of its rows, issued back to back.  Idle lanes (past
// d_k) load a live lane's piece instead of branching around the load, and zero it afterwards.
template <class T>
__device__ __forceinline__ void load_tile(const uint8_t* head, const LaneId& l, RawRow<T::BITS> (&raw)[T::RPL]) {
    const int cc = l.cg < T::LPR ? l.cg : T::LPR - 1;
#pragma unroll
    for (int j = 0; j < T::RPL; ++j)
        raw[j] = load_row<T::BITS>(head + size_t(row_of<T>(l, j)) * T::ROW_BYTES + cc * T::LANE_BYTES);
}
template <class T>
__device__ __forceinline__ void mask_tile(const LaneId& l, RawRow<T::BITS> (&raw)[T::RPL]) {
    if constexpr (T::LPR < T::LPRP) {
        const bool live = l.cg < T::LPR;
        const RawRow<T::BITS> z = zero_row<T::BITS>();
#pragma unroll
        for (int j = 0; j < T::RPL; ++j) {
            raw[j].v.x = live ? raw[j].v.x : z.v.x;
            raw[j].v.y = live ? raw[j].v.y : z.v.y;
            if constexpr (T::BITS == 8) {
                raw[j].v.z = live ? raw[j].v.z : z.v.z;
                raw[j].v.w = live ? raw[j].v.w : z.v.w;
            }
        }
    }
}

// The raw fp16 scale of (row j, this lane's key group) for every row of the lane; scale_value() turns it into fp32
// (0 for lanes whose group lies past d_k).
template <class T>
__device__ __forceinline__ void load_scales(const uint16_t* sc_head, const LaneId& l, uint16_t (&sc)[T::RPL]) {
    int gi = (l.cg * CPL) / T::GROUP;
    gi = gi < T::NG ? gi : T::NG - 1;
#pragma unroll
    for (int j = 0; j < T::RPL; ++j) sc[j] = sc_head[size_t(row_of<T>(l, j)) * T::NG + gi];
}
template <class T>
__device__ __forceinline__ void scale_values(const uint16_t (&raw)[T::RPL], const LaneId& l, float (&sc)[T::RPL]) {
    const bool ok = (l.cg * CPL) / T::GROUP < T::NG;
#pragma unroll
    for (int j = 0; j < T::RPL; ++j) sc[j] = ok ? f16_to_f32(raw[j]) : 0.0f;
}

// A small register vector passed by value, so that selects between its elements stay selects (an array passed by
// reference would let the optimizer turn `c ? p[a] : p[b]` into a dynamically indexed load from scratch memory).
template <int N>
struct FVec {
    float v[N];
};

// Butterfly levels LV .. 0 over N row sums.  Levels at or above the scale-group size reduce-scatter (the lane whose
// bit is clear keeps the lower half and adds the partner's lower half); below it the lanes of a group already hold
// equal values and each just takes its share.  N halves per level; RPLP values end as NOWN.
template <class T, int LV, int N>
__device__ __forceinline__ FVec<(N >> (LV + 1))> butterfly(FVec<N> p, int cg) {
    const bool hi = (cg >> LV) & 1;
    FVec<N / 2> o;
#pragma unroll
    for (int t = 0; t < N / 2; ++t) {
        const float lo_v = p.v[t], hi_v = p.v[N / 2 + t];
        if constexpr (LV >= T::LVL_GRP) o.v[t] = (hi ? hi_v : lo_v) + partner<LV>(hi ? lo_v : hi_v);
        else o.v[t] = hi ? hi_v : lo_v;
    }
    if constexpr (LV > 0) return butterfly<T, LV - 1, N / 2>(o, cg);
    else return o;
}

// Per-lane partial row sums p[v][j] (this lane's 16 columns of row j against read-out vector v) -> full row sums of
// the rows the lane owns.  Inside a key group the partial sums are added first and multiplied by the group's scale,
// then the scaled group sums are added across the row (the reference's "(group sum) x scale, group by group",
// _fold_triton.py:191-196, here in a fixed butterfly order).
template <class T, int NV>
__device__ __forceinline__ void reduce_rows(const float (&p)[NV][T::RPLP], const float (&sc)[T::RPL],
                                            const LaneId& l, float (&own)[NV][T::NOWN]) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        FVec<T::RPLP> g;
#pragma unroll
        for (int j = 0; j < T::RPLP; ++j) {
            if (j < T::RPL) g.v[j] = block_sum<T::LPG>(p[v][j]) * sc[j < T::RPL ? j : 0];
            else g.v[j] = 0.0f;
        }
        const FVec<T::NOWN> o = butterfly<T, T::LVL_ROW - 1, T::RPLP>(g, l.cg);
#pragma unroll
        for (int t = 0; t < T::NOWN; ++t) own[v][t] = o.v[t];
    }
}

// Row dot products of the whole tile against NV read-out vectors whose 16-column pieces sit in x[v][].
template <class T, int NV>
__device__ __forceinline__ void tile_dots(const RawRow<T::BITS> (&raw)[T::RPL], const float (&x)[NV][CPL],
                                          float (&p)[NV][T::RPLP]) {
#pragma unroll
    for (int j = 0; j < T::RPLP; ++j) {
        if (j < T::RPL) {
            float c[CPL];
            decode_row<T::BITS>(raw[j], c);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                float s = c[0] * x[v][0];
#pragma unroll
                for (int t = 1; t < CPL; ++t) s = __builtin_fmaf(c[t], x[v][t], s);
                p[v][j] = s;
            }
        } else {
#pragma unroll
            for (int v = 0; v < NV; ++v) p[v][j] = 0.0f;
        }
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
// the decode buffer.  All loads below are unconditional (indices clamped into the live range) so that they can be
// issued back to back ahead of the state tile; dead slots and idle lanes are masked after the fact with selects.
// ---------------------------------------------------------------------------------------------------------------
template <class T>
struct BufAddr {                       // one (sequence, head)'s buffer fields
    uint8_t* KB;                       // [m][DK] int8 or bf16, of the head's KEY head
    uint8_t* UB;                       // [m][DV] int8 or bf16
    uint16_t* KBS;                     // [m] fp16 (int8 buffer)
    uint16_t* UBS;                     // [m] fp16 (int8 buffer)
};

// Raw delta values of the rows this lane owns, every slot: ub[i][t] = UB[min(i, m-1)][row t].
template <class T>
__device__ __forceinline__ void load_ub(const uint8_t* UB, int m, const LaneId& l, int jown,
                                        int32_t (&ub)[T::MMAX][T::NOWN]) {
#pragma unroll
    for (int i = 0; i < T::MMAX; ++i) {
        const int ic = i < m ? i : m - 1;
#pragma unroll
        for (int t = 0; t < T::NOWN; ++t) {
            int r = row_of<T>(l, jown + t);
            r = r < T::DV ? r : T::DV - 1;
            if constexpr (T::QBUF) ub[i][t] = reinterpret_cast<const int8_t*>(UB)[ic * T::DV + r];
            else ub[i][t] = reinterpret_cast<const uint16_t*>(UB)[ic * T::DV + r];
        }
    }
}
template <class T>
__device__ __forceinline__ float ub_value(int32_t raw) {
    if constexpr (T::QBUF) return float(raw);
    else return bf16_to_f32(uint16_t(raw));
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
// (reference `_coefs`, _fold_triton.py:260-272).  `gb` = the lane's slots' G (one per pass).  When the buffer is
// about to be folded the dequantized keys of slots 0 .. m-2 are staged in LDS for the fold.
template <class T, int NV>
__device__ __forceinline__ void buffer_coefs(const KeyBuf<T>& kbuf, const float (&gb)[KeyBuf<T>::KT], float gcur,
                                             int n, int m, bool full, const float (&x)[NV][CPL], const LaneId& l,
                                             float* lds_k, float (&c)[NV][T::MMAX]) {
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
            cl[v][t] = i < n ? dec * p : 0.0f;
        }
        if (full && i < m - 1) stage_kpiece<T>(lds_k, i, l, kb);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) c[v][i] = lane_bcast(cl[v][i / T::RG], (i % T::RG) * T::LPRP);
}

// Append the current token's value row: int8 with one absmax scale over the whole row (`us`, stored by lane 0), or
// bf16.  ur = the value as stored, dequantized (what the fold must use for slot n).
template <class T>
__device__ __forceinline__ void append_values(const float (&u)[T::NOWN], float us, const BufAddr<T>& a, int n,
                                              const LaneId& l, int jown, float (&ur)[T::NOWN]) {
    if (T::QBUF && l.lane == 0) a.UBS[n] = f32_to_f16(us);
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const int r = row_of<T>(l, jown + t);
        const bool valid = jown + t < T::RPL;
        if constexpr (T::QBUF) {
            const float c = round_buf(u[t], us);
            ur[t] = c * us;
            if (valid) reinterpret_cast<int8_t*>(a.UB)[n * T::DV + r] = int8_t(int(c));
        } else {
            const uint16_t hb = f32_to_bf16(u[t]);
            ur[t] = bf16_to_f32(hb);
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
// Stage the fold's value operand: lds_u[i][row] = f_i x U_i[row] for every slot (slot m-1: the value just appended);
// f_i = the slot's decay ratio held by lane i of `decf` (KDA passes 1).
template <class T>
__device__ __forceinline__ void stage_values(const int32_t (&ub)[T::MMAX][T::NOWN], float ubs_l, float decf,
                                             const float (&ur)[T::NOWN], int m, const LaneId& l, int jown,
                                             float* lds_u) {
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const int r = row_of<T>(l, jown + t);
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            if (i < m) {
                float uv = ub_value<T>(ub[i][t]);
                if constexpr (T::QBUF) uv = uv * lane_bcast(ubs_l, i);
                if (i == m - 1) uv = ur[t];
                if (jown + t >= T::RPL) uv = 0.0f;
                lds_u[i * T::UROW + r] = lane_bcast(decf, i) * uv;
            }
        }
    }
}
template <class T>
__device__ __forceinline__ void stage_key(const float (&kr)[T::NE], int slot, const LaneId& l, float* lds_k) {
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        if (e < T::LPRP * CPL) lds_k[slot * T::KROW + kpos<T>(e)] = e < T::DK ? kr[t] : 0.0f;
    }
}

// The fold: S = colmul * S_0 + sum_i du_i (x) kx_i over all m buffer slots in slot order, re-quantized in place
// (reference: _fused_triton.py:278-394 `_fold_head`; KDA _kda_triton.py:217-316; Mamba2 _mamba2_triton.py:213-332).
//   lds_k   [m][KROW]   the folded keys kx_i (GDN / Mamba2: the buffered keys; KDA: keys times their decay ratio)
//   lds_u   [m][UROW]   the folded values du_i (GDN / Mamba2: decay ratio x delta value; KDA: delta value)
//   colmul  this lane's 16 column factors on the dequantized old state (GDN / Mamba2: exp(G_m) in every column)
// Four rows per lane are in flight at a time; the register-resident rows are rotated down between rounds so that
// the loop stays rolled.  Each lane rewrites exactly the codes it read; the lowest lane of a key group stores the
// group's scale.  Codes are rint(S / scale) with the exact quotient wherever the reciprocal product is within
// |q| 2^-22 of a rounding boundary (rint_quot_fast / the wave-uniform exact pass).
template <class T>
__device__ __forceinline__ void fold_tile(RawRow<T::BITS> (&raw)[T::RPL], float (&sc)[T::RPL],
                                          const float (&colmul)[CPL], const float* lds_k, const float* lds_u, int m,
                                          uint8_t* head, uint16_t* sc_head, const LaneId& l) {
    constexpr int FR = 4;
    const bool live = l.cg < T::LPR;
    const int gi = (l.cg * CPL) / T::GROUP;
    const bool lead = live && (l.cg % T::LPG) == 0 && gi < T::NG;
    const float margin = 0.5f - (T::QMAX + 2.0f) * 2.384185791015625e-07f;      // 2^-22
#pragma unroll 1
    for (int j0 = 0; j0 < T::RPL; j0 += FR) {
        float acc[FR][CPL];
#pragma unroll
        for (int jj = 0; jj < FR; ++jj) {
            float c[CPL];
            decode_row<T::BITS>(raw[jj], c);
#pragma unroll
            for (int t = 0; t < CPL; ++t) acc[jj][t] = (c[t] * sc[jj]) * colmul[t];
        }
#pragma unroll 1
        for (int i = 0; i < m; ++i) {
            float kx[CPL];
            lds_piece<T>(lds_k + i * T::KROW, l.cg, kx);
#pragma unroll
            for (int jj = 0; jj < FR; ++jj) {
                const float du = lds_u[i * T::UROW + row_of<T>(l, j0 + jj)];
#pragma unroll
                for (int t = 0; t < CPL; ++t) acc[jj][t] = __builtin_fmaf(du, kx[t], acc[jj][t]);
            }
        }
#pragma unroll
        for (int jj = 0; jj < FR; ++jj) {
            float amax = 0.0f;
#pragma unroll
            for (int t = 0; t < CPL; ++t) amax = fmaxf(amax, fabsf(acc[jj][t]));
            amax = block_max<T::LPG>(amax);
            const float s = fp16_scale(amax, T::QMAX);
            const float r = 1.0f / s;
            const int row = row_of<T>(l, j0 + jj);
            if (lead) sc_head[size_t(row) * T::NG + gi] = f32_to_f16(s);
            float q[CPL];
            bool near = false;
#pragma unroll
            for (int t = 0; t < CPL; ++t) {
                const float qq = acc[jj][t] * r;
                const float c = rintf(qq);
                near |= fabsf(qq - c) >= margin;
                q[t] = c;
            }
            if (__builtin_amdgcn_ballot_w64(near) != 0) {          // some lane sits next to a rounding boundary
#pragma unroll
                for (int t = 0; t < CPL; ++t) q[t] = rintf(acc[jj][t] / s);
            }
#pragma unroll
            for (int t = 0; t < CPL; ++t) q[t] = fminf(fmaxf(q[t], -T::QMAX), T::QMAX);
            if (live) store_row<T::BITS>(head + size_t(row) * T::ROW_BYTES + l.cg * T::LANE_BYTES,
                                         encode_row<T::BITS>(q));
        }
        // rotate the remaining rows into place for the next round
#pragma unroll
        for (int j = 0; j + FR < T::RPL; ++j) { raw[j] = raw[j + FR]; sc[j] = sc[j + FR]; }
    }
}

}  // namespace sq
