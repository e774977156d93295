// The state tile of one (sequence, value head) in one wavefront: geometry, the streaming read of the stored codes
// with the row dot products and their cross-lane reduction, the decode buffer, and the fold (advance across the
// full buffer + re-quantize in place).  Shared by the Gated DeltaNet, KDA and Mamba2 step kernels.
//
// Resource plan (what keeps four wavefronts per SIMD resident): the codes stream through a window of LPRP rows per
// lane (32 VGPRs for int8), refilled row by row; the small operands (buffered values, scales) are fetched with one
// coalesced 128-bit load per lane and parked in LDS until needed; the fold reads the codes a second time (from L2 /
// Infinity Cache: they were read microseconds earlier) instead of pinning them in registers; the fold's LDS
// operands overlay the front end's.
#pragma once
#include "sq_device.cuh"

namespace sq {

// Compile-time geometry.  A row of DK codes is cut into DK/16 pieces of 16 columns; LPRP (that count rounded up to a
// power of two) consecutive lanes hold one row, lanes past DK/16 idle (d_k = 96: 6 of 8).  The wavefront therefore
// covers RG = 64/LPRP rows per load and a lane sees rows rg, rg + RG, rg + 2 RG, ...  Rows are handled in blocks of
// LPRP per lane (one reduce-scatter each), after which every lane owns one row of the block.
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
    static constexpr int NOWN = (RPL + LPRP - 1) / LPRP;  // row blocks per lane = rows a lane owns
    static constexpr int RPLP = NOWN * LPRP;              // rows per lane, padded to whole blocks
    static constexpr int NG = (DK + GROUP - 1) / GROUP;   // stored key groups per row (last may be ragged)
    static_assert(GROUP % CPL == 0 && GROUP >= CPL, "key group must be a multiple of 16");
    static constexpr int LPG = (GROUP / CPL < LPRP) ? GROUP / CPL : LPRP;   // lanes sharing one scale
    static constexpr int LVL_ROW = ilog2(LPRP);           // butterfly levels across a row
    static constexpr int LVL_GRP = ilog2(LPG);            // ... of which inside one scale group
    static constexpr int ROW_BYTES = BITS == 4 ? DK / 2 : DK;
    static constexpr int LANE_BYTES = BITS == 4 ? CPL / 2 : CPL;
    static constexpr float QMAX = float((1 << (BITS - 1)) - 1);
    static constexpr int NE = (DK + WAVE - 1) / WAVE;     // elements of a d_k vector per lane (element = lane + 64 t)
    static constexpr int BE = QBUF ? 1 : 2;               // bytes per buffer element (int8 / bf16)
    static constexpr int KPAD = CPL + 4;                  // LDS stride of a 16-column piece (spreads the banks)
    static constexpr int KROW = LPRP * KPAD;              // floats per d_k vector in LDS
    static constexpr int UROW = RPLP * RG;                // floats per d_v vector in LDS
    static constexpr int UB_BYTES = round_up(MMAX * DV * BE, 16);
    static constexpr int SC_BYTES = round_up(DV * NG * 2, 16);
};

// LDS plan of a step kernel that stages NX d_k vectors.  Front end: the vectors, the raw buffered values, the raw
// scales.  Fold: folded keys, folded values, column multipliers.  The two overlay each other.
template <class T, int NX>
struct LdsPlan {
    static constexpr int X = 0;
    static constexpr int UB = X + NX * T::KROW * 4;
    static constexpr int SC = UB + T::UB_BYTES;
    static constexpr int FRONT = SC + T::SC_BYTES;
    static constexpr int FK = 0;
    static constexpr int FU = FK + T::MMAX * T::KROW * 4;
    static constexpr int FC = FU + T::MMAX * T::UROW * 4;
    static constexpr int FOLD = FC + T::KROW * 4;
    static constexpr int BYTES = FRONT > FOLD ? FRONT : FOLD;
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

// Which row of a block of LPRP a lane owns after the block's reduction.  Every butterfly level halves the candidate
// range; the lane whose bit is set takes the upper half.
template <class T>
__device__ __forceinline__ int own_in_block(const LaneId& l) {
    int off = 0, n = T::LPRP;
#pragma unroll
    for (int lv = T::LVL_ROW - 1; lv >= 0; --lv) {
        n >>= 1;
        if ((l.cg >> lv) & 1) off += n;
    }
    return off;
}
// The head row a lane owns in block b (may lie past d_v in a padded last block: `owned_valid`).
template <class T>
__device__ __forceinline__ int owned_row(const LaneId& l, int b) {
    return row_of<T>(l, b * T::LPRP + own_in_block<T>(l));
}
template <class T>
__device__ __forceinline__ bool owned_valid(const LaneId& l, int b) {
    return b * T::LPRP + own_in_block<T>(l) < T::RPL;
}

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
// cross-lane reduction of one block of LPRP rows
// ---------------------------------------------------------------------------------------------------------------
// A small register vector passed by value, so that selects between its elements stay selects (an array passed by
// reference would let the optimizer turn `c ? p[a] : p[b]` into a dynamically indexed load from scratch memory).
template <int N>
struct FVec {
    float v[N];
};

// Butterfly levels LV .. 0 over N values.  Levels >= GRP reduce-scatter (the lane whose bit is clear keeps the lower
// half and adds the partner's lower half); below GRP the lanes already hold equal values and each takes its share.
template <int GRP, int LV, int N>
__device__ __forceinline__ FVec<(N >> (LV + 1))> butterfly(FVec<N> p, int cg) {
    const bool hi = (cg >> LV) & 1;
    FVec<N / 2> o;
#pragma unroll
    for (int t = 0; t < N / 2; ++t) {
        const float lo_v = p.v[t], hi_v = p.v[N / 2 + t];
        if constexpr (LV >= GRP) o.v[t] = (hi ? hi_v : lo_v) + partner<LV>(hi ? lo_v : hi_v);
        else o.v[t] = hi ? hi_v : lo_v;
    }
    if constexpr (LV > 0) return butterfly<GRP, LV - 1, N / 2>(o, cg);
    else return o;
}

// Partial sums p[t] (this lane's 16 columns of block row t against one read-out vector) -> the full, scaled row sum
// of the row the lane owns.  Inside a key group the partial sums are added first and multiplied by the group's scale,
// then the scaled group sums are added across the row (the reference's "(group sum) x scale, group by group",
// _fold_triton.py:191-196, here in a fixed butterfly order).  sc_lds: the head's raw fp16 scales [row][group].
template <class T>
__device__ __forceinline__ float reduce_block(FVec<T::LPRP> p, int b, const uint16_t* sc_lds, const LaneId& l) {
    const int gi = (l.cg * CPL) / T::GROUP;
    const bool has_group = gi < T::NG;
    if constexpr (T::LPG == T::LPRP) {                      // one group per row: reduce first, scale the owned row
        const FVec<1> o = butterfly<0, T::LVL_ROW - 1, T::LPRP>(p, l.cg);
        int r = owned_row<T>(l, b);
        r = r < T::DV ? r : T::DV - 1;
        return o.v[0] * f16_to_f32(sc_lds[r * T::NG]);
    } else {
#pragma unroll
        for (int t = 0; t < T::LPRP; ++t) {
            int r = row_of<T>(l, b * T::LPRP + t);
            r = r < T::DV ? r : T::DV - 1;
            const float s = has_group ? f16_to_f32(sc_lds[r * T::NG + (has_group ? gi : 0)]) : 0.0f;
            p.v[t] = block_sum<T::LPG>(p.v[t]) * s;
        }
        return butterfly<T::LVL_GRP, T::LVL_ROW - 1, T::LPRP>(p, l.cg).v[0];
    }
}

// ---------------------------------------------------------------------------------------------------------------
// the streaming pass over the stored codes
// ---------------------------------------------------------------------------------------------------------------
template <class T>
struct Window {
    RawRow<T::BITS> row[T::LPRP];
};
template <class T>
__device__ __forceinline__ const uint8_t* lane_codes(const uint8_t* head, const LaneId& l) {
    const int cc = l.cg < T::LPR ? l.cg : T::LPR - 1;       // idle lanes shadow a live one (masked later)
    return head + l.rg * T::ROW_BYTES + cc * T::LANE_BYTES;
}
// Issue the loads of block 0.
template <class T>
__device__ __forceinline__ void window_init(const uint8_t* lane_base, Window<T>& w) {
#pragma unroll
    for (int t = 0; t < T::LPRP; ++t)
        if (t < T::RPL) w.row[t] = load_row<T::BITS>(lane_base + t * (T::RG * T::ROW_BYTES));
}
// Row dot products of the whole tile against NV read-out vectors (16-column pieces in x[v][]), block by block; the
// window row just consumed is refilled with the same row of the next block.  own[v][b] = S0 x_v at the row the lane
// owns in block b.
template <class T, int NV>
__device__ __forceinline__ void state_pass(const uint8_t* lane_base, Window<T>& w, const float (&x)[NV][CPL],
                                           const uint16_t* sc_lds, const LaneId& l, float (&own)[NV][T::NOWN]) {
    const bool live = l.cg < T::LPR;
#pragma unroll
    for (int b = 0; b < T::NOWN; ++b) {
        FVec<T::LPRP> p[NV];
#pragma unroll
        for (int t = 0; t < T::LPRP; ++t) {
            const int j = b * T::LPRP + t;
            if (j < T::RPL) {
                float c[CPL];
                decode_row<T::BITS>(w.row[t], c);
                if (j + T::LPRP < T::RPL)
                    w.row[t] = load_row<T::BITS>(lane_base + (j + T::LPRP) * (T::RG * T::ROW_BYTES));
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    float s = c[0] * x[v][0];
#pragma unroll
                    for (int k = 1; k < CPL; ++k) s = __builtin_fmaf(c[k], x[v][k], s);
                    p[v].v[t] = live ? s : 0.0f;
                }
            } else {
#pragma unroll
                for (int v = 0; v < NV; ++v) p[v].v[t] = 0.0f;
            }
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) own[v][b] = reduce_block<T>(p[v], b, sc_lds, l);
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
// The codes and scales are read again from memory, four rows per lane at a time.  Each lane rewrites exactly the codes
// it read; the lowest lane of a key group stores the group's scale.  Codes are rint(S x (1/scale)) with the correctly
// rounded reciprocal: against rint(S / scale) that moves a code by one step only where the quotient lies within
// |q| 2^-24 of a rounding boundary (a few codes per million, the same order as the accumulation-order mismatches).
template <class T, bool COLVEC>
__device__ __forceinline__ void fold_tile(const float* lds_k, const float* lds_u, const float* lds_c, float cmul, int m,
                                          uint8_t* head, uint16_t* sc_head, const LaneId& l) {
    constexpr int FR = 4;
    const bool live = l.cg < T::LPR;
    int gi = (l.cg * CPL) / T::GROUP;
    const bool has_group = gi < T::NG;
    gi = has_group ? gi : T::NG - 1;
    const bool lead = live && (l.cg % T::LPG) == 0 && has_group;
    uint8_t* lane_base = const_cast<uint8_t*>(lane_codes<T>(head, l));
    float colmul[COLVEC ? CPL : 1];
    if constexpr (COLVEC) lds_piece<T>(lds_c, l.cg, colmul);
    else colmul[0] = cmul;
#pragma unroll 1
    for (int j0 = 0; j0 < T::RPL; j0 += FR) {
        RawRow<T::BITS> raw[FR];
        uint16_t scr[FR];
#pragma unroll
        for (int jj = 0; jj < FR; ++jj) {
            raw[jj] = load_row<T::BITS>(lane_base + (j0 + jj) * (T::RG * T::ROW_BYTES));
            scr[jj] = sc_head[row_of<T>(l, j0 + jj) * T::NG + gi];
        }
        float acc[FR][CPL];
#pragma unroll
        for (int jj = 0; jj < FR; ++jj) {
            float c[CPL];
            decode_row<T::BITS>(raw[jj], c);
            const float s = (live && has_group) ? f16_to_f32(scr[jj]) : 0.0f;
#pragma unroll
            for (int t = 0; t < CPL; ++t) acc[jj][t] = (c[t] * s) * colmul[COLVEC ? t : 0];
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
            if (lead) sc_head[row * T::NG + gi] = f32_to_f16(s);
            if (live)
                store_row<T::BITS>(lane_base + (j0 + jj) * (T::RG * T::ROW_BYTES), quantize_row<T::BITS>(acc[jj], r));
        }
    }
}

}  // namespace sq
