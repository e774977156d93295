// Gated DeltaNet packed decode step: one launch, one wavefront per (batch row, value head).
//
// Replaces the reference's fused Triton step (/root/reference/src/statequant/kernels/_fused_triton.py:48-190) with
// the same arithmetic per head:
//   prep     q, k l2-normalised (eps inside the sqrt), the gates, c_q[i] = (a_n/a_i) k_i.q, c_k[i] likewise
//   state    the stored codes streamed once through a register window; S0 q, S0 k as integer dot products against
//            fixed-point digit planes of q, k; buffer term as a slot-ordered fma chain; u = beta (v - a sk),
//            o = a sq + (k.q) u
//   append   G_n, the delta value (int8 with one absmax scale over the row, or bf16), the key (first head of a
//            GQA group only)
//   fold     buffer full: S = a_m S0 + sum_i (a_m/a_i) u_i k_i^T, re-quantized in place
//   advance  running decay and this head's copy of the counter
// Every load a tile needs is issued before the first use of any of them (small operands first, then the first
// block of the state tile), so a wavefront pays one memory round trip after the slot index, not one per operand.
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

// Where one tile's fields live.
template <class T>
struct GdnAddr {
    int b, h, hk;
    bool live;                         // false: padding row (slot index <= 0)
    uint64_t obase;
    uint8_t* Sh;
    uint16_t* SCh;
    BufAddr<T> buf;
    float* GBh;
    float* gcp;
    int32_t* np;
};
template <class T>
__device__ __forceinline__ GdnAddr<T> gdn_addr(const GdnParams& p, const TileId& t, int32_t slot) {
    GdnAddr<T> a;
    a.b = t.b; a.h = t.h; a.hk = t.hk;
    a.live = !(p.idx && slot <= 0);
    const uint32_t seq = a.live ? uint32_t(slot) : 0u;
    const uint32_t m = p.m, h = a.h, hk = a.hk;
    a.obase = (uint64_t(uint32_t(a.b)) * uint32_t(p.hv) + h) * T::DV;
    a.Sh = field(p.st.S, seq, p.st.sS, h * (T::DV * T::ROW_BYTES));
    a.SCh = field(p.st.SC, seq, p.st.sSC, h * T::SC_ELEMS);
    a.buf.KB = p.st.KB + (uint64_t(seq) * p.st.sKB + hk * m * T::DK) * T::BE;
    a.buf.UB = p.st.UB + (uint64_t(seq) * p.st.sUB + h * m * T::DV) * T::BE;
    a.buf.KBS = field(p.st.KBS, seq, p.st.sKBS, hk * m);
    a.buf.UBS = field(p.st.UBS, seq, p.st.sUBS, h * m);
    a.GBh = field(p.st.GB, seq, p.st.sGB, h * m);
    a.gcp = field(p.st.GCUR, seq, p.st.sGC, h);
    a.np = field(p.st.NPTR, seq, p.st.sN, h);
    return a;
}

// Everything a tile's step reads before its state pass, as issued loads: counters, buffer, inputs, the first block of
// the state tile.  Raw bits only; nothing here waits for memory.
template <class T>
struct GdnFront {
    static constexpr int KT = KeyBuf<T>::KT;
    int n;
    float gcur;
    uint16_t ubs_raw;
    float gb_lane;
    Staged<T::UB_BYTES> st_ub;
    Staged<T::SC_BYTES> st_sc;
    KeyBuf<T> kbuf;
    float gb[KT];
    uint32_t qr[T::NE], kr[T::NE], kxr[T::NE];
    uint32_t g0, g1, g2, g3;
    uint32_t vr[T::NOWN];
    Window<T> win;
};
// The token's own operands: q, k, v and the gate.  Their addresses need the batch row only, not the slot, so they are
// issued while the slot index is still on its way.
template <class T>
__device__ __forceinline__ void gdn_issue_inputs(const GdnParams& p, const TileId& a, const LaneId& l, GdnFront<T>& f) {
    constexpr int DK = T::DK, DV = T::DV;
    const int gqa = p.gqa;
    const int hq = p.qk_per_key_head ? a.hk : a.h;
    const bool own_key = !p.qk_per_key_head && gqa > 1;          // the buffered key is the group's first head's
    const uint32_t b = a.b, h = a.h;
    const void* qb = advance(p.q, p.q_dt, uint64_t(b) * p.s_q + uint32_t(hq) * DK);
    const void* kb = advance(p.k, p.k_dt, uint64_t(b) * p.s_k + uint32_t(hq) * DK);
    const void* kxb = advance(p.k, p.k_dt, uint64_t(b) * p.s_k + uint32_t(a.hk * gqa) * DK);
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        uint32_t e = l.lane + WAVE * t;
        e = e < DK ? e : DK - 1;
        f.qr[t] = load_raw(qb, p.q_dt, e);
        f.kr[t] = load_raw(kb, p.k_dt, e);
        f.kxr[t] = own_key ? load_raw(kxb, p.k_dt, e) : 0u;
    }
    // gate: a, b [rows, hv], A_log, dt_bias [hv];  no gate: the same four slots carry g, beta and two dummies
    // (the C ABI points them at g), so the loads need no branch
    f.g0 = load_raw_uniform(p.a, p.a_dt, uint64_t(b) * p.s_a + h);
    f.g1 = load_raw_uniform(p.bt, p.bt_dt, uint64_t(b) * p.s_bt + h);
    f.g2 = load_raw_uniform(p.A_log, p.A_log_dt, h);
    f.g3 = load_raw_uniform(p.dt_bias, p.dt_bias_dt, h);
    const void* vb = advance(p.v, p.v_dt, uint64_t(b) * p.s_v + h * DV);
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        uint32_t r = owned_row<T>(l, t);
        r = r < DV ? r : DV - 1;
        f.vr[t] = load_raw(vb, p.v_dt, r);
    }
}

// The slot's side: counters, the first blocks of the state tile, the scales, the live part of the decode buffer.
template <class T>
__device__ __forceinline__ void gdn_issue(const GdnParams& p, const GdnAddr<T>& a, const LaneId& l, GdnFront<T>& f) {
    constexpr int DV = T::DV;
    const int m = p.m;
    f.n = *a.np & (m - 1);
    f.gcur = *a.gcp;
    window_init<T>(lane_codes<T>(a.Sh, l), f.win);
    if constexpr (!T::FLT) stage_load(reinterpret_cast<const uint8_t*>(a.SCh), T::SC_ELEMS * 2, l.lane, f.st_sc);
    // the buffer last, and only its live slots (the fill count is a scalar load issued first: by now it is here)
    const int nl = f.n > 0 ? f.n : 1;
    const int lm = l.lane < nl ? l.lane : nl - 1;
    f.ubs_raw = 0;
    if constexpr (T::QBUF) f.ubs_raw = a.buf.UBS[lm];
    f.gb_lane = a.GBh[lm];                                       // lane i: slot i's cumulative decay
    stage_load(a.buf.UB, nl * DV * T::BE, l.lane, f.st_ub);
    load_keybuf<T>(a.buf, nl, l, f.kbuf);
#pragma unroll
    for (int t = 0; t < GdnFront<T>::KT; ++t) { const int i = l.rg + T::RG * t; f.gb[t] = a.GBh[i < nl ? i : nl - 1]; }
}

// Register target: four wavefronts per SIMD (what the tile's LDS admits), except the 128 x 128 int8 tile with
// value-axis groups, which spills at 128 registers and is faster at three (136 registers: 45.6 -> 43.5 us per launch).
template <class T, int SPEC>
__global__ __launch_bounds__(WAVE, (T::AXV && T::BITS == 8 && T::DK == 128 && T::DV == 128) ? 3 : 4)
void gdn_step_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ order, int per_xcd,
                     int hv, int hv_shift, const GdnParams args) {
    GdnParams p = args;
    assume_serving_case<SPEC>(p);                            // SPEC: see sq_params.h
    using L = LdsPlan<T, 2>;
    __shared__ __attribute__((aligned(16))) uint8_t lds[L::BYTES];
    float* lds_q = reinterpret_cast<float*>(lds + L::X);
    float* lds_kn = lds_q + T::KROW;
    uint8_t* lds_ub = lds + L::UB;
    uint16_t* lds_sc = reinterpret_cast<uint16_t*>(lds + L::SC);
    uint8_t* lds_b = lds + L::B;
    float* lds_xs = reinterpret_cast<float*>(lds + L::XS);
    uint8_t* lds_a = lds + L::A;
    float* lds_own = reinterpret_cast<float*>(lds + L::OWN);
    float* lds_k = reinterpret_cast<float*>(lds + L::FK);          // the fold's operands overlay the above
    float* lds_u = reinterpret_cast<float*>(lds + L::FU);

    const int gqa = p.gqa;
    const int m = p.m;
    constexpr int DK = T::DK, DV = T::DV;
    constexpr int KT = KeyBuf<T>::KT;
    const bool own_key = !p.qk_per_key_head && gqa > 1;
    const LaneId l = lane_id<T>();
    TileId tid = tile_id_lead<SPEC>(order, per_xcd, hv, hv_shift);          // from the leading arguments
    const int32_t slot = idx ? idx[tid.b] : tid.b;               // scalar load: on its way while the inputs are issued
    tid.hk = p.gqa_shift >= 0 ? tid.h >> p.gqa_shift : tid.h / p.gqa;
    GdnFront<T> F;
    gdn_issue_inputs<T>(p, tid, l, F);
    const GdnAddr<T> A = gdn_addr<T>(p, tid, slot);
    void* const outp = advance(p.out, p.out_dt, A.obase);
    if (!A.live) {                                                // padding row: zero output, touch nothing else
        for (int r = l.lane; r < DV; r += WAVE) store_f(outp, p.out_dt, r, 0.0f);
        return;
    }
    gdn_issue<T>(p, A, l, F);
    const int h = A.h;
    const int n = F.n;
    const float gcur = F.gcur;
    const uint8_t* lane_base = lane_codes<T>(A.Sh, l);

    // ---- prep: q, k (fla's l2 normalisation), gates ----
    const bool full = n == m - 1;
    float qe[T::NE], ke[T::NE], kxe[T::NE];
    float ssq = 0.0f, ssk = 0.0f, ssx = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const bool in = l.lane + WAVE * t < DK;
        qe[t] = in ? raw_to_f(F.qr[t], p.q_dt) : 0.0f;
        ke[t] = in ? raw_to_f(F.kr[t], p.k_dt) : 0.0f;
        kxe[t] = in ? raw_to_f(F.kxr[t], p.k_dt) : 0.0f;
        ssq = __builtin_fmaf(qe[t], qe[t], ssq);
        ssk = __builtin_fmaf(ke[t], ke[t], ssk);
        ssx = __builtin_fmaf(kxe[t], kxe[t], ssx);
    }
    const float nq = sqrtf(wave_sum(ssq) + 1e-6f);
    const float nk = sqrtf(wave_sum(ssk) + 1e-6f);
    float kqp = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        qe[t] = qe[t] / nq * p.scale;
        ke[t] = ke[t] / nk;
        kqp = __builtin_fmaf(ke[t], qe[t], kqp);
        const int e = l.lane + WAVE * t;
        if (e < T::LPRP * CPL) { lds_q[kpos<T>(e)] = qe[t]; lds_kn[kpos<T>(e)] = ke[t]; }
    }
    {
        float xe[2][T::NE];
#pragma unroll
        for (int t = 0; t < T::NE; ++t) { xe[0][t] = qe[t]; xe[1][t] = ke[t]; }
        if constexpr (!T::AXV && !T::FLT) stage_planes<T, 2>(xe, l, lds_b, lds_xs);
    }
    stage_store(lds_ub, m * DV * T::BE, l.lane, F.st_ub);
    if constexpr (!T::FLT) stage_store(reinterpret_cast<uint8_t*>(lds_sc), T::SC_ELEMS * 2, l.lane, F.st_sc);
    const float kq = wave_sum(kqp);
    if (own_key) {
        const float nx = sqrtf(wave_sum(ssx) + 1e-6f);
#pragma unroll
        for (int t = 0; t < T::NE; ++t) kxe[t] = kxe[t] / nx;
    } else {
#pragma unroll
        for (int t = 0; t < T::NE; ++t) kxe[t] = ke[t];
    }
    float g, beta;
    if (p.gate) {
        const float x = raw_to_f(F.g0, p.a_dt) + raw_to_f(F.g3, p.dt_bias_dt);
        const float sp = x <= 20.0f ? logf(1.0f + expf(x)) : x;
        g = -expf(raw_to_f(F.g2, p.A_log_dt)) * sp;
        beta = 1.0f / (1.0f + expf(-raw_to_f(F.g1, p.bt_dt)));
    } else {
        g = raw_to_f(F.g0, p.a_dt);
        beta = raw_to_f(F.g1, p.bt_dt);
    }
    const float alpha = expf(gcur);
    const float a = expf(g);
    const float gnew = gcur + g;
    float ubs[T::MMAX];
#pragma unroll
    for (int i = 0; i < T::MMAX; ++i) ubs[i] = T::QBUF ? lane_bcast(f16_to_f32(F.ubs_raw), i) : 1.0f;
    wave_sync();
    float x[2][CPL];
    lds_piece<T>(lds_q, l.cg, x[0]);
    lds_piece<T>(lds_kn, l.cg, x[1]);

    // ---- buffer coefficients ----
    float c[2][T::MMAX];
    buffer_coefs<T, 2>(F.kbuf, F.gb, gcur, n, x, l, c);

    // ---- state pass ----
    float own[2][T::NOWN];
    float xe2[2][T::NE];
#pragma unroll
    for (int t = 0; t < T::NE; ++t) { xe2[0][t] = qe[t]; xe2[1][t] = ke[t]; }
    state_pass<T, 2>(lane_base, F.win, lds_b, lds_xs, lds_sc, lds_a, lds_own, l, xe2, own);

    const KeyBuf<T>& kbuf = F.kbuf;
    const float gb_lane = F.gb_lane;
    const uint32_t (&vr)[T::NOWN] = F.vr;

    // ---- the rows this lane owns: buffer term, u, o ----
    float u[T::NOWN], amax = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const bool valid = owned_valid<T>(l, t);
        int r = owned_row<T>(l, t);
        r = r < DV ? r : DV - 1;
        float sqk[2] = {alpha * own[0][t], alpha * own[1][t]};
        buffer_term<T, 2>(lds_ub, ubs, c, n, m, r, sqk);
        const float sq = sqk[0], sk = sqk[1];
        const float vt = raw_to_f(vr[t], p.v_dt);
        u[t] = beta * __builtin_fmaf(-a, sk, vt);
        const float o = __builtin_fmaf(kq, u[t], a * sq);
        if (valid) store_f(outp, p.out_dt, r, o);
        else u[t] = 0.0f;
        amax = fmaxf(amax, fabsf(u[t]));
    }

    // ---- append ----
    float us = 1.0f, ks = 1.0f;
    if constexpr (T::QBUF) {
        us = fp16_scale(wave_max(amax), 127.0f);
        float kmax = 0.0f;
#pragma unroll
        for (int t = 0; t < T::NE; ++t) kmax = fmaxf(kmax, fabsf(kxe[t]));
        ks = fp16_scale(wave_max(kmax), 127.0f);
    }
    float ur[T::NOWN], kr[T::NE];                         // value / key as stored, dequantized
    append_values<T>(u, us, A.buf, n, l, ur);
    append_key<T>(kxe, ks, A.buf, n, int(h) == A.hk * gqa, l, kr);
    if (l.lane == 0) A.GBh[n] = gnew;

    // ---- advance: here unless the buffer is full (then behind the fold, to zero), so that the running decay and
    //      the count do not stay in registers across the fold ----
    if (!full && l.lane == 0) {
        *A.gcp = gnew;
        *A.np = n + 1;
    }
    // ---- fold ----
    if (full) {
        float uo[T::NOWN][T::MMAX];
        fold_fetch_values<T>(lds_ub, ubs, ur, m, l, uo);
        const float decf = l.lane < m - 1 ? expf(gnew - gb_lane) : 1.0f;     // a_m / a_i; current token: 1
        float f[T::MMAX];
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) f[i] = lane_bcast(decf, i);
        wave_sync();                                  // the front end's LDS is dead from here on
        fold_stage_values<T>(uo, f, m, l, lds_u);
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const int i = l.rg + T::RG * t;
            float kb[CPL];
            decode_kpiece<T>(kbuf.piece[t], f16_to_f32(kbuf.kbs[t]), l, kb);
            if (i < m - 1) stage_kpiece<T>(lds_k, i, l, kb);
        }
        fold_stage_key<T>(kr, m - 1, l, lds_k);
        wave_sync();
        if constexpr (T::AXV) fold_tile_v<T, false>(lds_k, lds_u, nullptr, expf(gnew), m, A.Sh, A.SCh, l);
        else fold_tile<T, false>(lds_k, lds_u, nullptr, expf(gnew), m, A.Sh, A.SCh, l);
        if (l.lane == 0) {
            *A.gcp = 0.0f;
            *A.np = 0;
        }
    }
}

template <class T, int SPEC>
int launch_gdn(const GdnParams& p, hipStream_t stream) {
    hipLaunchKernelGGL((gdn_step_kernel<T, SPEC>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p.idx, p.order, p.per_xcd,
                       p.hv, p.hv_shift, p);
    return int(hipGetLastError());
}

}  // namespace sq
