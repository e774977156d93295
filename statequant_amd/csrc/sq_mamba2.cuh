// Mamba2 / SSD packed decode step: one launch, one wavefront per (batch row, head).
//
// Replaces the reference's `_m2_step` (/root/reference/src/statequant/kernels/_mamba2_triton.py:48-197): key = B of
// the head's group (shared like a GQA key), query = C, buffered value u = dt x, scalar decay exp(A dt); no delta
// term, no normalisation:
//   y_n = a_n [alpha S0 C + sum_{i<n} (alpha/alpha_i) (B_i.C) u_i] + (B_n.C) u_n + D x_n
//   fold (buffer full): S = alpha_m S0 + sum_i (alpha_m/alpha_i) u_i B_i^T, re-quantized in place
// Structure (loads up front, streamed tile, LDS staging, fold overlay) as in the GDN step.
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

// Occupancy target: four wavefronts per SIMD; the d_state-256 tile does not fit 128 registers, and asked for two it
// is compiled at 234 without spills (asked for four the compiler gives up at 364, one wavefront per SIMD).
template <class T, int SPEC>
__global__ __launch_bounds__(WAVE, T::DK > 128 ? 2 : 4)
void mamba2_step_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ order, int per_xcd, int hv, int hv_shift, const Mamba2Params args) {
    Mamba2Params p = args;
    assume_serving_case<SPEC>(p);                            // SPEC: see sq_params.h
    using L = LdsPlan<T, 1, 1>;
    __shared__ __attribute__((aligned(16))) uint8_t lds[L::BYTES];
    float* lds_cv = reinterpret_cast<float*>(lds + L::X);
    uint8_t* lds_ub = lds + L::UB;
    uint16_t* lds_sc = reinterpret_cast<uint16_t*>(lds + L::SC);
    uint8_t* lds_b = lds + L::B;
    float* lds_xs = reinterpret_cast<float*>(lds + L::XS);
    uint8_t* lds_a = lds + L::A;
    float* lds_own = reinterpret_cast<float*>(lds + L::OWN);
    float* lds_k = reinterpret_cast<float*>(lds + L::FK);
    float* lds_u = reinterpret_cast<float*>(lds + L::FU);

    const LaneId l = lane_id<T>();
    const TileId tid = tile_id_lead<SPEC>(order, per_xcd, hv, hv_shift);   // from the leading arguments
    const uint32_t b = tid.b, h = tid.h, hk = p.gqa_shift >= 0 ? tid.h >> p.gqa_shift : tid.h / p.gqa;
    const int gqa = p.gqa;
    const int m = p.m;
    const uint32_t um = m;
    constexpr int DK = T::DK, DV = T::DV;
    constexpr int KT = KeyBuf<T>::KT;

    const int32_t slot = idx ? idx[b] : int32_t(b);              // scalar load: on its way while the inputs are issued
    // the token's own operands first: their addresses need the batch row only, not the slot
    uint32_t cr[T::NE], br[T::NE];
    const void* cb = advance(p.C, p.C_dt, uint64_t(b) * p.s_C + hk * DK);
    const void* bb = advance(p.B, p.B_dt, uint64_t(b) * p.s_B + hk * DK);
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        uint32_t e = l.lane + WAVE * t;
        e = e < DK ? e : DK - 1;
        cr[t] = load_raw(cb, p.C_dt, e);
        br[t] = load_raw(bb, p.B_dt, e);
    }
    const uint32_t dtr = load_raw_uniform(p.dt, p.dt_dt, uint64_t(b) * p.s_dt + h);
    const uint32_t ar = load_raw_uniform(p.A, p.A_dt, h);
    const uint32_t dbr = load_raw_uniform(p.dt_bias, p.dt_bias_dt, h);     // absent: the C ABI points them at A,
    const uint32_t ddr = load_raw_uniform(p.D, p.D_dt, h);                 // so the loads need no branch
    uint32_t xr_raw[T::NOWN];
    const void* xb = advance(p.x, p.x_dt, uint64_t(b) * p.s_x + h * DV);
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        uint32_t r = owned_row<T>(l, t);
        r = r < DV ? r : DV - 1;
        xr_raw[t] = load_raw(xb, p.x_dt, r);
    }
    void* const outp = advance(p.out, p.out_dt, uint64_t(b) * p.s_out + h * DV);
    if (idx && slot <= 0) {
        for (int r = l.lane; r < DV; r += WAVE) store_f(outp, p.out_dt, r, 0.0f);
        return;
    }
    const uint32_t seq = slot;

    uint8_t* Sh = field(p.st.S, seq, p.st.sS, h * (DV * T::ROW_BYTES));
    uint16_t* SCh = field(p.st.SC, seq, p.st.sSC, h * T::SC_ELEMS);
    BufAddr<T> buf;
    buf.KB = p.st.KB + (uint64_t(seq) * p.st.sKB + hk * um * DK) * T::BE;
    buf.UB = p.st.UB + (uint64_t(seq) * p.st.sUB + h * um * DV) * T::BE;
    buf.KBS = field(p.st.KBS, seq, p.st.sKBS, hk * um);
    buf.UBS = field(p.st.UBS, seq, p.st.sUBS, h * um);
    float* GBh = field(p.st.GB, seq, p.st.sGB, h * um);
    float* gcp = field(p.st.GCUR, seq, p.st.sGC, h);
    int32_t* np = field(p.st.NPTR, seq, p.st.sN, h);
    const uint8_t* lane_base = lane_codes<T>(Sh, l);

    // ---- issue the slot's loads: the state first, the buffer last and only its live slots (the fill count is a
    // scalar load issued first; by then it is here) ----
    const int n = *np & (m - 1);
    const float gcur = *gcp;
    Window<T> win;
    window_init<T>(lane_base, win);
    Staged<T::SC_BYTES> st_sc;
    if constexpr (!T::FLT) stage_load(reinterpret_cast<const uint8_t*>(SCh), T::SC_ELEMS * 2, l.lane, st_sc);
    const int nl = n > 0 ? n : 1;
    const int lm = l.lane < nl ? l.lane : nl - 1;
    uint16_t ubs_raw = 0;
    if constexpr (T::QBUF) ubs_raw = buf.UBS[lm];
    const float gb_lane = GBh[lm];
    Staged<T::UB_BYTES> st_ub;
    stage_load(buf.UB, nl * DV * T::BE, l.lane, st_ub);
    KeyBuf<T> kbuf;
    load_keybuf<T>(buf, nl, l, kbuf);
    float gb[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) { const int i = l.rg + T::RG * t; gb[t] = GBh[i < nl ? i : nl - 1]; }

    // ---- prep: B, C of the group, dt, decay ----
    const bool full = n == m - 1;
    float ce[T::NE], kxe[T::NE];
    float bcp = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        ce[t] = e < DK ? raw_to_f(cr[t], p.C_dt) : 0.0f;
        kxe[t] = e < DK ? raw_to_f(br[t], p.B_dt) : 0.0f;
        bcp = __builtin_fmaf(kxe[t], ce[t], bcp);
        if (e < T::LPRP * CPL) lds_cv[kpos<T>(e)] = ce[t];
    }
    {
        float xe[1][T::NE];
#pragma unroll
        for (int t = 0; t < T::NE; ++t) xe[0][t] = ce[t];
        if constexpr (!T::AXV && !T::FLT) stage_planes<T, 1>(xe, l, lds_b, lds_xs);
    }
    stage_store(lds_ub, m * DV * T::BE, l.lane, st_ub);
    if constexpr (!T::FLT) stage_store(reinterpret_cast<uint8_t*>(lds_sc), T::SC_ELEMS * 2, l.lane, st_sc);
    const float bc = wave_sum(bcp);
    float dt = raw_to_f(dtr, p.dt_dt);
    if (p.has_dt_bias) dt = dt + raw_to_f(dbr, p.dt_bias_dt);
    if (p.dt_softplus) dt = dt <= 20.0f ? logf(1.0f + expf(dt)) : dt;
    if (p.dt_clamp) dt = fminf(fmaxf(dt, p.dt_min), p.dt_max);
    const float g = raw_to_f(ar, p.A_dt) * dt;                   // rounded on its own (no contraction into gcur + g)
    const float a = expf(g);
    const float dd = p.has_D ? raw_to_f(ddr, p.D_dt) : 0.0f;
    const float alpha = expf(gcur);
    const float gnew = gcur + g;
    float ubs[T::MMAX];
#pragma unroll
    for (int i = 0; i < T::MMAX; ++i) ubs[i] = T::QBUF ? lane_bcast(f16_to_f32(ubs_raw), i) : 1.0f;
    wave_sync();
    float x[1][CPL];
    lds_piece<T>(lds_cv, l.cg, x[0]);

    // ---- buffer coefficients c[i] = (alpha / alpha_i) B_i . C ----
    float c[1][T::MMAX];
    buffer_coefs<T, 1>(kbuf, gb, gcur, n, x, l, c);

    // ---- state pass ----
    float own[1][T::NOWN];
    float xe1[1][T::NE];
#pragma unroll
    for (int t = 0; t < T::NE; ++t) xe1[0][t] = ce[t];
    state_pass<T, 1>(lane_base, win, lds_b, lds_xs, lds_sc, lds_a, lds_own, l, xe1, own);

    // ---- owned rows: y, and the value to buffer ----
    float u[T::NOWN], amax = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const bool valid = owned_valid<T>(l, t);
        int r = owned_row<T>(l, t);
        r = r < DV ? r : DV - 1;
        float sq1[1] = {alpha * own[0][t]};
        buffer_term<T, 1>(lds_ub, ubs, c, n, m, r, sq1);
        const float sq = sq1[0];
        const float xr = valid ? raw_to_f(xr_raw[t], p.x_dt) : 0.0f;
        u[t] = dt * xr;
        float y = __builtin_fmaf(bc, u[t], a * sq);
        if (p.has_D) y = __builtin_fmaf(dd, xr, y);
        if (valid) store_f(outp, p.out_dt, r, y);
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
    float ur[T::NOWN], kr[T::NE];
    append_values<T>(u, us, buf, n, l, ur);
    append_key<T>(kxe, ks, buf, n, int(h) == hk * gqa, l, kr);
    if (l.lane == 0) GBh[n] = gnew;

    // ---- fold ----
    if (full) {
        float uo[T::NOWN][T::MMAX];
        fold_fetch_values<T>(lds_ub, ubs, ur, m, l, uo);
        const float decf = l.lane < m - 1 ? expf(gnew - gb_lane) : 1.0f;
        float f[T::MMAX];
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) f[i] = lane_bcast(decf, i);
        wave_sync();
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
        if constexpr (T::AXV) fold_tile_v<T, false>(lds_k, lds_u, nullptr, expf(gnew), m, Sh, SCh, l);
        else fold_tile<T, false>(lds_k, lds_u, nullptr, expf(gnew), m, Sh, SCh, l);
    }

    if (l.lane == 0) {
        *gcp = full ? 0.0f : gnew;
        *np = full ? 0 : n + 1;
    }
}

template <class T, int SPEC>
int launch_mamba2(const Mamba2Params& p, hipStream_t stream) {
    hipLaunchKernelGGL((mamba2_step_kernel<T, SPEC>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p.idx, p.order, p.per_xcd,
                       p.hv, p.hv_shift, p);
    return int(hipGetLastError());
}

}  // namespace sq
