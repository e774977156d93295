// Gated DeltaNet packed decode step: one launch, one wavefront per (batch row, value head).
//
// Replaces the reference's fused Triton step (/root/reference/src/statequant/kernels/_fused_triton.py:48-190) with
// the same arithmetic per head:
//   prep     q, k l2-normalised (eps inside the sqrt), the gates, c_q[i] = (a_n/a_i) k_i.q, c_k[i] likewise
//   state    the stored codes read ONCE into registers; S0 q, S0 k by 16-column pieces + butterfly reduction;
//            buffer term as a slot-ordered fma chain; u = beta (v - a sk), o = a sq + (k.q) u
//   append   G_n, the delta value (int8 with one absmax scale over the row, or bf16), the key (first head of a
//            GQA group only)
//   fold     buffer full: S = a_m S0 + sum_i (a_m/a_i) u_i k_i^T from the codes still in registers (no second read
//            of the state), re-quantized in place
//   advance  running decay and this head's copy of the counter
// Every load the step needs is issued before the first use of any of them (small operands first, then the state
// tile), so a wavefront pays one memory round trip after the slot index, not one per operand.
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

template <class T>
__global__ __launch_bounds__(WAVE) void gdn_step_kernel(const GdnParams p) {
    __shared__ __attribute__((aligned(16))) float lds[T::LDS_FLOATS];
    float* lds_k = lds;
    float* lds_u = lds + T::MMAX * T::KROW;
    float* lds_q = lds_u + T::MMAX * T::UROW;
    float* lds_kn = lds_q + T::KROW;

    const LaneId l = lane_id<T>();
    const int tile = xcd_tile(blockIdx.x, gridDim.x);
    const int b = tile / p.hv;
    const int h = tile - b * p.hv;
    const int gqa = p.hv / p.hk;
    const int hk = h / gqa;
    const int m = p.m;
    constexpr int DK = T::DK, DV = T::DV;
    constexpr int KT = KeyBuf<T>::KT;

    const int64_t seq = p.idx ? int64_t(p.idx[b]) : int64_t(b);
    const int64_t obase = (int64_t(b) * p.hv + h) * DV;
    if (p.idx && seq <= 0) {                                     // padding row: zero output, touch nothing else
        for (int r = l.lane; r < DV; r += WAVE) store_f(p.out, p.out_dt, obase + r, 0.0f);
        return;
    }

    // ---- addresses ----
    uint8_t* Sh = p.st.S + seq * p.st.sS + int64_t(h) * (DV * T::ROW_BYTES);
    uint16_t* SCh = p.st.SC + seq * p.st.sSC + int64_t(h) * (DV * T::NG);
    constexpr int BE = T::QBUF ? 1 : 2;                           // bytes per buffer element
    BufAddr<T> buf;
    buf.KB = p.st.KB + (seq * p.st.sKB + int64_t(hk) * m * DK) * BE;
    buf.UB = p.st.UB + (seq * p.st.sUB + int64_t(h) * m * DV) * BE;
    buf.KBS = p.st.KBS + seq * p.st.sKBS + int64_t(hk) * m;
    buf.UBS = p.st.UBS + seq * p.st.sUBS + int64_t(h) * m;
    float* GBh = p.st.GB + seq * p.st.sGB + int64_t(h) * m;
    float* gcp = p.st.GCUR + seq * p.st.sGC + h;
    int32_t* np = p.st.NPTR + seq * p.st.sN + h;
    const int jown = own_first<T>(l);
    const int hq = p.qk_per_key_head ? hk : h;
    const bool own_key = !p.qk_per_key_head && gqa > 1;          // the buffered key is the group's first head's

    // ---- issue every load: counters, buffer, inputs, then the state tile ----
    const int n = *np & (m - 1);
    const float gcur = *gcp;
    const int lm = l.lane < m ? l.lane : m - 1;
    uint16_t ubs_raw = 0;
    if constexpr (T::QBUF) ubs_raw = buf.UBS[lm];
    const float gb_lane = GBh[lm];                                // lane i: slot i's cumulative decay
    int32_t ub[T::MMAX][T::NOWN];
    load_ub<T>(buf.UB, m, l, jown, ub);
    KeyBuf<T> kbuf;
    load_keybuf<T>(buf, m, l, kbuf);
    float gb[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) { const int i = l.rg + T::RG * t; gb[t] = GBh[i < m ? i : m - 1]; }
    uint32_t qr[T::NE], kr_[T::NE], kxr[T::NE];
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        int e = l.lane + WAVE * t;
        e = e < DK ? e : DK - 1;
        qr[t] = load_raw(p.q, p.q_dt, int64_t(b) * p.s_q + int64_t(hq) * DK + e);
        kr_[t] = load_raw(p.k, p.k_dt, int64_t(b) * p.s_k + int64_t(hq) * DK + e);
        kxr[t] = own_key ? load_raw(p.k, p.k_dt, int64_t(b) * p.s_k + int64_t(hk * gqa) * DK + e) : 0u;
    }
    // gate: a, b [rows, hv], A_log, dt_bias [hv];  no gate: the same four slots carry g, beta and two dummies
    // (the C ABI points them at g), so the loads need no branch
    const uint32_t g0 = load_raw_uniform(p.a, p.a_dt, int64_t(b) * p.s_a + h);
    const uint32_t g1 = load_raw_uniform(p.bt, p.bt_dt, int64_t(b) * p.s_bt + h);
    const uint32_t g2 = load_raw_uniform(p.A_log, p.A_log_dt, h);
    const uint32_t g3 = load_raw_uniform(p.dt_bias, p.dt_bias_dt, h);
    uint32_t vr[T::NOWN];
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        int r = row_of<T>(l, jown + t);
        r = r < DV ? r : DV - 1;
        vr[t] = load_raw(p.v, p.v_dt, int64_t(b) * p.s_v + int64_t(h) * DV + r);
    }
    RawRow<T::BITS> raw[T::RPL];
    load_tile<T>(Sh, l, raw);
    uint16_t scr[T::RPL];
    load_scales<T>(SCh, l, scr);

    // ---- prep: q, k (fla's l2 normalisation), gates ----
    const bool full = n == m - 1;
    float qe[T::NE], ke[T::NE], kxe[T::NE];
    float ssq = 0.0f, ssk = 0.0f, ssx = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const bool in = l.lane + WAVE * t < DK;
        qe[t] = in ? raw_to_f(qr[t], p.q_dt) : 0.0f;
        ke[t] = in ? raw_to_f(kr_[t], p.k_dt) : 0.0f;
        kxe[t] = in ? raw_to_f(kxr[t], p.k_dt) : 0.0f;
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
        const float x = raw_to_f(g0, p.a_dt) + raw_to_f(g3, p.dt_bias_dt);
        const float sp = x <= 20.0f ? logf(1.0f + expf(x)) : x;
        g = -expf(raw_to_f(g2, p.A_log_dt)) * sp;
        beta = 1.0f / (1.0f + expf(-raw_to_f(g1, p.bt_dt)));
    } else {
        g = raw_to_f(g0, p.a_dt);
        beta = raw_to_f(g1, p.bt_dt);
    }
    const float alpha = expf(gcur);
    const float a = expf(g);
    const float gnew = gcur + g;
    const float ubs_l = T::QBUF ? f16_to_f32(ubs_raw) : 1.0f;
    __syncthreads();
    float x[2][CPL];
    lds_piece<T>(lds_q, l.cg, x[0]);
    lds_piece<T>(lds_kn, l.cg, x[1]);

    // ---- buffer coefficients ----
    float c[2][T::MMAX];
    buffer_coefs<T, 2>(kbuf, gb, gcur, n, m, full, x, l, lds_k, c);

    // ---- state pass ----
    mask_tile<T>(l, raw);
    float sc[T::RPL];
    scale_values<T>(scr, l, sc);
    float part[2][T::RPLP];
    tile_dots<T, 2>(raw, x, part);
    float own[2][T::NOWN];
    reduce_rows<T, 2>(part, sc, l, own);

    // ---- the rows this lane owns: buffer term, u, o ----
    float u[T::NOWN], amax = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const int r = row_of<T>(l, jown + t);
        const bool valid = jown + t < T::RPL;
        float sq = alpha * own[0][t];
        float sk = alpha * own[1][t];
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            float uv = ub_value<T>(ub[i][t]);
            if constexpr (T::QBUF) uv = uv * lane_bcast(ubs_l, i);
            uv = i < n ? uv : 0.0f;                               // dead slots may hold anything: discard
            sq = __builtin_fmaf(uv, c[0][i], sq);
            sk = __builtin_fmaf(uv, c[1][i], sk);
        }
        const float vt = raw_to_f(vr[t], p.v_dt);
        u[t] = beta * __builtin_fmaf(-a, sk, vt);
        const float o = __builtin_fmaf(kq, u[t], a * sq);
        if (valid) store_f(p.out, p.out_dt, obase + r, o);
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
    float ur[T::NOWN], kr[T::NE];                                 // value / key as stored, dequantized
    append_values<T>(u, us, buf, n, l, jown, ur);
    append_key<T>(kxe, ks, buf, n, (h % gqa) == 0, l, kr);
    if (l.lane == 0) GBh[n] = gnew;

    // ---- fold ----
    if (full) {
        const float decf = l.lane < m - 1 ? expf(gnew - gb_lane) : 1.0f;     // a_m / a_i; the current token's: 1
        stage_values<T>(ub, ubs_l, decf, ur, m, l, jown, lds_u);
        stage_key<T>(kr, m - 1, l, lds_k);
        __syncthreads();
        const float alphan = expf(gnew);
        float colmul[CPL];
#pragma unroll
        for (int k = 0; k < CPL; ++k) colmul[k] = alphan;
        fold_tile<T>(raw, sc, colmul, lds_k, lds_u, m, Sh, SCh, l);
    }

    // ---- advance ----
    if (l.lane == 0) {
        *gcp = full ? 0.0f : gnew;
        *np = full ? 0 : n + 1;
    }
}

template <class T>
int launch_gdn(const GdnParams& p, hipStream_t stream) {
    hipLaunchKernelGGL(gdn_step_kernel<T>, dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p);
    return int(hipGetLastError());
}

}  // namespace sq
