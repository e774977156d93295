// KDA (Kimi Delta Attention: gated delta rule with a decay per key channel) packed decode step: one launch, one
// wavefront per (batch row, head).
//
// Replaces the reference's `_kda_step` (/root/reference/src/statequant/kernels/_kda_triton.py:38-149).  Per head, with
// G_n = G_{n-1} + g_n (vectors over d_k), A = exp(G_n):
//   c_x[i] = sum_j k_i[j] exp(G_n[j] - G_i[j]) x[j]              (x = q, k; slots i < n)
//   S'^T x = S0^T (A * x) + sum_i c_x[i] u_i;   u = beta (v - S'^T k);   o = S'^T q + (k.q) u
//   fold (buffer full): S = S0 diag(A) + sum_i u_i (exp(G_n - G_i) * k_i)^T, re-quantized in place
// The buffer keeps the cumulative decay per channel: GB is [h, m, d_k], GCUR is [h, d_k].  No grouped keys.
// Structure (loads up front, streamed tile, LDS staging, fold overlay) as in the GDN step.
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"
#include "sq_timeline.cuh"

namespace sq {

// exp of a decay or a decay ratio on the hardware's 2^x (1 ulp) after one multiplication by log2 e: a relative error of
// about |x| 2^-24, what the reference's device code (Triton's exp) has as well; the step takes m d_k + d_k of them per
// head, and the library exp's range reduction costs six times the instructions.
__device__ __forceinline__ float kda_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }

template <class T, int SPEC>
__global__ __launch_bounds__(WAVE, 4)
void kda_step_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ order, int per_xcd,
                     int hv, int hv_shift, SQ_TL_PARAM const KdaParams args) {
    SQ_MARK(0);                                                   // entry
    KdaParams p = args;
    assume_serving_case<SPEC>(p);                            // SPEC: see sq_params.h
    using L = LdsPlan<T, 3, 2>;                                   // q, k (normalised), G_n
    __shared__ __attribute__((aligned(16))) uint8_t lds[L::BYTES];
    float* lds_q = reinterpret_cast<float*>(lds + L::X);
    float* lds_kn = lds_q + T::KROW;
    float* lds_g = lds_kn + T::KROW;
    uint8_t* lds_ub = lds + L::UB;
    uint16_t* lds_sc = reinterpret_cast<uint16_t*>(lds + L::SC);
    uint8_t* lds_b = lds + L::B;
    float* lds_xs = reinterpret_cast<float*>(lds + L::XS);
    uint8_t* lds_a = lds + L::A;
    float* lds_own = reinterpret_cast<float*>(lds + L::OWN);
    float* lds_k = reinterpret_cast<float*>(lds + L::FK);
    float* lds_u = reinterpret_cast<float*>(lds + L::FU);
    float* lds_c = reinterpret_cast<float*>(lds + L::FC);

    const LaneId l = lane_id<T>();
    const TileId tid = tile_id_lead<SPEC>(order, per_xcd, hv, hv_shift);   // from the leading arguments
    const uint32_t b = tid.b, h = tid.h;
    const int m = p.m;
    const uint32_t um = m;
    constexpr int DK = T::DK, DV = T::DV;
    constexpr int KT = KeyBuf<T>::KT;

    const int32_t slot = idx ? idx[b] : int32_t(b);              // scalar load: on its way while the inputs are issued
    // the token's own operands first: their addresses need the batch row only, not the slot
    uint32_t qr[T::NE], kr_[T::NE], gr[T::NE];
    const void* qb = advance(p.q, p.q_dt, uint64_t(b) * p.s_q + h * DK);
    const void* kb_ = advance(p.k, p.k_dt, uint64_t(b) * p.s_k + h * DK);
    const void* gb_ = advance(p.g, p.g_dt, uint64_t(b) * p.s_g + h * DK);
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        uint32_t e = l.lane + WAVE * t;
        e = e < DK ? e : DK - 1;
        qr[t] = load_raw(qb, p.q_dt, e);
        kr_[t] = load_raw(kb_, p.k_dt, e);
        gr[t] = load_raw(gb_, p.g_dt, e);
    }
    const uint32_t betar = load_raw_uniform(p.beta, p.beta_dt, uint64_t(b) * p.s_beta + h);
    uint32_t vr[T::NOWN];
    const void* vb = advance(p.v, p.v_dt, uint64_t(b) * p.s_v + h * DV);
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        uint32_t r = owned_row<T>(l, t);
        r = r < DV ? r : DV - 1;
        vr[t] = load_raw(vb, p.v_dt, r);
    }
    void* const outp = advance(p.out, p.out_dt, uint64_t(b) * p.s_out + h * DV);
    if (idx && slot <= 0) {
        for (int r = l.lane; r < DV; r += WAVE) store_f(outp, p.out_dt, r, 0.0f);
        return;
    }
    SQ_MARK(1);                                                   // slot known, the token's loads issued
    const uint32_t seq = slot;

    uint8_t* Sh = field(p.st.S, seq, p.st.sS, h * (DV * T::ROW_BYTES));
    uint16_t* SCh = field(p.st.SC, seq, p.st.sSC, h * T::SC_ELEMS);
    BufAddr<T> buf;
    buf.KB = p.st.KB + (uint64_t(seq) * p.st.sKB + h * um * DK) * T::BE;
    buf.UB = p.st.UB + (uint64_t(seq) * p.st.sUB + h * um * DV) * T::BE;
    buf.KBS = field(p.st.KBS, seq, p.st.sKBS, h * um);
    buf.UBS = field(p.st.UBS, seq, p.st.sUBS, h * um);
    float* GBh = field(p.st.GB, seq, p.st.sGB, h * um * DK);
    float* gch = field(p.st.GCUR, seq, p.st.sGC, h * DK);
    int32_t* np = field(p.st.NPTR, seq, p.st.sN, h);
    const uint8_t* lane_base = lane_codes<T>(Sh, l);
    const int cc = l.cg < T::LPR ? l.cg : T::LPR - 1;

    // ---- issue the slot's loads: the state first, the buffer last and only its live slots (the fill count is a
    // scalar load issued first; by then it is here) ----
    const int n = *np & (m - 1);
    Window<T> win;
    window_init<T>(lane_base, win);
    Staged<T::SC_BYTES> st_sc;
    if constexpr (!T::FLT) stage_load(reinterpret_cast<const uint8_t*>(SCh), T::SC_ELEMS * 2, l.lane, st_sc);
    float gc[T::NE];
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        uint32_t e = l.lane + WAVE * t;
        e = e < DK ? e : DK - 1;
        gc[t] = gch[e];
    }
    const int nl = n > 0 ? n : 1;
    uint16_t ubs_raw = 0;
    if constexpr (T::QBUF) ubs_raw = buf.UBS[l.lane < nl ? l.lane : nl - 1];
    Staged<T::UB_BYTES> st_ub;
    stage_load(buf.UB, nl * DV * T::BE, l.lane, st_ub);
    KeyBuf<T> kbuf;
    load_keybuf<T>(buf, nl, l, kbuf);
    float4 gbp[KT][CPL / 4];                                      // the lane's piece of G_i of its slot(s)
#pragma unroll
    for (int t = 0; t < KT; ++t) {
        const int i = l.rg + T::RG * t;
        const float4* g4 = reinterpret_cast<const float4*>(GBh + (i < nl ? i : nl - 1) * DK + cc * CPL);
#pragma unroll
        for (int k = 0; k < CPL / 4; ++k) gbp[t][k] = g4[k];
    }

    SQ_MARK(2);                                                   // fill count here, every load issued

    // ---- prep: q, k normalised, the running decay per channel ----
    const bool full = n == m - 1;
    float qe[T::NE], ke[T::NE], gn[T::NE];
    float ssq = 0.0f, ssk = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const bool in = l.lane + WAVE * t < DK;
        qe[t] = in ? raw_to_f(qr[t], p.q_dt) : 0.0f;
        ke[t] = in ? raw_to_f(kr_[t], p.k_dt) : 0.0f;
        gn[t] = in ? gc[t] + raw_to_f(gr[t], p.g_dt) : 0.0f;
        ssq = __builtin_fmaf(qe[t], qe[t], ssq);
        ssk = __builtin_fmaf(ke[t], ke[t], ssk);
    }
    const float nq = sqrtf(wave_sum(ssq) + 1e-6f);
    const float nk = sqrtf(wave_sum(ssk) + 1e-6f);
    float kqp = 0.0f;
    float xa[2][T::NE];                                           // A * q, A * k: what the stored state is read against
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        qe[t] = qe[t] / nq * p.scale;
        ke[t] = ke[t] / nk;
        kqp = __builtin_fmaf(ke[t], qe[t], kqp);
        const int e = l.lane + WAVE * t;
        const float A = e < DK ? kda_exp(gn[t]) : 0.0f;
        xa[0][t] = A * qe[t];
        xa[1][t] = A * ke[t];
        if (e < T::LPRP * CPL) {
            const int pos = kpos<T>(e);
            lds_q[pos] = qe[t];
            lds_kn[pos] = ke[t];
            lds_g[pos] = gn[t];
        }
    }
    if constexpr (!T::AXV && !T::FLT) stage_planes<T, 2>(xa, l, lds_b, lds_xs);
    stage_store(lds_ub, m * DV * T::BE, l.lane, st_ub);
    if constexpr (!T::FLT) stage_store(reinterpret_cast<uint8_t*>(lds_sc), T::SC_ELEMS * 2, l.lane, st_sc);
    const float kq = wave_sum(kqp);
    const float beta = raw_to_f(betar, p.beta_dt);
    float ubs[T::MMAX];
#pragma unroll
    for (int i = 0; i < T::MMAX; ++i) ubs[i] = T::QBUF ? lane_bcast(f16_to_f32(ubs_raw), i) : 1.0f;
    wave_sync();
    SQ_MARK(3);                                                   // vectors, scales, buffered values here and staged

    // ---- buffer coefficients with the per-channel decay ratio folded into the buffered key ----
    float cqk[2][T::MMAX];
    {
        float xn[2][CPL], gp[CPL];
        lds_piece<T>(lds_q, l.cg, xn[0]);
        lds_piece<T>(lds_kn, l.cg, xn[1]);
        lds_piece<T>(lds_g, l.cg, gp);
        float cq_l[KT], ck_l[KT];
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const int i = l.rg + T::RG * t;
            float kb[CPL];
            decode_kpiece<T>(kbuf.piece[t], f16_to_f32(kbuf.kbs[t]), l, kb);
            const bool alive = i < n;                             // dead slots may hold anything: discard
            float pq = 0.0f, pk = 0.0f;
#pragma unroll
            for (int k = 0; k < CPL / 4; ++k) {
                const float4 gi = gbp[t][k];
                const float gv[4] = {gi.x, gi.y, gi.z, gi.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float kd = alive ? kb[4 * k + e] * kda_exp(gp[4 * k + e] - gv[e]) : 0.0f;
                    if (k == 0 && e == 0) { pq = kd * xn[0][0]; pk = kd * xn[1][0]; }
                    else {
                        pq = __builtin_fmaf(kd, xn[0][4 * k + e], pq);
                        pk = __builtin_fmaf(kd, xn[1][4 * k + e], pk);
                    }
                }
            }
            cq_l[t] = block_sum<T::LPRP>(pq);
            ck_l[t] = block_sum<T::LPRP>(pk);
        }
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            cqk[0][i] = lane_bcast(cq_l[i / T::RG], (i % T::RG) * T::LPRP);
            cqk[1][i] = lane_bcast(ck_l[i / T::RG], (i % T::RG) * T::LPRP);
        }
    }

    SQ_MARK(4);                                                   // buffered keys and decays here, coefficients done

    // ---- state pass against A*q, A*k ----
    float own[2][T::NOWN];
    state_pass<T, 2>(lane_base, win, lds_b, lds_xs, lds_sc, lds_a, lds_own, l, xa, own);
    SQ_MARK(5);                                                   // state pass done (all codes here)

    float u[T::NOWN], amax = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const bool valid = owned_valid<T>(l, t);
        int r = owned_row<T>(l, t);
        r = r < DV ? r : DV - 1;
        float sqk[2] = {own[0][t], own[1][t]};
        buffer_term<T, 2>(lds_ub, ubs, cqk, n, m, r, sqk);
        const float sq = sqk[0], sk = sqk[1];
        const float vt = raw_to_f(vr[t], p.v_dt);
        u[t] = beta * (vt - sk);
        const float o = __builtin_fmaf(kq, u[t], sq);
        if (valid) store_f(outp, p.out_dt, r, o);
        else u[t] = 0.0f;
        amax = fmaxf(amax, fabsf(u[t]));
    }

    SQ_MARK(6);                                                   // outputs stored
    // ---- append: decay vector, delta value, key ----
    float us = 1.0f, ks = 1.0f;
    if constexpr (T::QBUF) {
        us = fp16_scale(wave_max(amax), 127.0f);
        float kmax = 0.0f;
#pragma unroll
        for (int t = 0; t < T::NE; ++t) kmax = fmaxf(kmax, fabsf(ke[t]));
        ks = fp16_scale(wave_max(kmax), 127.0f);
    }
    float ur[T::NOWN], kr[T::NE];
    append_values<T>(u, us, buf, n, l, ur);
    append_key<T>(ke, ks, buf, n, true, l, kr);
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        if (e < DK) GBh[n * DK + e] = gn[t];
    }

    SQ_MARK(7);                                                   // appended
    // the running decay: stored here unless the buffer is full (then it restarts at zero, stored behind the fold), so
    // that it does not have to stay in registers across the fold
    if (!full) {
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const int e = l.lane + WAVE * t;
            if (e < DK) gch[e] = gn[t];
        }
    }
    // ---- fold ----
    if (full) {
        float uo[T::NOWN][T::MMAX];
        fold_fetch_values<T>(lds_ub, ubs, ur, m, l, uo);
        float gp[CPL];
        lds_piece<T>(lds_g, l.cg, gp);
        float f[T::MMAX];
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) f[i] = 1.0f;            // the decay ratio sits on the keys, per channel
        wave_sync();                                          // the front end's LDS is dead from here on
        fold_stage_values<T>(uo, f, m, l, lds_u);
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const int i = l.rg + T::RG * t;
            float kb[CPL];
            decode_kpiece<T>(kbuf.piece[t], f16_to_f32(kbuf.kbs[t]), l, kb);
#pragma unroll
            for (int k = 0; k < CPL / 4; ++k) {
                const float4 gi = gbp[t][k];
                kb[4 * k] = kb[4 * k] * kda_exp(gp[4 * k] - gi.x);
                kb[4 * k + 1] = kb[4 * k + 1] * kda_exp(gp[4 * k + 1] - gi.y);
                kb[4 * k + 2] = kb[4 * k + 2] * kda_exp(gp[4 * k + 2] - gi.z);
                kb[4 * k + 3] = kb[4 * k + 3] * kda_exp(gp[4 * k + 3] - gi.w);
            }
            if (i < m - 1) stage_kpiece<T>(lds_k, i, l, kb);
        }
        fold_stage_key<T>(kr, m - 1, l, lds_k);                   // the current token's decay ratio is exp(0) = 1
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const int e = l.lane + WAVE * t;
            if (e < T::LPRP * CPL) lds_c[kpos<T>(e)] = e < DK ? kda_exp(gn[t]) : 0.0f;     // = A
        }
        wave_sync();
        if constexpr (T::AXV) fold_tile_v<T, true>(lds_k, lds_u, lds_c, 1.0f, m, Sh, SCh, l);
        else fold_tile<T, true>(lds_k, lds_u, lds_c, 1.0f, m, Sh, SCh, l);
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const int e = l.lane + WAVE * t;
            if (e < DK) gch[e] = 0.0f;
        }
    }

    // ---- advance (the running decay of a full buffer is stored at the end of the fold) ----
    if (l.lane == 0) *np = full ? 0 : n + 1;
    SQ_MARK(8);                                                   // folded (a full buffer), counters advanced
}

template <class T, int SPEC>
int launch_kda(const KdaParams& p, hipStream_t stream) {
#ifdef SQ_TIMELINE
    hipLaunchKernelGGL((kda_step_kernel<T, SPEC>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p.idx, p.order, p.per_xcd,
                       p.hv, p.hv_shift, sq_timeline_buffer().p, sq_timeline_buffer().cap, p);
#else
    hipLaunchKernelGGL((kda_step_kernel<T, SPEC>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p.idx, p.order, p.per_xcd,
                       p.hv, p.hv_shift, p);
#endif
    return int(hipGetLastError());
}

}  // namespace sq
