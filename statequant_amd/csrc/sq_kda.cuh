// KDA (Kimi Delta Attention: gated delta rule with a decay per key channel) packed decode step: one launch, one
// wavefront per (batch row, head).
//
// Replaces the reference's `_kda_step` (/root/reference/src/statequant/kernels/_kda_triton.py:38-149).  Per head, with
// G_n = G_{n-1} + g_n (vectors over d_k), A = exp(G_n):
//   c_x[i] = sum_j k_i[j] exp(G_n[j] - G_i[j]) x[j]              (x = q, k; slots i < n)
//   S'^T x = S0^T (A * x) + sum_i c_x[i] u_i;   u = beta (v - S'^T k);   o = S'^T q + (k.q) u
//   fold (buffer full): S = S0 diag(A) + sum_i u_i (exp(G_n - G_i) * k_i)^T, re-quantized in place
// The buffer keeps the cumulative decay per channel: GB is [h, m, d_k], GCUR is [h, d_k].  No grouped keys.
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

template <class T>
__global__ __launch_bounds__(WAVE) void kda_step_kernel(const KdaParams p) {
    // folded keys, folded values, then five d_k vectors: q, k (normalised), A*q, A*k, G_n
    __shared__ __attribute__((aligned(16))) float lds[T::MMAX * T::KROW + T::MMAX * T::UROW + 5 * T::KROW];
    float* lds_k = lds;
    float* lds_u = lds + T::MMAX * T::KROW;
    float* lds_q = lds_u + T::MMAX * T::UROW;
    float* lds_kn = lds_q + T::KROW;
    float* lds_qa = lds_kn + T::KROW;
    float* lds_ka = lds_qa + T::KROW;
    float* lds_g = lds_ka + T::KROW;

    const LaneId l = lane_id<T>();
    const int tile = xcd_tile(blockIdx.x, gridDim.x);
    const int b = tile / p.hv;
    const int h = tile - b * p.hv;
    const int m = p.m;
    constexpr int DK = T::DK, DV = T::DV;

    const int64_t seq = p.idx ? int64_t(p.idx[b]) : int64_t(b);
    const int64_t obase = int64_t(b) * p.s_out + int64_t(h) * DV;
    if (p.idx && seq <= 0) {
        for (int r = l.lane; r < DV; r += WAVE) store_f(p.out, p.out_dt, obase + r, 0.0f);
        return;
    }

    uint8_t* Sh = p.st.S + seq * p.st.sS + int64_t(h) * (DV * T::ROW_BYTES);
    uint16_t* SCh = p.st.SC + seq * p.st.sSC + int64_t(h) * (DV * T::NG);
    RawRow<T::BITS> raw[T::RPL];
    load_tile<T>(Sh, l, raw);
    float sc[T::RPL];
    load_scales<T>(SCh, l, sc);

    constexpr int BE = T::QBUF ? 1 : 2;
    uint8_t* KBh = p.st.KB + (seq * p.st.sKB + int64_t(h) * m * DK) * BE;
    uint8_t* UBh = p.st.UB + (seq * p.st.sUB + int64_t(h) * m * DV) * BE;
    uint16_t* KBSh = p.st.KBS + seq * p.st.sKBS + int64_t(h) * m;
    uint16_t* UBSh = p.st.UBS + seq * p.st.sUBS + int64_t(h) * m;
    float* GBh = p.st.GB + seq * p.st.sGB + int64_t(h) * m * DK;
    float* gch = p.st.GCUR + seq * p.st.sGC + int64_t(h) * DK;
    int32_t* np = p.st.NPTR + seq * p.st.sN + h;

    const int n = *np & (m - 1);
    const bool full = n == m - 1;

    float ubs_l = 1.0f;
    if (T::QBUF && l.lane < m) ubs_l = f16_to_f32(UBSh[l.lane]);

    const int jown = own_first<T>(l);
    float ub[T::MMAX][T::NOWN];
#pragma unroll
    for (int i = 0; i < T::MMAX; ++i)
#pragma unroll
        for (int t = 0; t < T::NOWN; ++t) {
            const int r = row_of<T>(l, jown + t);
            float x = 0.0f;
            if (i < m && jown + t < T::RPL) {
                if constexpr (T::QBUF) x = float(reinterpret_cast<const int8_t*>(UBh)[i * DV + r]);
                else x = bf16_to_f32(reinterpret_cast<const uint16_t*>(UBh)[i * DV + r]);
            }
            ub[i][t] = x;
        }

    // ---- prep: q, k normalised, the running decay per channel ----
    float qe[T::NE], ke[T::NE], gn[T::NE];
    float ssq = 0.0f, ssk = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        const int64_t off = int64_t(h) * DK + e;
        qe[t] = e < DK ? load_f(p.q, p.q_dt, int64_t(b) * p.s_q + off) : 0.0f;
        ke[t] = e < DK ? load_f(p.k, p.k_dt, int64_t(b) * p.s_k + off) : 0.0f;
        gn[t] = e < DK ? gch[e] + load_f(p.g, p.g_dt, int64_t(b) * p.s_g + off) : 0.0f;
        ssq = __builtin_fmaf(qe[t], qe[t], ssq);
        ssk = __builtin_fmaf(ke[t], ke[t], ssk);
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
        if (e < T::LPRP * CPL) {
            const float A = e < DK ? expf(gn[t]) : 0.0f;
            const int pos = kpos<T>(e);
            lds_q[pos] = qe[t];
            lds_kn[pos] = ke[t];
            lds_qa[pos] = A * qe[t];
            lds_ka[pos] = A * ke[t];
            lds_g[pos] = gn[t];
        }
    }
    const float kq = wave_sum(kqp);
    const float beta = load_f(p.beta, p.beta_dt, int64_t(b) * p.s_beta + h);
    __syncthreads();
    float xn[2][CPL], gp[CPL];
    lds_piece<T>(lds_q, l.cg, xn[0]);
    lds_piece<T>(lds_kn, l.cg, xn[1]);
    lds_piece<T>(lds_g, l.cg, gp);

    // ---- buffer coefficients with the per-channel decay ratio folded into the buffered key ----
    float cq[T::MMAX], ck[T::MMAX];
    {
        constexpr int KT = (T::MMAX + T::RG - 1) / T::RG;
        float cq_l[KT], ck_l[KT];
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const int i = l.rg + T::RG * t;
            float kd[CPL];
#pragma unroll
            for (int c = 0; c < CPL; ++c) kd[c] = 0.0f;
            if (i < m && l.cg < T::LPR && (i < n || (full && i < m - 1))) {
                float kb[CPL];
                if constexpr (T::QBUF) {
                    RawRow<8> rr = load_row<8>(KBh + i * DK + l.cg * CPL);
                    decode_row<8>(rr, kb);
                    const float ksc = f16_to_f32(KBSh[i]);
#pragma unroll
                    for (int c = 0; c < CPL; ++c) kb[c] = kb[c] * ksc;
                } else {
                    const uint16_t* kp = reinterpret_cast<const uint16_t*>(KBh) + i * DK + l.cg * CPL;
#pragma unroll
                    for (int c = 0; c < CPL; ++c) kb[c] = bf16_to_f32(kp[c]);
                }
                const float4* g4 = reinterpret_cast<const float4*>(GBh + i * DK + l.cg * CPL);
#pragma unroll
                for (int c = 0; c < CPL / 4; ++c) {
                    const float4 gi = g4[c];
                    kd[4 * c] = kb[4 * c] * expf(gp[4 * c] - gi.x);
                    kd[4 * c + 1] = kb[4 * c + 1] * expf(gp[4 * c + 1] - gi.y);
                    kd[4 * c + 2] = kb[4 * c + 2] * expf(gp[4 * c + 2] - gi.z);
                    kd[4 * c + 3] = kb[4 * c + 3] * expf(gp[4 * c + 3] - gi.w);
                }
            }
            float pq = kd[0] * xn[0][0], pk = kd[0] * xn[1][0];
#pragma unroll
            for (int c = 1; c < CPL; ++c) {
                pq = __builtin_fmaf(kd[c], xn[0][c], pq);
                pk = __builtin_fmaf(kd[c], xn[1][c], pk);
            }
            pq = block_sum<T::LPRP>(pq);
            pk = block_sum<T::LPRP>(pk);
            cq_l[t] = i < n ? pq : 0.0f;
            ck_l[t] = i < n ? pk : 0.0f;
            if (full && i < m - 1) {
                float4* d4 = reinterpret_cast<float4*>(lds_k + i * T::KROW + l.cg * T::KPAD);
#pragma unroll
                for (int c = 0; c < CPL / 4; ++c)
                    d4[c] = make_float4(kd[4 * c], kd[4 * c + 1], kd[4 * c + 2], kd[4 * c + 3]);
            }
        }
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            cq[i] = lane_bcast(cq_l[i / T::RG], (i % T::RG) * T::LPRP);
            ck[i] = lane_bcast(ck_l[i / T::RG], (i % T::RG) * T::LPRP);
        }
    }

    // ---- state pass against A*q, A*k ----
    float x[2][CPL];
    lds_piece<T>(lds_qa, l.cg, x[0]);
    lds_piece<T>(lds_ka, l.cg, x[1]);
    float part[2][T::RPLP];
    tile_dots<T, 2>(raw, x, part);
    float own[2][T::NOWN];
    reduce_rows<T, 2>(part, sc, l, own);

    float u[T::NOWN], amax = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const int r = row_of<T>(l, jown + t);
        const bool valid = jown + t < T::RPL;
        float sq = own[0][t];
        float sk = own[1][t];
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            float uv = ub[i][t];
            if constexpr (T::QBUF) uv = uv * lane_bcast(ubs_l, i);
            uv = i < n ? uv : 0.0f;
            sq = __builtin_fmaf(uv, cq[i], sq);
            sk = __builtin_fmaf(uv, ck[i], sk);
        }
        const float vt = valid ? load_f(p.v, p.v_dt, int64_t(b) * p.s_v + int64_t(h) * DV + r) : 0.0f;
        u[t] = beta * (vt - sk);
        const float o = __builtin_fmaf(kq, u[t], sq);
        if (valid) store_f(p.out, p.out_dt, obase + r, o);
        else u[t] = 0.0f;
        amax = fmaxf(amax, fabsf(u[t]));
    }

    // ---- append: decay vector, delta value, key ----
    float us = 1.0f, ks = 1.0f;
    float ur[T::NOWN];
    if constexpr (T::QBUF) {
        us = fp16_scale(wave_max(amax), 127.0f);
        float kmax = 0.0f;
#pragma unroll
        for (int t = 0; t < T::NE; ++t) kmax = fmaxf(kmax, fabsf(ke[t]));
        ks = fp16_scale(wave_max(kmax), 127.0f);
        if (l.lane == 0) { UBSh[n] = f32_to_f16(us); KBSh[n] = f32_to_f16(ks); }
    }
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const int r = row_of<T>(l, jown + t);
        if constexpr (T::QBUF) {
            const float c = round_buf(u[t], us);
            ur[t] = c * us;
            if (jown + t < T::RPL) reinterpret_cast<int8_t*>(UBh)[n * DV + r] = int8_t(int(c));
        } else {
            const uint16_t hb = f32_to_bf16(u[t]);
            ur[t] = bf16_to_f32(hb);
            if (jown + t < T::RPL) reinterpret_cast<uint16_t*>(UBh)[n * DV + r] = hb;
        }
    }
    float kr[T::NE];
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        if constexpr (T::QBUF) {
            const float c = round_buf(ke[t], ks);
            kr[t] = c * ks;
            if (e < DK) reinterpret_cast<int8_t*>(KBh)[n * DK + e] = int8_t(int(c));
        } else {
            const uint16_t hb = f32_to_bf16(ke[t]);
            kr[t] = bf16_to_f32(hb);
            if (e < DK) reinterpret_cast<uint16_t*>(KBh)[n * DK + e] = hb;
        }
        if (e < DK) GBh[n * DK + e] = gn[t];
    }

    // ---- fold ----
    if (full) {
#pragma unroll
        for (int t = 0; t < T::NOWN; ++t) {
            const int r = row_of<T>(l, jown + t);
#pragma unroll
            for (int i = 0; i < T::MMAX; ++i) {
                if (i < m) {
                    float uv = ub[i][t];
                    if constexpr (T::QBUF) uv = uv * lane_bcast(ubs_l, i);
                    if (i == m - 1) uv = ur[t];
                    lds_u[i * T::UROW + r] = uv;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const int e = l.lane + WAVE * t;
            if (e < T::LPRP * CPL) lds_k[(m - 1) * T::KROW + kpos<T>(e)] = e < DK ? kr[t] : 0.0f;   // decay ratio 1
        }
        __syncthreads();
        float colmul[CPL];
#pragma unroll
        for (int c = 0; c < CPL; ++c) colmul[c] = expf(gp[c]);      // = A on this lane's columns
        fold_tile<T>(raw, sc, colmul, lds_k, lds_u, m, Sh, SCh, l);
    }

    // ---- advance ----
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        if (e < DK) gch[e] = full ? 0.0f : gn[t];
    }
    if (l.lane == 0) *np = full ? 0 : n + 1;
}

template <class T>
int launch_kda(const KdaParams& p, hipStream_t stream) {
    hipLaunchKernelGGL(kda_step_kernel<T>, dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p);
    return int(hipGetLastError());
}

}  // namespace sq
