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

    const int64_t seq = p.idx ? int64_t(p.idx[b]) : int64_t(b);
    const int64_t obase = (int64_t(b) * p.hv + h) * DV;
    if (p.idx && seq <= 0) {                                     // padding row: zero output, touch nothing else
        for (int r = l.lane; r < DV; r += WAVE) store_f(p.out, p.out_dt, obase + r, 0.0f);
        return;
    }

    // ---- the state tile and everything else that only depends on the slot: issue the loads first ----
    uint8_t* Sh = p.st.S + seq * p.st.sS + int64_t(h) * (DV * T::ROW_BYTES);
    uint16_t* SCh = p.st.SC + seq * p.st.sSC + int64_t(h) * (DV * T::NG);
    RawRow<T::BITS> raw[T::RPL];
    load_tile<T>(Sh, l, raw);
    float sc[T::RPL];
    load_scales<T>(SCh, l, sc);

    constexpr int BE = T::QBUF ? 1 : 2;                           // bytes per buffer element
    uint8_t* KBh = p.st.KB + (seq * p.st.sKB + int64_t(hk) * m * DK) * BE;
    uint8_t* UBh = p.st.UB + (seq * p.st.sUB + int64_t(h) * m * DV) * BE;
    uint16_t* KBSh = p.st.KBS + seq * p.st.sKBS + int64_t(hk) * m;
    uint16_t* UBSh = p.st.UBS + seq * p.st.sUBS + int64_t(h) * m;
    float* GBh = p.st.GB + seq * p.st.sGB + int64_t(h) * m;
    float* gcp = p.st.GCUR + seq * p.st.sGC + h;
    int32_t* np = p.st.NPTR + seq * p.st.sN + h;

    const int n = *np & (m - 1);
    const float gcur = *gcp;
    const bool full = n == m - 1;

    // per-slot scalars: lane i holds slot i's
    float ubs_l = 1.0f;
    if (T::QBUF && l.lane < m) ubs_l = f16_to_f32(UBSh[l.lane]);

    // delta values of the rows this lane will own, all slots (dead slots are discarded below, never multiplied)
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

    // ---- prep: q, k (fla's l2 normalisation), gates ----
    const int hq = p.qk_per_key_head ? hk : h;
    float qe[T::NE], ke[T::NE], kxe[T::NE];
    float ssq = 0.0f, ssk = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        qe[t] = e < DK ? load_f(p.q, p.q_dt, int64_t(b) * p.s_q + int64_t(hq) * DK + e) : 0.0f;
        ke[t] = e < DK ? load_f(p.k, p.k_dt, int64_t(b) * p.s_k + int64_t(hq) * DK + e) : 0.0f;
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
        kxe[t] = ke[t];
        kqp = __builtin_fmaf(ke[t], qe[t], kqp);
        const int e = l.lane + WAVE * t;
        if (e < T::LPRP * CPL) { lds_q[kpos<T>(e)] = qe[t]; lds_kn[kpos<T>(e)] = ke[t]; }
    }
    const float kq = wave_sum(kqp);
    if (!p.qk_per_key_head && gqa > 1) {                          // the buffered key is the group's first head's
        float ss = 0.0f;
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const int e = l.lane + WAVE * t;
            kxe[t] = e < DK ? load_f(p.k, p.k_dt, int64_t(b) * p.s_k + int64_t(hk * gqa) * DK + e) : 0.0f;
            ss = __builtin_fmaf(kxe[t], kxe[t], ss);
        }
        const float nx = sqrtf(wave_sum(ss) + 1e-6f);
#pragma unroll
        for (int t = 0; t < T::NE; ++t) kxe[t] = kxe[t] / nx;
    }
    float g, beta;
    if (p.gate) {
        const float x = load_f(p.a, p.a_dt, int64_t(b) * p.s_a + h) + load_f(p.dt_bias, p.dt_bias_dt, h);
        const float sp = x <= 20.0f ? logf(1.0f + expf(x)) : x;
        g = -expf(load_f(p.A_log, p.A_log_dt, h)) * sp;
        const float bx = load_f(p.bt, p.bt_dt, int64_t(b) * p.s_bt + h);
        beta = 1.0f / (1.0f + expf(-bx));
    } else {
        g = load_f(p.g, p.g_dt, int64_t(b) * p.s_g + h);
        beta = load_f(p.beta, p.beta_dt, int64_t(b) * p.s_beta + h);
    }
    const float alpha = expf(gcur);
    const float a = expf(g);
    const float gnew = gcur + g;
    __syncthreads();
    float x[2][CPL];
    lds_piece<T>(lds_q, l.cg, x[0]);
    lds_piece<T>(lds_kn, l.cg, x[1]);

    // ---- buffer coefficients: the key buffer as a small tile, slot = row group (+ RG per pass) ----
    float cq[T::MMAX], ck[T::MMAX];
    {
        constexpr int KT = (T::MMAX + T::RG - 1) / T::RG;
        float cq_l[KT], ck_l[KT];
#pragma unroll
        for (int t = 0; t < KT; ++t) {
            const int i = l.rg + T::RG * t;
            float kb[CPL];
#pragma unroll
            for (int c = 0; c < CPL; ++c) kb[c] = 0.0f;
            float dec = 0.0f;
            if (i < m) {
                if (l.cg < T::LPR) {
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
                }
                dec = expf(gcur - GBh[i]);
            }
            float pq = kb[0] * x[0][0], pk = kb[0] * x[1][0];
#pragma unroll
            for (int c = 1; c < CPL; ++c) {
                pq = __builtin_fmaf(kb[c], x[0][c], pq);
                pk = __builtin_fmaf(kb[c], x[1][c], pk);
            }
            pq = block_sum<T::LPRP>(pq);
            pk = block_sum<T::LPRP>(pk);
            const bool alive = i < n;
            cq_l[t] = alive ? dec * pq : 0.0f;
            ck_l[t] = alive ? dec * pk : 0.0f;
            if (full && i < m - 1) {                               // the fold wants the dequantized keys
                float4* d4 = reinterpret_cast<float4*>(lds_k + i * T::KROW + l.cg * T::KPAD);
#pragma unroll
                for (int c = 0; c < CPL / 4; ++c)
                    d4[c] = make_float4(kb[4 * c], kb[4 * c + 1], kb[4 * c + 2], kb[4 * c + 3]);
            }
        }
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            cq[i] = lane_bcast(cq_l[i / T::RG], (i % T::RG) * T::LPRP);
            ck[i] = lane_bcast(ck_l[i / T::RG], (i % T::RG) * T::LPRP);
        }
    }

    // ---- state pass ----
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
            float uv = ub[i][t];
            if constexpr (T::QBUF) uv = uv * lane_bcast(ubs_l, i);
            uv = i < n ? uv : 0.0f;
            sq = __builtin_fmaf(uv, cq[i], sq);
            sk = __builtin_fmaf(uv, ck[i], sk);
        }
        const float vt = valid ? load_f(p.v, p.v_dt, int64_t(b) * p.s_v + int64_t(h) * DV + r) : 0.0f;
        u[t] = beta * __builtin_fmaf(-a, sk, vt);
        const float o = __builtin_fmaf(kq, u[t], a * sq);
        if (valid) store_f(p.out, p.out_dt, obase + r, o);
        else u[t] = 0.0f;
        amax = fmaxf(amax, fabsf(u[t]));
    }

    // ---- append ----
    float us = 1.0f, ks = 1.0f;
    float ur[T::NOWN];                                             // the delta value as stored (dequantized)
    if constexpr (T::QBUF) {
        us = fp16_scale(wave_max(amax), 127.0f);
        float kmax = 0.0f;
#pragma unroll
        for (int t = 0; t < T::NE; ++t) kmax = fmaxf(kmax, fabsf(kxe[t]));
        ks = fp16_scale(wave_max(kmax), 127.0f);
        if (l.lane == 0) UBSh[n] = f32_to_f16(us);
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
    float kr[T::NE];                                               // the key as stored (dequantized)
    const bool first = (h % gqa) == 0;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        if constexpr (T::QBUF) {
            const float c = round_buf(kxe[t], ks);
            kr[t] = c * ks;
            if (first && e < DK) reinterpret_cast<int8_t*>(KBh)[n * DK + e] = int8_t(int(c));
        } else {
            const uint16_t hb = f32_to_bf16(kxe[t]);
            kr[t] = bf16_to_f32(hb);
            if (first && e < DK) reinterpret_cast<uint16_t*>(KBh)[n * DK + e] = hb;
        }
    }
    if (l.lane == 0) {
        GBh[n] = gnew;
        if (T::QBUF && first) KBSh[n] = f32_to_f16(ks);
    }

    // ---- fold ----
    if (full) {
        // decay ratio a_m / a_i per slot (lane i: slot i; the current token's is exp(0) = 1)
        float decf = 1.0f;
        if (l.lane < m - 1) decf = expf(gnew - GBh[l.lane]);
#pragma unroll
        for (int t = 0; t < T::NOWN; ++t) {
            const int r = row_of<T>(l, jown + t);
#pragma unroll
            for (int i = 0; i < T::MMAX; ++i) {
                if (i < m) {
                    float uv = ub[i][t];
                    if constexpr (T::QBUF) uv = uv * lane_bcast(ubs_l, i);
                    if (i == m - 1) uv = ur[t];
                    lds_u[i * T::UROW + r] = lane_bcast(decf, i) * uv;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < T::NE; ++t) {
            const int e = l.lane + WAVE * t;
            if (e < T::LPRP * CPL) lds_k[(m - 1) * T::KROW + kpos<T>(e)] = e < DK ? kr[t] : 0.0f;
        }
        __syncthreads();
        const float alphan = expf(gnew);
        float colmul[CPL];
#pragma unroll
        for (int c = 0; c < CPL; ++c) colmul[c] = alphan;
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
