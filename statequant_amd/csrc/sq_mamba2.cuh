// Mamba2 / SSD packed decode step: one launch, one wavefront per (batch row, head).
//
// Replaces the reference's `_m2_step` (/root/reference/src/statequant/kernels/_mamba2_triton.py:48-197): key = B of
// the head's group (shared like a GQA key), query = C, buffered value u = dt x, scalar decay exp(A dt); no delta
// term, no normalisation:
//   y_n = a_n [alpha S0 C + sum_{i<n} (alpha/alpha_i) (B_i.C) u_i] + (B_n.C) u_n + D x_n
//   fold (buffer full): S = alpha_m S0 + sum_i (alpha_m/alpha_i) u_i B_i^T, re-quantized in place
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

template <class T>
__global__ __launch_bounds__(WAVE) void mamba2_step_kernel(const Mamba2Params p) {
    __shared__ __attribute__((aligned(16))) float lds[T::LDS_FLOATS];
    float* lds_k = lds;
    float* lds_u = lds + T::MMAX * T::KROW;
    float* lds_c = lds_u + T::MMAX * T::UROW;

    const LaneId l = lane_id<T>();
    const int tile = xcd_tile(blockIdx.x, gridDim.x);
    const int b = tile / p.hv;
    const int h = tile - b * p.hv;
    const int gqa = p.hv / p.hk;
    const int hk = h / gqa;
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

    // ---- prep: B, C of the group, dt, decay ----
    float ce[T::NE], kxe[T::NE];
    float bcp = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NE; ++t) {
        const int e = l.lane + WAVE * t;
        ce[t] = e < DK ? load_f(p.C, p.C_dt, int64_t(b) * p.s_C + int64_t(hk) * DK + e) : 0.0f;
        kxe[t] = e < DK ? load_f(p.B, p.B_dt, int64_t(b) * p.s_B + int64_t(hk) * DK + e) : 0.0f;
        bcp = __builtin_fmaf(kxe[t], ce[t], bcp);
        if (e < T::LPRP * CPL) lds_c[kpos<T>(e)] = ce[t];
    }
    const float bc = wave_sum(bcp);
    float dt = load_f(p.dt, p.dt_dt, int64_t(b) * p.s_dt + h);
    if (p.dt_bias) dt = dt + load_f(p.dt_bias, p.dt_bias_dt, h);
    if (p.dt_softplus) dt = dt <= 20.0f ? logf(1.0f + expf(dt)) : dt;
    if (p.dt_clamp) dt = fminf(fmaxf(dt, p.dt_min), p.dt_max);
    const float g = load_f(p.A, p.A_dt, h) * dt;                 // rounded on its own (no contraction into gcur + g)
    const float a = expf(g);
    const float dd = p.D ? load_f(p.D, p.D_dt, h) : 0.0f;
    const float alpha = expf(gcur);
    const float gnew = gcur + g;
    __syncthreads();
    float x[1][CPL];
    lds_piece<T>(lds_c, l.cg, x[0]);

    // ---- buffer coefficients c[i] = (alpha / alpha_i) B_i . C ----
    float cq[T::MMAX];
    {
        constexpr int KT = (T::MMAX + T::RG - 1) / T::RG;
        float cq_l[KT];
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
            float pq = kb[0] * x[0][0];
#pragma unroll
            for (int c = 1; c < CPL; ++c) pq = __builtin_fmaf(kb[c], x[0][c], pq);
            pq = block_sum<T::LPRP>(pq);
            cq_l[t] = i < n ? dec * pq : 0.0f;
            if (full && i < m - 1) {
                float4* d4 = reinterpret_cast<float4*>(lds_k + i * T::KROW + l.cg * T::KPAD);
#pragma unroll
                for (int c = 0; c < CPL / 4; ++c)
                    d4[c] = make_float4(kb[4 * c], kb[4 * c + 1], kb[4 * c + 2], kb[4 * c + 3]);
            }
        }
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) cq[i] = lane_bcast(cq_l[i / T::RG], (i % T::RG) * T::LPRP);
    }

    // ---- state pass ----
    float part[1][T::RPLP];
    tile_dots<T, 1>(raw, x, part);
    float own[1][T::NOWN];
    reduce_rows<T, 1>(part, sc, l, own);

    // ---- owned rows: y, and the value to buffer ----
    float u[T::NOWN], amax = 0.0f;
#pragma unroll
    for (int t = 0; t < T::NOWN; ++t) {
        const int r = row_of<T>(l, jown + t);
        const bool valid = jown + t < T::RPL;
        float sq = alpha * own[0][t];
#pragma unroll
        for (int i = 0; i < T::MMAX; ++i) {
            float uv = ub[i][t];
            if constexpr (T::QBUF) uv = uv * lane_bcast(ubs_l, i);
            uv = i < n ? uv : 0.0f;
            sq = __builtin_fmaf(uv, cq[i], sq);
        }
        const float xr = valid ? load_f(p.x, p.x_dt, int64_t(b) * p.s_x + int64_t(h) * DV + r) : 0.0f;
        u[t] = dt * xr;
        float y = __builtin_fmaf(bc, u[t], a * sq);
        if (p.D) y = __builtin_fmaf(dd, xr, y);
        if (valid) store_f(p.out, p.out_dt, obase + r, y);
        amax = fmaxf(amax, fabsf(u[t]));
    }

    // ---- append ----
    float us = 1.0f, ks = 1.0f;
    float ur[T::NOWN];
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
    float kr[T::NE];
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

    if (l.lane == 0) {
        *gcp = full ? 0.0f : gnew;
        *np = full ? 0 : n + 1;
    }
}

template <class T>
int launch_mamba2(const Mamba2Params& p, hipStream_t stream) {
    hipLaunchKernelGGL(mamba2_step_kernel<T>, dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p);
    return int(hipGetLastError());
}

}  // namespace sq
