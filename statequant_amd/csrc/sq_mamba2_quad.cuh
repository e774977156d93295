// Mamba2 / SSD packed decode step, one workgroup per (batch row, GH heads of one B / C group): the heads share C
// (the read-out vector, its digit planes), B (this token's key, its rounded copy for the buffer) and every product
// with the buffered keys; every wavefront owns NB 32-row blocks of one head's state (int4 / int8 codes, key-axis
// scale groups; geometry and building blocks in sq_quad.cuh).
//
// Same arithmetic per head as the one-wavefront kernel of sq_mamba2.cuh (the reference's `_m2_step`,
// /root/reference/src/statequant/kernels/_mamba2_triton.py:48-197):
//   u_n = dt x_n,  y_n = a_n [alpha S0 C + sum_{i<n} (alpha / alpha_i) (B_i . C) u_i] + (B_n . C) u_n + D x_n
//   fold (buffer full): S = alpha_m S0 + sum_i (alpha_m / alpha_i) u_i B_i^T, re-quantized out of LDS
// Division of labour inside the workgroup as in the Gated DeltaNet kernel (sq_gdn_quad.cuh): all loads first, one
// wavefront each for C and B, per head dt and the decays, then per wavefront the state pass, its share of the
// buffered keys, its rows' epilogue, append and fold.
#pragma once
#include "sq_gdn_quad.cuh"

namespace sq {

template <class T, class Q>
struct Mamba2Loads {
    uint16_t sc[Q::NB][T::NG];             // scales of rows (block bi, lane % 32)
    Raw4<T::QBUF> uraw[Q::UT], kraw[Q::KT];
    uint16_t kbs[Q::KT], ubs;
    float gbl, gcur;
    int np;
    uint32_t xr[Q::NE], xr2[Q::NE], g0, g1, g2, g3, vr;
};

// SPEC = 1 compiles the serving case in (as in the Gated DeltaNet kernel): bf16 x / B / C / out, fp32 dt, A, D and
// dt_bias, head counts that are powers of two.  SPEC = 0 reads all of it from the arguments.
template <class T, int NB, int GH, int WPE, int SPEC>
__global__ __launch_bounds__((Quad<T, NB, GH>::THREADS), WPE)
void mamba2_quad_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ order, int per_xcd, int hv, int hv_shift,
                     const uint8_t* codes,
                        uint32_t codes_stride, const int32_t* counters, uint32_t counters_stride, uint32_t start_ramp,
                        const Mamba2Params p) {
    constexpr bool FIX = SPEC > 0;
    const int x_dt = FIX ? int(BF16) : p.x_dt, B_dt = FIX ? int(BF16) : p.B_dt, C_dt = FIX ? int(BF16) : p.C_dt;
    const int out_dt = FIX ? int(BF16) : p.out_dt, dt_dt = FIX ? int(F32) : p.dt_dt, A_dt = FIX ? int(F32) : p.A_dt;
    const int D_dt = FIX ? int(F32) : p.D_dt, dt_bias_dt = FIX ? int(F32) : p.dt_bias_dt;
    using Q = Quad<T, NB, GH>;
    using L = QuadLds<T, NB, GH, 2, 1>;
    constexpr int DK = T::DK, DV = T::DV, NW = Q::NW, NWH = Q::NWH, MM = T::MMAX, NE = Q::NE, NG = T::NG;
    constexpr int RQ = 1 % NW, RK = 3 % NW, RX = 2 % NW;          // which wavefront plays which shared role
    __shared__ __attribute__((aligned(16))) uint8_t lds[L::BYTES];
    uint8_t* lds_kbr = lds + L::KBR;
    float* lds_xn = reinterpret_cast<float*>(lds + L::XN);         // [0]: C, [1]: B
    uint8_t* lds_pl = lds + L::PL;
    float* lds_xs = reinterpret_cast<float*>(lds + L::XS);
    float* lds_dots = reinterpret_cast<float*>(lds + L::DOTS);
    float* lds_kbsf = reinterpret_cast<float*>(lds + L::KBSF);
    float* lds_red = reinterpret_cast<float*>(lds + L::RED);

    const int lane0 = threadIdx.x & (WAVE - 1);
    const int w = __builtin_amdgcn_readfirstlane(int(threadIdx.x) >> 6);
    const int hl = w / NWH, wh = w % NWH;                         // head of the group, wavefront of the head
    const int m = p.m;
    uint8_t* lds_ubr = lds + L::UBR + hl * (MM * DV * T::BE);     // this head's buffered values
    float* lds_ubsf = reinterpret_cast<float*>(lds + L::UBSF) + hl * MM;
    float* lds_scal = reinterpret_cast<float*>(lds + L::SCAL) + hl * 8;
    float* lds_gsc = reinterpret_cast<float*>(lds + L::SCAL) + GH * 8;   // the group's scalars (B . C)
    float* lds_gbf = reinterpret_cast<float*>(lds + L::GBF) + hl * MM;
    uint16_t* lds_sc = reinterpret_cast<uint16_t*>(lds + L::SC) + hl * (DV * NG);
    uint8_t* my_codes = lds + L::CODES + hl * Q::HEAD + wh * NB * Q::BLK;
    static_assert((WAVE / Q::CPR) % (Q::SWD * Q::SWM) == 0 || Q::NLD == 1, "swizzle period");

    // ---- this workgroup's item: (batch row, head group), dealt so that every XCD walks a contiguous range ----
    const int ngrp = hv / GH;
    int b, grp, slot;
    {
        const int wg = blockIdx.x;
        const int item = per_xcd ? (wg & 7) * per_xcd + (wg >> 3) : wg;
        b = (FIX || hv_shift >= 0) ? item >> (hv_shift - ilog2(GH)) : item / ngrp;
        grp = item - b * ngrp;
        if (order) b = order[b];                    // the caller's dispatch order: position -> batch row
        slot = idx ? idx[b] : b;
    }
    const uint32_t h = grp * GH + hl;
    const uint32_t hk = (FIX || p.gqa_shift >= 0) ? h >> p.gqa_shift : h / uint32_t(p.gqa);

    const int lane = lane0;
    const int n32 = lane & 31, kb = lane >> 5;
    // the row of the head this lane finishes after the pass (NB = 2: the wavefront's halves take a block each)
    const int row = (wh * NB + (NB == 2 ? kb : 0)) * T::MR + n32;

    Mamba2Loads<T, Q> F;
    // ---- issue every load: first the token's own operands (their addresses need the batch row only; being older
    //      than the row blocks they are back before them) ...
    if constexpr (RQ == RK) {                                     // a single wavefront carries both vectors
        if (w == RQ) {
            load_vec<NE>(advance(p.C, C_dt, uint64_t(uint32_t(b)) * p.s_C + hk * DK), C_dt, lane, F.xr);
            load_vec<NE>(advance(p.B, B_dt, uint64_t(uint32_t(b)) * p.s_B + hk * DK), B_dt, lane, F.xr2);
        }
    } else if (w == RQ || w == RK) {
        const bool isq = w == RQ;
        const void* base = isq ? advance(p.C, C_dt, uint64_t(uint32_t(b)) * p.s_C + hk * DK)
                               : advance(p.B, B_dt, uint64_t(uint32_t(b)) * p.s_B + hk * DK);
        load_vec<NE>(base, isq ? C_dt : B_dt, lane, F.xr);
    }
    if (wh == 0) {
        F.g0 = load_raw_uniform(p.dt, dt_dt, uint64_t(uint32_t(b)) * p.s_dt + h);
        F.g1 = load_raw_uniform(p.A, A_dt, h);
        F.g2 = load_raw_uniform(p.dt_bias, dt_bias_dt, h);      // absent: the C ABI points them at A, so the loads
        F.g3 = load_raw_uniform(p.D, D_dt, h);                  // need no branch
    }
    F.vr = load_raw(advance(p.x, x_dt, uint64_t(uint32_t(b)) * p.s_x + h * DV), x_dt, uint32_t(row));
    void* const outp = advance(p.out, out_dt, uint64_t(uint32_t(b)) * p.s_out + h * DV);
    if (idx && slot <= 0) {                              // padding row: zero output, touch nothing else
        for (int r = wh * WAVE + lane; r < DV; r += NWH * WAVE) store_f(outp, out_dt, r, 0.0f);
        return;
    }
    // ... then the slot's big side, from the preloaded leading arguments alone: the row blocks, straight into their
    // LDS image, and the fill counter (a scalar load; sq_quad.cuh) behind them ...
    quad_start_wait<Q, WPE>(start_ramp);                  // the launch's first workgroups: spread over a ramp
    quad_dma_blocks<Q, NB>(field(codes, uint32_t(slot), codes_stride, h * (DV * T::ROW_BYTES)) + wh * NB * Q::BLK, my_codes, lane);
    F.np = quad_dma_counter(field(counters, uint32_t(slot), counters_stride, h));
    __builtin_amdgcn_sched_barrier(0);
    // ... and the rest of the slot
    const uint32_t seq = slot, um = m;
    uint8_t* const Sh = field(p.st.S, seq, p.st.sS, h * (DV * T::ROW_BYTES));
    float* const gcp = field(p.st.GCUR, seq, p.st.sGC, h);
    int32_t* const np = field(p.st.NPTR, seq, p.st.sN, h);
    F.gcur = *gcp;
    uint16_t* const SCh = field(p.st.SC, seq, p.st.sSC, h * T::SC_ELEMS);
    uint8_t* const KBp = p.st.KB + (uint64_t(seq) * p.st.sKB + hk * um * DK) * T::BE;
    uint8_t* const UBp = p.st.UB + (uint64_t(seq) * p.st.sUB + h * um * DV) * T::BE;
    uint16_t* const KBSp = field(p.st.KBS, seq, p.st.sKBS, hk * um);
    uint16_t* const UBSp = field(p.st.UBS, seq, p.st.sUBS, h * um);
    float* const GBh = field(p.st.GB, seq, p.st.sGB, h * um);
#pragma unroll
    for (int bi = 0; bi < NB; ++bi)
#pragma unroll
        for (int g = 0; g < NG; ++g) F.sc[bi][g] = stream_load(SCh + uint32_t(((wh * NB + bi) * T::MR + n32) * NG + g));
    // the buffer, live slots only (the others repeat the last live one: no new memory traffic); the fill count,
    // requested ahead of the row blocks, is here by now
    quad_dma_counter_wait(F.np);
    const uint32_t nfill = uint32_t(F.np & (m - 1));
    const uint32_t nl = nfill > 0 ? nfill : 1u;
    // buffered values of this wavefront's rows: lane (slot = lane / LU + SU t, rows 4 (lane % LU) ..)
#pragma unroll
    for (int t = 0; t < Q::UT; ++t) {
        const uint32_t i = lane / Q::LU + Q::SU * t;
        const uint32_t ic = i < nl ? i : nl - 1;
        F.uraw[t] = stream_raw4<T::QBUF>(UBp + (ic * DV + wh * Q::RW + 4 * (lane % Q::LU)) * T::BE);
    }
    // buffered keys, dealt over the workgroup: lane (slot = SPP (NW t + w) + lane / LPS, columns 4 (lane % LPS) ..)
#pragma unroll
    for (int t = 0; t < Q::KT; ++t) {
        const uint32_t i = Q::SPP * (NW * t + w) + lane / Q::LPS;
        const uint32_t ic = i < nl ? i : nl - 1;
        F.kraw[t] = stream_raw4<T::QBUF>(KBp + (ic * DK + 4 * (lane % Q::LPS)) * T::BE);
        F.kbs[t] = T::QBUF ? KBSp[ic] : uint16_t(0);
    }
    {   // per slot of this head, lane i: cumulative decay and value scale
        const uint32_t li = uint32_t(lane) < nl ? lane : 0;
        F.gbl = GBh[li];
        F.ubs = T::QBUF ? UBSp[li] : uint16_t(0);
    }
    // every load is in flight from here on: keep the compiler from sinking any of them to its use, and from
    // scheduling a use (a conversion, with its wait) up among them
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    // ---- shared roles: C (planes + fp32 copy), B (fp32 copy) ----
    auto role_vector = [&](const uint32_t (&raw)[NE], int dt, int v) {
        float xe[NE];
#pragma unroll
        for (int t = 0; t < NE; ++t) xe[t] = vec_elem<NE>(raw, dt, t);
        if constexpr (NE == 1) lds_xn[v * DK + lane] = xe[0];
        else if constexpr (NE == 2) *reinterpret_cast<float2*>(lds_xn + v * DK + 2 * lane) = make_float2(xe[0], xe[1]);
        else *reinterpret_cast<float4*>(lds_xn + v * DK + 4 * lane) = make_float4(xe[0], xe[1], xe[2], xe[3]);
        if (v == 0) quad_stage_planes<T, NE>(xe, 0, lane, lds_pl, lds_xs);
    };
    if constexpr (RQ == RK) {
        if (w == RQ) {
            role_vector(F.xr, C_dt, 0);
            role_vector(F.xr2, B_dt, 1);
        }
    } else {
        if (w == RQ) role_vector(F.xr, C_dt, 0);
        if (w == RK) role_vector(F.xr, B_dt, 1);
    }
    if (wh == 0) {                                       // this head's step size and decays
        float dt = raw_to_f(F.g0, dt_dt);
        if (p.has_dt_bias) dt = dt + raw_to_f(F.g2, dt_bias_dt);
        if (p.dt_softplus) dt = dt <= 20.0f ? logf(1.0f + expf(dt)) : dt;
        if (p.dt_clamp) dt = fminf(fmaxf(dt, p.dt_min), p.dt_max);
        const float g = raw_to_f(F.g1, A_dt) * dt;     // rounded on its own (no contraction into gcur + g)
        if (lane == 0) {
            lds_scal[0] = dt;
            lds_scal[1] = expf(F.gcur);
            lds_scal[2] = expf(g);
            lds_scal[3] = F.gcur + g;
            lds_scal[4] = p.has_D ? raw_to_f(F.g3, D_dt) : 0.0f;
        }
    }
    // ---- the loads land: LDS images of the row blocks, scales, raw buffer pieces ----
    const int n = F.np & (m - 1);
    const float gcur = F.gcur;
    const uint32_t vr = F.vr;
    uint16_t scw[NB][NG];
#pragma unroll
    for (int bi = 0; bi < NB; ++bi)
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            scw[bi][g] = F.sc[bi][g];
            if (kb == 0) lds_sc[((wh * NB + bi) * T::MR + n32) * NG + g] = F.sc[bi][g];
        }
#pragma unroll
    for (int t = 0; t < Q::UT; ++t) {
        const int i = lane / Q::LU + Q::SU * t;
        if (i < m) store_raw4<T::QBUF>(lds_ubr + (i * DV + wh * Q::RW + 4 * (lane % Q::LU)) * T::BE, F.uraw[t]);
    }
#pragma unroll
    for (int t = 0; t < Q::KT; ++t) {
        const int i = Q::SPP * (NW * t + w) + lane / Q::LPS;
        if (i < m) {
            store_raw4<T::QBUF>(lds_kbr + (i * DK + 4 * (lane % Q::LPS)) * T::BE, F.kraw[t]);
            if (T::QBUF && lane % Q::LPS == 0) lds_kbsf[i] = f16_to_f32(F.kbs[t]);
        }
    }
    if (wh == 0 && lane < m) {
        lds_gbf[lane] = F.gbl;
        if constexpr (T::QBUF) lds_ubsf[lane] = f16_to_f32(F.ubs);
    }
    quad_dma_landed();                                             // the row blocks are in LDS
    const bool full = n == m - 1;
    lds_barrier();

    // ---- every wavefront: state pass over its row blocks (one read-out vector: the lanes of the upper half idle) ----
    float sq;                                            // (S0 C)[row], scales applied
    {
        v4i aop[T::NKS];
        quad_fetch_planes<T, 1>(lds_pl, lane, aop);
        float xs[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) xs[g] = lds_xs[g];
        float own[NB];
#pragma unroll
        for (int bi = 0; bi < NB; ++bi) {
            float sc[NG];
#pragma unroll
            for (int g = 0; g < NG; ++g) sc[g] = f16_to_f32(scw[bi][g]);
            own[bi] = quad_block_pass<Q, T>(my_codes + bi * Q::BLK, aop, xs, sc, lane);
        }
        if constexpr (NB == 2) {                         // lane (n, kb) takes over row n of block kb
            const auto r = __builtin_amdgcn_permlane32_swap(as_u32(own[0]), as_u32(own[1]), false, false);
            sq = as_f32(r[0]);
        } else {
            sq = pair32(own[0]).lo;
        }
    }
    // ---- B_i . C of this wavefront's share of the slots ----
    {
        float x[4];
        {
            const float4 f = *reinterpret_cast<const float4*>(lds_xn + 4 * (lane % Q::LPS));
            x[0] = f.x; x[1] = f.y; x[2] = f.z; x[3] = f.w;
        }
#pragma unroll
        for (int t = 0; t < Q::KT; ++t) {
            const int i = Q::SPP * (NW * t + w) + lane / Q::LPS;
            const int ic = i < m ? i : m - 1;
            float kf[4];
            decode_raw4<T::QBUF>(load_raw4<T::QBUF>(lds_kbr + (ic * DK + 4 * (lane % Q::LPS)) * T::BE), kf);
            if constexpr (T::QBUF) {
                const float s = lds_kbsf[ic];
#pragma unroll
                for (int c = 0; c < 4; ++c) kf[c] = kf[c] * s;
            }
            float pr = kf[0] * x[0];
#pragma unroll
            for (int c = 1; c < 4; ++c) pr = __builtin_fmaf(kf[c], x[c], pr);
            pr = lanes_sum<Q::LPS>(pr);
            if (lane % Q::LPS == 0 && i < MM) lds_dots[i] = pr;
        }
    }
    // ---- B . C ----
    if (w == RK) {
        float bcp = 0.0f;
#pragma unroll
        for (int t = 0; t < NE; ++t) bcp = __builtin_fmaf(lds_xn[DK + NE * lane + t], lds_xn[NE * lane + t], bcp);
        bcp = lanes_sum<WAVE>(bcp);
        if (lane == 0) lds_gsc[0] = bcp;
    }
    lds_barrier();                                       // the raw keys of slot n may be overwritten from here on

    // ---- the buffered key of this token: the rounded B, for this workgroup's folds and (first head group of the
    //      B / C group only) for the slot ----
    if (w == RX) {
        float kxe[NE], kmax = 0.0f;
#pragma unroll
        for (int t = 0; t < NE; ++t) {
            kxe[t] = lds_xn[DK + NE * lane + t];
            kmax = fmaxf(kmax, fabsf(kxe[t]));
        }
        float ks = 1.0f;
        if constexpr (T::QBUF) ks = fp16_scale(lanes_max<WAVE>(kmax), 127.0f);
        const bool write = h - hl == hk * uint32_t(p.gqa);
        if (T::QBUF && lane == 0) {
            lds_kbsf[n] = ks;
            if (write) KBSp[n] = f32_to_f16(ks);
        }
        if constexpr (T::QBUF) {
            uint32_t pk = 0;
#pragma unroll
            for (int t = 0; t < NE; ++t) pk |= (uint32_t(int(round_buf(kxe[t], ks))) & 0xFFu) << (8 * t);
            uint8_t* dl = lds_kbr + n * DK + NE * lane;
            uint8_t* dg = KBp + n * DK + NE * lane;
            if constexpr (NE == 1) { *dl = uint8_t(pk); if (write) *dg = uint8_t(pk); }
            else if constexpr (NE == 2) {
                *reinterpret_cast<uint16_t*>(dl) = uint16_t(pk);
                if (write) *reinterpret_cast<uint16_t*>(dg) = uint16_t(pk);
            } else {
                *reinterpret_cast<uint32_t*>(dl) = pk;
                if (write) *reinterpret_cast<uint32_t*>(dg) = pk;
            }
        } else {
#pragma unroll
            for (int t = 0; t < NE; ++t) {
                const uint16_t hb = f32_to_bf16(kxe[t]);
                reinterpret_cast<uint16_t*>(lds_kbr)[n * DK + NE * lane + t] = hb;
                if (write) reinterpret_cast<uint16_t*>(KBp)[n * DK + NE * lane + t] = hb;
            }
        }
    }

    // ---- this wavefront's rows: buffer term, u, y ----
    const float dt = lds_scal[0], alpha = lds_scal[1], a = lds_scal[2], gnew = lds_scal[3], dd = lds_scal[4];
    const float bc = lds_gsc[0];
    // coefficients of the head's slots, lane i: c[i] = exp(gcur - G_i) (B_i . C), times the slot's value scale; dead
    // slots (i >= n) may hold anything: select, never multiply
    const int li = lane < m ? lane : 0;
    float cq;
    {
        const float dec = expf(gcur - lds_gbf[li]);
        const float dq = lds_dots[li];
        const float us_i = T::QBUF ? lds_ubsf[li] : 1.0f;
        cq = lane < n ? (T::QBUF ? (dec * dq) * us_i : dec * dq) : 0.0f;
    }
    float uv[MM];
#pragma unroll
    for (int i = 0; i < MM; ++i) uv[i] = lds_raw<T::QBUF>(lds_ubr, (i < m ? i : 0) * DV + row);
    float accq = alpha * sq;
#pragma unroll
    for (int i = 0; i < MM; ++i) {
        const float u_i = T::QBUF ? uv[i] : (i < n ? uv[i] : 0.0f);
        accq = __builtin_fmaf(u_i, lane_bcast(cq, i), accq);
    }
    const float xt = raw_to_f(vr, x_dt);
    const float u = dt * xt;
    float y = __builtin_fmaf(bc, u, a * accq);
    if (p.has_D) y = __builtin_fmaf(dd, xt, y);
    if (NB == 2 || kb == 0) store_f(outp, out_dt, row, y);

    // ---- append ----
    float us = 1.0f;
    if constexpr (T::QBUF) {
        float amax = lanes_max<WAVE>(fabsf(u));
        if constexpr (NWH > 1) {
            if (lane == 0) lds_red[w] = amax;
            lds_barrier();
#pragma unroll
            for (int ww = 0; ww < NWH; ++ww) amax = fmaxf(amax, lds_red[hl * NWH + ww]);
        }
        us = fp16_scale(amax, 127.0f);
        if (wh == 0 && lane == 0) { UBSp[n] = f32_to_f16(us); lds_ubsf[n] = us; }
    }
    if (NB == 2 || kb == 0) {
        if constexpr (T::QBUF) {
            const int8_t c = int8_t(int(round_buf(u, us)));
            reinterpret_cast<int8_t*>(UBp)[n * DV + row] = c;
            reinterpret_cast<int8_t*>(lds_ubr)[n * DV + row] = c;
        } else {
            const uint16_t hb = f32_to_bf16(u);
            reinterpret_cast<uint16_t*>(UBp)[n * DV + row] = hb;
            reinterpret_cast<uint16_t*>(lds_ubr)[n * DV + row] = hb;
        }
    }
    if (wh == 0 && lane == 0) {
        GBh[n] = gnew;
        *gcp = full ? 0.0f : gnew;                       // advance
        *np = full ? 0 : n + 1;
    }

    // ---- fold ----
    if (full) {
        lds_barrier();                                   // `full` is the same in every head of a slot
        constexpr int MT4 = (MM + 3) / 4, CL = DK / 4;
        // lane offsets derived anew (from a copy of the lane id the compiler cannot trace back), so that the ones
        // formed at the top of the kernel are not kept in registers all the way to here
        int lf = lane;
        asm volatile("" : "+v"(lf));
        const int fn = lf & 15, fq = lf >> 4;
        const int swzf = swz<Q>(lf / Q::CPR, lf % Q::CPR);
        float decf[MT4];                                 // decay ratios a_m / a_i of the lane's slots 4 t + q
#pragma unroll
        for (int t = 0; t < MT4; ++t) {
            const int sl = 4 * t + fq;
            decf[t] = sl < m - 1 ? expf(gnew - lds_gbf[sl < m - 1 ? sl : 0]) : 1.0f;
        }
        const float cmul = expf(gnew);
        const int fg = (fq * CL) / T::KGROUP;
        FoldKeys<T> kop;
        quad_fold_keys<T>(lds_kbr, lds_kbsf, m, lf, kop);
#pragma unroll
        for (int bi = 0; bi < NB; ++bi) {
            uint8_t* blk = my_codes + bi * Q::BLK;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int frow = (wh * NB + bi) * T::MR + 16 * hf + fn;
                float bop[MT4];
#pragma unroll
                for (int t = 0; t < MT4; ++t) {
                    const int sl = 4 * t + fq;
                    const int sc_ = sl < m ? sl : 0;
                    float fv = lds_raw<T::QBUF>(lds_ubr, sc_ * DV + frow);
                    if constexpr (T::QBUF) fv = fv * lds_ubsf[sc_];
                    fv = decf[t] * fv;
                    bop[t] = sl < m ? fv : 0.0f;
                }
                quad_fold_half<Q, T>(blk, hf, kop, bop, cmul, f16_to_f32(lds_sc[frow * NG + fg]),
                                            SCh + frow * NG + fg, lf);
            }
            wave_sync();
#pragma unroll
            for (int t = 0; t < Q::NLD; ++t)
                stream_store(reinterpret_cast<v4u*>(Sh + (wh * NB + bi) * Q::BLK + t * 1024 + lf * 16),
                             *reinterpret_cast<const v4u*>(blk + t * 1024 + swzf));
        }
    }
}

template <class T, int NB, int GH, int WPE, int SPEC>
int launch_mamba2_quad(const Mamba2Params& p0, hipStream_t stream) {
    Mamba2Params p = p0;
    p.per_xcd = (p.per_xcd % GH == 0) ? p.per_xcd / GH : 0;          // dealing over head groups
    const uint32_t grid = uint32_t(p.rows) * uint32_t(p.hv / GH);
    hipLaunchKernelGGL((mamba2_quad_kernel<T, NB, GH, WPE, SPEC>), dim3(grid), dim3(Quad<T, NB, GH>::THREADS),
                       quad_lds_pad(), stream, p.idx, p.order, p.per_xcd, p.hv, p.hv_shift, p.st.S, p.st.sS, p.st.NPTR, p.st.sN,
                       quad_start_ramp<Quad<T, NB, GH>, WPE>(grid, 24), p);
    return int(hipGetLastError());
}

}  // namespace sq
