// Gated DeltaNet packed decode step, one workgroup per (batch row, key head): the GH value heads of the key head
// share q, k, the buffered keys and everything computed from them; every wavefront owns NB 32-row blocks of one
// value head's state (int4 / int8 codes, key-axis scale groups; geometry and building blocks in sq_quad.cuh).
//
// Same arithmetic per head as the one-wavefront kernel of sq_gdn.cuh (the reference's fused Triton step,
// /root/reference/src/statequant/kernels/_fused_triton.py:48-190).  Division of labour inside the workgroup:
//   issue            every wavefront: its row blocks, their scales, its rows of v and of the buffered values, its
//                    share of the buffered keys, its head's decays and counters -- all in flight before any is used
//   roles            one wavefront each: q (l2 norm, scale, digit planes);  k (l2 norm, digit planes);  per head the
//                    gates and decays;  then everything lands in LDS                                       [barrier]
//   per wavefront    its row blocks' S0 q, S0 k on the matrix core;  K_i . q, K_i . k of its share of the slots;
//                    one wavefront: k . q and this token's buffered key                                    [barrier]
//                    buffer term, u, o for its rows;  max |u| of the head                                  [barrier]
//                    append;  with a full buffer: fold of its row blocks out of LDS, stored back           [barrier]
// Requires q and k given per key head (or one value head per key head): with per-value-head q / k and grouped keys
// the one-wavefront kernel runs instead.
#pragma once
#include "sq_gdn.cuh"
#include "sq_quad.cuh"
#include "sq_timeline.cuh"

namespace sq {

// NE consecutive elements of a float vector of run-time dtype, one load per lane, kept AS LOADED: w holds the
// lane's NE fp32 words, or its NE 16-bit patterns packed two per word (NE = 1: the pattern itself).  Nothing is
// computed from the loaded words here -- not even the split of a packed pair -- because any use would make the
// wavefront wait for this load before it has issued the ones behind it; `vec_elem` unpacks at the point of use.
// The vector's base must be 16-byte aligned.
template <int NE>
__device__ __forceinline__ void load_vec(const void* base, int dt, int lane, uint32_t (&w)[NE]) {
    if (dt == F32) {
        if constexpr (NE == 1) w[0] = reinterpret_cast<const uint32_t*>(base)[lane];
        else if constexpr (NE == 2) {
            const v2u x = reinterpret_cast<const v2u*>(base)[lane];
            w[0] = x.x; w[1] = x.y;
        } else {
            const v4u x = reinterpret_cast<const v4u*>(base)[lane];
            w[0] = x.x; w[1] = x.y; w[2] = x.z; w[3] = x.w;
        }
    } else {
        if constexpr (NE == 1) w[0] = reinterpret_cast<const uint16_t*>(base)[lane];
        else if constexpr (NE == 2) {
            w[0] = reinterpret_cast<const uint32_t*>(base)[lane];
            w[1] = 0;
        } else {
            const v2u x = reinterpret_cast<const v2u*>(base)[lane];
            w[0] = x.x; w[1] = x.y; w[2] = 0; w[3] = 0;
        }
    }
}
// Element t of what `load_vec` loaded, as fp32.
template <int NE>
__device__ __forceinline__ float vec_elem(const uint32_t (&w)[NE], int dt, int t) {
    if (dt == F32) return as_f32(w[t]);
    const uint32_t h = NE == 1 ? w[0] : (w[t / 2] >> (16 * (t % 2))) & 0xFFFFu;
    return raw_to_f(h, dt);
}

// Everything a wavefront loads for one item, as issued loads (raw bits; nothing here waits for memory).
template <class T, class Q>
struct GdnLoads {
    uint16_t sc[Q::NB][T::NG];             // scales of rows (block bi, lane % 32)
    Raw4<T::QBUF> uraw[Q::UT], kraw[Q::KT];
    uint16_t kbs[Q::KT], ubs;
    float gbl, gcur;
    int np;
    uint32_t xr[Q::NE], xr2[Q::NE], g0, g1, g2, g3, vr;
};

// SPEC > 0 compiles the serving cases in, so that dtypes and options cost no scalar branches on the way to the first
// load (measured on the 128 x 128 int8 step: 35.4 -> 34.2 us per launch): bf16 q / k / v / out,
// head counts that are powers of two, and  1: g and beta given as fp32;  2: the gate formed in the kernel from bf16
// a, b and fp32 A_log, dt_bias.  SPEC = 0 reads all of it from the arguments.
template <class T, int NB, int GH, int WPE, int SPEC>
__global__ __launch_bounds__((Quad<T, NB, GH>::THREADS), WPE)
void gdn_quad_kernel(const int32_t* __restrict__ idx, const int32_t* __restrict__ order, int per_xcd, int hv, int hv_shift,
                     const uint8_t* codes,
                     uint32_t codes_stride, const int32_t* counters, uint32_t counters_stride, uint32_t start_ramp,
                     SQ_TL_PARAM const GdnParams p) {
    SQ_MARK(0);                                                   // entry
    // the leading arguments (copies of fields of `p`) are what the slot index load, the fill counter and the row blocks
    // need: as separate scalar arguments they are preloaded into registers at wave launch, so those requests go out
    // without waiting for the argument block
    constexpr bool FIX = SPEC > 0;
    const int q_dt = FIX ? int(BF16) : p.q_dt, k_dt = FIX ? int(BF16) : p.k_dt, v_dt = FIX ? int(BF16) : p.v_dt;
    const int out_dt = FIX ? int(BF16) : p.out_dt;
    const int a_dt = SPEC == 1 ? int(F32) : SPEC == 2 ? int(BF16) : p.a_dt;
    const int bt_dt = SPEC == 1 ? int(F32) : SPEC == 2 ? int(BF16) : p.bt_dt;
    const int A_log_dt = FIX ? int(F32) : p.A_log_dt, dt_bias_dt = FIX ? int(F32) : p.dt_bias_dt;
    const bool gate = SPEC == 1 ? false : SPEC == 2 ? true : p.gate != 0;
    using Q = Quad<T, NB, GH>;
    using L = QuadLds<T, NB, GH, 2, 2>;
    constexpr int DK = T::DK, DV = T::DV, NW = Q::NW, NWH = Q::NWH, MM = T::MMAX, NE = Q::NE, NG = T::NG;
    constexpr int RQ = 1 % NW, RK = 3 % NW, RX = 2 % NW;          // which wavefront plays which shared role
    __shared__ __attribute__((aligned(16))) uint8_t lds[L::BYTES];
    uint8_t* lds_kbr = lds + L::KBR;
    float* lds_xn = reinterpret_cast<float*>(lds + L::XN);
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
    float* lds_gsc = reinterpret_cast<float*>(lds + L::SCAL) + GH * 8;   // the group's scalars (k . q)
    float* lds_gbf = reinterpret_cast<float*>(lds + L::GBF) + hl * MM;
    uint16_t* lds_sc = reinterpret_cast<uint16_t*>(lds + L::SC) + hl * (DV * NG);
    uint8_t* my_codes = lds + L::CODES + hl * Q::HEAD + wh * NB * Q::BLK;
    static_assert((WAVE / Q::CPR) % (Q::SWD * Q::SWM) == 0 || Q::NLD == 1, "swizzle period");

    // ---- this workgroup's item: (batch row, head group), dealt so that every XCD walks a contiguous range ----
    const int ngrp = hv / GH;                                     // head groups per batch row
    TileId tid;
    int32_t slot;
    {
        const int wg = blockIdx.x;
        const int item = per_xcd ? (wg & 7) * per_xcd + (wg >> 3) : wg;
        tid.b = (FIX || hv_shift >= 0) ? item >> (hv_shift - ilog2(GH)) : item / ngrp;
        tid.h = (item - tid.b * ngrp) * GH + hl;
        if (order) tid.b = order[tid.b];            // the caller's dispatch order: position -> batch row
        SQ_MARK(1);                                               // item known (the leading arguments are here)
        slot = idx ? idx[tid.b] : tid.b;
        tid.hk = (FIX || p.gqa_shift >= 0) ? tid.h >> p.gqa_shift : tid.h / p.gqa;
    }
    const int lane = lane0;
    const int n32 = lane & 31, kb = lane >> 5;
    // the row of the head this lane finishes after the pass (NB = 2: the wavefront's halves take a block each)
    const int row = (wh * NB + (NB == 2 ? kb : 0)) * T::MR + n32;

    GdnLoads<T, Q> F;
    // ---- issue every load: first the token's own operands (their addresses need the batch row only: they go out
    //      while the slot index is on its way, and being older than the row blocks they are back before them) ...
    {
        const uint32_t b = tid.b, h = tid.h;
        if constexpr (RQ == RK) {                                 // a single wavefront carries both vectors
            if (w == RQ) {
                load_vec<NE>(advance(p.q, q_dt, uint64_t(b) * p.s_q + uint32_t(tid.hk) * DK), q_dt, lane, F.xr);
                load_vec<NE>(advance(p.k, k_dt, uint64_t(b) * p.s_k + uint32_t(tid.hk) * DK), k_dt, lane, F.xr2);
            }
        } else if (w == RQ || w == RK) {
            const bool isq = w == RQ;
            const void* base = isq ? advance(p.q, q_dt, uint64_t(b) * p.s_q + uint32_t(tid.hk) * DK)
                                   : advance(p.k, k_dt, uint64_t(b) * p.s_k + uint32_t(tid.hk) * DK);
            load_vec<NE>(base, isq ? q_dt : k_dt, lane, F.xr);
        }
        if (wh == 0) {
            F.g0 = load_raw_uniform(p.a, a_dt, uint64_t(b) * p.s_a + h);
            F.g1 = load_raw_uniform(p.bt, bt_dt, uint64_t(b) * p.s_bt + h);
            if constexpr (SPEC != 1) {                            // without a gate they alias g (readable, unused)
                F.g2 = load_raw_uniform(p.A_log, A_log_dt, h);
                F.g3 = load_raw_uniform(p.dt_bias, dt_bias_dt, h);
            } else {
                F.g2 = F.g3 = 0;
            }
        }
        F.vr = load_raw(advance(p.v, v_dt, uint64_t(b) * p.s_v + h * DV), v_dt, uint32_t(row));
    }
    if (idx && slot <= 0) {                              // padding row: zero output, touch nothing of a slot
        void* const o0 = advance(p.out, out_dt, (uint64_t(uint32_t(tid.b)) * uint32_t(p.hv) + uint32_t(tid.h)) * DV);
        for (int r = wh * WAVE + lane; r < DV; r += NWH * WAVE) store_f(o0, out_dt, r, 0.0f);
        return;
    }
    SQ_MARK(2);                                                   // slot known, the token's loads issued
    // ... then the slot's big side, from the preloaded arguments alone: the row blocks, straight into their LDS image,
    // and the fill counter (a scalar load; sq_quad.cuh) -- behind the row blocks, because the first wait for any
    // scalar load, the argument block's included, waits for it as well ...
    quad_start_wait<Q, WPE>(start_ramp);                  // the launch's first workgroups: spread over a ramp
    quad_dma_blocks<Q, NB>(field(codes, uint32_t(slot), codes_stride, uint32_t(tid.h) * (DV * T::ROW_BYTES)) + wh * NB * Q::BLK,
                           my_codes, lane);
    SQ_MARK(3);                                                   // row blocks issued
    F.np = quad_dma_counter(field(counters, uint32_t(slot), counters_stride, uint32_t(tid.h)));
    __builtin_amdgcn_sched_barrier(0);
    SQ_MARK(4);                                                   // counter issued
    // ... and the rest of the slot: running decay, scales, and -- once the fill counter is here -- the live part of
    // the decode buffer
    const GdnAddr<T> A = gdn_addr<T>(p, tid, slot);
    void* const outp = advance(p.out, out_dt, A.obase);
    F.gcur = *A.gcp;
    {
#pragma unroll
        for (int bi = 0; bi < NB; ++bi)
#pragma unroll
            for (int g = 0; g < NG; ++g) F.sc[bi][g] = stream_load(A.SCh + uint32_t(((wh * NB + bi) * T::MR + n32) * NG + g));
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
            F.uraw[t] = stream_raw4<T::QBUF>(A.buf.UB + (ic * DV + wh * Q::RW + 4 * (lane % Q::LU)) * T::BE);
        }
        // buffered keys, dealt over the workgroup: lane (slot = SPP (NW t + w) + lane / LPS, columns 4 (lane % LPS) ..)
#pragma unroll
        for (int t = 0; t < Q::KT; ++t) {
            const uint32_t i = Q::SPP * (NW * t + w) + lane / Q::LPS;
            const uint32_t ic = i < nl ? i : nl - 1;
            F.kraw[t] = stream_raw4<T::QBUF>(A.buf.KB + (ic * DK + 4 * (lane % Q::LPS)) * T::BE);
            F.kbs[t] = T::QBUF ? A.buf.KBS[ic] : uint16_t(0);
        }
        // per slot of this head, lane i: cumulative decay and value scale
        const uint32_t li = uint32_t(lane) < nl ? lane : 0;
        F.gbl = A.GBh[li];
        F.ubs = T::QBUF ? A.buf.UBS[li] : uint16_t(0);
    }
    // every load of the item is in flight from here on: keep the compiler from sinking any of them to its use, and
    // from scheduling a use (a conversion, with its wait) up among them
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    SQ_MARK(5);                                                   // fill count here, buffer loads issued

    // ---- shared roles (their inputs were issued first) ----
    auto role_vector = [&](const uint32_t (&raw)[NE], int dt, float post, int v) {
        float xe[NE], ss = 0.0f;
#pragma unroll
        for (int t = 0; t < NE; ++t) {
            xe[t] = vec_elem<NE>(raw, dt, t);
            ss = __builtin_fmaf(xe[t], xe[t], ss);
        }
        const float nrm = sqrtf(lanes_sum<WAVE>(ss) + 1e-6f);
#pragma unroll
        for (int t = 0; t < NE; ++t) xe[t] = xe[t] / nrm * post;
        if constexpr (NE == 1) lds_xn[v * DK + lane] = xe[0];
        else if constexpr (NE == 2) *reinterpret_cast<float2*>(lds_xn + v * DK + 2 * lane) = make_float2(xe[0], xe[1]);
        else *reinterpret_cast<float4*>(lds_xn + v * DK + 4 * lane) = make_float4(xe[0], xe[1], xe[2], xe[3]);
        quad_stage_planes<T, NE>(xe, v, lane, lds_pl, lds_xs);
    };
    if constexpr (RQ == RK) {
        if (w == RQ) {
            role_vector(F.xr, q_dt, p.scale, 0);
            role_vector(F.xr2, k_dt, 1.0f, 1);
        }
    } else {
        if (w == RQ) role_vector(F.xr, q_dt, p.scale, 0);
        if (w == RK) role_vector(F.xr, k_dt, 1.0f, 1);
    }
    if (wh == 0) {                                   // this head's gates and decays
        float g, beta;
        if (gate) {
            const float x = raw_to_f(F.g0, a_dt) + raw_to_f(F.g3, dt_bias_dt);
            const float sp = x <= 20.0f ? logf(1.0f + expf(x)) : x;
            g = -expf(raw_to_f(F.g2, A_log_dt)) * sp;
            beta = 1.0f / (1.0f + expf(-raw_to_f(F.g1, bt_dt)));
        } else {
            g = raw_to_f(F.g0, a_dt);
            beta = raw_to_f(F.g1, bt_dt);
        }
        if (lane == 0) {
            lds_scal[0] = beta;
            lds_scal[1] = expf(F.gcur);
            lds_scal[2] = expf(g);
            lds_scal[3] = F.gcur + g;
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
    SQ_MARK(6);                                                   // roles done, every load landed in LDS
    lds_barrier();
    SQ_MARK(7);                                                   // first barrier passed

    // ---- every wavefront: state pass over its row blocks ----
    float sq, sk;                                    // (S0 q)[row], (S0 k)[row], scales applied
    {
        v4i aop[T::NKS];
        quad_fetch_planes<T, 2>(lds_pl, lane, aop);
        float xs[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) xs[g] = lds_xs[kb * NG + g];
        float own[NB];
#pragma unroll
        for (int bi = 0; bi < NB; ++bi) {
            float sc[NG];
#pragma unroll
            for (int g = 0; g < NG; ++g) sc[g] = f16_to_f32(scw[bi][g]);
            own[bi] = quad_block_pass<Q, T>(my_codes + bi * Q::BLK, aop, xs, sc, lane);
        }
        if constexpr (NB == 2) {                     // lane (n, kb) takes over row n of block kb: both sums
            const auto r = __builtin_amdgcn_permlane32_swap(as_u32(own[0]), as_u32(own[1]), false, false);
            sq = as_f32(r[0]);
            sk = as_f32(r[1]);
        } else {
            const Pair qk = pair32(own[0]);
            sq = qk.lo;
            sk = qk.hi;
        }
    }
#ifdef SQ_TIMELINE
    asm volatile("" ::"v"(sq), "v"(sk));                          // the sums are here before the mark is taken
#endif
    SQ_MARK(8);                                                   // state pass done
    // ---- K_i . q, K_i . k of this wavefront's share of the slots ----
    {
        float x[2][4];
#pragma unroll
        for (int v = 0; v < 2; ++v) {
            const float4 f = *reinterpret_cast<const float4*>(lds_xn + v * DK + 4 * (lane % Q::LPS));
            x[v][0] = f.x; x[v][1] = f.y; x[v][2] = f.z; x[v][3] = f.w;
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
#pragma unroll
            for (int v = 0; v < 2; ++v) {
                float pr = kf[0] * x[v][0];
#pragma unroll
                for (int c = 1; c < 4; ++c) pr = __builtin_fmaf(kf[c], x[v][c], pr);
                pr = lanes_sum<Q::LPS>(pr);
                if (lane % Q::LPS == 0 && i < MM) lds_dots[v * MM + i] = pr;
            }
        }
    }
    // ---- k . q ----
    if (w == RK) {
        float kqp = 0.0f;
#pragma unroll
        for (int t = 0; t < NE; ++t) kqp = __builtin_fmaf(lds_xn[DK + NE * lane + t], lds_xn[NE * lane + t], kqp);
        kqp = lanes_sum<WAVE>(kqp);
        if (lane == 0) lds_gsc[0] = kqp;
    }
    SQ_MARK(9);                                                   // buffer dot products done
    lds_barrier();                                   // the raw keys of slot n may be overwritten from here on
    SQ_MARK(10);                                                  // second barrier passed

    // ---- the buffered key of this token: the rounded k, for this workgroup's folds and (first head group of
    //      the key head only) for the slot ----
    if (w == RX) {
        float kxe[NE], kmax = 0.0f;
#pragma unroll
        for (int t = 0; t < NE; ++t) {
            kxe[t] = lds_xn[DK + NE * lane + t];
            kmax = fmaxf(kmax, fabsf(kxe[t]));
        }
        float ks = 1.0f;
        if constexpr (T::QBUF) ks = fp16_scale(lanes_max<WAVE>(kmax), 127.0f);
        const bool write = tid.h - hl == tid.hk * p.gqa;
        if (T::QBUF && lane == 0) {
            lds_kbsf[n] = ks;
            if (write) A.buf.KBS[n] = f32_to_f16(ks);
        }
        if constexpr (T::QBUF) {
            uint32_t pk = 0;
#pragma unroll
            for (int t = 0; t < NE; ++t) pk |= (uint32_t(int(round_buf(kxe[t], ks))) & 0xFFu) << (8 * t);
            uint8_t* dl = lds_kbr + n * DK + NE * lane;
            uint8_t* dg = A.buf.KB + n * DK + NE * lane;
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
                if (write) reinterpret_cast<uint16_t*>(A.buf.KB)[n * DK + NE * lane + t] = hb;
            }
        }
    }

    // ---- this wavefront's rows: buffer term, u, o ----
    const float beta = lds_scal[0], alpha = lds_scal[1], a = lds_scal[2], gnew = lds_scal[3];
    const float kq = lds_gsc[0];
    // coefficients of the head's slots, lane i: c_x[i] = exp(gcur - G_i) (K_i . x), times the slot's value scale;
    // dead slots (i >= n) may hold anything: select, never multiply
    const int li = lane < m ? lane : 0;
    float cq, ck;
    {
        const float dec = expf(gcur - lds_gbf[li]);
        const float dq = lds_dots[li], dk_ = lds_dots[MM + li];
        const float us_i = T::QBUF ? lds_ubsf[li] : 1.0f;
        const bool alive = lane < n;
        cq = alive ? (T::QBUF ? (dec * dq) * us_i : dec * dq) : 0.0f;
        ck = alive ? (T::QBUF ? (dec * dk_) * us_i : dec * dk_) : 0.0f;
    }
    // every slot's value is fetched up front (one wait for all of them), dead slots then add c = 0 times a finite
    // int8 value, or are skipped (bf16 values of a dead slot may be NaNs)
    float uv[MM];
#pragma unroll
    for (int i = 0; i < MM; ++i) uv[i] = lds_raw<T::QBUF>(lds_ubr, (i < m ? i : 0) * DV + row);
    float accq = alpha * sq, acck = alpha * sk;
#pragma unroll
    for (int i = 0; i < MM; ++i) {
        const float u_i = T::QBUF ? uv[i] : (i < n ? uv[i] : 0.0f);
        accq = __builtin_fmaf(u_i, lane_bcast(cq, i), accq);
        acck = __builtin_fmaf(u_i, lane_bcast(ck, i), acck);
    }
    const float vt = raw_to_f(vr, v_dt);
    const float u = beta * __builtin_fmaf(-a, acck, vt);
    const float o = __builtin_fmaf(kq, u, a * accq);
    if (NB == 2 || kb == 0) store_f(outp, out_dt, row, o);
    SQ_MARK(11);                                                  // output stored

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
#ifdef SQ_TIMELINE
        asm volatile("" ::"v"(amax));
#endif
        SQ_MARK(12);                                              // largest |u| of the head known (a barrier)
        us = fp16_scale(amax, 127.0f);
        if (wh == 0 && lane == 0) { A.buf.UBS[n] = f32_to_f16(us); lds_ubsf[n] = us; }
    }
    if (NB == 2 || kb == 0) {
        if constexpr (T::QBUF) {
            const int8_t c = int8_t(int(round_buf(u, us)));
            reinterpret_cast<int8_t*>(A.buf.UB)[n * DV + row] = c;
            reinterpret_cast<int8_t*>(lds_ubr)[n * DV + row] = c;
        } else {
            const uint16_t hb = f32_to_bf16(u);
            reinterpret_cast<uint16_t*>(A.buf.UB)[n * DV + row] = hb;
            reinterpret_cast<uint16_t*>(lds_ubr)[n * DV + row] = hb;
        }
    }
    if (wh == 0 && lane == 0) {
        A.GBh[n] = gnew;
        *A.gcp = full ? 0.0f : gnew;                 // advance
        *A.np = full ? 0 : n + 1;
    }

    SQ_MARK(13);                                                  // appended, counters advanced
    // ---- fold ----
    if (full) {
        lds_barrier();                               // `full` is the same in every head of a slot
        constexpr int MT4 = (MM + 3) / 4, CL = DK / 4;
        // what the fold derives from the lane id it derives anew (from a copy the compiler cannot trace back): offsets
        // formed at the top of the kernel would otherwise be kept in registers all the way to here
        int lf = lane;
        asm volatile("" : "+v"(lf));
        const int fn = lf & 15, fq = lf >> 4;
        const int swzf = swz<Q>(lf / Q::CPR, lf % Q::CPR);
        // decay ratios a_m / a_i of the lane's slots 4 t + q (this token: 1)
        float decf[MT4];
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
                    float uv = lds_raw<T::QBUF>(lds_ubr, sc_ * DV + frow);
                    if constexpr (T::QBUF) uv = uv * lds_ubsf[sc_];
                    uv = decf[t] * uv;
                    bop[t] = sl < m ? uv : 0.0f;
                }
                quad_fold_half<Q, T>(blk, hf, kop, bop, cmul, f16_to_f32(lds_sc[frow * NG + fg]),
                                            A.SCh + frow * NG + fg, lf);
            }
            wave_sync();
#pragma unroll
            for (int t = 0; t < Q::NLD; ++t)
                stream_store(reinterpret_cast<v4u*>(A.Sh + (wh * NB + bi) * Q::BLK + t * 1024 + lf * 16),
                             *reinterpret_cast<const v4u*>(blk + t * 1024 + swzf));
        }
    }
    SQ_MARK(14);                                                  // fold done and stored (if any)
}

template <class T, int NB, int GH, int WPE, int SPEC>
int launch_gdn_quad(const GdnParams& p0, hipStream_t stream) {
    GdnParams p = p0;
    p.per_xcd = (p.per_xcd % GH == 0) ? p.per_xcd / GH : 0;          // dealing over head groups
    const uint32_t grid = uint32_t(p.rows) * uint32_t(p.hv / GH);
    const uint32_t stag = quad_start_ramp<Quad<T, NB, GH>, WPE>(grid, 32);
#ifdef SQ_TIMELINE
    const SqTimelineBuf tl = sq_timeline_buffer();
    hipLaunchKernelGGL((gdn_quad_kernel<T, NB, GH, WPE, SPEC>), dim3(grid), dim3(Quad<T, NB, GH>::THREADS),
                       quad_lds_pad(), stream, p.idx, p.order, p.per_xcd, p.hv, p.hv_shift, p.st.S, p.st.sS, p.st.NPTR, p.st.sN, stag,
                       tl.p, tl.cap, p);
#else
    hipLaunchKernelGGL((gdn_quad_kernel<T, NB, GH, WPE, SPEC>), dim3(grid), dim3(Quad<T, NB, GH>::THREADS),
                       quad_lds_pad(), stream, p.idx, p.order, p.per_xcd, p.hv, p.hv_shift, p.st.S, p.st.sS, p.st.NPTR, p.st.sN, stag, p);
#endif
    return int(hipGetLastError());
}

}  // namespace sq
