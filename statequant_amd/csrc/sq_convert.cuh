// The two operations either side of the decode step (prefill hands a state over / takes it back):
//   pack   fp32 value-major state -> stored codes + fp16 scales, into given sequences, buffers emptied
//          (reference: kernels/fold.py:123-147 `pack_vk`, kernels/slots.py:236-252 `write`)
//   read   the stored state advanced across its pending buffer, as fp32 value-major
//          S_n = a_n S_0 + sum_{i<n} (a_n / a_i) u_i k_i^T;  KDA: decays per key channel
//          (reference: kernels/slots.py:210-233, kernels/kda.py:351-372)
// Both are plain streaming kernels, one wavefront per (sequence, value head): rows in the row shape of the fold
// (LPRP lanes per row, 16 columns per lane), d_v and m taken at run time.  They are bound by the fp32 side of the
// transfer (pack reads 4 bytes per code it writes, read writes 4 bytes per code it reads).
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

// geometry carrier: only the d_k-shaped members of Tile are used here
template <int BITS, int DK, int GROUP, bool QBUF>
using RowTile = Tile<BITS, DK, 128, GROUP, QBUF, 16>;

template <int BITS, int DK, int GROUP>
__global__ __launch_bounds__(WAVE) void pack_kernel(const PackParams p) {
    using T = RowTile<BITS, DK, GROUP, true>;
    const LaneId l = lane_id<T>();
    const uint32_t b = blockIdx.x / uint32_t(p.hv), h = blockIdx.x - b * uint32_t(p.hv);
    const int32_t slot = p.idx ? p.idx[b] : int32_t(b);
    if (p.idx && slot <= 0) return;
    const uint32_t seq = slot, dv = p.dv;
    const float* src = p.src + (uint64_t(b) * p.s_src + uint64_t(h) * dv * DK);
    uint8_t* Sh = field(p.S, seq, p.sS, h * (dv * T::ROW_BYTES));
    uint16_t* SCh = field(p.SC, seq, p.sSC, h * (dv * T::NG));
    const bool live = l.cg < T::LPR;
    const int cc = live ? l.cg : T::LPR - 1;
    int gi = (l.cg * CPL) / GROUP;
    const bool has_group = gi < T::NG;
    gi = has_group ? gi : T::NG - 1;
    const bool lead = live && (l.cg % T::LPG) == 0 && has_group;
    for (uint32_t r0 = 0; r0 < dv; r0 += T::RG) {
        const uint32_t row = r0 + l.rg;
        const bool in = row < dv;
        const float4* s4 = reinterpret_cast<const float4*>(src + (in ? row : dv - 1) * DK + cc * CPL);
        float x[CPL];
#pragma unroll
        for (int t = 0; t < CPL / 4; ++t) {
            const float4 f = s4[t];
            x[4 * t] = f.x; x[4 * t + 1] = f.y; x[4 * t + 2] = f.z; x[4 * t + 3] = f.w;
        }
        float amax = 0.0f;
#pragma unroll
        for (int t = 0; t < CPL; ++t) amax = fmaxf(amax, live ? fabsf(x[t]) : 0.0f);
        amax = block_max<T::LPG>(amax);
        const float s = fp16_scale(amax, T::QMAX);
        float q[CPL];
#pragma unroll
        for (int t = 0; t < CPL; ++t) q[t] = fminf(fmaxf(rintf(x[t] / s), -T::QMAX), T::QMAX);
        if (in && live) store_row<BITS>(Sh + row * T::ROW_BYTES + l.cg * T::LANE_BYTES, encode_row<BITS>(q));
        if (in && lead) SCh[row * T::NG + gi] = f32_to_f16(s);
    }
    // empty the buffer: counter copy of this head, running decay of this head
    if (p.NPTR && l.lane == 0) *field(p.NPTR, seq, p.sN, h) = 0;
    if (p.GCUR)
        for (uint32_t e = l.lane; e < uint32_t(p.gcur_per_head); e += WAVE)
            *field(p.GCUR, seq, p.sGC, h * uint32_t(p.gcur_per_head) + e) = 0.0f;
}

template <int BITS, int DK, int GROUP>
int launch_pack(const PackParams& p, hipStream_t stream) {
    hipLaunchKernelGGL((pack_kernel<BITS, DK, GROUP>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p);
    return int(hipGetLastError());
}

// LDS (dynamic): keys x decay ratio [m][KROW] fp32, values [m][dv] fp32
template <int BITS, int DK, int GROUP, bool QBUF, bool KDA>
__global__ __launch_bounds__(WAVE) void read_kernel(const ReadParams p) {
    using T = RowTile<BITS, DK, GROUP, QBUF>;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int m = p.m;
    const uint32_t um = m, dv = p.dv;
    float* lds_k = reinterpret_cast<float*>(lds);
    float* lds_u = lds_k + m * T::KROW;
    const LaneId l = lane_id<T>();
    const uint32_t b = blockIdx.x / uint32_t(p.hv), h = blockIdx.x - b * uint32_t(p.hv);
    const uint32_t hk = h / uint32_t(p.gqa);
    float* out = p.out + (uint64_t(b) * p.s_out + uint64_t(h) * dv * DK);
    const int32_t slot = p.idx ? p.idx[b] : int32_t(b);
    if (p.idx && slot <= 0) return;
    const uint32_t seq = slot;
    const uint8_t* Sh = field(p.st.S, seq, p.st.sS, h * (dv * T::ROW_BYTES));
    const uint16_t* SCh = field(p.st.SC, seq, p.st.sSC, h * (dv * T::NG));
    const uint8_t* KB = p.st.KB + (uint64_t(seq) * p.st.sKB + hk * um * DK) * T::BE;
    const uint8_t* UB = p.st.UB + (uint64_t(seq) * p.st.sUB + h * um * dv) * T::BE;
    const uint16_t* KBS = field(p.st.KBS, seq, p.st.sKBS, hk * um);
    const uint16_t* UBS = field(p.st.UBS, seq, p.st.sUBS, h * um);
    const float* GBh = field(p.st.GB, seq, p.st.sGB, h * um * (KDA ? DK : 1));
    const float* gch = field(p.st.GCUR, seq, p.st.sGC, h * (KDA ? DK : 1));
    const int n = *field(p.st.NPTR, seq, p.st.sN, 0u) & (m - 1);     // the first head's copy, as the reference reads it
    const bool live = l.cg < T::LPR;
    const int cc = live ? l.cg : T::LPR - 1;

    // keys, times their decay ratio, dead slots as zeros
    float alpha_p[CPL];                                           // this lane's columns of a_n
    float gcp[CPL];
#pragma unroll
    for (int t = 0; t < CPL; ++t) {
        gcp[t] = KDA ? gch[cc * CPL + t] : gch[0];
        alpha_p[t] = expf(gcp[t]);
    }
    BufAddr<T> ba;
    ba.KB = const_cast<uint8_t*>(KB);
    for (int i0 = 0; i0 < m; i0 += T::RG) {
        const int i = i0 + l.rg;
        const int ic = i < m ? i : m - 1;
        const KPiece<QBUF> kp = load_kpiece<T>(ba.KB, ic, m, l);
        const float ks = QBUF ? f16_to_f32(KBS[ic]) : 1.0f;
        float kb[CPL];
        decode_kpiece<T>(kp, ks, l, kb);
        const bool alive = i < n;
#pragma unroll
        for (int t = 0; t < CPL; ++t) {
            const float gi = KDA ? GBh[ic * DK + cc * CPL + t] : GBh[ic];
            kb[t] = alive ? kb[t] * expf(gcp[t] - gi) : 0.0f;
        }
        if (i < m) stage_kpiece<T>(lds_k, i, l, kb);
    }
    for (uint32_t e = l.lane; e < um * dv; e += WAVE) {
        const uint32_t i = e / dv;
        float u;
        if constexpr (QBUF) u = float(reinterpret_cast<const int8_t*>(UB)[e]) * f16_to_f32(UBS[i]);
        else u = bf16_to_f32(reinterpret_cast<const uint16_t*>(UB)[e]);
        lds_u[e] = int(i) < n ? u : 0.0f;
    }
    __syncthreads();

    int gi = (l.cg * CPL) / GROUP;
    const bool has_group = gi < T::NG;
    gi = has_group ? gi : T::NG - 1;
    constexpr int RR = 2;                                         // rows per pass over the buffered keys
    for (uint32_t r0 = 0; r0 < dv; r0 += RR * T::RG) {
        uint32_t row[RR], rc[RR];
        float acc[RR][CPL];
#pragma unroll
        for (int k = 0; k < RR; ++k) {
            row[k] = r0 + k * T::RG + l.rg;
            rc[k] = row[k] < dv ? row[k] : dv - 1;
            float c[CPL];
            decode_row<BITS>(load_row<BITS>(Sh + rc[k] * T::ROW_BYTES + cc * T::LANE_BYTES), c);
            const float s = has_group ? f16_to_f32(SCh[rc[k] * T::NG + gi]) : 0.0f;
#pragma unroll
            for (int t = 0; t < CPL; ++t) acc[k][t] = alpha_p[t] * (c[t] * s);
        }
        for (int i = 0; i < n; ++i) {                             // live slots only
            float kx[CPL];
            lds_piece<T>(lds_k + i * T::KROW, l.cg, kx);
#pragma unroll
            for (int k = 0; k < RR; ++k) {
                const float du = lds_u[i * dv + rc[k]];
#pragma unroll
                for (int t = 0; t < CPL; ++t) acc[k][t] = __builtin_fmaf(du, kx[t], acc[k][t]);
            }
        }
#pragma unroll
        for (int k = 0; k < RR; ++k)
            if (row[k] < dv && live) {
                float4* o4 = reinterpret_cast<float4*>(out + row[k] * DK + l.cg * CPL);
#pragma unroll
                for (int t = 0; t < CPL / 4; ++t)
                    o4[t] = make_float4(acc[k][4 * t], acc[k][4 * t + 1], acc[k][4 * t + 2], acc[k][4 * t + 3]);
            }
    }
}

template <int BITS, int DK, int GROUP, bool QBUF, bool KDA>
int launch_read(const ReadParams& p, hipStream_t stream) {
    using T = RowTile<BITS, DK, GROUP, QBUF>;
    const size_t lds = size_t(p.m) * (T::KROW + p.dv) * sizeof(float);
    hipLaunchKernelGGL((read_kernel<BITS, DK, GROUP, QBUF, KDA>), dim3(p.rows * p.hv), dim3(WAVE), lds, stream, p);
    return int(hipGetLastError());
}

}  // namespace sq
