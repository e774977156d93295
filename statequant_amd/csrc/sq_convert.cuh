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

// LDS (dynamic): keys x decay ratio [m][DK] fp32, values [m][dv] fp32.
// Column split of the output pass: a lane takes NCH chunks of 4 columns, chunk t = columns 4 LPR t + 4 cg .. + 3, so
// that the LPR lanes of a row write 16 LPR consecutive bytes with every store instruction (whole 128-byte lines for
// d_k = 128) -- with 16 consecutive columns per lane each store would scatter 16-byte pieces 64 bytes apart.
template <int BITS, int DK, int GROUP, bool QBUF, bool KDA>
__global__ __launch_bounds__(WAVE) void read_kernel(const ReadParams p) {
    using T = RowTile<BITS, DK, GROUP, QBUF>;
    constexpr int NCH = CPL / 4;
    constexpr int CSTEP = 4 * T::LPR;                             // columns between a lane's chunks
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int m = p.m;
    const uint32_t um = m, dv = p.dv;
    float* lds_k = reinterpret_cast<float*>(lds);
    float* lds_u = lds_k + m * DK;
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

    // keys of the live slots, times their decay ratio (slot = row group + RG x pass, 16 consecutive columns per lane)
    for (int i0 = 0; i0 < n; i0 += T::RG) {
        const int i = i0 + l.rg;
        const int ic = i < n ? i : n - 1;
        const KPiece<QBUF> kp = load_kpiece<T>(KB, ic, n, l);
        const float ks = QBUF ? f16_to_f32(KBS[ic]) : 1.0f;
        float kb[CPL];
        decode_kpiece<T>(kp, ks, l, kb);
#pragma unroll
        for (int t = 0; t < CPL; ++t) {
            const float gi = KDA ? GBh[ic * DK + cc * CPL + t] : GBh[ic];
            const float gc = KDA ? gch[cc * CPL + t] : gch[0];
            kb[t] = kb[t] * expf(gc - gi);
        }
        if (i < n && live) {
            float4* d4 = reinterpret_cast<float4*>(lds_k + i * DK + l.cg * CPL);
#pragma unroll
            for (int c = 0; c < CPL / 4; ++c) d4[c] = make_float4(kb[4 * c], kb[4 * c + 1], kb[4 * c + 2], kb[4 * c + 3]);
        }
    }
    for (uint32_t e = l.lane; e < uint32_t(n) * dv; e += WAVE) {
        const uint32_t i = e / dv;
        float u;
        if constexpr (QBUF) u = float(reinterpret_cast<const int8_t*>(UB)[e]) * f16_to_f32(UBS[i]);
        else u = bf16_to_f32(reinterpret_cast<const uint16_t*>(UB)[e]);
        lds_u[e] = u;
    }
    float alpha_p[NCH][4];                                        // a_n at this lane's columns
#pragma unroll
    for (int t = 0; t < NCH; ++t)
#pragma unroll
        for (int c = 0; c < 4; ++c) alpha_p[t][c] = expf(KDA ? gch[t * CSTEP + 4 * cc + c] : gch[0]);
    __syncthreads();

    constexpr int RR = 2;                                         // rows per pass over the buffered keys
    for (uint32_t r0 = 0; r0 < dv; r0 += RR * T::RG) {
        uint32_t row[RR], rc[RR];
        float acc[RR][NCH][4];
#pragma unroll
        for (int k = 0; k < RR; ++k) {
            row[k] = r0 + k * T::RG + l.rg;
            rc[k] = row[k] < dv ? row[k] : dv - 1;
#pragma unroll
            for (int t = 0; t < NCH; ++t) {
                const int col = t * CSTEP + 4 * cc;
                const float s = f16_to_f32(SCh[rc[k] * T::NG + col / GROUP]);
                float c4[4];
                if constexpr (BITS == 8) {
                    const uint32_t w = *reinterpret_cast<const uint32_t*>(Sh + rc[k] * T::ROW_BYTES + col);
#pragma unroll
                    for (int c = 0; c < 4; ++c) c4[c] = s8_to_f(w, c);
                } else {
                    const uint32_t w = *reinterpret_cast<const uint16_t*>(Sh + rc[k] * T::ROW_BYTES + col / 2);
#pragma unroll
                    for (int c = 0; c < 4; ++c) c4[c] = float(int32_t((w >> (4 * c)) & 0xFu) - 8);
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[k][t][c] = alpha_p[t][c] * (c4[c] * s);
            }
        }
        for (int i = 0; i < n; ++i) {                             // live slots only
            float4 kx[NCH];
#pragma unroll
            for (int t = 0; t < NCH; ++t) kx[t] = *reinterpret_cast<const float4*>(lds_k + i * DK + t * CSTEP + 4 * cc);
#pragma unroll
            for (int k = 0; k < RR; ++k) {
                const float du = lds_u[i * dv + rc[k]];
#pragma unroll
                for (int t = 0; t < NCH; ++t) {
                    acc[k][t][0] = __builtin_fmaf(du, kx[t].x, acc[k][t][0]);
                    acc[k][t][1] = __builtin_fmaf(du, kx[t].y, acc[k][t][1]);
                    acc[k][t][2] = __builtin_fmaf(du, kx[t].z, acc[k][t][2]);
                    acc[k][t][3] = __builtin_fmaf(du, kx[t].w, acc[k][t][3]);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < RR; ++k)
            if (row[k] < dv && live) {
#pragma unroll
                for (int t = 0; t < NCH; ++t)
                    *reinterpret_cast<float4*>(out + row[k] * DK + t * CSTEP + 4 * l.cg) =
                        make_float4(acc[k][t][0], acc[k][t][1], acc[k][t][2], acc[k][t][3]);
            }
    }
}

template <int BITS, int DK, int GROUP, bool QBUF, bool KDA>
int launch_read(const ReadParams& p, hipStream_t stream) {
    using T = RowTile<BITS, DK, GROUP, QBUF>;
    const size_t lds = size_t(p.m) * (DK + p.dv) * sizeof(float);
    hipLaunchKernelGGL((read_kernel<BITS, DK, GROUP, QBUF, KDA>), dim3(p.rows * p.hv), dim3(WAVE), lds, stream, p);
    return int(hipGetLastError());
}

}  // namespace sq
