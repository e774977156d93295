// The two operations either side of the decode step (prefill hands a state over / takes it back):
//   pack   fp32 value-major state -> stored codes + fp16 scales, into given sequences, buffers emptied
//          (reference: kernels/fold.py:123-147 `pack_vk`, kernels/slots.py:236-252 `write`)
//   read   the stored state advanced across its pending buffer, as fp32 value-major
//          S_n = a_n S_0 + sum_{i<n} (a_n / a_i) u_i k_i^T;  KDA: decays per key channel
//          (reference: kernels/slots.py:210-233, kernels/kda.py:351-372)
// Both are plain streaming kernels, one wavefront per (sequence, value head): rows in the row shape of the fold
// (LPRP lanes per row, 16 columns per lane), d_v and m taken at run time.  Value-axis scale groups (32 rows of one key
// column share a scale) pack with a column shape instead (a lane owns two neighbouring columns of a 32-row block);
// the unquantized state (bf16 / fp32) packs as a cast.  They are bound by the fp32 side of the
// transfer (pack reads 4 bytes per code it writes, read writes 4 bytes per code it reads).
#pragma once
#include "sq_tile.cuh"
#include "sq_params.h"

namespace sq {

// geometry carrier: only the d_k-shaped members of Tile are used here
template <int BITS, int DK, int GROUP, bool QBUF, bool AXV = false>
using RowTile = Tile<BITS, DK, 128, GROUP, QBUF, 16, AXV>;

// Empty a sequence's buffer: this head's counter copy and running decay.
__device__ __forceinline__ void reset_counters(const PackParams& p, uint32_t seq, uint32_t h, int lane) {
    if (p.NPTR && lane == 0) {
        *field(p.NPTR, seq, p.sN, h) = 0;
        if (h + 1 == uint32_t(p.hv))                         // the last head also clears the copies no head owns
            for (uint32_t e = p.hv; e < uint32_t(p.nptr_copies); ++e) *field(p.NPTR, seq, p.sN, e) = 0;
    }
    if (p.GCUR)
        for (uint32_t e = lane; e < uint32_t(p.gcur_per_head); e += WAVE)
            *field(p.GCUR, seq, p.sGC, h * uint32_t(p.gcur_per_head) + e) = 0.0f;
}

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
        const Divisor ds = scale_divisor(s);                 // x / s below is the IEEE quotient (sq_device.cuh)
        float q[CPL];
#pragma unroll
        for (int t = 0; t < CPL; ++t) q[t] = fminf(fmaxf(rintf(div_by(x[t], ds)), -T::QMAX), T::QMAX);
        if (in && live) store_row<BITS>(Sh + row * T::ROW_BYTES + l.cg * T::LANE_BYTES, encode_row<BITS>(q));
        if (in && lead) SCh[row * T::NG + gi] = f32_to_f16(s);
    }
    reset_counters(p, seq, h, l.lane);
}

// Value-axis groups of G rows (fold.py:139-146): scales [dv / G][DK].  A lane owns columns 2 lane, 2 lane + 1 and
// walks the G rows of a group twice (absmax, then codes) with the group's 2 G values in registers.
template <int BITS, int DK, int G>
__global__ __launch_bounds__(WAVE) void pack_v_kernel(const PackParams p) {
    constexpr float QMAX = float((1 << (BITS - 1)) - 1);
    constexpr int ROW_BYTES = DK * BITS / 8;
    static_assert(DK % 2 == 0 && DK <= 2 * WAVE, "two columns per lane");
    const int lane = threadIdx.x;
    const uint32_t b = blockIdx.x / uint32_t(p.hv), h = blockIdx.x - b * uint32_t(p.hv);
    const int32_t slot = p.idx ? p.idx[b] : int32_t(b);
    if (p.idx && slot <= 0) return;
    const uint32_t seq = slot, dv = p.dv;
    const float* src = p.src + (uint64_t(b) * p.s_src + uint64_t(h) * dv * DK);
    uint8_t* Sh = field(p.S, seq, p.sS, h * (dv * ROW_BYTES));
    uint16_t* SCh = field(p.SC, seq, p.sSC, h * ((dv / G) * DK));
    const bool live = 2 * lane < DK;
    const int c0 = live ? 2 * lane : DK - 2;
    for (uint32_t r0 = 0; r0 < dv; r0 += G) {
        float2 x[G];
#pragma unroll
        for (int r = 0; r < G; ++r) x[r] = *reinterpret_cast<const float2*>(src + (r0 + r) * DK + c0);
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int r = 0; r < G; ++r) { a0 = fmaxf(a0, fabsf(x[r].x)); a1 = fmaxf(a1, fabsf(x[r].y)); }
        const float s0 = fp16_scale(a0, QMAX), s1 = fp16_scale(a1, QMAX);
        if (live)
            *reinterpret_cast<uint32_t*>(SCh + (r0 / G) * DK + c0) = uint32_t(f32_to_f16(s0)) | (uint32_t(f32_to_f16(s1)) << 16);
        const Divisor d0 = scale_divisor(s0), d1 = scale_divisor(s1);      // IEEE quotients (sq_device.cuh)
#pragma unroll
        for (int r = 0; r < G; ++r) {
            const int q0 = int(fminf(fmaxf(rintf(div_by(x[r].x, d0)), -QMAX), QMAX));
            const int q1 = int(fminf(fmaxf(rintf(div_by(x[r].y, d1)), -QMAX), QMAX));
            uint8_t* row = Sh + (r0 + r) * ROW_BYTES;
            if (live) {
                if constexpr (BITS == 8)
                    *reinterpret_cast<uint16_t*>(row + c0) = uint16_t((q0 & 0xFF) | ((q1 & 0xFF) << 8));
                else
                    row[lane] = uint8_t((q0 + 8) | ((q1 + 8) << 4));
            }
        }
    }
    reset_counters(p, seq, h, lane);
}

// The unquantized state: a cast to bf16 (round to nearest even) or a copy (fp32), [dv][DK] per head.
template <int BITS, int DK>
__global__ __launch_bounds__(WAVE) void pack_f_kernel(const PackParams p) {
    static_assert(DK % 4 == 0, "four columns per lane and step");
    const int lane = threadIdx.x;
    const uint32_t b = blockIdx.x / uint32_t(p.hv), h = blockIdx.x - b * uint32_t(p.hv);
    const int32_t slot = p.idx ? p.idx[b] : int32_t(b);
    if (p.idx && slot <= 0) return;
    const uint32_t seq = slot, n = p.dv * DK;
    const float* src = p.src + (uint64_t(b) * p.s_src + uint64_t(h) * n);
    uint8_t* Sh = field(p.S, seq, p.sS, h * (n * (BITS / 8)));
    for (uint32_t e = 4 * lane; e < n; e += 4 * WAVE) {
        const float4 f = *reinterpret_cast<const float4*>(src + e);
        if constexpr (BITS == 16)
            *reinterpret_cast<uint2*>(Sh + 2 * e) =
                make_uint2(uint32_t(f32_to_bf16(f.x)) | (uint32_t(f32_to_bf16(f.y)) << 16),
                           uint32_t(f32_to_bf16(f.z)) | (uint32_t(f32_to_bf16(f.w)) << 16));
        else
            *reinterpret_cast<float4*>(Sh + 4 * e) = f;
    }
    reset_counters(p, seq, h, lane);
}

// AXV: value-axis groups of GROUP rows; BITS 16 / 32: the unquantized state (GROUP = DK).
template <int BITS, int DK, int GROUP, bool AXV>
int launch_pack(const PackParams& p, hipStream_t stream) {
    if constexpr (BITS >= 16) hipLaunchKernelGGL((pack_f_kernel<BITS, DK>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p);
    else if constexpr (AXV) hipLaunchKernelGGL((pack_v_kernel<BITS, DK, GROUP>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p);
    else hipLaunchKernelGGL((pack_kernel<BITS, DK, GROUP>), dim3(p.rows * p.hv), dim3(WAVE), 0, stream, p);
    return int(hipGetLastError());
}

// LDS (dynamic): keys x decay ratio [m][DK] fp32, values [m][dv] fp32.
// Column split of the output pass: a lane takes NCH chunks of 4 columns, chunk t = columns 4 LPR t + 4 cg .. + 3, so
// that the LPR lanes of a row write 16 LPR consecutive bytes with every store instruction (whole 128-byte lines for
// d_k = 128) -- with 16 consecutive columns per lane each store would scatter 16-byte pieces 64 bytes apart.
template <int BITS, int DK, int GROUP, bool QBUF, bool KDA, bool AXV>
__global__ __launch_bounds__(WAVE) void read_kernel(const ReadParams p) {
    using T = RowTile<BITS, DK, GROUP, QBUF, AXV>;
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
    if (p.idx && slot <= 0) {                                      // padding row: a zero state, nothing of a slot read
        float4* o4 = reinterpret_cast<float4*>(out);
        for (uint32_t e = l.lane; e < dv * DK / 4; e += WAVE) o4[e] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        return;
    }
    const uint32_t seq = slot;
    const uint8_t* Sh = field(p.st.S, seq, p.st.sS, h * (dv * T::ROW_BYTES));
    const uint16_t* SCh = field(p.st.SC, seq, p.st.sSC, AXV ? h * ((dv / GROUP) * DK) : h * (dv * T::NG));
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
                float s4[4], c4[4];
                if constexpr (T::FLT) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) s4[c] = 1.0f;
                } else if constexpr (AXV) {                       // one scale per (group of rows, column)
                    const uint2 w = *reinterpret_cast<const uint2*>(SCh + (rc[k] / GROUP) * DK + col);
                    s4[0] = f16_to_f32(uint16_t(w.x)); s4[1] = f16_to_f32(uint16_t(w.x >> 16));
                    s4[2] = f16_to_f32(uint16_t(w.y)); s4[3] = f16_to_f32(uint16_t(w.y >> 16));
                } else {
                    const float s = f16_to_f32(SCh[rc[k] * T::NG + col / GROUP]);
#pragma unroll
                    for (int c = 0; c < 4; ++c) s4[c] = s;
                }
                if constexpr (BITS == 32) {
                    const float4 w = *reinterpret_cast<const float4*>(Sh + rc[k] * T::ROW_BYTES + 4 * col);
                    c4[0] = w.x; c4[1] = w.y; c4[2] = w.z; c4[3] = w.w;
                } else if constexpr (BITS == 16) {
                    const uint2 w = *reinterpret_cast<const uint2*>(Sh + rc[k] * T::ROW_BYTES + 2 * col);
                    c4[0] = as_f32(w.x << 16); c4[1] = as_f32(w.x & 0xFFFF0000u);
                    c4[2] = as_f32(w.y << 16); c4[3] = as_f32(w.y & 0xFFFF0000u);
                } else if constexpr (BITS == 8) {
                    const uint32_t w = *reinterpret_cast<const uint32_t*>(Sh + rc[k] * T::ROW_BYTES + col);
#pragma unroll
                    for (int c = 0; c < 4; ++c) c4[c] = s8_to_f(w, c);
                } else {
                    const uint32_t w = *reinterpret_cast<const uint16_t*>(Sh + rc[k] * T::ROW_BYTES + col / 2);
#pragma unroll
                    for (int c = 0; c < 4; ++c) c4[c] = float(int32_t((w >> (4 * c)) & 0xFu) - 8);
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[k][t][c] = alpha_p[t][c] * (c4[c] * s4[c]);
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

template <int BITS, int DK, int GROUP, bool QBUF, bool KDA, bool AXV>
int launch_read(const ReadParams& p, hipStream_t stream) {
    const size_t lds = size_t(p.m) * (DK + p.dv) * sizeof(float);
    hipLaunchKernelGGL((read_kernel<BITS, DK, GROUP, QBUF, KDA, AXV>), dim3(p.rows * p.hv), dim3(WAVE), lds, stream, p);
    return int(hipGetLastError());
}

// A dispatch order for the step kernels (their `order` argument; no counterpart in the reference) for batches whose
// sequences fill their buffers on different steps.  A row that folds on the coming step keeps its workgroups half
// again as long as the others; where the batch order puts such rows decides when the launch ends: the step kernels
// deal eight contiguous ranges of rows to the GPU's eight XCDs, which do not share work, so the folding rows should
// be spread evenly over the ranges, and inside a range neither at the front (their writes then come in one burst)
// nor in the last round of workgroups (they then end after everything else).  order[position] = batch row: every
// range of R = rows / 8 positions gets F / 8 of the F folding rows (the first F % 8 ranges one more), one after
// every s - 1 other rows from the start of the range, s = max(2, R / (4 f)) for a range with f of them -- its first
// quarter (measured best on every kernel here: the one-wavefront kernels' folding tiles live three times as long as
// the others and must start early; a first half costs them 20 %, the very front 1-2 % on all), more where more than
// every eighth row folds; the other rows (padding rows among them) keep their order.  The identity for
// rows % 8 != 0, fewer than 64 rows, no folding row, or more than every second row of a range folding.
// One workgroup; ranks by ballots and a running count.
constexpr int FO_THREADS = 256;
template <int THREADS>                               // (a template only so that the header can hold it)
__global__ __launch_bounds__(THREADS) void fold_order_kernel(const int32_t* idx, const int32_t* NPTR, uint32_t sN,
                                                                int m, int rows, int32_t* order) {
    constexpr int NWV = THREADS / WAVE;
    __shared__ int wave_count[2][NWV];
    const int tid = threadIdx.x, lane = tid % WAVE, wv = tid / WAVE;
    auto folds = [&](int r) {
        if (r >= rows) return false;
        const int32_t slot = idx ? idx[r] : r;
        if (idx && slot <= 0) return false;
        return (NPTR[uint64_t(uint32_t(slot)) * sN] & (m - 1)) == m - 1;
    };
    int cnt = 0;
    for (int r0 = 0; r0 < rows; r0 += THREADS) cnt += __popcll(__builtin_amdgcn_ballot_w64(folds(r0 + tid)));
    if (lane == 0) wave_count[0][wv] = cnt;
    __syncthreads();
    int F = 0;
    for (int w = 0; w < NWV; ++w) F += wave_count[0][w];
    __syncthreads();
    const int R = rows / 8, fq = F / 8, fr = F % 8;
    if (rows % 8 != 0 || rows < 64 || F == 0 || 2 * ((F + 7) / 8) > R) {
        for (int r = tid; r < rows; r += THREADS) order[r] = r;
        return;
    }
    int base_f = 0, base_p = 0;
    for (int r0 = 0; r0 < rows; r0 += THREADS) {
        const int r = r0 + tid;
        const bool f = folds(r), pl = r < rows && !f;
        const unsigned long long bf = __builtin_amdgcn_ballot_w64(f), bp = __builtin_amdgcn_ballot_w64(pl);
        const unsigned long long below = (1ull << lane) - 1ull;
        if (lane == 0) { wave_count[0][wv] = __popcll(bf); wave_count[1][wv] = __popcll(bp); }
        __syncthreads();
        int kf = base_f + __popcll(bf & below), kp = base_p + __popcll(bp & below);
        for (int w = 0; w < NWV; ++w) {
            if (w < wv) { kf += wave_count[0][w]; kp += wave_count[1][w]; }
            base_f += wave_count[0][w];
            base_p += wave_count[1][w];
        }
        __syncthreads();                             // the counts are rewritten on the next turn
        if (f) {
            const int c = kf % 8, j = kf / 8, fc = fq + (c < fr);
            const int s = max(2, R / (4 * fc));
            order[c * R + s * j + s - 1] = r;
        } else if (pl) {
            int t = kp, c = 0;
            for (; c < 7; ++c) {
                const int n = R - (fq + (c < fr));
                if (t < n) break;
                t -= n;
            }
            const int fc = fq + (c < fr);
            int pos = t;
            if (fc > 0) {
                const int s = max(2, R / (4 * fc));
                pos = t < (s - 1) * fc ? t + t / (s - 1) : t + fc;
            }
            order[c * R + pos] = r;
        }
    }
}


}  // namespace sq
