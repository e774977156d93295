// Mixed-width GGA / STEP slot with the FP8 write window (PW-S m): one decode token per (batch row, value head).
//
// Replaces the reference's `_gga_step`, `_gga_advance`, `_gga_store`, `_gga_load`
// (/root/reference/src/statequant/kernels/_gga_triton.py:207-340) and the dual-axis fit they call
// (`_fit_parts`, /root/reference/src/statequant/kernels/_stepquant_triton.py:41-69).  Per slot (byte offsets):
//   0            int32 [4]: n (queued pairs), head (ring index of the oldest pair)
//   offs[h]      head h at its frozen width b: fp16 [d_k, d_v] (b = 16), or codes [d_k, d_v b / 8] packed
//                little-endian along d_v (u = z + qmax; b = 2: u = (z + 3) / 2), row factors fp16 [d_k] (b = 2: one
//                per 32 value columns, [d_k, d_v / 32]) and column factors fp16 [d_v]; the state is (r c) z
//   qoff + h qsz the head's window: P e4m3 [m, d_k], V e4m3 [m, d_v], PS fp32 [m], VS fp32 [m] (a ring)
// One token (Algorithm 1 of the method, as the reference implements it):
//   O_pre = a (O - beta k (k^T O));  queued left factors p_i <- R(a (p_i - beta k (k^T p_i)))  (R: FP8 per vector);
//   o = O_pre^T q + sum_i (p_i^T q) v_i + (beta k^T q) v;  window full: the oldest pair is merged, O_pre += p_0 v_0^T;
//   the state is re-fitted at its width and re-packed in place; (R(beta k), R(v)) is queued.  Pivots (b = 16) and
//   slots without a window take the new write into the state: O = Q(O_pre + beta k v^T).
//
// A workgroup of four wavefronts holds the head's [d_k, d_v] tile in registers.  Wavefront w owns a quarter of the
// columns and all rows: lane (tr, q) = (lane / 4, lane % 4) owns the columns tc CT .. tc CT + CT - 1 (tc = 4 w + q,
// CT = d_v / 16) of the rows s 16 + tr.  Sums along d_k -- the step and the fit take six of them per column -- stay
// inside a wavefront (two DPP row rotations and two lane swaps, no LDS, no barrier); the one sum along d_v (the row
// factors of the fit) is a quad reduction plus one exchange of per-wavefront partials through LDS.
#pragma once
#include "sq_device.cuh"
#include "sq_params.h"

namespace sq {

constexpr int GGA_THREADS = 256;
constexpr int GGA_WAVES = GGA_THREADS / WAVE;
constexpr int GGA_MMAX = 8;
constexpr int GGA_GROUP = 32;

template <int DK_, int DV_>
struct GgaTile {
    static constexpr int DK = DK_, DV = DV_;
    static constexpr int CT = DV / 16;                  // columns per thread
    static constexpr int RPT = DK / 16;                 // rows per thread
    static constexpr int NE = DK / WAVE;                // a key vector's elements per lane (one wavefront per vector)
    static constexpr int NV = DV / WAVE;
    static constexpr int NG = DV / GGA_GROUP;           // row-factor groups of a two-bit head
    static_assert(DK % WAVE == 0 && DV % WAVE == 0 && CT % 4 == 0, "built for d_k, d_v multiples of 64");
};

struct GgaThread {
    int tid, lane, wave, tc, tr;
};
__device__ __forceinline__ GgaThread gga_thread() {
    GgaThread t;
    t.tid = threadIdx.x;
    t.lane = t.tid & (WAVE - 1);
    t.wave = t.tid >> 6;
    t.tc = t.wave * 4 + (t.lane & 3);
    t.tr = t.lane >> 2;
    return t;
}

__host__ __device__ constexpr int gga_qmax(int b) { return b == 2 ? 3 : (1 << (b - 1)) - 1; }
__host__ __device__ constexpr int gga_code_bytes(int b, int dk, int dv) { return dk * dv * b / 8; }

// fp16 with the fit's clamp: [2^-24, 65504], round to nearest even.
__device__ __forceinline__ float gga_half(float x) { return float(_Float16(fminf(fmaxf(x, FP16_TINY), 65504.0f))); }

// The fit's divisions go through `div_rc` / `rcp_f16` (sq_device.cuh): reciprocals once per row or column, IEEE
// quotients at a third of the instructions.
__device__ __forceinline__ float gga_div(float x, float d, float rc) { return div_rc(x, d, rc); }
__device__ __forceinline__ float gga_rcp_f16(float d) { return rcp_f16(d); }

// ---------------------------------------------------------------------------------------------------------------
// sums / maxima along d_k: every thread ends with the totals of its CT columns (the same value in all row groups)
// ---------------------------------------------------------------------------------------------------------------
// The partner's value across 16 / 32 lanes and the lane's own, as one VALU swap each (v_permlane16_swap exchanges the
// odd 16-lane rows of its first operand with the even rows of its second, v_permlane32_swap the upper half of the
// first with the lower half of the second; fed the same register twice they leave both values of a pair in both of
// its lanes, in the same order, so the combined value is bit-identical across the pair).
template <bool MAX>
__device__ __forceinline__ float gga_pair16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(as_u32(v), as_u32(v), false, false);
    return MAX ? fmaxf(as_f32(r[0]), as_f32(r[1])) : as_f32(r[0]) + as_f32(r[1]);
}
template <bool MAX>
__device__ __forceinline__ float gga_pair32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(as_u32(v), as_u32(v), false, false);
    return MAX ? fmaxf(as_f32(r[0]), as_f32(r[1])) : as_f32(r[0]) + as_f32(r[1]);
}

constexpr int DPP_ROR4 = 0x124, DPP_ROR8 = 0x128;      // row_ror: lane i of a 16-lane row reads lane (i + n) % 16

// Sum / maximum over the 16 row groups of a wavefront (lanes with the same lane % 4): every lane ends with the total
// of its CT columns, bit-identical across the lanes of a column (each step combines a pair symmetrically).
template <class T, int K, bool MAX>
__device__ __forceinline__ void gga_col_allreduce(float (&p)[K][T::CT]) {
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
        for (int e = 0; e < T::CT; ++e) {
            float v = p[k][e];
            v = MAX ? fmaxf(v, dpp<DPP_ROR8>(v)) : v + dpp<DPP_ROR8>(v);
            v = MAX ? fmaxf(v, dpp<DPP_ROR4>(v)) : v + dpp<DPP_ROR4>(v);
            p[k][e] = gga_pair32<MAX>(gga_pair16<MAX>(v));
        }
}

// ---------------------------------------------------------------------------------------------------------------
// a thread's CT codes of one row: NB = CT B / 8 bytes, little-endian bit string
// ---------------------------------------------------------------------------------------------------------------
template <int NB>
__device__ __forceinline__ uint64_t gga_load_bytes(const uint8_t* p) {
    if constexpr (NB == 8) {
        const uint2 v = *reinterpret_cast<const uint2*>(p);
        return uint64_t(v.x) | (uint64_t(v.y) << 32);
    } else if constexpr (NB == 4) {
        return *reinterpret_cast<const uint32_t*>(p);
    } else if constexpr (NB == 2) {
        return *reinterpret_cast<const uint16_t*>(p);
    } else if constexpr (NB == 1) {
        return *p;
    } else if constexpr (NB == 6) {
        const uint16_t* h = reinterpret_cast<const uint16_t*>(p);
        return uint64_t(h[0]) | (uint64_t(h[1]) << 16) | (uint64_t(h[2]) << 32);
    } else {
        static_assert(NB == 3, "bytes per thread and row");
        return uint64_t(p[0]) | (uint64_t(p[1]) << 8) | (uint64_t(p[2]) << 16);
    }
}
template <int NB>
__device__ __forceinline__ void gga_store_bytes(uint8_t* p, uint64_t v) {
    if constexpr (NB == 8) {
        *reinterpret_cast<uint2*>(p) = make_uint2(uint32_t(v), uint32_t(v >> 32));
    } else if constexpr (NB == 4) {
        *reinterpret_cast<uint32_t*>(p) = uint32_t(v);
    } else if constexpr (NB == 2) {
        *reinterpret_cast<uint16_t*>(p) = uint16_t(v);
    } else if constexpr (NB == 1) {
        *p = uint8_t(v);
    } else if constexpr (NB == 6) {
        uint16_t* h = reinterpret_cast<uint16_t*>(p);
        h[0] = uint16_t(v);
        h[1] = uint16_t(v >> 16);
        h[2] = uint16_t(v >> 32);
    } else {
        static_assert(NB == 3, "bytes per thread and row");
        p[0] = uint8_t(v);
        p[1] = uint8_t(v >> 8);
        p[2] = uint8_t(v >> 16);
    }
}

// Head state of width B at S -> the thread's x[s][e] (reference: `_load_head`, _gga_triton.py:131-143).
template <class T, int B>
__device__ __forceinline__ void gga_load_head(const uint8_t* S, const GgaThread& t, float (&x)[T::RPT][T::CT]) {
    constexpr int CT = T::CT, RPT = T::RPT, DK = T::DK, DV = T::DV;
    if constexpr (B == 16) {
        const uint16_t* H = reinterpret_cast<const uint16_t*>(S);
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const int i = s * 16 + t.tr;
#pragma unroll
            for (int e4 = 0; e4 < CT; e4 += 4) {
                const uint2 v = *reinterpret_cast<const uint2*>(H + i * DV + t.tc * CT + e4);
                x[s][e4 + 0] = f16_to_f32(uint16_t(v.x));
                x[s][e4 + 1] = f16_to_f32(uint16_t(v.x >> 16));
                x[s][e4 + 2] = f16_to_f32(uint16_t(v.y));
                x[s][e4 + 3] = f16_to_f32(uint16_t(v.y >> 16));
            }
        }
    } else {
        constexpr int NB = CT * B / 8;
        constexpr int RB = DV * B / 8;                                     // bytes of a row of codes
        const uint16_t* R = reinterpret_cast<const uint16_t*>(S + gga_code_bytes(B, DK, DV));
        const uint16_t* C = R + (B == 2 ? DK * T::NG : DK);
        uint64_t raw[RPT];
        uint16_t rr[RPT];
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const int i = s * 16 + t.tr;
            raw[s] = gga_load_bytes<NB>(S + i * RB + t.tc * NB);
            rr[s] = B == 2 ? R[i * T::NG + (t.tc * CT) / GGA_GROUP] : R[i];
        }
        float c[CT];
#pragma unroll
        for (int e = 0; e < CT; ++e) c[e] = f16_to_f32(C[t.tc * CT + e]);
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const float r = f16_to_f32(rr[s]);
#pragma unroll
            for (int e = 0; e < CT; ++e) {
                const int u = int((raw[s] >> (e * B)) & ((1u << B) - 1));
                const float z = B == 2 ? float(2 * u - 3) : float(u - gga_qmax(B));
                x[s][e] = (r * c[e]) * z;
            }
        }
    }
}

template <int B>
__device__ __forceinline__ float gga_encode(float y) {
    if constexpr (B == 2) return (y >= 0.0f ? 1.0f : -1.0f) * (fabsf(y) >= 2.0f ? 3.0f : 1.0f);
    else return fminf(fmaxf(rintf(y), -float(gga_qmax(B))), float(gga_qmax(B)));
}

// STEP's dual-axis fit of the thread block's tile x at width B, packed at S (reference: `_store_head` ->
// `_fit_parts`): row factors r = half(sqrt(max(mean_j |x|, 1e-20) / w)), column factors c = half(max_i |x / r| /
// qmax), codes, one w^2-weighted least-squares refit of c with the codes fixed, codes again.  Divisions and the
// square root are IEEE, as in torch.  `wrow[s]` = w of the thread's rows.
template <class T, int B>
__device__ __forceinline__ void gga_fit_store(uint8_t* S, float (&x)[T::RPT][T::CT], const float (&wrow)[T::RPT],
                                              float* red, const GgaThread& t) {
    constexpr int CT = T::CT, RPT = T::RPT, DK = T::DK, DV = T::DV;
    if constexpr (B == 16) {
        uint16_t* H = reinterpret_cast<uint16_t*>(S);
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const int i = s * 16 + t.tr;
#pragma unroll
            for (int e4 = 0; e4 < CT; e4 += 4) {
                uint2 v;
                v.x = uint32_t(f32_to_f16(x[s][e4])) | (uint32_t(f32_to_f16(x[s][e4 + 1])) << 16);
                v.y = uint32_t(f32_to_f16(x[s][e4 + 2])) | (uint32_t(f32_to_f16(x[s][e4 + 3])) << 16);
                *reinterpret_cast<uint2*>(H + i * DV + t.tc * CT + e4) = v;
            }
        }
    } else {
        constexpr int NB = CT * B / 8;
        constexpr int RB = DV * B / 8;
        constexpr float QMAX = float(gga_qmax(B));
        constexpr int RN = B == 2 ? GGA_GROUP / CT : 16;                    // threads sharing one row factor
        uint16_t* R = reinterpret_cast<uint16_t*>(S + gga_code_bytes(B, DK, DV));
        uint16_t* C = R + (B == 2 ? DK * T::NG : DK);
        float rf[RPT], asum[RPT];
        float y0[RPT][CT];
        float cmax[1][CT];
#pragma unroll
        for (int e = 0; e < CT; ++e) cmax[0][e] = 0.0f;
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            float a = 0.0f;
#pragma unroll
            for (int e = 0; e < CT; ++e) a = a + fabsf(x[s][e]);
            asum[s] = block_sum<4>(a);                      // over the wavefront's 4 CT columns
        }
        constexpr bool OWN = B == 2 && 4 * CT >= GGA_GROUP;       // a two-bit group lies inside one wavefront's columns
        if constexpr (!OWN) {
            if ((t.lane & 3) == 0) {
#pragma unroll
                for (int s = 0; s < RPT; ++s) red[(s * 16 + t.tr) * GGA_WAVES + t.wave] = asum[s];
            }
            __syncthreads();
#pragma unroll
            for (int s = 0; s < RPT; ++s) {
                const float4 w4 = *reinterpret_cast<const float4*>(red + (s * 16 + t.tr) * GGA_WAVES);
                if constexpr (B == 2) asum[s] = t.wave < 2 ? w4.x + w4.y : w4.z + w4.w;     // d_v = 64: two wavefronts
                else asum[s] = (w4.x + w4.y) + (w4.z + w4.w);
            }
        }
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const float a = asum[s] * (1.0f / float(RN * CT));
            rf[s] = gga_half(sqrtf(fmaxf(a, 1e-20f) / wrow[s]));
            const float rrc = gga_rcp_f16(rf[s]);
#pragma unroll
            for (int e = 0; e < CT; ++e) {
                y0[s][e] = gga_div(x[s][e], rf[s], rrc);
                cmax[0][e] = fmaxf(cmax[0][e], fabsf(y0[s][e]));
            }
        }
        gga_col_allreduce<T, 1, true>(cmax);
        float c[CT], crc[CT];
        float nd[2][CT];
#pragma unroll
        for (int e = 0; e < CT; ++e) {
            // max_i (|y| / qmax) = (max_i |y|) / qmax: division is monotonic
            c[e] = gga_half(gga_div(cmax[0][e], QMAX, 1.0f / QMAX));
            crc[e] = gga_rcp_f16(c[e]);
            nd[0][e] = nd[1][e] = 0.0f;
        }
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const float ww = wrow[s] * wrow[s];
#pragma unroll
            for (int e = 0; e < CT; ++e) {
                const float vv = rf[s] * gga_encode<B>(gga_div(y0[s][e], c[e], crc[e]));
                nd[0][e] = __builtin_fmaf(ww * vv, x[s][e], nd[0][e]);
                nd[1][e] = __builtin_fmaf(ww, vv * vv, nd[1][e]);
            }
        }
        gga_col_allreduce<T, 2, false>(nd);
#pragma unroll
        for (int e = 0; e < CT; ++e) {
            c[e] = gga_half(nd[1][e] > 0.0f ? nd[0][e] / fmaxf(nd[1][e], 1e-30f) : c[e]);
            crc[e] = gga_rcp_f16(c[e]);
        }
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const int i = s * 16 + t.tr;
            uint64_t bits = 0;
#pragma unroll
            for (int e = 0; e < CT; ++e) {
                const float z = gga_encode<B>(gga_div(y0[s][e], c[e], crc[e]));
                const int u = B == 2 ? (int(z) + 3) >> 1 : int(z) + gga_qmax(B);
                bits |= uint64_t(uint32_t(u)) << (e * B);
            }
            gga_store_bytes<NB>(S + i * RB + t.tc * NB, bits);
            if (B == 2) {
                if ((t.tc & (RN - 1)) == 0) R[i * T::NG + (t.tc * CT) / GGA_GROUP] = f32_to_f16(rf[s]);
            } else if (t.tc == 0) {
                R[i] = f32_to_f16(rf[s]);
            }
        }
        if (t.tr == 0) {
#pragma unroll
            for (int e = 0; e < CT; ++e) C[t.tc * CT + e] = f32_to_f16(c[e]);
        }
    }
}

template <class T>
__device__ __forceinline__ void gga_load_any(const uint8_t* S, int bits, const GgaThread& t, float (&x)[T::RPT][T::CT]) {
    if (bits == 16) gga_load_head<T, 16>(S, t, x);
    else if (bits == 8) gga_load_head<T, 8>(S, t, x);
    else if (bits == 6) gga_load_head<T, 6>(S, t, x);
    else if (bits == 4) gga_load_head<T, 4>(S, t, x);
    else gga_load_head<T, 2>(S, t, x);
}
template <class T>
__device__ __forceinline__ void gga_store_any(uint8_t* S, int bits, float (&x)[T::RPT][T::CT], const float (&wrow)[T::RPT],
                                              float* red, const GgaThread& t) {
    if (bits == 16) gga_fit_store<T, 16>(S, x, wrow, red, t);
    else if (bits == 8) gga_fit_store<T, 8>(S, x, wrow, red, t);
    else if (bits == 6) gga_fit_store<T, 6>(S, x, wrow, red, t);
    else if (bits == 4) gga_fit_store<T, 4>(S, x, wrow, red, t);
    else gga_fit_store<T, 2>(S, x, wrow, red, t);
}

// ---------------------------------------------------------------------------------------------------------------
// FP8 (E4M3, finite, no infinities) vectors, one wavefront per vector, N elements per lane (reference: `_fp8_enc`,
// _gga_triton.py:182-190; torch's cast rounds to nearest even, and so does the hardware conversion)
// ---------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float fp8_to_f32(uint32_t byte) { return __builtin_amdgcn_cvt_f32_fp8(int(byte), 0); }
__device__ __forceinline__ uint32_t f32_to_fp8(float y) {
    return uint32_t(__builtin_amdgcn_cvt_pk_fp8_f32(y, 0.0f, 0, false)) & 0xFFu;
}
// codes, scale s = amax / 448 and the reconstruction of x (0 -> 0)
template <int N>
__device__ __forceinline__ float fp8_encode(const float (&x)[N], uint32_t (&code)[N], float (&rec)[N]) {
    float am = 0.0f;
#pragma unroll
    for (int t = 0; t < N; ++t) am = fmaxf(am, fabsf(x[t]));
    const float s = wave_max(am) / 448.0f;
    const float safe = s > 0.0f ? s : 1.0f;
#pragma unroll
    for (int t = 0; t < N; ++t) {
        code[t] = f32_to_fp8(fminf(fmaxf(x[t] / safe, -448.0f), 448.0f));
        rec[t] = s > 0.0f ? fp8_to_f32(code[t]) * safe : 0.0f;
    }
    return s;
}
template <int N>
__device__ __forceinline__ void fp8_store(uint8_t* p, int lane, const uint32_t (&code)[N]) {
    if constexpr (N == 2) reinterpret_cast<uint16_t*>(p)[lane] = uint16_t(code[0] | (code[1] << 8));
    else p[lane] = uint8_t(code[0]);
}
template <int N>
__device__ __forceinline__ void fp8_load(const uint8_t* p, int lane, uint32_t (&code)[N]) {
    if constexpr (N == 2) {
        const uint32_t v = reinterpret_cast<const uint16_t*>(p)[lane];
        code[0] = v & 0xFFu;
        code[1] = v >> 8;
    } else {
        code[0] = p[lane];
    }
}

// ---------------------------------------------------------------------------------------------------------------
// the decode step
// ---------------------------------------------------------------------------------------------------------------
template <class T>
struct GgaLds {
    float kn[T::DK], qn[T::DK], r0[T::DK];
    float coef[GGA_MMAX];
    float red[GGA_WAVES * T::DK];                 // the fit's row sums: one partial per wavefront and row
};

template <class T>
__global__ __launch_bounds__(GGA_THREADS, 2) void gga_step_kernel(const GgaParams p) {
    constexpr int CT = T::CT, RPT = T::RPT, DK = T::DK, DV = T::DV, NE = T::NE, NV = T::NV;
    __shared__ __attribute__((aligned(16))) GgaLds<T> L;
    const GgaThread t = gga_thread();
    // head-major order: workgroups that run together work on the same head, hence on the same width, and share the
    // instructions of one of the five width paths (each path is ~40 KB of straight-line code)
    const uint32_t h = blockIdx.x / uint32_t(p.rows), b = blockIdx.x - h * uint32_t(p.rows);
    const uint32_t bh = b * uint32_t(p.hv) + h;
    const uint32_t hk = h / uint32_t(p.gqa);
    void* const outp = advance(p.out, p.out_dt, uint64_t(bh) * DV);
    const int32_t seq = p.idx[b];
    if (seq <= 0) {
        if (t.tid < DV) store_f(outp, p.out_dt, t.tid, 0.0f);
        return;
    }
    uint8_t* const base = p.blob + uint64_t(seq) * p.slot_stride;
    const int bits = p.bits[h];
    uint8_t* const S = base + p.offs[h];
    const bool window = p.pw && bits != 16;
    const int m = p.m;
    int n = 0, hd = 0;
    if (window) {
        n = reinterpret_cast<const int32_t*>(base)[0];
        hd = reinterpret_cast<const int32_t*>(base)[1];
        n = n < 0 ? 0 : n > m ? m : n;
        hd = hd < 0 ? 0 : hd >= m ? m - 1 : hd;
    }
    uint8_t* const qb = base + p.qoff + uint64_t(h) * p.qsz;
    uint8_t* const PP = qb;
    uint8_t* const VP = qb + m * DK;
    float* const PS = reinterpret_cast<float*>(qb + m * (DK + DV));
    float* const VS = PS + m;

    // ---- q, k of the key head (every wavefront on its own: lane l holds elements l NE .. l NE + NE - 1), gates ----
    const void* qp = advance(p.q, p.q_dt, uint64_t(b) * p.s_q + hk * DK);
    const void* kp = advance(p.k, p.k_dt, uint64_t(b) * p.s_k + hk * DK);
    uint32_t qr[NE], kr[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        qr[e] = load_raw(qp, p.q_dt, t.lane * NE + e);
        kr[e] = load_raw(kp, p.k_dt, t.lane * NE + e);
    }
    const uint32_t ar = load_raw_uniform(p.a, p.a_dt, uint64_t(b) * p.s_a + h);
    const uint32_t btr = load_raw_uniform(p.bt, p.bt_dt, uint64_t(b) * p.s_bt + h);
    const uint32_t alr = load_raw_uniform(p.A_log, p.A_log_dt, h);
    const uint32_t dbr = load_raw_uniform(p.dt_bias, p.dt_bias_dt, h);
    // the thread's columns of v, and of the queued right factors
    const void* vp = advance(p.v, p.v_dt, uint64_t(b) * p.s_v + h * DV);
    uint32_t vr[CT];
#pragma unroll
    for (int e = 0; e < CT; ++e) vr[e] = load_raw(vp, p.v_dt, t.tc * CT + e);
    uint32_t vq[GGA_MMAX][CT / 4];
    float vs[GGA_MMAX];
    if (window) {
#pragma unroll
        for (int oi = 0; oi < GGA_MMAX; ++oi) {
            const int jj = (hd + oi) % m;
            const bool live = oi < n;
#pragma unroll
            for (int w4 = 0; w4 < CT / 4; ++w4)
                vq[oi][w4] = live ? reinterpret_cast<const uint32_t*>(VP + jj * DV + t.tc * CT)[w4] : 0u;
            vs[oi] = live ? VS[jj] : 0.0f;
        }
    }
    float wrow[RPT];
#pragma unroll
    for (int s = 0; s < RPT; ++s) wrow[s] = p.w[h * DK + s * 16 + t.tr];

    float x[RPT][CT];
    gga_load_any<T>(S, bits, t, x);

    float qe[NE], ke[NE], ssq = 0.0f, ssk = 0.0f;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        qe[e] = raw_to_f(qr[e], p.q_dt);
        ke[e] = raw_to_f(kr[e], p.k_dt);
        ssq = __builtin_fmaf(qe[e], qe[e], ssq);
        ssk = __builtin_fmaf(ke[e], ke[e], ssk);
    }
    const float nq = sqrtf(wave_sum(ssq) + 1e-6f);
    const float nk = sqrtf(wave_sum(ssk) + 1e-6f);
    float a, beta;
    if (p.gate) {
        const float xg = raw_to_f(ar, p.a_dt) + raw_to_f(dbr, p.dt_bias_dt);
        const float sp = xg <= 20.0f ? logf(1.0f + expf(xg)) : xg;
        a = expf(-expf(raw_to_f(alr, p.A_log_dt)) * sp);
        beta = 1.0f / (1.0f + expf(-raw_to_f(btr, p.bt_dt)));
    } else {
        a = expf(raw_to_f(ar, p.a_dt));
        beta = raw_to_f(btr, p.bt_dt);
    }
    float bke[NE], bkq = 0.0f;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        qe[e] = qe[e] / nq * p.scale;
        ke[e] = ke[e] / nk;
        bke[e] = beta * ke[e];
        bkq = bkq + bke[e] * qe[e];
    }
    bkq = wave_sum(bkq);
    if (t.wave == 0) {
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            L.kn[t.lane * NE + e] = ke[e];
            L.qn[t.lane * NE + e] = qe[e];
        }
    }

    // ---- the queued left factors: propagate, re-encode, read out (wavefront w: entries w, w + 4) ----
    const bool full = window && n == m;
    if (window) {
        for (int oi = t.wave; oi < n; oi += GGA_WAVES) {
            const int jj = (hd + oi) % m;
            uint32_t code[NE];
            fp8_load<NE>(PP + jj * DK, t.lane, code);
            const float ps = PS[jj];
            float pv[NE], kpp = 0.0f;
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                pv[e] = fp8_to_f32(code[e]) * ps;
                kpp = kpp + ke[e] * pv[e];
            }
            kpp = wave_sum(kpp);
            float ap[NE], rec[NE];
#pragma unroll
            for (int e = 0; e < NE; ++e) ap[e] = a * (pv[e] - bke[e] * kpp);
            const float sc = fp8_encode<NE>(ap, code, rec);
            if (!(full && oi == 0)) {                      // the oldest pair of a full window leaves it below
                fp8_store<NE>(PP + jj * DK, t.lane, code);
                if (t.lane == 0) PS[jj] = sc;
            }
            float cf = 0.0f;
#pragma unroll
            for (int e = 0; e < NE; ++e) cf = cf + rec[e] * qe[e];
            cf = wave_sum(cf);
            if (t.lane == 0) L.coef[oi] = cf;
            if (oi == 0) {
#pragma unroll
                for (int e = 0; e < NE; ++e) L.r0[t.lane * NE + e] = rec[e];
            }
        }
    }
    __syncthreads();

    // ---- O_pre = a (O - beta k (k^T O)), its read-out ----
    float krow[RPT], qrow[RPT];
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
        krow[s] = L.kn[s * 16 + t.tr];
        qrow[s] = L.qn[s * 16 + t.tr];
    }
    float acc[1][CT];
#pragma unroll
    for (int e = 0; e < CT; ++e) acc[0][e] = 0.0f;
#pragma unroll
    for (int s = 0; s < RPT; ++s)
#pragma unroll
        for (int e = 0; e < CT; ++e) acc[0][e] = __builtin_fmaf(krow[s], x[s][e], acc[0][e]);
    gga_col_allreduce<T, 1, false>(acc);
    float kO[CT];
#pragma unroll
    for (int e = 0; e < CT; ++e) {
        kO[e] = acc[0][e];
        acc[0][e] = 0.0f;
    }
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
        const float bk = beta * krow[s];
#pragma unroll
        for (int e = 0; e < CT; ++e) {
            x[s][e] = a * __builtin_fmaf(-bk, kO[e], x[s][e]);
            acc[0][e] = __builtin_fmaf(x[s][e], qrow[s], acc[0][e]);
        }
    }
    gga_col_allreduce<T, 1, false>(acc);
    float ve[CT], o[CT];
#pragma unroll
    for (int e = 0; e < CT; ++e) {
        ve[e] = raw_to_f(vr[e], p.v_dt);
        o[e] = acc[0][e] + bkq * ve[e];
    }

    if (window) {
        // read-out of the queued pairs (oldest first), the merge of the evicted one
#pragma unroll
        for (int oi = 0; oi < GGA_MMAX; ++oi) {
            if (oi < n) {
                const float cf = L.coef[oi];
#pragma unroll
                for (int e = 0; e < CT; ++e) {
                    const float vt = fp8_to_f32((vq[oi][e / 4] >> (8 * (e % 4))) & 0xFFu) * vs[oi];
                    o[e] = o[e] + cf * vt;
                }
            }
        }
        if (full) {
            float v0[CT];
#pragma unroll
            for (int e = 0; e < CT; ++e) v0[e] = fp8_to_f32((vq[0][e / 4] >> (8 * (e % 4))) & 0xFFu) * vs[0];
#pragma unroll
            for (int s = 0; s < RPT; ++s) {
                const float r0 = L.r0[s * 16 + t.tr];
#pragma unroll
                for (int e = 0; e < CT; ++e) x[s][e] = __builtin_fmaf(r0, v0[e], x[s][e]);
            }
        }
    } else {
        // pivots and slots without a window: the new write goes into the state
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
            const float bk = beta * krow[s];
#pragma unroll
            for (int e = 0; e < CT; ++e) x[s][e] = __builtin_fmaf(bk, ve[e], x[s][e]);
        }
    }
    if (t.tr == 0) {
#pragma unroll
        for (int e = 0; e < CT; ++e) store_f(outp, p.out_dt, t.tc * CT + e, o[e]);
    }

    // ---- re-fit and re-pack in place ----
    gga_store_any<T>(S, bits, x, wrow, L.red, t);

    // ---- queue (R(beta k), R(v)).  A full window's new pair replaces the oldest one, whose right factor every
    // wavefront has read for the merge: the barrier puts the store behind all of those reads (each wavefront used its
    // copy before it got here).
    if (window) {
        __syncthreads();
        const int jn = n < m ? (hd + n) % m : hd;
        if (t.wave == 0) {
            uint32_t code[NE];
            float rec[NE];
            const float sc = fp8_encode<NE>(bke, code, rec);
            fp8_store<NE>(PP + jn * DK, t.lane, code);
            if (t.lane == 0) PS[jn] = sc;
        } else if (t.wave == 1) {
            float vv[NV];
#pragma unroll
            for (int e = 0; e < NV; ++e) vv[e] = raw_to_f(load_raw(vp, p.v_dt, t.lane * NV + e), p.v_dt);
            uint32_t code[NV];
            float rec[NV];
            const float sc = fp8_encode<NV>(vv, code, rec);
            fp8_store<NV>(VP + jn * DV, t.lane, code);
            if (t.lane == 0) VS[jn] = sc;
        }
    }
}

// Counters of the stepped slots, after the step (all heads of a slot read them): reference `_gga_advance`.
template <class T>
__global__ void gga_advance_kernel(uint8_t* blob, uint64_t slot_stride, const int32_t* idx, int rows, int m) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= rows) return;
    const int32_t seq = idx[b];
    if (seq <= 0) return;
    int32_t* ct = reinterpret_cast<int32_t*>(blob + uint64_t(seq) * slot_stride);
    const int n = ct[0], hd = ct[1];
    ct[0] = n + 1 < m ? n + 1 : m;
    ct[1] = n == m ? (hd + 1) % m : hd;
}

// Fit + pack canonical states X [rows, hv, d_k, d_v] fp32 into slots idx; zero the counters (reference `_gga_store`).
template <class T>
__global__ __launch_bounds__(GGA_THREADS, 2) void gga_store_kernel(const GgaParams p) {
    constexpr int CT = T::CT, RPT = T::RPT, DK = T::DK, DV = T::DV;
    __shared__ __attribute__((aligned(16))) float red[GGA_WAVES * DK];
    const GgaThread t = gga_thread();
    // head-major order: workgroups that run together work on the same head, hence on the same width, and share the
    // instructions of one of the five width paths (each path is ~40 KB of straight-line code)
    const uint32_t h = blockIdx.x / uint32_t(p.rows), b = blockIdx.x - h * uint32_t(p.rows);
    const uint32_t bh = b * uint32_t(p.hv) + h;
    const int32_t seq = p.idx[b];
    if (seq <= 0) return;
    uint8_t* const base = p.blob + uint64_t(seq) * p.slot_stride;
    const float* X = p.X + uint64_t(bh) * (DK * DV);
    float x[RPT][CT], wrow[RPT];
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
        const int i = s * 16 + t.tr;
        wrow[s] = p.w[h * DK + i];
#pragma unroll
        for (int e4 = 0; e4 < CT; e4 += 4) {
            const float4 v = *reinterpret_cast<const float4*>(X + i * DV + t.tc * CT + e4);
            x[s][e4] = v.x; x[s][e4 + 1] = v.y; x[s][e4 + 2] = v.z; x[s][e4 + 3] = v.w;
        }
    }
    gga_store_any<T>(base + p.offs[h], p.bits[h], x, wrow, red, t);
    if (h == 0 && t.tid < 2) reinterpret_cast<int32_t*>(base)[t.tid] = 0;
}

// Unpack slots idx into canonical fp32 Y [rows, hv, d_k, d_v]: the stored state without the window (`_gga_load`).
template <class T>
__global__ __launch_bounds__(GGA_THREADS, 2) void gga_load_kernel(const GgaParams p) {
    constexpr int CT = T::CT, RPT = T::RPT, DK = T::DK, DV = T::DV;
    const GgaThread t = gga_thread();
    // head-major order: workgroups that run together work on the same head, hence on the same width, and share the
    // instructions of one of the five width paths (each path is ~40 KB of straight-line code)
    const uint32_t h = blockIdx.x / uint32_t(p.rows), b = blockIdx.x - h * uint32_t(p.rows);
    const uint32_t bh = b * uint32_t(p.hv) + h;
    const int32_t seq = p.idx[b];
    float* Y = p.Y + uint64_t(bh) * (DK * DV);
    float x[RPT][CT];
    if (seq > 0) {
        gga_load_any<T>(p.blob + uint64_t(seq) * p.slot_stride + p.offs[h], p.bits[h], t, x);
    } else {
#pragma unroll
        for (int s = 0; s < RPT; ++s)
#pragma unroll
            for (int e = 0; e < CT; ++e) x[s][e] = 0.0f;
    }
#pragma unroll
    for (int s = 0; s < RPT; ++s)
#pragma unroll
        for (int e4 = 0; e4 < CT; e4 += 4)
            *reinterpret_cast<float4*>(Y + (s * 16 + t.tr) * DV + t.tc * CT + e4) =
                make_float4(x[s][e4], x[s][e4 + 1], x[s][e4 + 2], x[s][e4 + 3]);
}

// op: 0 step (+ advance), 1 store, 2 load
template <class T>
int launch_gga(const GgaParams& p, int op, hipStream_t stream) {
    const dim3 grid(p.rows * p.hv), block(GGA_THREADS);
    if (op == 0) {
        hipLaunchKernelGGL(gga_step_kernel<T>, grid, block, 0, stream, p);
        if (p.pw)
            hipLaunchKernelGGL(gga_advance_kernel<T>, dim3((p.rows + 63) / 64), dim3(64), 0, stream, p.blob, p.slot_stride,
                               p.idx, p.rows, p.m);
    } else if (op == 1) {
        hipLaunchKernelGGL(gga_store_kernel<T>, grid, block, 0, stream, p);
    } else {
        hipLaunchKernelGGL(gga_load_kernel<T>, grid, block, 0, stream, p);
    }
    return int(hipGetLastError());
}

}  // namespace sq
