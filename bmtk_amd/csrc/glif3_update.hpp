// The GLIF3 per-element update shared by the stand-alone step kernel and the
// fused simulation kernels.  Restates NEST glif_psc::update for
// after_spike_currents only (how bmtk instantiates nest:glif_lif_asc_psc,
// bmtk/simulator/pointnet/glif_utils.py:301-320).  The operation order is fixed
// and the file is compiled with -ffp-contract=off, so results are reproducible
// to the bit against a scalar fp32 evaluation of the same expressions.
#pragma once

#include "common.hpp"

namespace bmtk {

struct Glif3Elem {
    float V, asc[GLIF3_NASC], y1[GLIF3_NREC], y2[GLIF3_NREC];
    int ref;
};

// Propagators of one table column, loaded once per element.
struct Glif3Prop {
    float P33, P30, th, Ur;
    int n_ref;
    float c[GLIF3_NASC], d[GLIF3_NASC], r[GLIF3_NASC], amp[GLIF3_NASC];
    float P11[GLIF3_NREC], P31[GLIF3_NREC], P32[GLIF3_NREC], psc0[GLIF3_NREC];

    __device__ __forceinline__ void load(const float *__restrict__ prop, int64_t stride, int64_t col)
    {
        const float *p = prop + col;
        P33 = p[GLIF3_P33 * stride];
        P30 = p[GLIF3_P30 * stride];
        th = p[GLIF3_TH * stride];
        Ur = p[GLIF3_UR * stride];
        n_ref = (int)p[GLIF3_NREF * stride];
#pragma unroll
        for (int a = 0; a < GLIF3_NASC; ++a) {
            c[a] = p[(GLIF3_C0 + a) * stride];
            d[a] = p[(GLIF3_D0 + a) * stride];
            r[a] = p[(GLIF3_R0 + a) * stride];
            amp[a] = p[(GLIF3_AMP0 + a) * stride];
        }
#pragma unroll
        for (int k = 0; k < GLIF3_NREC; ++k) {
            P11[k] = p[(GLIF3_P11_0 + k) * stride];
            P31[k] = p[(GLIF3_P31_0 + k) * stride];
            P32[k] = p[(GLIF3_P32_0 + k) * stride];
            psc0[k] = p[(GLIF3_PSC0_0 + k) * stride];
        }
    }
};

// A class table small enough for LDS is copied there as it lies in device memory, [quantity][class], sixteen bytes
// per lane and load, four loads asked for before the first is stored; ``prop`` must be 16-byte aligned.  Threads of
// one wavefront then read a quantity of their own classes: two lanes meet in a bank only when their classes differ
// by a multiple of the bank count, with this layout as with a transposed one.  The caller synchronises.
template <int kThreads>
__device__ __forceinline__ void stage_class_table(float *__restrict__ lds, const float *__restrict__ prop, int n_words)
{
    const int n4 = n_words >> 2;
    const float4 *src = reinterpret_cast<const float4 *>(prop);
    float4 *dst = reinterpret_cast<float4 *>(lds);
    for (int base = 0; base < n4; base += 4 * kThreads) {
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = base + j * kThreads + (int)threadIdx.x;
            v[j] = src[i < n4 ? i : 0];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = base + j * kThreads + (int)threadIdx.x;
            if (i < n4) dst[i] = v[j];
        }
    }
    for (int i = (n4 << 2) + (int)threadIdx.x; i < n_words; i += kThreads) lds[i] = prop[i];
}

// Advance one element by one step.  syn[r]: weight sum arriving on receptor r
// in this step; I: external current.  Returns true on a spike and then sets
// *frac to the fraction of the step at which U crossed threshold.
__device__ __forceinline__ bool glif3_update(Glif3Elem &s, const Glif3Prop &p, float h, const float syn[GLIF3_NREC],
                                             float I, float *frac)
{
    const float v_old = s.V;
    float U = v_old;
    bool spike = false;
    if (s.ref > 0) {
        // refractory: U is held; on leaving, U and the after-spike currents are reset
        s.ref -= 1;
        if (s.ref == 0) {
#pragma unroll
            for (int a = 0; a < GLIF3_NASC; ++a) s.asc[a] = p.amp[a] + s.asc[a] * p.r[a];
            U = p.Ur;
        }
    } else {
        float S = 0.0f;
#pragma unroll
        for (int a = 0; a < GLIF3_NASC; ++a) {
            S = S + p.c[a] * s.asc[a];
            s.asc[a] = s.asc[a] * p.d[a];
        }
        U = v_old * p.P33 + (I + S) * p.P30;
#pragma unroll
        for (int k = 0; k < GLIF3_NREC; ++k) U = U + (p.P31[k] * s.y1[k] + p.P32[k] * s.y2[k]);
        if (U > p.th) {
            spike = true;
            s.ref = p.n_ref;
            *frac = (p.th - v_old) / (U - v_old);
        }
    }
    s.V = U;
    // alpha-shaped PSCs advance every step, refractory or not
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        const float P21 = h * p.P11[k];
        const float a1 = s.y1[k], a2 = s.y2[k];
        s.y2[k] = P21 * a1 + p.P11[k] * a2;
        s.y1[k] = a1 * p.P11[k] + syn[k] * p.psc0[k];
    }
    return spike;
}

__device__ __forceinline__ void glif3_load(Glif3Elem &s, const float *V, const float *asc, const float *y1,
                                           const float *y2, const int32_t *ref, int64_t ne, int64_t e)
{
    s.V = V[e];
    s.ref = ref[e];
#pragma unroll
    for (int a = 0; a < GLIF3_NASC; ++a) s.asc[a] = asc[a * ne + e];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        s.y1[k] = y1[k * ne + e];
        s.y2[k] = y2[k * ne + e];
    }
}

__device__ __forceinline__ void glif3_store(const Glif3Elem &s, float *V, float *asc, float *y1, float *y2,
                                            int32_t *ref, int64_t ne, int64_t e)
{
    V[e] = s.V;
    ref[e] = s.ref;
#pragma unroll
    for (int a = 0; a < GLIF3_NASC; ++a) asc[a * ne + e] = s.asc[a];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        y1[k * ne + e] = s.y1[k];
        y2[k * ne + e] = s.y2[k];
    }
}

}  // namespace bmtk
