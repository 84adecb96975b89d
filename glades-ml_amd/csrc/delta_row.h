// Output delta, loss and metrics of one row of at most 64 outputs held one per lane: shared by the
// element-wise output-delta kernel and by the fused kernel of narrow output layers.
#pragma once
#include "ghip_internal.h"

__device__ __forceinline__ float ghip_wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float ghip_wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Row b of the canonical output layer: softmax (if asked), per-sample loss = sum over outputs of the
// reference's cost (gmath.cpp:272-321 without the 1/dataSize), the reference's accuracy term
// (network.cpp:541-547), argmax agreement under gmath.cpp:412-455 with the confusion-matrix count
// (cmatrix.cpp:57-98), and delta = dLoss/dz.  Lane o < a.n passes output o in `v` (pre-softmax logit
// or activated output), the other lanes -3.0e38f, and its target in `yv` (ghip_delta_target: the
// caller may ask for it long before it has the output); all 64 lanes call.  Writes P (if
// a.store_p), D and Dbf as the arguments ask; returns this lane's delta (0 for lanes past the row).
__device__ __forceinline__ float ghip_delta_target(const DeltaArgs& a, int b, int lane)
{
    return (a.Y && lane < a.n) ? a.Y[(long long)b * a.ldy + lane] : 0.0f;
}
__device__ __forceinline__ float ghip_delta_row64(const DeltaArgs& a, int b, int lane, float v, float yv,
                                                  double& loss, double& accs, double& corr)
{
    const bool softmax = a.act == GHIP_SOFTMAX;
    const bool sig_bce = (a.act == GHIP_SIGMOID || a.act == GHIP_SIGMOIDP) && a.cost == GHIP_CLASSIFICATION;
    float* p = a.P + (long long)b * a.ldp;
    const int o = lane;
    float inv = 1.0f;
    if (softmax) {
        const float mx = ghip_wave_max(v);
        v = (o < a.n) ? expf(v - mx) : 0.0f;
        inv = 1.0f / ghip_wave_sum(v);
    }
    float l = 0.0f, ac = 0.0f, d = 0.0f;
    float bp = 0.0f, by = 0.0f;  // running maxima for the argmax rule (start at 0, strict >)
    int ip = 0x7fffffff, iy = 0x7fffffff;
    if (o < a.n) {
        float pv = v;
        if (softmax) {
            pv = pv * inv;
            if (a.store_p) p[o] = pv;
            if (yv != 0.0f) l += -(yv * logf(fmaxf(pv, 1e-30f)));
            d = pv - yv;
        } else {
            l += ghip_cost<false>(yv, pv, 1.0f, a.cost);
            d = sig_bce ? (pv - yv) : ghip_cost_der(yv, pv, a.cost) * ghip_act_der_canon(pv, a.act, a.act_param);
        }
        ac += ghip_accuracy_term(pv, yv);
        if (pv > bp) { bp = pv; ip = o; }
        if (yv > by) { by = yv; iy = o; }
        if (a.D) a.D[(long long)b * a.n + o] = d;
        if (a.Dbf) a.Dbf[(long long)b * (a.ldd ? a.ldd : a.n) + o] = ghip_f32_to_bf16(d);
    }
    // argmax across lanes: largest value, lowest index on ties; "no element above 0" = none
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        float ov = __shfl_xor(bp, s, 64); int oi = __shfl_xor(ip, s, 64);
        if (ov > bp || (ov == bp && oi < ip)) { bp = ov; ip = oi; }
        ov = __shfl_xor(by, s, 64); oi = __shfl_xor(iy, s, 64);
        if (ov > by || (ov == by && oi < iy)) { by = ov; iy = oi; }
    }
    loss += (double)ghip_wave_sum(l);
    accs += (double)ghip_wave_sum(ac);
    if (ip == iy) corr += 1.0;
    // CMatrix::addResult (cmatrix.cpp:57-98): row = expected class, column = predicted
    if (a.cm && lane == 0 && ip != 0x7fffffff && iy != 0x7fffffff) atomicAdd(&a.cm[(long long)iy * a.n + ip], 1);
    return d;
}
