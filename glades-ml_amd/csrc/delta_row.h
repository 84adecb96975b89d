// Output delta, loss and metrics of rows of at most 64 outputs held one per lane: shared by the
// element-wise output-delta kernel, by the fused kernel of narrow output layers and by the persistent
// kernel of narrow networks.  SEG (a power of two, the number of lanes a row takes) lets a wavefront
// finish 64 / SEG rows at once when the rows are short: every cross-lane step stays inside a segment.
#pragma once
#include "ghip_internal.h"

template <int SEG = 64>
__device__ __forceinline__ float ghip_seg_max(float v)
{
#pragma unroll
    for (int o = SEG / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
template <int SEG = 64>
__device__ __forceinline__ float ghip_seg_sum(float v)
{
#pragma unroll
    for (int o = SEG / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float ghip_wave_max(float v) { return ghip_seg_max<64>(v); }
__device__ __forceinline__ float ghip_wave_sum(float v) { return ghip_seg_sum<64>(v); }

// One row of the canonical output layer per segment of SEG lanes: softmax (if asked), per-sample loss = sum
// over outputs of the reference's cost (gmath.cpp:272-321 without the 1/dataSize), the reference's accuracy
// term (network.cpp:541-547), argmax agreement under gmath.cpp:412-455 with the confusion-matrix count
// (cmatrix.cpp:57-98), and delta = dLoss/dz.  The lane at place o < a.n of its segment passes output o of the
// segment's row in `v` (pre-softmax logit or activated output), the other lanes -3.0e38f, and its target in
// `yv`; all 64 lanes call.  `b` is the lane's row where the function stores (P if a.store_p, D, Dbf: as the
// arguments ask).  The row's loss, accuracy-term sum and class agreement are ADDED to loss / accs / corr in
// every lane of the segment (a caller that adds up lanes counts one lane per segment).  Returns the lane's
// delta (0 for lanes past the row).
__device__ __forceinline__ float ghip_delta_target(const DeltaArgs& a, int b, int lane)
{
    return (a.Y && lane < a.n) ? a.Y[(long long)b * a.ldy + lane] : 0.0f;
}
template <int SEG>
__device__ __forceinline__ float ghip_delta_row_seg(const DeltaArgs& a, long long b, int lane, float v, float yv,
                                                    double& loss, double& accs, double& corr)
{
    const bool softmax = a.act == GHIP_SOFTMAX;
    const bool sig_bce = (a.act == GHIP_SIGMOID || a.act == GHIP_SIGMOIDP) && a.cost == GHIP_CLASSIFICATION;
    float* p = a.P + b * a.ldp;
    const int o = lane & (SEG - 1);
    float inv = 1.0f;
    if (softmax) {
        const float mx = ghip_seg_max<SEG>(v);
        v = (o < a.n) ? expf(v - mx) : 0.0f;
        inv = 1.0f / ghip_seg_sum<SEG>(v);
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
        if (a.D) a.D[b * a.n + o] = d;
        if (a.Dbf) a.Dbf[b * (a.ldd ? a.ldd : a.n) + o] = ghip_f32_to_bf16(d);
    }
    // argmax across the segment: largest value, lowest index on ties; "no element above 0" = none
#pragma unroll
    for (int s = SEG / 2; s > 0; s >>= 1) {
        float ov = __shfl_xor(bp, s, 64); int oi = __shfl_xor(ip, s, 64);
        if (ov > bp || (ov == bp && oi < ip)) { bp = ov; ip = oi; }
        ov = __shfl_xor(by, s, 64); oi = __shfl_xor(iy, s, 64);
        if (ov > by || (ov == by && oi < iy)) { by = ov; iy = oi; }
    }
    loss += (double)ghip_seg_sum<SEG>(l);
    accs += (double)ghip_seg_sum<SEG>(ac);
    if (ip == iy) corr += 1.0;
    // CMatrix::addResult (cmatrix.cpp:57-98): row = expected class, column = predicted
    if (a.cm && o == 0 && ip != 0x7fffffff && iy != 0x7fffffff) atomicAdd(&a.cm[(long long)iy * a.n + ip], 1);
    return d;
}
__device__ __forceinline__ float ghip_delta_row64(const DeltaArgs& a, int b, int lane, float v, float yv,
                                                  double& loss, double& accs, double& corr)
{
    return ghip_delta_row_seg<64>(a, b, lane, v, yv, loss, accs, corr);
}
