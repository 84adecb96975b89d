// HBM-bound kernels of the canonical path: output delta / loss / metrics, bias updates of the bf16
// path, precision conversion, transposition, per-row e4m3 quantisation.  (The weight updates live in
// the weight-gradient GEMMs' epilogues.)

#include "ghip_internal.h"
#include "delta_row.h"

namespace {

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ double wave_sum_d(double v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Output layer of the canonical mode: softmax (if asked), per-sample loss = sum over outputs of
// the reference's cost (gmath.cpp:272-321 without the 1/dataSize), the reference's accuracy term
// (network.cpp:541-547), argmax agreement under gmath.cpp:412-455, and delta = dLoss/dz.
// One wavefront per row, kRowsPerWave rows per wavefront, 4 wavefronts per workgroup.  A row of
// up to 64*kRegs outputs is read from memory once and kept in registers (lane j-th value =
// column j*64 + lane): one exp per element, and the softmax passes cost no extra HBM traffic.
constexpr int kRowsPerWave = 2;

template <int kRegs>  // row held in kRegs registers per lane (n <= 64 * kRegs); 0: read from memory on every pass
__global__ void __launch_bounds__(256) output_delta_kernel(DeltaArgs a)
{
    constexpr bool kInRegs = kRegs > 0;
    if (blockIdx.x == 0 && threadIdx.x < 4 && a.acc_clear) a.acc_clear[threadIdx.x] = 0.0;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * 4 + w) * kRowsPerWave;
    double loss = 0.0, accs = 0.0, corr = 0.0;
    const bool softmax = a.act == GHIP_SOFTMAX;
    const bool sig_bce = (a.act == GHIP_SIGMOID || a.act == GHIP_SIGMOIDP) && a.cost == GHIP_CLASSIFICATION;
    for (int rr = 0; rr < kRowsPerWave; ++rr) {
        const int b = row0 + rr;
        if (b >= a.B) break;
        if constexpr (kRegs == 1) {  // a row of at most 64 outputs, one per lane
            ghip_delta_row64(a, b, lane, (lane < a.n) ? a.P[(long long)b * a.ldp + lane] : -3.0e38f, ghip_delta_target(a, b, lane),
                             loss, accs, corr);
            continue;
        }
        float* p = a.P + (long long)b * a.ldp;
        const float* y = a.Y ? a.Y + (long long)b * a.ldy : nullptr;
        float reg[kRegs > 0 ? kRegs : 1];
        float inv = 1.0f, mx = 0.0f;
        if (kInRegs) {
#pragma unroll
            for (int j = 0; j < kRegs; ++j) {
                const int o = j * 64 + lane;
                reg[j] = (o < a.n) ? p[o] : -3.0e38f;
            }
        }
        if (softmax) {
            float m = -3.0e38f;
            if (kInRegs) {
#pragma unroll
                for (int j = 0; j < kRegs; ++j) m = fmaxf(m, reg[j]);
            } else {
                for (int o = lane; o < a.n; o += 64) m = fmaxf(m, p[o]);
            }
            mx = wave_max(m);
            float s = 0.0f;
            if (kInRegs) {
#pragma unroll
                for (int j = 0; j < kRegs; ++j) {
                    const int o = j * 64 + lane;
                    reg[j] = (o < a.n) ? expf(reg[j] - mx) : 0.0f;
                    s += reg[j];
                }
            } else {
                for (int o = lane; o < a.n; o += 64) s += expf(p[o] - mx);
            }
            inv = 1.0f / wave_sum(s);
        }
        float l = 0.0f, ac = 0.0f;
        float bp = 0.0f, by = 0.0f;  // running maxima for the argmax rule (start at 0, strict >)
        int ip = 0x7fffffff, iy = 0x7fffffff;
        auto element = [&](int o, float pv) {
            const float yv = y ? y[o] : 0.0f;
            float d;
            if (softmax) {
                pv = kInRegs ? pv * inv : expf(pv - mx) * inv;
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
        };
        if (kInRegs) {
#pragma unroll
            for (int j = 0; j < kRegs; ++j) {
                const int o = j * 64 + lane;
                if (o < a.n) element(o, reg[j]);
            }
        } else {
            for (int o = lane; o < a.n; o += 64) element(o, p[o]);
        }
        // argmax across lanes: largest value, lowest index on ties; "no element above 0" = none
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            float ov = __shfl_xor(bp, o, 64); int oi = __shfl_xor(ip, o, 64);
            if (ov > bp || (ov == bp && oi < ip)) { bp = ov; ip = oi; }
            ov = __shfl_xor(by, o, 64); oi = __shfl_xor(iy, o, 64);
            if (ov > by || (ov == by && oi < iy)) { by = ov; iy = oi; }
        }
        loss += (double)wave_sum(l);
        accs += (double)wave_sum(ac);
        if (ip == iy) corr += 1.0;
        // CMatrix::addResult (cmatrix.cpp:57-98): row = expected class, column = predicted
        if (a.cm && lane == 0 && ip != 0x7fffffff && iy != 0x7fffffff) atomicAdd(&a.cm[(long long)iy * a.n + ip], 1);
    }
    __shared__ double red[4][3];
    if (lane == 0) { red[w][0] = loss; red[w][1] = accs; red[w][2] = corr; }
    __syncthreads();
    if (threadIdx.x < 3) {
        double v = red[0][threadIdx.x] + red[1][threadIdx.x] + red[2][threadIdx.x] + red[3][threadIdx.x];
        atomicAdd(&a.acc[threadIdx.x], v);
    }
}

// The same for rows whose length is a multiple of 4 and at most 256 * Q: one row per wavefront,
// lane l owns columns 4*(j*64 + l) .. +3 for j < Q.  The row's outputs and targets are requested
// together as 16-byte loads before anything is computed (one memory round trip per row), deltas
// leave as 16-byte (fp32) or 8-byte (bf16) stores.
template <int Q>
__global__ void __launch_bounds__(256) output_delta_vec4_kernel(DeltaArgs a)
{
    if (blockIdx.x == 0 && threadIdx.x < 4 && a.acc_clear) a.acc_clear[threadIdx.x] = 0.0;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    double loss = 0.0, accs = 0.0, corr = 0.0;
    const bool softmax = a.act == GHIP_SOFTMAX;
    const bool sig_bce = (a.act == GHIP_SIGMOID || a.act == GHIP_SIGMOIDP) && a.cost == GHIP_CLASSIFICATION;
    // a bounded grid walks the rows: the three sums reach the accumulators once per workgroup (the
    // same-address double atomics of one workgroup per 4 rows took longer than the rows themselves)
    for (int b = blockIdx.x * 4 + w; b < a.B; b += gridDim.x * 4) {
        float* p = a.P + (long long)b * a.ldp;
        const float* y = a.Y ? a.Y + (long long)b * a.ldy : nullptr;
        float4 pr[Q], yr[Q];
#pragma unroll
        for (int j = 0; j < Q; ++j) {
            const int o = (j * 64 + lane) * 4;
            pr[j] = (o < a.n) ? *reinterpret_cast<const float4*>(p + o) : make_float4(-3.0e38f, -3.0e38f, -3.0e38f, -3.0e38f);
        }
#pragma unroll
        for (int j = 0; j < Q; ++j) {
            const int o = (j * 64 + lane) * 4;
            yr[j] = (y && o < a.n) ? *reinterpret_cast<const float4*>(y + o) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
        float inv = 1.0f;
        if (softmax) {
            float m = -3.0e38f;
#pragma unroll
            for (int j = 0; j < Q; ++j) m = fmaxf(fmaxf(m, fmaxf(pr[j].x, pr[j].y)), fmaxf(pr[j].z, pr[j].w));
            const float mx = wave_max(m);
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < Q; ++j) {
                const bool ok = (j * 64 + lane) * 4 < a.n;
                pr[j].x = ok ? expf(pr[j].x - mx) : 0.0f; pr[j].y = ok ? expf(pr[j].y - mx) : 0.0f;
                pr[j].z = ok ? expf(pr[j].z - mx) : 0.0f; pr[j].w = ok ? expf(pr[j].w - mx) : 0.0f;
                s += (pr[j].x + pr[j].y) + (pr[j].z + pr[j].w);
            }
            inv = 1.0f / wave_sum(s);
        }
        float l = 0.0f, ac = 0.0f;
        float bp = 0.0f, by = 0.0f;  // running maxima for the argmax rule (start at 0, strict >)
        int ip = 0x7fffffff, iy = 0x7fffffff;
        auto element = [&](int o, float& pv, float yv) -> float {
            float d;
            if (softmax) {
                pv = pv * inv;
                if (yv != 0.0f) l += -(yv * logf(fmaxf(pv, 1e-30f)));
                d = pv - yv;
            } else {
                l += ghip_cost<false>(yv, pv, 1.0f, a.cost);
                d = sig_bce ? (pv - yv) : ghip_cost_der(yv, pv, a.cost) * ghip_act_der_canon(pv, a.act, a.act_param);
            }
            ac += ghip_accuracy_term(pv, yv);
            if (pv > bp) { bp = pv; ip = o; }
            if (yv > by) { by = yv; iy = o; }
            return d;
        };
#pragma unroll
        for (int j = 0; j < Q; ++j) {
            const int o = (j * 64 + lane) * 4;
            if (o < a.n) {
                float4 d;
                d.x = element(o, pr[j].x, yr[j].x); d.y = element(o + 1, pr[j].y, yr[j].y);
                d.z = element(o + 2, pr[j].z, yr[j].z); d.w = element(o + 3, pr[j].w, yr[j].w);
                if (a.store_p) *reinterpret_cast<float4*>(p + o) = pr[j];
                if (a.D) *reinterpret_cast<float4*>(a.D + (long long)b * a.n + o) = d;
                if (a.Dbf) {
                    uint2 h;
                    h.x = (uint32_t)ghip_f32_to_bf16(d.x) | ((uint32_t)ghip_f32_to_bf16(d.y) << 16);
                    h.y = (uint32_t)ghip_f32_to_bf16(d.z) | ((uint32_t)ghip_f32_to_bf16(d.w) << 16);
                    *reinterpret_cast<uint2*>(a.Dbf + (long long)b * (a.ldd ? a.ldd : a.n) + o) = h;
                }
            }
        }
        // argmax across lanes: largest value, lowest index on ties; "no element above 0" = none
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            float ov = __shfl_xor(bp, o, 64); int oi = __shfl_xor(ip, o, 64);
            if (ov > bp || (ov == bp && oi < ip)) { bp = ov; ip = oi; }
            ov = __shfl_xor(by, o, 64); oi = __shfl_xor(iy, o, 64);
            if (ov > by || (ov == by && oi < iy)) { by = ov; iy = oi; }
        }
        loss += (double)wave_sum(l);
        accs += (double)wave_sum(ac);
        if (ip == iy) corr += 1.0;
        // CMatrix::addResult (cmatrix.cpp:57-98): row = expected class, column = predicted
        if (a.cm && lane == 0 && ip != 0x7fffffff && iy != 0x7fffffff) atomicAdd(&a.cm[(long long)iy * a.n + ip], 1);
    }
    __shared__ double red[4][3];
    if (lane == 0) { red[w][0] = loss; red[w][1] = accs; red[w][2] = corr; }
    __syncthreads();
    if (threadIdx.x < 3) {
        double v = red[0][threadIdx.x] + red[1][threadIdx.x] + red[2][threadIdx.x] + red[3][threadIdx.x];
        atomicAdd(&a.acc[threadIdx.x], v);
    }
}

// bf16 delta^T, K-blocked [B / 64][n][64]: one wavefront per channel, 16-byte loads (B is a multiple of 64)
__device__ __forceinline__ void bias_from_deltaT(int block, const uint16_t* __restrict__ DT, int n, int B, int batch,
                                                 float* __restrict__ bias, float* __restrict__ vb, float lr, float mom)
{
    const int lane = threadIdx.x & 63;
    const int o = block * 4 + (threadIdx.x >> 6);
    if (o >= n) return;
    // eight 16-byte pieces per plane of 64 batch rows; plane p of channel o starts at (p * n + o) * 64
    auto piece = [&](int k) { return *reinterpret_cast<const uint4*>(DT + ((long long)(k >> 3) * n + o) * 64 + (k & 7) * 8); };
    float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const int nq = B >> 3;
    for (int k0 = 0; k0 < nq; k0 += 256) {  // four independent 16-byte loads in flight per lane
        uint4 q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = k0 + u * 64 + lane;
            q[u] = (k < nq) ? piece(k) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const unsigned int wds[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) s4[u] += __uint_as_float(wds[j] << 16) + __uint_as_float(wds[j] & 0xffff0000u);
        }
    }
    float s = wave_sum((s4[0] + s4[1]) + (s4[2] + s4[3]));
    if (lane == 0) {
        const float g = s / (float)batch;
        const float d = lr * g + mom * vb[o];
        vb[o] = d;
        bias[o] = bias[o] - d;
    }
}

// bias update from per-tile-row partial column sums [tiles][n]: a thread per channel adds them in order
__device__ __forceinline__ void bias_from_partials(int o, const float* __restrict__ part, int tiles, int n, int B,
                                                   float* __restrict__ bias, float* __restrict__ vb, float lr, float mom)
{
    if (o >= n) return;
    float s = 0.0f;
    int k = 0;
    for (; k + 8 <= tiles; k += 8) {  // eight independent loads in flight, added in a fixed order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = part[(long long)(k + u) * n + o];
        s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    }
    for (; k < tiles; ++k) s += part[(long long)k * n + o];
    const float g = s / (float)B;
    const float d = lr * g + mom * vb[o];
    vb[o] = d;
    bias[o] = bias[o] - d;
}

// every layer's bias update of a step: a workgroup finds its layer by its index in the grid
__global__ void __launch_bounds__(256) bias_update_step_kernel(BiasStepArgs a)
{
    int k = 0;
    while (k + 1 < a.count && (int)blockIdx.x >= a.e[k + 1].first_block) ++k;
    const BiasStepArgs::Entry& e = a.e[k];
    const int block = blockIdx.x - e.first_block;
    if (e.part) bias_from_partials(block * 256 + threadIdx.x, e.part, e.tiles, e.n, e.batch, e.bias, e.vb, e.lr, e.mom);
    else bias_from_deltaT(block, e.DT, e.n, e.rows, e.batch, e.bias, e.vb, e.lr, e.mom);
}

template <typename T>
__global__ void __launch_bounds__(256) fill_kernel(T* p, long long n, T v)
{
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long stride = (long long)gridDim.x * 256;
    for (; i < n; i += stride) p[i] = v;
}

// 64x64 tile through LDS: dst[r][c] = bf16(src[r][c]) and the K-blocked transposed copy
// dstT[r / 64][c][r % 64]; src fp32 or bf16
// The source has src_rows x src_cols elements (row pitch src_cols); what lies outside it is written as zero.
template <typename SrcT>
__global__ void __launch_bounds__(256)
convert_transpose_kernel(const SrcT* __restrict__ src, int src_rows, int src_cols, uint16_t* __restrict__ dst,
                         uint16_t* __restrict__ dstT, int rows, int cols)
{
    __shared__ uint16_t tile[64][64 + 2];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int j = ty; j < 64; j += 4) {
        const int r = r0 + j, c = c0 + tx;
        uint16_t v = 0;
        if (r < rows && c < cols) {
            if (r < src_rows && c < src_cols) {
                if (sizeof(SrcT) == 4) v = ghip_f32_to_bf16(((const float*)src)[(long long)r * src_cols + c]);
                else v = ((const uint16_t*)src)[(long long)r * src_cols + c];
            }
            if (dst) dst[(long long)r * cols + c] = v;
        }
        tile[j][tx] = v;
    }
    __syncthreads();
    if (dstT) {
        for (int j = ty; j < 64; j += 4) {
            const int c = c0 + j, r = r0 + tx;
            if (r < rows && c < cols) dstT[((long long)blockIdx.y * cols + c) * 64 + tx] = tile[tx][j];
        }
    }
}

// bf16 transposition (K-blocked destination, dstT[r / 64][c][r % 64]) with 16-byte global accesses: a
// 64 x 64 tile enters LDS row by row (8 lanes per source row) and leaves column by column (each lane
// gathers 8 values of one source column; a tile's 64 destination rows of 128 bytes are contiguous).
// rows and cols are multiples of 64 here; other shapes take the kernel above.
__global__ void __launch_bounds__(256)
bf16_transpose64_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dstT, int rows, int cols)
{
    __shared__ uint16_t tile[64][64 + 2];  // 33 dwords per row: column walks rotate over the banks
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int sub = threadIdx.x & 7, line = threadIdx.x >> 3;  // 8 lanes per 128-byte line, 32 lines per pass
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int r = line + 32 * h;
        const uint4 v = *reinterpret_cast<const uint4*>(src + (long long)(r0 + r) * cols + c0 + sub * 8);
        uint32_t* t32 = reinterpret_cast<uint32_t*>(&tile[r][sub * 8]);
        t32[0] = v.x; t32[1] = v.y; t32[2] = v.z; t32[3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int c = line + 32 * h;  // source column = destination row
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            o[k] = (uint32_t)tile[sub * 8 + 2 * k][c] | ((uint32_t)tile[sub * 8 + 2 * k + 1][c] << 16);
        *reinterpret_cast<uint4*>(dstT + ((long long)blockIdx.y * cols + c0 + c) * 64 + sub * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// one workgroup per row: amax (or a given amax), scale = amax/448, q = e4m3(x / scale)
template <typename SrcT>
__global__ void __launch_bounds__(256)
quant_rows_kernel(const SrcT* __restrict__ src, int rows, int cols, uint8_t* __restrict__ q,
                  float* __restrict__ scale, unsigned int* __restrict__ amax_bits, int consume)
{
    const int r = blockIdx.x;
    const SrcT* x = src + (long long)r * cols;
    __shared__ float red[4];
    float amax;
    if (amax_bits) {
        amax = __uint_as_float(amax_bits[r]);
        if (consume) {  // every lane has its copy: the entry goes back to zero for the next producer
            __syncthreads();
            if (threadIdx.x == 0) amax_bits[r] = 0u;
        }
    } else {
        float m = 0.0f;
        for (int c = threadIdx.x; c < cols; c += 256) {
            float v = (sizeof(SrcT) == 4) ? ((const float*)x)[c] : ghip_bf16_to_f32(((const uint16_t*)x)[c]);
            m = fmaxf(m, fabsf(v));
        }
        m = wave_max(m);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
        __syncthreads();
        amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    }
    const float sc = (amax > 0.0f) ? __fdiv_rn(amax, 448.0f) : 1.0f;
    if (threadIdx.x == 0) scale[r] = sc;
    uint8_t* qr = q + (long long)r * cols;
    for (int c = threadIdx.x; c < cols; c += 256) {
        float v = (sizeof(SrcT) == 4) ? ((const float*)x)[c] : ghip_bf16_to_f32(((const uint16_t*)x)[c]);
        qr[c] = ghip_f32_to_e4m3(__fdiv_rn(v, sc));
    }
}

// The same for bf16 rows whose length is a multiple of 8: 16-byte loads, 8-byte stores, the row
// read from memory once (a thread keeps up to kQuantKeep chunks of 8 values between the amax pass
// and the conversion pass; longer rows re-read the rest), hardware e4m3 conversion (round to
// nearest even; inputs are clamped to +-448 first, so nothing overflows).
constexpr int kQuantKeep = 4;
__device__ __forceinline__ uint32_t e4m3x4(float a, float b, float c, float d)
{
    a = fminf(fmaxf(a, -448.0f), 448.0f); b = fminf(fmaxf(b, -448.0f), 448.0f);
    c = fminf(fmaxf(c, -448.0f), 448.0f); d = fminf(fmaxf(d, -448.0f), 448.0f);
    int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
    return (uint32_t)v;
}
__global__ void __launch_bounds__(256)
quant_rows_bf16x8_kernel(const uint16_t* __restrict__ src, int cols, uint8_t* __restrict__ q,
                         float* __restrict__ scale, unsigned int* __restrict__ amax_bits, int consume)
{
    const int r = blockIdx.x;
    const uint4* x = reinterpret_cast<const uint4*>(src + (long long)r * cols);
    uint2* qr = reinterpret_cast<uint2*>(q + (long long)r * cols);
    const int nchunk = cols >> 3;
    __shared__ unsigned int red[4];
    uint4 keep[kQuantKeep];
#pragma unroll
    for (int u = 0; u < kQuantKeep; ++u) {
        const int c = threadIdx.x + u * 256;
        keep[u] = (c < nchunk) ? x[c] : make_uint4(0u, 0u, 0u, 0u);
    }
    float amax;
    if (amax_bits) {
        amax = __uint_as_float(amax_bits[r]);
        if (consume) {  // every lane has its copy: the entry goes back to zero for the next producer
            __syncthreads();
            if (threadIdx.x == 0) amax_bits[r] = 0u;
        }
    } else {
        // bf16 magnitudes order like their bit patterns
        unsigned int m = 0;
        auto upd = [&](const uint4& v) {
            const unsigned int wds[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const unsigned int lo = wds[j] & 0x7fffu, hi = (wds[j] >> 16) & 0x7fffu;
                m = m > lo ? m : lo;
                m = m > hi ? m : hi;
            }
        };
#pragma unroll
        for (int u = 0; u < kQuantKeep; ++u) upd(keep[u]);
        for (int c = threadIdx.x + kQuantKeep * 256; c < nchunk; c += 256) upd(x[c]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { const unsigned int other = (unsigned int)__shfl_xor((int)m, o, 64); m = m > other ? m : other; }
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
        __syncthreads();
        unsigned int mm = red[0] > red[1] ? red[0] : red[1];
        const unsigned int m2 = red[2] > red[3] ? red[2] : red[3];
        mm = mm > m2 ? mm : m2;
        amax = __uint_as_float(mm << 16);
    }
    const float sc = (amax > 0.0f) ? __fdiv_rn(amax, 448.0f) : 1.0f;
    if (threadIdx.x == 0) scale[r] = sc;
    // x / sc for the whole row with the reciprocal taken once: the hardware's approximation refined by
    // one Newton step, then per element the product, its exact remainder and one correction.  That is
    // the correctly rounded quotient unless the true one lies within ~2^-20 of a unit in the last
    // place of a rounding boundary; quotients are at most 448 in magnitude here, so the scaling an IEEE
    // division needs for its exceptional ranges (8 divisions of a dozen instructions each per 16 bytes
    // made this kernel bound by arithmetic, not by memory) has nothing to do.
    float rcp = __frcp_rn(sc);
    rcp = __fmaf_rn(__fmaf_rn(-sc, rcp, 1.0f), rcp, rcp);
    auto quot = [&](float xv) {
        const float q0 = __fmul_rn(xv, rcp);
        return __fmaf_rn(__fmaf_rn(-q0, sc, xv), rcp, q0);
    };
    auto conv = [&](const uint4& v) -> uint2 {
        const unsigned int wds[4] = {v.x, v.y, v.z, v.w};
        float f[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = quot(__uint_as_float(wds[j] << 16));
            f[2 * j + 1] = quot(__uint_as_float(wds[j] & 0xffff0000u));
        }
        uint2 o;
        o.x = e4m3x4(f[0], f[1], f[2], f[3]);
        o.y = e4m3x4(f[4], f[5], f[6], f[7]);
        return o;
    };
#pragma unroll
    for (int u = 0; u < kQuantKeep; ++u) {
        const int c = threadIdx.x + u * 256;
        if (c < nchunk) qr[c] = conv(keep[u]);
    }
    for (int c = threadIdx.x + kQuantKeep * 256; c < nchunk; c += 256) qr[c] = conv(x[c]);
}

// Block-scaled e4m3 quantisation of bf16 rows: a lane per 8 values, four lanes per 32-element block, sixteen per
// stage dword (see ghip_quant_rows_mx)
__global__ void __launch_bounds__(256)
quant_rows_mx_kernel(const uint16_t* __restrict__ src, long long chunks, int chunks_per_row, uint8_t* __restrict__ q,
                     unsigned int* __restrict__ scale, int ld_scale)
{
    const long long c = (long long)blockIdx.x * 256 + threadIdx.x;   // chunks_per_row is a multiple of 16: a wavefront never straddles rows' dwords
    if (c >= chunks) return;
    const uint4 v = reinterpret_cast<const uint4*>(src)[c];
    unsigned int m = ghip_bf16x8_amax15(v.x, v.y, v.z, v.w);
    unsigned int o = (unsigned int)__shfl_xor((int)m, 1, 64); m = m > o ? m : o;
    o = (unsigned int)__shfl_xor((int)m, 2, 64); m = m > o ? m : o;
    const int eb = ghip_mx_scale_byte(m);
    reinterpret_cast<uint2*>(q)[c] = ghip_mx_quant8(v.x, v.y, v.z, v.w, eb);
    unsigned int sd = (unsigned int)eb | ((unsigned int)__shfl_down(eb, 4, 64) << 8);
    sd |= (unsigned int)__shfl_down((int)sd, 8, 64) << 16;
    const long long row = c / chunks_per_row;
    const int cc = (int)(c % chunks_per_row);
    if ((threadIdx.x & 15) == 0) scale[(long long)(cc >> 4) * ld_scale + row] = sd;
}

inline int grid_for(long long n, int cap = 65535 * 4)
{
    long long b = (n + 255) / 256;
    if (b > cap) b = cap;
    if (b < 1) b = 1;
    return (int)b;
}

}  // namespace

__global__ void __launch_bounds__(256) mask_rows_kernel(const float* X, const uint8_t* __restrict__ drop, int ld_drop,
                                                        long long total, int cols, float* out)
{
    for (long long k = (long long)blockIdx.x * 256 + threadIdx.x; k < total; k += (long long)gridDim.x * 256) {
        const long long r = k / cols;
        const int c = (int)(k - r * cols);
        out[k] = drop[r * ld_drop + c] ? 0.0f : X[k];
    }
}

hipError_t ghip_mask_rows(const float* X, const uint8_t* drop, int ld_drop, int rows, int cols, float* out, hipStream_t s)
{
    const long long total = (long long)rows * cols;
    if (total <= 0) return hipSuccess;
    long long blocks = (total + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(mask_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, s, X, drop, ld_drop, total, cols, out);
    return hipGetLastError();
}

hipError_t ghip_output_delta(const DeltaArgs& a, hipStream_t s)
{
    const bool vec_ok = (a.n % 4) == 0 && a.n <= 2048 && (a.ldp % 4) == 0 && (!a.Y || (a.ldy % 4) == 0) &&
                        ((uintptr_t)a.P % 16) == 0 && ((uintptr_t)a.Y % 16) == 0 && ((uintptr_t)a.D % 16) == 0 && ((uintptr_t)a.Dbf % 8) == 0;
    if (vec_ok) {
        const int groups = (a.B + 3) / 4;
        const dim3 grid4(groups < 1024 ? groups : 1024);
        if (a.n <= 256) hipLaunchKernelGGL(output_delta_vec4_kernel<1>, grid4, dim3(256), 0, s, a);
        else if (a.n <= 512) hipLaunchKernelGGL(output_delta_vec4_kernel<2>, grid4, dim3(256), 0, s, a);
        else if (a.n <= 1024) hipLaunchKernelGGL(output_delta_vec4_kernel<4>, grid4, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(output_delta_vec4_kernel<8>, grid4, dim3(256), 0, s, a);
        return hipGetLastError();
    }
    const int rows_per_block = 4 * kRowsPerWave;
    const dim3 grid((a.B + rows_per_block - 1) / rows_per_block);
    if (a.n <= 64) hipLaunchKernelGGL(output_delta_kernel<1>, grid, dim3(256), 0, s, a);
    else if (a.n <= 256) hipLaunchKernelGGL(output_delta_kernel<4>, grid, dim3(256), 0, s, a);
    else if (a.n <= 1024) hipLaunchKernelGGL(output_delta_kernel<16>, grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL(output_delta_kernel<0>, grid, dim3(256), 0, s, a);
    return hipGetLastError();
}



hipError_t ghip_bias_update_step(BiasStepArgs& a, hipStream_t s)
{
    int blocks = 0;
    for (int k = 0; k < a.count; ++k) {
        a.e[k].first_block = blocks;
        blocks += a.e[k].part ? (a.e[k].n + 255) / 256 : (a.e[k].n + 3) / 4;
    }
    a.blocks = blocks;
    if (blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(bias_update_step_kernel, dim3(blocks), dim3(256), 0, s, a);
    return hipGetLastError();
}

hipError_t ghip_fill_f32(float* p, long long n, float v, hipStream_t s)
{
    hipLaunchKernelGGL(fill_kernel<float>, dim3(grid_for(n, 2048)), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}
hipError_t ghip_fill_f64(double* p, long long n, double v, hipStream_t s)
{
    hipLaunchKernelGGL(fill_kernel<double>, dim3(grid_for(n, 2048)), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}
hipError_t ghip_fill_u32(unsigned int* p, long long n, unsigned int v, hipStream_t s)
{
    hipLaunchKernelGGL(fill_kernel<unsigned int>, dim3(grid_for(n, 2048)), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}

hipError_t ghip_f32_to_bf16_2d(const float* src, uint16_t* dst, uint16_t* dstT, int rows, int cols, hipStream_t s)
{
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    hipLaunchKernelGGL(convert_transpose_kernel<float>, grid, dim3(256), 0, s, src, rows, cols, dst, dstT, rows, cols);
    return hipGetLastError();
}

hipError_t ghip_f32_to_bf16_2d_pad(const float* src, int src_rows, int src_cols, uint16_t* dst, uint16_t* dstT, int rows, int cols, hipStream_t s)
{
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    hipLaunchKernelGGL(convert_transpose_kernel<float>, grid, dim3(256), 0, s, src, src_rows, src_cols, dst, dstT, rows, cols);
    return hipGetLastError();
}

hipError_t ghip_bf16_transpose(const uint16_t* src, uint16_t* dstT, int rows, int cols, hipStream_t s)
{
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    if ((rows % 64) == 0 && (cols % 64) == 0 && ((uintptr_t)src % 16) == 0 && ((uintptr_t)dstT % 16) == 0) {
        hipLaunchKernelGGL(bf16_transpose64_kernel, grid, dim3(256), 0, s, src, dstT, rows, cols);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(convert_transpose_kernel<uint16_t>, grid, dim3(256), 0, s, src, rows, cols, (uint16_t*)nullptr, dstT, rows, cols);
    return hipGetLastError();
}

hipError_t ghip_quant_rows_mx(const uint16_t* src, int rows, int cols, uint8_t* q, unsigned int* scale, int ld_scale, hipStream_t s)
{
    if (rows <= 0 || cols <= 0 || (cols % 128) || ld_scale < rows || ((uintptr_t)src % 16) || ((uintptr_t)q % 8)) return hipErrorInvalidValue;
    const long long chunks = (long long)rows * (cols / 8);
    hipLaunchKernelGGL(quant_rows_mx_kernel, dim3((unsigned int)((chunks + 255) / 256)), dim3(256), 0, s, src, chunks, cols / 8, q, scale, ld_scale);
    return hipGetLastError();
}

hipError_t ghip_quant_rows_e4m3(const void* src, int src_is_bf16, int rows, int cols, uint8_t* q,
                                float* scale, unsigned int* amax_bits, int consume_amax, hipStream_t s)
{
    if (src_is_bf16 && (cols % 8) == 0 && ((uintptr_t)src % 16) == 0 && ((uintptr_t)q % 8) == 0)
        hipLaunchKernelGGL(quant_rows_bf16x8_kernel, dim3(rows), dim3(256), 0, s, (const uint16_t*)src, cols, q, scale, amax_bits, consume_amax);
    else if (src_is_bf16)
        hipLaunchKernelGGL(quant_rows_kernel<uint16_t>, dim3(rows), dim3(256), 0, s, (const uint16_t*)src, rows, cols, q, scale, amax_bits, consume_amax);
    else
        hipLaunchKernelGGL(quant_rows_kernel<float>, dim3(rows), dim3(256), 0, s, (const float*)src, rows, cols, q, scale, amax_bits, consume_amax);
    return hipGetLastError();
}
