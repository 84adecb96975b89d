// Low-precision GEMM for the wide canonical layers: C[M][N] = A[M][K] * B[N][K]^T with both
// operands K-contiguous, bf16 (v_mfma_f32_32x32x16_bf16) or e4m3 (v_mfma_scale_f32_32x32x64_f8f6f4
// with unit block scales), fp32 accumulation, fused epilogues.
//
// The three products of a training step are all brought to this one operand form by keeping
// transposed copies that the producing epilogues write for free (the GEMMs are compute bound
// by a factor of ~5 in HBM terms):
//   forward   H_{l+1} = squash(H_l W^T + b)   A = H_l [B][n_in],      B = W [n_out][n_in]
//   back-prop D_l = (D_{l+1} W) .* f'(H_l)    A = D_{l+1} [B][n_out], B = W^T [n_in][n_out]
//   gradient  G = D_{l+1}^T H_l               A = D^T [n_out][B],     B = H_l^T [n_in][B]
//             fused with the SGD + momentum + L1/L2 update of the fp32 master weights, which
//             also writes the bf16 W and W^T used by the next step.
//
// Tile: a workgroup of 8 wavefronts laid out 2 (M) x 4 (N); each wavefront owns MI x NI
// accumulators of 32x32.  MI = 4, NI = 2 gives the 256 x 256 tile (128 x 64 per wavefront, 128
// accumulator VGPRs) used whenever it fills the 256 CUs; MI = 2, NI = 1 gives a 128 x 128 tile for
// the products that would otherwise leave most CUs idle (the 1024-wide output layer), MI = 4, NI = 1
// a 256 x 128 tile for that layer's fp32-output forward product.
// K advances in stages of 128 bytes per row (64 bf16 / 128 e4m3: whole cache lines).  The 160 KB of
// LDS are a ring of five 32 KB operand half-stages (one operand of one stage each) filled by
// LDS-direct global loads (global_load_lds_dwordx4 from inline assembly: no VGPR staging, no
// ds_write, and no waits but the explicit s_waitcnt vmcnt(N) in front of the barriers).  The
// half-stages go round the ring as X0 Y0 X1 Y1 ...: X (A, as a rule) is requested two stages ahead
// of its use, its loads spread one by one between the MFMAs of the stage in between; Y (B) one stage
// ahead, its loads back to back right behind the barrier that frees their slot.  The wait that
// closes a stage leaves X's loads in flight.  (A ring of 64-byte-row stages with more of them in
// flight was measured too: same loop time, because every 128-byte line then travels from L2 twice.)
// Operands whose K runs over the batch (the weight gradient's, back-propagation's W^T) are read from
// K-blocked copies, [K / 64][rows][64], where a tile's stage is one contiguous block.
// 16-byte chunks are XOR-swizzled with the row index so that the per-lane 16-byte operand reads
// spread over all 64 banks.  Workgroup ids are remapped so that each XCD (ids congruent mod 8 share
// an L2) walks a compact block of tiles.

#include "ghip_internal.h"

#include <string.h>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int NT = 512;
constexpr int SKB = 128;  // bytes of K per stage row (64 bf16 / 128 e4m3): one full cache line

// LDS has 64 banks of 4 bytes: a 16-byte-per-lane read is served 16 lanes per clock.  A stage
// row is 128 B = 32 banks, so row parity picks the bank half and (row >> 1) & 7 rotates the
// chunk: 16 consecutive rows reading one logical chunk touch 16 distinct (half, chunk) slots.
__device__ __forceinline__ int swz(int row, int chunk) { return (row << 7) + (((chunk ^ (row >> 1)) & 7) << 4); }

// Activation and its derivative in a branch-free parametric form (filled on the host by
// resolve_act): the epilogues apply them to up to 128 accumulators per lane, and a switch over the
// activation id replicated that often does not fit the instruction cache.
template <bool PLAIN>
__device__ __forceinline__ float lp_squash(float z, const GemmLpArgs::ActForm& a)
{
    float v = (z < a.thr) ? a.a0 * z + a.b0 : a.a1 * z + a.b1;
    if (PLAIN) return v;
    if (a.trans) v = a.ta * __frcp_rn(1.0f + __expf(-a.tk * z)) + a.tb;
    v = (z < a.clo) ? a.vlo : v;
    v = (z > a.chi) ? a.vhi : v;
    return v;
}
__device__ __forceinline__ float lp_act_der(float y, const GemmLpArgs::ActForm& a)
{
    const float poly = a.c0 + a.c1 * y + a.c2 * y * y;
    const float stp = (y > 0.0f) ? a.dhi : a.dlo;
    return a.step ? stp : poly;
}

// Operand fragments of one K sub-step for this wavefront: MI row blocks of A, NI of B.
// bf16: 16 bytes per lane per block (K = 16); e4m3: 32 bytes per lane per block (K = 64).
template <bool FP8, int MI, int NI> struct Frags { v4i a[MI][FP8 ? 2 : 1], b[NI][FP8 ? 2 : 1]; };

// e4m3: the 64 bytes of K of one MFMA are four 16-byte chunks, and the instruction takes chunks lh and 2 + lh
// from the lane pair (row, lh = 0 / 1): its first 32-element scale block is the FIRST 16 bytes of both lanes,
// its second block the second 16 bytes (established with a probe that doubles one lane's scale byte), and the
// block scale of lane (row, lh) applies to block lh.  Reading the chunks in that order makes the blocks runs
// of 32 consecutive K, as the producers of the scales define them.
template <bool FP8, int MI, int NI>
__device__ __forceinline__ void load_frags(Frags<FP8, MI, NI>& f, const unsigned char* sa, const unsigned char* sb,
                                           int ks, int wm, int wn, int l31, int lh)
{
    constexpr int H = FP8 ? 2 : 1;
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int h = 0; h < H; ++h)
            f.a[mi][h] = *reinterpret_cast<const v4i*>(sa + swz(wm + mi * 32 + l31, FP8 ? ks * 4 + h * 2 + lh : ks * 2 + lh));
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int h = 0; h < H; ++h)
            f.b[ni][h] = *reinterpret_cast<const v4i*>(sb + swz(wn + ni * 32 + l31, FP8 ? ks * 4 + h * 2 + lh : ks * 2 + lh));
}

// the same in two parts: row block mi of A, and all of B
template <bool FP8, int MI, int NI>
__device__ __forceinline__ void load_frag_a(Frags<FP8, MI, NI>& f, const unsigned char* sa, int ks, int mi, int wm, int l31, int lh)
{
    constexpr int H = FP8 ? 2 : 1;
#pragma unroll
    for (int h = 0; h < H; ++h)
        f.a[mi][h] = *reinterpret_cast<const v4i*>(sa + swz(wm + mi * 32 + l31, FP8 ? ks * 4 + h * 2 + lh : ks * 2 + lh));
}
template <bool FP8, int MI, int NI>
__device__ __forceinline__ void load_frags_b(Frags<FP8, MI, NI>& f, const unsigned char* sb, int ks, int wn, int l31, int lh)
{
    constexpr int H = FP8 ? 2 : 1;
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int h = 0; h < H; ++h)
            f.b[ni][h] = *reinterpret_cast<const v4i*>(sb + swz(wn + ni * 32 + l31, FP8 ? ks * 4 + h * 2 + lh : ks * 2 + lh));
}

typedef __attribute__((address_space(3))) unsigned char* lptr_t;

// LDS-direct load of one 1 KiB slab: lane i's 16 bytes land at lds_slab + 16*i.
// Issued from inline assembly on purpose: the compiler then keeps no book on it, and the only
// waits on these loads are the explicit s_waitcnt vmcnt(N) before the barriers (with the builtin
// it drains all of them, vmcnt(0), in front of LDS reads it cannot tell apart from the stage
// being filled).  M0 carries the LDS byte address of the slab; loads return in order.
__device__ __forceinline__ void lds_direct_16(const unsigned char* src, unsigned int lds_slab)
{
    const unsigned int dst_u = __builtin_amdgcn_readfirstlane(lds_slab);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst_u) : "memory", "m0");
}
// The same with a wavefront-uniform base address and a 32-bit per-lane byte offset: the main loop
// advances the base with scalar arithmetic and keeps one offset register per operand and slab parity.
__device__ __forceinline__ void lds_direct_16s(const unsigned char* sbase, unsigned int voff, unsigned int lds_slab)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(sbase), "s"(lds_slab) : "memory", "m0");
}

// One dword per lane from a wavefront-uniform base plus a per-lane byte offset plus OFF, into a register the
// compiler takes for written at once: like the operand loads it is waited for by the explicit counts alone.
template <int OFF>
__device__ __forceinline__ void load_dword_s(unsigned int& dst, const void* sbase, unsigned int voff)
{
    asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(sbase), "n"(OFF) : "memory");
}

// 16 bytes per lane the same way: an operand half-stage on its way to LDS through registers (see the main loop)
__device__ __forceinline__ void load_x4_s(v4i& dst, const void* sbase, unsigned int voff)
{
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}

constexpr int cmax(int a, int b) { return a > b ? a : b; }
template <int V> struct IC { static constexpr int value = V; };

// MFMAs of one K sub-step with NDMA LDS-direct loads of the running fill spread between them:
// BEFORE MFMAs of the fill's span have been issued before this group; load number i goes out once
// (i + 1) * STEP MFMAs of the span have, STEP = SPAN / (NDMA + 1).  A wavefront that issues all its
// loads back to back stalls on the address unit (16 clocks per load, shared by the 8 wavefronts),
// and the matrix pipe of its SIMD idles with it.
// OPSEL: the byte of sa[mi] that holds this sub-step's E8M0 scale of the lane's block of A (e4m3 only; 0x7f = 1)
// row(mi) runs once the MFMAs that read row block mi of A have been issued (the rolling fragment loads: the block's
// registers are free for the next sub-step's block from there on).
template <bool FP8, int MI, int NI, int SPAN, int NDMA, int BEFORE, int OPSEL = 0, typename Dma, typename Row>
__device__ __forceinline__ void mma_group(v16f (&acc)[MI][NI], const Frags<FP8, MI, NI>& f, Dma&& dma, const unsigned int (&sa)[MI], Row&& row)
{
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            if constexpr (!FP8) {
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, f.a[mi][0]),
                                                                      __builtin_bit_cast(bf16x8, f.b[ni][0]), acc[mi][ni], 0, 0, 0);
            } else {
                const v8i av = v8i{f.a[mi][0][0], f.a[mi][0][1], f.a[mi][0][2], f.a[mi][0][3],
                                   f.a[mi][1][0], f.a[mi][1][1], f.a[mi][1][2], f.a[mi][1][3]};
                const v8i bv = v8i{f.b[ni][0][0], f.b[ni][0][1], f.b[ni][0][2], f.b[ni][0][3],
                                   f.b[ni][1][0], f.b[ni][1][1], f.b[ni][1][2], f.b[ni][1][3]};
                acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc[mi][ni], 0, 0, OPSEL, (int)sa[mi], 0, 0x7f7f7f7f);
            }
            if constexpr (NDMA > 0) {
                const int m = BEFORE + mi * NI + ni;
                constexpr int STEP = SPAN / (NDMA + 1) > 0 ? SPAN / (NDMA + 1) : 1;
                static_assert(SPAN >= NDMA, "the span has room for every load");
                auto before = [](int mm) { return mm / STEP < NDMA ? mm / STEP : NDMA; };  // loads out before MFMA mm
                const int lo = before(m);
                const int hi = (m + 1 >= SPAN) ? NDMA : before(m + 1);
                if (m < SPAN && hi > lo) {
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int d = lo; d < hi; ++d) dma(d);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (ni == NI - 1) row(mi);
        }
}

// LDS of one workgroup: a ring of five operand half-stages during the K loop, then the staging area of the epilogue.
template <int MI, int NI>
constexpr int lp_lds_bytes()
{
    constexpr int TM = 64 * MI, TN = 128 * NI;
    return cmax(5 * cmax(TM, TN) * SKB, cmax(TM * (2 * TN + 16), TN * (2 * TM + 16)));
}

// One tile of one product, by the whole workgroup.  `id` numbers the product's tiles so that consecutive
// numbers are neighbours in the output (the caller hands each XCD a contiguous range of them); smem is the
// workgroup's LDS block of lp_lds_bytes<MI, NI>() bytes, 1 KiB aligned.
template <bool FP8, int EPI, int MI, int NI>
__device__ __forceinline__ void gemm_lp_tile(const GemmLpArgs& g, int id, unsigned char* smem)
{
    constexpr int TM = 64 * MI, TN = 128 * NI;       // tile
    constexpr int WM = 32 * MI, WN = 32 * NI;        // per wavefront
    constexpr int A_BYTES = TM * SKB, B_BYTES = TN * SKB;
    constexpr int SLOT = cmax(A_BYTES, B_BYTES);     // one operand stage
    constexpr int NSLOT = 5;
    constexpr int PITCH = 2 * TN + 16;               // staged bf16 output row [TM][TN]: +16 rotates banks, keeps alignment
    constexpr int PITCH_T = 2 * TM + 16;             // staged transposed row [TN][TM]
    static_assert(lp_lds_bytes<MI, NI>() == cmax(NSLOT * SLOT, cmax(TM * PITCH, TN * PITCH_T)), "the ring and the staging area fit");

    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int l31 = lane & 31, lh = lane >> 5;
    constexpr bool kDgrad = (EPI == LP_DGRAD || EPI == LP_DGRAD_MASK);   // back-propagation: derivative from the activations / from their signs
    constexpr bool kMask = (EPI == LP_DGRAD_MASK);

    // ---- walk the tiles in column groups of 8 rows
    const int tiles_m = g.M / TM, tiles_n = g.N / TN;
    constexpr int GROUP = 8;
    const int per_group = GROUP * tiles_n;
    const int gidx = id / per_group;
    const int first_m = gidx * GROUP;
    const int gsize = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    const int tm = first_m + (id % per_group) % gsize;
    const int tn = (id % per_group) / gsize;
    const int bm = tm * TM, bn = tn * TN;

    constexpr int ES = FP8 ? 1 : 2;                                   // bytes per operand element
    const long long ldk = (long long)g.K * ES;                        // bytes of K per row
    const long long lda = (long long)(g.lda ? g.lda : g.K) * ES;      // row pitches in bytes
    const long long ldb = (long long)(g.ldb ? g.ldb : g.K) * ES;
    const long long ksA = g.kstrideA ? g.kstrideA : SKB, ksB = g.kstrideB ? g.kstrideB : SKB;  // bytes from stage to stage
    const unsigned char* gA = (const unsigned char*)g.A + (long long)bm * lda;
    const unsigned char* gB = (const unsigned char*)g.B + (long long)bn * ldb;

    const int wm = (w >> 2) * WM, wn = (w & 3) * WN;

    v16f acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mi][ni][i] = 0.0f;

    const int nk = (int)(ldk / SKB);  // stages along K

    // ---- operand stages.  Stage j of A is TM rows x 128 B, of B TN rows x 128 B; both are
    // sequences of 1 KiB slabs of 8 rows, one LDS-direct load each: lane i lands at row i/8,
    // physical chunk i%8 of its slab, so it fetches the logical chunk that the swizzle maps there
    // (every load covers whole 128-byte lines).  A wavefront moves PWA + PWB slabs per stage.
    // The ring holds the half-stages A0 B0 A1 B1 ... in slots 0 1 2 3 4 0 1 ...: B(j+1) is requested
    // as soon as the barrier that ends stage j-1 has freed its slot, A(j+2) while stage j is consumed,
    // so A has two stages of lead and B one, and the wait that ends stage j leaves the A loads in flight.
    constexpr int PWA = TM / 64, PWB = TN / 64;
    const int ws = __builtin_amdgcn_readfirstlane(w);
    static_assert(PWA % 2 == 0 && PWB % 2 == 0 && PWA < 8, "slab parity and the vmcnt immediate assume this");
    // e4m3 with block-scaled activations: the E8M0 scales of A, one byte per row and 32 elements of K, lie
    // stage-major, [K / 128][ld_scale] dwords (a dword = the four blocks of one row in one stage).  Each lane
    // fetches the dwords of its MI rows straight into registers, two stages ahead together with the first X
    // load; five register sets, one per ring position, so that no value ever moves between registers while
    // its load may still be in flight.
    constexpr bool kMX = FP8 && (EPI == LP_FP8_ACT_MX || EPI == LP_FP8_F32_MX);
    unsigned int sc[NSLOT][MI];
    const unsigned int* const scw = kMX ? g.a_scale + bm + (ws >> 2) * WM : nullptr;
    const unsigned int scv = (unsigned int)l31 * 4u;
    auto load_scales = [&](auto setc, int st) {
        constexpr int S = decltype(setc)::value;
        const unsigned int* const base = scw + (long long)(st < nk ? st : nk - 1) * g.ld_scale;
        load_dword_s<0>(sc[S][0], base, scv);
        if constexpr (MI > 1) load_dword_s<128>(sc[S][1], base, scv);
        if constexpr (MI > 2) load_dword_s<256>(sc[S][2], base, scv);
        if constexpr (MI > 3) load_dword_s<384>(sc[S][3], base, scv);
        static_assert(MI <= 4, "one load per 32-row block");
    };
    if constexpr (kMX) { load_scales(IC<0>{}, 0); load_scales(IC<1>{}, 1); }
    else {
#pragma unroll
        for (int i = 0; i < NSLOT; ++i)
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) sc[i][mi] = 0x7f7f7f7fu;
    }
    const unsigned int smem_u = (unsigned int)(uintptr_t)((lptr_t)smem);
    unsigned int voffA[2], voffB[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {  // slab parity decides bit 2 of (row >> 1)
        const unsigned int chunk = ((lane & 7) ^ (p * 4 + (lane >> 4))) & 7;
        voffA[p] = (unsigned int)(lane >> 3) * (unsigned int)lda + (chunk << 4);
        voffB[p] = (unsigned int)(lane >> 3) * (unsigned int)ldb + (chunk << 4);
    }
    const unsigned char* const gAw = gA + (long long)(ws * PWA * 8) * lda;
    const unsigned char* const gBw = gB + (long long)(ws * PWB * 8) * ldb;
    auto dmaA = [&](int slot, int st, int jj) {
        const long long kb = (long long)(st < nk ? st : nk - 1) * ksA;  // past the end: refetch, never read
        lds_direct_16s(gAw + (long long)(jj * 8) * lda + kb, voffA[jj & 1], smem_u + slot * SLOT + (ws * PWA + jj) * 1024);
    };
    auto dmaB = [&](int slot, int st, int jj) {
        const long long kb = (long long)(st < nk ? st : nk - 1) * ksB;
        lds_direct_16s(gBw + (long long)(jj * 8) * ldb + kb, voffB[jj & 1], smem_u + slot * SLOT + (ws * PWB + jj) * 1024);
    };
    // X is the operand with two stages of lead, Y the one with one: A and B, except in the 128 x 128-tile
    // weight gradient, which runs 10 % faster with its B operand (the activations, a forward pass old)
    // in the place with more lead; the 256 x 256-tile kernels measure the same either way
    constexpr bool kSwap = !FP8 && EPI == LP_WGRAD_SGD && TM == 128;
    static_assert(!kSwap || PWA == PWB, "operands that change places in the ring have equally many slabs");
    auto dmaX = [&](int slot, int st, int jj) { if constexpr (kSwap) dmaB(slot, st, jj); else dmaA(slot, st, jj); };
    auto dmaY = [&](int slot, int st, int jj) { if constexpr (kSwap) dmaA(slot, st, jj); else dmaB(slot, st, jj); };
    constexpr int OA = kSwap ? 1 : 0, OB = kSwap ? 0 : 1;  // places of A and B within a stage's pair of slots
    // The bf16 128-row tiles (two workgroups to a CU, the global->LDS path their bound) take Y's half-stages through
    // registers.  Straight into LDS, a half-stage can only be asked for once its slot is free, one stage ahead of its
    // use.  A register set per stage parity holds Y(j+2) from the start of stage j until the middle of stage j+1, when
    // it is written to the slot that stage j's barrier freed: a stage and a half in flight for 2 x PWB x 4 registers
    // (the narrow layer's weight gradient runs 16 % faster).  The 256 x 256 tiles lose 3 to 7 % that way, with the loads
    // in one go behind the barrier or spread between the MFMAs alike, and keep the direct path: each operand's loads
    // alone cost their loop 3 %, both together 35 % -- its bound is what the path delivers, not how early it is asked.
    constexpr int RY = (!FP8 && MI * NI < 8) ? PWB : 0;   // slabs of Y per wavefront that go through registers
    constexpr bool kRegY = RY > 0;
    v4i yreg[2][RY > 0 ? RY : 1];
    auto ldY = [&](auto setc, int st, int jj) {
        constexpr int S = decltype(setc)::value;
        if constexpr (kSwap) {
            const long long kb = (long long)(st < nk ? st : nk - 1) * ksA;
            load_x4_s(yreg[S][jj], gAw + (long long)(jj * 8) * lda + kb, voffA[jj & 1]);
        } else {
            const long long kb = (long long)(st < nk ? st : nk - 1) * ksB;
            load_x4_s(yreg[S][jj], gBw + (long long)(jj * 8) * ldb + kb, voffB[jj & 1]);
        }
    };
    auto wrY = [&](auto setc, int slot) {   // lane i's 16 bytes to where the direct load puts them: slab + 16 i
        constexpr int S = decltype(setc)::value;
#pragma unroll
        for (int jj = 0; jj < RY; ++jj)
            *reinterpret_cast<v4i*>(smem + slot * SLOT + (ws * PWB + jj) * 1024 + lane * 16) = yreg[S][jj];
    };
#pragma unroll
    for (int jj = 0; jj < PWA; ++jj) dmaX(0, 0, jj);
#pragma unroll
    for (int jj = 0; jj < PWB; ++jj) dmaY(1, 0, jj);
#pragma unroll
    for (int jj = 0; jj < RY; ++jj) ldY(IC<1>{}, 1, jj);
#pragma unroll
    for (int jj = 0; jj < PWA; ++jj) dmaX(2, 1, jj);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (PWA + RY));  // A0 and B0 have landed
    __builtin_amdgcn_s_barrier();

    typedef Frags<FP8, MI, NI> F;
    F f0, f1;
    load_frags<FP8, MI, NI>(f0, smem + OA * SLOT, smem + OB * SLOT, 0, wm, wn, l31, lh);

    // One stage (P = j mod 5 fixes the slots at compile time).  Sub-steps are software pipelined:
    // each one requests the next sub-step's B fragments, then issues its MFMAs with the fill's loads
    // between them and, behind the MFMAs that read a row block of A, the request for the next
    // sub-step's block (the compiler places the waits for these LDS reads).  The last sub-step waits
    // for B(j+1), meets the other wavefronts (bare s_barrier: the explicit counts are exactly what has
    // to be visible) and requests the first fragments of stage j+1.  The 256 x 256 e4m3 tile runs its
    // two sub-steps in sequence on one fragment set.
    constexpr int KS = FP8 ? 2 : 4;
    constexpr int G = MI * NI;
    constexpr bool kDouble = !(FP8 && G > 2);
    constexpr int MASK_WORDS = MI * NI * 16 / 32;   // a lane's accumulators, one bit each
    // loads a stage's closing wait leaves in flight: X(j+2), and Y(j+2) on its way to registers / the scale dwords
    constexpr int VM_STAGE = PWA + (kMX ? MI : 0) + RY;
    // ... and the wait in the middle of a stage for the registers of Y(j+1): X(j+1), Y(j+2) and X(j+2) were asked for later
    constexpr int VM_MID = 2 * PWA + PWB;
    static_assert(VM_STAGE <= 15 && VM_MID <= 15, "the counts fit the low four bits of the wait's immediate");
    // Y's loads go out as early as their slot allows, back to back right behind the barrier that closes
    // the stage before (spread over the stage with X's, they cost the bf16 training step 5 % and the e4m3
    // products 7 %), and only X's, which have a stage more, are spread between the MFMAs.  What the loop
    // waits for is the path from L2 to LDS as a whole: without any loads the 256 x 256 bf16 loop keeps the
    // matrix pipes busy (1.07 us per stage), with either operand's loads alone it takes 3 % longer, with both
    // 45 % (1.56 us): 64 KB per stage and CU are 15 TB/s over the chip at the matrix pipes' rate, and the
    // path delivers 10 to 11 in this loop.
    auto stage = [&](auto Pc, auto Qc, int j) {
        constexpr int P = decltype(Pc)::value;
        constexpr int Q = decltype(Qc)::value;   // j mod 2: the register set that holds Y(j+2); the other one turns over in this stage
        // The slots' offsets reach the fragment reads as scalars the compiler cannot fold: folded, every (slot, sub-step,
        // operand) combination becomes an address register of its own, kept across the whole loop (24 of them)
        auto slot_at = [&](auto slot_c) {
            unsigned int off;
            asm volatile("s_mov_b32 %0, %1" : "=s"(off) : "i"(decltype(slot_c)::value * SLOT));
            return smem + off;
        };
        const unsigned char* const RA = slot_at(IC<(2 * P + OA) % NSLOT>{});
        const unsigned char* const RB = slot_at(IC<(2 * P + OB) % NSLOT>{});
        const unsigned char* const NA = slot_at(IC<(2 * P + 2 + OA) % NSLOT>{});
        const unsigned char* const NB = slot_at(IC<(2 * P + 2 + OB) % NSLOT>{});
        auto dma = [&](int d) {
            if constexpr (kMX) { if (d == 0) load_scales(IC<(P + 2) % NSLOT>{}, j + 2); }
            dmaX((2 * P + 4) % NSLOT, j + 2, d);
        };
        auto none = [](int) {};
        // this stage's scale dwords landed before the wait that closed the stage before; lane (row, lh) scales
        // blocks lh (first sub-step) and 2 + lh (second): bytes 0 and 2 once the dword is shifted by 8 lh bits
        unsigned int sa[MI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) sa[mi] = kMX ? sc[P][mi] >> (8 * lh) : 0x7f7f7f7fu;
        auto next_y = [&]() {  // the next stage's Y loads: their slot is free once this stage's closing barrier is passed
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int d = RY; d < PWB; ++d) dmaY((2 * P + 5) % NSLOT, j + 2, d);   // straight into LDS: one stage ahead
#pragma unroll
            for (int d = 0; d < RY; ++d) ldY(IC<(Q + 1) & 1>{}, j + 3, d);        // by way of registers: two
            __builtin_amdgcn_sched_barrier(0);
        };
        auto norow = [](int) {};
        if constexpr (!kDouble) {
            constexpr int SPAN = 2 * G;
            mma_group<FP8, MI, NI, SPAN, PWA, 0, 0>(acc, f0, dma, sa, norow);
            load_frags<FP8, MI, NI>(f0, RA, RB, 1, wm, wn, l31, lh);
            mma_group<FP8, MI, NI, SPAN, PWA, G, 2>(acc, f0, dma, sa, norow);
            __builtin_amdgcn_s_waitcnt(0x0070 | VM_STAGE);  // vmcnt(VM_STAGE) lgkmcnt(0)
            __builtin_amdgcn_s_barrier();
            next_y();
            load_frags<FP8, MI, NI>(f0, NA, NB, 0, wm, wn, l31, lh);
        } else {
            constexpr int SPAN = (KS - 1) * G;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                F& cur = (ks & 1) ? f1 : f0;
                F& nxt = (ks & 1) ? f0 : f1;
                // The next sub-step's fragments: B's at the head of this one, A's block by block behind the MFMAs that
                // read the block before it (one set of A fragments and a block in transit instead of two sets)
                const unsigned char* const FA = (ks + 1 < KS) ? RA : NA;
                const int fks = (ks + 1 < KS) ? ks + 1 : 0;
                auto row = [&](int mi) {
                    __builtin_amdgcn_sched_barrier(0);
                    load_frag_a<FP8, MI, NI>(nxt, FA, fks, mi, wm, l31, lh);
                    __builtin_amdgcn_sched_barrier(0);
                };
                if (ks + 1 < KS) {
                    load_frags_b<FP8, MI, NI>(nxt, RB, ks + 1, wn, l31, lh);
                    if constexpr (kRegY) {
                        if (ks == KS - 2) {   // all of X(j+2) has been asked for by now (see mma_group): the count below holds
                            static_assert((2 * G) / ((KS - 1) * G / (PWA + 1) > 0 ? (KS - 1) * G / (PWA + 1) : 1) >= PWA, "X's loads are out after two sub-steps");
                            __builtin_amdgcn_sched_barrier(0);
                            __builtin_amdgcn_s_waitcnt(0x0F70 | VM_MID);  // Y(j+1) is in its registers
                            __builtin_amdgcn_sched_barrier(0);
                            wrY(IC<(Q + 1) & 1>{}, (2 * P + 3) % NSLOT);   // Y's place in stage j+1's pair of slots
                        }
                    }
                } else {
                    __builtin_amdgcn_s_waitcnt(0x0070 | VM_STAGE);  // vmcnt(VM_STAGE) lgkmcnt(0)
                    __builtin_amdgcn_s_barrier();
                    next_y();
                    load_frags_b<FP8, MI, NI>(nxt, NB, 0, wn, l31, lh);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (ks == 0) mma_group<FP8, MI, NI, SPAN, PWA, 0, 0>(acc, cur, dma, sa, row);
                else if (ks == 1 && KS > 2) mma_group<FP8, MI, NI, SPAN, PWA, G>(acc, cur, dma, sa, row);
                else if (ks == 2 && KS > 3) mma_group<FP8, MI, NI, SPAN, PWA, 2 * G>(acc, cur, dma, sa, row);
                else mma_group<FP8, MI, NI, 1, 0, 0, FP8 ? 2 : 0>(acc, cur, none, sa, row);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    // what the first stage's waits are for (X1 went out with the ring's first fill)
#pragma unroll
    for (int d = RY; d < PWB; ++d) dmaY(3, 1, d);
#pragma unroll
    for (int d = 0; d < RY; ++d) ldY(IC<0>{}, 2, d);
    if constexpr (kRegY) {
        for (int j = 0;;) {
            stage(IC<0>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<1>{}, IC<1>{}, j); if (++j == nk) break;
            stage(IC<2>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<3>{}, IC<1>{}, j); if (++j == nk) break;
            stage(IC<4>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<0>{}, IC<1>{}, j); if (++j == nk) break;
            stage(IC<1>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<2>{}, IC<1>{}, j); if (++j == nk) break;
            stage(IC<3>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<4>{}, IC<1>{}, j); if (++j == nk) break;
        }
    } else {
        for (int j = 0;;) {
            stage(IC<0>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<1>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<2>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<3>{}, IC<0>{}, j); if (++j == nk) break;
            stage(IC<4>{}, IC<0>{}, j); if (++j == nk) break;
        }
    }
    // nothing may still be writing this workgroup's LDS when its wavefronts retire -- nor the registers of the loads
    // that were asked for past the last stage: those registers stay taken until the wait is over (the compiler,
    // which keeps no book on these loads, would hand them to the epilogue's first values otherwise)
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kRegY) {
#pragma unroll
        for (int jj = 0; jj < RY; ++jj) asm volatile("" : : "v"(yreg[0][jj]), "v"(yreg[1][jj]));
    }
    if constexpr (kMX) {
#pragma unroll
        for (int i = 0; i < NSLOT; ++i)
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) asm volatile("" : : "v"(sc[i][mi]));
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- epilogue.  Accumulator layout of a 32x32 tile: lane -> column lane%32,
    //      register i -> row 8*(i/4) + 4*(lane/32) + i%4  (4 consecutive rows per register quad).
    //      bf16 results leave through LDS so that global memory only sees 16-byte-per-lane stores
    //      of whole tile rows (direct stores from this layout are 2 bytes per lane, and 8 bytes per
    //      lane with a row-sized stride for the transposed copy).
    const int M = g.M, N = g.N;
    __builtin_amdgcn_s_barrier();  // every wavefront is done with the ring

    if constexpr (kMask) {
        // The activation below is a step in its derivative (ReLU, leaky ReLU): f' takes one of two values by the sign of
        // the activation, and the forward product that stored the activations left those signs, a bit per element in
        // the order of the accumulators of the workgroup that computed them -- which is this workgroup's order: same
        // rows, same units, same tile.  16 bytes per lane instead of a 128 KB tile through LDS.
        const unsigned int* mw = g.mask_in + ((long long)(tm * tiles_n + tn) * NT + t) * MASK_WORDS;
        unsigned int bits[MASK_WORDS];
#pragma unroll
        for (int k = 0; k < MASK_WORDS; ++k) bits[k] = mw[k];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int b = (mi * NI + ni) * 16 + i;
                    acc[mi][ni][i] *= ((bits[b >> 5] >> (b & 31)) & 1u) ? g.ap.dhi : g.ap.dlo;
                }
    }
    if constexpr (EPI == LP_DGRAD) {
        // activation tile [TM][TN] bf16 -> LDS (row pitch 2*TN bytes) with LDS-direct loads
        constexpr int LPR = TN / 8;         // lanes per tile row (16 bytes each)
        constexpr int RPS = 64 / LPR;       // rows per 1 KiB slab
        constexpr int PER_WAVE = TM / RPS / 8;
        const unsigned char* aux = (const unsigned char*)g.aux + ((long long)bm * N + bn) * 2;
#pragma unroll
        for (int j = 0; j < PER_WAVE; ++j) {
            const int slab = w * PER_WAVE + j;
            const int row = slab * RPS + lane / LPR;
            lds_direct_16(aux + (long long)row * N * 2 + ((lane % LPR) << 4), (unsigned int)(uintptr_t)((lptr_t)smem) + slab * 1024);
        }
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = wm + mi * 32 + 8 * (i >> 2) + 4 * lh + (i & 3);
                    const int col = wn + ni * 32 + l31;
                    const uint16_t hv = *reinterpret_cast<const uint16_t*>(smem + row * (2 * TN) + col * 2);
                    acc[mi][ni][i] *= lp_act_der(ghip_bf16_to_f32(hv), g.ap);
                }
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_s_barrier();
    }

    constexpr bool kActMX = (EPI == LP_FP8_ACT_MX);   // e4m3 codes + block scales out, through the same bf16 staging
    constexpr bool kBf16Out = (EPI == LP_FWD_ACT || kDgrad || EPI == LP_WGRAD_SGD || EPI == LP_FP8_ACT || kActMX);
    constexpr bool kFwd = (EPI == LP_FWD_ACT || EPI == LP_FWD_F32), kF8 = (EPI == LP_FP8_ACT || EPI == LP_FP8_F32 || kMX);
    uint2 pk[MI][NI][4];  // bf16 results, 4 consecutive rows packed per entry
    float cbias[NI], cscale[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int col = bn + wn + ni * 32 + l31;
        cbias[ni] = (kFwd && g.bias) ? g.bias[col] : 0.0f;
        cscale[ni] = kF8 ? g.col_scale[col] : 1.0f;
    }
    // Two copies of the element loop, chosen once per launch: piecewise-linear activations
    // (ReLU, leaky, linear, step) take four instructions per element, the general form a dozen.
    const bool pad_tile = g.n_valid > 0 && bn + TN > g.n_valid;   // only the tiles of the last columns can hold padding
    auto finish = [&](auto plain_c) {
        constexpr bool PLAIN = decltype(plain_c)::value;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            // weight gradient: the master weights and momentum of a whole 32-row block are asked for together,
            // ahead of the arithmetic and of any store (element by element, each load pair would wait out a round
            // trip to memory before the next one could leave: 128 round trips per lane were the update's time)
            float mw[4][NI][4], mv[4][NI][4];
            if constexpr (EPI == LP_WGRAD_SGD) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            mw[q][ni][r] = g.master[(long long)(bm + wm + mi * 32 + 8 * q + 4 * lh + r) * N + bn + wn + ni * 32 + l31];
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            mv[q][ni][r] = g.mom[(long long)(bm + wm + mi * 32 + 8 * q + 4 * lh + r) * N + bn + wn + ni * 32 + l31];
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int row0 = bm + wm + mi * 32 + 8 * q + 4 * lh;
                float rs[4] = {1.0f, 1.0f, 1.0f, 1.0f};
                if constexpr (kF8 && !kMX) {
                    const float4 r4 = *reinterpret_cast<const float4*>(g.row_scale + row0);
                    rs[0] = r4.x; rs[1] = r4.y; rs[2] = r4.z; rs[3] = r4.w;
                }
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const int col = bn + wn + ni * 32 + l31;
                    float o[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const long long idx = (long long)(row0 + r) * N + col;
                        const float v = acc[mi][ni][q * 4 + r];
                        if constexpr (kFwd) {
                            o[r] = lp_squash<PLAIN>(v + cbias[ni], g.ap);
                        } else if constexpr (kMX) {
                            o[r] = lp_squash<PLAIN>(__fmul_rn(v, cscale[ni]), g.ap);   // the rows' scales went in block by block
                        } else if constexpr (kF8) {
                            o[r] = lp_squash<PLAIN>(__fmul_rn(v, __fmul_rn(rs[r], cscale[ni])), g.ap);
                        } else if constexpr (EPI == LP_WGRAD_SGD) {
                            const float wv = mw[q][ni][r];
                            const float sg = (wv > 0.0f) ? 1.0f : ((wv < 0.0f) ? -1.0f : 0.0f);
                            const float gr = v * g.gscale + g.wd1 * sg + g.wd2 * wv;
                            const float d = g.lr * gr + g.momf * mv[q][ni][r];
                            g.mom[idx] = d;
                            o[r] = wv - d;
                            g.master[idx] = o[r];
                        } else {
                            o[r] = v;
                        }
                        if constexpr (EPI == LP_FWD_F32 || EPI == LP_FP8_F32 || EPI == LP_FP8_F32_MX) ((float*)g.out)[idx] = o[r];
                    }
                    if constexpr (EPI == LP_FWD_ACT || EPI == LP_FP8_ACT || kActMX) {
                        // units past the layer's width are padding: they stay zero whatever the activation makes of 0
                        if (pad_tile && col >= g.n_valid) { o[0] = 0.0f; o[1] = 0.0f; o[2] = 0.0f; o[3] = 0.0f; }
                    }
                    if constexpr (EPI == LP_FP8_ACT || kActMX) {
                        // single output: straight into the row-major staging area
                        const unsigned int p01 = ghip_f32x2_to_bf16x2(o[0], o[1]), p23 = ghip_f32x2_to_bf16x2(o[2], o[3]);
                        unsigned char* d0 = smem + (wm + mi * 32 + 8 * q + 4 * lh) * PITCH + (wn + ni * 32 + l31) * 2;
                        *reinterpret_cast<uint16_t*>(d0) = (uint16_t)(p01 & 0xffffu);
                        *reinterpret_cast<uint16_t*>(d0 + PITCH) = (uint16_t)(p01 >> 16);
                        *reinterpret_cast<uint16_t*>(d0 + 2 * PITCH) = (uint16_t)(p23 & 0xffffu);
                        *reinterpret_cast<uint16_t*>(d0 + 3 * PITCH) = (uint16_t)(p23 >> 16);
                    } else if constexpr (kBf16Out) {
                        pk[mi][ni][q].x = ghip_f32x2_to_bf16x2(o[0], o[1]);
                        pk[mi][ni][q].y = ghip_f32x2_to_bf16x2(o[2], o[3]);
                    }
                }
            }
        }
    };
    if ((kFwd || kF8) && !g.ap.plain) finish(IC<0>{});
    else finish(IC<1>{});
    if constexpr (EPI == LP_FWD_ACT) {
        if (g.mask_out) {   // the signs of the stored activations, for the back-propagation product of this tile (see there)
            unsigned int bits[MASK_WORDS];
#pragma unroll
            for (int k = 0; k < MASK_WORDS; ++k) bits[k] = 0u;
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint2 v = pk[mi][ni][q];
                        // a bf16 is positive where its 16 bits, read as a signed integer, are
                        const unsigned int four = ((short)(v.x & 0xffffu) > 0 ? 1u : 0u) | ((short)(v.x >> 16) > 0 ? 2u : 0u) |
                                                  ((short)(v.y & 0xffffu) > 0 ? 4u : 0u) | ((short)(v.y >> 16) > 0 ? 8u : 0u);
                        const int b = (mi * NI + ni) * 16 + q * 4;
                        bits[b >> 5] |= four << (b & 31);
                    }
            unsigned int* mw = g.mask_out + ((long long)(tm * tiles_n + tn) * NT + t) * MASK_WORDS;
#pragma unroll
            for (int k = 0; k < MASK_WORDS; ++k) mw[k] = bits[k];
        }
    }
    // back-propagation also leaves the column sums of the deltas it stores (the bias gradient of
    // the layer below), per tile row so that the caller adds them in a fixed order
    float csum[NI];
    if constexpr (kDgrad) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            float s = 0.0f;
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint2 v = pk[mi][ni][q];
                    s += (__uint_as_float(v.x << 16) + __uint_as_float(v.x & 0xffff0000u)) +
                         (__uint_as_float(v.y << 16) + __uint_as_float(v.y & 0xffff0000u));
                }
            csum[ni] = s + __shfl_xor(s, 32, 64);
        }
    }
    if constexpr (kBf16Out) {
        // transposed copy first: LDS_T[n][m], a lane's 4 consecutive rows are 8 contiguous bytes
        if ((EPI == LP_FWD_ACT || kDgrad || EPI == LP_WGRAD_SGD) && g.outT) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int rl = wm + mi * 32 + 8 * q + 4 * lh, cl = wn + ni * 32 + l31;
                        *reinterpret_cast<uint2*>(smem + cl * PITCH_T + rl * 2) = pk[mi][ni][q];
                    }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();
            constexpr int LPR = TM / 8, RPI = 64 / LPR;   // lanes per transposed row, rows per instruction
            // plain: outT[n][m]; K-blocked for the weight gradient (K = m): outT[m / 64][n][m % 64], where
            // the 128-byte pieces of a transposed row go to planes N x 128 bytes apart and the tile's rows
            // follow one another within a plane
            unsigned char* dstT = g.outT_blocked ? (unsigned char*)g.outT + ((long long)(bm >> 6) * N + bn) * 128
                                                 : (unsigned char*)g.outT + ((long long)bn * M + bm) * 2;
            const long long rowT = g.outT_blocked ? 128 : (long long)M * 2;
            const long long planeT = g.outT_blocked ? (long long)N * 128 : 128;
#pragma unroll
            for (int i = 0; i < (TN / 8) / RPI; ++i) {
                const int nl = w * (TN / 8) + i * RPI + lane / LPR;
                const int lc = (lane % LPR) << 4;
                const v4i val = *reinterpret_cast<const v4i*>(smem + nl * PITCH_T + lc);
                *reinterpret_cast<v4i*>(dstT + (long long)nl * rowT + (long long)(lc >> 7) * planeT + (lc & 127)) = val;
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();
        }
        // row-major copy: LDS[m][n] (back-propagation's last product has no reader for it: the deltas of the first
        // hidden layer are only read transposed, by the first layer's weight gradient)
        const bool row_major = !(kDgrad && !g.out);
        if (row_major) {
        if constexpr (EPI != LP_FP8_ACT && !kActMX)
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int rl = wm + mi * 32 + 8 * q + 4 * lh, cl = wn + ni * 32 + l31;
                    unsigned char* d0 = smem + rl * PITCH + cl * 2;
                    *reinterpret_cast<uint16_t*>(d0) = (uint16_t)(pk[mi][ni][q].x & 0xffffu);
                    *reinterpret_cast<uint16_t*>(d0 + PITCH) = (uint16_t)(pk[mi][ni][q].x >> 16);
                    *reinterpret_cast<uint16_t*>(d0 + 2 * PITCH) = (uint16_t)(pk[mi][ni][q].y & 0xffffu);
                    *reinterpret_cast<uint16_t*>(d0 + 3 * PITCH) = (uint16_t)(pk[mi][ni][q].y >> 16);
                }
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_s_barrier();
        constexpr int LPR = TN / 8, RPI = 64 / LPR, NIT = (TM / 8) / RPI;
        if constexpr (kActMX) {
            // The next layer's A operand, made here: every run of 32 outputs of a row (four lanes' 8 values) gets its
            // power-of-two scale (ghip_mx_scale_byte) and is stored as e4m3 codes of the bf16-rounded values over
            // that scale; the scale's E8M0 byte goes where the consuming product's lanes fetch it (a_scale's layout)
            unsigned char* dq = (unsigned char*)g.out + (long long)bm * N + bn;
#pragma unroll
            for (int i = 0; i < NIT; ++i) {
                const int ml = w * (TM / 8) + i * RPI + lane / LPR;
                const int lc = lane % LPR;
                const v4i val = *reinterpret_cast<const v4i*>(smem + ml * PITCH + (lc << 4));
                const unsigned int u0 = (unsigned int)val[0], u1 = (unsigned int)val[1], u2 = (unsigned int)val[2], u3 = (unsigned int)val[3];
                unsigned int m = ghip_bf16x8_amax15(u0, u1, u2, u3);
                unsigned int o1 = (unsigned int)__shfl_xor((int)m, 1, 64); m = m > o1 ? m : o1;
                o1 = (unsigned int)__shfl_xor((int)m, 2, 64); m = m > o1 ? m : o1;
                const int eb = ghip_mx_scale_byte(m);
                *reinterpret_cast<uint2*>(dq + (long long)ml * N + (lc << 3)) = ghip_mx_quant8(u0, u1, u2, u3, eb);
                // the four blocks of a 128-wide run of outputs = the next product's stage: bytes of lanes 0, 4, 8, 12 of
                // every 16 make one dword
                unsigned int sd = (unsigned int)eb | ((unsigned int)__shfl_down(eb, 4, 64) << 8);
                sd |= (unsigned int)__shfl_down((int)sd, 8, 64) << 16;
                if ((lane & 15) == 0) g.out_scale[(long long)((bn >> 7) + (lc >> 4)) * g.ld_out_scale + bm + ml] = sd;
            }
            return;
        }
        unsigned char* dst = (unsigned char*)g.out + ((long long)bm * N + bn) * 2;
        unsigned int am[NIT];
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int ml = w * (TM / 8) + i * RPI + lane / LPR;
            const int lc = (lane % LPR) << 4;
            const v4i val = *reinterpret_cast<const v4i*>(smem + ml * PITCH + lc);
            *reinterpret_cast<v4i*>(dst + (long long)ml * N * 2 + lc) = val;
            if constexpr (EPI == LP_FP8_ACT) {
                // row amax of the stored values for the next layer's per-row scale: bf16 magnitudes
                // order like their bit patterns, so the maximum is taken on 15-bit integers
                unsigned int m = 0;
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const unsigned int u = (unsigned int)val[d];
                    const unsigned int lo = u & 0x7fffu, hi = (u >> 16) & 0x7fffu;
                    m = m > lo ? m : lo;
                    m = m > hi ? m : hi;
                }
                am[i] = m;
            }
        }
        if constexpr (EPI == LP_FP8_ACT) {
            // the NIT reductions side by side, so that their cross-lane steps overlap
#pragma unroll
            for (int o = LPR / 2; o > 0; o >>= 1)
#pragma unroll
                for (int i = 0; i < NIT; ++i) {
                    const unsigned int other = (unsigned int)__shfl_xor((int)am[i], o, 64);
                    am[i] = am[i] > other ? am[i] : other;
                }
            if (lane % LPR == 0)
#pragma unroll
                for (int i = 0; i < NIT; ++i) atomicMax(&g.row_amax_bits[bm + w * (TM / 8) + i * RPI + lane / LPR], am[i] << 16);
        }
        }
    }
    if constexpr (kDgrad) {
        if (g.colsum) {
            float* red = reinterpret_cast<float*>(smem);  // [2][TN]: one row per wavefront row
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();  // the staged tile has been read
            if (lh == 0)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) red[(w >> 2) * TN + wn + ni * 32 + l31] = csum[ni];
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();
            if (t < TN) g.colsum[(long long)tm * N + bn + t] = red[t] + red[TN + t];
        }
    }
}

// XCD-aware tile order of a launch over one product: workgroups whose ids are congruent mod 8 run on one
// XCD (and share its L2); each XCD gets a contiguous range of tile numbers.
__device__ __forceinline__ int xcd_tile_id(int block, int nb)
{
    return (nb & 7) == 0 ? (block & 7) * (nb >> 3) + (block >> 3) : block;
}

template <bool FP8, int EPI, int MI, int NI>
__global__ void __launch_bounds__(NT) gemm_lp_kernel(GemmLpArgs g)
{
    __shared__ __attribute__((aligned(1024))) unsigned char smem[lp_lds_bytes<MI, NI>()];
    gemm_lp_tile<FP8, EPI, MI, NI>(g, xcd_tile_id(blockIdx.x, (g.M / (64 * MI)) * (g.N / (128 * NI))), smem);
}

// The 256 x 256-tile weight gradients of a training step as ONE launch: they are independent of one another once the
// back-propagation chain is through.  A workgroup looks up its product and tile in a schedule the host lays out
// (ghip_gemm_lp_wgrad_plan).  Without a launch boundary after every layer a CU that has finished a tile's update goes
// on with the next layer's tile while its neighbours still write theirs: measured 2 to 4 % less than a launch per
// layer.  (Also measured, and not kept: starting half of the CUs, or half of the XCDs, late, so that the two halves
// never update at the same time.  It recovers about half of the delay it costs and no more.)
struct GemmLpGroupArgs {
    GemmLpArgs p[GHIP_GEMM_LP_GROUP_MAX];
    const unsigned int* sched;   // per workgroup: bits 24..30 = product, bits 0..23 = tile number
};
__global__ void __launch_bounds__(NT) gemm_lp_wgrad_group_kernel(GemmLpGroupArgs grp)
{
    __shared__ __attribute__((aligned(1024))) unsigned char smem[lp_lds_bytes<4, 2>()];
    const unsigned int e = grp.sched[blockIdx.x];
    gemm_lp_tile<false, LP_WGRAD_SGD, 4, 2>(grp.p[(e >> 24) & 0x7f], (int)(e & 0xffffffu), smem);
}

// 256 x 256 tiles when they give every CU at least one workgroup, else 128 x 128.
constexpr int kCUs = 256;
inline bool use_small_tile(int M, int N) { return (long long)(M / 256) * (N / 256) < kCUs; }
// In between, for the fp32-output forward product of a narrow last layer: 256 x 128 tiles where those fill the
// CUs.  Two 128 x 128 workgroups per CU ask the global->LDS path for 124 bytes per clock at the matrix
// cores' rate, twice what it moves; one 256 x 128 workgroup asks for 46.
inline bool use_tall_tile(int M, int N) { return (long long)(M / 256) * (N / 128) >= kCUs; }

template <bool FP8, int EPI>
hipError_t launch(const GemmLpArgs& a, hipStream_t s)
{
    if constexpr (!FP8 && EPI == LP_FWD_F32) {
        if (use_small_tile(a.M, a.N) && use_tall_tile(a.M, a.N)) {
            const int nb = (a.M / 256) * (a.N / 128);
            hipLaunchKernelGGL((gemm_lp_kernel<FP8, EPI, 4, 1>), dim3(nb), dim3(NT), 0, s, a);
            return hipGetLastError();
        }
    }
    if (use_small_tile(a.M, a.N)) {
        const int nb = (a.M / 128) * (a.N / 128);
        hipLaunchKernelGGL((gemm_lp_kernel<FP8, EPI, 2, 1>), dim3(nb), dim3(NT), 0, s, a);
    } else {
        const int nb = (a.M / 256) * (a.N / 256);
        hipLaunchKernelGGL((gemm_lp_kernel<FP8, EPI, 4, 2>), dim3(nb), dim3(NT), 0, s, a);
    }
    return hipGetLastError();
}

void resolve_act(GemmLpArgs& g)
{
    GemmLpArgs::ActForm& a = g.ap;
    const float inf = __builtin_huge_valf(), p = g.act_param;
    a = GemmLpArgs::ActForm{-inf, 0.f, 0.f, 1.f, 0.f, 1.f, 1.f, 0.f, -inf, 0.f, inf, 0.f, 0, 0, 0, 1.f, 1.f, 1.f, 0.f, 0.f};
    switch (g.act) {
    case GHIP_TANH:     a.trans = 1; a.tk = 2.f; a.ta = 2.f; a.tb = -1.f; a.c0 = 1.f; a.c2 = -1.f; break;
    case GHIP_TANHP:    a.trans = 1; a.tk = 2.f; a.ta = 2.f; a.tb = -1.f; a.c0 = 1.f; a.c2 = -1.f;
                        a.clo = p - 1.f; a.vlo = -1.f; a.chi = 1.f - p; a.vhi = 1.f; break;
    case GHIP_SIGMOID:  a.trans = 1; a.c0 = 0.f; a.c1 = 1.f; a.c2 = -1.f; break;
    case GHIP_SIGMOIDP: a.trans = 1; a.c0 = 0.f; a.c1 = 1.f; a.c2 = -1.f;
                        a.clo = p; a.vlo = 0.01f; a.chi = 1.f - p; a.vhi = 0.99f; break;
    case GHIP_RELU:     a.thr = GHIP_OUTLIER; a.a0 = 0.f; a.step = 1; a.dhi = 1.f; a.dlo = 0.f; break;
    case GHIP_LEAKY:    a.thr = GHIP_OUTLIER; a.a0 = p; a.step = 1; a.dhi = 1.f; a.dlo = p; break;
    case GHIP_LINEAR:   a.a1 = p; a.c0 = p; break;
    case GHIP_STEP:     a.thr = p; a.a0 = 0.f; a.a1 = 0.f; a.b1 = 1.f; a.c0 = 0.f; break;
    default: break;
    }
    a.plain = (!a.trans && a.clo == -inf && a.chi == inf) ? 1 : 0;
}

}  // namespace

int ghip_gemm_lp_tile_m(int M, int N) { return use_small_tile(M, N) ? 128 : 256; }

bool ghip_gemm_lp_shape_ok(int M, int N, int K, int fp8)
{
    const int kq = fp8 ? 256 : 128;  // two stages of 128 bytes of K per pass of the main loop
    return M > 0 && N > 0 && K > 0 && (M % 256) == 0 && (N % 256) == 0 && (K % kq) == 0;
}

// what the kernels assume of a product's shapes, pitches and addresses
static bool operands_ok(const GemmLpArgs& a_)
{
    if (!ghip_gemm_lp_shape_ok(a_.M, a_.N, a_.K, a_.fp8)) return false;
    // the LDS-direct loads move 16 bytes per lane: operand rows start on 16-byte boundaries, pitches cover K
    const int es = a_.fp8 ? 1 : 2;
    // (a K-blocked operand's pitch is one stage's 128 bytes and its stages lie kstride bytes apart)
    const bool pitchA_ok = a_.kstrideA ? ((long long)a_.lda * es == 128 && a_.kstrideA % 128 == 0) : (!a_.lda || a_.lda >= a_.K);
    const bool pitchB_ok = a_.kstrideB ? ((long long)a_.ldb * es == 128 && a_.kstrideB % 128 == 0) : (!a_.ldb || a_.ldb >= a_.K);
    return pitchA_ok && pitchB_ok && !(a_.lda && ((long long)a_.lda * es) % 16) && !(a_.ldb && ((long long)a_.ldb * es) % 16) &&
           (((uintptr_t)a_.A | (uintptr_t)a_.B) % 16) == 0;
}

// Schedule of a grouped weight-gradient launch over `count` products of M[i] x N[i] outputs, all of them 256 x 256-tile
// products (ghip_gemm_lp_tile_m): one entry per workgroup.  Workgroup b runs on XCD b % 8, and a CU takes one
// workgroup at a time (the kernel asks for all of its LDS), so entries b, b + 8, b + 16, ... are what one XCD's CUs
// work through in order: every XCD gets a contiguous eighth of each product's tiles (its CUs then share operand
// rows in its L2), the products in the caller's order.  Returns the number of workgroups, -1 if it does not apply.
int ghip_gemm_lp_wgrad_plan(const int* M, const int* N, int count, unsigned int* sched, int cap)
{
    if (count < 1 || count > GHIP_GEMM_LP_GROUP_MAX) return -1;
    int total = 0;
    bool by_xcd = true;
    for (int i = 0; i < count; ++i) {
        if (use_small_tile(M[i], N[i])) return -1;
        const int nb = (M[i] / 256) * (N[i] / 256);
        if (nb > 0xffffff) return -1;
        by_xcd = by_xcd && (nb % 8) == 0;
        total += nb;
    }
    if (total > cap) return -1;
    int k = 0;
    if (!by_xcd) {
        for (int i = 0; i < count; ++i)
            for (int t = 0; t < (M[i] / 256) * (N[i] / 256); ++t) sched[k++] = ((unsigned int)i << 24) | (unsigned int)t;
        return total;
    }
    for (int i = 0; i < count; ++i) {
        const int per = (M[i] / 256) * (N[i] / 256) / 8;
        for (int t = 0; t < per; ++t)
            for (int x = 0; x < 8; ++x) sched[k++] = ((unsigned int)i << 24) | (unsigned int)(x * per + t);
    }
    return total;
}

hipError_t ghip_gemm_lp_wgrad_group(const GemmLpArgs* a, int count, const unsigned int* dev_sched, int blocks, hipStream_t s)
{
    if (count < 1 || count > GHIP_GEMM_LP_GROUP_MAX || !dev_sched || blocks < 1) return hipErrorInvalidValue;
    GemmLpGroupArgs grp;
    memset(&grp, 0, sizeof(grp));
    int total = 0;
    for (int i = 0; i < count; ++i) {
        if (a[i].fp8 || a[i].epilogue != LP_WGRAD_SGD || !operands_ok(a[i]) || use_small_tile(a[i].M, a[i].N) || !a[i].out) return hipErrorInvalidValue;
        grp.p[i] = a[i];
        resolve_act(grp.p[i]);
        total += (a[i].M / 256) * (a[i].N / 256);
    }
    if (total != blocks) return hipErrorInvalidValue;   // the schedule was laid out for other products
    grp.sched = dev_sched;
    hipLaunchKernelGGL(gemm_lp_wgrad_group_kernel, dim3(blocks), dim3(NT), 0, s, grp);
    return hipGetLastError();
}

hipError_t ghip_gemm_lp(const GemmLpArgs& a_, hipStream_t s)
{
    if (!operands_ok(a_)) return hipErrorInvalidValue;
    if (!a_.out && !(a_.epilogue == LP_DGRAD && a_.outT)) return hipErrorInvalidValue;   // only back-propagation may leave the row-major copy out
    GemmLpArgs a = a_;
    resolve_act(a);
    if (!a.fp8) {
        switch (a.epilogue) {
        case LP_FWD_ACT: return launch<false, LP_FWD_ACT>(a, s);
        case LP_FWD_F32: return launch<false, LP_FWD_F32>(a, s);
        case LP_DGRAD:
            if (a.mask_in && a.ap.step) return launch<false, LP_DGRAD_MASK>(a, s);
            return launch<false, LP_DGRAD>(a, s);
        case LP_WGRAD_SGD: return launch<false, LP_WGRAD_SGD>(a, s);
        }
    } else {
        const bool mx = a.epilogue == LP_FP8_ACT_MX || a.epilogue == LP_FP8_F32_MX;
        // block-scaled activations: a dword of scales per row and stage, at least M rows to a stage
        if (mx && (!a.a_scale || a.ld_scale < a.M || ((uintptr_t)a.a_scale % 4))) return hipErrorInvalidValue;
        if (a.epilogue == LP_FP8_ACT_MX && (!a.out_scale || a.ld_out_scale < a.M || ((uintptr_t)a.out % 8))) return hipErrorInvalidValue;
        switch (a.epilogue) {
        case LP_FP8_ACT: return launch<true, LP_FP8_ACT>(a, s);
        case LP_FP8_F32: return launch<true, LP_FP8_F32>(a, s);
        case LP_FP8_ACT_MX: return launch<true, LP_FP8_ACT_MX>(a, s);
        case LP_FP8_F32_MX: return launch<true, LP_FP8_F32_MX>(a, s);
        }
    }
    return hipErrorInvalidValue;
}
