// Flash-attention forward + forward-mode JVP for gfx950 (MI355X, CDNA4): kernels and C ABI.
//
// What is computed (one pass over K/V per 128-query tile, online softmax):
//     S  = Q K^T s                 P = softmax(S)            O  = P V
//     dS = (dQ K^T + Q dK^T) s     H = P * dS   r = rowsum H dO = P dV + H V - r O
//     LSE = logsumexp(S)
// This is the arithmetic of the reference's Triton kernel
// (cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py:47-153 loop, :299-309 init,
// :367-378 epilogue) with the same rounding points: P and H are rounded to the 16-bit input type
// before the P.V-type products while the row sums l and r are accumulated in fp32 from the
// unrounded values (:111-119, :134-146).  Unlike the reference, P dV and H V share ONE fp32
// accumulator (the reference keeps acc_A and acc_B apart but only ever uses their sum, :369).
//
// How it is laid out for CDNA4:
//   * Scores are computed TRANSPOSED: S^T = K Q^T with v_mfma_f32_32x32x16 (K rows are the A operand,
//     32 query columns per wavefront are the B operand).  A lane then owns one query column and 16 of
//     every 32 keys, so the softmax row reductions are in-lane plus ONE exchange with lane^32, and the
//     fp32 S^T registers, once converted to 16-bit, ARE the B operand of O^T = V^T P^T -- no LDS or
//     cross-lane shuffle between the two GEMM stages.
//   * K, V (and dK, dV) are re-tiled ONCE per call by `pack_kv_kernel` into "LDS images": for every
//     32-key tile, the exact byte order in which the MFMA A-operand fragments are consumed
//     (1 KB per fragment = 64 lanes x 16 B, V already transposed and key-permuted to match the
//     S^T register layout).  The attention kernel then moves tiles L2 -> LDS with direct-to-LDS
//     buffer loads (buffer_load_dwordx4 ... lds, no VGPR staging) and reads fragments back with
//     conflict-free linear ds_read_b128.  Re-tiling costs one extra read+write of K/V (<1 % of the
//     call at L=84480) and removes every transpose / swizzle / tail check from the hot loop.
//   * One workgroup = 128 query rows = 8 wavefronts, two per SIMD, in two ROLES.  A single CDNA wavefront overlaps
//     its own VALU and MFMA instructions poorly (4 VALU per MFMA already cost 25 % of the MFMA rate), two wavefronts
//     on one SIMD overlap freely, and one wavefront cannot hold Q, dQ, the scores and both 32 x 128 fp32
//     accumulators in the 256 registers that two-per-SIMD leaves it.  So wavefront w (< 4) is a SCORE wavefront:
//     Q, dQ fragments, the score MFMAs of the next tile interleaved with the softmax VALU work of the current one,
//     the running max / row sums; and wavefront w + 4 (same SIMD) is the OUTPUT wavefront of the same 32 rows: both
//     accumulators and the P.V-type MFMAs.  P^T, H^T (already 16-bit MFMA B operands) and the rescale factor go
//     from one to the other through double-buffered LDS slots, one step apart.
//   * LDS: ring of 4 K parts and ring of 3 V parts (K, dK / V^T, dV^T of 32 keys each), filled 2-3 tiles ahead by
//     the output wavefronts; hand-over slots; 146 KB at d = 128 with tangents.  One bare s_barrier per 32-key step
//     publishes fills and hand-over (a __syncthreads() would also drain every wavefront's LDS operand prefetch).
//   * Forward only (no tangents) runs a different, symmetric kernel (attn_fwd_sym_kernel below): there the softmax
//     VALU work per MFMA is three times higher and a wavefront's state is small, so 12 wavefronts (three per SIMD)
//     each do everything for their own 32 rows and P^T never leaves registers.
//   * Query-tile index is the fastest grid dimension, so the 256 workgroups in flight sweep the same
//     head's K/V images and share them through the per-XCD L2s and the Infinity Cache; workgroups of
//     one XCD start their (order-free) sweep a few tiles apart so they do not hit one L2 channel at once.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>

#include <atomic>
#include <mutex>
#include <set>
#include <type_traits>
#include <utility>

#include "cosmos_attn_hip.h"

namespace {

#include "attn_common_gfx950.h"

constexpr int kBlockM = 128;       // query rows per workgroup (4 wavefronts x 32)
constexpr int kBlockN = 32;        // keys per tile
constexpr int kPackThreads = 256;

enum { MODE_FWD = 0, MODE_JVP_Q = 1, MODE_JVP_FULL = 2 };

// Geometry of one packed KV tile ("LDS image") of kBlockN = 32 keys.  Sections in order: K, dK (the
// "K part"), V^T, dV^T (the "V part"); dK / dV^T only with tangents on k/v.  Every section is a run of
// 1 KB MFMA A-operand fragments (64 lanes x 16 B):
//   K-type fragment c (c < dqk/16):            lane l holds K[l%32][16 c + 8 (l/32) .. +7]
//   V^T-type fragment (db, c) (c < 2), index 2 db + c:
//                                              lane l, slot s holds V[16 c + 8 (s/4) + 4 (l/32) + s%4][32 db + l%32]
// (the key order inside a V^T fragment is the order in which the S^T accumulator registers of
// v_mfma_f32_32x32x16 hold keys, so P^T needs no shuffle to become the B operand).
struct TileGeom {
    int nc, ndb, k_frags, vt_frags, kpart_frags, tile_frags;
    __host__ __device__ TileGeom(int dqk, int dv, bool full)
        : nc(dqk / 16), ndb((dv + 31) / 32), k_frags(dqk / 16), vt_frags(2 * ((dv + 31) / 32)),
          kpart_frags((dqk / 16) * (full ? 2 : 1)),
          tile_frags(((dqk / 16) + 2 * ((dv + 31) / 32)) * (full ? 2 : 1)) {}
};

struct PackParams {
    const uint16_t *k, *v, *tk, *tv;   // tk/tv may be null (then no tangent sections)
    int64_t k_sb, k_sh, k_sl, v_sb, v_sh, v_sl;
    uint4* out;
    int H, Lkv, dqk, dv, n_tiles;
};

// grid (ceil(n_tiles / 2), B*H); every 16-byte unit of a tile image is produced by one thread.
__global__ void __launch_bounds__(kPackThreads) pack_kv_kernel(const PackParams p) {
    const int bh = blockIdx.y, b = bh / p.H, h = bh % p.H;
    const bool full = p.tk != nullptr;
    const TileGeom g(p.dqk, p.dv, full);
    const int64_t k_off = (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
    const int64_t v_off = (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
    const int units = g.tile_frags * 64;
    for (int tt = 0; tt < 2; ++tt) {
        const int t = blockIdx.x * 2 + tt;
        if (t >= p.n_tiles) break;
        uint4* dst = p.out + ((size_t)bh * p.n_tiles + t) * (size_t)(g.tile_frags * (kFragBytes / 16));
        for (int u = threadIdx.x; u < units; u += kPackThreads) {
            int frag = u >> 6;
            const int l = u & 63, i = l & 31, hh = l >> 5;
            uint4 val = make_uint4(0u, 0u, 0u, 0u);
            if (frag < g.kpart_frags) {
                const uint16_t* src = p.k;
                if (frag >= g.k_frags) { frag -= g.k_frags; src = p.tk; }
                const int key = t * kBlockN + i;
                if (key < p.Lkv) val = *reinterpret_cast<const uint4*>(src + k_off + (int64_t)key * p.k_sl + 16 * frag + 8 * hh);
            } else {
                frag -= g.kpart_frags;
                const uint16_t* src = p.v;
                if (frag >= g.vt_frags) { frag -= g.vt_frags; src = p.tv; }
                const int db = frag >> 1, c = frag & 1;
                const int d = 32 * db + i;
                uint16_t e[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    const int key = t * kBlockN + 16 * c + 8 * (s >> 2) + 4 * hh + (s & 3);
                    e[s] = (key < p.Lkv && d < p.dv) ? src[v_off + (int64_t)key * p.v_sl + d] : (uint16_t)0;
                }
                val.x = e[0] | ((uint32_t)e[1] << 16); val.y = e[2] | ((uint32_t)e[3] << 16);
                val.z = e[4] | ((uint32_t)e[5] << 16); val.w = e[6] | ((uint32_t)e[7] << 16);
            }
            dst[u] = val;
        }
    }
}

struct AttnParams {
    const void *q, *tq;
    int64_t q_sb, q_sh, q_sl;
    void *o, *to;
    int64_t o_sb, o_sh, o_sl;
    float* lse;
    const char* kv;            // packed tiles [B*H][n_tiles][tile bytes]
    const int32_t* key_lens;   // nullable
    int H, Lq, Lkv, n_tiles, causal;
    float sm_scale, scale_log2;
    // 1-D grid: workgroups [0, n_full) each own a (query block, head) pair; the remaining n_rem pairs are cut into
    // `splits` key ranges, one workgroup each, which leave unnormalised partial results for attn_combine_kernel.
    // slot = (pair - n_full) * splits + split; block_m = query rows per workgroup (128, or 384 forward only)
    int n_qt, n_full, n_rem, splits;
    // attn_qstream_kernel: BH = batch * heads (the kernel deals the (query block, head) pairs out over its workgroups itself)
    int BH, q_chunk;
    float* part_acc;           // [slot][block_m][d_v] accumulators; with tangents [slot][block_m][2][d_v] (O, T)
    float4* part_stat;         // [slot][block_m]: (running max in log2 units, row sum of P, row sum of H, 0)
};

extern __shared__ __attribute__((aligned(1024))) char smem[];

constexpr int kAttnThreads = 512;   // 4 score wavefronts + 4 output wavefronts, two per SIMD
constexpr int kRingK = 4;           // LDS ring depth, K parts
constexpr int kRingV = 3;           // LDS ring depth, V parts

// Compile-time geometry shared by both roles and the host.
template <int DQK, int DV, int MODE>
struct AttnCfg {
    static constexpr int NC = DQK / 16;             // 16-wide d chunks of the QK^T contraction
    static constexpr int NDB = (DV + 31) / 32;      // 32-row blocks of O^T
    static constexpr bool JVP = MODE != MODE_FWD, FULL = MODE == MODE_JVP_FULL;
    static constexpr int K_FR = NC, VT_FR = 2 * NDB;
    static constexpr int KP_FR = K_FR * (FULL ? 2 : 1), VP_FR = VT_FR * (FULL ? 2 : 1);
    static constexpr int KP_BYTES = KP_FR * kFragBytes, VP_BYTES = VP_FR * kFragBytes;
    static constexpr int TILE_BYTES = KP_BYTES + VP_BYTES;
    static constexpr int DK_OFF = K_FR * kFragBytes;     // inside the K part
    static constexpr int DVT_OFF = VT_FR * kFragBytes;   // inside the V part
    static constexpr int KP_LOADS = (KP_FR + 3) / 4, VP_LOADS = (VP_FR + 3) / 4;   // per output wavefront per tile (they issue all fills)
    static constexpr int GROUP_LOADS = KP_LOADS + VP_LOADS;
    static constexpr int MFMA_PER_C = FULL ? 3 : (JVP ? 2 : 1);
    // P^T (and H^T) of one tile as MFMA B operands: 2 (4) fragments per score wavefront, double-buffered
    static constexpr int PH_FR = JVP ? 4 : 2;
    static constexpr int PH_BYTES = PH_FR * kFragBytes;
    static constexpr int KRING_OFF = 0;
    static constexpr int VRING_OFF = kRingK * KP_BYTES;
    static constexpr int PH_OFF = VRING_OFF + kRingV * VP_BYTES;
    static constexpr int ALPHA_OFF = PH_OFF + 2 * 4 * PH_BYTES;      // [2 stages][4 wavefronts][64 lanes] floats
    static constexpr int LDS_BYTES = ALPHA_OFF + 2 * 4 * 256;
};

template <typename C>
__device__ __forceinline__ void issue_group(const LoadJob& j) {
    static_assert(C::KP_LOADS <= 4 && C::VP_LOADS <= 4, "a part has at most 16 fragments");
    issue_part<C::VP_LOADS>(j.rsrc, j.v_dst, j.lane_off, j.v_src);
    issue_part<C::KP_LOADS>(j.rsrc, j.k_dst, j.lane_off, j.k_src);
}

// ---------------------------------------------------------------------------------------------------------------
// Score wavefront: owns 32 query rows' Q, dQ fragments and softmax statistics.  Per step it issues the score
// MFMAs of the NEXT tile interleaved with the softmax VALU work of the current one, and hands P^T, H^T (16-bit
// MFMA B operands) and the rescale factor of the tile to its output wavefront through LDS.
template <typename T, int DQK, int DV, int MODE>
struct ScoreWave {
    typedef AttnCfg<DQK, DV, MODE> C;
    typedef typename VecOf<T>::v8 V8;
    static constexpr int NC = C::NC;
    static constexpr bool JVP = C::JVP, FULL = C::FULL;
    static constexpr int PD = COSMOS_ATTN_PREFETCH_SCORE;    // LDS operand fetches run this many chunks ahead of use

    // Scores of one tile as this lane sees them: its query column x 16 of the tile's 32 keys (element e is key
    // 8 (e/4) + 4 (lane/32) + e%4 of the tile) -- the accumulator registers of the score MFMAs themselves.
    struct Scores { f32x16 s, ds; };

    V8 qf[NC], tqf[NC];
    float m_run, l_run, r_run;
    float scale_log2, sm_scale;
    int lane;

    __device__ __forceinline__ V8 lds_frag(const char* base, int frag) const {
        return *reinterpret_cast<const V8*>(base + frag * kFragBytes + lane * 16);
    }

    __device__ __forceinline__ static float lane_max(const Scores& x) {
        float mx = x.s[0];
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, x.s[e]);
        return mx;
    }

    // Rare path (last tile of a ragged / padded key range, causal diagonal): masked keys (>= kv_len, or above the
    // diagonal when causal) get score -inf, hence p = 0 and H = 0.
    __device__ __forceinline__ static void mask_scores(Scores& x, int key0, int kv_len, bool causal, int row) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int key = key0 + 8 * (e >> 2) + (e & 3);
            const bool ok = key < kv_len && (!causal || key <= row);
            x.s[e] = ok ? x.s[e] : -INFINITY;
        }
    }

    // Fold a tile's lane-local score max into the running max.  Returns the factor by which everything accumulated
    // so far must be rescaled before this tile is added (exactly 1 when no row's max moved).
    __device__ __forceinline__ float update_max(float mx) {
        {   // max with lane ^ 32 (the other half of the same query column)
            float lo, hi;
            both_halves(mx, lo, hi);
            mx = fmaxf(lo, hi);
        }
        const float m_new = fmaxf(m_run, mx * scale_log2);
        float alpha = 1.0f;
        if (__any(m_new > m_run + max_slack_of<T>(JVP))) {
            alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= alpha;
            r_run *= alpha;
            m_run = m_new;
        }
        return alpha;
    }

    // Softmax of element e of this lane's 16:  p = exp2(s c - m), l += p ;  H = p dS s, r += H.  Both rounded to
    // 16-bit MFMA operands.
    __device__ __forceinline__ void softmax_elem(const Scores& x, V8* pf, V8* hf, int e) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(x.s[e], scale_log2, -m_run));
        l_run += p;
        pf[e >> 3][e & 7] = (T)p;
        if (JVP) {
            const float hv = p * (x.ds[e] * sm_scale);
            r_run += hv;
            hf[e >> 3][e & 7] = (T)hv;
        }
    }

    // One step: softmax of the tile whose scores are in `x` (already folded into m_run; `alpha` is the rescale
    // factor that goes with it) interleaved with the score MFMAs of the next tile (K part `kpart`) into `xn`.
    // P^T / H^T go to `ph_out`, `alpha` to `alpha_out` (LDS addresses).
    // `after_chunk(c)` runs right after the MFMAs of d chunk c, the last use of qf[c] / tqf[c] in the step.
    struct NoHook { __device__ __forceinline__ void operator()(int) const {} };
    template <class F = NoHook>
    __device__ __forceinline__ void step(const Scores& x, Scores& xn, const char* kpart, unsigned ph_out, unsigned alpha_out, float alpha, F after_chunk = F()) {
        V8 pf[2], hf[2];
        V8 fa[NC], fb[NC];
        asm volatile("ds_write_b32 %0, %1" ::"v"(alpha_out + 4 * lane), "v"(alpha) : "memory");
#pragma unroll
        for (int i = 0; i < PD && i < NC; ++i) { fa[i] = lds_frag(kpart, i); if (FULL) fb[i] = lds_frag(kpart + C::DK_OFF, i); }
#pragma unroll
        for (int e = 0; e < 16; ++e) { xn.s[e] = 0.f; xn.ds[e] = 0.f; }
        constexpr int EPC = 16 / NC;   // softmax elements dealt out per chunk (NC <= 8)
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            SCHED_FENCE();
            if (c + PD < NC) { fa[c + PD] = lds_frag(kpart, c + PD); if (FULL) fb[c + PD] = lds_frag(kpart + C::DK_OFF, c + PD); }
            SCHED_FENCE();
            xn.s = mfma32(fa[c], qf[c], xn.s);
#pragma unroll
            for (int k = 0; k < EPC; ++k)
                if (k * C::MFMA_PER_C / EPC == 0) softmax_elem(x, pf, hf, c * EPC + k);
            SCHED_FENCE();
            if (JVP) {
                xn.ds = mfma32(fa[c], tqf[c], xn.ds);
#pragma unroll
                for (int k = 0; k < EPC; ++k)
                    if (k * C::MFMA_PER_C / EPC == 1) softmax_elem(x, pf, hf, c * EPC + k);
                SCHED_FENCE();
            }
            if (FULL) {
                xn.ds = mfma32(fb[c], qf[c], xn.ds);
#pragma unroll
                for (int k = 0; k < EPC; ++k)
                    if (k * C::MFMA_PER_C / EPC == 2) softmax_elem(x, pf, hf, c * EPC + k);
                SCHED_FENCE();
            }
            after_chunk(c);
        }
        // hand P^T, H^T over (asm stores: a visible LDS store would make the compiler wait for vmcnt(0), i.e. for
        // the direct-to-LDS fills in flight)
        const unsigned pa = ph_out + 16 * lane;
        asm volatile("ds_write_b128 %0, %1" ::"v"(pa), "v"(pf[0]) : "memory");
        asm volatile("ds_write_b128 %0, %1 offset:1024" ::"v"(pa), "v"(pf[1]) : "memory");
        if (JVP) {
            asm volatile("ds_write_b128 %0, %1 offset:2048" ::"v"(pa), "v"(hf[0]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:3072" ::"v"(pa), "v"(hf[1]) : "memory");
        }
    }

    // scores of the first tile (prologue)
    __device__ __forceinline__ void scores_plain(Scores& x, const char* kpart) const {
#pragma unroll
        for (int e = 0; e < 16; ++e) { x.s[e] = 0.f; x.ds[e] = 0.f; }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const V8 kf = lds_frag(kpart, c);
            if (JVP) x.ds = mfma32(kf, tqf[c], x.ds);
            x.s = mfma32(kf, qf[c], x.s);
            if (FULL) x.ds = mfma32(lds_frag(kpart + C::DK_OFF, c), qf[c], x.ds);
        }
    }
};

// ---------------------------------------------------------------------------------------------------------------
// Output wavefront: owns the fp32 accumulators O^T and T^T (= (P dV + H V)^T; the reference keeps the two terms
// apart, JVP:134-146, but only ever uses their sum, JVP:369) of the same 32 query rows.
template <typename T, int DQK, int DV, int MODE>
struct OutputWave {
    typedef AttnCfg<DQK, DV, MODE> C;
    typedef typename VecOf<T>::v8 V8;
    static constexpr int NDB = C::NDB;
    static constexpr bool JVP = C::JVP, FULL = C::FULL;
    static constexpr int NB = 2 * NDB;      // MFMA groups of a step, g = c * NDB + db
    static constexpr int PD = COSMOS_ATTN_PREFETCH_OUTPUT;

    f32x16 acc[NDB], acct[NDB];
    int lane;

    __device__ __forceinline__ V8 lds_frag(const char* base, int frag) const {
        return *reinterpret_cast<const V8*>(base + frag * kFragBytes + lane * 16);
    }
    __device__ __forceinline__ void fetch_group(int g, const char* vpart, V8& a, V8& b) const {
        const int c = g / NDB, db = g % NDB;
        a = lds_frag(vpart, 2 * db + c);
        if (FULL) b = lds_frag(vpart + C::DVT_OFF, 2 * db + c);
    }

    // One step: O^T = alpha O^T + V^T P^T ;  T^T = alpha T^T + V^T H^T + dV^T P^T
    __device__ __forceinline__ void step(const char* vpart, const char* ph_in, const char* alpha_in) {
        const float alpha = *reinterpret_cast<const float*>(alpha_in + 4 * lane);
        V8 pf[2], hf[2];
        pf[0] = lds_frag(ph_in, 0); pf[1] = lds_frag(ph_in, 1);
        if (JVP) { hf[0] = lds_frag(ph_in, 2); hf[1] = lds_frag(ph_in, 3); }
        V8 fa[NB], fb[NB];
#pragma unroll
        for (int i = 0; i < PD && i < NB; ++i) fetch_group(i, vpart, fa[i], fb[i]);
        if (__any(alpha != 1.0f)) {   // some row's max moved (wavefront-uniform, rare after the first tiles)
            // v_mul_legacy_f32: 0 * x = 0 for every x, so a factor of zero clears an accumulator whatever it holds (the
            // query-streaming kernel starts a block that way instead of with a clearing pass of its own); for factors
            // in (0, 1] it is the ordinary product.
#pragma unroll
            for (int i = 0; i < NDB; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    asm("v_mul_legacy_f32 %0, %1, %2" : "=v"(acc[i][e]) : "v"(alpha), "v"(acc[i][e]));
                    if (JVP) asm("v_mul_legacy_f32 %0, %1, %2" : "=v"(acct[i][e]) : "v"(alpha), "v"(acct[i][e]));
                }
            }
        }
#pragma unroll
        for (int g = 0; g < NB; ++g) {
            const int c = g / NDB, db = g % NDB;
            SCHED_FENCE();
            if (g + PD < NB) fetch_group(g + PD, vpart, fa[g + PD], fb[g + PD]);
            SCHED_FENCE();
            acc[db] = mfma32(fa[g], pf[c], acc[db]);
            if (JVP) acct[db] = mfma32(fa[g], hf[c], acct[db]);
            if (FULL) acct[db] = mfma32(fb[g], pf[c], acct[db]);
        }
        SCHED_FENCE();
    }
};

template <typename T, int DQK, int DV, int MODE>
__global__ void __attribute__((amdgpu_flat_work_group_size(kAttnThreads, kAttnThreads), amdgpu_waves_per_eu(2, 2)))
attn_fwd_jvp_kernel(const AttnParams p) {
    static_assert(MODE != MODE_FWD, "forward only is attn_fwd_sym_kernel's job");
    typedef AttnCfg<DQK, DV, MODE> C;
    typedef ScoreWave<T, DQK, DV, MODE> SW;
    typedef OutputWave<T, DQK, DV, MODE> OW;
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr int NC = C::NC, NDB = C::NDB;
    constexpr bool JVP = C::JVP;
    constexpr int KP_BYTES = C::KP_BYTES, VP_BYTES = C::VP_BYTES, TILE_BYTES = C::TILE_BYTES;
    // s_waitcnt immediate: vmcnt(n), expcnt / lgkmcnt left at their maxima.  At the top of step s the fills of the
    // V part of tile s-1 and the K part of tile s+1 must have landed; issued after them (in this order) and still
    // allowed in flight: K(s+2), V(s), K(s+3).
    constexpr int IN_FLIGHT = 2 * C::KP_LOADS + C::VP_LOADS;
    constexpr int WAIT_FILLS = (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14) | 0x0F70;

    // 1-D grid: block id -> (pair, key range); pair = query block + n_qt * (batch * H + head)
    const int bid = blockIdx.x;
    const bool partial = bid >= p.n_full && p.splits > 1;
    const int pair = partial ? p.n_full + (bid - p.n_full) / p.splits : bid;
    const int split = partial ? (bid - p.n_full) % p.splits : 0;
    const int qt = pair % p.n_qt, bh = pair / p.n_qt, b = bh / p.H, h = bh % p.H;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool score_role = wave < 4;            // wavefronts w and w + 4 (same SIMD) serve query rows 32 w .. 32 w + 31
    const int qw = wave & 3;
    const int j = lane & 31, hh = lane >> 5;
    const int row0 = qt * kBlockM + qw * 32;     // first query row of this wavefront pair
    const int row = row0 + j;                    // this lane's query row (lanes l and l^32 share it)

    int kv_len = p.Lkv;
    if (p.key_lens) { const int kl = p.key_lens[b]; kv_len = kl < kv_len ? (kl < 0 ? 0 : kl) : kv_len; }
    int n_tiles_all = (kv_len + kBlockN - 1) / kBlockN;
    if (p.causal) { const int lim = (qt * kBlockM + kBlockM + kBlockN - 1) / kBlockN; n_tiles_all = n_tiles_all < lim ? n_tiles_all : lim; }
    // this workgroup's share of the sweep: positions [u_lo, u_lo + n_tiles)  (the whole sweep unless the pair is cut)
    const int u_lo = partial ? (int)((int64_t)split * n_tiles_all / p.splits) : 0;
    const int n_tiles = partial ? (int)((int64_t)(split + 1) * n_tiles_all / p.splits) - u_lo : n_tiles_all;

    char* const kring = smem + C::KRING_OFF;
    char* const vring = smem + C::VRING_OFF;
    // buffer resource over this (batch, head)'s packed tiles: raw (stride 0), num_records in bytes
    const __amdgpu_buffer_rsrc_t kv_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.kv) + (size_t)bh * p.n_tiles * TILE_BYTES, 0, p.n_tiles * TILE_BYTES, 0x00020000);
    // Sweep order.  The softmax recurrences do not care in which order the KV tiles arrive, so a workgroup may
    // start its sweep at any tile and wrap around: position u of the sweep is tile (u + shift) mod n.  Workgroups
    // that share one XCD's L2 (workgroup ids congruent mod 8) start a few tiles apart, so that the first one to
    // reach a tile takes the L2 miss and the ones behind it hit.  The shift is a fixed function of the workgroup id:
    // results are bitwise reproducible from run to run.
    const int n_sweep = n_tiles_all > 0 ? n_tiles_all : 1;
    // (not with causal masking: there the first tile of the sweep must be tile 0, the one tile in which every query row
    // sees a key, so that the running max is finite from the first step on)
    const int shift = p.causal ? 0 : (((pair >> 3) & 31) * COSMOS_ATTN_SWEEP_STAGGER) % n_sweep;
    auto tile_at = [&](int u) { return __builtin_amdgcn_readfirstlane((u_lo + u + shift) % n_sweep); };
    auto wrap_inc = [&](int t) { ++t; return t >= n_sweep ? t - n_sweep : t; };
    const int k_run = ((qw * C::KP_LOADS) % C::KP_FR) * kFragBytes, v_run = ((qw * C::VP_LOADS) % C::VP_FR) * kFragBytes;
    // tk / tv: tiles whose K part / V part the group copies; ku / vu: sweep positions that pick the ring slots
    auto make_job = [&](int tk, int ku, int tv, int vu) {
        LoadJob jb;
        jb.rsrc = kv_rsrc; jb.lane_off = lane * 16;
        jb.k_src = tk * TILE_BYTES + k_run; jb.k_dst = kring + (ku % kRingK) * KP_BYTES + k_run;
        jb.v_src = tv * TILE_BYTES + KP_BYTES + v_run; jb.v_dst = vring + (vu % kRingV) * VP_BYTES + v_run;
        return jb;
    };
    // Fill stream, in issue order:  K(0) K(1) K(2) [V(0) K(3)] | step 0: [V(1) K(4)] | step 1: [V(2) K(5)] | ...
    // (positions past the end of the sweep wrap around: that data is loaded but never used, so that every
    // wavefront always issues the same number of loads)
    // The output wavefronts issue all fills (their instruction stream has room; the score wavefronts' has not).
    if (!score_role) {
#pragma unroll
        for (int u = 0; u < 3; ++u) {
            const LoadJob jb = make_job(tile_at(u), u, 0, 0);
            issue_part<C::KP_LOADS>(jb.rsrc, jb.k_dst, jb.lane_off, jb.k_src);
        }
        issue_group<C>(make_job(tile_at(3), 3, tile_at(0), 0));
    }

    const bool causal = p.causal != 0;
    // wavefront-uniform: does tile t hold a key some row of this wavefront must not see?
    auto need_mask = [&](int t) { return (t * kBlockN + kBlockN > kv_len) || (causal && (t * kBlockN + kBlockN - 1 > row0)); };
    // LDS byte offsets (from `smem`) of this wavefront pair's hand-over slots; stage k adds k * 4 * PH_BYTES / k * 4 * 256
    const unsigned ph_base = C::PH_OFF + qw * C::PH_BYTES, alpha_base = C::ALPHA_OFF + qw * 256;
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;   // LDS address of smem[0], for asm stores
    int t_v = tile_at(1), t_k = tile_at(4);

    if (score_role) {
        SW w;
        w.lane = lane;
        w.scale_log2 = p.scale_log2;
        w.sm_scale = p.sm_scale;
        {   // Q (and dQ) fragments: B operand of S^T = K Q^T; lane holds Q[row][16 c + 8 hh .. +7]
            const int64_t off = (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + (int64_t)row * p.q_sl + 8 * hh;
            const T* qp = reinterpret_cast<const T*>(p.q) + off;
            const T* tqp = reinterpret_cast<const T*>(p.tq) + off;
            const bool live = row < p.Lq;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                V8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                w.qf[c] = live ? *reinterpret_cast<const V8*>(qp + 16 * c) : z;
                if (JVP) w.tqf[c] = live ? *reinterpret_cast<const V8*>(tqp + 16 * c) : z;
            }
        }
        w.m_run = -INFINITY;   // running row max of the scaled scores, log2 domain (same in lanes l and l^32)
        w.l_run = 0.f;         // this lane's partial row sum of p (the two half rows are added in the epilogue)
        w.r_run = 0.f;         // this lane's partial row sum of H

        typename SW::Scores sc0, sc1;   // scores of the current / next tile, swapping roles every step
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): Q, dQ are here
        __builtin_amdgcn_s_barrier();         // ... and so is the K part of the first tile
        asm volatile("" ::: "memory");
        float alpha = 1.0f;
        // fold a tile's scores into the running max (masking them first where the tile needs it)
        auto fold = [&](typename SW::Scores& x, int t) {
            if (need_mask(t)) SW::mask_scores(x, t * kBlockN + 4 * hh, kv_len, causal, row);
            alpha = w.update_max(SW::lane_max(x));
        };
        w.scores_plain(sc0, kring);
        if (n_tiles > 0) fold(sc0, tile_at(0));
        // Step s: softmax of tile s (scores in `cur`), scores of tile s+1 into `nxt` (K part resident since the barrier
        // at the top of the step), statistics of tile s+1.
        auto body = [&](int s, typename SW::Scores& cur, typename SW::Scores& nxt) {
            // own P^T / H^T stores of step s-1 done (lgkmcnt(0)); the barrier then says so of every score wavefront,
            // that the fills of V(s-1), K(s+1) landed, and that every wavefront finished step s-1
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (s < n_tiles) {
                w.step(cur, nxt, kring + ((s + 1) % kRingK) * KP_BYTES, lds0 + ph_base + (s & 1) * 4 * C::PH_BYTES,
                       lds0 + alpha_base + (s & 1) * 4 * 256, alpha);
                if (s + 1 < n_tiles) fold(nxt, t_v);
            }
            t_v = wrap_inc(t_v);   // tile at sweep position s + 2
        };
        for (int s = 0; s <= n_tiles; s += 2) {
            body(s, sc0, sc1);
            if (s + 1 <= n_tiles) body(s + 1, sc1, sc0);
        }
        __builtin_amdgcn_s_waitcnt(0x0070);   // drain the (unused) trailing fills and the last stores
        __builtin_amdgcn_s_barrier();         // the output wavefronts have read the last alpha
        // ---- epilogue, statistics: 1 / l and r / l to the output wavefront ; LSE = (m + log2 l) ln 2 ----
        const float l_tot = w.l_run + __shfl_xor(w.l_run, 32);
        const float r_tot = w.r_run + __shfl_xor(w.r_run, 32);
        const float inv_l = 1.0f / l_tot;
        const float r_over_l = r_tot * inv_l;
        asm volatile("ds_write_b32 %0, %1" ::"v"(lds0 + alpha_base + 4 * lane), "v"(inv_l) : "memory");
        asm volatile("ds_write_b32 %0, %1" ::"v"(lds0 + alpha_base + 4 * 256 + 4 * lane), "v"(r_over_l) : "memory");
        __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        if (partial) {   // a key range only: leave the statistics for attn_combine_kernel
            if (hh == 0) {
                const int64_t slot = (int64_t)(pair - p.n_full) * p.splits + split;
                p.part_stat[slot * kBlockM + qw * 32 + j] = make_float4(w.m_run, l_tot, r_tot, 0.f);
            }
        } else if (row < p.Lq && p.lse && hh == 0) {
            p.lse[(int64_t)bh * p.Lq + row] = (w.m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
        }
    } else {
        OW w;
        w.lane = lane;
#pragma unroll
        for (int i = 0; i < NDB; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) { w.acc[i][e] = 0.f; if (JVP) w.acct[i][e] = 0.f; }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // Step s: accumulate tile s-1 (P^T, H^T, alpha written by the score wavefront during step s-1).
        for (int s = 0; s <= n_tiles; ++s) {
            __builtin_amdgcn_s_waitcnt(WAIT_FILLS);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue_group<C>(make_job(t_k, s + 4, t_v, s + 1));
            if (s > 0)
                w.step(vring + ((s - 1) % kRingV) * VP_BYTES, smem + ph_base + ((s - 1) & 1) * 4 * C::PH_BYTES,
                       smem + alpha_base + ((s - 1) & 1) * 4 * 256);
            t_v = wrap_inc(t_v); t_k = wrap_inc(t_k);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // ---- epilogue, outputs: O = acc / l ; dO = (T - (r / l) acc) / l ----
        const float inv_l = *reinterpret_cast<const float*>(smem + alpha_base + 4 * lane);
        const float r_over_l = *reinterpret_cast<const float*>(smem + alpha_base + 4 * 256 + 4 * lane);
        if (partial) {   // a key range only: leave the unnormalised accumulators for attn_combine_kernel
            const int64_t slot = (int64_t)(pair - p.n_full) * p.splits + split;
            float* pa = p.part_acc + (slot * kBlockM + qw * 32 + j) * (JVP ? 2 * DV : DV);
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d = 32 * db + 8 * g + 4 * hh;
                    if (d < DV) {
                        *reinterpret_cast<float4*>(pa + d) = make_float4(w.acc[db][4 * g], w.acc[db][4 * g + 1], w.acc[db][4 * g + 2], w.acc[db][4 * g + 3]);
                        if (JVP) *reinterpret_cast<float4*>(pa + DV + d) = make_float4(w.acct[db][4 * g], w.acct[db][4 * g + 1], w.acct[db][4 * g + 2], w.acct[db][4 * g + 3]);
                    }
                }
            }
        } else if (row < p.Lq) {
            const int64_t off = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)row * p.o_sl;
            T* op = reinterpret_cast<T*>(p.o) + off;
            T* top = reinterpret_cast<T*>(p.to) + off;
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d = 32 * db + 8 * g + 4 * hh;   // registers 4g..4g+3 are 4 consecutive d
                    if (d < DV) {
                        V4 ov, tov;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float of = w.acc[db][4 * g + r] * inv_l;
                            ov[r] = (T)of;
                            if (JVP) tov[r] = (T)((w.acct[db][4 * g + r] - r_over_l * w.acc[db][4 * g + r]) * inv_l);
                        }
                        *reinterpret_cast<V4*>(op + d) = ov;
                        if (JVP) *reinterpret_cast<V4*>(top + d) = tov;
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Short key sequences (text cross-attention: a few hundred keys against tens of thousands of queries).  With 16 key
// tiles per query block the kernel above spends more time starting and finishing a workgroup (query load, first fills,
// normalisation, output stores: none of it overlapped with anything) than sweeping the keys.  Here a workgroup keeps
// going: it serves a run of consecutive query blocks of one (batch, head) as ONE stream of steps.  The K/V tiles of the
// head keep circulating through the LDS rings without a gap (the sweep of the next query block starts where the last
// one ended, modulo the tile count).  Same roles, rings, hand-over and arithmetic as attn_fwd_jvp_kernel; no causal
// mask, no key-range split.  All three tangent modes (forward only runs here too: at these lengths the fixed costs
// decide).
//
// At these lengths a query block's own memory traffic (Q, dQ in; O, dO out: 128 KB) weighs as much as its key sweep, and
// the two only overlap if the traffic is spread over the sweep: a block's 64 KB of stores issued in one step queue up
// in the compute unit's memory pipeline in front of the K/V fills of the following steps and stall them (measured: the
// stores then cost their full drain time on top of the sweep).  So, except with tangents on k and v (no LDS left):
//   * an output wavefront normalises a finished block into a private LDS region (whole rows, 16-byte chunks XOR-swizzled
//     by row so that neither side has bank conflicts) and goes on accumulating the next block;
//   * the score wavefront of the pair drains that region to memory a few 1 KB stores per step during the first steps of
//     the next block's sweep (16-byte stores covering whole rows).  Its vector-memory counter is not the one that tracks
//     the fills, so nobody ever waits for a store to retire;
//   * once the region is empty again, the output wavefront copies the next block's Q / dQ rows into it (direct-to-LDS
//     loads covering whole rows, one step before the block's end), and the score wavefront reads its fragments from there
//     at the start of the block's last step, the first to need them.  A block's steps: results of the last block written
//     to the region / drained / next rows copied / next rows read.
// With tangents on k and v the output wavefronts store from their accumulators right after a block's last accumulation
// step, and the score wavefront fetches the next block's Q / dQ rows from memory into the registers of the current ones,
// d chunk by d chunk, as the block's last score computation lets go of them (no second register set, no copies).
// For all this a block has at least kStreamMinTiles steps (a row of fewer valid tiles walks fully masked ones as well).
constexpr int kNumXCDs = 8;           // MI355X: 8 accelerator dies of 32 compute units, workgroup ids dealt round-robin
constexpr int kStreamMinTiles = 4;
constexpr int kStreamStagger = 2;     // tiles between the sweep starts of the workgroups of an XCD
constexpr int kStreamBlockCost = 5;   // what starting and finishing a query block costs, in half steps (measured: about 2.5 steps)

template <int DV, int MODE>
struct StreamStores {
    static constexpr bool JVP = MODE != MODE_FWD;
    static constexpr bool TRICKLE = MODE != MODE_JVP_FULL;
    static constexpr int NT = JVP ? 2 : 1;                            // tensors stored: O (and dO)
    static constexpr int DVP = DV < 32 ? DV : 32 * ((DV + 31) / 32);   // channels stored (DV = 16: half an accumulator block)
    static constexpr int CPR = DVP / 8;                  // 16-byte chunks per row
    static constexpr int ROW_BYTES = DVP * 2;
    static constexpr int RPS = 64 / CPR;                 // rows one wavefront-wide 16-byte store covers
    static constexpr int SPT = 32 / RPS;                 // such stores per tensor, wavefront and block
    static constexpr int NS = NT * SPT;
    static constexpr int XP_BYTES = TRICKLE ? NT * 32 * ROW_BYTES : 0;   // LDS region per wavefront pair
    static constexpr int N_DIRECT = (DVP / 8) * NT;      // stores per output wavefront and block when storing from the accumulators
};

template <typename T, int DQK, int DV, int MODE>
__global__ void __attribute__((amdgpu_flat_work_group_size(kAttnThreads, kAttnThreads), amdgpu_waves_per_eu(2, 2)))
attn_qstream_kernel(const AttnParams p) {
    typedef AttnCfg<DQK, DV, MODE> C;
    typedef ScoreWave<T, DQK, DV, MODE> SW;
    typedef OutputWave<T, DQK, DV, MODE> OW;
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr int NC = C::NC, NDB = C::NDB;
    constexpr bool JVP = C::JVP;
    constexpr int KP_BYTES = C::KP_BYTES, VP_BYTES = C::VP_BYTES, TILE_BYTES = C::TILE_BYTES;
    typedef StreamStores<DV, MODE> ST;
    constexpr bool TRICKLE = ST::TRICKLE;
    constexpr int STAT_OFF = C::LDS_BYTES;        // [2 query-block parities][inv_l, r / l][4 wavefronts][64 lanes] floats
    constexpr int XP_OFF = STAT_OFF + 2 * 2 * 4 * 256;   // [4 wavefront pairs] finished blocks on their way out (TRICKLE)
    // vmcnt immediates (see attn_fwd_jvp_kernel): the newest IN_FLIGHT fills may still be in flight at the top of a
    // step; when an output wavefront stored a query block from its accumulators in the step before, so may the N_STORES
    // stores issued behind them (vector memory operations of a wavefront retire in issue order).
    constexpr int IN_FLIGHT = 2 * C::KP_LOADS + C::VP_LOADS;
    constexpr int N_STORES = ST::N_DIRECT;
    static_assert(IN_FLIGHT + N_STORES < 64, "vmcnt is a 6-bit counter");
    constexpr int WAIT_FILLS = (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14) | 0x0F70;
    constexpr int WAIT_FILLS_STORES = ((IN_FLIGHT + N_STORES) & 15) | (((IN_FLIGHT + N_STORES) >> 4) << 14) | 0x0F70;

    const int bid = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool score_role = wave < 4;
    const int qw = wave & 3;
    const int j = lane & 31, hh = lane >> 5;

    // Which (query block, head) pairs this workgroup serves.  All pairs, in the order (batch, head, query block), form one
    // line of work; a pair of batch row b weighs 2 n_b + kStreamBlockCost half steps (n_b key tiles per block, plus what
    // starting and finishing a block costs), and the gridDim.x workgroups cut the line into pieces of equal weight (the
    // host launches a multiple of the number of compute units: no thin last round, whatever the key lengths of the rows).
    // A piece may run over the end of a head: the workgroup then serves it as several streams, one after the other.
    auto tiles_of = [&](int bb) {
        int len = p.Lkv;
        if (p.key_lens) { const int kl = __builtin_amdgcn_readfirstlane(p.key_lens[bb]); len = kl < len ? (kl < 0 ? 0 : kl) : len; }
        const int nt = (len + kBlockN - 1) / kBlockN;
        return nt < kStreamMinTiles ? kStreamMinTiles : nt;
    };
    // (everything below is the same in all lanes; said explicitly, so that it lives in scalar registers)
    auto uniform64 = [](int64_t v) {
        const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)((uint64_t)v >> 32));
        return (int64_t)(((uint64_t)hi << 32) | lo);
    };
    const int n_batch = p.BH / p.H;
    const int64_t per_row = (int64_t)p.H * p.n_qt;          // pairs of one batch row
    int64_t total_w = 0;
    for (int bb = 0; bb < n_batch; ++bb) total_w += per_row * (2 * tiles_of(bb) + kStreamBlockCost);
    // first pair at or after weight position x on the line
    auto locate = [&](int64_t x) {
        int64_t cum = 0;
        for (int bb = 0; bb < n_batch; ++bb) {
            const int64_t w = 2 * tiles_of(bb) + kStreamBlockCost, span = per_row * w;
            if (x < cum + span) return bb * per_row + (x - cum + w - 1) / w;
            cum += span;
        }
        return n_batch * per_row;
    };
    // Piece number: workgroups are dealt to the 8 XCDs in turn (id mod 8), and each XCD has an L2 of its own, so the pieces
    // are numbered such that an XCD's workgroups get one contiguous eighth of the line -- a few heads' K/V images per L2
    // instead of all of them (the grid is a multiple of 8).
    const int piece = (bid % kNumXCDs) * ((int)gridDim.x / kNumXCDs) + bid / kNumXCDs;
    const int64_t pair_lo = uniform64(locate(total_w * piece / (int64_t)gridDim.x)), pair_hi = uniform64(locate(total_w * (piece + 1) / (int64_t)gridDim.x));

    for (int64_t pair = pair_lo; pair < pair_hi;) {
    const int bh = (int)(pair / p.n_qt), b = bh / p.H, h = bh % p.H;
    const int qt0 = (int)(pair % p.n_qt);                                      // first query block of this stream
    const int nq = (int)(pair_hi - pair < (int64_t)(p.n_qt - qt0) ? pair_hi - pair : (int64_t)(p.n_qt - qt0));   // its query blocks (>= 1)
    pair += nq;

    int kv_len = p.Lkv;
    if (p.key_lens) { const int kl = __builtin_amdgcn_readfirstlane(p.key_lens[b]); kv_len = kl < kv_len ? (kl < 0 ? 0 : kl) : kv_len; }
    // key tiles per query block: at least kStreamMinTiles (a finished block drains, and the next block's rows are touched,
    // fetched and waited for, during the sweep).  Tiles past the last valid key are fully masked; past the end of the
    // packed buffer the fills deliver zeros.
    const int n_valid = (kv_len + kBlockN - 1) / kBlockN;
    const int n = n_valid < kStreamMinTiles ? kStreamMinTiles : n_valid;
    const int n_flat = nq * n;                     // steps of the whole stream: position f = query block f / n, tile f % n

    char* const kring = smem + C::KRING_OFF;
    char* const vring = smem + C::VRING_OFF;
    const __amdgpu_buffer_rsrc_t kv_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.kv) + (size_t)bh * p.n_tiles * TILE_BYTES, 0, p.n_tiles * TILE_BYTES, 0x00020000);
    // position f of the stream reads tile (f + shift) mod n: one shift for all query blocks, so the tiles keep arriving
    // in the same cyclic order across block boundaries and the fills issued ahead of a boundary are the next block's first
    // (a sweep with fully masked tiles starts at tile 0: the first tile of a block must have a valid key, or the running max
    // would still be -inf when the exponentials refer to it)
    const int shift = n_valid < n ? 0 : (((bid >> 3) & 31) * kStreamStagger) % n;
    auto tile_at = [&](int u) { return __builtin_amdgcn_readfirstlane((u + shift) % n); };
    auto wrap_inc = [&](int t) { ++t; return t >= n ? t - n : t; };
    const int k_run = ((qw * C::KP_LOADS) % C::KP_FR) * kFragBytes, v_run = ((qw * C::VP_LOADS) % C::VP_FR) * kFragBytes;
    auto make_job = [&](int tk, int ku, int tv, int vu) {
        LoadJob jb;
        jb.rsrc = kv_rsrc; jb.lane_off = lane * 16;
        jb.k_src = tk * TILE_BYTES + k_run; jb.k_dst = kring + (ku % kRingK) * KP_BYTES + k_run;
        jb.v_src = tv * TILE_BYTES + KP_BYTES + v_run; jb.v_dst = vring + (vu % kRingV) * VP_BYTES + v_run;
        return jb;
    };
    if (!score_role) {   // fill stream, in issue order:  K(0) K(1) K(2) [V(0) K(3)] | step 0: [V(1) K(4)] | step 1: [V(2) K(5)] | ...
#pragma unroll
        for (int u = 0; u < 3; ++u) {
            const LoadJob jb = make_job(tile_at(u), u, 0, 0);
            issue_part<C::KP_LOADS>(jb.rsrc, jb.k_dst, jb.lane_off, jb.k_src);
        }
        issue_group<C>(make_job(tile_at(3), 3, tile_at(0), 0));
    }

    auto need_mask = [&](int t) { return t * kBlockN + kBlockN > kv_len; };
    const unsigned ph_base = C::PH_OFF + qw * C::PH_BYTES, alpha_base = C::ALPHA_OFF + qw * 256, stat_base = STAT_OFF + qw * 256;
    const unsigned xp_base = XP_OFF + qw * ST::XP_BYTES;
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    int t_v = tile_at(1), t_k = tile_at(4);

    if (score_role) {
        SW w;
        w.lane = lane;
        w.scale_log2 = p.scale_log2;
        w.sm_scale = p.sm_scale;
        // Q (and dQ) fragments of a query block: B operand of S^T = K Q^T; lane holds Q[row][16 c + 8 hh .. +7] (rows past
        // Lq read the last row instead: their results are never stored).  Addresses are a wavefront-uniform base (scalar
        // registers) plus a 32-bit lane offset (the launch code sends only tensors here whose heads span less than 2 GiB):
        // no 64-bit per-lane pointers live across the steps.
        const char* const q_head = reinterpret_cast<const char*>(p.q) + ((int64_t)b * p.q_sb + (int64_t)h * p.q_sh) * 2;
        const char* const tq_head = reinterpret_cast<const char*>(JVP ? p.tq : p.q) + ((int64_t)b * p.q_sb + (int64_t)h * p.q_sh) * 2;
        auto q_off = [&](int qt) {
            int row = qt * kBlockM + qw * 32 + j;
            row = row < p.Lq ? row : p.Lq - 1;
            return ((unsigned)row * (unsigned)p.q_sl + 8u * hh) * 2u;
        };
        {
            const unsigned off = q_off(qt0);
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                w.qf[c] = *reinterpret_cast<const V8*>(q_head + off + 32 * c);
                if (JVP) w.tqf[c] = *reinterpret_cast<const V8*>(tq_head + off + 32 * c);
            }
        }
        w.m_run = -INFINITY;
        w.l_run = 0.f;
        w.r_run = 0.f;
        // The next block's rows replace the current ones in place.  With tangents on k and v: step n-2 of a block computes
        // the block's last scores, and right after the MFMAs of d chunk c it fetches chunk c of the next block into the
        // same registers; step n-1 (the next block's first scores) then waits chunk by chunk.  That leaves a load one step
        // to arrive, enough from the L2 but not from memory: step 0 of the block touches every 128-byte line of those rows
        // (4 bytes per lane).  Such a fetch is 16-byte pieces of 32 different rows per instruction, 32 cache lines each:
        // 2000 cycles per block during which the fills queue up behind it.  In the other modes the rows therefore come
        // through the LDS region of the pair, which is free once the last block's results have left it: the output
        // wavefront copies them there during step n-2 with direct-to-LDS loads that cover whole lines (4 rows of 256 bytes
        // per instruction at d = 128), XOR-swizzled like the results, and this wavefront reads them at the top of step n-1.
        // The touches stay (the copy then hits the L2).
        constexpr int Q_LINES = (2 * DQK + 127) / 128;   // lines per row (at most 2: lane half hh takes line hh)
        int warm_q = 0, warm_tq = 0;
        // A finished block drains during steps 1 .. n-3 of the next one (then the region takes the next block's rows).
        // The stores go out in batches of DB (reads from the region first, then the stores: one wait per batch), a whole
        // number of batches per step.  Everything this wavefront does sits on the critical path of the step (one instruction
        // every few cycles, whatever its kind), so a store is kept to a handful of instructions: addresses are a scalar
        // base per head and tensor plus 32-bit offsets, batch and store numbers are compile-time inside a batch.
        constexpr int DB = ST::NS < 4 ? ST::NS : 4;
        static_assert(ST::RPS >= ST::CPR || (DB * ST::RPS) % ST::CPR == 0, "the swizzle key of a batch's stores depends on the position in the batch only");
        const int drain_steps = n - 3;
        const int st_per_step = ((ST::NS + drain_steps - 1) / drain_steps + DB - 1) / DB * DB;
        // store number i of a query block's results: tensor i / SPT, rows (i % SPT) RPS .. + RPS - 1 of this wavefront's 32;
        // lane l stores chunk l % CPR of row l / CPR of those
        const int rr = lane / ST::CPR, ch = lane % ST::CPR;
        const unsigned x_lane = rr * ST::ROW_BYTES + ((ch ^ (rr & (ST::CPR - 1))) << 4);
        const unsigned o_lane = ((unsigned)rr * (unsigned)p.o_sl + 8u * ch) * 2u;
        const int64_t o_head = ((int64_t)b * p.o_sb + (int64_t)h * p.o_sh) * 2;
        char* const o_base = reinterpret_cast<char*>(p.o) + o_head;
        char* const to_base = reinterpret_cast<char*>(JVP ? p.to : p.o) + o_head;
        const unsigned o_rps = (unsigned)ST::RPS * (unsigned)p.o_sl * 2u;       // bytes from one store's rows to the next one's
        auto drain_batch = [&](int qt, int i0, auto whole) {
            // store i0 + k: tensor t, row group g.  A batch lies inside one tensor (t and the first group g0 are scalars, the
            // rest compile-time) unless a tensor has fewer stores than a batch: then there is one batch, i0 = 0.
            constexpr bool ONE_T = ST::SPT >= DB;
            const int t0 = ONE_T ? i0 / ST::SPT : 0, g0 = ONE_T ? i0 % ST::SPT : 0;
            const char* const src = smem + xp_base + t0 * 32 * ST::ROW_BYTES + g0 * ST::RPS * ST::ROW_BYTES;
            const int r0 = qt * kBlockM + qw * 32 + g0 * ST::RPS;
            const unsigned off0 = (unsigned)r0 * (unsigned)p.o_sl * 2u + o_lane;
            V8 val[DB];
#pragma unroll
            for (int k = 0; k < DB; ++k) {
                const int tk = ONE_T ? 0 : k / ST::SPT, gk = ONE_T ? k : k % ST::SPT;
                constexpr unsigned none = 0;
                const unsigned sw = ST::RPS < ST::CPR ? (unsigned)((gk * ST::RPS) & (ST::CPR - 1)) << 4 : none;   // row g RPS + rr has swizzle key (g RPS + rr) mod CPR
                val[k] = *reinterpret_cast<const V8*>(src + tk * 32 * ST::ROW_BYTES + gk * ST::RPS * ST::ROW_BYTES + (x_lane ^ sw));
            }
#pragma unroll
            for (int k = 0; k < DB; ++k) {
                const int tk = ONE_T ? t0 : k / ST::SPT, gk = ONE_T ? k : k % ST::SPT;
                char* const base = tk ? to_base : o_base;
                const unsigned off = off0 + gk * o_rps;
                // (a compiler-generated store, not inline assembly: after a store of more than 8 bytes the data registers
                // must not be overwritten for two cycles, which the compiler only knows to respect for its own stores)
                if (decltype(whole)::value || r0 + gk * ST::RPS + rr < p.Lq)
                    __builtin_nontemporal_store(val[k], reinterpret_cast<V8*>(base + off));
            }
        };
        auto drain = [&](int qt, int lo, int hi) {
            if ((qt + 1) * kBlockM <= p.Lq) {       // all rows of the block exist (every block but a head's last)
                for (int i = lo; i < hi; i += DB) drain_batch(qt, i, std::true_type());
            } else {
                for (int i = lo; i < hi; i += DB) drain_batch(qt, i, std::false_type());
            }
        };

        typename SW::Scores sc0, sc1;
        __builtin_amdgcn_s_barrier();         // the K part of the first tile is in LDS (the output wavefronts waited for it)
        asm volatile("" ::: "memory");
        float alpha = 1.0f;
        auto fold = [&](typename SW::Scores& x, int t) {
            if (need_mask(t)) SW::mask_scores(x, t * kBlockN + 4 * hh, kv_len, false, 0);
            alpha = w.update_max(SW::lane_max(x));
        };
        w.scores_plain(sc0, kring);
        fold(sc0, tile_at(0));
        alpha = 0.0f;                            // a block's first tile: the output wavefront's rescaling pass clears its accumulators
        int f = 0, qi = 0;                       // position in the stream, and its query block
        bool more = nq > 1;                      // is there a block after block qi?
        // Step f = position s_in of block qi's sweep: softmax of the tile at position f (scores in `cur`), scores of position
        // f+1 into `nxt`, its statistics.  Three kinds, as separate code: steps 0 .. n-3 of a block; step n-2, which refills
        // the Q / dQ registers from memory with tangents on k and v (a plain step otherwise); step n-1, which waits for
        // them chunk by chunk, or reads them from the LDS region, and closes the block.  (Apart, so that the compiler sees
        // every fetch waited for inside the pair of steps that issues it and puts no waits for it -- which would wait for
        // the drain stores as well -- into the other steps.)
        typedef std::integral_constant<int, 0> Plain;
        typedef std::integral_constant<int, 1> Refill;
        typedef std::integral_constant<int, 2> Last;
        auto one = [&](auto kind, typename SW::Scores& cur, typename SW::Scores& nxt, int s_in) {
            constexpr int KIND = decltype(kind)::value;
            __builtin_amdgcn_s_waitcnt(0xC07F);      // own LDS stores of step f-1 done
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const unsigned ph_out = lds0 + ph_base + (f & 1) * 4 * C::PH_BYTES, alpha_out = lds0 + alpha_base + (f & 1) * 4 * 256;
            const char* const kpart = kring + ((f + 1) % kRingK) * KP_BYTES;
            if (KIND == 0 && more && s_in == 0) {
                const unsigned off = q_off(qt0 + qi + 1) - 16u * hh + (Q_LINES > 1 ? 128u * hh : 0u);
                warm_q = *reinterpret_cast<const int*>(q_head + off);
                if (JVP) warm_tq = *reinterpret_cast<const int*>(tq_head + off);
            }
            if (KIND == 2 && TRICKLE && more) {
                // the next block's rows, from the pair's LDS region: 16-byte piece k = 2 c + hh of row j sits at position
                // k ^ (j mod CPR) of the row
                const char* const src = smem + xp_base + j * ST::ROW_BYTES;
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const unsigned pos = (unsigned)((2 * c + hh) ^ (j & (ST::CPR - 1))) << 4;
                    w.qf[c] = *reinterpret_cast<const V8*>(src + pos);
                    if (JVP) w.tqf[c] = *reinterpret_cast<const V8*>(src + 32 * ST::ROW_BYTES + pos);
                }
            }
            if (KIND == 1 && !TRICKLE && more) {
                const unsigned off = q_off(qt0 + qi + 1);
                w.step(cur, nxt, kpart, ph_out, alpha_out, alpha, [&](int c) {
                    w.qf[c] = __builtin_nontemporal_load(reinterpret_cast<const V8*>(q_head + off + 32 * c));
                    if (JVP) w.tqf[c] = __builtin_nontemporal_load(reinterpret_cast<const V8*>(tq_head + off + 32 * c));
                });
            } else {
                w.step(cur, nxt, kpart, ph_out, alpha_out, alpha);
            }
            if (KIND == 2) asm volatile("" ::"v"(warm_q), "v"(warm_tq));   // the touches are done with (keeps their registers theirs until here)
            if (TRICKLE && KIND == 0 && qi > 0 && s_in > 0) {
                const int lo = (s_in - 1) * st_per_step, hi = lo + st_per_step;
                drain(qt0 + qi - 1, lo, hi < ST::NS ? hi : ST::NS);
            }
            if (KIND == 2) {
                // statistics of the finished block: 1 / l and r / l to the output wavefront, LSE = (m + log2 l) ln 2
                float l_lo, l_hi, r_lo, r_hi;
                both_halves(w.l_run, l_lo, l_hi);
                both_halves(w.r_run, r_lo, r_hi);
                const float l_tot = l_lo + l_hi, r_tot = r_lo + r_hi;
                const float inv_l = 1.0f / l_tot;
                const float r_over_l = r_tot * inv_l;
                const unsigned sa = lds0 + stat_base + (qi & 1) * 2 * 4 * 256 + 4 * lane;
                asm volatile("ds_write_b32 %0, %1" ::"v"(sa), "v"(inv_l) : "memory");
                asm volatile("ds_write_b32 %0, %1 offset:1024" ::"v"(sa), "v"(r_over_l) : "memory");
                const int row = (qt0 + qi) * kBlockM + qw * 32 + j;
                if (row < p.Lq && p.lse && hh == 0)
                    p.lse[(int64_t)bh * p.Lq + row] = (w.m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
                w.m_run = -INFINITY; w.l_run = 0.f; w.r_run = 0.f;
            }
            if (f + 1 < n_flat) fold(nxt, t_v);
            if (KIND == 2) alpha = 0.0f;         // the next block's first tile: see above
            t_v = wrap_inc(t_v);   // tile at position f + 2
            ++f;
        };
        // sc0 and sc1 swap roles every step; a block always starts and ends with the current scores in sc0 (after an odd
        // number of steps the scores move back: 32 register copies per block)
        for (qi = 0; qi < nq; ++qi) {
            more = qi + 1 < nq;
            int s_in = 0;
            for (; s_in + 2 <= n - 2; s_in += 2) {
                one(Plain(), sc0, sc1, s_in);
                one(Plain(), sc1, sc0, s_in + 1);
            }
            if (s_in < n - 2) {
                one(Plain(), sc0, sc1, s_in);
                sc0 = sc1;
            }
            one(Refill(), sc0, sc1, n - 2);
            one(Last(), sc1, sc0, n - 1);
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);      // step n_flat: the output wavefronts accumulate the last tile
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (TRICKLE) {   // the last block: its region was written during the last step
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            drain(qt0 + nq - 1, 0, ST::NS);
        }
    } else {
        OW w;
        w.lane = lane;
        auto zero_acc = [&]() {
#pragma unroll
            for (int i = 0; i < NDB; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) { w.acc[i][e] = 0.f; if (JVP) w.acct[i][e] = 0.f; }
            }
        };
        zero_acc();
        // TRICKLE: the next block's Q (and dQ) rows of this pair go to the pair's LDS region during the score wavefront's
        // step n-2, as direct-to-LDS loads of 1 KB each that cover whole rows (RPS rows per load, SPT loads per tensor):
        // lane l fills 16-byte position l % CPR of row l / CPR with piece (l % CPR) ^ (row mod CPR) of that row, the
        // swizzle the results use.  Rows past Lq lie outside the buffer resource and arrive as zeros.
        const int64_t q_head_off = ((int64_t)b * p.q_sb + (int64_t)h * p.q_sh) * 2;
        const unsigned q_extent = (unsigned)(p.Lq - 1) * (unsigned)p.q_sl * 2u + 2u * DQK;
        const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char*>(reinterpret_cast<const char*>(p.q)) + q_head_off, 0, q_extent, 0x00020000);
        const __amdgpu_buffer_rsrc_t tq_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char*>(reinterpret_cast<const char*>(JVP ? p.tq : p.q)) + q_head_off, 0, q_extent, 0x00020000);
        const int c_rr = lane / ST::CPR, c_ch = lane % ST::CPR;
        const unsigned c_row = (unsigned)c_rr * (unsigned)p.q_sl * 2u;
        const unsigned c_piece = c_ch ^ (c_rr & (ST::CPR - 1));
        auto copy_rows = [&](int qt) {
            const unsigned row0 = qt * kBlockM + qw * 32;
#pragma unroll
            for (int t = 0; t < ST::NT; ++t) {
#pragma unroll
                for (int g = 0; g < ST::SPT; ++g) {
                    constexpr unsigned none = 0;
                    const unsigned sw = ST::RPS < ST::CPR ? (unsigned)((g * ST::RPS) & (ST::CPR - 1)) : none;
                    const int voff = (int)(c_row + ((c_piece ^ sw) << 4));
                    const int soff = (int)((row0 + g * ST::RPS) * (unsigned)p.q_sl * 2u);
                    lds_load<0>(t ? tq_rsrc : q_rsrc, smem + xp_base + t * 32 * ST::ROW_BYTES + g * ST::RPS * ST::ROW_BYTES, voff, soff);
                }
            }
        };
        constexpr int WAIT_COPIED = ((C::KP_LOADS + C::VP_LOADS) & 15) | (((C::KP_LOADS + C::VP_LOADS) >> 4) << 14) | 0x0F70;
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        int qi = 0, s_in = 0;
        int pos = 0, qb = 0;                     // the score wavefront's position in its block, and that block
        bool stored = false;                     // did the previous step issue output stores? (wavefront-uniform)
        bool copied = false;                     // did the previous step issue the copy of the next block's rows?
        // Step f: accumulate the tile at position f-1 (P^T, H^T, alpha written by the score wavefront during step f-1);
        // if that was the last tile of its query block, normalise the block, send it off and start the next one from zero.
        for (int f = 0; f <= n_flat; ++f) {
            // (after a copy -- issued ahead of that step's fills -- only those fills may still be in flight)
            if (copied) __builtin_amdgcn_s_waitcnt(WAIT_COPIED);
            else if (stored) __builtin_amdgcn_s_waitcnt(WAIT_FILLS_STORES);
            else __builtin_amdgcn_s_waitcnt(WAIT_FILLS);
            stored = false; copied = false;
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (TRICKLE && pos == n - 2 && qb + 1 < nq) { copy_rows(qt0 + qb + 1); copied = true; }
            if (++pos == n) { pos = 0; ++qb; }
            issue_group<C>(make_job(t_k, f + 4, t_v, f + 1));
            if (f > 0) {
                w.step(vring + ((f - 1) % kRingV) * VP_BYTES, smem + ph_base + ((f - 1) & 1) * 4 * C::PH_BYTES,
                       smem + alpha_base + ((f - 1) & 1) * 4 * 256);
                if (++s_in == n) {
                    // O = acc / l ; dO = (T - (r / l) acc) / l   (statistics published by the barrier at the top of this step)
                    const char* st = smem + stat_base + (qi & 1) * 2 * 4 * 256 + 4 * lane;
                    const float inv_l = *reinterpret_cast<const float*>(st);
                    const float r_over_l = *reinterpret_cast<const float*>(st + 1024);
                    const int row0 = (qt0 + qi) * kBlockM + qw * 32;
                    if constexpr (TRICKLE) {
                        // accumulator lane (j, hh) holds channels 32 db + 8 g + 4 hh .. +3 of row j: 8 bytes of 16-byte chunk
                        // 4 db + g, which goes to chunk position (4 db + g) ^ (j mod CPR) of row j of the region
                        // (the row address is made opaque here so that the chunk addresses are computed on the spot, one XOR
                        // each, instead of being kept in registers across the whole stream)
                        unsigned xw = lds0 + xp_base + j * ST::ROW_BYTES + 8 * hh + ((j & (ST::CPR - 1)) << 4);
                        asm volatile("" : "+v"(xw));
#pragma unroll
                        for (int db = 0; db < NDB; ++db) {
#pragma unroll
                            for (int g = 0; g < 4; ++g) {
                                if (32 * db + 8 * g < DV) {
                                    const unsigned a = xw ^ ((4 * db + g) << 4);
                                    V4 ov, tov;
#pragma unroll
                                    for (int r = 0; r < 4; ++r) {
                                        ov[r] = (T)(w.acc[db][4 * g + r] * inv_l);
                                        if (JVP) tov[r] = (T)((w.acct[db][4 * g + r] - r_over_l * w.acc[db][4 * g + r]) * inv_l);
                                    }
                                    asm volatile("ds_write_b64 %0, %1" ::"v"(a), "v"(ov) : "memory");
                                    if (JVP) asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(a), "v"(tov), "n"(32 * ST::ROW_BYTES) : "memory");
                                }
                            }
                        }
                        __builtin_amdgcn_s_waitcnt(0xC07F);   // the region is complete before the next barrier publishes it
                    } else if (row0 < p.Lq) {           // wavefront-uniform: every wavefront that stores issues all N_STORES stores
                        const int row = row0 + j;
                        const int64_t off = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)row * p.o_sl;
                        T* op = reinterpret_cast<T*>(p.o) + off;
                        T* top = reinterpret_cast<T*>(p.to) + off;
                        if (row < p.Lq) {
#pragma unroll
                            for (int db = 0; db < NDB; ++db) {
#pragma unroll
                                for (int g = 0; g < 4; ++g) {
                                    const int d = 32 * db + 8 * g + 4 * hh;   // registers 4g..4g+3 are 4 consecutive d
                                    if (32 * db + 8 * g < DV) {
                                        V4 ov, tov;
#pragma unroll
                                        for (int r = 0; r < 4; ++r) {
                                            ov[r] = (T)(w.acc[db][4 * g + r] * inv_l);
                                            if (JVP) tov[r] = (T)((w.acct[db][4 * g + r] - r_over_l * w.acc[db][4 * g + r]) * inv_l);
                                        }
                                        asm volatile("global_store_dwordx2 %0, %1, off" ::"v"(op + d), "v"(ov) : "memory");
                                        if (JVP) asm volatile("global_store_dwordx2 %0, %1, off" ::"v"(top + d), "v"(tov) : "memory");
                                    }
                                }
                            }
                        }
                        stored = row0 + 32 <= p.Lq;     // all rows live: every store instruction had a live lane
                    }
                    s_in = 0; ++qi;                    // (the next block's first tile arrives with a factor of zero)
                }
            }
            t_v = wrap_inc(t_v); t_k = wrap_inc(t_k);
        }
        if (TRICKLE) __builtin_amdgcn_s_barrier();   // hands the last block to the score wavefronts
        __builtin_amdgcn_s_waitcnt(0x0F70);   // drain the (unused) trailing fills before the LDS is released (or reused by the next stream)
    }
    }   // streams of this workgroup
}

#include "attn_wide_gfx950.h"

// ---------------------------------------------------------------------------------------------------------------
// Forward only.  Without tangents a wavefront's whole state (Q fragments, one 32 x d_v accumulator, two score sets)
// fits the 256 registers that two wavefronts per SIMD leave it, and the softmax VALU work per MFMA is three times
// that of the tangent modes -- too much for one score wavefront per pair.  So all 8 wavefronts do the same thing,
// each for its own 32 query rows (256 per workgroup): score MFMAs of the next 32 keys interleaved with the softmax of
// the current ones, then the P.V MFMAs, with P^T never leaving registers.  The workgroup synchronises (and refills
// the LDS rings) once per 64 keys: a step is two such half steps.
constexpr int kSymWaves = 12;        // wavefronts per workgroup, three per SIMD
constexpr int kSymBlockM = 32 * kSymWaves;     // query rows per workgroup
constexpr int kSymRing = 4;         // LDS ring depth in steps (pairs of packed tiles), K slots and V slots

template <int DQK, int DV>
struct SymCfg {
    static constexpr int NC = DQK / 16, NDB = (DV + 31) / 32;
    static constexpr int K_FR = NC, VT_FR = 2 * NDB;                       // fragments per packed tile
    static constexpr int KP_BYTES = K_FR * kFragBytes, VP_BYTES = VT_FR * kFragBytes, TILE_BYTES = KP_BYTES + VP_BYTES;
    static constexpr int KS_BYTES = 2 * KP_BYTES, VS_BYTES = 2 * VP_BYTES;   // ring slots: the parts of two packed tiles
    static constexpr int K_LOADS = (2 * K_FR + 7) / 8, V_LOADS = (2 * VT_FR + 7) / 8;   // per wavefront per step
    static_assert(K_LOADS <= 2 && V_LOADS <= 2 && (K_LOADS == 1 || K_FR % 2 == 0) && (V_LOADS == 1 || VT_FR % 2 == 0), "runs stay inside a tile");
    static constexpr int GROUP_LOADS = K_LOADS + V_LOADS;
    static constexpr int KRING_OFF = 0, VRING_OFF = kSymRing * KS_BYTES;
    static constexpr int LDS_BYTES = VRING_OFF + kSymRing * VS_BYTES;
};

template <typename T, int DQK, int DV>
struct SymWave {
    typedef SymCfg<DQK, DV> C;
    typedef typename VecOf<T>::v8 V8;
    static constexpr int NC = C::NC, NDB = C::NDB;
    static constexpr int NB = 2 * NDB;      // P.V MFMA groups of a tile, (c, db) at index c * NDB + db
    static constexpr int PD = COSMOS_ATTN_PREFETCH_GROUPS;

    V8 qf[NC];
    f32x16 acc[NDB];
    float m_run, l_run, scale_log2;
    int lane;

    __device__ __forceinline__ V8 lds_frag(const char* base, int frag) const {
        return *reinterpret_cast<const V8*>(base + frag * kFragBytes + lane * 16);
    }
    // this lane's scores of a tile: its query column x 16 of the 32 keys (element e is key 8 (e/4) + 4 (lane/32) + e%4)
    __device__ __forceinline__ static float lane_max(const f32x16& s) {
        float mx = s[0];
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s[e]);
        return mx;
    }
    __device__ __forceinline__ static void mask_scores(f32x16& s, int key0, int kv_len, bool causal, int row) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int key = key0 + 8 * (e >> 2) + (e & 3);
            const bool ok = key < kv_len && (!causal || key <= row);
            s[e] = ok ? s[e] : -INFINITY;
        }
    }
    // fold the lane-local max of a tile's scores into the running max; returns the rescale factor (1 if no row moved)
    __device__ __forceinline__ float update_max(float mx) {
        {   // max with lane ^ 32 (the other half of the same query column)
            float lo, hi;
            both_halves(mx, lo, hi);
            mx = fmaxf(lo, hi);
        }
        const float m_new = fmaxf(m_run, mx * scale_log2);
        float alpha = 1.0f;
        if (__any(m_new > m_run + kMaxSlack)) {
            alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= alpha;
            m_run = m_new;
        }
        return alpha;
    }
    __device__ __forceinline__ void scores_plain(f32x16& x, const char* kpart) const {
#pragma unroll
        for (int e = 0; e < 16; ++e) x[e] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) x = mfma32(lds_frag(kpart, c), qf[c], x);
    }

    // Half a step (32 keys).  Stage A: scores of the next tile (K part `kpart`) into `xn`, interleaved with the softmax
    // of the current one (`x`, already folded into m_run) into the 16-bit operands P^T.  Then rescale by `alpha`
    // (the factor that goes with `x`) if some row's max moved, and stage B: O^T += V^T P^T over the V part `vpart`.
    __device__ __forceinline__ void half_step(const f32x16& x, f32x16& xn, const char* kpart, const char* vpart, float alpha) {
        V8 pf[2];
        constexpr int EPC = 16 / NC;   // softmax elements dealt out per d chunk
        V8 fa[NC];
#pragma unroll
        for (int i = 0; i < PD && i < NC; ++i) fa[i] = lds_frag(kpart, i);
#pragma unroll
        for (int e = 0; e < 16; ++e) xn[e] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            SCHED_FENCE();
            if (c + PD < NC) fa[c + PD] = lds_frag(kpart, c + PD);
            SCHED_FENCE();
            xn = mfma32(fa[c], qf[c], xn);
#pragma unroll
            for (int k = 0; k < EPC; ++k) {
                const int e = c * EPC + k;
                const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], scale_log2, -m_run));
                l_run += p;
                pf[e >> 3][e & 7] = (T)p;
            }
        }
        SCHED_FENCE();
        V8 fv[NB];
#pragma unroll
        for (int i = 0; i < PD && i < NB; ++i) fv[i] = lds_frag(vpart, 2 * (i % NDB) + i / NDB);
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int i = 0; i < NDB; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][e] *= alpha;
            }
        }
#pragma unroll
        for (int g = 0; g < NB; ++g) {
            const int c = g / NDB, db = g % NDB;
            SCHED_FENCE();
            if (g + PD < NB) fv[g + PD] = lds_frag(vpart, 2 * ((g + PD) % NDB) + (g + PD) / NDB);
            SCHED_FENCE();
            acc[db] = mfma32(fv[g], pf[c], acc[db]);
        }
        SCHED_FENCE();
    }
};

template <typename T, int DQK, int DV>
__global__ void __attribute__((amdgpu_flat_work_group_size(64 * kSymWaves, 64 * kSymWaves), amdgpu_waves_per_eu(3, 3)))
attn_fwd_sym_kernel(const AttnParams p) {
    typedef SymCfg<DQK, DV> C;
    typedef SymWave<T, DQK, DV> W;
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr int NC = C::NC, NDB = C::NDB;
    constexpr int TILE_BYTES = C::TILE_BYTES, KS_BYTES = C::KS_BYTES, VS_BYTES = C::VS_BYTES;
    // K(s), V(s): the K parts / V parts of the two packed tiles at sweep position s ("step tile" g = tiles 2g, 2g+1).
    // Step s: half step 0 = scores of tile (s,1) | softmax and P.V of tile (s,0); half step 1 = scores of tile (s+1,0) |
    // softmax and P.V of tile (s,1).  It reads K(s), K(s+1), V(s) and issues the fills of K(s+3), V(s+3) into the slots
    // of K(s-1), V(s-1), dead since the barrier.  At the top of step s the fills issued up to step s-2 must have
    // landed; those of step s-1 may be in flight.
    constexpr int IN_FLIGHT = C::GROUP_LOADS;
    constexpr int WAIT_FILLS = (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14) | 0x0F70;

    // 1-D grid: block id -> (pair, key range); pair = query block + n_qt * (batch * H + head)
    const int bid = blockIdx.x;
    const bool partial = bid >= p.n_full && p.splits > 1;
    const int pair = partial ? p.n_full + (bid - p.n_full) / p.splits : bid;
    const int split = partial ? (bid - p.n_full) % p.splits : 0;
    const int qt = pair % p.n_qt, bh = pair / p.n_qt, b = bh / p.H, h = bh % p.H;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int row0 = qt * kSymBlockM + wave * 32;   // first query row of this wavefront
    const int row = row0 + j;                       // this lane's query row (lanes l and l^32 share it)

    int kv_len = p.Lkv;
    if (p.key_lens) { const int kl = p.key_lens[b]; kv_len = kl < kv_len ? (kl < 0 ? 0 : kl) : kv_len; }
    int n_tiles = (kv_len + kBlockN - 1) / kBlockN;
    if (p.causal) { const int lim = (qt * kSymBlockM + kSymBlockM + kBlockN - 1) / kBlockN; n_tiles = n_tiles < lim ? n_tiles : lim; }
    const int n_steps_all = (n_tiles + 1) / 2;   // (a last step tile that sticks out past n_tiles is masked like any tail)
    // this workgroup's share of the sweep: positions [u_lo, u_lo + n_steps)
    const int u_lo = partial ? (int)((int64_t)split * n_steps_all / p.splits) : 0;
    const int n_steps = partial ? (int)((int64_t)(split + 1) * n_steps_all / p.splits) - u_lo : n_steps_all;

    char* const kring = smem + C::KRING_OFF;
    char* const vring = smem + C::VRING_OFF;
    // reads past the end of the buffer (second tile of a last, odd step) return zeros
    const __amdgpu_buffer_rsrc_t kv_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.kv) + (size_t)bh * p.n_tiles * TILE_BYTES, 0, p.n_tiles * TILE_BYTES, 0x00020000);
    // sweep order (in step tiles): see attn_fwd_jvp_kernel
    const int n_sweep = n_steps_all > 0 ? n_steps_all : 1;
    const int shift = p.causal ? 0 : (((pair >> 3) & 31) * COSMOS_ATTN_SWEEP_STAGGER) % n_sweep;
    auto tile_at = [&](int u) { return __builtin_amdgcn_readfirstlane((u_lo + u + shift) % n_sweep); };
    auto wrap_inc = [&](int t) { ++t; return t >= n_sweep ? t - n_sweep : t; };
    // this wavefront's run of fragments inside a K slot / V slot (never crosses a packed tile)
    const int kf0 = (wave * C::K_LOADS) % (2 * C::K_FR), vf0 = (wave * C::V_LOADS) % (2 * C::VT_FR);
    const int k_src_run = (kf0 / C::K_FR) * TILE_BYTES + (kf0 % C::K_FR) * kFragBytes;
    const int v_src_run = (vf0 / C::VT_FR) * TILE_BYTES + C::KP_BYTES + (vf0 % C::VT_FR) * kFragBytes;
    auto fill = [&](int g, int u) {
        if (wave >= 8) return;   // eight wavefronts cover a slot
        issue_part<C::K_LOADS>(kv_rsrc, kring + (u % kSymRing) * KS_BYTES + kf0 * kFragBytes, lane * 16, g * 2 * TILE_BYTES + k_src_run);
        issue_part<C::V_LOADS>(kv_rsrc, vring + (u % kSymRing) * VS_BYTES + vf0 * kFragBytes, lane * 16, g * 2 * TILE_BYTES + v_src_run);
    };
#pragma unroll
    for (int u = 0; u < 3; ++u) fill(tile_at(u), u);

    W w;
    w.lane = lane;
    w.scale_log2 = p.scale_log2;
    {
        const int64_t off = (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + (int64_t)row * p.q_sl + 8 * hh;
        const T* qp = reinterpret_cast<const T*>(p.q) + off;
        const bool live = row < p.Lq;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            V8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            w.qf[c] = live ? *reinterpret_cast<const V8*>(qp + 16 * c) : z;
        }
    }
#pragma unroll
    for (int i = 0; i < NDB; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) w.acc[i][e] = 0.f;
    }
    w.m_run = -INFINITY;
    w.l_run = 0.f;

    const bool causal = p.causal != 0;
    auto need_mask = [&](int t) { return (t * kBlockN + kBlockN > kv_len) || (causal && (t * kBlockN + kBlockN - 1 > row0)); };
    float alpha = 1.0f;
    // fold the scores of packed tile pt into the running max (masking them first where the tile needs it)
    auto fold = [&](f32x16& x, int pt) {
        if (need_mask(pt)) W::mask_scores(x, pt * kBlockN + 4 * hh, kv_len, causal, row);
        alpha = w.update_max(W::lane_max(x));
    };
    f32x16 sc0, sc1;   // scores of the current / next tile, swapping roles every half step
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): Q and this wavefront's share of the first fills are here
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    w.scores_plain(sc0, kring);
    if (n_steps > 0) fold(sc0, 2 * tile_at(0));
    int g_cur = tile_at(0), g_nxt = tile_at(1), g_fill = tile_at(3);
    for (int s = 0; s < n_steps; ++s) {
        __builtin_amdgcn_s_waitcnt(WAIT_FILLS);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        fill(g_fill, s + 3);
        const char* kslot = kring + (s % kSymRing) * KS_BYTES;
        const char* vslot = vring + (s % kSymRing) * VS_BYTES;
        {
            const float a = alpha;
            w.half_step(sc0, sc1, kslot + C::KP_BYTES, vslot, a);
            fold(sc1, 2 * g_cur + 1);
        }
        {
            const float a = alpha;
            w.half_step(sc1, sc0, kring + ((s + 1) % kSymRing) * KS_BYTES, vslot + C::VP_BYTES, a);
            if (s + 1 < n_steps) fold(sc0, 2 * g_nxt);
        }
        g_cur = g_nxt; g_nxt = wrap_inc(g_nxt); g_fill = wrap_inc(g_fill);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // drain the (unused) trailing fills before the LDS is released

    // ---- epilogue: O = acc / l ; LSE = (m + log2 l) ln 2 ----
    const float l_tot = w.l_run + __shfl_xor(w.l_run, 32);
    if (partial) {
        // a key range only: leave acc, m, l as they are for attn_combine_kernel (rows past Lq are written too and
        // never combined)
        const int64_t slot = (int64_t)(pair - p.n_full) * p.splits + split;
        const int wrow = wave * 32 + j;
        float* pa = p.part_acc + (slot * kSymBlockM + wrow) * DV;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * db + 8 * g + 4 * hh;
                if (d < DV)
                    *reinterpret_cast<float4*>(pa + d) = make_float4(w.acc[db][4 * g], w.acc[db][4 * g + 1], w.acc[db][4 * g + 2], w.acc[db][4 * g + 3]);
            }
        }
        if (hh == 0) p.part_stat[slot * kSymBlockM + wrow] = make_float4(w.m_run, l_tot, 0.f, 0.f);
        return;
    }
    const float inv_l = 1.0f / l_tot;
    if (row < p.Lq) {
        T* op = reinterpret_cast<T*>(p.o) + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)row * p.o_sl;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * db + 8 * g + 4 * hh;   // registers 4g..4g+3 are 4 consecutive d
                if (d < DV) {
                    V4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (T)(w.acc[db][4 * g + r] * inv_l);
                    *reinterpret_cast<V4*>(op + d) = ov;
                }
            }
        }
        if (p.lse && hh == 0) p.lse[(int64_t)bh * p.Lq + row] = (w.m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
    }
}

// Merge the key-range partial results of one query row:  M = max m_i,  w_i = 2^(m_i - M),  L = sum l_i w_i,
// O = sum acc_i w_i / L,  LSE = (M + log2 L) ln 2; with tangents also T = sum accT_i w_i, R = sum r_i w_i and
// dO = (T - (R / L) sum acc_i w_i) / L.  One thread per (row, 4 output channels); fixed order over the ranges.
template <typename T, bool JVP>
__global__ void __launch_bounds__(256) attn_combine_kernel(const AttnParams p, int dv, int block_m) {
    typedef typename VecOf<T>::v4 V4;
    const int tpr = dv / 4;                                   // threads per row
    const int64_t r = (int64_t)blockIdx.x * (256 / tpr) + threadIdx.x / tpr;   // row among the split pairs' rows
    const int c = (threadIdx.x % tpr) * 4;
    const int pair_i = (int)(r / block_m), wrow = (int)(r % block_m);
    const int pair = p.n_full + pair_i;
    const int qt = pair % p.n_qt, bh = pair / p.n_qt, b = bh / p.H, h = bh % p.H;
    const int row = qt * block_m + wrow;
    if (pair_i >= p.n_rem || row >= p.Lq) return;
    const int64_t slot0 = (int64_t)pair_i * p.splits;
    const int acc_w = JVP ? 2 * dv : dv;                      // floats per row in part_acc
    float M = -INFINITY;
    for (int i = 0; i < p.splits; ++i) M = fmaxf(M, p.part_stat[(slot0 + i) * block_m + wrow].x);
    float L = 0.f, R = 0.f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f), t = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int i = 0; i < p.splits; ++i) {
        const float4 st = p.part_stat[(slot0 + i) * block_m + wrow];
        const float wgt = __builtin_amdgcn_exp2f(st.x - M);
        const float* pa = p.part_acc + ((slot0 + i) * block_m + wrow) * acc_w + c;
        const float4 a = *reinterpret_cast<const float4*>(pa);
        L += st.y * wgt;
        o.x += a.x * wgt; o.y += a.y * wgt; o.z += a.z * wgt; o.w += a.w * wgt;
        if (JVP) {
            const float4 at = *reinterpret_cast<const float4*>(pa + dv);
            R += st.z * wgt;
            t.x += at.x * wgt; t.y += at.y * wgt; t.z += at.z * wgt; t.w += at.w * wgt;
        }
    }
    const float inv_l = 1.0f / L;
    const int64_t off = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)row * p.o_sl + c;
    V4 ov;
    ov[0] = (T)(o.x * inv_l); ov[1] = (T)(o.y * inv_l); ov[2] = (T)(o.z * inv_l); ov[3] = (T)(o.w * inv_l);
    *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.o) + off) = ov;
    if (JVP) {
        const float r_over_l = R * inv_l;
        V4 tv;
        tv[0] = (T)((t.x - r_over_l * o.x) * inv_l); tv[1] = (T)((t.y - r_over_l * o.y) * inv_l);
        tv[2] = (T)((t.z - r_over_l * o.z) * inv_l); tv[3] = (T)((t.w - r_over_l * o.w) * inv_l);
        *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.to) + off) = tv;
    }
    if (p.lse && c == 0) p.lse[(int64_t)bh * p.Lq + row] = (M + __builtin_log2f(L)) * 0.6931471805599453f;
}

// ------------------------------------------------------------------------------------------------ host
typedef void (*attn_kernel_t)(const AttnParams);

template <typename T, int DQK, int DV>
attn_kernel_t pick_mode(int mode) {
    switch (mode) {
        case MODE_FWD: return attn_fwd_sym_kernel<T, DQK, DV>;
        case MODE_JVP_Q: return attn_fwd_jvp_kernel<T, DQK, DV, MODE_JVP_Q>;
        default: return attn_fwd_jvp_kernel<T, DQK, DV, MODE_JVP_FULL>;
    }
}
template <typename T, int DQK>
attn_kernel_t pick_dv(int dv, int mode) {
    switch (dv) {
        case 16: return pick_mode<T, DQK, 16>(mode);
        case 32: return pick_mode<T, DQK, 32>(mode);
        case 64: return pick_mode<T, DQK, 64>(mode);
        case 128: return pick_mode<T, DQK, 128>(mode);
        default: return nullptr;
    }
}
template <typename T>
attn_kernel_t pick_dqk(int dqk, int dv, int mode) {
#ifdef COSMOS_ATTN_ONLY_D128   // development builds: instantiate the d=128 kernels only
    return (dqk == 128 && dv == 128) ? pick_mode<T, 128, 128>(mode) : nullptr;
#endif
    switch (dqk) {
        case 16: return pick_dv<T, 16>(dv, mode);
        case 32: return pick_dv<T, 32>(dv, mode);
        case 64: return pick_dv<T, 64>(dv, mode);
        case 128: return pick_dv<T, 128>(dv, mode);
        default: return nullptr;
    }
}


// the query-streaming kernel is built for equal head dims (what cross-attention in the DiT uses)
template <typename T, int D>
attn_kernel_t pick_stream_mode(int mode) {
    switch (mode) {
        case MODE_FWD: return attn_qstream_kernel<T, D, D, MODE_FWD>;
        case MODE_JVP_Q: return attn_qstream_kernel<T, D, D, MODE_JVP_Q>;
        default: return attn_qstream_kernel<T, D, D, MODE_JVP_FULL>;
    }
}
template <typename T>
attn_kernel_t pick_stream(int dqk, int dv, int mode) {
    if (dqk != dv) return nullptr;
    switch (dqk) {
#ifndef COSMOS_ATTN_ONLY_D128
        case 16: return pick_stream_mode<T, 16>(mode);
        case 32: return pick_stream_mode<T, 32>(mode);
        case 64: return pick_stream_mode<T, 64>(mode);
#endif
        case 128: return pick_stream_mode<T, 128>(mode);
        default: return nullptr;
    }
}

int mode_of(const cosmos_attn_desc* d) {
    if (!d->tq && !d->tk && !d->tv) return MODE_FWD;
    if (d->tq && !d->tk && !d->tv) return MODE_JVP_Q;
    if (d->tq && d->tk && d->tv) return MODE_JVP_FULL;
    return -1;
}

size_t tile_bytes_of(const cosmos_attn_desc* d) {
    const TileGeom g(d->d_qk, d->d_v, mode_of(d) == MODE_JVP_FULL);
    return (size_t)g.tile_frags * kFragBytes;
}
// LDS of the attention kernel: K ring, V ring, P^T/H^T hand-over buffers, rescale factors (AttnCfg::LDS_BYTES)
size_t lds_bytes_of(const cosmos_attn_desc* d) {
    const int mode = mode_of(d);
    const TileGeom g(d->d_qk, d->d_v, mode == MODE_JVP_FULL);
    const size_t kp = (size_t)g.kpart_frags * kFragBytes, vp = (size_t)(g.tile_frags - g.kpart_frags) * kFragBytes;
    if (mode == MODE_FWD) return (size_t)kSymRing * 2 * (kp + vp);   // SymCfg::LDS_BYTES
    const size_t ph = 4 * kFragBytes;
    return kRingK * kp + kRingV * vp + 2 * 4 * ph + 2 * 4 * 256;
}
int n_tiles_of(const cosmos_attn_desc* d) { return (d->Lkv + kBlockN - 1) / kBlockN; }
// workspace = packed tiles [B*H][n_tiles][tile bytes]
size_t tiles_bytes_of(const cosmos_attn_desc* d) { return (size_t)d->B * d->H * n_tiles_of(d) * tile_bytes_of(d); }

// How the (query block, head) pairs are dealt out (see choose_splits): the pairs of a partly filled last round of
// workgroups are cut along the keys, and a small second kernel merges the ranges.
// a head dim of 256 goes to attn_wide_kernel
bool is_wide(const cosmos_attn_desc* d) { return d->d_qk == 256 || d->d_v == 256; }
struct SplitPlan { int block_m, n_qt, n_pairs, n_full, n_rem, splits; };
SplitPlan plan_split(const cosmos_attn_desc* d) {
    SplitPlan s;
    const bool fwd = mode_of(d) == MODE_FWD;
    s.block_m = fwd ? kSymBlockM : kBlockM;
    s.n_qt = (d->Lq + s.block_m - 1) / s.block_m;
    s.n_pairs = s.n_qt * d->B * d->H;
    s.n_rem = 0; s.splits = 1; s.n_full = s.n_pairs;
    if (d->causal || d->key_lens || is_wide(d)) return s;          // key ranges of equal work only; not for head dim 256
    const int rem = s.n_pairs % kNumCUs;
    const int n_steps = fwd ? (n_tiles_of(d) + 1) / 2 : n_tiles_of(d);   // barrier steps: 64 keys forward only, 32 with tangents
    const int splits = choose_splits(rem, n_steps);
    if (splits < 2) return s;
    s.n_rem = rem; s.n_full = s.n_pairs - rem; s.splits = splits;
    return s;
}
// Short key sequences go to attn_qstream_kernel: number of workgroups (0 = use the other kernels).  The kernel cuts the
// line of (query block, head) pairs into pieces of equal weight itself, so the launch is a small multiple of the number
// of compute units (every unit gets the same number of equal pieces); it pays from a few blocks per workgroup on.
// cosmos_attn_set_stream_override() replaces the choice (tuning and tests); nothing in the per-call path reads the environment.
constexpr int kStreamMaxTiles = 64;       // up to 2048 keys
constexpr int kStreamGroupsPerCU = 1;       // one workgroup fills a compute unit (8 wavefronts, 2 per SIMD at 256 registers): a single round
constexpr int kStreamMinPairs = 1024;     // four blocks per workgroup: from there on the stream is faster than one workgroup per block (measured)
std::atomic<int> g_stream_chunk{0};       // query blocks per workgroup (1 = never stream), 0 = the library's own choice
std::atomic<int> g_stream_groups{0};      // number of workgroups, 0 = the library's own choice
int stream_groups_of(const cosmos_attn_desc* d) {
    if (d->causal || d->d_qk != d->d_v || n_tiles_of(d) > kStreamMaxTiles) return 0;
    // the kernel addresses q and o inside a head with 32-bit byte offsets
    if ((int64_t)d->Lq * d->q_stride[2] >= ((int64_t)1 << 30) || (int64_t)d->Lq * d->o_stride[2] >= ((int64_t)1 << 30)) return 0;
    const int n_qt = (d->Lq + kBlockM - 1) / kBlockM;
    const int64_t pairs = (int64_t)n_qt * d->B * d->H;
    if (const int chunk = g_stream_chunk.load(std::memory_order_relaxed)) {
        if (chunk < 2 || pairs < 2) return 0;
        const int64_t groups = ((pairs + chunk - 1) / chunk + 7) / 8 * 8;     // a multiple of the number of XCDs
        return groups > (1 << 30) ? 0 : (int)groups;
    }
    if (const int groups = g_stream_groups.load(std::memory_order_relaxed)) return (groups + 7) / 8 * 8;
    return pairs >= kStreamMinPairs ? kNumCUs * kStreamGroupsPerCU : 0;
}
// LDS of attn_qstream_kernel: the layout of attn_fwd_jvp_kernel (AttnCfg::LDS_BYTES) + the per-block statistics slots
size_t stream_lds_bytes_of(const cosmos_attn_desc* d) {
    const int mode = mode_of(d);
    const TileGeom g(d->d_qk, d->d_v, mode == MODE_JVP_FULL);
    const size_t kp = (size_t)g.kpart_frags * kFragBytes, vp = (size_t)(g.tile_frags - g.kpart_frags) * kFragBytes;
    const size_t ph = (mode == MODE_FWD ? 2 : 4) * kFragBytes;
    const int dvp = d->d_v < 32 ? d->d_v : 32 * ((d->d_v + 31) / 32);
    const size_t xp = mode == MODE_JVP_FULL ? 0 : (size_t)4 * (mode == MODE_FWD ? 1 : 2) * 32 * dvp * 2;   // StreamStores::XP_BYTES per wavefront pair
    return kRingK * kp + kRingV * vp + 2 * 4 * ph + 2 * 4 * 256 + 2 * 2 * 4 * 256 + xp;
}
size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
// partial results of the split pairs: fp32 accumulators (O, and T with tangents), then the row statistics
size_t partial_acc_bytes(const cosmos_attn_desc* d, const SplitPlan& s) {
    const size_t per_row = (size_t)d->d_v * (mode_of(d) == MODE_FWD ? 1 : 2) * sizeof(float);
    return align256((size_t)s.n_rem * s.splits * s.block_m * per_row);
}
size_t partial_bytes_of(const cosmos_attn_desc* d) {
    const SplitPlan s = plan_split(d);
    if (s.splits < 2) return 0;
    return partial_acc_bytes(d, s) + align256((size_t)s.n_rem * s.splits * s.block_m * sizeof(float4));
}

int validate(const cosmos_attn_desc* d) {
    if (!d) return COSMOS_ATTN_BAD_ARG;
    if (d->abi_version != COSMOS_ATTN_ABI_VERSION) return COSMOS_ATTN_BAD_ARG;
    if (d->B <= 0 || d->H <= 0 || d->Lq <= 0 || d->Lkv <= 0) return COSMOS_ATTN_BAD_ARG;
    if (!d->q || !d->k || !d->v || !d->o) return COSMOS_ATTN_BAD_ARG;
    const int mode = mode_of(d);
    if (mode < 0) return COSMOS_ATTN_BAD_ARG;          // tangents must be: none, q only, or all three
    if (mode != MODE_FWD && !d->to) return COSMOS_ATTN_BAD_ARG;
    if (d->dtype != COSMOS_ATTN_BF16 && d->dtype != COSMOS_ATTN_FP16) return COSMOS_ATTN_UNSUPPORTED;
    if (!(head_dim_ok(d->d_qk) || d->d_qk == 256) || !(head_dim_ok(d->d_v) || d->d_v == 256)) return COSMOS_ATTN_BAD_SHAPE;
    if (d->causal && d->Lq != d->Lkv) return COSMOS_ATTN_BAD_SHAPE;
    if (d->causal && d->key_lens) return COSMOS_ATTN_BAD_ARG;
    if (!aligned16(d->q) || !aligned16(d->k) || !aligned16(d->v) || !aligned16(d->o)) return COSMOS_ATTN_BAD_STRIDE;
    if ((d->tq && !aligned16(d->tq)) || (d->tk && !aligned16(d->tk)) || (d->tv && !aligned16(d->tv)) ||
        (d->to && !aligned16(d->to)))
        return COSMOS_ATTN_BAD_STRIDE;
    if (!strides_ok(d->q_stride) || !strides_ok(d->k_stride) || !strides_ok(d->v_stride) || !strides_ok(d->o_stride))
        return COSMOS_ATTN_BAD_STRIDE;
    if ((int64_t)d->B * d->H * ((d->Lq + kBlockM - 1) / kBlockM) > ((int64_t)1 << 30)) return COSMOS_ATTN_BAD_SHAPE;   // 1-D grid, 32-bit pair index
    if ((int64_t)n_tiles_of(d) * (int64_t)tile_bytes_of(d) >= (int64_t)1 << 31) return COSMOS_ATTN_BAD_SHAPE;   // 32-bit buffer offsets per head
    return COSMOS_ATTN_OK;
}


}  // namespace

extern "C" {

COSMOS_ATTN_API int cosmos_attn_abi_version(void) { return COSMOS_ATTN_ABI_VERSION; }

COSMOS_ATTN_API const char* cosmos_attn_status_string(int status) {
    switch (status) {
        case COSMOS_ATTN_OK: return "ok";
        case COSMOS_ATTN_BAD_ARG: return "bad argument (null pointer, non-positive size, ABI version, or tangent set other than none / q only / q,k,v)";
        case COSMOS_ATTN_BAD_SHAPE: return "bad shape (head dims must be in {16,32,64,128,256}; causal needs Lq == Lkv)";
        case COSMOS_ATTN_BAD_STRIDE: return "bad stride or alignment (16-byte aligned bases, strides multiple of 8 elements, innermost stride 1)";
        case COSMOS_ATTN_UNSUPPORTED: return "unsupported dtype or head dim (bf16/fp16 only)";
        case COSMOS_ATTN_WORKSPACE_TOO_SMALL: return "workspace too small or null";
        case COSMOS_ATTN_LAUNCH_FAILED: return "kernel launch failed";
        case COSMOS_ATTN_WRONG_DEVICE: return "the current device is not a whole MI355X (gfx950 with 256 compute units in 8 XCDs): the kernels' workgroup-to-XCD maps assume it";
        case COSMOS_ATTN_STATIC_SCRATCH_EXCEEDED: return "problem needs more workspace than the library's static scratch array holds (cosmos_attn_static_scratch_bytes); use cosmos_attn_fwd_jvp with a caller-provided workspace";
        default: return "unknown status";
    }
}

COSMOS_ATTN_API void cosmos_attn_set_stream_override(int blocks_per_workgroup, int workgroups) {
    g_stream_chunk.store(blocks_per_workgroup > 0 ? blocks_per_workgroup : 0, std::memory_order_relaxed);
    g_stream_groups.store(workgroups > 0 ? workgroups : 0, std::memory_order_relaxed);
}

COSMOS_ATTN_API size_t cosmos_attn_workspace_bytes(const cosmos_attn_desc* d) {
    if (validate(d) != COSMOS_ATTN_OK) return 0;
    return align256(tiles_bytes_of(d)) + partial_bytes_of(d);
}

COSMOS_ATTN_API size_t cosmos_attn_packed_bytes(const cosmos_attn_desc* d) {
    if (validate(d) != COSMOS_ATTN_OK) return 0;
    return align256(tiles_bytes_of(d));
}

COSMOS_ATTN_API int cosmos_attn_pack_kv(const cosmos_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    const int st = validate(d);
    if (st != COSMOS_ATTN_OK) return st;
    if (!workspace || workspace_bytes < align256(tiles_bytes_of(d)) || !aligned16(workspace)) return COSMOS_ATTN_WORKSPACE_TOO_SMALL;
    PackParams pp;
    const bool full = mode_of(d) == MODE_JVP_FULL;
    pp.k = (const uint16_t*)d->k; pp.v = (const uint16_t*)d->v;
    pp.tk = full ? (const uint16_t*)d->tk : nullptr; pp.tv = full ? (const uint16_t*)d->tv : nullptr;
    pp.k_sb = d->k_stride[0]; pp.k_sh = d->k_stride[1]; pp.k_sl = d->k_stride[2];
    pp.v_sb = d->v_stride[0]; pp.v_sh = d->v_stride[1]; pp.v_sl = d->v_stride[2];
    pp.out = (uint4*)workspace;
    pp.H = d->H; pp.Lkv = d->Lkv; pp.dqk = d->d_qk; pp.dv = d->d_v; pp.n_tiles = n_tiles_of(d);
    hipLaunchKernelGGL(pack_kv_kernel, dim3((pp.n_tiles + 1) / 2, d->B * d->H), dim3(kPackThreads), 0, (hipStream_t)stream, pp);
    return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
}

}  // extern "C"

namespace {
typedef void (*wide_kernel_t)(const AttnParams, int, int);
template <typename T>
wide_kernel_t pick_wide(int mode) {
    switch (mode) {
        case MODE_FWD: return attn_wide_kernel<T, MODE_FWD>;
        case MODE_JVP_Q: return attn_wide_kernel<T, MODE_JVP_Q>;
        default: return attn_wide_kernel<T, MODE_JVP_FULL>;
    }
}
int run_wide(const cosmos_attn_desc* d, const void* workspace, void* stream) {
    const int mode = mode_of(d);
    AttnParams ap = {};
    ap.q = d->q; ap.tq = d->tq;
    ap.q_sb = d->q_stride[0]; ap.q_sh = d->q_stride[1]; ap.q_sl = d->q_stride[2];
    ap.o = d->o; ap.to = d->to;
    ap.o_sb = d->o_stride[0]; ap.o_sh = d->o_stride[1]; ap.o_sl = d->o_stride[2];
    ap.lse = d->lse;
    ap.kv = (const char*)workspace;
    ap.key_lens = d->key_lens;
    ap.H = d->H; ap.Lq = d->Lq; ap.Lkv = d->Lkv; ap.n_tiles = n_tiles_of(d); ap.causal = d->causal;
    ap.sm_scale = d->sm_scale; ap.scale_log2 = d->sm_scale * 1.4426950408889634f;
    const int64_t blocks = (int64_t)((d->Lq + 31) / 32) * d->B * d->H;
    if (blocks > ((int64_t)1 << 31) - 1) return COSMOS_ATTN_BAD_SHAPE;
    wide_kernel_t fn = d->dtype == COSMOS_ATTN_BF16 ? pick_wide<__bf16>(mode) : pick_wide<_Float16>(mode);
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3(64 * kWideWaves), 0, (hipStream_t)stream, ap, (int)d->d_qk, (int)d->d_v);
    return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
}
// `scratch`: where key-range partial results may go (null: never split).  cosmos_attn_run only reads its workspace, so
// that several runs may share one re-tiled K/V image; the one-call entry point owns the workspace and passes its tail.
int run_impl(const cosmos_attn_desc* d, const void* workspace, size_t workspace_bytes, void* scratch, void* stream) {
    const int st = validate(d);
    if (st != COSMOS_ATTN_OK) return st;
    // the two-stage run never cuts key ranges: it needs the image only
    const size_t need = scratch ? cosmos_attn_workspace_bytes(d) : align256(tiles_bytes_of(d));
    if (!workspace || workspace_bytes < need || !aligned16(workspace)) return COSMOS_ATTN_WORKSPACE_TOO_SMALL;
    if (!device_is_whole_mi355x()) return COSMOS_ATTN_WRONG_DEVICE;
    const int mode = mode_of(d);
    if (is_wide(d)) return run_wide(d, workspace, stream);
    attn_kernel_t fn = d->dtype == COSMOS_ATTN_BF16 ? pick_dqk<__bf16>(d->d_qk, d->d_v, mode)
                                                    : pick_dqk<_Float16>(d->d_qk, d->d_v, mode);
    if (!fn) return COSMOS_ATTN_UNSUPPORTED;
    AttnParams ap;
    ap.q = d->q; ap.tq = d->tq;
    ap.q_sb = d->q_stride[0]; ap.q_sh = d->q_stride[1]; ap.q_sl = d->q_stride[2];
    ap.o = d->o; ap.to = d->to;
    ap.o_sb = d->o_stride[0]; ap.o_sh = d->o_stride[1]; ap.o_sl = d->o_stride[2];
    ap.lse = d->lse;
    ap.kv = (const char*)workspace;
    ap.key_lens = d->key_lens;
    ap.H = d->H; ap.Lq = d->Lq; ap.Lkv = d->Lkv; ap.n_tiles = n_tiles_of(d); ap.causal = d->causal;
    ap.sm_scale = d->sm_scale; ap.scale_log2 = d->sm_scale * 1.4426950408889634f;
    ap.BH = d->B * d->H; ap.q_chunk = 0;
    ap.n_qt = (d->Lq + kBlockM - 1) / kBlockM; ap.n_full = ap.n_rem = 0; ap.splits = 1;
    ap.part_acc = nullptr; ap.part_stat = nullptr;
    if (const int groups = stream_groups_of(d)) {   // short key sequences: `groups` workgroups stream the query blocks
        attn_kernel_t sfn = d->dtype == COSMOS_ATTN_BF16 ? pick_stream<__bf16>(d->d_qk, d->d_v, mode)
                                                         : pick_stream<_Float16>(d->d_qk, d->d_v, mode);
        if (sfn) {
            const size_t slds = stream_lds_bytes_of(d);
            if (!allow_lds((const void*)sfn, slds)) return COSMOS_ATTN_LAUNCH_FAILED;
            const int64_t sblocks = groups;
            hipLaunchKernelGGL(sfn, dim3((unsigned)sblocks), dim3(kAttnThreads), slds, (hipStream_t)stream, ap);
            return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
        }
    }
    const size_t lds = lds_bytes_of(d);
    if (!allow_lds((const void*)fn, lds)) return COSMOS_ATTN_LAUNCH_FAILED;
    SplitPlan sp = plan_split(d);
    if (!scratch) { sp.n_full = sp.n_pairs; sp.n_rem = 0; sp.splits = 1; }
    ap.n_qt = sp.n_qt; ap.n_full = sp.n_full; ap.n_rem = sp.n_rem; ap.splits = sp.splits;
    ap.part_acc = nullptr; ap.part_stat = nullptr;
    if (sp.splits > 1) {
        ap.part_acc = (float*)scratch;
        ap.part_stat = (float4*)((char*)scratch + partial_acc_bytes(d, sp));
    }
    const int64_t blocks = (int64_t)sp.n_full + (int64_t)sp.n_rem * sp.splits;
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3(mode == MODE_FWD ? 64 * kSymWaves : kAttnThreads), lds, (hipStream_t)stream, ap);
    if (hipGetLastError() != hipSuccess) return COSMOS_ATTN_LAUNCH_FAILED;
    if (sp.splits > 1) {
        const int rows_per_block = 256 / (d->d_v / 4);
        const int64_t rows = (int64_t)sp.n_rem * sp.block_m;
        const dim3 cgrid((unsigned)((rows + rows_per_block - 1) / rows_per_block));
        const bool bf16 = d->dtype == COSMOS_ATTN_BF16, jvp = mode != MODE_FWD;
        auto cfn = jvp ? (bf16 ? attn_combine_kernel<__bf16, true> : attn_combine_kernel<_Float16, true>)
                       : (bf16 ? attn_combine_kernel<__bf16, false> : attn_combine_kernel<_Float16, false>);
        hipLaunchKernelGGL(cfn, cgrid, dim3(256), 0, (hipStream_t)stream, ap, d->d_v, sp.block_m);
        if (hipGetLastError() != hipSuccess) return COSMOS_ATTN_LAUNCH_FAILED;
    }
    return COSMOS_ATTN_OK;
}
}  // namespace

extern "C" {

COSMOS_ATTN_API int cosmos_attn_run(const cosmos_attn_desc* d, const void* workspace, size_t workspace_bytes, void* stream) {
    return run_impl(d, workspace, workspace_bytes, nullptr, stream);
}

COSMOS_ATTN_API int cosmos_attn_fwd_jvp(const cosmos_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    const int st = cosmos_attn_pack_kv(d, workspace, workspace_bytes, stream);
    if (st != COSMOS_ATTN_OK) return st;
    void* scratch = partial_bytes_of(d) ? (char*)workspace + align256(tiles_bytes_of(d)) : nullptr;
    return run_impl(d, workspace, workspace_bytes, scratch, stream);
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------------------------
// The same call for callers that cannot allocate (code under graph capture, serving loops, harnesses that forbid it):
// the workspace (re-tiled K/V image + key-range partial results) is a device array that is part of this library's
// code object.  Every GPU the library runs on holds its own copy, at its own address, until the process ends; the array's
// name is only a handle on the host, so its address on the current device is looked up once per device and kept.
namespace {
constexpr size_t kStaticScratchBytes = (size_t)COSMOS_ATTN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};       // device address of `scratch`, per device ordinal (null: not looked up yet)
std::mutex g_scratch_mu;

// device address of the current device's copy of `scratch` (null on failure)
void* static_scratch_ptr() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { (void)hipGetLastError(); return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) { (void)hipGetLastError(); return nullptr; }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" {

COSMOS_ATTN_API size_t cosmos_attn_static_scratch_bytes(void) { return kStaticScratchBytes; }

COSMOS_ATTN_API int cosmos_attn_fwd_jvp_static(const cosmos_attn_desc* d, void* stream) {
    const int st = validate(d);
    if (st != COSMOS_ATTN_OK) return st;
    const size_t need = cosmos_attn_workspace_bytes(d);
    if (need > kStaticScratchBytes) return COSMOS_ATTN_STATIC_SCRATCH_EXCEEDED;
    void* const ws = static_scratch_ptr();
    if (!ws) return COSMOS_ATTN_LAUNCH_FAILED;
    // nothing in the workspace has to start at zero: the re-tiling kernel writes every byte of the image (padding
    // included) and every key range writes its whole slot of partial results before the merge kernel reads it
    return cosmos_attn_fwd_jvp(d, ws, need, stream);
}

}  // extern "C"
