// Flash-attention backward (reverse mode through O) for gfx950 (MI355X, CDNA4): kernels and C ABI.
//
// Given dO and the forward's O and LSE:
//     P  = exp(S s - LSE),  S = Q K^T          D  = rowsum(dO * O)
//     dP = dO V^T                              dS = P * (dP - D)
//     dV = P^T dO         dK = s dS^T Q        dQ = s dS K
// This replaces the flash-attn calls of the reference's `_attention.backward`
// (cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py:505-561): same inputs (q, k, v, o, lse, dout),
// same outputs (dq, dk, dv), gradient through O only, equal head dims required (:507-509).
//
// Kernels with the structure of the forward kernel (wavefronts specialised by role, two per SIMD; operands handed over
// through LDS; stream tiles of 32 rows re-tiled once per call into 1 KB MFMA A-operand fragments and moved L2 -> LDS with
// direct-to-LDS loads):
//   * dK/dV kernel: a workgroup owns 128 keys (K, V rows are the stationary B operands) and streams query tiles:
//       scores  Sq = Q k^T,  dPq = dO v^T  (rows = streamed queries, columns = own keys),
//       U = P, W = dS as 16-bit B operands,   dV^T += dO^T U,   dK^T += Q^T W.
//     LSE and D vary along the streamed rows; they travel with the stream as one extra fragment per tile.
//     Head dim 128: attn_dkdv_quad_kernel (four roles per 64 keys, attn_bwd_quad_gfx950.h), which can also keep every dS tile
//     in memory; other head dims: attn_bwd_kernel<T, D, KIND_DKDV> (score wavefront + output wavefront per 32 keys).
//   * dQ from kept dS (head dim 128, when the workspace budget allows): attn_dq_from_ds_kernel streams the 16-bit dS tiles
//     back once, dQ^T += K^T W with W = dS^T -- five matrix products per call in all, as the reference counts them.
//   * dQ by recomputation (otherwise): attn_bwd_kernel<T, D, KIND_DQ>: a workgroup owns 128 queries (Q, dO rows stationary)
//     and streams key tiles:  S^T = K q^T,  dP^T = V dO^T,   W = dS^T,   dQ^T += K^T W  (P computed a second time: seven products).
// No atomics: results are bitwise reproducible.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include <mutex>
#include <set>
#include <type_traits>
#include <utility>

#include "cosmos_attn_hip.h"

namespace {

#include "attn_common_gfx950.h"

constexpr int kRows = 32;           // rows (queries or keys) per stream tile and per wavefront pair
constexpr int kBlock = 128;         // stationary rows per workgroup (4 wavefront pairs)
constexpr int kBwdThreads = 512;    // 4 score wavefronts + 4 output wavefronts
constexpr int kPackThreads = 256;
constexpr int kRingS = 4;           // LDS ring depth, score-side parts
constexpr int kRingO = 3;           // LDS ring depth, output-side parts
constexpr int kRingStats = 5;       // LDS ring depth, per-row statistics fragments (dK/dV kernel)

enum { KIND_DQ = 0, KIND_DKDV = 1 };

// Geometry of a stream tile (32 rows) and of the LDS, per kernel kind and head dim.
// Stream tile image, in order:  score-side part [A1: NC K-type fragments][A2: NC K-type fragments],
//                               output-side part [C1: 2 NDB V^T-type fragments]([C2: 2 NDB V^T-type fragments]),
//                               (statistics fragment).
//   dQ kernel (key tiles):      A1 = K, A2 = V, C1 = K^T.
//   dK/dV kernel (query tiles): A1 = Q, A2 = dO, C1 = dO^T, C2 = Q^T, statistics = LSE log2(e) and D of the 32 queries.
// Fragment layouts as in the forward kernel:
//   K-type fragment c:          lane l holds X[l%32][16 c + 8 (l/32) .. +7]
//   V^T-type fragment 2 db + c: lane l, slot s holds X[16 c + 8 (s/4) + 4 (l/32) + s%4][32 db + l%32]
//   statistics fragment:        floats [0,32): LSE log2(e) of row 8 (e/4) + 4 hh + e%4 at index 16 hh + e; floats [32,64): D likewise.
template <int D, int KIND>
struct BwdCfg {
    static constexpr int NC = D / 16, NDB = (D + 31) / 32;
    static constexpr bool DKDV = KIND == KIND_DKDV;
    static constexpr int SP_FR = 2 * NC, OP_FR = 2 * NDB * (DKDV ? 2 : 1), ST_FR = DKDV ? 1 : 0;
    static constexpr int SP_BYTES = SP_FR * kFragBytes, OP_BYTES = OP_FR * kFragBytes;
    static constexpr int TILE_BYTES = (SP_FR + OP_FR + ST_FR) * kFragBytes;
    static constexpr int A2_OFF = NC * kFragBytes;          // inside the score-side part
    static constexpr int C2_OFF = 2 * NDB * kFragBytes;     // inside the output-side part
    static constexpr int SP_LOADS = (SP_FR + 3) / 4, OP_LOADS = (OP_FR + 3) / 4;   // per output wavefront per tile
    static constexpr int GROUP_LOADS = SP_LOADS + OP_LOADS + ST_FR;
    static constexpr int PH_FR = DKDV ? 4 : 2;              // hand-over fragments per wavefront pair per stage
    static constexpr int PH_BYTES = PH_FR * kFragBytes;
    static constexpr int SRING_OFF = 0;
    static constexpr int ORING_OFF = kRingS * SP_BYTES;
    static constexpr int PH_OFF = ORING_OFF + kRingO * OP_BYTES;
    static constexpr int ST_OFF = PH_OFF + 2 * 4 * PH_BYTES;
    static constexpr int LDS_BYTES = ST_OFF + (DKDV ? kRingStats * kFragBytes : 0);
};

// ---------------------------------------------------------------------------------------------- per-row statistics
struct StatsParams {
    const uint16_t *o, *dout;
    int64_t o_sb, o_sh, o_sl, g_sb, g_sh, g_sl;
    const float* lse;      // [B,H,Lq]
    float2* stats;         // [B*H][Lq] : (LSE log2 e, D)
    int H, Lq, d, bf16;
};

__device__ __forceinline__ float half_bits_to_float(uint16_t h, int bf16) {
    if (bf16) return __builtin_bit_cast(float, (uint32_t)h << 16);
    return (float)__builtin_bit_cast(_Float16, h);
}

// D[row] = sum_d dO[row][d] O[row][d] in fp32 (8 lanes per row, 16-byte loads), LSE rescaled to base 2
__global__ void __launch_bounds__(kPackThreads) bwd_stats_kernel(const StatsParams p) {
    const int bh = blockIdx.y, b = bh / p.H, h = bh % p.H;
    const int row = blockIdx.x * (kPackThreads / 8) + threadIdx.x / 8, part = threadIdx.x % 8;
    float acc = 0.f;
    if (row < p.Lq) {
        const uint16_t* op = p.o + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)row * p.o_sl;
        const uint16_t* gp = p.dout + (int64_t)b * p.g_sb + (int64_t)h * p.g_sh + (int64_t)row * p.g_sl;
        for (int c = part * 8; c < p.d; c += 64) {
            const uint4 ov = *reinterpret_cast<const uint4*>(op + c), gv = *reinterpret_cast<const uint4*>(gp + c);
            const uint32_t ow[4] = {ov.x, ov.y, ov.z, ov.w}, gw[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc += half_bits_to_float((uint16_t)(ow[i] & 0xFFFF), p.bf16) * half_bits_to_float((uint16_t)(gw[i] & 0xFFFF), p.bf16);
                acc += half_bits_to_float((uint16_t)(ow[i] >> 16), p.bf16) * half_bits_to_float((uint16_t)(gw[i] >> 16), p.bf16);
            }
        }
    }
    acc += __shfl_xor(acc, 1); acc += __shfl_xor(acc, 2); acc += __shfl_xor(acc, 4);
    if (row < p.Lq && part == 0)
        p.stats[(int64_t)bh * p.Lq + row] = make_float2(p.lse[(int64_t)bh * p.Lq + row] * 1.4426950408889634f, acc);
}

// ---------------------------------------------------------------------------------------------- stream re-tiling
// Order of the 16-byte units (row q of the tile, 16-channel chunk cK, half hK: 8 channels) inside a K-type section of the
// query stream of attn_dkdv_quad_kernel, which reads the same units linearly (ds_read_b128, lane = row) and transposed
// (ds_read_b64_tr_b16): both without bank conflicts in this order (attn_bwd_quad_gfx950.h).
__host__ __device__ constexpr int quad_unit_slot(int q, int cK, int hK) {
    return 16 * ((q >> 4) + 2 * hK + 4 * cK) + ((q & 3) + 4 * (((q >> 2) & 3) ^ (hK + 2 * (cK & 1))));
}

struct PackSrc { const uint16_t* ptr; int64_t sb, sh, sl; };
struct PackBwdParams {
    PackSrc a1, a2, c1, c2;      // the K-type sections and the V^T-type sections (n_vt of them: 0, 1 or 2)
    const float2* stats;         // null: no statistics fragment
    uint4* out;
    int H, L, d, n_tiles, nc, ndb, tile_frags;
    int n_vt;                    // number of V^T-type sections
    int swz;                     // K-type sections in the unit order of attn_dkdv_quad_kernel (quad_unit_slot) instead of fragment by fragment
};

// grid (n_tiles, B*H); every 16-byte unit of a tile image is produced by one thread.
__global__ void __launch_bounds__(kPackThreads) pack_stream_kernel(const PackBwdParams p) {
    const int bh = blockIdx.y, b = bh / p.H, h = bh % p.H, t = blockIdx.x;
    uint4* dst = p.out + ((size_t)bh * p.n_tiles + t) * (size_t)(p.tile_frags * (kFragBytes / 16));
    const int ktype_frags = 2 * p.nc, vt_frags = 2 * p.ndb;
    const int units = p.tile_frags * 64;
    for (int u = threadIdx.x; u < units; u += kPackThreads) {
        int frag = u >> 6;
        const int l = u & 63, i = l & 31, hh = l >> 5;
        uint4 val = make_uint4(0u, 0u, 0u, 0u);
        int where = u;           // 16-byte unit of the tile image this value goes to
        if (frag < ktype_frags) {
            const int sec = frag < p.nc ? 0 : 1;
            const PackSrc& s = sec ? p.a2 : p.a1;
            frag -= sec * p.nc;
            const int row = t * kRows + i;
            if (row < p.L)
                val = *reinterpret_cast<const uint4*>(s.ptr + (int64_t)b * s.sb + (int64_t)h * s.sh + (int64_t)row * s.sl + 16 * frag + 8 * hh);
            if (p.swz) where = sec * p.nc * 64 + quad_unit_slot(i, frag, hh);
        } else if (frag < ktype_frags + vt_frags * p.n_vt) {
            frag -= ktype_frags;
            const PackSrc& s = frag < vt_frags ? p.c1 : p.c2;
            if (frag >= vt_frags) frag -= vt_frags;
            const int db = frag >> 1, c = frag & 1;
            const int d = 32 * db + i;
            const uint16_t* base = s.ptr + (int64_t)b * s.sb + (int64_t)h * s.sh;
            uint16_t e[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int row = t * kRows + 16 * c + 8 * (k >> 2) + 4 * hh + (k & 3);
                e[k] = (row < p.L && d < p.d) ? base[(int64_t)row * s.sl + d] : (uint16_t)0;
            }
            val.x = e[0] | ((uint32_t)e[1] << 16); val.y = e[2] | ((uint32_t)e[3] << 16);
            val.z = e[4] | ((uint32_t)e[5] << 16); val.w = e[6] | ((uint32_t)e[7] << 16);
        } else if (l < 16) {
            // statistics fragment: lanes 0..7 hold the 32 LSE values, lanes 8..15 the 32 D values; rows past the
            // end get LSE = +inf (so P = 0) and D = 0
            float f[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int idx = 4 * (l & 7) + k, shh = idx >> 4, e = idx & 15;
                const int row = t * kRows + 8 * (e >> 2) + 4 * shh + (e & 3);
                const bool live = row < p.L;
                const float2 st = live ? p.stats[(int64_t)bh * p.L + row] : make_float2(INFINITY, 0.f);
                f[k] = l < 8 ? st.x : st.y;
            }
            val = make_uint4(__builtin_bit_cast(uint32_t, f[0]), __builtin_bit_cast(uint32_t, f[1]),
                             __builtin_bit_cast(uint32_t, f[2]), __builtin_bit_cast(uint32_t, f[3]));
        }
        dst[where] = val;
    }
}

// ---------------------------------------------------------------------------------------------- main kernels
struct BwdParams {
    const void *st1, *st2;             // stationary operands: rows of (q, dout) for dQ, of (k, v) for dK/dV
    int64_t s1_sb, s1_sh, s1_sl, s2_sb, s2_sh, s2_sl;
    void *out1, *out2;                 // dq | dv, dk
    int64_t o1_sb, o1_sh, o1_sl, o2_sb, o2_sh, o2_sl;
    const float2* stats;               // [B*H][Lq]
    const char* stream;                // packed stream tiles [B*H][n_tiles][tile bytes]
    int H, L_stat, L_stream, n_tiles, causal;
    float sm_scale, scale_log2;
    // 1-D grid: workgroups [0, n_full) each own a (block of 128 stationary rows, head) pair; the remaining n_rem pairs
    // are cut into `splits` ranges of the stream, one workgroup each, which leave fp32 partial sums for bwd_combine_kernel
    int n_blk, n_full, n_rem, splits;
    float* part;                       // [(pair - n_full) * splits + split][kBlock][D] (dQ) or [..][kBlock][2][D] (dV, dK)
    // A launch serves the heads [bh0, bh0 + pairs / n_blk) of the call (one group of heads at a time when dS is kept).
    int bh0;
    // dK/dV kernel that keeps dS: every 32 x 32 tile of dS = P * (dP - D) it forms is also written, as the two 1 KB operand
    // fragments the score wavefront hands over, to ds[local head][query tile][key tile] (2 KB each) for attn_dq_from_ds_kernel
    char* ds;
    int64_t ds_head_bytes;             // n_q_tiles * n_kt_pad * 2048
    int n_kt_pad;                      // key tiles per query tile in `ds`: 4 * number of 128-key blocks
};

extern __shared__ __attribute__((aligned(1024))) char smem[];

constexpr int kBwdSweepStagger = 2;   // tiles between the sweep starts of workgroups that share an L2 (3 as in the forward kernels: dQ kernel 1 % slower, 25 % more traffic)

template <typename T, int D, int KIND>
struct BwdScoreWave {
    typedef BwdCfg<D, KIND> C;
    typedef typename VecOf<T>::v8 V8;
    static constexpr int NC = C::NC;
    static constexpr bool DKDV = C::DKDV;
    static constexpr int PD = COSMOS_ATTN_PREFETCH_GROUPS;

    // this lane's share of a 32 x 32 score tile: its stationary row (column of the transposed tile) x 16 of the 32
    // streamed rows (element e is streamed row 8 (e/4) + 4 (lane/32) + e%4)
    struct Scores { f32x16 s, dp; };

    V8 b1[NC], b2[NC];      // stationary B operands: (q, dO) rows or (k, v) rows
    float l2, dd;           // dQ kernel: LSE log2(e) and D of this lane's query
    float scale_log2;
    int lane;

    __device__ __forceinline__ V8 lds_frag(const char* base, int frag) const {
        return *reinterpret_cast<const V8*>(base + frag * kFragBytes + lane * 16);
    }

    // P = exp2(S c - LSE'),  dS = P (dP - D) for element e; rounded to 16-bit MFMA B operands
    __device__ __forceinline__ void elem(const Scores& x, const float* l2v, const float* ddv, V8* uf, V8* wf, int e) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(x.s[e], scale_log2, -(DKDV ? l2v[e] : l2)));
        const float w = p * (x.dp[e] - (DKDV ? ddv[e] : dd));
        if (DKDV) uf[e >> 3][e & 7] = (T)p;
        wf[e >> 3][e & 7] = (T)w;
    }

    // One step: elementwise work on the tile whose scores are in `x` (statistics fragment `stats` in the dK/dV
    // kernel) interleaved with the score MFMAs of the next tile (score-side part `spart`) into `xn`.
    __device__ __forceinline__ void step(const Scores& x, Scores& xn, const char* spart, const char* stats, unsigned ph_out) {
        V8 uf[2], wf[2];
        V8 fa[NC], fb[NC];
        float l2v[16], ddv[16];
#pragma unroll
        for (int i = 0; i < PD && i < NC; ++i) { fa[i] = lds_frag(spart, i); fb[i] = lds_frag(spart + C::A2_OFF, i); }
        if (DKDV) {
            const int hh = lane >> 5;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 a = *reinterpret_cast<const float4*>(stats + 64 * hh + 16 * i);
                const float4 b = *reinterpret_cast<const float4*>(stats + 128 + 64 * hh + 16 * i);
                l2v[4 * i] = a.x; l2v[4 * i + 1] = a.y; l2v[4 * i + 2] = a.z; l2v[4 * i + 3] = a.w;
                ddv[4 * i] = b.x; ddv[4 * i + 1] = b.y; ddv[4 * i + 2] = b.z; ddv[4 * i + 3] = b.w;
            }
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) { xn.s[e] = 0.f; xn.dp[e] = 0.f; }
        constexpr int EPC = 16 / NC;   // elements dealt out per chunk (NC <= 8), half behind each of its two MFMAs
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            SCHED_FENCE();
            if (c + PD < NC) { fa[c + PD] = lds_frag(spart, c + PD); fb[c + PD] = lds_frag(spart + C::A2_OFF, c + PD); }
            SCHED_FENCE();
            xn.s = mfma32(fa[c], b1[c], xn.s);
#pragma unroll
            for (int k = 0; k < EPC; ++k)
                if (k * 2 / EPC == 0) elem(x, l2v, ddv, uf, wf, c * EPC + k);
            SCHED_FENCE();
            xn.dp = mfma32(fb[c], b2[c], xn.dp);
#pragma unroll
            for (int k = 0; k < EPC; ++k)
                if (k * 2 / EPC == 1) elem(x, l2v, ddv, uf, wf, c * EPC + k);
            SCHED_FENCE();
        }
        // hand-over (asm stores: a visible LDS store would make the compiler wait for vmcnt(0), i.e. for the
        // direct-to-LDS fills in flight)
        const unsigned pa = ph_out + 16 * lane;
        if (DKDV) {
            asm volatile("ds_write_b128 %0, %1" ::"v"(pa), "v"(uf[0]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:1024" ::"v"(pa), "v"(uf[1]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:2048" ::"v"(pa), "v"(wf[0]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:3072" ::"v"(pa), "v"(wf[1]) : "memory");
        } else {
            asm volatile("ds_write_b128 %0, %1" ::"v"(pa), "v"(wf[0]) : "memory");
            asm volatile("ds_write_b128 %0, %1 offset:1024" ::"v"(pa), "v"(wf[1]) : "memory");
        }
    }

    // scores of the first tile (prologue)
    __device__ __forceinline__ void scores_plain(Scores& x, const char* spart) const {
#pragma unroll
        for (int e = 0; e < 16; ++e) { x.s[e] = 0.f; x.dp[e] = 0.f; }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            x.s = mfma32(lds_frag(spart, c), b1[c], x.s);
            x.dp = mfma32(lds_frag(spart + C::A2_OFF, c), b2[c], x.dp);
        }
    }
};

template <typename T, int D, int KIND>
struct BwdOutputWave {
    typedef BwdCfg<D, KIND> C;
    typedef typename VecOf<T>::v8 V8;
    static constexpr int NDB = C::NDB;
    static constexpr bool DKDV = C::DKDV;
    static constexpr int NB = 2 * NDB;      // MFMA groups of a step, g = c * NDB + db
    static constexpr int PD = COSMOS_ATTN_PREFETCH_GROUPS;

    f32x16 acc1[NDB], acc2[NDB];   // dQ^T | dV^T, dK^T
    int lane;

    __device__ __forceinline__ V8 lds_frag(const char* base, int frag) const {
        return *reinterpret_cast<const V8*>(base + frag * kFragBytes + lane * 16);
    }
    __device__ __forceinline__ void fetch_group(int g, const char* opart, V8& a, V8& b) const {
        const int c = g / NDB, db = g % NDB;
        a = lds_frag(opart, 2 * db + c);
        if (DKDV) b = lds_frag(opart + C::C2_OFF, 2 * db + c);
    }

    // dQ^T += K^T W       |       dV^T += dO^T U ;  dK^T += Q^T W
    template <typename Fill>
    __device__ __forceinline__ void step(const char* opart, const char* ph_in, Fill&& fill) {
        V8 uf[2], wf[2];
        if (DKDV) { uf[0] = lds_frag(ph_in, 0); uf[1] = lds_frag(ph_in, 1); wf[0] = lds_frag(ph_in, 2); wf[1] = lds_frag(ph_in, 3); }
        else { wf[0] = lds_frag(ph_in, 0); wf[1] = lds_frag(ph_in, 1); }
        V8 fa[NB], fb[NB];
#pragma unroll
        for (int i = 0; i < PD && i < NB; ++i) fetch_group(i, opart, fa[i], fb[i]);
        SCHED_FENCE();
        fill();
        SCHED_FENCE();
#pragma unroll
        for (int g = 0; g < NB; ++g) {
            const int c = g / NDB, db = g % NDB;
            SCHED_FENCE();
            if (g + PD < NB) fetch_group(g + PD, opart, fa[g + PD], fb[g + PD]);
            SCHED_FENCE();
            if (DKDV) {
                acc1[db] = mfma32(fa[g], uf[c], acc1[db]);
                acc2[db] = mfma32(fb[g], wf[c], acc2[db]);
            } else {
                acc1[db] = mfma32(fa[g], wf[c], acc1[db]);
            }
        }
        SCHED_FENCE();
    }
};

template <typename T, int D, int KIND>
__global__ void __attribute__((amdgpu_flat_work_group_size(kBwdThreads, kBwdThreads), amdgpu_waves_per_eu(2, 2)))
attn_bwd_kernel(const BwdParams p) {
    typedef BwdCfg<D, KIND> C;
    typedef BwdScoreWave<T, D, KIND> SW;
    typedef BwdOutputWave<T, D, KIND> OW;
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr int NC = C::NC, NDB = C::NDB;
    constexpr bool DKDV = C::DKDV;
    constexpr int SP_BYTES = C::SP_BYTES, OP_BYTES = C::OP_BYTES, TILE_BYTES = C::TILE_BYTES;
    // s_waitcnt immediate: vmcnt(n), expcnt / lgkmcnt left at their maxima.  At the top of step s the fills of the
    // output-side part of tile s-1 and the score-side part (and statistics) of tile s+1 must have landed; issued
    // after them and still allowed in flight: S(s+2), then the whole groups of steps s-1 ... wait for the rest.
    constexpr int IN_FLIGHT = 2 * (C::SP_LOADS + C::ST_FR) + C::OP_LOADS;
    constexpr int WAIT_FILLS = (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14) | 0x0F70;

    const int bid = blockIdx.x;
    const bool partial = bid >= p.n_full && p.splits > 1;
    const int pair = partial ? p.n_full + (bid - p.n_full) / p.splits : bid;
    const int split = partial ? (bid - p.n_full) % p.splits : 0;
    const int blk = pair % p.n_blk, bhl = pair / p.n_blk, bh = p.bh0 + bhl, b = bh / p.H, h = bh % p.H;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool score_role = wave < 4;            // wavefronts w and w + 4 (same SIMD) serve stationary rows 32 w .. 32 w + 31
    const int qw = wave & 3;
    const int j = lane & 31, hh = lane >> 5;
    const int row0 = blk * kBlock + qw * kRows;  // first stationary row of this wavefront pair
    const int row = row0 + j;                    // this lane's stationary row (lanes l and l^32 share it)

    // Stream tiles this workgroup must visit.  Causal (key j visible to query i iff j <= i, equal lengths):
    //   dQ kernel (stream = keys):     tiles [0, ceil((last query of the block + 1) / 32))
    //   dK/dV kernel (stream = queries): tiles [first key of the block / 32, n)
    int t_lo = 0, t_hi = p.n_tiles;
    if (p.causal) {
        if (DKDV) t_lo = (blk * kBlock) / kRows;
        else { const int lim = (blk * kBlock + kBlock + kRows - 1) / kRows; t_hi = t_hi < lim ? t_hi : lim; }
    }
    if (partial) {   // this workgroup's range of the stream (never with causal masking)
        const int n = p.n_tiles;
        t_lo = (int)((int64_t)split * n / p.splits);
        t_hi = (int)((int64_t)(split + 1) * n / p.splits);
    }
    const int n_steps = t_hi > t_lo ? t_hi - t_lo : 0;

    char* const sring = smem + C::SRING_OFF;
    char* const oring = smem + C::ORING_OFF;
    char* const string = smem + C::ST_OFF;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.stream) + (size_t)bh * p.n_tiles * TILE_BYTES, 0, p.n_tiles * TILE_BYTES, 0x00020000);
    // Sweep order: accumulation is order-free, so workgroups that share an XCD's L2 start a few tiles apart and wrap
    // around (a fixed function of the workgroup id: results stay bitwise reproducible).
    const int n_sweep = n_steps > 0 ? n_steps : 1;
    const int shift = (((pair >> 3) & 31) * kBwdSweepStagger) % n_sweep;
    auto tile_at = [&](int u) { return __builtin_amdgcn_readfirstlane(t_lo + (u + shift) % n_sweep); };
    auto wrap_inc = [&](int t) { ++t; return t >= t_lo + n_sweep ? t - n_sweep : t; };
    const int s_run = ((qw * C::SP_LOADS) % C::SP_FR) * kFragBytes, o_run = ((qw * C::OP_LOADS) % C::OP_FR) * kFragBytes;
    // fill of the score-side part (and statistics) of tile ts into ring position su, of the output-side part of tile to into ou
    auto fill_s = [&](int ts, int su) {
        issue_part<C::SP_LOADS>(rsrc, sring + (su % kRingS) * SP_BYTES + s_run, lane * 16, ts * TILE_BYTES + s_run);
        if (DKDV) lds_load<0>(rsrc, string + (su % kRingStats) * kFragBytes, lane * 16, ts * TILE_BYTES + SP_BYTES + OP_BYTES);
    };
    auto fill_o = [&](int to, int ou) {
        issue_part<C::OP_LOADS>(rsrc, oring + (ou % kRingO) * OP_BYTES + o_run, lane * 16, to * TILE_BYTES + SP_BYTES + o_run);
    };
    // Fill stream, in issue order:  S(0) S(1) S(2) [O(0) S(3)] | step 0: [O(1) S(4)] | step 1: [O(2) S(5)] | ...
    if (!score_role) {
#pragma unroll
        for (int u = 0; u < 3; ++u) fill_s(tile_at(u), u);
        fill_o(tile_at(0), 0);
        fill_s(tile_at(3), 3);
    }

    const bool causal = p.causal != 0;
    // wavefront-uniform: does stream tile t hold an element some lane of this wavefront must mask (causal diagonal)?
    //   dQ:    key (streamed) > query (stationary)   possible iff last key of tile > first query of the pair
    //   dK/dV: key (stationary) > query (streamed)   possible iff last key of the pair > first query of the tile
    // The dQ kernel also masks the streamed keys past the end (their K rows are zero, so P would be exp(-LSE), and
    // an overflowing P times a zero K^T entry is NaN).  Streamed queries past the end need no mask: LSE = +inf.
    auto need_mask = [&](int t) {
        if (!DKDV && t * kRows + kRows > p.L_stream) return true;
        if (!causal) return false;
        return DKDV ? (row0 + kRows - 1 > t * kRows) : (t * kRows + kRows - 1 > row0);
    };
    const unsigned ph_base = C::PH_OFF + qw * C::PH_BYTES;
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;   // LDS address of smem[0], for asm stores
    int t_o = tile_at(1), t_s = tile_at(4);

    if (score_role) {
        SW w;
        w.lane = lane;
        w.scale_log2 = p.scale_log2;
        {   // stationary rows as MFMA B operands: lane holds X[row][16 c + 8 hh .. +7]
            const T* p1 = reinterpret_cast<const T*>(p.st1) + (int64_t)b * p.s1_sb + (int64_t)h * p.s1_sh + (int64_t)row * p.s1_sl + 8 * hh;
            const T* p2 = reinterpret_cast<const T*>(p.st2) + (int64_t)b * p.s2_sb + (int64_t)h * p.s2_sh + (int64_t)row * p.s2_sl + 8 * hh;
            const bool live = row < p.L_stat;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                V8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                w.b1[c] = live ? *reinterpret_cast<const V8*>(p1 + 16 * c) : z;
                w.b2[c] = live ? *reinterpret_cast<const V8*>(p2 + 16 * c) : z;
            }
            w.l2 = INFINITY; w.dd = 0.f;   // rows past the end: P = 0
            if (!DKDV && live) { const float2 st = p.stats[(int64_t)bh * p.L_stat + row]; w.l2 = st.x; w.dd = st.y; }
        }
        // masked elements get score -inf, hence P = 0 and dS = 0
        auto mask = [&](typename SW::Scores& x, int t) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int srow = t * kRows + 8 * (e >> 2) + 4 * hh + (e & 3);   // streamed row of element e
                const bool ok = DKDV ? (!causal || row <= srow) : (srow < p.L_stream && (!causal || srow <= row));   // key <= query
                x.s[e] = ok ? x.s[e] : -INFINITY;
            }
        };
        typename SW::Scores sc0, sc1;   // scores of the current / next tile, swapping roles every step
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the stationary rows are here
        __builtin_amdgcn_s_barrier();         // ... and so is the first stream tile
        asm volatile("" ::: "memory");
        w.scores_plain(sc0, sring);
        if (n_steps > 0 && need_mask(tile_at(0))) mask(sc0, tile_at(0));
        auto body = [&](int s, typename SW::Scores& cur, typename SW::Scores& nxt) {
            __builtin_amdgcn_s_waitcnt(0xC07F);   // own hand-over stores of step s-1 done (lgkmcnt(0))
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (s < n_steps) {
                w.step(cur, nxt, sring + ((s + 1) % kRingS) * SP_BYTES, string + (s % kRingStats) * kFragBytes,
                       lds0 + ph_base + (s & 1) * 4 * C::PH_BYTES);
                if (s + 1 < n_steps && need_mask(t_o)) mask(nxt, t_o);
            }
            t_o = wrap_inc(t_o);   // tile at sweep position s + 2
        };
        for (int s = 0; s <= n_steps; s += 2) {
            body(s, sc0, sc1);
            if (s + 1 <= n_steps) body(s + 1, sc1, sc0);
        }
        __builtin_amdgcn_s_waitcnt(0x0070);
    } else {
        OW w;
        w.lane = lane;
#pragma unroll
        for (int i = 0; i < NDB; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) { w.acc1[i][e] = 0.f; w.acc2[i][e] = 0.f; }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // Step s: accumulate tile s-1 (operands handed over by the score wavefront during step s-1).
        for (int s = 0; s <= n_steps; ++s) {
            __builtin_amdgcn_s_waitcnt(WAIT_FILLS);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // O(s+1) overwrites O(s-2), S(s+4) overwrites S(s), statistics(s+4) overwrite statistics(s-1): all dead
            auto fill = [&]() { fill_o(t_o, s + 1); fill_s(t_s, s + 4); };
            if (s > 0)
                w.step(oring + ((s - 1) % kRingO) * OP_BYTES, smem + ph_base + ((s - 1) & 1) * 4 * C::PH_BYTES, fill);
            else
                fill();
            t_o = wrap_inc(t_o); t_s = wrap_inc(t_s);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // drain the (unused) trailing fills before the LDS is released
        // ---- epilogue: dQ = s dQ^T   |   dV = dV^T, dK = s dK^T ----
        if (partial) {   // a range of the stream only: leave the sums for bwd_combine_kernel
            const int64_t slot = (int64_t)(pair - p.n_full) * p.splits + split;
            float* pa = p.part + (slot * kBlock + qw * kRows + j) * (DKDV ? 2 * D : D);
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d = 32 * db + 8 * g + 4 * hh;
                    if (d < D) {
                        *reinterpret_cast<float4*>(pa + d) = make_float4(w.acc1[db][4 * g], w.acc1[db][4 * g + 1], w.acc1[db][4 * g + 2], w.acc1[db][4 * g + 3]);
                        if (DKDV) *reinterpret_cast<float4*>(pa + D + d) = make_float4(w.acc2[db][4 * g], w.acc2[db][4 * g + 1], w.acc2[db][4 * g + 2], w.acc2[db][4 * g + 3]);
                    }
                }
            }
        } else if (row < p.L_stat) {
            T* o1 = reinterpret_cast<T*>(p.out1) + (int64_t)b * p.o1_sb + (int64_t)h * p.o1_sh + (int64_t)row * p.o1_sl;
            T* o2 = DKDV ? reinterpret_cast<T*>(p.out2) + (int64_t)b * p.o2_sb + (int64_t)h * p.o2_sh + (int64_t)row * p.o2_sl : nullptr;
            const float s1 = DKDV ? 1.0f : p.sm_scale;
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d = 32 * db + 8 * g + 4 * hh;   // registers 4g..4g+3 are 4 consecutive d
                    if (d < D) {
                        V4 v1, v2;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            v1[r] = (T)(w.acc1[db][4 * g + r] * s1);
                            if (DKDV) v2[r] = (T)(w.acc2[db][4 * g + r] * p.sm_scale);
                        }
                        *reinterpret_cast<V4*>(o1 + d) = v1;
                        if (DKDV) *reinterpret_cast<V4*>(o2 + d) = v2;
                    }
                }
            }
        }
    }
}

#include "attn_bwd_quad_gfx950.h"

// ---------------------------------------------------------------------------------------------- head dim 256
// At d = 256 the stationary rows of a wavefront are 128 registers and its accumulators up to 256, and a stream tile is
// 49 / 97 KB: the kernels above do not fit.  This one is built for being right rather than fast (no Cosmos configuration
// has this head dim): no LDS, no roles, no barriers.  A workgroup is four wavefronts that serve the SAME 32 stationary
// rows; each computes the whole 32 x 32 tile of scores and dP for itself (A fragments read straight from the re-tiled
// stream in memory), forms U = P and W = dS, and accumulates its own quarter of the channels (32-channel blocks w and
// w + 4).  Same arithmetic and rounding points as attn_bwd_kernel; the head dim is a run-time value.
constexpr int kWideMaxNC = 16;
constexpr int kWideWaves = 4;
constexpr int kWideDbPerWave = 2;

template <typename T, int KIND>
__global__ void __launch_bounds__(64 * kWideWaves) attn_bwd_wide_kernel(const BwdParams p, int d) {
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr bool DKDV = KIND == KIND_DKDV;
    const int nc = d / 16, ndb = (d + 31) / 32;
    const int sp_frags = 2 * nc, op_frags = 2 * ndb * (DKDV ? 2 : 1);
    const int tile_bytes = (sp_frags + op_frags + (DKDV ? 1 : 0)) * kFragBytes;

    const int pair = blockIdx.x;
    const int blk = pair % p.n_blk, bh = pair / p.n_blk, b = bh / p.H, h = bh % p.H;   // n_blk: blocks of 32 stationary rows
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int row0 = blk * kRows, row = row0 + j;
    const bool causal = p.causal != 0;

    int t_lo = 0, t_hi = p.n_tiles;
    if (causal) {
        if (DKDV) t_lo = row0 / kRows;
        else { const int lim = (row0 + kRows + kRows - 1) / kRows; t_hi = t_hi < lim ? t_hi : lim; }
    }
    V8 b1[kWideMaxNC], b2[kWideMaxNC];   // stationary B operands: (q, dO) rows or (k, v) rows
    float l2 = INFINITY, dd = 0.f;       // dQ kernel: LSE log2(e) and D of this lane's query (rows past the end: P = 0)
    {
        const bool live = row < p.L_stat;
        const T* p1 = reinterpret_cast<const T*>(p.st1) + (int64_t)b * p.s1_sb + (int64_t)h * p.s1_sh + (int64_t)(live ? row : 0) * p.s1_sl + 8 * hh;
        const T* p2 = reinterpret_cast<const T*>(p.st2) + (int64_t)b * p.s2_sb + (int64_t)h * p.s2_sh + (int64_t)(live ? row : 0) * p.s2_sl + 8 * hh;
        const V8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < kWideMaxNC; ++c) {
            b1[c] = z; b2[c] = z;
            if (c < nc && live) { b1[c] = *reinterpret_cast<const V8*>(p1 + 16 * c); b2[c] = *reinterpret_cast<const V8*>(p2 + 16 * c); }
        }
        if (!DKDV && live) { const float2 st = p.stats[(int64_t)bh * p.L_stat + row]; l2 = st.x; dd = st.y; }
    }
    f32x16 acc1[kWideDbPerWave], acc2[kWideDbPerWave];   // dQ^T | dV^T, dK^T
#pragma unroll
    for (int i = 0; i < kWideDbPerWave; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) { acc1[i][e] = 0.f; acc2[i][e] = 0.f; }
    }
    const char* const head = p.stream + (size_t)bh * p.n_tiles * tile_bytes;
    auto frag = [&](const char* tile, int f) { return *reinterpret_cast<const V8*>(tile + (size_t)f * kFragBytes + lane * 16); };

    for (int t = t_lo; t < t_hi; ++t) {
        const char* const tile = head + (size_t)t * tile_bytes;
        f32x16 sc, dp;
#pragma unroll
        for (int e = 0; e < 16; ++e) { sc[e] = 0.f; dp[e] = 0.f; }
#pragma unroll
        for (int c = 0; c < kWideMaxNC; ++c) {
            if (c < nc) {
                sc = mfma32(frag(tile, c), b1[c], sc);
                dp = mfma32(frag(tile, nc + c), b2[c], dp);
            }
        }
        float l2v[16], ddv[16];
        if (DKDV) {   // statistics of the 32 streamed queries: LSE log2(e) at float index 16 hh + e, D at 32 + 16 hh + e
            const float* st = reinterpret_cast<const float*>(tile + (size_t)(sp_frags + op_frags) * kFragBytes);
#pragma unroll
            for (int e = 0; e < 16; ++e) { l2v[e] = st[16 * hh + e]; ddv[e] = st[32 + 16 * hh + e]; }
        }
        V8 uf[2], wf[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int srow = t * kRows + 8 * (e >> 2) + 4 * hh + (e & 3);   // streamed row of element e
            const bool ok = DKDV ? (!causal || row <= srow) : (srow < p.L_stream && (!causal || srow <= row));   // key <= query
            const float se = ok ? sc[e] : -INFINITY;
            const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(se, p.scale_log2, -(DKDV ? l2v[e] : l2)));
            const float we = pe * (dp[e] - (DKDV ? ddv[e] : dd));
            uf[e >> 3][e & 7] = (T)pe;
            wf[e >> 3][e & 7] = (T)we;
        }
#pragma unroll
        for (int i = 0; i < kWideDbPerWave; ++i) {
            const int db = wave + kWideWaves * i;
            if (db < ndb) {
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    if (DKDV) {
                        acc1[i] = mfma32(frag(tile, sp_frags + 2 * db + c), uf[c], acc1[i]);               // dV^T += dO^T U
                        acc2[i] = mfma32(frag(tile, sp_frags + 2 * ndb + 2 * db + c), wf[c], acc2[i]);     // dK^T += Q^T W
                    } else {
                        acc1[i] = mfma32(frag(tile, sp_frags + 2 * db + c), wf[c], acc1[i]);               // dQ^T += K^T W
                    }
                }
            }
        }
    }
    // dQ = s dQ^T   |   dV = dV^T, dK = s dK^T
    if (row < p.L_stat) {
        T* o1 = reinterpret_cast<T*>(p.out1) + (int64_t)b * p.o1_sb + (int64_t)h * p.o1_sh + (int64_t)row * p.o1_sl;
        T* o2 = DKDV ? reinterpret_cast<T*>(p.out2) + (int64_t)b * p.o2_sb + (int64_t)h * p.o2_sh + (int64_t)row * p.o2_sl : o1;
        const float s1 = DKDV ? 1.0f : p.sm_scale;
#pragma unroll
        for (int i = 0; i < kWideDbPerWave; ++i) {
            const int db = wave + kWideWaves * i;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int ch = 32 * db + 8 * g + 4 * hh;
                if (db < ndb && ch < d) {
                    V4 v1, v2;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        v1[r] = (T)(acc1[i][4 * g + r] * s1);
                        v2[r] = (T)(acc2[i][4 * g + r] * p.sm_scale);
                    }
                    *reinterpret_cast<V4*>(o1 + ch) = v1;
                    if (DKDV) *reinterpret_cast<V4*>(o2 + ch) = v2;
                }
            }
        }
    }
}

// Add the partial sums of the ranges of one stationary row (fixed order), scale, round, store.
// One thread per (row, 4 channels).
template <typename T, bool DKDV>
__global__ void __launch_bounds__(256) bwd_combine_kernel(const BwdParams p, int D) {
    typedef typename VecOf<T>::v4 V4;
    const int tpr = D / 4;
    const int64_t r = (int64_t)blockIdx.x * (256 / tpr) + threadIdx.x / tpr;
    const int c = (threadIdx.x % tpr) * 4;
    const int pair_i = (int)(r / kBlock), wrow = (int)(r % kBlock);
    const int pair = p.n_full + pair_i;
    const int blk = pair % p.n_blk, bh = p.bh0 + pair / p.n_blk, b = bh / p.H, h = bh % p.H;
    const int row = blk * kBlock + wrow;
    if (pair_i >= p.n_rem || row >= p.L_stat) return;
    const int W = DKDV ? 2 * D : D;
    float4 a1 = make_float4(0.f, 0.f, 0.f, 0.f), a2 = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int i = 0; i < p.splits; ++i) {
        const float* pa = p.part + (((int64_t)pair_i * p.splits + i) * kBlock + wrow) * W + c;
        const float4 x = *reinterpret_cast<const float4*>(pa);
        a1.x += x.x; a1.y += x.y; a1.z += x.z; a1.w += x.w;
        if (DKDV) {
            const float4 y = *reinterpret_cast<const float4*>(pa + D);
            a2.x += y.x; a2.y += y.y; a2.z += y.z; a2.w += y.w;
        }
    }
    const float s1 = DKDV ? 1.0f : p.sm_scale;
    V4 v1;
    v1[0] = (T)(a1.x * s1); v1[1] = (T)(a1.y * s1); v1[2] = (T)(a1.z * s1); v1[3] = (T)(a1.w * s1);
    *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.out1) + (int64_t)b * p.o1_sb + (int64_t)h * p.o1_sh + (int64_t)row * p.o1_sl + c) = v1;
    if (DKDV) {
        V4 v2;
        v2[0] = (T)(a2.x * p.sm_scale); v2[1] = (T)(a2.y * p.sm_scale); v2[2] = (T)(a2.z * p.sm_scale); v2[3] = (T)(a2.w * p.sm_scale);
        *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.out2) + (int64_t)b * p.o2_sb + (int64_t)h * p.o2_sh + (int64_t)row * p.o2_sl + c) = v2;
    }
}


// ---------------------------------------------------------------------------------------------- dQ from kept dS
// When the dK/dV kernel keeps its 16-bit dS tiles, dQ = s dS K is one product per tile instead of three (no second
// computation of S and dP): a pass that streams dS from memory once and is bound by that stream (2 bytes per score
// element; K^T comes from the L2).  A workgroup owns 256 queries, one 32-query tile per wavefront (8 wavefronts, two per
// SIMD); per 32-key step a wavefront copies its own 2 KB dS tile and an eighth of the shared 32-key K^T part into an LDS
// ring with direct-to-LDS loads kDsRing - 1 steps ahead, and accumulates dQ^T += K^T W with W = dS^T.
// A dS tile lies in memory in the 16-byte units the dK/dV kernel's wavefront held -- one key, eight queries -- and is
// wanted with lane = query, eight keys per lane: the transposing LDS read (ds_read_b64_tr_b16) does that.  Within a
// group of 16 lanes, lane i passes the address of 8 bytes (row i of a 16 x 4 matrix M of 16-bit values) and receives
// M[i/4 + 4k][i%4], k = 0..3.  A row of M here is one key's dS for 4 consecutive queries, so lane (query, half hh) gets, for
// key chunk c and read t, the keys 16 c + 8 t + 4 hh + k -- the order in which a V^T-type fragment of K^T holds them.
constexpr int kDsLoadPolicy = 2;     // cache policy bits of the dS loads: non-temporal (each tile is read once; 4 % faster than plain loads)
constexpr int kDsRing = 6;            // steps of dS / K^T in flight per workgroup
constexpr int kDqWaves = 8;           // query tiles per workgroup
constexpr int kDqThreads = 64 * kDqWaves;

struct DqFromDsParams {
    const char* ds;                    // [local head][n_q_tiles][n_kt_pad][2 KB]
    int64_t ds_head_bytes;
    int n_kt_pad;
    const char* kt_img;                // K^T stream: [B*H][n_k_tiles][2 NDB fragments]
    void* dq;
    int64_t o_sb, o_sh, o_sl;
    int H, Lq, Lkv, n_q_tiles, n_k_tiles, n_blk, bh0, causal;
    float sm_scale;
};

template <int D>
struct DqCfg {
    static constexpr int NDB = (D + 31) / 32;
    static constexpr int KT_FR = 2 * NDB, KT_BYTES = KT_FR * kFragBytes;
    static constexpr int W_BYTES = 2 * kFragBytes;                       // one dS tile
    static constexpr int SLOT_BYTES = kDqWaves * W_BYTES + KT_BYTES;
    static constexpr int LDS_BYTES = kDsRing * SLOT_BYTES;
    static constexpr int LOADS = 3;                                      // per wavefront per step: 2 (dS tile) + 1 (K^T fragment)
};

typedef short s16x4 __attribute__((ext_vector_type(4)));

template <typename T, int D>
__global__ void __attribute__((amdgpu_flat_work_group_size(kDqThreads, kDqThreads), amdgpu_waves_per_eu(2, 2)))
attn_dq_from_ds_kernel(const DqFromDsParams p) {
    typedef DqCfg<D> C;
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr int NDB = C::NDB;
    // vmcnt(n): the loads of the newest kDsRing - 2 steps may still be in flight
    constexpr int IN_FLIGHT = C::LOADS * (kDsRing - 2);
    constexpr int WAIT_LOADS = (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14) | 0x0F70;

    const int blk = blockIdx.x % p.n_blk, bhl = blockIdx.x / p.n_blk, bh = p.bh0 + bhl, b = bh / p.H, h = bh % p.H;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int qt = blk * kDqWaves + wave;          // this wavefront's query tile
    const bool live_tile = qt < p.n_q_tiles;
    const int row = qt * kRows + j;

    // key tiles this workgroup walks: all, or up to its last query's diagonal when causal
    int n_steps = p.n_k_tiles;
    if (p.causal) { const int lim = blk * kDqWaves + kDqWaves; n_steps = n_steps < lim ? n_steps : lim; }

    // this wavefront's run of dS tiles (one query tile, all key tiles: contiguous), and the head's K^T stream
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.ds) + (int64_t)bhl * p.ds_head_bytes + (int64_t)(live_tile ? qt : 0) * p.n_kt_pad * C::W_BYTES, 0,
        live_tile ? p.n_kt_pad * C::W_BYTES : 0, 0x00020000);   // no tile: every load returns zeros
    const __amdgpu_buffer_rsrc_t rs_k = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.kt_img) + (size_t)bh * p.n_k_tiles * C::KT_BYTES, 0, p.n_k_tiles * C::KT_BYTES, 0x00020000);
    const int kfrag = wave % C::KT_FR;             // the K^T fragment this wavefront copies (copied redundantly when there are fewer than 8)
    auto issue = [&](int u) {                      // loads of sweep position u (clamped: positions past the end repeat the last tile, unused)
        const int t = __builtin_amdgcn_readfirstlane(u < n_steps ? u : n_steps - 1);
        char* slot = smem + (u % kDsRing) * C::SLOT_BYTES;
        lds_load<0, kDsLoadPolicy>(rs_w, slot + wave * C::W_BYTES, lane * 16, t * C::W_BYTES);
        lds_load<kFragBytes, kDsLoadPolicy>(rs_w, slot + wave * C::W_BYTES, lane * 16, t * C::W_BYTES);
        lds_load<0>(rs_k, slot + kDqWaves * C::W_BYTES + kfrag * kFragBytes, lane * 16, t * C::KT_BYTES + kfrag * kFragBytes);
    };
#pragma unroll
    for (int u = 0; u < kDsRing - 1; ++u) issue(u);

    f32x16 acc[NDB];
#pragma unroll
    for (int i = 0; i < NDB; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
    }
    // transposing read: byte offset, inside a dS tile, of the 8 bytes this lane passes for key chunk 0, read 0
    //   group g = lane / 16: queries 16 (g % 2) .. + 15, key half g / 2;  lane i of the group passes row r = i:
    //   queries 16 (g%2) + 4 (r%4) .. + 3 of key 4 (g/2) + r/4  (+ 16 c + 8 t).  In the tile the 16-byte unit (query half c' = g%2,
    //   key, lane half hh' = r%2 of the wavefront that formed it) sits at slot 16 (key / 4) + 8 c' + 4 hh' + key % 4, and the lane
    //   wants its second 8 bytes when (r%4)/2: the 32 lanes of a pass touch 256 consecutive bytes, every bank once.
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;   // LDS address of smem[0]
    const int g16 = lane >> 4, r16 = lane & 15;
    const unsigned tr_off = (unsigned)(256 * (g16 >> 1) + 128 * (g16 & 1) + 64 * (r16 & 1) + 16 * (r16 >> 2) + 8 * ((r16 & 3) >> 1));

    auto step = [&](int s) {
        const char* slot = smem + (s % kDsRing) * C::SLOT_BYTES;
        // (written out: the compiler takes the builtin of this read for an access that may alias the direct-to-LDS loads in
        // flight and puts vmcnt(0) in front of it, which would end the prefetch; it does not see through the asm, so the
        // wait for the four results is in the block as well)
        const unsigned wt = lds0 + (unsigned)((s % kDsRing) * C::SLOT_BYTES + wave * C::W_BYTES) + tr_off;
        s16x4 t00, t01, t10, t11;
        asm volatile("ds_read_b64_tr_b16 %0, %4\n\t"
                     "ds_read_b64_tr_b16 %1, %4 offset:512\n\t"
                     "ds_read_b64_tr_b16 %2, %4 offset:1024\n\t"
                     "ds_read_b64_tr_b16 %3, %4 offset:1536\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(t00), "=&v"(t01), "=&v"(t10), "=&v"(t11) : "v"(wt) : "memory");
        V8 wf[2];
        wf[0] = __builtin_shufflevector(__builtin_bit_cast(V4, t00), __builtin_bit_cast(V4, t01), 0, 1, 2, 3, 4, 5, 6, 7);
        wf[1] = __builtin_shufflevector(__builtin_bit_cast(V4, t10), __builtin_bit_cast(V4, t11), 0, 1, 2, 3, 4, 5, 6, 7);
        // dead operands become zeros: tiles the (causal) dK/dV kernel never formed, keys past the end of the last tile
        const bool unformed = p.causal && (s / 4) * 4 > qt;
        if (unformed || !live_tile || s * kRows + kRows > p.Lkv) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = s * kRows + 16 * c + 8 * (e >> 2) + 4 * hh + (e & 3);
                    if (unformed || !live_tile || key >= p.Lkv) wf[c][e] = (T)0.0f;
                }
            }
        }
        const char* kt = slot + kDqWaves * C::W_BYTES + lane * 16;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
#pragma unroll
            for (int c = 0; c < 2; ++c)
                acc[db] = mfma32(*reinterpret_cast<const V8*>(kt + (2 * db + c) * kFragBytes), wf[c], acc[db]);
        }
    };
    for (int s = 0; s < n_steps; ++s) {
        __builtin_amdgcn_s_waitcnt(WAIT_LOADS);
        __builtin_amdgcn_s_barrier();          // everybody's loads of step s have landed, everybody is done reading step s - 1
        asm volatile("" ::: "memory");
        issue(s + kDsRing - 1);                // into the slot of step s - 1
        step(s);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);        // drain the trailing loads before the LDS is released
    if (live_tile && row < p.Lq) {
        T* o1 = reinterpret_cast<T*>(p.dq) + (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)row * p.o_sl;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * db + 8 * g + 4 * hh;   // registers 4g..4g+3 are 4 consecutive channels
                if (d < D) {
                    V4 v1;
#pragma unroll
                    for (int r = 0; r < 4; ++r) v1[r] = (T)(acc[db][4 * g + r] * p.sm_scale);
                    *reinterpret_cast<V4*>(o1 + d) = v1;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------ host
typedef void (*bwd_kernel_t)(const BwdParams);

typedef void (*dq_from_ds_kernel_t)(const DqFromDsParams);

// Keeping dS pays where the two products it saves are large next to the 4 bytes per score element it moves: head dim 128.
inline bool spill_head_dim(int d) { return d == 128; }
// head dim 128: the four-role dK/dV kernel, with or without keeping dS (the other head dims: attn_bwd_kernel<T, D, KIND_DKDV>)
template <typename T>
bwd_kernel_t pick_dkdv_quad(int d, bool keep_ds) {
    if (d != 128) return nullptr;
    return keep_ds ? attn_dkdv_quad_kernel<T, 128, true> : attn_dkdv_quad_kernel<T, 128, false>;
}
inline size_t dkdv_lds_bytes(int d, size_t two_role) { return d == 128 ? (size_t)QuadCfg<128>::LDS_BYTES : two_role; }
template <typename T>
dq_from_ds_kernel_t pick_dq_from_ds(int d) { return d == 128 ? attn_dq_from_ds_kernel<T, 128> : nullptr; }

template <typename T, int KIND>
bwd_kernel_t pick_bwd(int d) {
#ifdef COSMOS_ATTN_ONLY_D128   // development builds: instantiate the d=128 kernels only
    return d == 128 ? attn_bwd_kernel<T, 128, KIND> : nullptr;
#endif
    switch (d) {
        case 16: return attn_bwd_kernel<T, 16, KIND>;
        case 32: return attn_bwd_kernel<T, 32, KIND>;
        case 64: return attn_bwd_kernel<T, 64, KIND>;
        case 128: return attn_bwd_kernel<T, 128, KIND>;
        default: return nullptr;
    }
}

struct BwdGeom {
    int nc, ndb;
    size_t q_tile_bytes, k_tile_bytes, lds_dkdv, lds_dq;
    int n_q_tiles, n_k_tiles;
    size_t stats_bytes, q_img_bytes, k_img_bytes;
    explicit BwdGeom(const cosmos_attn_bwd_desc* d) {
        nc = d->d / 16; ndb = (d->d + 31) / 32;
        quad = d->d == 128;   // attn_dkdv_quad_kernel: one copy of the query stream ([Q | dO | statistics])
        q_tile_bytes = (size_t)(quad ? 2 * nc + 1 : 2 * nc + 4 * ndb + 1) * kFragBytes;
        k_tile_bytes = (size_t)(2 * nc + 2 * ndb) * kFragBytes;
        lds_dkdv = (size_t)kRingS * 2 * nc * kFragBytes + (size_t)kRingO * 4 * ndb * kFragBytes + 2 * 4 * 4 * kFragBytes + kRingStats * kFragBytes;
        lds_dq = (size_t)kRingS * 2 * nc * kFragBytes + (size_t)kRingO * 2 * ndb * kFragBytes + 2 * 4 * 2 * kFragBytes;
        n_q_tiles = (d->Lq + kRows - 1) / kRows; n_k_tiles = (d->Lkv + kRows - 1) / kRows;
        const size_t bh = (size_t)d->B * d->H;
        stats_bytes = ((bh * d->Lq * sizeof(float2)) + 1023) / 1024 * 1024;
        q_img_bytes = bh * n_q_tiles * q_tile_bytes;
        k_img_bytes = bh * n_k_tiles * k_tile_bytes;
        if (d->d == 256) {   // attn_bwd_wide_kernel: blocks of 32 stationary rows, never cut
            dkdv = Plan{(d->Lkv + kRows - 1) / kRows, (d->Lkv + kRows - 1) / kRows * (int)bh, (d->Lkv + kRows - 1) / kRows * (int)bh, 0, 1};
            dq = Plan{(d->Lq + kRows - 1) / kRows, (d->Lq + kRows - 1) / kRows * (int)bh, (d->Lq + kRows - 1) / kRows * (int)bh, 0, 1};
            part_bytes = 0;
            return;
        }
        const int n_kblk = (d->Lkv + kBlock - 1) / kBlock;
        // Keep dS?  Its tiles for one head take n_q_tiles * n_kt_pad * 2 KB; heads are served in groups that fit the budget
        // (desc->max_ds_mib: 0 = kDefaultDsMiB, > 0 = that many MiB, < 0 = never keep dS).
        n_kt_pad = 4 * n_kblk;
        ds_head_bytes = (size_t)n_q_tiles * n_kt_pad * 2 * kFragBytes;
        const int64_t budget = d->max_ds_mib < 0 ? 0 : (int64_t)(d->max_ds_mib > 0 ? d->max_ds_mib : kDefaultDsMiB) << 20;
        if (spill_head_dim(d->d) && (int64_t)ds_head_bytes <= budget && (int64_t)n_kt_pad * 2 * kFragBytes < ((int64_t)1 << 31)) {
            spill = true;
            const int64_t fit = budget / (int64_t)ds_head_bytes;
            group = (int)(fit < (int64_t)bh ? fit : (int64_t)bh);
            ds_bytes = (size_t)group * ds_head_bytes;
            k_tile_bytes = (size_t)(2 * ndb) * kFragBytes;            // the key stream holds K^T alone
            k_img_bytes = bh * n_k_tiles * k_tile_bytes;
        }
        dkdv = plan(n_kblk, spill ? group : (int)bh, n_q_tiles, d->causal != 0);
        dq = plan((d->Lq + kBlock - 1) / kBlock, (int)bh, n_k_tiles, d->causal != 0);
        size_t p1 = (size_t)dkdv.n_rem * dkdv.splits * kBlock * 2 * d->d * sizeof(float);
        if (spill && bh % group) {   // the last, smaller group has a plan of its own
            const Plan last = plan(n_kblk, (int)(bh % group), n_q_tiles, d->causal != 0);
            const size_t p3 = (size_t)last.n_rem * last.splits * kBlock * 2 * d->d * sizeof(float);
            p1 = p1 > p3 ? p1 : p3;
        }
        const size_t p2 = spill ? 0 : (size_t)dq.n_rem * dq.splits * kBlock * d->d * sizeof(float);
        part_bytes = ((p1 > p2 ? p1 : p2) + 1023) / 1024 * 1024;     // the two kernels run one after the other
    }
    static constexpr int kDefaultDsMiB = 32 * 1024;
    bool quad = false;
    bool spill = false;
    int group = 0, n_kt_pad = 0;        // heads per group; key tiles per query tile in the dS buffer
    size_t ds_head_bytes = 0, ds_bytes = 0;
    // How the (block of stationary rows, head) pairs of a kernel are dealt out (see choose_splits): the pairs of a partly
    // filled last round of workgroups are cut along the stream and bwd_combine_kernel adds the ranges up.
    struct Plan { int n_blk, n_pairs, n_full, n_rem, splits; };
    static Plan plan(int n_blk, int bh, int n_stream_tiles, bool causal) {
        Plan s;
        s.n_blk = n_blk; s.n_pairs = n_blk * bh; s.n_full = s.n_pairs; s.n_rem = 0; s.splits = 1;
        const int rem = s.n_pairs % kNumCUs;
        const int splits = causal ? 1 : choose_splits(rem, n_stream_tiles);
        if (splits < 2) return s;
        s.n_rem = rem; s.n_full = s.n_pairs - rem; s.splits = splits;
        return s;
    }
    Plan dkdv, dq;
    size_t part_bytes;
};

int validate_bwd(const cosmos_attn_bwd_desc* d) {
    if (!d) return COSMOS_ATTN_BAD_ARG;
    if (d->abi_version != COSMOS_ATTN_ABI_VERSION) return COSMOS_ATTN_BAD_ARG;
    if (d->B <= 0 || d->H <= 0 || d->Lq <= 0 || d->Lkv <= 0) return COSMOS_ATTN_BAD_ARG;
    if (!d->q || !d->k || !d->v || !d->o || !d->dout || !d->lse || !d->dq || !d->dk || !d->dv) return COSMOS_ATTN_BAD_ARG;
    if (d->dtype != COSMOS_ATTN_BF16 && d->dtype != COSMOS_ATTN_FP16) return COSMOS_ATTN_UNSUPPORTED;
    if (!head_dim_ok(d->d) && d->d != 256) return COSMOS_ATTN_BAD_SHAPE;
    if (d->causal && d->Lq != d->Lkv) return COSMOS_ATTN_BAD_SHAPE;
    const void* ptrs[] = {d->q, d->k, d->v, d->o, d->dout, d->dq, d->dk, d->dv};
    for (const void* ptr : ptrs) if (!aligned16(ptr)) return COSMOS_ATTN_BAD_STRIDE;
    const int64_t* strides[] = {d->q_stride, d->k_stride, d->v_stride, d->o_stride, d->dout_stride, d->dq_stride, d->dk_stride, d->dv_stride};
    for (const int64_t* s : strides) if (!strides_ok(s)) return COSMOS_ATTN_BAD_STRIDE;
    if ((int64_t)d->B * d->H > 65535) return COSMOS_ATTN_BAD_SHAPE;   // grid.y limit of the re-tiling kernels
    const BwdGeom g(d);
    if ((int64_t)g.n_q_tiles * (int64_t)g.q_tile_bytes >= (int64_t)1 << 31) return COSMOS_ATTN_BAD_SHAPE;   // 32-bit buffer offsets per head
    if ((int64_t)g.n_k_tiles * (int64_t)g.k_tile_bytes >= (int64_t)1 << 31) return COSMOS_ATTN_BAD_SHAPE;
    return COSMOS_ATTN_OK;
}

PackSrc src_of(const void* ptr, const int64_t* s) { return PackSrc{(const uint16_t*)ptr, s[0], s[1], s[2]}; }

}  // namespace

extern "C" {

COSMOS_ATTN_API size_t cosmos_attn_bwd_workspace_bytes(const cosmos_attn_bwd_desc* d) {
    if (validate_bwd(d) != COSMOS_ATTN_OK) return 0;
    const BwdGeom g(d);
    return g.stats_bytes + g.q_img_bytes + g.k_img_bytes + g.part_bytes + g.ds_bytes;
}

COSMOS_ATTN_API int cosmos_attn_bwd(const cosmos_attn_bwd_desc* d, void* workspace, size_t workspace_bytes, void* stream_) {
    const int st = validate_bwd(d);
    if (st != COSMOS_ATTN_OK) return st;
    if (!workspace || workspace_bytes < cosmos_attn_bwd_workspace_bytes(d) || !aligned16(workspace)) return COSMOS_ATTN_WORKSPACE_TOO_SMALL;
    if (!device_is_whole_mi355x()) return COSMOS_ATTN_WRONG_DEVICE;
    hipStream_t stream = (hipStream_t)stream_;
    const BwdGeom g(d);
    const bool bf16 = d->dtype == COSMOS_ATTN_BF16;
    const bool wide = d->d == 256;
    bwd_kernel_t k_dkdv = bf16 ? pick_bwd<__bf16, KIND_DKDV>(d->d) : pick_bwd<_Float16, KIND_DKDV>(d->d);
    if (bwd_kernel_t quad = bf16 ? pick_dkdv_quad<__bf16>(d->d, false) : pick_dkdv_quad<_Float16>(d->d, false)) k_dkdv = quad;
    const size_t lds_dkdv = dkdv_lds_bytes(d->d, g.lds_dkdv);
    bwd_kernel_t k_dq = bf16 ? pick_bwd<__bf16, KIND_DQ>(d->d) : pick_bwd<_Float16, KIND_DQ>(d->d);
    if (!wide && (!k_dkdv || !k_dq)) return COSMOS_ATTN_UNSUPPORTED;
    char* ws = (char*)workspace;
    float2* stats = (float2*)ws;
    char* q_img = ws + g.stats_bytes;
    char* k_img = q_img + g.q_img_bytes;
    float* part = (float*)(k_img + g.k_img_bytes);
    char* ds = (char*)part + g.part_bytes;
    const int BH = d->B * d->H;
    auto launch = [&](bwd_kernel_t fn, size_t lds, const BwdGeom::Plan& pl, BwdParams& bp, bool is_dkdv) {
        bp.n_blk = pl.n_blk; bp.n_full = pl.n_full; bp.n_rem = pl.n_rem; bp.splits = pl.splits; bp.part = part;
        if (wide) {
            auto wfn = is_dkdv ? (bf16 ? attn_bwd_wide_kernel<__bf16, KIND_DKDV> : attn_bwd_wide_kernel<_Float16, KIND_DKDV>)
                               : (bf16 ? attn_bwd_wide_kernel<__bf16, KIND_DQ> : attn_bwd_wide_kernel<_Float16, KIND_DQ>);
            hipLaunchKernelGGL(wfn, dim3((unsigned)pl.n_pairs), dim3(64 * kWideWaves), 0, stream, bp, (int)d->d);
            return true;
        }
        if (!allow_lds((const void*)fn, lds)) return false;
        hipLaunchKernelGGL(fn, dim3((unsigned)(pl.n_full + pl.n_rem * pl.splits)), dim3(kBwdThreads), lds, stream, bp);
        if (pl.splits > 1) {
            const int rows_per_block = 256 / (d->d / 4);
            const dim3 cgrid((unsigned)(((int64_t)pl.n_rem * kBlock + rows_per_block - 1) / rows_per_block));
            auto cfn = is_dkdv ? (bf16 ? bwd_combine_kernel<__bf16, true> : bwd_combine_kernel<_Float16, true>)
                               : (bf16 ? bwd_combine_kernel<__bf16, false> : bwd_combine_kernel<_Float16, false>);
            hipLaunchKernelGGL(cfn, cgrid, dim3(256), 0, stream, bp, d->d);
        }
        return true;
    };

    {   // per-query statistics
        StatsParams sp;
        sp.o = (const uint16_t*)d->o; sp.dout = (const uint16_t*)d->dout;
        sp.o_sb = d->o_stride[0]; sp.o_sh = d->o_stride[1]; sp.o_sl = d->o_stride[2];
        sp.g_sb = d->dout_stride[0]; sp.g_sh = d->dout_stride[1]; sp.g_sl = d->dout_stride[2];
        sp.lse = d->lse; sp.stats = stats; sp.H = d->H; sp.Lq = d->Lq; sp.d = d->d; sp.bf16 = bf16 ? 1 : 0;
        hipLaunchKernelGGL(bwd_stats_kernel, dim3((d->Lq + kPackThreads / 8 - 1) / (kPackThreads / 8), BH), dim3(kPackThreads), 0, stream, sp);
    }
    {   // query stream: Q, dO, dO^T, Q^T, statistics
        PackBwdParams pp;
        pp.a1 = src_of(d->q, d->q_stride); pp.a2 = src_of(d->dout, d->dout_stride);
        pp.c1 = src_of(d->dout, d->dout_stride); pp.c2 = src_of(d->q, d->q_stride);
        pp.n_vt = g.quad ? 0 : 2; pp.swz = g.quad ? 1 : 0;
        pp.stats = stats; pp.out = (uint4*)q_img;
        pp.H = d->H; pp.L = d->Lq; pp.d = d->d; pp.n_tiles = g.n_q_tiles; pp.nc = g.nc; pp.ndb = g.ndb;
        pp.tile_frags = (int)(g.q_tile_bytes / kFragBytes);
        hipLaunchKernelGGL(pack_stream_kernel, dim3(g.n_q_tiles, BH), dim3(kPackThreads), 0, stream, pp);
    }
    {   // key stream: K, V, K^T  (K^T alone when dS is kept: the pass that reads it forms no scores)
        PackBwdParams pp;
        pp.a1 = src_of(d->k, d->k_stride); pp.a2 = src_of(d->v, d->v_stride);
        pp.c1 = src_of(d->k, d->k_stride); pp.c2 = PackSrc{nullptr, 0, 0, 0};
        pp.n_vt = 1; pp.swz = 0;
        pp.stats = nullptr; pp.out = (uint4*)k_img;
        pp.H = d->H; pp.L = d->Lkv; pp.d = d->d; pp.n_tiles = g.n_k_tiles; pp.nc = g.spill ? 0 : g.nc; pp.ndb = g.ndb;
        pp.tile_frags = (int)(g.k_tile_bytes / kFragBytes);
        hipLaunchKernelGGL(pack_stream_kernel, dim3(g.n_k_tiles, BH), dim3(kPackThreads), 0, stream, pp);
    }
    if (hipGetLastError() != hipSuccess) return COSMOS_ATTN_LAUNCH_FAILED;

    BwdParams bp;
    bp.stats = stats; bp.H = d->H; bp.causal = d->causal;
    bp.sm_scale = d->sm_scale; bp.scale_log2 = d->sm_scale * 1.4426950408889634f;
    bp.bh0 = 0; bp.ds = nullptr; bp.ds_head_bytes = 0; bp.n_kt_pad = 0;
    auto set_dkdv = [&]() {   // dK, dV: stationary keys, streamed queries
        bp.st1 = d->k; bp.s1_sb = d->k_stride[0]; bp.s1_sh = d->k_stride[1]; bp.s1_sl = d->k_stride[2];
        bp.st2 = d->v; bp.s2_sb = d->v_stride[0]; bp.s2_sh = d->v_stride[1]; bp.s2_sl = d->v_stride[2];
        bp.out1 = d->dv; bp.o1_sb = d->dv_stride[0]; bp.o1_sh = d->dv_stride[1]; bp.o1_sl = d->dv_stride[2];
        bp.out2 = d->dk; bp.o2_sb = d->dk_stride[0]; bp.o2_sh = d->dk_stride[1]; bp.o2_sl = d->dk_stride[2];
        bp.stream = q_img; bp.L_stat = d->Lkv; bp.L_stream = d->Lq; bp.n_tiles = g.n_q_tiles;
    };
    if (g.spill) {
        // dS kept: per group of heads, the dK/dV kernel (which writes the group's dS tiles), then the pass that turns them into dQ
        bwd_kernel_t k_spill = bf16 ? pick_dkdv_quad<__bf16>(d->d, true) : pick_dkdv_quad<_Float16>(d->d, true);
        dq_from_ds_kernel_t k_ds = bf16 ? pick_dq_from_ds<__bf16>(d->d) : pick_dq_from_ds<_Float16>(d->d);
        if (!k_spill || !k_ds) return COSMOS_ATTN_UNSUPPORTED;
        const size_t lds_ds = (size_t)kDsRing * (kDqWaves * 2 * kFragBytes + 2 * g.ndb * kFragBytes);
        if (!allow_lds((const void*)k_ds, lds_ds)) return COSMOS_ATTN_LAUNCH_FAILED;
        set_dkdv();
        bp.ds = ds; bp.ds_head_bytes = (int64_t)g.ds_head_bytes; bp.n_kt_pad = g.n_kt_pad;
        DqFromDsParams qp;
        qp.ds = ds; qp.ds_head_bytes = (int64_t)g.ds_head_bytes; qp.n_kt_pad = g.n_kt_pad; qp.kt_img = k_img;
        qp.dq = d->dq; qp.o_sb = d->dq_stride[0]; qp.o_sh = d->dq_stride[1]; qp.o_sl = d->dq_stride[2];
        qp.H = d->H; qp.Lq = d->Lq; qp.Lkv = d->Lkv; qp.n_q_tiles = g.n_q_tiles; qp.n_k_tiles = g.n_k_tiles;
        qp.n_blk = (g.n_q_tiles + kDqWaves - 1) / kDqWaves; qp.causal = d->causal; qp.sm_scale = d->sm_scale;
        for (int bh0 = 0; bh0 < BH; bh0 += g.group) {
            const int heads = BH - bh0 < g.group ? BH - bh0 : g.group;
            const BwdGeom::Plan pl = heads == g.group ? g.dkdv : BwdGeom::plan(g.dkdv.n_blk, heads, g.n_q_tiles, d->causal != 0);
            bp.bh0 = bh0;
            if (!launch(k_spill, lds_dkdv, pl, bp, true)) return COSMOS_ATTN_LAUNCH_FAILED;
            qp.bh0 = bh0;
            hipLaunchKernelGGL(k_ds, dim3((unsigned)(qp.n_blk * heads)), dim3(kDqThreads), lds_ds, stream, qp);
        }
        return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
    }
    {
        set_dkdv();
        if (!launch(k_dkdv, lds_dkdv, g.dkdv, bp, true)) return COSMOS_ATTN_LAUNCH_FAILED;
    }
    {   // dQ: stationary queries, streamed keys
        bp.st1 = d->q; bp.s1_sb = d->q_stride[0]; bp.s1_sh = d->q_stride[1]; bp.s1_sl = d->q_stride[2];
        bp.st2 = d->dout; bp.s2_sb = d->dout_stride[0]; bp.s2_sh = d->dout_stride[1]; bp.s2_sl = d->dout_stride[2];
        bp.out1 = d->dq; bp.o1_sb = d->dq_stride[0]; bp.o1_sh = d->dq_stride[1]; bp.o1_sl = d->dq_stride[2];
        bp.out2 = nullptr; bp.o2_sb = bp.o2_sh = bp.o2_sl = 0;
        bp.stream = k_img; bp.L_stat = d->Lq; bp.L_stream = d->Lkv; bp.n_tiles = g.n_k_tiles;
        if (!launch(k_dq, g.lds_dq, g.dq, bp, false)) return COSMOS_ATTN_LAUNCH_FAILED;
    }
    return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
}

}  // extern "C"
