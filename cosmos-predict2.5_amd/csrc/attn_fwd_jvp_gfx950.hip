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
//     64-key tile, the exact byte order in which the MFMA A-operand fragments are consumed
//     (1 KB per fragment = 64 lanes x 16 B, V already transposed and key-permuted to match the
//     S^T register layout).  The attention kernel then moves tiles HBM/L2 -> LDS with direct-to-LDS
//     loads (global_load_lds_dwordx4, no VGPR staging) and reads fragments back with conflict-free
//     linear ds_read_b128.  Re-tiling costs one extra read+write of K/V (<1 % of the call at L=84480)
//     and removes every transpose / swizzle / tail check from the hot loop.
//   * One workgroup = 4 wavefronts = 128 query rows; 1 wavefront per SIMD with the full 512-register
//     budget (Q, dQ fragments and both fp32 accumulators stay in registers for the whole KV sweep);
//     LDS holds two tile buffers (2 x 64 KB at d=128 with tangents) so the next tile streams in while
//     the current one is consumed; one workgroup barrier per tile.
//   * Query-tile index is the fastest grid dimension, so the 256 workgroups in flight sweep the same
//     head's K/V images together and share them through the per-XCD L2s and the Infinity Cache.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "cosmos_attn_hip.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

template <typename T> struct VecOf;
template <> struct VecOf<__bf16> { typedef bf16x8 v8; typedef bf16x4 v4; };
template <> struct VecOf<_Float16> { typedef f16x8 v8; typedef f16x4 v4; };

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

constexpr int kBlockM = 128;       // query rows per workgroup (4 wavefronts x 32)
constexpr int kBlockN = 64;        // keys per tile
constexpr int kThreads = 256;
constexpr int kFragBytes = 1024;   // one MFMA A-operand fragment: 64 lanes x 16 B

enum { MODE_FWD = 0, MODE_JVP_Q = 1, MODE_JVP_FULL = 2 };

// Geometry of one packed KV tile ("LDS image").  Sections in order: K, V^T, dK, dV^T (the last two only
// with tangents on k/v).  K-type fragment (kb, c): lane l holds K[32 kb + l%32][16 c + 8 (l/32) .. +7].
// V^T-type fragment (db, c): lane l, slot s holds V[16 c + 8 (s/4) + 4 (l/32) + s%4][32 db + l%32].
struct TileGeom {
    int nc, ndb, k_frags, vt_frags, tile_frags;
    __host__ __device__ TileGeom(int dqk, int dv, bool full)
        : nc(dqk / 16), ndb((dv + 31) / 32), k_frags(2 * (dqk / 16)), vt_frags(4 * ((dv + 31) / 32)),
          tile_frags((2 * (dqk / 16) + 4 * ((dv + 31) / 32)) * (full ? 2 : 1)) {}
};

struct PackParams {
    const uint16_t *k, *v, *tk, *tv;   // tk/tv may be null (then no tangent sections)
    int64_t k_sb, k_sh, k_sl, v_sb, v_sh, v_sl;
    uint4* out;
    int H, Lkv, dqk, dv, n_tiles;
};

// grid (n_tiles, B*H); every 16-byte unit of the tile image is produced by one thread.
__global__ void __launch_bounds__(kThreads) pack_kv_kernel(const PackParams p) {
    const int t = blockIdx.x, bh = blockIdx.y, b = bh / p.H, h = bh % p.H;
    const bool full = p.tk != nullptr;
    const TileGeom g(p.dqk, p.dv, full);
    uint4* dst = p.out + ((size_t)bh * p.n_tiles + t) * (size_t)(g.tile_frags * (kFragBytes / 16));
    const int64_t k_off = (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
    const int64_t v_off = (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
    const int units = g.tile_frags * 64;
    for (int u = threadIdx.x; u < units; u += kThreads) {
        int frag = u >> 6;
        const int l = u & 63, i = l & 31, hh = l >> 5;
        const uint16_t *ksrc = p.k, *vsrc = p.v;
        if (frag >= g.k_frags + g.vt_frags) { frag -= g.k_frags + g.vt_frags; ksrc = p.tk; vsrc = p.tv; }
        uint4 val = make_uint4(0u, 0u, 0u, 0u);
        if (frag < g.k_frags) {
            const int kb = frag / g.nc, c = frag % g.nc;
            const int key = t * kBlockN + 32 * kb + i;
            if (key < p.Lkv) val = *reinterpret_cast<const uint4*>(ksrc + k_off + (int64_t)key * p.k_sl + 16 * c + 8 * hh);
        } else {
            const int f = frag - g.k_frags, db = f >> 2, c = f & 3;
            const int d = 32 * db + i;
            uint16_t e[8];
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int key = t * kBlockN + 16 * c + 8 * (s >> 2) + 4 * hh + (s & 3);
                e[s] = (key < p.Lkv && d < p.dv) ? vsrc[v_off + (int64_t)key * p.v_sl + d] : (uint16_t)0;
            }
            val.x = e[0] | ((uint32_t)e[1] << 16); val.y = e[2] | ((uint32_t)e[3] << 16);
            val.z = e[4] | ((uint32_t)e[5] << 16); val.w = e[6] | ((uint32_t)e[7] << 16);
        }
        dst[u] = val;
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
};

extern __shared__ __attribute__((aligned(1024))) char smem[];

__device__ __forceinline__ void load_tile_to_lds(const char* src_lane, char* dst, int wave, int tile_frags) {
    // each wavefront-level instruction moves one 1 KB fragment: LDS address = dst + lane * 16
    for (int f = wave; f < tile_frags; f += 4) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src_lane + f * kFragBytes),
                                         (__attribute__((address_space(3))) void*)(dst + f * kFragBytes), 16, 0, 0);
    }
}

template <typename T, int DQK, int DV, int MODE>
__global__ void __attribute__((amdgpu_flat_work_group_size(kThreads, kThreads), amdgpu_waves_per_eu(1, 1)))
attn_fwd_jvp_kernel(const AttnParams p) {
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr int NC = DQK / 16;             // 16-wide d chunks of the QK^T contraction
    constexpr int NDB = (DV + 31) / 32;      // 32-row blocks of O^T
    constexpr bool JVP = MODE != MODE_FWD, FULL = MODE == MODE_JVP_FULL;
    constexpr int K_FR = 2 * NC, VT_FR = 4 * NDB;
    constexpr int TILE_FR = (K_FR + VT_FR) * (FULL ? 2 : 1);
    constexpr int TILE_BYTES = TILE_FR * kFragBytes;
    constexpr int VT_OFF = K_FR * kFragBytes, DK_OFF = (K_FR + VT_FR) * kFragBytes, DVT_OFF = DK_OFF + K_FR * kFragBytes;

    const int qt = blockIdx.x, bh = blockIdx.y, b = bh / p.H, h = bh % p.H;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int row0 = qt * kBlockM + wave * 32;   // first query row of this wavefront
    const int row = row0 + j;                    // this lane's query row (lanes l and l^32 share it)

    int kv_len = p.Lkv;
    if (p.key_lens) { const int kl = p.key_lens[b]; kv_len = kl < kv_len ? (kl < 0 ? 0 : kl) : kv_len; }
    int n_tiles = (kv_len + kBlockN - 1) / kBlockN;
    if (p.causal) { const int lim = (qt * kBlockM + kBlockM + kBlockN - 1) / kBlockN; n_tiles = n_tiles < lim ? n_tiles : lim; }

    const char* kv_lane = p.kv + (size_t)bh * p.n_tiles * TILE_BYTES + lane * 16;
    if (n_tiles > 0) load_tile_to_lds(kv_lane, smem, wave, TILE_FR);

    // Q (and dQ) fragments: B operand of S^T = K Q^T; lane holds Q[row][16 c + 8 hh .. +7]
    V8 qf[NC], tqf[JVP ? NC : 1];
    {
        const int64_t off = (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + (int64_t)row * p.q_sl + 8 * hh;
        const T* qp = reinterpret_cast<const T*>(p.q) + off;
        const T* tqp = reinterpret_cast<const T*>(p.tq) + off;
        const bool live = row < p.Lq;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            V8 z = {0, 0, 0, 0, 0, 0, 0, 0};
            qf[c] = live ? *reinterpret_cast<const V8*>(qp + 16 * c) : z;
            if (JVP) tqf[c] = live ? *reinterpret_cast<const V8*>(tqp + 16 * c) : z;
        }
    }

    f32x16 acc[NDB], acct[JVP ? NDB : 1];
#pragma unroll
    for (int i = 0; i < NDB; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) { acc[i][e] = 0.f; if (JVP) acct[i][e] = 0.f; }
    }
    float m_run = -INFINITY;   // running row max of the scaled scores in the log2 domain (same in lanes l, l^32)
    float l_run = 0.f;         // this lane's partial row sum of p   (the two half-rows are added in the epilogue)
    float r_run = 0.f;         // this lane's partial row sum of H

    for (int t = 0; t < n_tiles; ++t) {
        const char* buf = smem + (t & 1) * TILE_BYTES;
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's share of tile t has landed
        __syncthreads();                      // everyone's share landed; everyone is done with the other buffer
        if (t + 1 < n_tiles) load_tile_to_lds(kv_lane + (size_t)(t + 1) * TILE_BYTES, smem + ((t + 1) & 1) * TILE_BYTES, wave, TILE_FR);

        // ---- stage 1: S^T = K Q^T, dS^T = K dQ^T + dK Q^T for 2 blocks of 32 keys ----
        f32x16 s[2], ds[JVP ? 2 : 1];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) { s[kb][e] = 0.f; if (JVP) ds[kb][e] = 0.f; }
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const V8 kf = *reinterpret_cast<const V8*>(buf + (kb * NC + c) * kFragBytes + lane * 16);
                s[kb] = mfma32(kf, qf[c], s[kb]);
                if (JVP) ds[kb] = mfma32(kf, tqf[c], ds[kb]);
                if (FULL) {
                    const V8 dkf = *reinterpret_cast<const V8*>(buf + DK_OFF + (kb * NC + c) * kFragBytes + lane * 16);
                    ds[kb] = mfma32(dkf, qf[c], ds[kb]);
                }
            }
        }

        // ---- stage 2: online softmax on this lane's query column (32 of the tile's 64 keys) ----
        // register e of block kb is key  t*64 + 32 kb + 8 (e/4) + 4 hh + e%4
        const int key0 = t * kBlockN + 4 * hh;
        const bool need_mask = (t * kBlockN + kBlockN > kv_len) || (p.causal && (t * kBlockN + kBlockN - 1 > row0));
        if (need_mask) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = key0 + 32 * kb + 8 * (e >> 2) + (e & 3);
                    const bool ok = key < kv_len && (!p.causal || key <= row);
                    s[kb][e] = ok ? s[kb][e] : -INFINITY;
                }
            }
        }
        float mx = s[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[kb][e]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx * p.scale_log2);
        if (__any(m_new > m_run)) {   // wavefront-uniform: skip the rescale when no row's max moved (alpha == 1 exactly)
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= alpha;
            r_run *= alpha;
#pragma unroll
            for (int i = 0; i < NDB; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) { acc[i][e] *= alpha; if (JVP) acct[i][e] *= alpha; }
            }
            m_run = m_new;
        }
        V8 pf[4], hf[JVP ? 4 : 1];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kb][e], p.scale_log2, -m_run));
                l_run += pv;
                pf[2 * kb + (e >> 3)][e & 7] = (T)pv;
                if (JVP) {
                    const float hv = pv * (ds[kb][e] * p.sm_scale);
                    r_run += hv;
                    hf[2 * kb + (e >> 3)][e & 7] = (T)hv;
                }
            }
        }

        // ---- stage 3: O^T += V^T P^T ;  T^T += V^T H^T + dV^T P^T ----
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                const V8 vf = *reinterpret_cast<const V8*>(buf + VT_OFF + (db * 4 + c) * kFragBytes + lane * 16);
                acc[db] = mfma32(vf, pf[c], acc[db]);
                if (JVP) acct[db] = mfma32(vf, hf[c], acct[db]);
                if (FULL) {
                    const V8 dvf = *reinterpret_cast<const V8*>(buf + DVT_OFF + (db * 4 + c) * kFragBytes + lane * 16);
                    acct[db] = mfma32(dvf, pf[c], acct[db]);
                }
            }
        }
    }

    // ---- epilogue: O = acc / l ; dO = (T - r O) / l ; LSE = (m + log2 l) ln 2 ----
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float r_tot = r_run + __shfl_xor(r_run, 32);
    const float inv_l = 1.0f / l_tot;
    const float r_over_l = r_tot * inv_l;
    if (row < p.Lq) {
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
                        const float of = acc[db][4 * g + r] * inv_l;
                        ov[r] = (T)of;
                        if (JVP) tov[r] = (T)((acct[db][4 * g + r] - r_over_l * acc[db][4 * g + r]) * inv_l);
                    }
                    *reinterpret_cast<V4*>(op + d) = ov;
                    if (JVP) *reinterpret_cast<V4*>(top + d) = tov;
                }
            }
        }
        if (p.lse && hh == 0) p.lse[(int64_t)bh * p.Lq + row] = (m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
    }
}

// ------------------------------------------------------------------------------------------------ host
typedef void (*attn_kernel_t)(const AttnParams);

template <typename T, int DQK, int DV>
attn_kernel_t pick_mode(int mode) {
    switch (mode) {
        case MODE_FWD: return attn_fwd_jvp_kernel<T, DQK, DV, MODE_FWD>;
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
    switch (dqk) {
        case 16: return pick_dv<T, 16>(dv, mode);
        case 32: return pick_dv<T, 32>(dv, mode);
        case 64: return pick_dv<T, 64>(dv, mode);
        case 128: return pick_dv<T, 128>(dv, mode);
        default: return nullptr;
    }
}

bool head_dim_ok(int d) { return d == 16 || d == 32 || d == 64 || d == 128; }
bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }
bool strides_ok(const int64_t* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }

int mode_of(const cosmos_attn_desc* d) {
    if (!d->tq && !d->tk && !d->tv) return MODE_FWD;
    if (d->tq && !d->tk && !d->tv) return MODE_JVP_Q;
    if (d->tq && d->tk && d->tv) return MODE_JVP_FULL;
    return -1;
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
    if (d->d_qk == 256 || d->d_v == 256) return COSMOS_ATTN_UNSUPPORTED;
    if (!head_dim_ok(d->d_qk) || !head_dim_ok(d->d_v)) return COSMOS_ATTN_BAD_SHAPE;
    if (d->causal && d->Lq != d->Lkv) return COSMOS_ATTN_BAD_SHAPE;
    if (d->causal && d->key_lens) return COSMOS_ATTN_BAD_ARG;
    if (!aligned16(d->q) || !aligned16(d->k) || !aligned16(d->v) || !aligned16(d->o)) return COSMOS_ATTN_BAD_STRIDE;
    if ((d->tq && !aligned16(d->tq)) || (d->tk && !aligned16(d->tk)) || (d->tv && !aligned16(d->tv)) ||
        (d->to && !aligned16(d->to)))
        return COSMOS_ATTN_BAD_STRIDE;
    if (!strides_ok(d->q_stride) || !strides_ok(d->k_stride) || !strides_ok(d->v_stride) || !strides_ok(d->o_stride))
        return COSMOS_ATTN_BAD_STRIDE;
    if ((int64_t)d->B * d->H > 65535) return COSMOS_ATTN_BAD_SHAPE;   // grid.y limit
    return COSMOS_ATTN_OK;
}

size_t tile_bytes_of(const cosmos_attn_desc* d) {
    const TileGeom g(d->d_qk, d->d_v, mode_of(d) == MODE_JVP_FULL);
    return (size_t)g.tile_frags * kFragBytes;
}
int n_tiles_of(const cosmos_attn_desc* d) { return (d->Lkv + kBlockN - 1) / kBlockN; }

}  // namespace

extern "C" {

COSMOS_ATTN_API int cosmos_attn_abi_version(void) { return COSMOS_ATTN_ABI_VERSION; }

COSMOS_ATTN_API const char* cosmos_attn_status_string(int status) {
    switch (status) {
        case COSMOS_ATTN_OK: return "ok";
        case COSMOS_ATTN_BAD_ARG: return "bad argument (null pointer, non-positive size, ABI version, or tangent set other than none / q only / q,k,v)";
        case COSMOS_ATTN_BAD_SHAPE: return "bad shape (head dims must be in {16,32,64,128}; causal needs Lq == Lkv; B*H <= 65535)";
        case COSMOS_ATTN_BAD_STRIDE: return "bad stride or alignment (16-byte aligned bases, strides multiple of 8 elements, innermost stride 1)";
        case COSMOS_ATTN_UNSUPPORTED: return "unsupported dtype or head dim (bf16/fp16, head dim <= 128)";
        case COSMOS_ATTN_WORKSPACE_TOO_SMALL: return "workspace too small or null";
        case COSMOS_ATTN_LAUNCH_FAILED: return "kernel launch failed";
        default: return "unknown status";
    }
}

COSMOS_ATTN_API size_t cosmos_attn_workspace_bytes(const cosmos_attn_desc* d) {
    if (validate(d) != COSMOS_ATTN_OK) return 0;
    return (size_t)d->B * d->H * n_tiles_of(d) * tile_bytes_of(d);
}

COSMOS_ATTN_API int cosmos_attn_pack_kv(const cosmos_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    const int st = validate(d);
    if (st != COSMOS_ATTN_OK) return st;
    if (!workspace || workspace_bytes < cosmos_attn_workspace_bytes(d) || !aligned16(workspace)) return COSMOS_ATTN_WORKSPACE_TOO_SMALL;
    PackParams pp;
    const bool full = mode_of(d) == MODE_JVP_FULL;
    pp.k = (const uint16_t*)d->k; pp.v = (const uint16_t*)d->v;
    pp.tk = full ? (const uint16_t*)d->tk : nullptr; pp.tv = full ? (const uint16_t*)d->tv : nullptr;
    pp.k_sb = d->k_stride[0]; pp.k_sh = d->k_stride[1]; pp.k_sl = d->k_stride[2];
    pp.v_sb = d->v_stride[0]; pp.v_sh = d->v_stride[1]; pp.v_sl = d->v_stride[2];
    pp.out = (uint4*)workspace;
    pp.H = d->H; pp.Lkv = d->Lkv; pp.dqk = d->d_qk; pp.dv = d->d_v; pp.n_tiles = n_tiles_of(d);
    hipLaunchKernelGGL(pack_kv_kernel, dim3(pp.n_tiles, d->B * d->H), dim3(kThreads), 0, (hipStream_t)stream, pp);
    return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
}

COSMOS_ATTN_API int cosmos_attn_run(const cosmos_attn_desc* d, const void* workspace, size_t workspace_bytes, void* stream) {
    const int st = validate(d);
    if (st != COSMOS_ATTN_OK) return st;
    if (!workspace || workspace_bytes < cosmos_attn_workspace_bytes(d) || !aligned16(workspace)) return COSMOS_ATTN_WORKSPACE_TOO_SMALL;
    const int mode = mode_of(d);
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
    const size_t lds = 2 * tile_bytes_of(d);
    if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
        (void)hipGetLastError();
        return COSMOS_ATTN_LAUNCH_FAILED;
    }
    const int n_qt = (d->Lq + kBlockM - 1) / kBlockM;
    hipLaunchKernelGGL(fn, dim3(n_qt, d->B * d->H), dim3(kThreads), lds, (hipStream_t)stream, ap);
    return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
}

COSMOS_ATTN_API int cosmos_attn_fwd_jvp(const cosmos_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    const int st = cosmos_attn_pack_kv(d, workspace, workspace_bytes, stream);
    if (st != COSMOS_ATTN_OK) return st;
    return cosmos_attn_run(d, workspace, workspace_bytes, stream);
}

}  // extern "C"
