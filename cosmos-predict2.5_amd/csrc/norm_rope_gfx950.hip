// Fused per-head RMSNorm + rotary position embedding (+ their forward-mode tangents) for gfx950: kernel and C ABI.
//
// The step immediately before the attention call in the DiT's `Attention.compute_qkv`
// (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:405-415):
//     q = q_norm(q); k = k_norm(k)                      te.pytorch.RMSNorm(head_dim, eps=1e-6)   (:350-356)
//     q = apply_rotary_pos_emb(q, rope_emb, "bshd")     self-attention only                       (:409-414)
// with rope_emb the angles [L, 1, 1, D] = cat([t, h, w] * 2) built by the positional embedding (:648-658).
// Restated here from the published semantics of the two Transformer Engine ops (the library itself is not part of
// the reference checkout):
//     n = x * rsqrt(mean_d(x^2) + eps) * g                  rounded to the 16-bit element type (RMSNorm's output)
//     y[j]       = n[j] cos(a[j])       - n[j + D/2] sin(a[j])              j <  D/2      (rotate-half form,
//     y[j + D/2] = n[j + D/2] cos(a[j + D/2]) + n[j] sin(a[j + D/2])        j <  D/2       not interleaved)
// and, for a tangent dx of x (the JVP the distillation path needs for q, k as functions of the block input):
//     dn = g * (dx * r - x * r^3 * mean_d(x * dx)),   r = rsqrt(mean_d(x^2) + eps);      dy = rope(dn)  (rope is linear)
// One pass over x (and dx) -- every byte read once and written once -- instead of two kernels per tensor (four with
// tangents) with a 16-bit round trip through HBM between them.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "cosmos_attn_hip.h"

namespace {
// The tensors of these kernels are touched once: loads and stores that do not displace anything in the caches.
typedef unsigned nr_u32x2 __attribute__((ext_vector_type(2)));
#ifndef NR_PLAIN
__device__ __forceinline__ uint2 stream_load(const uint16_t* p) {
    const nr_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const nr_u32x2*>(p));
    return make_uint2(v[0], v[1]);
}
__device__ __forceinline__ void stream_store(uint16_t* p, uint2 v) {
    nr_u32x2 w; w[0] = v.x; w[1] = v.y;
    __builtin_nontemporal_store(w, reinterpret_cast<nr_u32x2*>(p));
}
#else
__device__ __forceinline__ uint2 stream_load(const uint16_t* p) { return *reinterpret_cast<const uint2*>(p); }
__device__ __forceinline__ void stream_store(uint16_t* p, uint2 v) { *reinterpret_cast<uint2*>(p) = v; }
#endif


constexpr int kThreads = 256;

struct NormRopeParams {
    const uint16_t *x, *tx;      // tx may be null
    uint16_t *y, *ty;
    const float* weight;         // [D] or null (ones)
    const float* angles;         // [S, D] or null (no rotation)
    int64_t x_sb, x_ss, x_sh, y_sb, y_ss, y_sh;
    int B, S, H, D;
    float eps;
    int heads_per_unit;          // heads served by one thread group: a multiple of kHeadsPerStep
    int head_groups;             // ceil(H / heads_per_unit)
    int64_t units;               // B * S * head_groups: one per thread group
};

template <bool BF16>
__device__ __forceinline__ void unpack4(const uint2& v, float* f) {
    if (BF16) {
        f[0] = __builtin_bit_cast(float, v.x << 16); f[1] = __builtin_bit_cast(float, v.x & 0xFFFF0000u);
        f[2] = __builtin_bit_cast(float, v.y << 16); f[3] = __builtin_bit_cast(float, v.y & 0xFFFF0000u);
    } else {
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        const half2_t a = __builtin_bit_cast(half2_t, v.x), b = __builtin_bit_cast(half2_t, v.y);
        f[0] = (float)a[0]; f[1] = (float)a[1]; f[2] = (float)b[0]; f[3] = (float)b[1];
    }
}
template <bool BF16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    if (BF16) {
        typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
        bf2_t r; r[0] = (__bf16)lo; r[1] = (__bf16)hi;
        return __builtin_bit_cast(uint32_t, r);
    } else {
        typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
        half2_t r; r[0] = (_Float16)lo; r[1] = (_Float16)hi;
        return __builtin_bit_cast(uint32_t, r);
    }
}
template <bool BF16>
__device__ __forceinline__ uint2 pack4(const float* f) {
    return make_uint2(pack2<BF16>(f[0], f[1]), pack2<BF16>(f[2], f[3]));
}
// round four values to the 16-bit type and back (the rounding point of a 16-bit intermediate tensor)
template <bool BF16>
__device__ __forceinline__ void round4(float* f) {
    const uint2 r = pack4<BF16>(f);
    unpack4<BF16>(r, f);
}

// Sum over the TPR (2, 4, 8, 16 or 32) adjacent lanes of a thread group, result in every lane, by data-parallel-primitive
// lane permutations (no LDS traffic): swap within pairs, swap pairs within quads, mirror within 8, mirror within 16.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
    return v + __builtin_bit_cast(float, moved);
}
template <int TPR>
__device__ __forceinline__ float group_sum(float v) {
    if (TPR >= 2) v = dpp_add<0xB1>(v);    // quad_perm [1, 0, 3, 2]
    if (TPR >= 4) v = dpp_add<0x4E>(v);    // quad_perm [2, 3, 0, 1]
    if (TPR >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
    if (TPR >= 16) v = dpp_add<0x140>(v);  // row_mirror
    if (TPR >= 32) v += __shfl_xor(v, 16);  // the other row of 16 lanes (head dim 256 only)
    return v;
}

// The kernel is bound by vector-ALU issue as much as by HBM (a 64-lane instruction takes four cycles on a 16-lane SIMD;
// at one pass over 16-bit data there is room for about 25 instructions per element pair before arithmetic, not memory,
// sets the time), so the work per element is kept minimal: the element type is a template parameter, the sines and
// cosines are shared by all heads of a position, and the rotation needs no exchange between lanes.
//
// TPR = D / 8 threads per row (2, 4, 8, 16 or 32: a power of two that divides the wavefront).  Thread `part` holds both
// members of four rotation pairs: elements [4 part, 4 part + 4) and [D/2 + 4 part, D/2 + 4 part + 4); the row statistics
// are summed over the TPR lanes by lane permutations.  A thread group serves `heads_per_unit` consecutive heads of one
// (batch, position), kHeadsPerStep at a time; the loads of a step are issued before their first use.
constexpr int kHeadsPerStep = 4;
constexpr int kMaxHeadsPerUnit = 16;

template <int TPR, bool TANGENT, bool BF16>
__global__ void __launch_bounds__(kThreads) norm_rope_kernel(const NormRopeParams p) {
    constexpr int D = TPR * 8;
    constexpr int HS = kHeadsPerStep;
    const int64_t unit = (int64_t)blockIdx.x * (kThreads / TPR) + threadIdx.x / TPR;
    const int part = threadIdx.x % TPR;
    const bool live = unit < p.units;
    // unit -> (b, s, head group), head group fastest (the [B, S, H, D] order of the projections' output)
    const int64_t uu = live ? unit : 0;
    const int h0 = (int)(uu % p.head_groups) * p.heads_per_unit;
    const int s = (int)((uu / p.head_groups) % p.S);
    const int b = (int)(uu / ((int64_t)p.head_groups * p.S));
    const int n_heads = live ? min(p.heads_per_unit, p.H - h0) : 0;   // heads this unit stores
    const int64_t xo = (int64_t)b * p.x_sb + (int64_t)s * p.x_ss + (int64_t)h0 * p.x_sh + 4 * part;
    const int64_t yo = (int64_t)b * p.y_sb + (int64_t)s * p.y_ss + (int64_t)h0 * p.y_sh + 4 * part;
    const uint16_t* xp = p.x + xo;
    const uint16_t* txp = TANGENT ? p.tx + xo : nullptr;
    uint16_t* yp = p.y + yo;
    uint16_t* typ = TANGENT ? p.ty + yo : nullptr;

    float g[8], sn[8], cs[8];   // [0, 4): the lower-half elements, [4, 8): their partners in the upper half
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        g[i] = p.weight ? p.weight[4 * part + i] : 1.0f;
        g[4 + i] = p.weight ? p.weight[D / 2 + 4 * part + i] : 1.0f;
    }
    if (p.angles) {
        const float4 a0 = *reinterpret_cast<const float4*>(p.angles + (int64_t)s * D + 4 * part);
        const float4 a1 = *reinterpret_cast<const float4*>(p.angles + (int64_t)s * D + D / 2 + 4 * part);
        const float lo[4] = {a0.x, a0.y, a0.z, a0.w}, hi[4] = {a1.x, a1.y, a1.z, a1.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) sincosf(lo[i], &sn[i], &cs[i]);
        // the DiT's table repeats the half vector (both members of a pair turn by the same angle): then one evaluation
        // serves both; any other table gets its own
        if (lo[0] == hi[0] && lo[1] == hi[1] && lo[2] == hi[2] && lo[3] == hi[3]) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { sn[4 + i] = sn[i]; cs[4 + i] = cs[i]; }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) sincosf(hi[i], &sn[4 + i], &cs[4 + i]);
        }
    }

    // the trip count is the same for every lane (the lane permutations need all lanes of a thread group): a unit whose
    // head range is cut short re-reads its first head in the surplus slots and stores nothing for them
    for (int hb = 0; hb < p.heads_per_unit; hb += HS) {
        uint2 xlo[HS], xhi[HS], dlo[HS], dhi[HS];
#pragma unroll
        for (int i = 0; i < HS; ++i) {
            const int64_t o = (hb + i < n_heads ? hb + i : 0) * p.x_sh;
            xlo[i] = stream_load(xp + o);
            xhi[i] = stream_load(xp + o + D / 2);
            if (TANGENT) {
                dlo[i] = stream_load(txp + o);
                dhi[i] = stream_load(txp + o + D / 2);
            }
        }
#pragma unroll
        for (int hh = 0; hh < HS; ++hh) {
            float x[8], dx[8];
            unpack4<BF16>(xlo[hh], x);
            unpack4<BF16>(xhi[hh], x + 4);
            if (TANGENT) { unpack4<BF16>(dlo[hh], dx); unpack4<BF16>(dhi[hh], dx + 4); }
            float ss = 0.f, sd = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) { ss += x[i] * x[i]; if (TANGENT) sd += x[i] * dx[i]; }
            ss = group_sum<TPR>(ss);
            if (TANGENT) sd = group_sum<TPR>(sd);
            const float r = rsqrtf(ss * (1.0f / D) + p.eps);
            const float c3 = TANGENT ? r * r * r * sd * (1.0f / D) : 0.f;

            float n[8], dn[8], y[8], dy[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                n[i] = x[i] * r * g[i];
                if (TANGENT) dn[i] = g[i] * (dx[i] * r - x[i] * c3);
            }
            // RMSNorm's output is a 16-bit tensor in the reference: keep that rounding point
            round4<BF16>(n); round4<BF16>(n + 4);
            if (TANGENT) { round4<BF16>(dn); round4<BF16>(dn + 4); }
            if (p.angles) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // rotate_half: the lower half takes -n[j + D/2], the upper half +n[j - D/2]
                    y[i] = n[i] * cs[i] - n[4 + i] * sn[i];
                    y[4 + i] = n[4 + i] * cs[4 + i] + n[i] * sn[4 + i];
                    if (TANGENT) {
                        dy[i] = dn[i] * cs[i] - dn[4 + i] * sn[i];
                        dy[4 + i] = dn[4 + i] * cs[4 + i] + dn[i] * sn[4 + i];
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) { y[i] = n[i]; if (TANGENT) dy[i] = dn[i]; }
            }
            if (hb + hh < n_heads) {
                const int64_t o = (hb + hh) * p.y_sh;
                stream_store(yp + o, pack4<BF16>(y));
                stream_store(yp + o + D / 2, pack4<BF16>(y + 4));
                if (TANGENT) {
                    stream_store(typ + o, pack4<BF16>(dy));
                    stream_store(typ + o + D / 2, pack4<BF16>(dy + 4));
                }
            }
        }
    }
}

typedef void (*norm_rope_kernel_t)(const NormRopeParams);

template <bool TANGENT, bool BF16>
norm_rope_kernel_t pick(int d) {
    switch (d) {
        case 16: return norm_rope_kernel<2, TANGENT, BF16>;
        case 32: return norm_rope_kernel<4, TANGENT, BF16>;
        case 64: return norm_rope_kernel<8, TANGENT, BF16>;
        case 128: return norm_rope_kernel<16, TANGENT, BF16>;
        case 256: return norm_rope_kernel<32, TANGENT, BF16>;
        default: return nullptr;
    }
}

// ------------------------------------------------------------------------------------------------ reverse mode
// Given dy = dL/dy:   dn = R^T dy (the rotation by the negated angles; the 16-bit rounding of n is passed straight through)
//                     dx = r (g dn) - x r^3 mean_d(x g dn),      dweight[j] = sum over rows of dn[j] x[j] r.
// Same thread layout as the forward kernel.  dweight: every thread sums its heads, the block's thread groups are added
// in a fixed order through LDS, and each block writes one row of partial sums; norm_rope_dweight_kernel adds the rows
// (fixed order again: the result is bitwise reproducible, no atomics).
struct NormRopeBwdParams {
    const uint16_t *x, *dy;
    uint16_t* dx;
    const float* weight;         // [D] or null (ones)
    const float* angles;         // [S, D] or null (no rotation)
    float* partials;             // [blocks, D] or null (no dweight wanted)
    int64_t x_sb, x_ss, x_sh, g_sb, g_ss, g_sh, o_sb, o_ss, o_sh;   // strides of x, dy, dx
    int B, S, H, D;
    float eps;
    int heads_per_unit, head_groups;
    int64_t units;
};

template <int TPR, bool BF16>
__global__ void __launch_bounds__(kThreads) norm_rope_bwd_kernel(const NormRopeBwdParams p) {
    constexpr int D = TPR * 8;
    constexpr int HS = kHeadsPerStep;
    constexpr int UPB = kThreads / TPR;          // units (thread groups) per block
    __shared__ float red[UPB * D];               // 8 KB for every D
    const int ug = threadIdx.x / TPR;
    const int64_t unit = (int64_t)blockIdx.x * UPB + ug;
    const int part = threadIdx.x % TPR;
    const bool live = unit < p.units;
    const int64_t uu = live ? unit : 0;
    const int h0 = (int)(uu % p.head_groups) * p.heads_per_unit;
    const int s = (int)((uu / p.head_groups) % p.S);
    const int b = (int)(uu / ((int64_t)p.head_groups * p.S));
    const int n_heads = live ? min(p.heads_per_unit, p.H - h0) : 0;
    const uint16_t* xp = p.x + (int64_t)b * p.x_sb + (int64_t)s * p.x_ss + (int64_t)h0 * p.x_sh + 4 * part;
    const uint16_t* gp = p.dy + (int64_t)b * p.g_sb + (int64_t)s * p.g_ss + (int64_t)h0 * p.g_sh + 4 * part;
    uint16_t* op = p.dx + (int64_t)b * p.o_sb + (int64_t)s * p.o_ss + (int64_t)h0 * p.o_sh + 4 * part;

    float g[8], sn[8], cs[8], wacc[8];   // [0, 4): the lower-half elements, [4, 8): their partners in the upper half
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        g[i] = p.weight ? p.weight[4 * part + i] : 1.0f;
        g[4 + i] = p.weight ? p.weight[D / 2 + 4 * part + i] : 1.0f;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) wacc[i] = 0.f;
    if (p.angles) {
        const float4 a0 = *reinterpret_cast<const float4*>(p.angles + (int64_t)s * D + 4 * part);
        const float4 a1 = *reinterpret_cast<const float4*>(p.angles + (int64_t)s * D + D / 2 + 4 * part);
        const float lo[4] = {a0.x, a0.y, a0.z, a0.w}, hi[4] = {a1.x, a1.y, a1.z, a1.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) sincosf(lo[i], &sn[i], &cs[i]);
        if (lo[0] == hi[0] && lo[1] == hi[1] && lo[2] == hi[2] && lo[3] == hi[3]) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { sn[4 + i] = sn[i]; cs[4 + i] = cs[i]; }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) sincosf(hi[i], &sn[4 + i], &cs[4 + i]);
        }
    }

    for (int hb = 0; hb < p.heads_per_unit; hb += HS) {
        uint2 xlo[HS], xhi[HS], glo[HS], ghi[HS];
#pragma unroll
        for (int i = 0; i < HS; ++i) {
            const int hsel = hb + i < n_heads ? hb + i : 0;   // surplus slots re-read the first head, store nothing
            xlo[i] = stream_load(xp + hsel * p.x_sh);
            xhi[i] = stream_load(xp + hsel * p.x_sh + D / 2);
            glo[i] = stream_load(gp + hsel * p.g_sh);
            ghi[i] = stream_load(gp + hsel * p.g_sh + D / 2);
        }
#pragma unroll
        for (int hh = 0; hh < HS; ++hh) {
            float x[8], dy[8], dn[8];
            unpack4<BF16>(xlo[hh], x);
            unpack4<BF16>(xhi[hh], x + 4);
            unpack4<BF16>(glo[hh], dy);
            unpack4<BF16>(ghi[hh], dy + 4);
            if (p.angles) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // transpose of  y_lo = n_lo c_lo - n_hi s_lo,  y_hi = n_hi c_hi + n_lo s_hi
                    dn[i] = dy[i] * cs[i] + dy[4 + i] * sn[4 + i];
                    dn[4 + i] = dy[4 + i] * cs[4 + i] - dy[i] * sn[i];
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) dn[i] = dy[i];
            }
            float ss = 0.f, sg = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) { ss += x[i] * x[i]; sg += x[i] * (g[i] * dn[i]); }
            ss = group_sum<TPR>(ss);
            sg = group_sum<TPR>(sg);
            const float r = rsqrtf(ss * (1.0f / D) + p.eps);
            const float c3 = r * r * r * sg * (1.0f / D);
            float dx[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) dx[i] = g[i] * dn[i] * r - x[i] * c3;
            if (hb + hh < n_heads) {
#pragma unroll
                for (int i = 0; i < 8; ++i) wacc[i] += dn[i] * x[i] * r;
                uint16_t* o = op + (int64_t)(hb + hh) * p.o_sh;
                stream_store(o, pack4<BF16>(dx));
                stream_store(o + D / 2, pack4<BF16>(dx + 4));
            }
        }
    }
    if (p.partials) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            red[ug * D + 4 * part + i] = wacc[i];
            red[ug * D + D / 2 + 4 * part + i] = wacc[4 + i];
        }
        __syncthreads();
        if (threadIdx.x < D) {
            float t = 0.f;
            for (int u = 0; u < UPB; ++u) t += red[u * D + threadIdx.x];
            p.partials[(int64_t)blockIdx.x * D + threadIdx.x] = t;
        }
    }
}

// dweight[j] = sum over `rows` of partials[row][j]: one block per channel, fixed order within a thread and across threads
__global__ void __launch_bounds__(kThreads) norm_rope_dweight_kernel(const float* partials, float* dweight, int64_t rows, int D) {
    __shared__ float red[kThreads];
    const int j = blockIdx.x;
    float t = 0.f;
    for (int64_t r = threadIdx.x; r < rows; r += kThreads) t += partials[r * D + j];
    red[threadIdx.x] = t;
    __syncthreads();
    for (int w = kThreads / 2; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) dweight[j] = red[0];
}

typedef void (*norm_rope_bwd_kernel_t)(const NormRopeBwdParams);

template <bool BF16>
norm_rope_bwd_kernel_t pick_bwd(int d) {
    switch (d) {
        case 16: return norm_rope_bwd_kernel<2, BF16>;
        case 32: return norm_rope_bwd_kernel<4, BF16>;
        case 64: return norm_rope_bwd_kernel<8, BF16>;
        case 128: return norm_rope_bwd_kernel<16, BF16>;
        case 256: return norm_rope_bwd_kernel<32, BF16>;
        default: return nullptr;
    }
}

// How the rows are dealt out to thread groups: as many heads per group as there are (up to 16) while that leaves enough
// groups to fill the chip.
struct UnitPlan { int heads_per_unit, head_groups; int64_t units, blocks; };
UnitPlan plan_units(int B, int S, int H, int D) {
    UnitPlan u;
    const int units_per_block = kThreads / (D / 8);
    const int64_t enough_units = (int64_t)units_per_block * 4096;
    u.heads_per_unit = kHeadsPerStep;
    while (u.heads_per_unit < kMaxHeadsPerUnit && u.heads_per_unit < H &&
           (int64_t)B * S * ((H + 2 * u.heads_per_unit - 1) / (2 * u.heads_per_unit)) >= enough_units)
        u.heads_per_unit *= 2;
    u.head_groups = (H + u.heads_per_unit - 1) / u.heads_per_unit;
    u.units = (int64_t)B * S * u.head_groups;
    u.blocks = (u.units + units_per_block - 1) / units_per_block;
    return u;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }
bool strides_ok(const int64_t* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }

}  // namespace

extern "C" {

COSMOS_ATTN_API int cosmos_norm_rope(const cosmos_norm_rope_desc* d, void* stream) {
    if (!d || d->abi_version != COSMOS_ATTN_ABI_VERSION) return COSMOS_ATTN_BAD_ARG;
    if (d->B <= 0 || d->S <= 0 || d->H <= 0) return COSMOS_ATTN_BAD_ARG;
    if (!d->x || !d->y || (d->tx != nullptr) != (d->ty != nullptr)) return COSMOS_ATTN_BAD_ARG;
    if (!(d->eps >= 0.f)) return COSMOS_ATTN_BAD_ARG;
    if (d->dtype != COSMOS_ATTN_BF16 && d->dtype != COSMOS_ATTN_FP16) return COSMOS_ATTN_UNSUPPORTED;
    if (d->D != 16 && d->D != 32 && d->D != 64 && d->D != 128 && d->D != 256) return COSMOS_ATTN_BAD_SHAPE;
    if (!aligned16(d->x) || !aligned16(d->y) || (d->tx && (!aligned16(d->tx) || !aligned16(d->ty)))) return COSMOS_ATTN_BAD_STRIDE;
    if (d->angles && !aligned16(d->angles)) return COSMOS_ATTN_BAD_STRIDE;
    if (!strides_ok(d->x_stride) || !strides_ok(d->y_stride)) return COSMOS_ATTN_BAD_STRIDE;
    NormRopeParams p;
    p.x = (const uint16_t*)d->x; p.tx = (const uint16_t*)d->tx; p.y = (uint16_t*)d->y; p.ty = (uint16_t*)d->ty;
    p.weight = d->weight; p.angles = d->angles;
    p.x_sb = d->x_stride[0]; p.x_ss = d->x_stride[1]; p.x_sh = d->x_stride[2];
    p.y_sb = d->y_stride[0]; p.y_ss = d->y_stride[1]; p.y_sh = d->y_stride[2];
    p.B = d->B; p.S = d->S; p.H = d->H; p.D = d->D;
    p.eps = d->eps;
    const UnitPlan u = plan_units(d->B, d->S, d->H, d->D);
    p.heads_per_unit = u.heads_per_unit; p.head_groups = u.head_groups; p.units = u.units;
    const int64_t blocks = u.blocks;
    if (blocks > 0x7FFFFFFF) return COSMOS_ATTN_BAD_SHAPE;
    const bool bf16 = d->dtype == COSMOS_ATTN_BF16;
    norm_rope_kernel_t fn = d->tx ? (bf16 ? pick<true, true>(d->D) : pick<true, false>(d->D))
                                  : (bf16 ? pick<false, true>(d->D) : pick<false, false>(d->D));
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, p);
    return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED;
}

static int validate_norm_rope_bwd(const cosmos_norm_rope_bwd_desc* d) {
    if (!d || d->abi_version != COSMOS_ATTN_ABI_VERSION) return COSMOS_ATTN_BAD_ARG;
    if (d->B <= 0 || d->S <= 0 || d->H <= 0) return COSMOS_ATTN_BAD_ARG;
    if (!d->x || !d->dy || !d->dx) return COSMOS_ATTN_BAD_ARG;
    if (!(d->eps >= 0.f)) return COSMOS_ATTN_BAD_ARG;
    if (d->dtype != COSMOS_ATTN_BF16 && d->dtype != COSMOS_ATTN_FP16) return COSMOS_ATTN_UNSUPPORTED;
    if (d->D != 16 && d->D != 32 && d->D != 64 && d->D != 128 && d->D != 256) return COSMOS_ATTN_BAD_SHAPE;
    if (!aligned16(d->x) || !aligned16(d->dy) || !aligned16(d->dx)) return COSMOS_ATTN_BAD_STRIDE;
    if (d->angles && !aligned16(d->angles)) return COSMOS_ATTN_BAD_STRIDE;
    if (!strides_ok(d->x_stride) || !strides_ok(d->dy_stride) || !strides_ok(d->dx_stride)) return COSMOS_ATTN_BAD_STRIDE;
    if (plan_units(d->B, d->S, d->H, d->D).blocks > 0x7FFFFFFF) return COSMOS_ATTN_BAD_SHAPE;
    return COSMOS_ATTN_OK;
}

COSMOS_ATTN_API size_t cosmos_norm_rope_bwd_workspace_bytes(const cosmos_norm_rope_bwd_desc* d) {
    if (validate_norm_rope_bwd(d) != COSMOS_ATTN_OK || !d->dweight) return 0;
    return (size_t)plan_units(d->B, d->S, d->H, d->D).blocks * d->D * sizeof(float);
}

COSMOS_ATTN_API int cosmos_norm_rope_bwd(const cosmos_norm_rope_bwd_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    const int st = validate_norm_rope_bwd(d);
    if (st != COSMOS_ATTN_OK) return st;
    const UnitPlan u = plan_units(d->B, d->S, d->H, d->D);
    const size_t need = d->dweight ? (size_t)u.blocks * d->D * sizeof(float) : 0;
    if (need && (!workspace || workspace_bytes < need)) return COSMOS_ATTN_WORKSPACE_TOO_SMALL;
    if (need && !aligned16(workspace)) return COSMOS_ATTN_BAD_STRIDE;
    NormRopeBwdParams p;
    p.x = (const uint16_t*)d->x; p.dy = (const uint16_t*)d->dy; p.dx = (uint16_t*)d->dx;
    p.weight = d->weight; p.angles = d->angles;
    p.partials = d->dweight ? (float*)workspace : nullptr;
    p.x_sb = d->x_stride[0]; p.x_ss = d->x_stride[1]; p.x_sh = d->x_stride[2];
    p.g_sb = d->dy_stride[0]; p.g_ss = d->dy_stride[1]; p.g_sh = d->dy_stride[2];
    p.o_sb = d->dx_stride[0]; p.o_ss = d->dx_stride[1]; p.o_sh = d->dx_stride[2];
    p.B = d->B; p.S = d->S; p.H = d->H; p.D = d->D;
    p.eps = d->eps;
    p.heads_per_unit = u.heads_per_unit; p.head_groups = u.head_groups; p.units = u.units;
    norm_rope_bwd_kernel_t fn = d->dtype == COSMOS_ATTN_BF16 ? pick_bwd<true>(d->D) : pick_bwd<false>(d->D);
    hipLaunchKernelGGL(fn, dim3((unsigned)u.blocks), dim3(kThreads), 0, (hipStream_t)stream, p);
    if (hipGetLastError() != hipSuccess) return COSMOS_ATTN_LAUNCH_FAILED;
    if (d->dweight) {
        hipLaunchKernelGGL(norm_rope_dweight_kernel, dim3((unsigned)d->D), dim3(kThreads), 0, (hipStream_t)stream,
                           (const float*)workspace, d->dweight, u.blocks, d->D);
        if (hipGetLastError() != hipSuccess) return COSMOS_ATTN_LAUNCH_FAILED;
    }
    return COSMOS_ATTN_OK;
}

}  // extern "C"
