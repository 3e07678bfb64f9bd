// Elementwise pieces of the DiT block with their forward-mode tangents, for gfx950: kernels and C ABI.
//
// The DiT block (cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py:1119-1242) wraps each of its three
// sub-layers as
//     n = LayerNorm(x) * (1 + scale) + shift            (:1166-1167; LayerNorm without affine parameters, eps 1e-6, :1031)
//     x = x + gate * sublayer(n)                         (:1199, :1231, :1241)
// with per-(batch, frame) modulation vectors shift / scale / gate (:1131-1162), and its MLP uses the exact GELU
// (:222-249).  When a tangent is carried through the block these steps become, in plain tensor-library ops, some thirty
// passes over tensors of hundreds of megabytes; here each is one pass:
//     ln_modulate_kernel      y = n (1 + scale) + shift,  ty = tn (1 + scale) + n tscale + tshift
//                             n = (x - mean) r,  tn = r (tc - n mean(n tc)),  tc = tx - mean(tx),  r = rsqrt(var + eps)
//     gated_residual_kernel   out = x + gate res,  tout = tx + tgate res + gate tres
//     gelu_kernel             a = h Phi(h),  ta = th (Phi(h) + h phi(h))
// All HBM-bound; 16-bit tensors, fp32 arithmetic, 16-byte accesses.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "cosmos_attn_hip.h"

namespace {

constexpr int kThreads = 256;

template <bool BF16>
__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (BF16) {
            f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
            f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xFFFF0000u);
        } else {
            typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
            const half2_t h = __builtin_bit_cast(half2_t, w[i]);
            f[2 * i] = (float)h[0];
            f[2 * i + 1] = (float)h[1];
        }
    }
}
template <bool BF16>
__device__ __forceinline__ uint4 pack8(const float* f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (BF16) {
            typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
            bf2_t r; r[0] = (__bf16)f[2 * i]; r[1] = (__bf16)f[2 * i + 1];
            w[i] = __builtin_bit_cast(uint32_t, r);
        } else {
            typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
            half2_t r; r[0] = (_Float16)f[2 * i]; r[1] = (_Float16)f[2 * i + 1];
            w[i] = __builtin_bit_cast(uint32_t, r);
        }
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// sum over the 64 lanes of the wavefront, result in every lane
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) v += __shfl_xor(v, m);
    return v;
}

// ------------------------------------------------------------------------------------------------ LayerNorm + modulation
struct LnModParams {
    const uint16_t *x, *tx;                      // [rows, D]; tx may be null
    const uint16_t *shift, *scale;               // [groups, D]
    const uint16_t *tshift, *tscale;             // [groups, D] or null (the modulation does not move)
    uint16_t *y, *ty;                            // [rows, D]
    int64_t rows;
    int D, rows_per_group;
    float eps;
};

// One wavefront per row; lane l holds the 8-element chunks l, l + 64, ... (NCH of them, D <= 512 NCH), so that the
// row stays in registers between the statistics and the output pass.
template <int NCH, bool TANGENT, bool BF16>
__global__ void __launch_bounds__(kThreads) ln_modulate_kernel(const LnModParams p) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= p.rows) return;     // whole wavefronts leave together: the shuffles below stay complete
    const int D = p.D;
    const uint16_t* xr = p.x + row * D;
    const uint16_t* txr = TANGENT ? p.tx + row * D : nullptr;
    float x[NCH][8], t[NCH][8];
    float sx = 0.f, st = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int off = 8 * (lane + 64 * c);
        const bool in = off < D;
        uint4 z = make_uint4(0u, 0u, 0u, 0u);
        unpack8<BF16>(in ? *reinterpret_cast<const uint4*>(xr + off) : z, x[c]);
        if (TANGENT) unpack8<BF16>(in ? *reinterpret_cast<const uint4*>(txr + off) : z, t[c]);
#pragma unroll
        for (int i = 0; i < 8; ++i) { sx += x[c][i]; if (TANGENT) st += t[c][i]; }
    }
    const float inv_d = 1.0f / D;
    const float mean = wave_sum(sx) * inv_d;
    const float tmean = TANGENT ? wave_sum(st) * inv_d : 0.f;
    float sv = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const bool in = 8 * (lane + 64 * c) < D;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            x[c][i] = in ? x[c][i] - mean : 0.f;
            if (TANGENT) t[c][i] = in ? t[c][i] - tmean : 0.f;
            sv += x[c][i] * x[c][i];
        }
    }
    const float r = rsqrtf(wave_sum(sv) * inv_d + p.eps);
    float sd = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { x[c][i] *= r; if (TANGENT) sd += x[c][i] * t[c][i]; }
    }
    const float s = TANGENT ? wave_sum(sd) * inv_d : 0.f;

    const int64_t grp = row / p.rows_per_group;
    const uint16_t* sh = p.shift + grp * D;
    const uint16_t* sc = p.scale + grp * D;
    const uint16_t* tsh = (TANGENT && p.tshift) ? p.tshift + grp * D : nullptr;
    const uint16_t* tsc = (TANGENT && p.tscale) ? p.tscale + grp * D : nullptr;
    uint16_t* yr = p.y + row * D;
    uint16_t* tyr = TANGENT ? p.ty + row * D : nullptr;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int off = 8 * (lane + 64 * c);
        if (off >= D) continue;
        float a[8], b[8], y[8];
        unpack8<BF16>(*reinterpret_cast<const uint4*>(sc + off), a);
        unpack8<BF16>(*reinterpret_cast<const uint4*>(sh + off), b);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = x[c][i] * (1.0f + a[i]) + b[i];
        *reinterpret_cast<uint4*>(yr + off) = pack8<BF16>(y);
        if (TANGENT) {
            float ty[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) ty[i] = r * (t[c][i] - x[c][i] * s) * (1.0f + a[i]);
            if (tsc) {
                float ta[8];
                unpack8<BF16>(*reinterpret_cast<const uint4*>(tsc + off), ta);
#pragma unroll
                for (int i = 0; i < 8; ++i) ty[i] += x[c][i] * ta[i];
            }
            if (tsh) {
                float tb[8];
                unpack8<BF16>(*reinterpret_cast<const uint4*>(tsh + off), tb);
#pragma unroll
                for (int i = 0; i < 8; ++i) ty[i] += tb[i];
            }
            *reinterpret_cast<uint4*>(tyr + off) = pack8<BF16>(ty);
        }
    }
}

typedef void (*ln_kernel_t)(const LnModParams);
template <bool TANGENT, bool BF16>
ln_kernel_t pick_ln(int d) {
    const int nch = (d + 511) / 512;
    if (nch <= 1) return ln_modulate_kernel<1, TANGENT, BF16>;
    if (nch <= 2) return ln_modulate_kernel<2, TANGENT, BF16>;
    if (nch <= 4) return ln_modulate_kernel<4, TANGENT, BF16>;
    if (nch <= 8) return ln_modulate_kernel<8, TANGENT, BF16>;
    if (nch <= 10) return ln_modulate_kernel<10, TANGENT, BF16>;
    if (nch <= 16) return ln_modulate_kernel<16, TANGENT, BF16>;
    return nullptr;
}

// ------------------------------------------------------------------------------------------------ gated residual
struct GatedResidualParams {
    const uint16_t *x, *tx, *res, *tres;         // [rows, D]; tx, tres null together
    const uint16_t *gate, *tgate;                // [groups, D]; tgate may be null
    uint16_t *out, *tout;                        // [rows, D]; may alias x, tx
    int64_t chunks;                              // rows * D / 8
    int D, rows_per_group;
};

template <bool TANGENT, bool BF16>
__global__ void __launch_bounds__(kThreads) gated_residual_kernel(const GatedResidualParams p) {
    const int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (c >= p.chunks) return;
    const int cpr = p.D / 8;                      // chunks per row
    const int64_t row = c / cpr;
    const int col = (int)(c - row * cpr) * 8;
    const int64_t g = (row / p.rows_per_group) * p.D + col;
    const int64_t o = c * 8;
    float x[8], res[8], gate[8], out[8];
    unpack8<BF16>(*reinterpret_cast<const uint4*>(p.x + o), x);
    unpack8<BF16>(*reinterpret_cast<const uint4*>(p.res + o), res);
    unpack8<BF16>(*reinterpret_cast<const uint4*>(p.gate + g), gate);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = x[i] + gate[i] * res[i];
    if (TANGENT) {
        float tx[8], tres[8], tout[8];
        unpack8<BF16>(*reinterpret_cast<const uint4*>(p.tx + o), tx);
        unpack8<BF16>(*reinterpret_cast<const uint4*>(p.tres + o), tres);
#pragma unroll
        for (int i = 0; i < 8; ++i) tout[i] = tx[i] + gate[i] * tres[i];
        if (p.tgate) {
            float tg[8];
            unpack8<BF16>(*reinterpret_cast<const uint4*>(p.tgate + g), tg);
#pragma unroll
            for (int i = 0; i < 8; ++i) tout[i] += tg[i] * res[i];
        }
        *reinterpret_cast<uint4*>(p.tout + o) = pack8<BF16>(tout);
    }
    *reinterpret_cast<uint4*>(p.out + o) = pack8<BF16>(out);
}

// ------------------------------------------------------------------------------------------------ GELU
struct GeluParams {
    const uint16_t *h, *th;                      // th may be null
    uint16_t *a, *ta;
    int64_t chunks;                              // elements / 8
};

template <bool TANGENT, bool BF16>
__global__ void __launch_bounds__(kThreads) gelu_kernel(const GeluParams p) {
    const int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (c >= p.chunks) return;
    const int64_t o = c * 8;
    float h[8], a[8], th[8], ta[8];
    unpack8<BF16>(*reinterpret_cast<const uint4*>(p.h + o), h);
    if (TANGENT) unpack8<BF16>(*reinterpret_cast<const uint4*>(p.th + o), th);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float cdf = 0.5f * (1.0f + erff(h[i] * 0.70710678118654752f));
        a[i] = h[i] * cdf;
        if (TANGENT) {
            const float pdf = 0.3989422804014327f * __expf(-0.5f * h[i] * h[i]);
            ta[i] = th[i] * (cdf + h[i] * pdf);
        }
    }
    *reinterpret_cast<uint4*>(p.a + o) = pack8<BF16>(a);
    if (TANGENT) *reinterpret_cast<uint4*>(p.ta + o) = pack8<BF16>(ta);
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }
bool dtype_ok(int dtype) { return dtype == COSMOS_ATTN_BF16 || dtype == COSMOS_ATTN_FP16; }
int launched() { return hipGetLastError() == hipSuccess ? COSMOS_ATTN_OK : COSMOS_ATTN_LAUNCH_FAILED; }

}  // namespace

extern "C" {

COSMOS_ATTN_API int cosmos_ln_modulate(const cosmos_ln_modulate_desc* d, void* stream) {
    if (!d || d->abi_version != COSMOS_ATTN_ABI_VERSION) return COSMOS_ATTN_BAD_ARG;
    if (d->rows <= 0 || d->D <= 0 || d->rows_per_group <= 0 || !(d->eps >= 0.f)) return COSMOS_ATTN_BAD_ARG;
    if (!d->x || !d->y || !d->shift || !d->scale) return COSMOS_ATTN_BAD_ARG;
    if ((d->tx != nullptr) != (d->ty != nullptr)) return COSMOS_ATTN_BAD_ARG;
    if (!d->tx && (d->tshift || d->tscale)) return COSMOS_ATTN_BAD_ARG;
    if (!dtype_ok(d->dtype)) return COSMOS_ATTN_UNSUPPORTED;
    if (d->D % 8 != 0 || d->rows % d->rows_per_group != 0) return COSMOS_ATTN_BAD_SHAPE;
    if (d->D > 8192) return COSMOS_ATTN_UNSUPPORTED;
    const void* ptrs[] = {d->x, d->tx, d->shift, d->scale, d->tshift, d->tscale, d->y, d->ty};
    for (const void* q : ptrs) if (q && !aligned16(q)) return COSMOS_ATTN_BAD_STRIDE;
    LnModParams p;
    p.x = (const uint16_t*)d->x; p.tx = (const uint16_t*)d->tx;
    p.shift = (const uint16_t*)d->shift; p.scale = (const uint16_t*)d->scale;
    p.tshift = (const uint16_t*)d->tshift; p.tscale = (const uint16_t*)d->tscale;
    p.y = (uint16_t*)d->y; p.ty = (uint16_t*)d->ty;
    p.rows = d->rows; p.D = d->D; p.rows_per_group = d->rows_per_group; p.eps = d->eps;
    const bool bf16 = d->dtype == COSMOS_ATTN_BF16;
    ln_kernel_t fn = d->tx ? (bf16 ? pick_ln<true, true>(d->D) : pick_ln<true, false>(d->D))
                           : (bf16 ? pick_ln<false, true>(d->D) : pick_ln<false, false>(d->D));
    const int64_t blocks = (d->rows + kThreads / 64 - 1) / (kThreads / 64);
    if (!fn || blocks > 0x7FFFFFFF) return COSMOS_ATTN_BAD_SHAPE;
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, p);
    return launched();
}

COSMOS_ATTN_API int cosmos_gated_residual(const cosmos_gated_residual_desc* d, void* stream) {
    if (!d || d->abi_version != COSMOS_ATTN_ABI_VERSION) return COSMOS_ATTN_BAD_ARG;
    if (d->rows <= 0 || d->D <= 0 || d->rows_per_group <= 0) return COSMOS_ATTN_BAD_ARG;
    if (!d->x || !d->res || !d->gate || !d->out) return COSMOS_ATTN_BAD_ARG;
    const bool tangent = d->tx != nullptr;
    if ((d->tres != nullptr) != tangent || (d->tout != nullptr) != tangent || (!tangent && d->tgate)) return COSMOS_ATTN_BAD_ARG;
    if (!dtype_ok(d->dtype)) return COSMOS_ATTN_UNSUPPORTED;
    if (d->D % 8 != 0 || d->rows % d->rows_per_group != 0) return COSMOS_ATTN_BAD_SHAPE;
    const void* ptrs[] = {d->x, d->tx, d->res, d->tres, d->gate, d->tgate, d->out, d->tout};
    for (const void* q : ptrs) if (q && !aligned16(q)) return COSMOS_ATTN_BAD_STRIDE;
    GatedResidualParams p;
    p.x = (const uint16_t*)d->x; p.tx = (const uint16_t*)d->tx; p.res = (const uint16_t*)d->res; p.tres = (const uint16_t*)d->tres;
    p.gate = (const uint16_t*)d->gate; p.tgate = (const uint16_t*)d->tgate;
    p.out = (uint16_t*)d->out; p.tout = (uint16_t*)d->tout;
    p.chunks = d->rows * (d->D / 8); p.D = d->D; p.rows_per_group = d->rows_per_group;
    const int64_t blocks = (p.chunks + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFF) return COSMOS_ATTN_BAD_SHAPE;
    const bool bf16 = d->dtype == COSMOS_ATTN_BF16;
    auto fn = tangent ? (bf16 ? gated_residual_kernel<true, true> : gated_residual_kernel<true, false>)
                      : (bf16 ? gated_residual_kernel<false, true> : gated_residual_kernel<false, false>);
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, p);
    return launched();
}

COSMOS_ATTN_API int cosmos_gelu(const cosmos_gelu_desc* d, void* stream) {
    if (!d || d->abi_version != COSMOS_ATTN_ABI_VERSION) return COSMOS_ATTN_BAD_ARG;
    if (d->n <= 0 || !d->h || !d->a || (d->th != nullptr) != (d->ta != nullptr)) return COSMOS_ATTN_BAD_ARG;
    if (!dtype_ok(d->dtype)) return COSMOS_ATTN_UNSUPPORTED;
    if (d->n % 8 != 0) return COSMOS_ATTN_BAD_SHAPE;
    const void* ptrs[] = {d->h, d->th, d->a, d->ta};
    for (const void* q : ptrs) if (q && !aligned16(q)) return COSMOS_ATTN_BAD_STRIDE;
    GeluParams p;
    p.h = (const uint16_t*)d->h; p.th = (const uint16_t*)d->th; p.a = (uint16_t*)d->a; p.ta = (uint16_t*)d->ta;
    p.chunks = d->n / 8;
    const int64_t blocks = (p.chunks + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFF) return COSMOS_ATTN_BAD_SHAPE;
    const bool bf16 = d->dtype == COSMOS_ATTN_BF16;
    auto fn = d->th ? (bf16 ? gelu_kernel<true, true> : gelu_kernel<true, false>)
                    : (bf16 ? gelu_kernel<false, true> : gelu_kernel<false, false>);
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, p);
    return launched();
}

}  // extern "C"
