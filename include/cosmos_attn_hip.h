/*
 * cosmos_attn_hip.h -- C ABI of the MI355X (gfx950) flash-attention forward + forward-mode
 * JVP (tangent) library.
 *
 * Plain C: pointers, sizes, strides, a hipStream_t passed as void*.  No torch types.
 * Every entry point is asynchronous on the given stream and never synchronises the device.
 * All device pointers must belong to the current HIP device.
 *
 * Reference interfaces replaced (paths relative to the reference checkout):
 *   JVP = cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py
 *   ATT = cosmos_predict2/_src/predict2/networks/attention.py
 *   networks/... = cosmos_predict2/_src/predict2/networks/...
 */
#ifndef COSMOS_ATTN_HIP_H
#define COSMOS_ATTN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define COSMOS_ATTN_ABI_VERSION 2
#define COSMOS_ATTN_API __attribute__((visibility("default")))

/* element types of q,k,v,tangents and of o,to (lse is always fp32) */
enum cosmos_attn_dtype {
    COSMOS_ATTN_BF16 = 0,
    COSMOS_ATTN_FP16 = 1
};

/* status codes (0 = ok).  The Python host maps BAD_SHAPE/BAD_STRIDE to AssertionError like the
 * reference's asserts (JVP:439-448) and UNSUPPORTED to NotImplementedError (ATT:107-108). */
enum cosmos_attn_status {
    COSMOS_ATTN_OK = 0,
    COSMOS_ATTN_BAD_ARG = 1,        /* null pointer / negative size */
    COSMOS_ATTN_BAD_SHAPE = 2,      /* head dim not in {16,32,64,128,256}, causal with Lq != Lkv */
    COSMOS_ATTN_BAD_STRIDE = 3,     /* misaligned base or stride (16-byte rows required) */
    COSMOS_ATTN_UNSUPPORTED = 4,    /* dtype / head-dim combination not built */
    COSMOS_ATTN_WORKSPACE_TOO_SMALL = 5,
    COSMOS_ATTN_LAUNCH_FAILED = 6,  /* hipGetLastError() != hipSuccess after a launch */
    COSMOS_ATTN_STATIC_SCRATCH_EXCEEDED = 7,  /* cosmos_attn_fwd_jvp_static: workspace need > COSMOS_ATTN_STATIC_SCRATCH_BYTES */
    COSMOS_ATTN_WRONG_DEVICE = 8    /* the current device does not report 256 compute units (a partitioned MI355X, another part):
                                       checked once per device at the first attention launch */
};

/* size of the static device array behind cosmos_attn_fwd_jvp_static (64 MiB) */
#define COSMOS_ATTN_STATIC_SCRATCH_BYTES (64u << 20)

/*
 * One attention call.  Tensors are [B, H, L, d] addressed through element strides
 * (batch, head, row); the innermost (d) stride is 1.  This covers both the heads-first
 * layout of the JVP entry (JVP:425-431) and a transposed view of the DiT's [B, S, H, D]
 * tensors (ATT:166-168) without a copy.  Tangents share the strides of their primals
 * (the reference asserts this, JVP:448).
 *
 * Replaces the argument list of the Triton launch JVP:462-496.
 */
typedef struct cosmos_attn_desc {
    int32_t abi_version;     /* COSMOS_ATTN_ABI_VERSION */
    int32_t dtype;           /* enum cosmos_attn_dtype */
    int32_t B, H;            /* batch, heads                                   (JVP:489-490) */
    int32_t Lq, Lkv;         /* query / key sequence lengths                   (JVP:491-492) */
    int32_t d_qk, d_v;       /* head dims, each in {16,32,64,128,256}          (JVP:444-445; 256 runs a slower kernel) */
    int32_t causal;          /* 1: key j visible to query i iff j <= i; needs Lq == Lkv (JVP:446) */
    float sm_scale;          /* softmax scale; caller resolves the default d_qk^-0.5 (JVP:449-450) */

    const void *q, *k, *v;   /* primals (device) */
    const void *tq, *tk, *tv;/* tangents (device); all NULL = forward only; tk == tv == NULL = tangent on q only */
    int64_t q_stride[3];     /* (batch, head, row) element strides of q and tq */
    int64_t k_stride[3];     /* of k and tk */
    int64_t v_stride[3];     /* of v and tv */

    void *o, *to;            /* outputs [B,H,Lq,d_v] in `dtype`; `to` may be NULL iff all tangents are NULL */
    int64_t o_stride[3];     /* (batch, head, row) element strides of o and to (d stride 1) */
    float *lse;              /* [B,H,Lq] fp32 contiguous: natural-log logsumexp of the scaled scores (JVP:367,376); may be NULL */

    const int32_t *key_lens; /* optional [B] int32 (device): keys >= key_lens[b] are masked out.  No counterpart in the
                                reference, which never masks (ATT:94-95 ignores k_lens); pinned by the torch oracle. */
} cosmos_attn_desc;

/* ABI version of the loaded library. */
COSMOS_ATTN_API int cosmos_attn_abi_version(void);

/* Human-readable text for a status code (static storage). */
COSMOS_ATTN_API const char *cosmos_attn_status_string(int status);

/*
 * Tuning and test hook, process-wide; no counterpart in the reference.  Short key sequences (text cross-attention) are
 * served by a kernel that streams consecutive query blocks through one workgroup; the library chooses when and with how
 * many workgroups.  blocks_per_workgroup > 1 forces that kernel with that many query blocks per workgroup, 1 turns it off,
 * 0 leaves the choice to the library; workgroups > 0 (used when blocks_per_workgroup is 0) sets the number of workgroups
 * directly.  (0, 0) restores the default.  Nothing in the per-call path reads the environment.
 */
COSMOS_ATTN_API void cosmos_attn_set_stream_override(int blocks_per_workgroup, int workgroups);

/*
 * Bytes of device workspace the call needs (K, V and their tangents re-tiled into the
 * kernel's LDS image).  0 on invalid descriptors.  The host allocates it however it likes
 * (the Python host uses torch's caching allocator) and may reuse it across calls on one stream.
 * No counterpart in the reference (Triton reads K/V in place).
 */
COSMOS_ATTN_API size_t cosmos_attn_workspace_bytes(const cosmos_attn_desc *desc);

/*
 * Forward + JVP:  o = softmax(q k^T s) v ;  to = d/de o(q+e tq, k+e tk, v+e tv)|_{e=0} ;  lse.
 * Forward only when all tangent pointers are NULL.
 * Replaces `_attention.forward` -> `_attn_fwd[grid](...)`  (JVP:436-502, JVP:176-378) and, forward only,
 * the SDPA / FA3 call of `attention()` (ATT:119-127, ATT:170-178).
 * Launches the re-tiling kernel and the attention kernel on `stream`; returns a status code.
 */
COSMOS_ATTN_API int cosmos_attn_fwd_jvp(const cosmos_attn_desc *desc, void *workspace, size_t workspace_bytes, void *stream);

/*
 * cosmos_attn_fwd_jvp without a workspace argument and without any allocation: the workspace is a static device array
 * inside the library (COSMOS_ATTN_STATIC_SCRATCH_BYTES = 64 MiB per GPU, held until the process ends).
 * No counterpart in the reference.  It is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The call itself calls no hipMalloc / hipFree and no
 * allocating library routine; inputs and outputs are the caller's, as in cosmos_attn_fwd_jvp, and results are bitwise
 * those of cosmos_attn_fwd_jvp.
 * A problem whose cosmos_attn_workspace_bytes() exceeds the array is refused with COSMOS_ATTN_STATIC_SCRATCH_EXCEEDED
 * (the text cross-attention of the 2B DiT, B=2 H=16 Lkv=512 d=128, needs 8 MiB; self-attention at L=84480 does not fit).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or threads)
 * race on it; calls on one stream are ordered and safe.
 */
COSMOS_ATTN_API size_t cosmos_attn_static_scratch_bytes(void);
COSMOS_ATTN_API int cosmos_attn_fwd_jvp_static(const cosmos_attn_desc *desc, void *stream);

/*
 * The two stages separately, for callers that reuse K/V across calls (e.g. cross-attention
 * against a fixed text context, JVP with several tangent directions on q only) and for profiling.
 *   cosmos_attn_packed_bytes : bytes of the re-tiled image alone (depends on B, H, Lkv, the head dims and on whether
 *                              k and v carry tangents; not on q): what the two calls below need as `workspace_bytes`
 *   cosmos_attn_pack_kv : k,v(,tk,tv) -> workspace
 *   cosmos_attn_run     : q(,tq), workspace -> o(,to), lse     (desc->k/v/tk/tv are only tested for NULL)
 * An image packed without tangents serves forward-only runs and runs with a tangent on q alike.
 */
COSMOS_ATTN_API size_t cosmos_attn_packed_bytes(const cosmos_attn_desc *desc);
COSMOS_ATTN_API int cosmos_attn_pack_kv(const cosmos_attn_desc *desc, void *workspace, size_t workspace_bytes, void *stream);
COSMOS_ATTN_API int cosmos_attn_run(const cosmos_attn_desc *desc, const void *workspace, size_t workspace_bytes, void *stream);

/*
 * Backward (reverse mode through O only).  Replaces the flash-attn calls of `_attention.backward`
 * (JVP:505-561: `_flash_attn_backward` JVP:514-531, `_flash_attn_varlen_backward` JVP:538-559): inputs q, k, v, the
 * forward's o and lse (`ctx.saved_tensors`, JVP:506) and dout; outputs dq, dk, dv (JVP:561).  Equal head dims are
 * required like the reference (JVP:507-509); causal needs Lq == Lkv (the forward's JVP:446).  Tensors are [B, H, L, d]
 * addressed through element strides (batch, head, row), innermost stride 1; every tensor has its own strides, so the
 * transposed views the reference hands to flash-attn (JVP:515-523) need no copies.
 */
typedef struct cosmos_attn_bwd_desc {
    int32_t abi_version;     /* COSMOS_ATTN_ABI_VERSION */
    int32_t dtype;           /* enum cosmos_attn_dtype: element type of q, k, v, o, dout, dq, dk, dv */
    int32_t B, H;
    int32_t Lq, Lkv;
    int32_t d;               /* head dim of q, k and v, in {16,32,64,128,256} */
    int32_t causal;
    float sm_scale;          /* the forward's softmax scale (`ctx.sm_scale`, JVP:499) */
    int32_t max_ds_mib;      /* workspace the call may spend on keeping the 16-bit dS tiles between its two passes, in MiB:
                                0 = library default (32 GiB), > 0 = that many, < 0 = never keep dS (the smallest workspace;
                                the scores are then computed a second time for dq).  Results are deterministic either way. */

    const void *q, *k, *v, *o, *dout;   /* device */
    const float *lse;        /* [B,H,Lq] fp32 contiguous, as written by the forward */
    void *dq, *dk, *dv;      /* outputs, device */
    int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3], dout_stride[3];
    int64_t dq_stride[3], dk_stride[3], dv_stride[3];
} cosmos_attn_bwd_desc;

/* Bytes of device workspace `cosmos_attn_bwd` needs (per-row statistics and the re-tiled query and key streams). */
COSMOS_ATTN_API size_t cosmos_attn_bwd_workspace_bytes(const cosmos_attn_bwd_desc *desc);

/* dq, dk, dv from dout.  Asynchronous on `stream`, no atomics (bitwise reproducible); returns a status code. */
COSMOS_ATTN_API int cosmos_attn_bwd(const cosmos_attn_bwd_desc *desc, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Fused per-head RMSNorm + rotary position embedding, with optional forward-mode tangent: the step before the attention
 * call in `Attention.compute_qkv` (networks/minimal_v4_dit.py:405-415: `q_norm` / `k_norm` = te.pytorch.RMSNorm(head_dim,
 * eps=1e-6) :350-356, then TE `apply_rotary_pos_emb(..., tensor_format="bshd", fused=True)` for self-attention :409-414,
 * with the angles [L,1,1,D] of networks/minimal_v4_dit.py:648-658).
 *     n = x * rsqrt(mean_d(x^2) + eps) * weight        (rounded to `dtype`, as RMSNorm's output tensor is)
 *     y = n * cos(angles) + rotate_half(n) * sin(angles)               rotate_half(n) = cat(-n[D/2:], n[:D/2])
 *     ty = d/de y(x + e tx)|_{e=0}
 * x, tx: [B, S, H, D] addressed through element strides (batch, sequence, head), innermost stride 1; y, ty likewise with
 * their own strides (so the result can be written heads-first).  One kernel launch; no workspace.
 */
typedef struct cosmos_norm_rope_desc {
    int32_t abi_version;     /* COSMOS_ATTN_ABI_VERSION */
    int32_t dtype;           /* enum cosmos_attn_dtype: element type of x, tx, y, ty */
    int32_t B, S, H, D;      /* D in {16,32,64,128,256} */
    float eps;               /* 1e-6 in the DiT */
    int32_t reserved;        /* 0 */
    const void *x, *tx;      /* device; tx may be NULL (then ty must be NULL) */
    const float *weight;     /* [D] fp32 (RMSNorm's gamma), device; NULL = ones */
    const float *angles;     /* [S, D] fp32 contiguous, device; NULL = no rotation (cross-attention keys, :409) */
    void *y, *ty;            /* outputs, device */
    int64_t x_stride[3];     /* (batch, sequence, head) element strides of x and tx */
    int64_t y_stride[3];     /* of y and ty */
} cosmos_norm_rope_desc;

COSMOS_ATTN_API int cosmos_norm_rope(const cosmos_norm_rope_desc *desc, void *stream);

/*
 * Reverse mode of cosmos_norm_rope (what autograd does for the RMSNorm and rotary ops of networks/minimal_v4_dit.py:405-415
 * during training): from dy = dL/dy,
 *     dn = R^T dy                      (rotation by the negated angles; RMSNorm's 16-bit rounding is passed straight through)
 *     dx = r (weight * dn) - x r^3 mean_d(x * weight * dn),      r = rsqrt(mean_d(x^2) + eps)
 *     dweight[j] = sum over all (b, s, h) of dn[j] x[j] r        (fp32, optional)
 * x, dy, dx: [B, S, H, D] through their own (batch, sequence, head) element strides.  dweight needs a workspace of
 * cosmos_norm_rope_bwd_workspace_bytes(desc) bytes (per-block partial sums, added in a fixed order: results are
 * bitwise reproducible); with dweight == NULL no workspace is needed.  Two launches (one without dweight).
 */
typedef struct cosmos_norm_rope_bwd_desc {
    int32_t abi_version;     /* COSMOS_ATTN_ABI_VERSION */
    int32_t dtype;           /* element type of x, dy, dx */
    int32_t B, S, H, D;
    float eps;
    int32_t reserved;        /* 0 */
    const void *x, *dy;      /* device */
    const float *weight;     /* [D] fp32 or NULL = ones */
    const float *angles;     /* [S, D] fp32 or NULL = no rotation */
    void *dx;                /* device */
    float *dweight;          /* [D] fp32, device; NULL = not wanted */
    int64_t x_stride[3];
    int64_t dy_stride[3];
    int64_t dx_stride[3];
} cosmos_norm_rope_bwd_desc;

COSMOS_ATTN_API size_t cosmos_norm_rope_bwd_workspace_bytes(const cosmos_norm_rope_bwd_desc *desc);
COSMOS_ATTN_API int cosmos_norm_rope_bwd(const cosmos_norm_rope_bwd_desc *desc, void *workspace, size_t workspace_bytes,
                                         void *stream);

/*
 * Elementwise steps of the DiT block with optional forward-mode tangents (networks/minimal_v4_dit.py:1119-1242), each one
 * pass over 16-bit tensors with fp32 arithmetic.  Tensors are dense row-major [rows, D]; a modulation vector [groups, D]
 * is shared by `rows_per_group` consecutive rows (the H*W tokens of one (batch, frame), :1150-1162).  Tangent pointers
 * are optional: all NULL = values only.
 *
 * cosmos_ln_modulate:     y = LayerNorm(x) * (1 + scale) + shift           (:1166-1167; no affine parameters, eps :1031)
 *                         ty = its derivative along (tx, tscale, tshift)    (tscale / tshift NULL = they do not move)
 * cosmos_gated_residual:  out = x + gate * res                               (:1199, :1231, :1241)
 *                         tout = tx + tgate * res + gate * tres              (out / tout may alias x / tx)
 * cosmos_gelu:            a = gelu(h) (exact, erf form: nn.GELU() of :225),  ta = th * gelu'(h)
 */
typedef struct cosmos_ln_modulate_desc {
    int32_t abi_version, dtype;
    int32_t D, rows_per_group;     /* D % 8 == 0, D <= 8192; rows % rows_per_group == 0 */
    float eps;
    int32_t reserved;
    int64_t rows;
    const void *x, *tx;            /* [rows, D] */
    const void *shift, *scale;     /* [rows / rows_per_group, D] */
    const void *tshift, *tscale;   /* same shape, or NULL */
    void *y, *ty;                  /* [rows, D] */
} cosmos_ln_modulate_desc;

typedef struct cosmos_gated_residual_desc {
    int32_t abi_version, dtype;
    int32_t D, rows_per_group;
    int64_t rows;
    const void *x, *tx, *res, *tres;   /* [rows, D]; tx, tres, tout NULL together */
    const void *gate, *tgate;          /* [rows / rows_per_group, D]; tgate may be NULL */
    void *out, *tout;
} cosmos_gated_residual_desc;

typedef struct cosmos_gelu_desc {
    int32_t abi_version, dtype;
    int64_t n;                         /* elements, n % 8 == 0 */
    const void *h, *th;                /* th, ta NULL together */
    void *a, *ta;
} cosmos_gelu_desc;

COSMOS_ATTN_API int cosmos_ln_modulate(const cosmos_ln_modulate_desc *desc, void *stream);
COSMOS_ATTN_API int cosmos_gated_residual(const cosmos_gated_residual_desc *desc, void *stream);
COSMOS_ATTN_API int cosmos_gelu(const cosmos_gelu_desc *desc, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* COSMOS_ATTN_HIP_H */
