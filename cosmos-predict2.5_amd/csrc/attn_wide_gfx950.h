// Head dim 256 (the reference accepts it, flash_attention_jvp_triton.py:444-445; no Cosmos configuration uses it).
// Included by attn_fwd_jvp_gfx950.hip inside its anonymous namespace.
//
// At d = 256 a 32-key tile of K, dK, V^T, dV^T is 64 KB (the LDS rings of the other kernels would need 224 KB) and the
// accumulators of 32 query rows are 512 registers, so this case gets a kernel of its own, built for being right rather
// than fast: no LDS, no roles, no barriers.  A workgroup is four wavefronts that serve the SAME 32 query rows; each
// computes the whole score tile for itself (S^T = K Q^T, dS^T = K dQ^T + dK Q^T with v_mfma_f32_32x32x16, the A fragments
// read straight from the re-tiled K/V image in memory: one 1 KB fragment is 64 lanes x 16 B there), runs the same online
// softmax, and accumulates its own quarter of the output channels (32-channel blocks w and w + 4 of O^T and T^T).
// Same arithmetic and rounding points as attn_fwd_jvp_kernel (flash_attention_jvp_triton.py:47-153, :299-309, :367-378).
// Head dims are run-time values here (any of 16 ... 256 each); the launch code sends only calls with a 256 this way.

constexpr int kWideMaxNC = 16;    // d_qk / 16
constexpr int kWideWaves = 4;
constexpr int kWideDbPerWave = 2; // 32-channel output blocks per wavefront: blocks w and w + 4

template <typename T, int MODE>
__global__ void __launch_bounds__(64 * kWideWaves) attn_wide_kernel(const AttnParams p, int dqk, int dv) {
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr bool JVP = MODE != MODE_FWD, FULL = MODE == MODE_JVP_FULL;
    const TileGeom g(dqk, dv, FULL);
    const int nc = g.nc, ndb = g.ndb;
    const int tile_bytes = g.tile_frags * kFragBytes;
    const int dk_frag0 = g.k_frags;                          // first dK fragment of a tile (FULL)
    const int v_frag0 = g.kpart_frags;                       // first V^T fragment
    const int dv_frag0 = g.kpart_frags + g.vt_frags;         // first dV^T fragment (FULL)

    const int pair = blockIdx.x;
    const int n_qt = (p.Lq + 31) / 32;
    const int qt = pair % n_qt, bh = pair / n_qt, b = bh / p.H, h = bh % p.H;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int row0 = qt * 32, row = row0 + j;

    int kv_len = p.Lkv;
    if (p.key_lens) { const int kl = p.key_lens[b]; kv_len = kl < kv_len ? (kl < 0 ? 0 : kl) : kv_len; }
    int n_tiles = (kv_len + kBlockN - 1) / kBlockN;
    const bool causal = p.causal != 0;
    if (causal) { const int lim = (row0 + 32 + kBlockN - 1) / kBlockN; n_tiles = n_tiles < lim ? n_tiles : lim; }

    // Q (and dQ) fragments: B operand of S^T = K Q^T; lane holds Q[row][16 c + 8 hh .. +7]
    V8 qf[kWideMaxNC], tqf[kWideMaxNC];
    {
        const bool live = row < p.Lq;
        const int64_t off = (int64_t)b * p.q_sb + (int64_t)h * p.q_sh + (int64_t)(live ? row : 0) * p.q_sl + 8 * hh;
        const T* qp = reinterpret_cast<const T*>(p.q) + off;
        const T* tqp = reinterpret_cast<const T*>(JVP ? p.tq : p.q) + off;
        const V8 z = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < kWideMaxNC; ++c) {
            qf[c] = z; tqf[c] = z;
            if (c < nc && live) {
                qf[c] = *reinterpret_cast<const V8*>(qp + 16 * c);
                if (JVP) tqf[c] = *reinterpret_cast<const V8*>(tqp + 16 * c);
            }
        }
    }
    f32x16 acc[kWideDbPerWave], acct[kWideDbPerWave];
#pragma unroll
    for (int i = 0; i < kWideDbPerWave; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) { acc[i][e] = 0.f; acct[i][e] = 0.f; }
    }
    float m_run = -INFINITY, l_run = 0.f, r_run = 0.f;
    const char* const head = p.kv + (size_t)bh * p.n_tiles * tile_bytes;
    auto frag = [&](const char* tile, int f) { return *reinterpret_cast<const V8*>(tile + (size_t)f * kFragBytes + lane * 16); };

    for (int t = 0; t < n_tiles; ++t) {
        const char* const tile = head + (size_t)t * tile_bytes;
        f32x16 s, ds;
#pragma unroll
        for (int e = 0; e < 16; ++e) { s[e] = 0.f; ds[e] = 0.f; }
#pragma unroll
        for (int c = 0; c < kWideMaxNC; ++c) {
            if (c < nc) {
                const V8 kf = frag(tile, c);
                s = mfma32(kf, qf[c], s);
                if (JVP) ds = mfma32(kf, tqf[c], ds);
                if (FULL) ds = mfma32(frag(tile, dk_frag0 + c), qf[c], ds);
            }
        }
        // masks: keys past kv_len, and above the diagonal when causal (element e is key 8 (e/4) + 4 hh + e%4 of the tile)
        if (t * kBlockN + kBlockN > kv_len || (causal && t * kBlockN + kBlockN - 1 > row0)) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int key = t * kBlockN + 4 * hh + 8 * (e >> 2) + (e & 3);
                const bool ok = key < kv_len && (!causal || key <= row);
                s[e] = ok ? s[e] : -INFINITY;
            }
        }
        float mx = s[0];
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s[e]);
        float lo, hi;
        both_halves(mx, lo, hi);
        const float m_new = fmaxf(m_run, fmaxf(lo, hi) * p.scale_log2);
        if (__any(m_new > m_run + max_slack_of<T>(JVP))) {
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            l_run *= alpha;
            r_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int i = 0; i < kWideDbPerWave; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) { acc[i][e] *= alpha; acct[i][e] *= alpha; }
            }
        }
        V8 pf[2], hf[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], p.scale_log2, -m_run));
            l_run += pe;
            pf[e >> 3][e & 7] = (T)pe;
            if (JVP) {
                const float hv = pe * (ds[e] * p.sm_scale);
                r_run += hv;
                hf[e >> 3][e & 7] = (T)hv;
            }
        }
#pragma unroll
        for (int i = 0; i < kWideDbPerWave; ++i) {
            const int db = wave + kWideWaves * i;
            if (db < ndb) {
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const V8 vf = frag(tile, v_frag0 + 2 * db + c);
                    acc[i] = mfma32(vf, pf[c], acc[i]);
                    if (JVP) acct[i] = mfma32(vf, hf[c], acct[i]);
                    if (FULL) acct[i] = mfma32(frag(tile, dv_frag0 + 2 * db + c), pf[c], acct[i]);
                }
            }
        }
    }
    // O = acc / l ; dO = (T - (r / l) acc) / l ; LSE = (m + log2 l) ln 2
    float l_lo, l_hi, r_lo, r_hi;
    both_halves(l_run, l_lo, l_hi);
    both_halves(r_run, r_lo, r_hi);
    const float l_tot = l_lo + l_hi, r_tot = r_lo + r_hi;
    const float inv_l = 1.0f / l_tot, r_over_l = r_tot * inv_l;
    if (row < p.Lq) {
        const int64_t off = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh + (int64_t)row * p.o_sl;
        T* op = reinterpret_cast<T*>(p.o) + off;
        T* top = reinterpret_cast<T*>(JVP ? p.to : p.o) + off;
#pragma unroll
        for (int i = 0; i < kWideDbPerWave; ++i) {
            const int db = wave + kWideWaves * i;
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int d = 32 * db + 8 * gq + 4 * hh;   // registers 4 gq .. 4 gq + 3 are 4 consecutive channels
                if (db < ndb && d < dv) {
                    V4 ov, tov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        ov[r] = (T)(acc[i][4 * gq + r] * inv_l);
                        tov[r] = (T)((acct[i][4 * gq + r] - r_over_l * acc[i][4 * gq + r]) * inv_l);
                    }
                    *reinterpret_cast<V4*>(op + d) = ov;
                    if (JVP) *reinterpret_cast<V4*>(top + d) = tov;
                }
            }
        }
        if (p.lse && wave == 0 && hh == 0) p.lse[(int64_t)bh * p.Lq + row] = (m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
    }
}
