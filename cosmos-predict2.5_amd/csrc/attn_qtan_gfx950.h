// Tangent on q only, short key sequences: text cross-attention under the forward-mode JVP (dK = dV = 0).
// Included by attn_fwd_jvp_gfx950.hip inside its anonymous namespace (uses AttnParams, StreamStores, the LDS-fill
// helpers and the streaming scheme of attn_qstream_kernel: one workgroup serves `q_chunk` consecutive query blocks of
// one (batch, head) as one stream of 32-key steps, finished blocks drain through LDS during the next block's sweep).
//
//     S  = Q K^T s      P = softmax(S)     O  = P V
//     dS = dQ K^T s     H = P * dS         r = rowsum H        dO = H V - r O
// (flash_attention_jvp_triton.py:86-152 with zero dK, dV: the Q dK^T and P dV products vanish.)
//
// Four matrix products per tile instead of six, but the same softmax arithmetic: with the role split of
// attn_fwd_jvp_kernel (score wavefront: both score products and all of the VALU work; output wavefront: both output
// products) the score wavefront alone decides the step time and the matrix pipe idles more than half of it.  Here the
// work of a 32-row pair is cut differently, so that both wavefronts of a SIMD carry about the same load:
//   * score wavefront:   S^T = K Q^T (8 MFMA at d = 128), running max, p = exp2(s c - m), row sum l; hands p over in
//                        fp32 (lane to same lane: the accumulator layouts of S^T and dS^T are the same);
//   * output wavefront:  dS^T = K dQ^T (8 MFMA), H = p dS s, row sum r, rounding of P^T and H^T to 16 bit, then
//                        O^T += V^T P^T and T^T += V^T H^T (16 MFMA).
// Per step f the score wavefront computes the scores of tile f+1 while it turns those of tile f into p; the output
// wavefront computes dS^T of tile f while it turns p and dS^T of tile f-1 into P^T, H^T, and then accumulates tile f-1.
// The rounding points are those of the other kernels (l and r from unrounded fp32 values, P and H rounded before the
// output products).
// LDS: K ring (4 parts: tiles f and f+1 in use, f+2 and f+3 arriving), V ring (3), p hand-over (2 stages x 4 pairs x
// 4 KB), rescale factors, 1 / l per finished block, and the regions of the finished blocks on their way out.

template <int DQK, int DV>
struct QtCfg {
    static constexpr int NC = DQK / 16, NDB = (DV + 31) / 32;
    static constexpr int K_FR = NC, VT_FR = 2 * NDB;
    static constexpr int KP_BYTES = K_FR * kFragBytes, VP_BYTES = VT_FR * kFragBytes, TILE_BYTES = KP_BYTES + VP_BYTES;
    static constexpr int KP_LOADS = (K_FR + 3) / 4, VP_LOADS = (VT_FR + 3) / 4;   // per output wavefront per tile
    static constexpr int P_BYTES = 4 * kFragBytes;           // p of one tile and one pair: 16 floats per lane
    static constexpr int KRING_OFF = 0;
    static constexpr int VRING_OFF = kRingK * KP_BYTES;
    static constexpr int P_OFF = VRING_OFF + kRingV * VP_BYTES;       // [2 stages][4 pairs][4 pieces][64 lanes] float4
    static constexpr int ALPHA_OFF = P_OFF + 2 * 4 * P_BYTES;         // [2 stages][4 pairs][64 lanes] floats
    static constexpr int STAT_OFF = ALPHA_OFF + 2 * 4 * 256;          // [2 block parities][4 pairs][64 lanes] floats: 1 / l
    static constexpr int XP_OFF = STAT_OFF + 2 * 4 * 256;             // [4 pairs] finished blocks on their way out
    typedef StreamStores<DV, MODE_JVP_Q> ST;
    static constexpr int LDS_BYTES = XP_OFF + 4 * ST::XP_BYTES;
};

template <typename T, int DQK, int DV>
__global__ void __attribute__((amdgpu_flat_work_group_size(kAttnThreads, kAttnThreads), amdgpu_waves_per_eu(2, 2)))
attn_qtan_kernel(const AttnParams p) {
    typedef QtCfg<DQK, DV> C;
    typedef typename C::ST ST;
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    constexpr int NC = C::NC, NDB = C::NDB, NB = 2 * NDB;
    constexpr int EPC = 16 / NC;   // score elements dealt out per d chunk
    constexpr int PD = COSMOS_ATTN_PREFETCH_GROUPS;
    constexpr int KP_BYTES = C::KP_BYTES, VP_BYTES = C::VP_BYTES, TILE_BYTES = C::TILE_BYTES;
    // At the top of step f the fills of V(f-1) and K(f+1) must have landed; issued after them and still allowed in
    // flight: V(f), K(f+2) (the group of step f-1), and the NC row fetches of dQ when step f-1 issued them.
    constexpr int IN_FLIGHT = C::KP_LOADS + C::VP_LOADS;
    constexpr int WAIT_FILLS = (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14) | 0x0F70;
    constexpr int WAIT_FILLS_ROWS = ((IN_FLIGHT + NC) & 15) | (((IN_FLIGHT + NC) >> 4) << 14) | 0x0F70;

    const int bid = blockIdx.x;
    const int bh = bid % p.BH, chunk = bid / p.BH, b = bh / p.H, h = bh % p.H;
    const int qt0 = chunk * p.q_chunk;                                         // first query block of this workgroup
    const int nq = p.n_qt - qt0 < p.q_chunk ? p.n_qt - qt0 : p.q_chunk;        // query blocks of this workgroup (>= 1)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool score_role = wave < 4;
    const int qw = wave & 3;
    const int j = lane & 31, hh = lane >> 5;

    int kv_len = p.Lkv;
    if (p.key_lens) { const int kl = p.key_lens[b]; kv_len = kl < kv_len ? (kl < 0 ? 0 : kl) : kv_len; }
    // key tiles per query block: at least two (see attn_qstream_kernel); tiles past the last valid key are fully masked
    int n = kv_len > 0 ? (kv_len + kBlockN - 1) / kBlockN : 1;
    if (n < 2) n = 2;
    const int n_flat = nq * n;                     // steps of the whole stream: position f = query block f / n, tile f % n

    char* const kring = smem + C::KRING_OFF;
    char* const vring = smem + C::VRING_OFF;
    const __amdgpu_buffer_rsrc_t kv_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.kv) + (size_t)bh * p.n_tiles * TILE_BYTES, 0, p.n_tiles * TILE_BYTES, 0x00020000);
    const int shift = (((bid >> 3) & 31) * COSMOS_ATTN_SWEEP_STAGGER) % n;
    auto tile_at = [&](int u) { return __builtin_amdgcn_readfirstlane((u + shift) % n); };
    auto wrap_inc = [&](int t) { ++t; return t >= n ? t - n : t; };
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    const unsigned p_base = C::P_OFF + qw * C::P_BYTES + 16 * lane, alpha_base = C::ALPHA_OFF + qw * 256 + 4 * lane;
    const unsigned stat_base = C::STAT_OFF + qw * 256 + 4 * lane, xp_base = C::XP_OFF + qw * ST::XP_BYTES;
    auto need_mask = [&](int t) { return t * kBlockN + kBlockN > kv_len; };
    auto lds_frag = [&](const char* base, int frag) { return *reinterpret_cast<const V8*>(base + frag * kFragBytes + lane * 16); };
    // byte offset of this lane's piece of Q / dQ inside its head for query block qt (rows past Lq read the last row)
    auto q_off = [&](int qt) {
        int row = qt * kBlockM + qw * 32 + j;
        row = row < p.Lq ? row : p.Lq - 1;
        return ((unsigned)row * (unsigned)p.q_sl + 8u * hh) * 2u;
    };
    typedef std::integral_constant<int, 0> KindA;
    typedef std::integral_constant<int, 1> KindB;
    typedef std::integral_constant<int, 2> KindC;

    if (score_role) {
        // ------------------------------------------------------------------------------------------ score wavefront
        const char* const q_head = reinterpret_cast<const char*>(p.q) + ((int64_t)b * p.q_sb + (int64_t)h * p.q_sh) * 2;
        const char* const tq_head = reinterpret_cast<const char*>(p.tq) + ((int64_t)b * p.q_sb + (int64_t)h * p.q_sh) * 2;
        V8 qf[NC];
        {
            const unsigned off = q_off(qt0);
#pragma unroll
            for (int c = 0; c < NC; ++c) qf[c] = *reinterpret_cast<const V8*>(q_head + off + 32 * c);
        }
        float m_run = -INFINITY, l_run = 0.f;
        const float scale_log2 = p.scale_log2;
        constexpr int Q_LINES = (2 * DQK + 127) / 128;
        int warm_q = 0, warm_tq = 0;
        // draining of finished blocks: see attn_qstream_kernel
        const int drain_steps = n > 3 ? n - 2 : 1;
        const int st_per_step = (ST::NS + drain_steps - 1) / drain_steps;
        const int rr = lane / ST::CPR, ch = lane % ST::CPR;
        const unsigned x_lane = rr * ST::ROW_BYTES + ((ch ^ (rr & (ST::CPR - 1))) << 4);
        const unsigned o_lane = ((unsigned)rr * (unsigned)p.o_sl + 8u * ch) * 2u;
        const int64_t o_head = ((int64_t)b * p.o_sb + (int64_t)h * p.o_sh) * 2;
        auto drain = [&](int qt, int lo, int hi) {
            for (int i = lo; i < hi; ++i) {
                const int t = i / ST::SPT, g = i % ST::SPT;
                const unsigned sw = ST::RPS < ST::CPR ? ((g * ST::RPS) & (ST::CPR - 1)) << 4 : 0;
                const V8 val = *reinterpret_cast<const V8*>(smem + xp_base + t * 32 * ST::ROW_BYTES + g * ST::RPS * ST::ROW_BYTES + (x_lane ^ sw));
                const int r0 = qt * kBlockM + qw * 32 + g * ST::RPS;
                char* const base = reinterpret_cast<char*>(t ? p.to : p.o) + o_head + (int64_t)r0 * p.o_sl * 2;
                if (r0 + rr < p.Lq) asm volatile("global_store_dwordx4 %0, %1, %2" ::"v"(o_lane), "v"(val), "s"(base) : "memory");
            }
        };
        auto lane_max = [](const f32x16& x) {
            float mx = x[0];
#pragma unroll
            for (int e = 1; e < 16; ++e) mx = fmaxf(mx, x[e]);
            return mx;
        };
        float alpha = 1.0f;
        // fold a tile's scores into the running max (masking them first where the tile needs it); sets alpha
        auto fold = [&](f32x16& x, int t) {
            if (need_mask(t)) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = t * kBlockN + 4 * hh + 8 * (e >> 2) + (e & 3);
                    x[e] = key < kv_len ? x[e] : -INFINITY;
                }
            }
            float lo, hi;
            both_halves(lane_max(x), lo, hi);
            const float m_new = fmaxf(m_run, fmaxf(lo, hi) * scale_log2);
            alpha = 1.0f;
            if (__any(m_new > m_run + kMaxSlack)) {
                alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                l_run *= alpha;
                m_run = m_new;
            }
        };
        f32x16 sc0, sc1;
        __builtin_amdgcn_s_barrier();         // the first K parts are in LDS (the output wavefronts waited for them)
        asm volatile("" ::: "memory");
        {
#pragma unroll
            for (int e = 0; e < 16; ++e) sc0[e] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) sc0 = mfma32(lds_frag(kring, c), qf[c], sc0);
        }
        fold(sc0, tile_at(0));
        int t_v = tile_at(1);
        int f = 0, qi = 0;
        bool more = nq > 1;
        // Step f = position s_in of block qi's sweep.  Kinds: A = steps 0 .. n-3; B = step n-2, which refills the Q
        // registers chunk by chunk as the block's last score product lets go of them; C = step n-1, which waits for them
        // chunk by chunk and closes the block.
        auto one = [&](auto kind, const f32x16& cur, f32x16& nxt, int s_in) {
            constexpr int KIND = decltype(kind)::value;
            __builtin_amdgcn_s_waitcnt(0xC07F);      // own LDS stores of step f-1 done
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const unsigned p_out = lds0 + p_base + (f & 1) * 4 * C::P_BYTES, alpha_out = lds0 + alpha_base + (f & 1) * 4 * 256;
            const char* const kpart = kring + ((f + 1) % kRingK) * KP_BYTES;
            if (KIND == 0 && more && s_in == 0) {   // touch the next block's rows (both tensors): they are in the L2 when fetched
                const unsigned off = q_off(qt0 + qi + 1) - 16u * hh + (Q_LINES > 1 ? 128u * hh : 0u);
                warm_q = *reinterpret_cast<const int*>(q_head + off);
                warm_tq = *reinterpret_cast<const int*>(tq_head + off);
            }
            const bool refill = KIND == 1 && more;
            const unsigned off_n = refill ? q_off(qt0 + qi + 1) : 0u;
            asm volatile("ds_write_b32 %0, %1" ::"v"(alpha_out), "v"(alpha) : "memory");
            V8 fa[NC];
#pragma unroll
            for (int i = 0; i < PD && i < NC; ++i) fa[i] = lds_frag(kpart, i);
#pragma unroll
            for (int e = 0; e < 16; ++e) nxt[e] = 0.f;
            f32x4 pv;
            auto softmax_chunk = [&](int c) {
#pragma unroll
                for (int k = 0; k < EPC; ++k) {
                    const int e = c * EPC + k;
                    const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(cur[e], scale_log2, -m_run));
                    l_run += pe;
                    pv[e & 3] = pe;
                    if ((e & 3) == 3) asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(p_out), "v"(pv), "n"((e >> 2) * kFragBytes) : "memory");
                }
            };
            if (refill) {
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    SCHED_FENCE();
                    if (c + PD < NC) fa[c + PD] = lds_frag(kpart, c + PD);
                    SCHED_FENCE();
                    nxt = mfma32(fa[c], qf[c], nxt);
                    softmax_chunk(c);
                    SCHED_FENCE();
                    qf[c] = *reinterpret_cast<const V8*>(q_head + off_n + 32 * c);
                }
            } else {
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    SCHED_FENCE();
                    if (c + PD < NC) fa[c + PD] = lds_frag(kpart, c + PD);
                    SCHED_FENCE();
                    nxt = mfma32(fa[c], qf[c], nxt);
                    softmax_chunk(c);
                    SCHED_FENCE();
                }
            }
            if (KIND == 2) asm volatile("" ::"v"(warm_q), "v"(warm_tq));
            if (KIND != 1 && qi > 0 && s_in > 0) {
                const int lo = (KIND == 2 ? drain_steps - 1 : s_in - 1) * st_per_step, hi = lo + st_per_step;
                drain(qt0 + qi - 1, lo, hi < ST::NS ? hi : ST::NS);
            }
            if (KIND == 2) {
                // the finished block: 1 / l to the output wavefront, LSE = (m + log2 l) ln 2
                float l_lo, l_hi;
                both_halves(l_run, l_lo, l_hi);
                const float l_tot = l_lo + l_hi;
                const float inv_l = 1.0f / l_tot;
                asm volatile("ds_write_b32 %0, %1" ::"v"(lds0 + stat_base + (qi & 1) * 4 * 256), "v"(inv_l) : "memory");
                const int row = (qt0 + qi) * kBlockM + qw * 32 + j;
                if (row < p.Lq && p.lse && hh == 0)
                    p.lse[(int64_t)bh * p.Lq + row] = (m_run + __builtin_log2f(l_tot)) * 0.6931471805599453f;
                m_run = -INFINITY; l_run = 0.f;
            }
            if (f + 1 < n_flat) fold(nxt, t_v);
            t_v = wrap_inc(t_v);   // tile at position f + 2
            ++f;
        };
        for (qi = 0; qi < nq; ++qi) {
            more = qi + 1 < nq;
            int s_in = 0;
            for (; s_in + 2 <= n - 2; s_in += 2) {
                one(KindA(), sc0, sc1, s_in);
                one(KindA(), sc1, sc0, s_in + 1);
            }
            if (s_in < n - 2) {
                one(KindA(), sc0, sc1, s_in);
                sc0 = sc1;
            }
            one(KindB(), sc0, sc1, n - 2);
            one(KindC(), sc1, sc0, n - 1);
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);      // step n_flat: the output wavefronts accumulate the last tile
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();            // the last block's region is complete
        asm volatile("" ::: "memory");
        drain(qt0 + nq - 1, 0, ST::NS);
    } else {
        // ----------------------------------------------------------------------------------------- output wavefront
        const char* const tq_head = reinterpret_cast<const char*>(p.tq) + ((int64_t)b * p.q_sb + (int64_t)h * p.q_sh) * 2;
        const int k_run = ((qw * C::KP_LOADS) % C::K_FR) * kFragBytes, v_run = ((qw * C::VP_LOADS) % C::VT_FR) * kFragBytes;
        auto fill_k = [&](int t, int u) {
            issue_part<C::KP_LOADS>(kv_rsrc, kring + (u % kRingK) * KP_BYTES + k_run, lane * 16, t * TILE_BYTES + k_run);
        };
        auto fill_v = [&](int t, int u) {
            issue_part<C::VP_LOADS>(kv_rsrc, vring + (u % kRingV) * VP_BYTES + v_run, lane * 16, t * TILE_BYTES + KP_BYTES + v_run);
        };
        // fill stream, in issue order:  K(0) K(1) K(2) V(0) | step 0: [V(1) K(3)] | step 1: [V(2) K(4)] | ...
#pragma unroll
        for (int u = 0; u < 3; ++u) fill_k(tile_at(u), u);
        fill_v(tile_at(0), 0);
        int t_v = tile_at(1), t_k = tile_at(3);

        V8 tqf[NC];
        {
            const unsigned off = q_off(qt0);
#pragma unroll
            for (int c = 0; c < NC; ++c) tqf[c] = *reinterpret_cast<const V8*>(tq_head + off + 32 * c);
        }
        f32x16 acc[NDB], acct[NDB];
        auto zero_acc = [&]() {
#pragma unroll
            for (int i = 0; i < NDB; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) { acc[i][e] = 0.f; acct[i][e] = 0.f; }
            }
        };
        zero_acc();
        float r_run = 0.f;
        const float sm_scale = p.sm_scale;
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        int f = 0, qi = 0;                       // position in the stream; query block of position f
        bool more = nq > 1;
        bool rows_in_flight = false;             // did the previous step fetch dQ rows? (they sit behind its fills in the queue)
        // Step f.  Kinds: A = position 0 of a block (waits chunk by chunk for the dQ rows fetched in the step before;
        // the tile it accumulates closes the previous block); B = positions 1 .. n-2; C = position n-1, the block's last
        // dS^T product, which refills the dQ registers chunk by chunk.
        //   phase 1: dS^T of tile f into `dn`, interleaved with p, dS^T (`dc`) of tile f-1 -> P^T, H^T, r
        //   phase 2: O^T, T^T += V^T P^T, V^T H^T of tile f-1
        auto one = [&](auto kind, const f32x16& dc, f32x16& dn) {
            constexpr int KIND = decltype(kind)::value;
            if (rows_in_flight) __builtin_amdgcn_s_waitcnt(WAIT_FILLS_ROWS); else __builtin_amdgcn_s_waitcnt(WAIT_FILLS);
            rows_in_flight = false;
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            fill_v(t_v, f + 1);
            fill_k(t_k, f + 3);
            const bool has_prev = KIND != 0 || f > 0, has_next = KIND != 0 || f < n_flat;
            const char* const kpart = kring + (f % kRingK) * KP_BYTES;
            const char* const p_in = smem + p_base + ((f - 1) & 1) * 4 * C::P_BYTES;
            V8 pf[2], hf[2];
            f32x4 pv[4];                              // p of tile f-1, fetched one piece of four elements ahead of its use
            float alpha = 1.0f;                       // rescale factor that goes with tile f-1: applies to what was summed before it
            if (has_prev) {
                pv[0] = *reinterpret_cast<const f32x4*>(p_in);
                alpha = *reinterpret_cast<const float*>(smem + alpha_base + ((f - 1) & 1) * 4 * 256);
                r_run *= alpha;
            }
            auto mix_chunk = [&](int c) {
#pragma unroll
                for (int k = 0; k < EPC; ++k) {
                    const int e = c * EPC + k;
                    if ((e & 3) == 0 && e < 12) pv[(e >> 2) + 1] = *reinterpret_cast<const f32x4*>(p_in + ((e >> 2) + 1) * kFragBytes);
                    const float pe = pv[e >> 2][e & 3];
                    const float hv = pe * (dc[e] * sm_scale);
                    r_run += hv;
                    pf[e >> 3][e & 7] = (T)pe;
                    hf[e >> 3][e & 7] = (T)hv;
                }
            };
            const bool refill = KIND == 2 && more;
            if (has_next) {
                const unsigned off_n = refill ? q_off(qt0 + qi + 1) : 0u;
                V8 fa[NC];
#pragma unroll
                for (int i = 0; i < PD && i < NC; ++i) fa[i] = lds_frag(kpart, i);
#pragma unroll
                for (int e = 0; e < 16; ++e) dn[e] = 0.f;
                if (refill) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        SCHED_FENCE();
                        if (c + PD < NC) fa[c + PD] = lds_frag(kpart, c + PD);
                        SCHED_FENCE();
                        dn = mfma32(fa[c], tqf[c], dn);
                        mix_chunk(c);
                        SCHED_FENCE();
                        tqf[c] = *reinterpret_cast<const V8*>(tq_head + off_n + 32 * c);
                    }
                    rows_in_flight = true;
                } else {
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        SCHED_FENCE();
                        if (c + PD < NC) fa[c + PD] = lds_frag(kpart, c + PD);
                        SCHED_FENCE();
                        dn = mfma32(fa[c], tqf[c], dn);
                        if (has_prev) mix_chunk(c);
                        SCHED_FENCE();
                    }
                }
            } else if (has_prev) {
#pragma unroll
                for (int c = 0; c < NC; ++c) mix_chunk(c);
            }
            if (has_prev) {
                const char* const vpart = vring + ((f - 1) % kRingV) * VP_BYTES;
                V8 fv[NB];
#pragma unroll
                for (int i = 0; i < PD && i < NB; ++i) fv[i] = lds_frag(vpart, 2 * (i % NDB) + i / NDB);
                if (__any(alpha != 1.0f)) {   // some row's max moved (wavefront-uniform, rare after the first tiles)
#pragma unroll
                    for (int i = 0; i < NDB; ++i) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) { acc[i][e] *= alpha; acct[i][e] *= alpha; }
                    }
                }
#pragma unroll
                for (int g = 0; g < NB; ++g) {
                    const int c = g / NDB, db = g % NDB;
                    SCHED_FENCE();
                    if (g + PD < NB) fv[g + PD] = lds_frag(vpart, 2 * ((g + PD) % NDB) + (g + PD) / NDB);
                    SCHED_FENCE();
                    acc[db] = mfma32(fv[g], pf[c], acc[db]);
                    acct[db] = mfma32(fv[g], hf[c], acct[db]);
                }
                SCHED_FENCE();
            }
            if (KIND == 0 && has_prev) {
                // tile f-1 closed block qi-1:  O = acc / l ;  dO = (T - (r / l) acc) / l
                const float inv_l = *reinterpret_cast<const float*>(smem + stat_base + ((qi - 1) & 1) * 4 * 256);
                float r_lo, r_hi;
                both_halves(r_run, r_lo, r_hi);
                const float r_over_l = (r_lo + r_hi) * inv_l;
                // accumulator lane (j, hh) holds channels 32 db + 8 g + 4 hh .. +3 of row j: 8 bytes of 16-byte chunk
                // 4 db + g, which goes to chunk position (4 db + g) ^ (j mod CPR) of row j of the region
                // (the row address is made opaque here so that the 16 chunk addresses are computed on the spot, one XOR
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
                                ov[r] = (T)(acc[db][4 * g + r] * inv_l);
                                tov[r] = (T)((acct[db][4 * g + r] - r_over_l * acc[db][4 * g + r]) * inv_l);
                            }
                            asm volatile("ds_write_b64 %0, %1" ::"v"(a), "v"(ov) : "memory");
                            asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(a), "v"(tov), "n"(32 * ST::ROW_BYTES) : "memory");
                        }
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xC07F);   // the region is complete before the next barrier publishes it
                zero_acc();
                r_run = 0.f;
            }
            t_v = wrap_inc(t_v); t_k = wrap_inc(t_k);
            ++f;
        };
        f32x16 d0, d1;
        // d0 and d1 swap roles every step; a block always starts with tile f-1's dS^T in d0
        for (qi = 0; qi < nq; ++qi) {
            more = qi + 1 < nq;
            one(KindA(), d0, d1);
            int s_in = 1;
            for (; s_in + 2 <= n - 1; s_in += 2) {
                one(KindB(), d1, d0);
                one(KindB(), d0, d1);
            }
            if (s_in < n - 1) {
                one(KindB(), d1, d0);
                d1 = d0;
            }
            one(KindC(), d1, d0);
        }
        one(KindA(), d0, d1);                    // step n_flat: the last tile, the last block
        __builtin_amdgcn_s_barrier();            // hands the last block to the score wavefronts
        __builtin_amdgcn_s_waitcnt(0x0F70);      // drain the (unused) trailing fills before the LDS is released
    }
}
