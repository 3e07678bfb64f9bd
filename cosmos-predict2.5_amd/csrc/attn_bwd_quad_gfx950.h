// dK/dV kernel of the backward for head dim 128, four wavefront roles ("quad").  Included inside the anonymous namespace of
// attn_bwd_gfx950.hip (uses BwdParams, kRows, kBlock, kBwdThreads, kBwdSweepStagger and attn_common_gfx950.h).
//
// Same mathematics and stream as attn_bwd_kernel<T, D, KIND_DKDV> (a workgroup owns 128 keys and streams 32-query tiles
// [Q | dO | dO^T | Q^T | LSE log2e, D]), other division of labour.  There every MFMA takes a fresh 1 KB A fragment from LDS
// and the four wavefront pairs of a workgroup each read the whole stream tile: 1.13 KB of LDS operand per MFMA.  Here a group of
// four wavefronts serves 64 keys, so that every stream fragment feeds two MFMAs, and each wavefront has one job:
//   S1  S = Q k^T for its 64 keys (K rows are register-resident B operands), U = P = exp2(S c - LSE') rounded to 16 bit,
//       handed over through LDS;
//   S2  dP = dO v^T (V rows register-resident), W = dS = U * (dP - D) rounded to 16 bit, handed over through LDS and,
//       when dS is kept, stored to memory;
//   O1  dV^T += dO^T U   (accumulators for 64 keys x 128 channels);
//   O2  dK^T += Q^T W.
// 16 MFMAs per wavefront and step for all four; the elementwise work is split between S1 and S2; 0.69 KB of LDS operand per
// MFMA.  Two such groups per workgroup (8 wavefronts, two per SIMD: one of S1 / S2 and one of O1 / O2).  W is formed from the
// ROUNDED P (the hand-over holds 16-bit values); the reference's kernel multiplies before rounding, the difference is one more
// relative rounding of 2^-9 (bf16) on dS.
//
// Pipeline, step s (tile = sweep position):   S1: MFMAs S(s+1) | U(s)      S2: MFMAs dP(s) | W(s-1)
//                                             O1: tile s-1                 O2: tile s-2
// LDS: rings of the four stream parts (Q 4 deep, dO 4, dO^T 3, Q^T 3: a part is fetched two to three steps before its one
// step of use), U and W hand-over (two stages each), statistics ring (6).  All direct-to-LDS fills are issued by the O
// wavefronts (nine 1 KB loads per wavefront and step); one s_barrier per step.

template <int D>
struct QuadCfg {
    static_assert(D == 128, "built for head dim 128");
    static constexpr int NC = D / 16, NDB = D / 32;
    static constexpr int KP_BYTES = NC * kFragBytes;          // Q part, dO part of a tile (K-type fragments)
    static constexpr int TP_BYTES = 2 * NDB * kFragBytes;     // dO^T part, Q^T part (V^T-type fragments)
    static constexpr int Q_SRC = 0, DO_SRC = KP_BYTES, DOT_SRC = 2 * KP_BYTES, QT_SRC = 2 * KP_BYTES + TP_BYTES, ST_SRC = 2 * KP_BYTES + 2 * TP_BYTES;
    static constexpr int TILE_BYTES = ST_SRC + kFragBytes;    // = the image of attn_bwd_kernel's query stream
    static constexpr int RQ = 4, RDO = 4, RDOT = 3, RQT = 3, RST = 6;
    static constexpr int HO_BYTES = 4 * kFragBytes;           // hand-over of one group and stage: 64 keys x 32 queries, 16 bit
    static constexpr int Q_OFF = 0;
    static constexpr int DO_OFF = Q_OFF + RQ * KP_BYTES;
    static constexpr int DOT_OFF = DO_OFF + RDO * KP_BYTES;
    static constexpr int QT_OFF = DOT_OFF + RDOT * TP_BYTES;
    static constexpr int U_OFF = QT_OFF + RQT * TP_BYTES;     // [2 stages][2 groups]
    static constexpr int W_OFF = U_OFF + 4 * HO_BYTES;
    static constexpr int ST_OFF = W_OFF + 4 * HO_BYTES;
    static constexpr int LDS_BYTES = ST_OFF + RST * kFragBytes;
    static constexpr int LOADS = 9;                           // per O wavefront and step: 2 fragments of each part + the statistics
    static constexpr int IN_FLIGHT = 14;                      // at the top of a step: all but the newest 14 loads must have landed
};

template <typename T, int D, bool SPILL>
__global__ void __attribute__((amdgpu_flat_work_group_size(kBwdThreads, kBwdThreads), amdgpu_waves_per_eu(2, 2)))
attn_dkdv_quad_kernel(const BwdParams p) {
    typedef QuadCfg<D> C;
    typedef typename VecOf<T>::v8 V8;
    typedef typename VecOf<T>::v4 V4;
    constexpr int NC = C::NC, NDB = C::NDB, NB = 2 * NDB;
    constexpr int PD = 2, PDO = 2;      // LDS operand fetches run this many MFMA groups ahead of use, S / O roles (4, 6, 8 for the O roles, 4 / 4: 1 % slower)
    constexpr int WAIT_FILLS = (C::IN_FLIGHT & 15) | ((C::IN_FLIGHT >> 4) << 14) | 0x0F70;

    const int bid = blockIdx.x;
    const bool partial = bid >= p.n_full && p.splits > 1;
    const int pair = partial ? p.n_full + (bid - p.n_full) / p.splits : bid;
    const int split = partial ? (bid - p.n_full) % p.splits : 0;
    const int blk = pair % p.n_blk, bhl = pair / p.n_blk, bh = p.bh0 + bhl, b = bh / p.H, h = bh % p.H;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool s_role = wave < 4;                 // waves 0..3: S1, S2 of group 0, S1, S2 of group 1; waves 4..7: O1, O2, O1, O2
    const bool second = (wave & 1) != 0;          // S2 / O2
    const int grp = (wave >> 1) & 1;
    const int ow = wave & 3;                      // O wavefronts: which quarter of each stream part this one copies
    const int j = lane & 31, hh = lane >> 5;
    const int row0 = blk * kBlock + grp * 64;     // first key of this group
    const bool causal = p.causal != 0;

    int t_lo = 0, t_hi = p.n_tiles;
    if (causal) t_lo = (blk * kBlock) / kRows;    // query tiles before the block's first key see none of its keys
    if (partial) {
        t_lo = (int)((int64_t)split * p.n_tiles / p.splits);
        t_hi = (int)((int64_t)(split + 1) * p.n_tiles / p.splits);
    }
    const int n = t_hi > t_lo ? t_hi - t_lo : 0;
    const int n_sweep = n > 0 ? n : 1;
    const int shift = (((pair >> 3) & 31) * kBwdSweepStagger) % n_sweep;
    auto tile_at = [&](int u) { return __builtin_amdgcn_readfirstlane(t_lo + (u + shift) % n_sweep); };
    auto wrap_inc = [&](int t) { ++t; return t >= t_lo + n_sweep ? t - n_sweep : t; };

    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(p.stream) + (size_t)bh * p.n_tiles * C::TILE_BYTES, 0, p.n_tiles * C::TILE_BYTES, 0x00020000);
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    auto frag = [&](const char* base, int f) { return *reinterpret_cast<const V8*>(base + f * kFragBytes + lane * 16); };

    // ---- fills (O wavefronts): this wavefront's two fragments of a part of tile t into ring slot u
    const int run = 2 * ow * kFragBytes;
    auto fill_part = [&](int src_off, int dst_off, int part_bytes, int ring, int t, int u) {
        issue_part<2>(rsrc, smem + dst_off + (u % ring) * part_bytes + run, lane * 16, t * C::TILE_BYTES + src_off + run);
    };
    auto fill_q = [&](int t, int u) {
        fill_part(C::Q_SRC, C::Q_OFF, C::KP_BYTES, C::RQ, t, u);
        lds_load<0>(rsrc, smem + C::ST_OFF + (u % C::RST) * kFragBytes, lane * 16, t * C::TILE_BYTES + C::ST_SRC);
    };
    auto fill_do = [&](int t, int u) { fill_part(C::DO_SRC, C::DO_OFF, C::KP_BYTES, C::RDO, t, u); };
    auto fill_dot = [&](int t, int u) { fill_part(C::DOT_SRC, C::DOT_OFF, C::TP_BYTES, C::RDOT, t, u); };
    auto fill_qt = [&](int t, int u) { fill_part(C::QT_SRC, C::QT_OFF, C::TP_BYTES, C::RQT, t, u); };
    if (!s_role) {   // what steps -3, -2, -1 would have issued
        fill_q(tile_at(0), 0); fill_do(tile_at(0), 0); fill_q(tile_at(1), 1);
        fill_do(tile_at(1), 1); fill_q(tile_at(2), 2);
        fill_dot(tile_at(0), 0); fill_do(tile_at(2), 2); fill_q(tile_at(3), 3);
    }

    const unsigned u_base = C::U_OFF + grp * C::HO_BYTES, w_base = C::W_OFF + grp * C::HO_BYTES;   // + stage * 2 * HO_BYTES

    if (s_role) {
        // ------------------------------------------------------------------------------------------ S1 / S2
        V8 breg[2][NC];             // stationary rows as B operands: K (S1) or V (S2) of keys row0 + 32 hf + j
        {
            const void* st = second ? p.st2 : p.st1;
            const int64_t sb = second ? p.s2_sb : p.s1_sb, sh = second ? p.s2_sh : p.s1_sh, sl = second ? p.s2_sl : p.s1_sl;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int row = row0 + 32 * hf + j;
                const T* ptr = reinterpret_cast<const T*>(st) + (int64_t)b * sb + (int64_t)h * sh + (int64_t)row * sl + 8 * hh;
                const bool live = row < p.L_stat;
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const V8 z = {0, 0, 0, 0, 0, 0, 0, 0};
                    breg[hf][c] = live ? *reinterpret_cast<const V8*>(ptr + 16 * c) : z;
                }
            }
        }
        f32x16 x0[2], x1[2];        // S (S1) or dP (S2) of two tiles, swapping roles every step; [key half]
        __builtin_amdgcn_s_waitcnt(0x0F70);   // the stationary rows are here
        __builtin_amdgcn_s_barrier();         // ... and so are the first stream tiles
        asm volatile("" ::: "memory");

        if (!second) {
            // ---------------------------------------------------------------- S1
            // causal: key (stationary) > query (streamed) possible iff last key of the group > first query of the tile
            auto need_mask = [&](int t) { return causal && row0 + 63 > t * kRows; };
            auto mask = [&](f32x16* x, int t) {
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int qrow = t * kRows + 8 * (e >> 2) + 4 * hh + (e & 3);
                        x[hf][e] = (row0 + 32 * hf + j <= qrow) ? x[hf][e] : -INFINITY;
                    }
                }
            };
            // scores of the first tile
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
                for (int e = 0; e < 16; ++e) x0[hf][e] = 0.f;
            }
            if (n > 0) {
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const V8 fa = frag(smem + C::Q_OFF, c);
                    x0[0] = mfma32(fa, breg[0][c], x0[0]);
                    x0[1] = mfma32(fa, breg[1][c], x0[1]);
                }
                if (need_mask(tile_at(0))) mask(x0, tile_at(0));
            }
            int t_next = tile_at(1);      // tile whose scores the step computes
            // one step: MFMAs of S(s+1) into xn (if NEXT) interleaved with U(s) from x (if CUR)
            auto step = [&](auto NEXT, auto CUR, const f32x16* x, f32x16* xn, int s) {
                constexpr bool next = decltype(NEXT)::value, cur = decltype(CUR)::value;
                const char* qpart = smem + C::Q_OFF + ((s + 1) % C::RQ) * C::KP_BYTES;
                const char* stats = smem + C::ST_OFF + (s % C::RST) * kFragBytes;
                V8 uf[2][2];
                V8 fa[NC];
                float l2v[16];
                if (next) {
#pragma unroll
                    for (int i = 0; i < PD; ++i) fa[i] = frag(qpart, i);
                }
                if (cur) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float4 a = *reinterpret_cast<const float4*>(stats + 64 * hh + 16 * i);
                        l2v[4 * i] = a.x; l2v[4 * i + 1] = a.y; l2v[4 * i + 2] = a.z; l2v[4 * i + 3] = a.w;
                    }
                }
                if (next) {
#pragma unroll
                    for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) xn[hf][e] = 0.f;
                    }
                }
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    SCHED_FENCE();
                    if (next && c + PD < NC) fa[c + PD] = frag(qpart, c + PD);
                    SCHED_FENCE();
#pragma unroll
                    for (int hf = 0; hf < 2; ++hf) {
                        if (next) xn[hf] = mfma32(fa[c], breg[hf][c], xn[hf]);
                        if (cur) {   // two elements of this key half behind each MFMA
#pragma unroll
                            for (int k = 0; k < 2; ++k) {
                                const int e = 2 * c + k;
                                const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(x[hf][e], p.scale_log2, -l2v[e]));
                                uf[hf][e >> 3][e & 7] = (T)pe;
                            }
                        }
                        SCHED_FENCE();
                    }
                }
                if (cur) {
                    const unsigned ua = lds0 + u_base + (s & 1) * 2 * C::HO_BYTES + 16 * lane;
                    asm volatile("ds_write_b128 %0, %1" ::"v"(ua), "v"(uf[0][0]) : "memory");
                    asm volatile("ds_write_b128 %0, %1 offset:1024" ::"v"(ua), "v"(uf[0][1]) : "memory");
                    asm volatile("ds_write_b128 %0, %1 offset:2048" ::"v"(ua), "v"(uf[1][0]) : "memory");
                    asm volatile("ds_write_b128 %0, %1 offset:3072" ::"v"(ua), "v"(uf[1][1]) : "memory");
                }
            };
            auto body = [&](int s, f32x16* cur, f32x16* nxt) {
                __builtin_amdgcn_s_waitcnt(0xC07F);   // own hand-over stores of the step before are done
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                if (s + 1 < n) {
                    step(std::true_type(), std::true_type(), cur, nxt, s);
                    if (need_mask(t_next)) mask(nxt, t_next);
                } else if (s < n) {
                    step(std::false_type(), std::true_type(), cur, nxt, s);
                }
                t_next = wrap_inc(t_next);
            };
            for (int s = 0; s <= n + 1; s += 2) {
                body(s, x0, x1);
                if (s + 1 <= n + 1) body(s + 1, x1, x0);
            }
        } else {
            // ---------------------------------------------------------------- S2
            // Inside a 2 KB tile the 16-byte unit (query half c', key, lane half hh) sits at slot 16 (key / 4) + 8 c' + 4 hh + key % 4: the
            // order in which the transposing reads of attn_dq_from_ds_kernel touch 256 consecutive bytes per pass (no bank conflicts).
            char* const ds_lane = SPILL ? p.ds + (int64_t)bhl * p.ds_head_bytes + ((int64_t)(4 * blk + 2 * grp) * 2 * kFragBytes + 16 * (16 * (j >> 2) + 4 * hh + (j & 3))) : nullptr;
            const int64_t ds_row = (int64_t)p.n_kt_pad * 2 * kFragBytes;
            int t_prev = tile_at(0);      // tile whose W the step forms (sweep position s - 1)
            // one step: MFMAs of dP(s) into xc (if CUR) interleaved with W(s-1) = U(s-1) * (dP(s-1) - D) from xp (if PREV)
            auto step = [&](auto CUR, auto PREV, f32x16* xc, const f32x16* xp, int s) {
                constexpr bool cur = decltype(CUR)::value, prev = decltype(PREV)::value;
                const char* dopart = smem + C::DO_OFF + (s % C::RDO) * C::KP_BYTES;
                const char* stats = smem + C::ST_OFF + ((s + C::RST - 1) % C::RST) * kFragBytes;
                const char* uin = smem + u_base + ((s + 1) & 1) * 2 * C::HO_BYTES;
                V8 ui[2][2], wf[2][2];
                V8 fb[NC];
                float ddv[16];
                if (prev) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) ui[i >> 1][i & 1] = frag(uin, i);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float4 a = *reinterpret_cast<const float4*>(stats + 128 + 64 * hh + 16 * i);
                        ddv[4 * i] = a.x; ddv[4 * i + 1] = a.y; ddv[4 * i + 2] = a.z; ddv[4 * i + 3] = a.w;
                    }
                }
                if (cur) {
#pragma unroll
                    for (int i = 0; i < PD; ++i) fb[i] = frag(dopart, i);
#pragma unroll
                    for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) xc[hf][e] = 0.f;
                    }
                }
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    SCHED_FENCE();
                    if (cur && c + PD < NC) fb[c + PD] = frag(dopart, c + PD);
                    SCHED_FENCE();
#pragma unroll
                    for (int hf = 0; hf < 2; ++hf) {
                        if (cur) xc[hf] = mfma32(fb[c], breg[hf][c], xc[hf]);
                        if (prev) {
#pragma unroll
                            for (int k = 0; k < 2; ++k) {
                                const int e = 2 * c + k;
                                const float we = (float)ui[hf][e >> 3][e & 7] * (xp[hf][e] - ddv[e]);
                                wf[hf][e >> 3][e & 7] = (T)we;
                            }
                        }
                        SCHED_FENCE();
                    }
                }
                if (prev) {
                    const unsigned wa = lds0 + w_base + ((s + 1) & 1) * 2 * C::HO_BYTES + 16 * lane;
                    asm volatile("ds_write_b128 %0, %1" ::"v"(wa), "v"(wf[0][0]) : "memory");
                    asm volatile("ds_write_b128 %0, %1 offset:1024" ::"v"(wa), "v"(wf[0][1]) : "memory");
                    asm volatile("ds_write_b128 %0, %1 offset:2048" ::"v"(wa), "v"(wf[1][0]) : "memory");
                    asm volatile("ds_write_b128 %0, %1 offset:3072" ::"v"(wa), "v"(wf[1][1]) : "memory");
                    if (SPILL) {   // the two 32-key tiles of dS of this group: [stream tile][4 blk + 2 grp + hf], this lane's 2 x 16 bytes each
                        char* dst = ds_lane + t_prev * ds_row;
                        __builtin_nontemporal_store(wf[0][0], reinterpret_cast<V8*>(dst));
                        __builtin_nontemporal_store(wf[0][1], reinterpret_cast<V8*>(dst + 128));
                        __builtin_nontemporal_store(wf[1][0], reinterpret_cast<V8*>(dst + 2 * kFragBytes));
                        __builtin_nontemporal_store(wf[1][1], reinterpret_cast<V8*>(dst + 2 * kFragBytes + 128));
                    }
                }
            };
            auto body = [&](int s, f32x16* cur, f32x16* prv) {
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                if (s >= 1 && s < n) step(std::true_type(), std::true_type(), cur, prv, s);
                else if (s < n) step(std::true_type(), std::false_type(), cur, prv, s);
                else if (s >= 1 && s == n) step(std::false_type(), std::true_type(), cur, prv, s);
                if (s >= 1 && s <= n) t_prev = wrap_inc(t_prev);
            };
            for (int s = 0; s <= n + 1; s += 2) {
                body(s, x0, x1);
                if (s + 1 <= n + 1) body(s + 1, x1, x0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0070);
    } else {
        // ------------------------------------------------------------------------------------------ O1 / O2
        f32x16 acc[2][NDB];         // dV^T (O1) or dK^T (O2): [key half][32-channel block]
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
            for (int i = 0; i < NDB; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[hf][i][e] = 0.f;
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        int t_qt = tile_at(0), t_dot = tile_at(1), t_do = tile_at(3), t_q = tile_at(4);
        const int lag = second ? 2 : 1;                       // O1 accumulates tile s-1, O2 tile s-2
        for (int s = 0; s <= n + 1; ++s) {
            __builtin_amdgcn_s_waitcnt(WAIT_FILLS);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const int u = s - lag;                             // sweep position accumulated in this step
            const bool active = u >= 0 && u < n;
            const char* apart = second ? smem + C::QT_OFF + ((u + C::RQT) % C::RQT) * C::TP_BYTES
                                       : smem + C::DOT_OFF + ((u + C::RDOT) % C::RDOT) * C::TP_BYTES;
            // U(u) was written in step u (stage u & 1), W(u) in step u + 1 (stage u & 1 as well)
            const char* hin = smem + (second ? w_base : u_base) + (u & 1) * 2 * C::HO_BYTES;
            V8 bf[2][2];
            V8 fa[NB];
            if (active) {
#pragma unroll
                for (int i = 0; i < 4; ++i) bf[i >> 1][i & 1] = frag(hin, i);
#pragma unroll
                for (int i = 0; i < PDO; ++i) fa[i] = frag(apart, 2 * (i % NDB) + i / NDB);
            }
            SCHED_FENCE();
            // Q^T(s), dO^T(s+1), dO(s+3), Q(s+4) + statistics(s+4): into slots that were read for the last time in step s-1 or before
            fill_qt(t_qt, s); fill_dot(t_dot, s + 1); fill_do(t_do, s + 3); fill_q(t_q, s + 4);
            t_qt = wrap_inc(t_qt); t_dot = wrap_inc(t_dot); t_do = wrap_inc(t_do); t_q = wrap_inc(t_q);
            SCHED_FENCE();
            if (active) {
#pragma unroll
                for (int g = 0; g < NB; ++g) {
                    const int c = g / NDB, db = g % NDB;
                    SCHED_FENCE();
                    if (g + PDO < NB) fa[g + PDO] = frag(apart, 2 * ((g + PDO) % NDB) + (g + PDO) / NDB);
                    SCHED_FENCE();
                    acc[0][db] = mfma32(fa[g], bf[0][c], acc[0][db]);
                    acc[1][db] = mfma32(fa[g], bf[1][c], acc[1][db]);
                }
            }
            SCHED_FENCE();
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // drain the (unused) trailing fills before the LDS is released
        // ---- epilogue: dV = dV^T (O1), dK = s dK^T (O2)
        const float sc = second ? p.sm_scale : 1.0f;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int wrow = grp * 64 + 32 * hf + j, row = blk * kBlock + wrow;
            if (partial) {   // a range of the stream only: leave the sums for bwd_combine_kernel ([row][dV | dK])
                const int64_t slot = (int64_t)(pair - p.n_full) * p.splits + split;
                float* pa = p.part + (slot * kBlock + wrow) * (2 * D) + (second ? D : 0);
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d = 32 * db + 8 * g + 4 * hh;
                        *reinterpret_cast<float4*>(pa + d) = make_float4(acc[hf][db][4 * g], acc[hf][db][4 * g + 1], acc[hf][db][4 * g + 2], acc[hf][db][4 * g + 3]);
                    }
                }
            } else if (row < p.L_stat) {
                T* out = second ? reinterpret_cast<T*>(p.out2) + (int64_t)b * p.o2_sb + (int64_t)h * p.o2_sh + (int64_t)row * p.o2_sl
                                : reinterpret_cast<T*>(p.out1) + (int64_t)b * p.o1_sb + (int64_t)h * p.o1_sh + (int64_t)row * p.o1_sl;
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d = 32 * db + 8 * g + 4 * hh;   // registers 4g..4g+3 are 4 consecutive channels
                        V4 v;
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] = (T)(acc[hf][db][4 * g + r] * sc);
                        *reinterpret_cast<V4*>(out + d) = v;
                    }
                }
            }
        }
    }
}
