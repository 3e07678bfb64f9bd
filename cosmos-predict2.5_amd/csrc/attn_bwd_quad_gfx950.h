// dK/dV kernel of the backward for head dim 128, four wavefront roles ("quad").  Included inside the anonymous namespace of
// attn_bwd_gfx950.hip (uses BwdParams, kRows, kBlock, kBwdThreads, kBwdSweepStagger and attn_common_gfx950.h).
//
// Same mathematics as attn_bwd_kernel<T, D, KIND_DKDV> (a workgroup owns 128 keys and streams 32-query tiles, there
// [Q | dO | dO^T | Q^T | LSE log2e, D]), other division of labour and a stream half the size.  There every MFMA takes a fresh 1 KB A fragment from LDS
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
//
// One copy of the stream.  A tile is [Q | dO | LSE log2e, D]: 32 rows x 128 channels of each tensor as 16-byte units
// (row q, 16-channel chunk cK, half hK: 8 channels).  S1 / S2 read them as MFMA A operands with ds_read_b128 (lane = row);
// O1 / O2 need the transposed operands (lane = channel, 8 rows per lane) and get them from the SAME units with the
// transposing read ds_read_b64_tr_b16 (within 16 lanes, lane i passes the address of 8 bytes -- row i of a 16 x 4 matrix M of
// 16-bit values -- and receives M[i/4 + 4k][i%4], k = 0..3): no second, transposed copy of the tile in memory, in the fills
// or in LDS.  For both kinds of read to be free of bank conflicts the units of a part are stored in the order
//     slot(q, cK, hK) = 16 (q/16 + 2 hK + 4 cK) + (q%4 + 4 ((q/4)%4 XOR (hK + 2 (cK%2)))):
// the 16 lanes of a ds_read_b128 pass (16 consecutive rows, one cK, one hK) and the 32 lanes of a transposing pass (4 rows x
// 2 chunks x 2 halves, both 8-byte halves of each unit) touch 256 consecutive-bank bytes each.  pack_stream_kernel writes the
// image in that order; the direct-to-LDS fills copy it linearly.
// LDS: rings of the two stream parts (Q 7 deep: fetched three steps before S1 uses it, kept until O2 has used it three steps
// later; dO 5 deep), U and W hand-over (two stages each), statistics ring (6).  All fills are issued by the O wavefronts (five
// 1 KB loads per wavefront and step); one s_barrier per step.  The O wavefronts' LDS reads are written as asm (the compiler
// would put vmcnt(0) in front of the transposing-read builtin: it takes it for an access that may alias the fills in flight),
// with their own lgkmcnt waits, each tied to the registers it makes valid.

template <int D>
struct QuadCfg {
    static_assert(D == 128, "built for head dim 128");
    static constexpr int NC = D / 16, NDB = D / 32;
    static constexpr int KP_BYTES = NC * kFragBytes;          // Q part, dO part of a tile
    static constexpr int Q_SRC = 0, DO_SRC = KP_BYTES, ST_SRC = 2 * KP_BYTES;
    static constexpr int TILE_FRAGS = 2 * NC + 1;
    static constexpr int TILE_BYTES = TILE_FRAGS * kFragBytes;
    static constexpr int RQ = 7, RDO = 5, RST = 6;
    static constexpr int HO_BYTES = 4 * kFragBytes;           // hand-over of one group and stage: 64 keys x 32 queries, 16 bit
    static constexpr int Q_OFF = 0;
    static constexpr int DO_OFF = Q_OFF + RQ * KP_BYTES;
    static constexpr int U_OFF = DO_OFF + RDO * KP_BYTES;     // [2 stages][2 groups]
    static constexpr int W_OFF = U_OFF + 4 * HO_BYTES;
    static constexpr int ST_OFF = W_OFF + 4 * HO_BYTES;
    static constexpr int LDS_BYTES = ST_OFF + RST * kFragBytes;
    static constexpr int LOADS = 5;                           // per O wavefront and step: 2 fragments of each part + the statistics
    static constexpr int IN_FLIGHT = 2 * LOADS;               // at the top of a step: all but the loads of the last two steps must have landed
};

typedef short quad_s16x4 __attribute__((ext_vector_type(4)));

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
    // A fragment cK of a stream part (lane = row j, half hh): byte offset of this lane's unit, for even / odd cK
    const int a_off[2] = {16 * quad_unit_slot(j, 0, hh), 16 * quad_unit_slot(j, 1, hh) - kFragBytes};
    auto afrag = [&](const char* part, int cK) { return *reinterpret_cast<const V8*>(part + cK * kFragBytes + a_off[cK & 1]); };

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
    if (!s_role) {   // what the steps before step 0 would have issued
        fill_q(tile_at(0), 0);
#pragma unroll
        for (int u = 0; u < 3; ++u) { fill_do(tile_at(u), u); fill_q(tile_at(u + 1), u + 1); }
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
                    const V8 fa = afrag(smem + C::Q_OFF, c);
                    x0[0] = mfma32(fa, breg[0][c], x0[0]);
                    x0[1] = mfma32(fa, breg[1][c], x0[1]);
                }
                if (need_mask(tile_at(0))) mask(x0, tile_at(0));
            }
            int t_next = tile_at(1);      // tile whose scores the step computes
            // one step: MFMAs of S(s+1) into xn (if NEXT) interleaved with U(s) from x (if CUR)
            float l2v[16];
            auto load_l2 = [&](const char* stats) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4 a = *reinterpret_cast<const float4*>(stats + 64 * hh + 16 * i);
                    l2v[4 * i] = a.x; l2v[4 * i + 1] = a.y; l2v[4 * i + 2] = a.z; l2v[4 * i + 3] = a.w;
                }
            };
            auto step = [&](auto NEXT, auto CUR, const f32x16* x, f32x16* xn, int s) {
                constexpr bool next = decltype(NEXT)::value, cur = decltype(CUR)::value;
                const char* qpart = smem + C::Q_OFF + ((s + 1) % C::RQ) * C::KP_BYTES;
                V8 uf[2][2];
                V8 fa[NC];
                if (next) {
#pragma unroll
                    for (int i = 0; i < PD; ++i) fa[i] = afrag(qpart, i);
                }
                if (cur) load_l2(smem + C::ST_OFF + (s % C::RST) * kFragBytes);
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
                    if (next && c + PD < NC) fa[c + PD] = afrag(qpart, c + PD);
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
            float ddv[16];
            auto load_dd = [&](const char* stats) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4 a = *reinterpret_cast<const float4*>(stats + 128 + 64 * hh + 16 * i);
                    ddv[4 * i] = a.x; ddv[4 * i + 1] = a.y; ddv[4 * i + 2] = a.z; ddv[4 * i + 3] = a.w;
                }
            };
            auto step = [&](auto CUR, auto PREV, f32x16* xc, const f32x16* xp, int s) {
                constexpr bool cur = decltype(CUR)::value, prev = decltype(PREV)::value;
                const char* dopart = smem + C::DO_OFF + (s % C::RDO) * C::KP_BYTES;
                const char* uin = smem + u_base + ((s + 1) & 1) * 2 * C::HO_BYTES;
                V8 ui[2][2], wf[2][2];
                V8 fb[NC];
                if (prev) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) ui[i >> 1][i & 1] = frag(uin, i);
                    load_dd(smem + C::ST_OFF + ((s + C::RST - 1) % C::RST) * kFragBytes);
                }
                if (cur) {
#pragma unroll
                    for (int i = 0; i < PD; ++i) fb[i] = afrag(dopart, i);
#pragma unroll
                    for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) xc[hf][e] = 0.f;
                    }
                }
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    SCHED_FENCE();
                    if (cur && c + PD < NC) fb[c + PD] = afrag(dopart, c + PD);
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
        int t_do = tile_at(3), t_q = tile_at(4);
        const int lag = second ? 2 : 1;                       // O1 accumulates tile s-1, O2 tile s-2
        // Transposing reads.  Lane (group g = lane / 16, r = lane % 16) is channel 16 (g%2) + r of a 32-channel block and key-index
        // half g/2 of the MFMA A operand; as a supplier of addresses it passes, for fragment (db, c) and read t, the 8 bytes of row
        // q = 16 c + 8 t + 4 (g/2) + r/4, channels 32 db + 16 (g%2) + 4 (r%4) .. + 3: unit (q, cK = 2 db + g%2, hK = (r%4)/2), its
        // second half when r is odd.  Byte offset in the part = 256 c + 2048 db + tr_off[t].
        const int g16 = lane >> 4, r16 = lane & 15, hK = (r16 & 3) >> 1;
        unsigned tr_off[2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
            tr_off[t] = (unsigned)(512 * hK + 1024 * (g16 & 1) + 16 * (r16 >> 2) + 64 * ((2 * t + (g16 >> 1)) ^ (hK + 2 * (g16 & 1))) + 8 * (r16 & 1));
// one MFMA group's A operand: fragment (db, c) = two transposing reads (t = 0, 1); IMM = 256 c + 2048 db
#define QUAD_TR_PAIR(g) asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%4\n\tds_read_b64_tr_b16 %1, %3 offset:%4" \
                                     : "=&v"(lo[g]), "=&v"(hi[g]) : "v"(ta0), "v"(ta1), "n"(256 * ((g) / NDB) + 2048 * ((g) % NDB)) : "memory")
// wait until at most N of this wavefront's LDS reads are outstanding; ties the registers the wait makes valid
#define QUAD_WAIT(N, g) asm volatile("s_waitcnt lgkmcnt(" #N ")" : "+v"(lo[g]), "+v"(hi[g]), "+v"(bf[0][0]), "+v"(bf[0][1]), "+v"(bf[1][0]), "+v"(bf[1][1]) :: "memory")
#define QUAD_GROUP(g) do { \
            const V8 fa = __builtin_shufflevector(__builtin_bit_cast(V4, lo[g]), __builtin_bit_cast(V4, hi[g]), 0, 1, 2, 3, 4, 5, 6, 7); \
            acc[0][(g) % NDB] = mfma32(fa, bf[0][(g) / NDB], acc[0][(g) % NDB]); \
            acc[1][(g) % NDB] = mfma32(fa, bf[1][(g) / NDB], acc[1][(g) % NDB]); } while (0)
        static_assert(NB == 8, "the MFMA groups below are written out for head dim 128");
        for (int s = 0; s <= n + 1; ++s) {
            __builtin_amdgcn_s_waitcnt(WAIT_FILLS);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const int u = s - lag;                             // sweep position accumulated in this step
            const bool active = u >= 0 && u < n;
            // O1: dO part of tile u; O2: Q part of tile u
            const unsigned part = lds0 + (second ? C::Q_OFF + ((u + C::RQ) % C::RQ) * C::KP_BYTES : C::DO_OFF + ((u + C::RDO) % C::RDO) * C::KP_BYTES);
            const unsigned ta0 = part + tr_off[0], ta1 = part + tr_off[1];
            // U(u) was written in step u (stage u & 1), W(u) in step u + 1 (stage u & 1 as well)
            const unsigned hin = lds0 + (second ? w_base : u_base) + (u & 1) * 2 * C::HO_BYTES + 16 * lane;
            V8 bf[2][2];
            quad_s16x4 lo[NB], hi[NB];
            if (active) {
                asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:1024\n\tds_read_b128 %2, %4 offset:2048\n\tds_read_b128 %3, %4 offset:3072"
                             : "=&v"(bf[0][0]), "=&v"(bf[0][1]), "=&v"(bf[1][0]), "=&v"(bf[1][1]) : "v"(hin) : "memory");
                QUAD_TR_PAIR(0); QUAD_TR_PAIR(1);
            }
            SCHED_FENCE();
            // dO(s+3), Q(s+4) + statistics(s+4): into slots that were read for the last time in step s-1 or before
            fill_do(t_do, s + 3); fill_q(t_q, s + 4);
            t_do = wrap_inc(t_do); t_q = wrap_inc(t_q);
            SCHED_FENCE();
            if (active) {
                QUAD_TR_PAIR(2); QUAD_WAIT(4, 0); QUAD_GROUP(0);
                QUAD_TR_PAIR(3); QUAD_WAIT(4, 1); QUAD_GROUP(1);
                QUAD_TR_PAIR(4); QUAD_WAIT(4, 2); QUAD_GROUP(2);
                QUAD_TR_PAIR(5); QUAD_WAIT(4, 3); QUAD_GROUP(3);
                QUAD_TR_PAIR(6); QUAD_WAIT(4, 4); QUAD_GROUP(4);
                QUAD_TR_PAIR(7); QUAD_WAIT(4, 5); QUAD_GROUP(5);
                QUAD_WAIT(2, 6); QUAD_GROUP(6);
                QUAD_WAIT(0, 7); QUAD_GROUP(7);
            }
            SCHED_FENCE();
        }
#undef QUAD_TR_PAIR
#undef QUAD_WAIT
#undef QUAD_GROUP
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
