// Pieces shared by the gfx950 attention kernels (forward + JVP, backward): vector types, the MFMA wrapper, the
// 1 KB operand-fragment constant, direct-to-LDS loads.  Included inside each translation unit's anonymous namespace.
#ifndef COSMOS_ATTN_COMMON_GFX950_H
#define COSMOS_ATTN_COMMON_GFX950_H

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

// A value that exists once per 32-lane half of a wavefront, made visible to both halves: afterwards, in every lane l,
// `lo` is what lane l % 32 held and `hi` what lane 32 + l % 32 held (one v_permlane32_swap, no LDS round trip).  The
// instruction is written out: given one value for both of its operands, the compiler's builtin treats its two results as
// equal and drops one of them.  (s_nop: the instruction may not directly follow the VALU write of its operands.)
__device__ __forceinline__ void both_halves(float x, float& lo, float& hi) {
    unsigned a = __builtin_bit_cast(unsigned, x), b = a;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    lo = __builtin_bit_cast(float, a);
    hi = __builtin_bit_cast(float, b);
}

constexpr int kFragBytes = 1024;   // one MFMA A-operand fragment: 64 lanes x 16 B
// The running row max that the softmax exponentials refer to is allowed to lag the true one: it moves (and everything
// summed so far is rescaled) only when some row of the wavefront has a score more than kMaxSlack above it, in log2
// units, so p = exp2(s c - m) stays below 2^kMaxSlack.  O = sum p v / sum p and LSE = m + log2 sum p hold for any
// reference m, and 16-bit rounding of p is relative, so nothing is lost; what is gained is that the rescaling pass over
// the accumulators, which otherwise runs in nearly every one of a sweep's first dozens of steps (in every step of a short
// sweep), runs about once per sweep.
constexpr float kMaxSlack = 6.0f;
// With tangents H = p dS s is rounded to the 16-bit type as well, and fp16 has the range for |dS s| up to 65504 only while
// p <= 1 (the reference's range, flash_attention_jvp_triton.py:114,141); a p of up to 2^6 would overflow from |dS s| ~ 1e3 on.
// So fp16 with tangents keeps the exact running max; bf16 (8 exponent bits) and the forward-only kernels use the slack.
template <typename T>
__device__ __host__ constexpr float max_slack_of(bool with_tangents) {
    return (with_tangents && __is_same(T, _Float16)) ? 0.0f : kMaxSlack;
}
#ifndef COSMOS_ATTN_PREFETCH_GROUPS
#define COSMOS_ATTN_PREFETCH_GROUPS 2   // LDS operand fetches run this many MFMA groups ahead of use
#endif
// The forward + JVP kernels' two roles have depths of their own.  The output wavefront runs 6 groups ahead (measured at the
// 2B 720p shape, score / output depth: 2/2 137-138 ms, 4/4 134.6-135, 2/6 133.3, 2/8 133.6, 4/8 134.5): it has the
// registers for it, and its MFMAs are what fills the gaps the score wavefront leaves in the pipe.
#ifndef COSMOS_ATTN_PREFETCH_SCORE
#define COSMOS_ATTN_PREFETCH_SCORE 2
#endif
#ifndef COSMOS_ATTN_PREFETCH_OUTPUT
#define COSMOS_ATTN_PREFETCH_OUTPUT 6
#endif
#ifndef COSMOS_ATTN_SWEEP_STAGGER
#define COSMOS_ATTN_SWEEP_STAGGER 3   // tiles between the sweep starts of workgroups that share an L2 (measured at the 2B 720p
                                      // shape: same time for 1 .. 4; traffic past the L2 56 / 48 / 36-38 / 26 / 26 / 82 GB at 0 / 1 / 2 / 3 / 4 / 6)
#endif

#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// What one wavefront copies per step (one "load group"): its share of the V part of one tile and of the K part
// of another, as VP_LOADS + KP_LOADS wavefront-level direct-to-LDS loads.  buffer_load ... lds (MUBUF) rather than
// global_load_lds: the compiler's wait-count pass treats the latter as a FLAT access that may touch LDS and then
// turns every later LDS wait into lgkmcnt(0).  One wavefront-level load moves one fragment: lane l's 16 bytes
// (voffset = 16 l) land at dst + 16 l.  The share is a contiguous run of fragments (parts with fewer fragments
// than wavefronts are copied redundantly), so one LDS base (M0) and one scalar offset serve the whole run and the
// fragment index travels in the instruction's immediate offset, which is added to both addresses.
struct LoadJob {
    __amdgpu_buffer_rsrc_t rsrc;
    int lane_off;            // 16 * lane
    int k_src, v_src;        // byte offsets of this wavefront's runs in the packed buffer
    char *k_dst, *v_dst;     // LDS destinations of the runs
};
template <int IMM, int AUX = 0>   // AUX: cache policy bits of the instruction (2 = non-temporal)
__device__ __forceinline__ void lds_load(__amdgpu_buffer_rsrc_t rsrc, char* dst, int lane_off, int src) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, lane_off, src, IMM, AUX);
}
template <int LOADS>
__device__ __forceinline__ void issue_part(__amdgpu_buffer_rsrc_t rsrc, char* dst, int lane_off, int src) {
    lds_load<0>(rsrc, dst, lane_off, src);
    if (LOADS > 1) lds_load<kFragBytes>(rsrc, dst, lane_off, src);
    if (LOADS > 2) lds_load<2 * kFragBytes>(rsrc, dst, lane_off, src);
    if (LOADS > 3) lds_load<3 * kFragBytes>(rsrc, dst, lane_off, src);
}

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per (device, kernel).  A kernel's LDS size is a compile-time
// constant of its instantiation, so the call never needs repeating; keeping it out of the steady state also keeps
// the entry points usable while a stream is being captured into a graph.  (Needs <mutex>, <set>, <utility>.)
inline bool allow_lds(const void* fn, size_t bytes) {
    static std::mutex mu;
    static std::set<std::pair<int, const void*>> done;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return false; }
    std::lock_guard<std::mutex> lock(mu);
    if (done.count(std::make_pair(dev, fn))) return true;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    done.insert(std::make_pair(dev, fn));
    return true;
}

// One workgroup of the attention kernels fits on a compute unit, so a launch of n_pairs equal workgroups runs in rounds
// of kNumCUs and a partly filled last round costs a whole one.  The `rem` workgroups of that round may instead be cut
// into S ranges of their stream (keys or queries) each: rem * S shorter workgroups that take ceil(rem S / kNumCUs) / S
// of a round, plus a merge kernel.  Returns the smallest S (1 = leave it) that minimises that cost, among the S that
// leave every range at least kMinStepsPerSplit barrier steps, if it saves at least a tenth of a round.
constexpr int kNumCUs = 256;          // MI355X
constexpr int kMaxSplits = 16;
constexpr int kMinStepsPerSplit = 4;
inline int choose_splits(int rem, int n_steps) {
    if (rem <= 0) return 1;
    int best = 1;
    double best_cost = 1.0;
    for (int S = 2; S <= kMaxSplits && S * kMinStepsPerSplit <= n_steps; ++S) {
        const double cost = (double)((rem * S + kNumCUs - 1) / kNumCUs) / S;
        if (cost < best_cost - 1e-9) { best_cost = cost; best = S; }
    }
    return best_cost <= 0.9 ? best : 1;
}

// The workgroup-to-XCD maps and the rounds-of-kNumCUs arithmetic of the attention kernels assume a whole MI355X (256 compute
// units).  A partitioned device (CPX / DPX modes) reports fewer and would silently get wrong piece maps: looked up once per
// device ordinal, refused with a status code.  (Needs <mutex>.)
inline bool device_is_whole_mi355x() {
    static std::mutex mu;
    static signed char state[64] = {};   // 0 = not looked up, 1 = yes, -1 = no
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return false; }
    std::lock_guard<std::mutex> lock(mu);
    if (state[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) { (void)hipGetLastError(); return false; }
        state[dev] = n == kNumCUs ? 1 : -1;
    }
    return state[dev] == 1;
}

inline bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }
inline bool strides_ok(const int64_t* s) { return s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0; }
inline bool head_dim_ok(int d) { return d == 16 || d == 32 || d == 64 || d == 128; }

#endif
