// ADKV hot-path kernels for MI355X (gfx950, wave64) and their C ABI (include/adkv_hip.h).
//
// Work decomposition.  Every (batch, head, channel) is an independent fp16 recurrence over the
// time axis (reference: src/adkv/kernel/gemv.cu:187-191).  A LANE owns CPL consecutive channels of
// one head; D/CPL lanes make a head; a wave64 carries 64*CPL/D heads.  One supergroup (8 tokens) of
// a head is D*4 contiguous bytes, which the head's lanes fetch as one run of 16-byte loads; loads
// for the next PF supergroups are in flight while the current one is decoded.
//
// The recurrence rounds to fp16 at every step, so it cannot be re-associated: a sequence can only be
// split where the exact state is known.  The encoder therefore can record the state every
// `ckpt_interval` tokens ("checkpoints", 4 bytes per channel each); given those, the decode kernels
// cut the time axis into segments that replay independently and bit-exactly.  Without checkpoints
// they replay from token 0 exactly like the reference.  More waves matter on this machine: a SIMD
// needs about four resident waves to issue packed-f16 instructions at full rate.
//
// The kernels keep the reference's call structure (encode / QK+append / OV+append) so that they are
// drop-ins for src/adkv/kernel/gemv.cu:368-414, 883-939, 1233-1288.
#include "adkv_device.h"

#include "../../include/adkv_hip.h"

#include <stdlib.h>

#include <atomic>
#include <initializer_list>
#include <mutex>
#include <type_traits>

#pragma clang fp contract(off)

namespace adkv {

constexpr int PF = 4; // supergroups in flight per lane (2, 6 and 8 were measured: no difference)

template <int D, int CPL>
struct Geo {
    static constexpr int LPH = D / CPL;       // lanes per head
    static constexpr int NP = CPL / 2;        // channel pairs per lane
    // a lane's CPL code words of one supergroup, loaded as 16-byte vectors (8 bytes when the lane
    // owns only two channels)
    using Vec = typename std::conditional<CPL >= 4, uint4, uint2>::type;
    static constexpr int WPV = sizeof(Vec) / 4; // 32-bit channel words per vector
    static constexpr int NV = CPL / WPV;        // vectors per lane per supergroup
    static constexpr int VPS = D / WPV;         // vectors per supergroup of one head
    static_assert(LPH == 32 || LPH == 64, "a head must fit in one wave");
    static_assert(CPL == 2 || CPL % 4 == 0, "two channels per lane, or a multiple of four");
};

__device__ __forceinline__ void vec_words(const uint4 &u, uint32_t *w)
{
    w[0] = u.x; w[1] = u.y; w[2] = u.z; w[3] = u.w;
}
__device__ __forceinline__ void vec_words(const uint2 &u, uint32_t *w)
{
    w[0] = u.x; w[1] = u.y;
}
__device__ __forceinline__ void words_vec(const uint32_t *w, uint4 &u) { u = make_uint4(w[0], w[1], w[2], w[3]); }
__device__ __forceinline__ void words_vec(const uint32_t *w, uint2 &u) { u = make_uint2(w[0], w[1]); }
template <typename V> __device__ __forceinline__ V vec_zero();
template <> __device__ __forceinline__ uint4 vec_zero<uint4>() { return make_uint4(0, 0, 0, 0); }
template <> __device__ __forceinline__ uint2 vec_zero<uint2>() { return make_uint2(0, 0); }

// The code stream is read exactly once: a non-temporal load keeps it from displacing the logits
// and weights (which the softmax and the next kernel read back) in the caches.  Measured on the
// headline shape: forward_qk -1 %, forward_ov -3 %, the softmax between them -12 %.
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef uint32_t u2v32 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 load_codes(const uint4 *p)
{
    const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_codes(const uint2 *p)
{
    const u2v32 v = __builtin_nontemporal_load(reinterpret_cast<const u2v32 *>(p));
    return make_uint2(v.x, v.y);
}

// How the time axis is cut.  seg_tokens is a multiple of ckpt_interval (itself a multiple of 8);
// segment s covers tokens [s*seg_tokens, min((s+1)*seg_tokens, T)) and starts from checkpoint
// s*seg_tokens/ckpt_interval - 1 (segment 0 starts from the initial parameters).
struct Seg {
    h1 *ckpt;           // [B*H, n_ckpt_cap, D, 2] (zp, sc) before token (j+1)*ckpt_interval; may be null
    int n_ckpt_cap;
    int ckpt_interval;  // 0 when ckpt is null
    int seg_tokens;     // >= T when there is one segment
    int nseg;
    long row_pitch;     // elements between rows of the logits / attention-weight matrix (>= T + 1)
    int act_bf16;       // q, the new token and the output are bfloat16 (see load_act2 / store_act2)
    int combine;        // ov_ft_kernel: the segments' partial outputs are added inside the workgroup
    // Per-head-table kernels only.  groups > 0: the context's `intervals` checkpoint intervals are
    // cut into `groups` groups of four segments of unequal length (uneven_cut).  phys_per_head:
    // workgroups launched per KV head; each walks through the head's virtual workgroups pw,
    // pw + phys_per_head, ... one after the other (same table, no barrier between them).
    int groups;
    int intervals;
    int phys_per_head;
    unsigned skew;      // shares of the four wave slots, oldest first, one byte each, in sixteenths
};

__host__ __device__ inline int ft_skew(unsigned skew, int k) { return (int)((skew >> (8 * k)) & 0xFFu); }
constexpr unsigned pack_skew(unsigned a, unsigned b, unsigned c, unsigned d) { return a | (b << 8) | (c << 16) | (d << 24); }

// First checkpoint interval of the seg-th segment IN TIME ORDER (seg == 4*groups: one past the
// last) when `intervals` intervals are cut into `groups` groups of four uneven segments.  Group g
// covers [intervals*g/groups, intervals*(g+1)/groups); inside it the shares are rounded down, every
// segment gets at least one interval, and what is left goes to the oldest slots first.  The
// shares are listed oldest wave slot first and laid out LATEST segment first: the oldest slot
// takes the group's last segment (the longest), the youngest its first (see segment_of_slot).
// Needs at least four intervals per group.  The same function plans on the host and indexes on
// the device.
__host__ __device__ inline int uneven_cut(int seg, int groups, int intervals, unsigned skew)
{
    const int g = seg >> 2, k = seg & 3;
    const int lo = (int)((long)intervals * g / groups);
    if (k == 0)
        return lo;
    const int n = (int)((long)intervals * (g + 1) / groups) - lo;
    int part[4], left = n; // by wave slot, oldest first
    for (int i = 0; i < 4; i++) {
        part[i] = n * ft_skew(skew, i) / 16;
        if (part[i] < 1)
            part[i] = 1;
        left -= part[i];
    }
    for (int i = 0; left > 0; i = (i + 1) & 3, left--)
        part[i]++;
    for (int i = 0; left < 0; i = (i + 1) & 3) // only when n is tiny: take from the longest
        if (part[i] > 1) {
            part[i]--;
            left++;
        }
    int c = lo;
    for (int i = 0; i < k; i++)
        c += part[3 - i];
    return c;
}

// Which segment (in time order) the waves of slot index `seg` work on.  interleave_segment gives
// quad k of a workgroup slot index k of a group of four, and quad k is wave slot k of its SIMDs
// (oldest first).  In an uneven plan the oldest slot takes the group's LAST segment: that is where
// the work after the loop is (ragged tail, appended token, published state: a chain of dependent
// memory operations), and the oldest slot's waves are the first to finish their loop, so that
// work runs while the other slots are still in theirs instead of at the very end of the launch.
__host__ __device__ inline int segment_of_slot(const Seg &sa, int seg) { return sa.groups ? seg ^ 3 : seg; }

// first token of the segment of slot index `seg` / of the one after it in time; whether it is the
// last of the context
__host__ __device__ inline int seg_begin(const Seg &sa, int seg)
{
    return sa.groups ? uneven_cut(seg ^ 3, sa.groups, sa.intervals, sa.skew) * sa.ckpt_interval : seg * sa.seg_tokens;
}
__host__ __device__ inline int seg_end(const Seg &sa, int seg)
{
    return sa.groups ? uneven_cut((seg ^ 3) + 1, sa.groups, sa.intervals, sa.skew) * sa.ckpt_interval
                     : (seg + 1) * sa.seg_tokens;
}
__host__ __device__ inline bool seg_is_last(const Seg &sa, int seg) { return segment_of_slot(sa, seg) == sa.nseg - 1; }

__device__ __forceinline__ float wave_xor_add(float v, int mask)
{
    return v + __shfl_xor(v, mask, 64);
}

// s + s[lane ^ 8]: DPP rotate by 8 within each row of 16 lanes (no LDS round trip).
__device__ __forceinline__ float xor8_add(float s)
{
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0x128 /*row_ror:8*/,
                                              0xF, 0xF, false);
    return s + __builtin_bit_cast(float, r);
}

typedef unsigned u2v __attribute__((ext_vector_type(2)));

// s + s[lane ^ 16] / s + s[lane ^ 32] through the gfx950 row/half swap instructions.  Both the copy
// and the results go through opaque asm statements: handed two identical values, or asked for the
// float sum of the two results directly, this compiler folds the pair into one register.
__device__ __forceinline__ float xor16_add(float s)
{
    unsigned a = __builtin_bit_cast(unsigned, s), b;
    asm volatile("v_mov_b32 %0, %1" : "=v"(b) : "v"(a));
    const u2v r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
    unsigned x = r.x, y = r.y;
    asm volatile("" : "+v"(x), "+v"(y));
    return __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
}

__device__ __forceinline__ float xor32_add(float s)
{
    unsigned a = __builtin_bit_cast(unsigned, s), b;
    asm volatile("v_mov_b32 %0, %1" : "=v"(b) : "v"(a));
    const u2v r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    unsigned x = r.x, y = r.y;
    asm volatile("" : "+v"(x), "+v"(y));
    return __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
}

// Sum over the LPH lanes of a head; every lane of the head gets the total.
template <int LPH>
__device__ __forceinline__ float head_allreduce(float v)
{
#pragma unroll
    for (int m = 1; m < LPH; m <<= 1)
        v = wave_xor_add(v, m);
    return v;
}

// a.x*b.x + a.y*b.y in fp32, as the three-operand form with a literal zero accumulator: the
// accumulating two-operand form the compiler picks needs its destination cleared first, one more
// vector instruction per token.  The leading wait state covers an operand that the instruction
// just before wrote as a packed 16-bit result (on this chip such a result cannot be forwarded to
// the very next instruction; the compiler pads its own code the same way).
__device__ __forceinline__ float dot2_from_zero(h2 a, h2 b)
{
    float d;
    asm("s_nop 0\n\tv_dot2_f32_f16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
}

// Sum of 8 per-lane partials over the 32 lanes of a head, scattered: afterwards every lane holds
// the total of ONE token, token_of_lane(lane), the same in the four lanes of a quad.
//   bit 3 of the lane (banks 0,1 | 2,3): keep tokens 0-3 | 4-7, add the partner's    8 instructions
//   bit 2 (banks 0,2 | 1,3):             keep tokens +0,+1 | +2,+3                      4
//   bit 4 (row 0 | 1 of the head):       v_permlane16_swap + add, keep token +0 | +1    2
//   bits 0,1: all-reduce inside the quad                                                2
// A masked DPP add writes only the banks of its mask and keeps the other lanes' destination; a
// DPP operand must not have been written by the two preceding instructions, which the order
// below guarantees inside the block and the leading s_nop for whatever precedes it.
__device__ __forceinline__ float reduce8_head32(const float *p)
{
    float r0, r1, r2, r3, s0, s1;
    asm volatile(
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %6, %6 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %1, %7, %7 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %2, %8, %8 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %3, %9, %9 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %0, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %1, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %2, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %3, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        // banks 0,2 take lane+4 (rotate right by 12), banks 1,3 take lane-4 (rotate right by 4)
        "v_add_f32_dpp %4, %0, %0 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %5, %1, %1 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %4, %2, %2 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %5, %3, %3 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "s_nop 1\n\t"
        "v_permlane16_swap_b32 %4, %5\n\t"
        "s_nop 1\n\t"
        "v_add_f32 %4, %4, %5\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %4, %4, %4 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %4, %4, %4 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0"
        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(s0), "=&v"(s1)
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]));
    return s0;
}

__device__ __forceinline__ int token_of_lane(int lane)
{
    const int bank = (lane >> 2) & 3, row = (lane >> 4) & 1;
    return 4 * (bank >> 1) + 2 * (bank & 1) + row;
}

// The same for a head of 16 lanes (one row): after the two masked steps a lane holds two tokens'
// sums over the four lanes that differ from it in bits 2 and 3; lanes with bit 1 clear keep the
// first and take the partner's (lane ^ 2) first, the others the second, and bit 0 is an all-reduce.
// Every PAIR of lanes ends with one token's total, token_of_lane16(lane).
__device__ __forceinline__ float reduce8_head16(const float *p)
{
    float r0, r1, r2, r3, s0, s1, keep, give;
    const unsigned long long odd_pairs = 0xCCCCCCCCCCCCCCCCull; // lanes with bit 1 set
    asm volatile(
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %1, %9, %9 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %2, %10, %10 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %3, %11, %11 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %0, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %1, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %2, %14, %14 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %3, %15, %15 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %4, %0, %0 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %5, %1, %1 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %4, %2, %2 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %5, %3, %3 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_cndmask_b32_e64 %6, %4, %5, %16\n\t"
        "v_cndmask_b32_e64 %7, %5, %4, %16\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %6, %7, %6 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %6, %6, %6 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0"
        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(s0), "=&v"(s1), "=&v"(keep), "=&v"(give)
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]), "s"(odd_pairs));
    return keep;
}

__device__ __forceinline__ int token_of_lane16(int lane)
{
    const int bank = (lane >> 2) & 3;
    return 4 * (bank >> 1) + 2 * (bank & 1) + ((lane >> 1) & 1);
}

// The same sum over a head of LPH lanes: a 64-lane head adds its two halves at the end (both then
// hold every token's total).
template <int LPH>
__device__ __forceinline__ float reduce8_head(const float *p)
{
    const float s = reduce8_head32(p);
    return LPH == 64 ? xor32_add(s) : s;
}

// (zp, sc) of CPL consecutive channels <-> the interleaved [channel][2] fp16 layout used for
// state_out and checkpoints.
template <int CPL>
__device__ __forceinline__ void store_state(h1 *dst, const Pair *st)
{
    h2 *so = reinterpret_cast<h2 *>(dst);
#pragma unroll
    for (int p = 0; p < CPL / 2; p++) {
        so[2 * p] = (h2){st[p].zp.x, st[p].sc.x};
        so[2 * p + 1] = (h2){st[p].zp.y, st[p].sc.y};
    }
}

template <int CPL>
__device__ __forceinline__ void load_state(const h1 *src, Pair *st)
{
    const h2 *so = reinterpret_cast<const h2 *>(src);
#pragma unroll
    for (int p = 0; p < CPL / 2; p++) {
        const h2 a = so[2 * p], b = so[2 * p + 1];
        st[p].zp = (h2){a.x, b.x};
        st[p].sc = (h2){a.y, b.y};
    }
}

// store_state for any channel count, including a single channel held in both halves of a pair
template <int CPL>
__device__ __forceinline__ void store_state_n(h1 *dst, const Pair *st)
{
    if (CPL >= 2)
        store_state<CPL>(dst, st);
    else
        *reinterpret_cast<h2 *>(dst) = (h2){st[0].zp.x, st[0].sc.x};
}

// Which (head, segment) this lane works on.  Every segment's run of units is padded to whole
// waves, so all lanes of a wave work on the same segment and everything derived from it (token
// range, trip counts) is wave-uniform: the decode loops then branch on scalars instead of masking
// lanes.  Units past the end are clamped to a valid one and flagged inactive: they compute but
// never store.
//
// Consecutive waves take DIFFERENT segments of the same sequences (interleave_segment): the last
// segment of a context is shorter than the others whenever the length is not a multiple of the
// segment size (a 640-token context cut at 512 is a 512-token and a 128-token segment), and with
// all short waves in one workgroup and all long ones in another, half the CUs went idle after a
// quarter of the launch (B=128: 640 tokens took as long as 1024).  Mixed, every SIMD holds long
// and short waves and the long ones speed up when the short ones leave (two waves issue nearly as
// fast as four).
//
// wave index -> (segment, wave within the segment).  A wave's SIMD is its index modulo 4 (a
// workgroup's waves go round the SIMDs), so the mapping works on quads of waves: quad q takes
// segment q mod nseg, and its four waves are four consecutive waves' worth of units of that
// segment; every SIMD then walks through the segments in turn.  Each segment's waves are padded
// to a multiple of four (pad4); padding waves leave right after the table is built.
__host__ __device__ inline int pad4(int n) { return (n + 3) & ~3; }
__host__ __device__ inline void interleave_segment(int wave, int nseg, int &seg, int &wave_in_seg)
{
    const int q = wave >> 2, g = q / nseg;
    seg = q - g * nseg;
    wave_in_seg = g * 4 + (wave & 3);
}

template <int LPH>
static inline long padded_units(int BH, int nseg)
{
    constexpr int UPW = 64 / LPH; // units per wave
    return (long)nseg * pad4((BH + UPW - 1) / UPW) * UPW;
}

template <int D, int CPL, int BLK>
struct Unit {
    int bx, seg, lh, c0;
    bool active, wave_active;
    __device__ __forceinline__ Unit(int BH, int nseg)
    {
        using G = Geo<D, CPL>;
        constexpr int UPW = 64 / G::LPH;
        const int waves_per_seg = (BH + UPW - 1) / UPW;
        const long gl = (long)blockIdx.x * BLK + threadIdx.x;
        lh = (int)(gl % G::LPH);
        const int wave = __builtin_amdgcn_readfirstlane((int)(gl >> 6));
        int sg, wis;
        interleave_segment(wave, nseg, sg, wis);
        const int b = wis * UPW + (int)((gl & 63) / G::LPH);
        wave_active = wis < waves_per_seg;
        active = wave_active && b < BH;
        seg = sg;
        bx = b < BH ? b : BH - 1;
        c0 = lh * CPL;
    }
};

// Parameters plus the state this segment starts from.
template <int D, int CPL>
__device__ __forceinline__ void init_pairs(Pair *st, const h1 *zp, const h1 *sc, const h1 *al,
                                           const h1 *be, const h1 *tg, int h, int bx, int c0, int seg,
                                           const Seg &sa)
{
#pragma unroll
    for (int p = 0; p < CPL / 2; p++)
        load_pair(st[p], zp, sc, al, be, tg, h * D + c0 + 2 * p);
    if (seg_begin(sa, seg) > 0) {
        const int j = seg_begin(sa, seg) / sa.ckpt_interval - 1;
        load_state<CPL>(sa.ckpt + (((size_t)bx * sa.n_ckpt_cap + j) * D + c0) * 2, st);
    }
}

// ---------------------------------------------------------------------------------------------
// encode_kv  (gemv.cu:168-308)
// ---------------------------------------------------------------------------------------------
// The state at token t depends on every code before it, so the encoder is one serial chain per
// channel and nothing but B*H*D is parallel.  A lane owns CPL consecutive channels (1 or 2, the
// launcher's choice).  With few channels every wave has a SIMD to itself and the time per token
// is the length of its instruction stream, so that stream is kept short: the dependent chain from
// one token's state to the next is mixed-precision fma -> mul -> rint -> med3 -> pack -> packed
// mul -> packed fma, input rows are loaded two groups of 8 tokens ahead with nothing waiting on
// them, codes are summed as signed q << 4t in floats (one fma each) and biased once by 0x8888...,
// row pointers advance by addition, checkpoints are found by comparison.
constexpr int ENC_PF = 3; // supergroup input buffers in rotation

// Where the new rows are: element strides between batches, heads and tokens (channels are
// contiguous).  The encoder reads each row once, 256 bytes per head, so a [B, T, H, D] projection
// output viewed as [B, H, T, D] can be quantised in place without a packed copy.
struct RowStrides {
    long b, h, t;
};

template <int BITS, int CPL, int BLK, bool BF16 = false>
__device__ __forceinline__ void encode_body(
    uint32_t *__restrict__ cache, const h1 *__restrict__ kv_new, RowStrides xs,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int BH, int H, int T0, int T, int D, int n_super_cap, const h1 *__restrict__ state_in,
    h1 *__restrict__ state_out, const Seg &sa)
{
    // Quantises tokens [T0, T) of a stream whose first T0 tokens are already in the cache; kv_new
    // holds the T - T0 new rows; state_in is the state after token T0-1 (ignored when T0 == 0).
    constexpr int NP = CPL >= 2 ? CPL / 2 : 1;
    constexpr int TPW = Code<BITS>::TPW; // tokens per channel word
    constexpr int G8 = TPW / 8;          // 8-token input groups per word
    const long total = (long)BH * D;
    long ci = ((long)blockIdx.x * BLK + threadIdx.x) * CPL;
    const bool active = ci < total;
    if (!active)
        ci = total - CPL;
    const int bx = (int)(ci / D), c0 = (int)(ci % D);
    const int h = bx % H;

    Pair st[NP];
    if (CPL >= 2) {
#pragma unroll
        for (int p = 0; p < NP; p++)
            load_pair(st[p], zp, sc, al, be, tg, h * D + c0 + 2 * p);
    } else {
        const int pi = h * D + c0;
        st[0].zp = splat(zp[pi]);
        st[0].sc = splat(sc[pi]);
        st[0].al = splat(al[pi]);
        st[0].be = splat(be[pi]);
        st[0].omt = splat((h1)1.0f) - st[0].be * splat(tg[pi]);
    }
    if (T0 > 0) {
        const h1 *si = state_in + ((size_t)bx * D + c0) * 2;
        if (CPL >= 2) {
            load_state<CPL>(si, st);
        } else {
            st[0].zp = splat(si[0]);
            st[0].sc = splat(si[1]);
        }
    }

    uint32_t *cw = cache + (size_t)bx * n_super_cap * D + c0;
    const h1 *xb = kv_new + (long)(bx / H) * xs.b + (long)h * xs.h + c0; // rows of tokens T0.. of this head

    // One token's CPL channels as NP aligned 32-bit words of the input row (an fp16 pair each; a
    // one-channel lane takes the word its channel lies in and shifts at use).  The loads carry no
    // arithmetic, and no 16-bit values the compiler would pack in pairs across the loop edge, so
    // nothing waits for a load until its token is quantised.
    using XW = uint32_t;
    const h1 *xbw = xb - (CPL == 1 ? (c0 & 1) : 0);
    const uint32_t xsh = CPL == 1 ? (uint32_t)(c0 & 1) * 16u : 0u;
    auto load_tok = [&](int t, XW *x) {
#pragma unroll
        for (int p = 0; p < NP; p++)
            x[p] = *reinterpret_cast<const XW *>(xbw + (long)(t - T0) * xs.t + 2 * p);
    };
    // reciprocal of the current scale, refreshed right after every update (see quantize_enc_fast)
    float rs[NP][2];
    auto refresh = [&](int p) {
        rs[p][0] = __builtin_amdgcn_rcpf((float)st[p].sc.x);
        rs[p][1] = CPL >= 2 ? __builtin_amdgcn_rcpf((float)st[p].sc.y) : rs[p][0];
    };
#pragma unroll
    for (int p = 0; p < NP; p++)
        refresh(p);
    // quantise one token with the current state, advance the state; qf = the codes as floats.
    // spec: branch-free speculative form (see quantize_enc_spec), the caller checks `worst`.
    uint32_t worst = 0u;
    auto advance = [&](auto spec, const XW *x, float *qf) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            XW xw = CPL == 1 ? x[p] >> xsh : x[p];
            if (BF16) {
                // bf16 -> fp32 is exact, fp32 -> fp16 rounds to nearest even: torch's .to(float16)
                const h1 lo = (h1)__uint_as_float(xw << 16);
                const h1 hi = CPL == 1 ? lo : (h1)__uint_as_float(xw & 0xFFFF0000u);
                xw = as_u32((h2){lo, hi});
            }
            const uint32_t zw = __builtin_bit_cast(uint32_t, st[p].zp);
            float q0, q1;
            if constexpr (decltype(spec)::value) {
                q0 = quantize_enc_spec<BITS, false>(xw, zw, rs[p][0], worst);
                q1 = CPL >= 2 ? quantize_enc_spec<BITS, true>(xw, zw, rs[p][1], worst) : q0;
            } else {
                q0 = quantize_enc_fast<BITS, false>(xw, zw, st[p].sc.x, rs[p][0]);
                q1 = CPL >= 2 ? quantize_enc_fast<BITS, true>(xw, zw, st[p].sc.y, rs[p][1]) : q0;
            }
            qf[CPL >= 2 ? 2 * p : 0] = q0;
            if (CPL >= 2)
                qf[2 * p + 1] = q1;
            const h2 q = pack_codes(q0, q1);
            update_pair_abs(st[p], pack_codes(__builtin_fabsf(q0), __builtin_fabsf(q1)), q * st[p].sc);
            refresh(p);
        }
    };
    using Exact = std::integral_constant<bool, false>;
    using Spec = std::integral_constant<bool, true>;
    // partial words: token slot known at run time only
    auto step = [&](const XW *x, int tt, uint32_t *w) {
        float qf[CPL];
        advance(Exact{}, x, qf);
#pragma unroll
        for (int c = 0; c < CPL; c++)
            w[c] += (uint32_t)(int)qf[c] << (BITS * tt);
    };
    // Checkpoints: entry j is the state before token (j+1)*interval.  Words are stored in order,
    // so the next boundary is tracked by comparison instead of a division per word.
    int ck_next = -1, ck_j = 0;
    if (sa.ckpt != nullptr) {
        const int first_end = (T0 / TPW) * TPW + TPW;
        ck_j = (first_end + sa.ckpt_interval - 1) / sa.ckpt_interval - 1;
        ck_next = (ck_j + 1) * sa.ckpt_interval;
    }
    // bias adds -QLO to the codes written now; keep selects codes of earlier tokens to preserve
    auto store_sg = [&](int sg, const uint32_t *w, uint32_t bias, uint32_t keep) {
        const int tend = sg * TPW + TPW;
        const bool ck_here = tend == ck_next;
        if (ck_here) {
            ck_next += sa.ckpt_interval;
            ck_j++;
        }
        if (!active)
            return;
        uint32_t *dst = cw + (size_t)sg * D;
        uint32_t o[CPL];
#pragma unroll
        for (int c = 0; c < CPL; c++)
            o[c] = w[c] + bias;
        if (keep) {
#pragma unroll
            for (int c = 0; c < CPL; c++)
                o[c] = (o[c] & ~keep) | (dst[c] & keep);
        }
        if (CPL == 4)
            *reinterpret_cast<uint4 *>(dst) = make_uint4(o[0], o[1], o[2], o[3]);
        else if (CPL == 2)
            *reinterpret_cast<uint2 *>(dst) = make_uint2(o[0], o[1]);
        else
            dst[0] = o[0];
        if (ck_here && tend <= T && ck_j - 1 < sa.n_ckpt_cap)
            store_state_n<CPL>(sa.ckpt + (((size_t)bx * sa.n_ckpt_cap + (ck_j - 1)) * D + c0) * 2, st);
    };

    auto nib_mask = [](int k) { return k >= TPW ? 0xFFFFFFFFu : ((1u << (BITS * k)) - 1u); };
    constexpr uint32_t BIAS = Code<BITS>::BIAS;

    // a stream that resumes inside a word first completes it (codes below T0 are kept)
    int t = T0;
    if ((t % TPW) && t < T) {
        const int lo = t % TPW, sg = t / TPW;
        uint32_t w[CPL];
#pragma unroll
        for (int c = 0; c < CPL; c++)
            w[c] = 0u;
        for (; t < T && t / TPW == sg; t++) {
            XW x[NP];
            load_tok(t, x);
            step(x, t % TPW, w);
        }
        const int hi = t / TPW == sg ? t % TPW : TPW;
        store_sg(sg, w, BIAS & nib_mask(hi) & ~nib_mask(lo), nib_mask(lo));
    }

    // full words: no per-token conditions, inputs ENC_PF-1 groups of 8 tokens ahead.  The loads
    // are unconditional (index clamped to the last group): a load under a condition has to land
    // before the code after the condition runs, which would expose the memory latency per group.
    const int sgb = t / TPW;                    // first full word
    const int nfull = (T - t) / TPW;
    const int ng = nfull * G8;
    XW xbuf[ENC_PF][8][NP];
    uint32_t w[CPL];
#pragma unroll
    for (int c = 0; c < CPL; c++)
        w[c] = 0u;
    // loads the next group of 8 rows; past the last group the same rows are loaded again
    const h1 *xnext = xbw + (long)(t - T0) * xs.t;
    int gnext = 0;
    auto load_next = [&](XW (*xg)[NP]) {
#pragma unroll
        for (int tt = 0; tt < 8; tt++) {
#pragma unroll
            for (int p = 0; p < NP; p++)
                xg[tt][p] = *reinterpret_cast<const XW *>(xnext + (long)tt * xs.t + 2 * p);
        }
        if (gnext < ng - 1) {
            xnext += 8 * xs.t;
            gnext++;
        }
    };
    // The codes of 16/BITS tokens fill 16 bits; their signed sum q << BITS*k is exact in one
    // float (|sum| < 2^20), one fma per code, and two halves make the 32-bit word.
    constexpr int TPA = 16 / BITS; // tokens per half word
    constexpr int NA = 8 / TPA;    // half words an 8-token group fills
    auto run_group = [&](auto spec, const XW (*xg)[NP], float (*acc)[NA]) {
#pragma unroll
        for (int tt = 0; tt < 8; tt++) {
            float qf[CPL];
            advance(spec, xg[tt], qf);
#pragma unroll
            for (int c = 0; c < CPL; c++) {
                if (tt % TPA == 0)
                    acc[c][tt / TPA] = qf[c];
                else
                    acc[c][tt / TPA] = __builtin_fmaf(qf[c], (float)(1u << (BITS * (tt % TPA))),
                                                      acc[c][tt / TPA]);
            }
        }
    };
    // Lanes of one channel belong to waves that have a SIMD to themselves (that is when the
    // launcher picks them), so they run a group speculatively without the per-token branch and
    // repeat it exactly from the saved state when any lane of the wave came near a rounding
    // boundary (about one group in sixty).
    constexpr bool SPECULATE = CPL == 1;
    auto do_group = [&](int g, const XW (*xg)[NP]) {
        float acc[CPL][NA];
        if (SPECULATE) {
            Pair saved[NP];
#pragma unroll
            for (int p = 0; p < NP; p++)
                saved[p] = st[p];
            worst = 0u;
            run_group(Spec{}, xg, acc);
            if (__any(worst >= __float_as_uint(ENC_SPEC_LIMIT))) {
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    st[p] = saved[p];
                    refresh(p);
                }
                run_group(Exact{}, xg, acc);
            }
        } else {
            run_group(Exact{}, xg, acc);
        }
#pragma unroll
        for (int c = 0; c < CPL; c++) {
            uint32_t v = (uint32_t)(int)acc[c][0];
            if (NA == 2)
                v += (uint32_t)(int)acc[c][NA - 1] << 16;
            w[c] += G8 == 1 ? v : v << (16 * (g % G8));
        }
        if (G8 == 1 || g % G8 == G8 - 1) {
            store_sg(sgb + g / G8, w, BIAS, 0u);
#pragma unroll
            for (int c = 0; c < CPL; c++)
                w[c] = 0u;
        }
    };
    if (ng > 0) {
#pragma unroll
        for (int i = 0; i < ENC_PF - 1; i++)
            load_next(xbuf[i]);
        int g0 = 0;
        for (; g0 + ENC_PF <= ng; g0 += ENC_PF) {
#pragma unroll
            for (int i = 0; i < ENC_PF; i++) {
                load_next(xbuf[(i + ENC_PF - 1) % ENC_PF]);
                do_group(g0 + i, xbuf[i]);
            }
        }
        // at most ENC_PF-1 groups left; their inputs are already in xbuf[0 .. ENC_PF-2]
#pragma unroll
        for (int i = 0; i < ENC_PF - 1; i++)
            if (g0 + i < ng)
                do_group(g0 + i, xbuf[i]);
    }
    // ragged last word: codes of the tokens present, zero fields after them
    t += nfull * TPW;
    if (t < T) {
        const int ntail = T - t;
#pragma unroll
        for (int c = 0; c < CPL; c++)
            w[c] = 0u;
        for (int tt = 0; tt < ntail; tt++) {
            XW x[NP];
            load_tok(t + tt, x);
            step(x, tt, w);
        }
        store_sg(t / TPW, w, BIAS & nib_mask(ntail), 0u);
    }
    if (state_out != nullptr && active)
        store_state_n<CPL>(state_out + ((size_t)bx * D + c0) * 2, st);
}

template <int BITS, int CPL, int BLK>
__global__ __launch_bounds__(BLK) void encode_kernel(
    uint32_t *__restrict__ cache, const h1 *__restrict__ kv_new,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int BH, int H, int T0, int T, int D, int n_super_cap, const h1 *__restrict__ state_in,
    h1 *__restrict__ state_out, Seg sa)
{
    const RowStrides packed = {(long)H * (T - T0) * D, (long)(T - T0) * D, (long)D};
    encode_body<BITS, CPL, BLK>(cache, kv_new, packed, zp, sc, al, be, tg, BH, H, T0, T, D, n_super_cap,
                                state_in, state_out, sa);
}

// Two tensors of one shape (the K and V rows of the same tokens) in one launch: blockIdx.y picks
// the tensor.  A prompt with few channels (small batch) leaves SIMDs idle when the tensors are
// encoded one after the other; together they run in the time of one.
struct EncTensor {
    uint32_t *cache;
    const h1 *kv_new, *zp, *sc, *al, *be, *tg, *state_in;
    h1 *state_out, *ckpt;
    RowStrides xs;
};

// BF16: the new rows are bfloat16 (same strides, in elements) and are rounded to fp16 on the fly.
template <int BITS, int CPL, int BLK, bool BF16>
__global__ __launch_bounds__(BLK) void encode_pair_kernel(EncTensor k, EncTensor v, int BH, int H,
                                                          int T0, int T, int D, int n_super_cap,
                                                          Seg sa)
{
    const EncTensor e = blockIdx.y ? v : k;
    sa.ckpt = e.ckpt;
    encode_body<BITS, CPL, BLK, BF16>(e.cache, e.kv_new, e.xs, e.zp, e.sc, e.al, e.be, e.tg, BH, H, T0,
                                      T, D, n_super_cap, e.state_in, e.state_out, sa);
}

// Shared tail of the two decode kernels: quantise the new token with the state after token T-1,
// patch it into slot T, return the fused dequant r16(q*sc + zp) per pair (gemv.cu:744-798,
// 1105-1157).  The state is NOT advanced.
template <int D, int CPL, int BITS = 4>
__device__ __forceinline__ void append_new_token(typename Geo<D, CPL>::Vec *cb, int T, const h1 *xnew, const Pair *st,
                                                 h2 *deq, bool active, int act_bf16 = 0)
{
    using G = Geo<D, CPL>;
    const int sg = T / Code<BITS>::TPW, tt = T % Code<BITS>::TPW;
#pragma unroll
    for (int v = 0; v < G::NV; v++) {
        typename G::Vec *slot = cb + (size_t)sg * G::VPS + v;
        typename G::Vec u = *slot;
        uint32_t w[G::WPV];
        vec_words(u, w);
#pragma unroll
        for (int pp = 0; pp < G::WPV / 2; pp++) {
            const int p = (G::WPV / 2) * v + pp;
            const h2 x = load_act2(xnew + 2 * p, act_bf16);
            const h2 q = append_pair<BITS>(w[2 * pp], w[2 * pp + 1], tt, x, st[p]);
            deq[p] = pk_fma(q, st[p].sc, st[p].zp);
        }
        if (active) {
            words_vec(w, u);
            *slot = u;
        }
    }
}

// What the last segment does once it holds the state after token T-1: hand it out, and record it
// as a checkpoint when token T opens a new checkpoint interval.
template <int D, int CPL>
__device__ __forceinline__ void publish_state(const Pair *st, h1 *state_out, const Seg &sa, int bx,
                                              int c0, int T)
{
    if (state_out != nullptr)
        store_state<CPL>(state_out + ((size_t)bx * D + c0) * 2, st);
    if (sa.ckpt != nullptr && T > 0 && T % sa.ckpt_interval == 0) {
        const int j = T / sa.ckpt_interval - 1;
        if (j < sa.n_ckpt_cap)
            store_state<CPL>(sa.ckpt + (((size_t)bx * sa.n_ckpt_cap + j) * D + c0) * 2, st);
    }
}

template <int D, int CPL>
__device__ __forceinline__ void pair_bytes_of(const typename Geo<D, CPL>::Vec *u, uint32_t (*nb)[2])
{
    using G = Geo<D, CPL>;
#pragma unroll
    for (int v = 0; v < G::NV; v++) {
        uint32_t w[G::WPV];
        vec_words(u[v], w);
#pragma unroll
        for (int pp = 0; pp < G::WPV / 2; pp++)
            pair_bytes(w[2 * pp], w[2 * pp + 1], nb[(G::WPV / 2) * v + pp][0], nb[(G::WPV / 2) * v + pp][1]);
    }
}

// ---------------------------------------------------------------------------------------------
// forward_qk  (gemv.cu:435-815)
// ---------------------------------------------------------------------------------------------
// Per lane and supergroup: 8 fp32 partial logits (v_dot2_f32_f16 over the lane's channel pairs).
// They are summed across the head's lanes and scattered by reduce8_head (masked DPP adds and row
// swaps, no LDS): afterwards every quad of lanes holds the total of one token.
template <int D, int CPL, int BLK>
__global__ __launch_bounds__(BLK) void qk_kernel(
    const h1 *__restrict__ q, uint4 *__restrict__ cache, const h1 *__restrict__ k_new,
    h1 *__restrict__ out,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int BH, int H, int T, int n_super_cap, h1 *__restrict__ state_out, Seg sa)
{
    using G = Geo<D, CPL>;
    // the only LDS object: the table sits at LDS offset 0 (its byte address is used as is)
    __shared__ uint2 smem[LUT_WORDS64];
    const uint2 *lut = smem;
    lut_fill(smem, threadIdx.x, BLK);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const uint32_t lane_copy = (uint32_t)(lane & (LUT_COPIES - 1)) * 8u;

    const Unit<D, CPL, BLK> un(BH, sa.nseg);
    if (!un.wave_active)
        return; // padding waves
    const int bx = un.bx, lh = un.lh, c0 = un.c0;
    const bool active = un.active;
    const bool last = seg_is_last(sa, un.seg);
    const int h = bx % H;

    Pair st[G::NP];
    h2 qv[G::NP];
    init_pairs<D, CPL>(st, zp, sc, al, be, tg, h, bx, c0, un.seg, sa);
#pragma unroll
    for (int p = 0; p < G::NP; p++)
        qv[p] = load_act2(q + (size_t)bx * D + c0 + 2 * p, sa.act_bf16);

    const int t0 = seg_begin(sa, un.seg);
    const int t1 = last ? T : seg_end(sa, un.seg);
    using Vec = typename G::Vec;
    Vec *cbh = reinterpret_cast<Vec *>(cache) + (size_t)bx * n_super_cap * G::VPS + lh * G::NV; // this head, this lane
    const Vec *cb = cbh + (size_t)(t0 >> 3) * G::VPS;                                           // this segment
    h1 *ob = out + (size_t)bx * sa.row_pitch + t0;
    const int nfull = (t1 - t0) >> 3;
    // the token whose total this lane's quad ends up with, and the one lane per token that stores
    // it (a 64-lane head holds every total twice, once per half)
    const int tk = token_of_lane(lane);
    const bool storer = active && (lane & 3) == 0 && (G::LPH == 32 || lane < 32);
    auto finish = [&](const float *part, int sg, int ntok) {
        const float s = reduce8_head<G::LPH>(part);
        if (storer && tk < ntok)
            ob[sg * 8 + tk] = (h1)s;
    };

    // ---- software pipeline over the full supergroups.  Global loads run PF supergroups ahead.
    // Table lookups run one supergroup ahead and are issued token by token between the arithmetic
    // of the current supergroup (the LDS counter holds only 15 outstanding operations, so issuing a
    // whole supergroup's lookups at once would stall on them).  The logits of supergroup sg-1 are
    // reduced and stored at the start of iteration sg, while the first lookups are in flight.
    // The lookup for the next supergroup goes into the slot the current token has just vacated, so
    // one supergroup's worth of registers holds both.
    auto token = [&](int t, uint2 (*e)[8], const uint32_t (*nb)[2], float &out_t) {
        float acc;
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            Pair &s = st[p];
            const h2 qs = as_h2(e[p][t].x) * s.sc;
            const h2 kh = qs + s.zp;
            if (p == 0)
                acc = dot2_from_zero(qv[p], kh);
            else
                acc = __builtin_amdgcn_fdot2(qv[p], kh, acc, false);
            update_pair_abs(s, as_h2(e[p][t].y), qs);
        }
        out_t = acc;
#pragma unroll
        for (int p = 0; p < G::NP; p++)
            e[p][t] = lut_get(lut, nb[p][t & 1], lane_copy, t >> 1);
        __builtin_amdgcn_sched_barrier(0);
    };

    Vec buf[PF][G::NV];
    uint2 lk[G::NP][8];
    uint32_t nb[G::NP][2];
    float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < PF; i++) {
#pragma unroll
        for (int v = 0; v < G::NV; v++)
            buf[i][v] = (i < nfull) ? load_codes(cb + (size_t)i * G::VPS + v) : vec_zero<Vec>();
    }
    if (nfull > 0) {
        pair_bytes_of<D, CPL>(buf[0], nb);
#pragma unroll
        for (int t = 0; t < 8; t++)
#pragma unroll
            for (int p = 0; p < G::NP; p++)
                lk[p][t] = lut_get(lut, nb[p][t & 1], lane_copy, t >> 1);
    }
    // One supergroup; i = its buffer in the rotation (compile-time).  Nothing in here is
    // conditional: the trip count is wave-uniform, the prefetch index is clamped, and the
    // reduction of the previous supergroup stores nothing when there is none (sg == 0).
    auto body = [&](int sg, auto ic) {
        constexpr int i = decltype(ic)::value;
        // bytes of supergroup sg+1 (stale data past the end: looked up, never used)
        pair_bytes_of<D, CPL>(buf[(i + 1) % PF], nb);
        {
            // unconditional, clamped to the segment's last supergroup: a load inside a branch
            // makes the next wait cover every load in flight, this one included
            const int sgp = min(sg + PF, nfull - 1);
#pragma unroll
            for (int v = 0; v < G::NV; v++)
                buf[i][v] = load_codes(cb + (size_t)sgp * G::VPS + v);
        }
        __builtin_amdgcn_sched_barrier(0);
        finish(part, sg - 1, sg > 0 ? 8 : 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 8; t++)
            token(t, lk, nb, part[t]);
    };
    rotate_over<PF>(nfull, body);
    if (nfull > 0)
        finish(part, nfull - 1, 8);
    if (!last)
        return;

    // ragged tail: T % 8 tokens of the last supergroup, state advances only for t < T
    // (gemv.cu:648-654)
    const int ntail = (t1 - t0) & 7;
    if (ntail) {
        float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int v = 0; v < G::NV; v++) {
            uint32_t w[G::WPV];
            vec_words(cb[(size_t)nfull * G::VPS + v], w);
#pragma unroll
            for (int pp = 0; pp < G::WPV / 2; pp++) {
                Pair &s = st[(G::WPV / 2) * v + pp];
                for (int tt = 0; tt < ntail; tt++) {
                    const uint32_t na = (w[2 * pp] >> (4 * tt)) & 0xFu;
                    const uint32_t nbb = (w[2 * pp + 1] >> (4 * tt)) & 0xFu;
                    const h2 qc = codes_to_h2((int)na - 8, (int)nbb - 8);
                    const h2 qs = qc * s.sc;
                    const float d = __builtin_amdgcn_fdot2(qv[(G::WPV / 2) * v + pp], qs + s.zp, 0.0f, false);
#pragma unroll
                    for (int k = 0; k < 8; k++)
                        part[k] += (k == tt) ? d : 0.0f;
                    update_pair(s, qc, qs);
                }
            }
        }
        finish(part, nfull, ntail);
    }

    if (active)
        publish_state<D, CPL>(st, state_out, sa, bx, c0, T);

    h2 deq[G::NP];
    append_new_token<D, CPL>(cbh, T, k_new + (size_t)bx * D + c0, st, deq, active, sa.act_bf16);
    float self = 0.0f;
#pragma unroll
    for (int p = 0; p < G::NP; p++)
        self = __builtin_amdgcn_fdot2(qv[p], deq[p], self, false);
    self = head_allreduce<G::LPH>(self);
    if (active && lh == 0)
        out[(size_t)bx * sa.row_pitch + T] = (h1)self;
}

// ---------------------------------------------------------------------------------------------
// forward_ov  (gemv.cu:946-1178)
// ---------------------------------------------------------------------------------------------
// acc[c] accumulates w_t * v_hat[t,c] in fp32 (fp16 operands, exact products: v_fma_mix_f32); the
// reference accumulates in fp16 for the whole sequence (gemv.cu:1087,1096).  With one segment the
// result is rounded to fp16 and stored; with several, each segment stores its fp32 partial into
// `partial` [nseg, B*H, D] and ov_finalize_kernel adds them up.
template <int D, int CPL, int BLK>
__global__ __launch_bounds__(BLK) void ov_kernel(
    const h1 *__restrict__ attn, uint4 *__restrict__ cache, const h1 *__restrict__ v_new,
    h1 *__restrict__ out, float *__restrict__ partial,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int BH, int H, int T, int n_super_cap, h1 *__restrict__ state_out, Seg sa)
{
    using G = Geo<D, CPL>;
    __shared__ uint2 lut[LUT_WORDS64];
    lut_fill(lut, threadIdx.x, BLK);
    __syncthreads();
    const uint32_t lane_copy = (uint32_t)(threadIdx.x & (LUT_COPIES - 1)) * 8u;

    const Unit<D, CPL, BLK> un(BH, sa.nseg);
    if (!un.wave_active)
        return; // padding waves
    const int bx = un.bx, lh = un.lh, c0 = un.c0;
    const bool active = un.active;
    const bool last = seg_is_last(sa, un.seg);
    const int h = bx % H;

    Pair st[G::NP];
    float acc[CPL];
    init_pairs<D, CPL>(st, zp, sc, al, be, tg, h, bx, c0, un.seg, sa);
#pragma unroll
    for (int c = 0; c < CPL; c++)
        acc[c] = 0.0f;
    // Four-channel (and wider) lanes contract on the matrix cores, as ov_ft_kernel does and for the
    // reason given there: B = the lane's dequantised pair at two tokens, A = (w[t], 0, w[t+1], 0)
    // from lane 0 of each group of four, (0, w[t], 0, w[t+1]) from lane 1, zeros from lanes 2, 3.
    constexpr bool MM = CPL >= 4;
    f4v acc4[G::NP];
#pragma unroll
    for (int p = 0; p < G::NP; p++)
        acc4[p] = (f4v){0.0f, 0.0f, 0.0f, 0.0f};
    const int role = threadIdx.x & 3;
    const uint32_t sel_a0 = role == 0 ? 0x0C0C0100u : role == 1 ? 0x01000C0Cu : 0x0C0C0C0Cu;
    const uint32_t sel_a1 = role == 0 ? 0x0C0C0302u : role == 1 ? 0x03020C0Cu : 0x0C0C0C0Cu;

    const int t0 = seg_begin(sa, un.seg);
    const int t1 = last ? T : seg_end(sa, un.seg);
    using Vec = typename G::Vec;
    Vec *cbh = reinterpret_cast<Vec *>(cache) + (size_t)bx * n_super_cap * G::VPS + lh * G::NV;
    const Vec *cb = cbh + (size_t)(t0 >> 3) * G::VPS;
    const h1 *wrow = attn + (size_t)bx * sa.row_pitch;
    const h1 *wb = wrow + t0;
    const int nfull = (t1 - t0) >> 3;

    auto load_w = [&](int sg) {
        uint4 r;
        __builtin_memcpy(&r, wb + (size_t)sg * 8, 16); // row base is only 2-byte aligned
        return r;
    };
    // one token of the current supergroup, followed by the lookups of the same token slot of the
    // next supergroup (see qk_kernel for why they are interleaved)
    auto token = [&](int t, uint2 (*e)[8], const uint32_t (*nb)[2], const uint4 wv) {
        const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
        const h2 wp = as_h2(ww[t >> 1]);
        const float wt = (t & 1) ? (float)wp.y : (float)wp.x;
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            Pair &s = st[p];
            const h2 qs = as_h2(e[p][t].x) * s.sc;
            const h2 vd = qs + s.zp;
            acc[2 * p] = __builtin_fmaf(wt, (float)vd.x, acc[2 * p]);
            acc[2 * p + 1] = __builtin_fmaf(wt, (float)vd.y, acc[2 * p + 1]);
            update_pair_abs(s, as_h2(e[p][t].y), qs);
        }
#pragma unroll
        for (int p = 0; p < G::NP; p++)
            e[p][t] = lut_get(lut, nb[p][t & 1], lane_copy, t >> 1);
        __builtin_amdgcn_sched_barrier(0);
    };

    // two tokens of the current supergroup on the matrix cores, then the lookups of the same two
    // slots of the next one
    auto token2 = [&](int t, uint2 (*e)[8], const uint32_t (*nb)[2], const uint4 wv) {
        const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
        const uint32_t w2 = ww[t >> 1];
        const h4v a = as_h4(__builtin_amdgcn_perm(w2, w2, sel_a0), __builtin_amdgcn_perm(w2, w2, sel_a1));
        uint32_t vd[G::NP][2];
#pragma unroll
        for (int k = 0; k < 2; k++)
#pragma unroll
            for (int p = 0; p < G::NP; p++) {
                Pair &s = st[p];
                const h2 qs = as_h2(e[p][t + k].x) * s.sc;
                vd[p][k] = as_u32(qs + s.zp);
                update_pair_abs(s, as_h2(e[p][t + k].y), qs);
            }
#pragma unroll
        for (int p = 0; p < G::NP; p++)
            acc4[p] = __builtin_amdgcn_mfma_f32_4x4x4f16(a, as_h4(vd[p][0], vd[p][1]), acc4[p], 0, 0, 0);
#pragma unroll
        for (int k = 0; k < 2; k++)
#pragma unroll
            for (int p = 0; p < G::NP; p++)
                e[p][t + k] = lut_get(lut, nb[p][(t + k) & 1], lane_copy, (t + k) >> 1);
        __builtin_amdgcn_sched_barrier(0);
    };

    Vec buf[PF][G::NV];
    uint4 wbuf[PF];
    uint2 lk[G::NP][8];
    uint32_t nb[G::NP][2];
#pragma unroll
    for (int i = 0; i < PF; i++) {
#pragma unroll
        for (int v = 0; v < G::NV; v++)
            buf[i][v] = (i < nfull) ? load_codes(cb + (size_t)i * G::VPS + v) : vec_zero<Vec>();
        wbuf[i] = (i < nfull) ? load_w(i) : make_uint4(0, 0, 0, 0);
    }
    if (nfull > 0) {
        pair_bytes_of<D, CPL>(buf[0], nb);
#pragma unroll
        for (int t = 0; t < 8; t++)
#pragma unroll
            for (int p = 0; p < G::NP; p++)
                lk[p][t] = lut_get(lut, nb[p][t & 1], lane_copy, t >> 1);
    }
    // one supergroup, nothing conditional in it (see qk_kernel); i = its buffer in the rotation
    auto body = [&](int sg, auto ic) {
        constexpr int i = decltype(ic)::value;
        pair_bytes_of<D, CPL>(buf[(i + 1) % PF], nb);
        const int sgp = min(sg + PF, nfull - 1);
#pragma unroll
        for (int v = 0; v < G::NV; v++)
            buf[i][v] = load_codes(cb + (size_t)sgp * G::VPS + v);
        __builtin_amdgcn_sched_barrier(0);
        if (MM) {
#pragma unroll
            for (int t = 0; t < 8; t += 2)
                token2(t, lk, nb, wbuf[i]);
        } else {
#pragma unroll
            for (int t = 0; t < 8; t++)
                token(t, lk, nb, wbuf[i]);
        }
        // the weights are reloaded once their last token is done: loading them earlier into a
        // second register set costs copies at the loop edge, which wait for the load they move
        wbuf[i] = load_w(sgp);
    };
    rotate_over<PF>(nfull, body);
    if (MM) {
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            acc[2 * p] = acc4[p].x;
            acc[2 * p + 1] = acc4[p].y;
        }
    }

    if (last) {
        const int ntail = (t1 - t0) & 7;
        if (ntail) {
#pragma unroll
            for (int v = 0; v < G::NV; v++) {
                uint32_t w[G::WPV];
                vec_words(cb[(size_t)nfull * G::VPS + v], w);
#pragma unroll
                for (int pp = 0; pp < G::WPV / 2; pp++) {
                    Pair &s = st[(G::WPV / 2) * v + pp];
                    for (int tt = 0; tt < ntail; tt++) {
                        const uint32_t na = (w[2 * pp] >> (4 * tt)) & 0xFu;
                        const uint32_t nbb = (w[2 * pp + 1] >> (4 * tt)) & 0xFu;
                        const h2 qc = codes_to_h2((int)na - 8, (int)nbb - 8);
                        const h2 qs = qc * s.sc;
                        const h2 vd = qs + s.zp;
                        const float wt = (float)wb[nfull * 8 + tt];
                        const int c = G::WPV * v + 2 * pp;
                        acc[c] = __builtin_fmaf(wt, (float)vd.x, acc[c]);
                        acc[c + 1] = __builtin_fmaf(wt, (float)vd.y, acc[c + 1]);
                        update_pair(s, qc, qs);
                    }
                }
            }
        }
        if (active)
            publish_state<D, CPL>(st, state_out, sa, bx, c0, T);

        h2 deq[G::NP];
        append_new_token<D, CPL>(cbh, T, v_new + (size_t)bx * D + c0, st, deq, active, sa.act_bf16);
        const float wT = (float)wrow[T];
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            acc[2 * p] = __builtin_fmaf(wT, (float)deq[p].x, acc[2 * p]);
            acc[2 * p + 1] = __builtin_fmaf(wT, (float)deq[p].y, acc[2 * p + 1]);
        }
    }
    if (!active)
        return;
    if (sa.nseg == 1) {
        h1 *o = out + (size_t)bx * D + c0;
#pragma unroll
        for (int p = 0; p < G::NP; p++)
            store_act2(o + 2 * p, acc[2 * p], acc[2 * p + 1], sa.act_bf16);
    } else {
        float2 *o = reinterpret_cast<float2 *>(partial + ((size_t)un.seg * BH + bx) * D + c0);
#pragma unroll
        for (int p = 0; p < G::NP; p++)
            o[p] = make_float2(acc[2 * p], acc[2 * p + 1]);
    }
}

// out[i] = fp16(sum over segments, in segment order, of partial[s][i])
__global__ __launch_bounds__(256) void ov_finalize_kernel(const float *__restrict__ partial,
                                                           h1 *__restrict__ out, long n, int nseg,
                                                           int act_bf16)
{
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 2; // n is even (whole heads)
    if (i >= n)
        return;
    float2 s = make_float2(0.0f, 0.0f);
    for (int k = 0; k < nseg; k++) {
        const float2 p = *reinterpret_cast<const float2 *>(partial + (size_t)k * n + i);
        s.x += p.x;
        s.y += p.y;
    }
    store_act2(out + i, s.x, s.y, act_bf16);
}

// The same sum for many segments (long contexts at small batch: 128 segments of a 32 768-token
// context leave the kernel above with 128 dependent additions per thread and few threads).  A
// workgroup owns 64 consecutive outputs: thread (r, j) adds the segments r, r+16, ... of outputs
// 4j..4j+3 in ascending order, then thread (0, j) adds the 16 subtotals in ascending r.  The order
// is fixed, so results are reproducible from run to run.
__global__ __launch_bounds__(256) void ov_finalize_wide_kernel(const float *__restrict__ partial,
                                                                h1 *__restrict__ out, long n, int nseg,
                                                                int act_bf16)
{
    __shared__ float4 sub[16][16];
    const int j = threadIdx.x & 15, r = threadIdx.x >> 4;
    const long i = ((long)blockIdx.x * 16 + j) * 4; // n is a multiple of 4 (whole heads)
    float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (i < n) {
        for (int k = r; k < nseg; k += 16) {
            const float4 p = *reinterpret_cast<const float4 *>(partial + (size_t)k * n + i);
            a.x += p.x;
            a.y += p.y;
            a.z += p.z;
            a.w += p.w;
        }
    }
    sub[r][j] = a;
    __syncthreads();
    if (r == 0 && i < n) {
#pragma unroll
        for (int k = 1; k < 16; k++) {
            const float4 p = sub[k][j];
            a.x += p.x;
            a.y += p.y;
            a.z += p.z;
            a.w += p.w;
        }
        store_act2(out + i, a.x, a.y, act_bf16);
        store_act2(out + i + 2, a.z, a.w, act_bf16);
    }
}

// ---------------------------------------------------------------------------------------------
// Rotary position embedding of q and k in one launch   (llama_adkv.py:336-337 calls transformers'
// apply_rotary_pos_emb: x * cos + rotate_half(x) * sin, ten elementwise launches)
// ---------------------------------------------------------------------------------------------
// Every operation is rounded to the activations' type the way torch's elementwise kernels round
// it (operands widened to fp32, one fp32 operation, result rounded to nearest even), so the
// output equals that of the torch expression bit for bit.  A row is one (batch, token, head)
// vector of D values; a lane takes two adjacent values of the first half and their partners in
// the second.
template <bool BF16>
__device__ __forceinline__ float act_to_f32(uint32_t bits16)
{
    if (BF16)
        return __uint_as_float(bits16 << 16);
    return (float)__builtin_bit_cast(h1, (uint16_t)bits16);
}
template <bool BF16>
__device__ __forceinline__ uint32_t f32_to_act(float f)
{
    if (BF16) {
        const uint32_t u = __float_as_uint(f);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u)
            return 0x7FC0u; // torch's bfloat16 NaN
        return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    }
    return (uint32_t)__builtin_bit_cast(uint16_t, (h1)f);
}
// r(r(x*c) + r(y*s)) with y already negated where rotate_half negates
template <bool BF16>
__device__ __forceinline__ uint32_t rope_one(uint32_t x, uint32_t c, uint32_t y, bool neg_y, uint32_t s)
{
    const float a = act_to_f32<BF16>(f32_to_act<BF16>(act_to_f32<BF16>(x) * act_to_f32<BF16>(c)));
    const float yy = neg_y ? -act_to_f32<BF16>(y) : act_to_f32<BF16>(y);
    const float b = act_to_f32<BF16>(f32_to_act<BF16>(yy * act_to_f32<BF16>(s)));
    return f32_to_act<BF16>(a + b);
}

struct RopeSide {
    const uint16_t *x;
    uint16_t *out;
    long sb, sh, st; // element strides of x over batch, head, token (channels contiguous)
    int heads;
};

// grid: (lanes of one token's Hq + H rows in workgroups of 256, token, batch)
template <bool BF16>
__global__ __launch_bounds__(256) void rope_kernel(RopeSide q, RopeSide k, const uint16_t *__restrict__ cos,
                                                   const uint16_t *__restrict__ sin, long cb, long ct,
                                                   int T, int D, int t0, int b0)
{
    const unsigned lpr = (unsigned)D >> 2;                   // lanes per row
    const unsigned idx = blockIdx.x * 256u + threadIdx.x;
    const unsigned hh = idx / lpr;
    if (hh >= (unsigned)(q.heads + k.heads))
        return;
    const int i = (int)(idx - hh * lpr) * 2;                 // first of this lane's two channels
    const int t = t0 + (int)blockIdx.y;
    const long b = (long)b0 + (long)blockIdx.z;
    const RopeSide &sd = hh < (unsigned)q.heads ? q : k;
    const int h = hh < (unsigned)q.heads ? (int)hh : (int)hh - q.heads;
    const uint16_t *x = sd.x + b * sd.sb + h * sd.sh + t * sd.st;
    uint16_t *o = sd.out + ((b * sd.heads + h) * T + t) * D;
    const uint16_t *c = cos + b * cb + t * ct, *s = sin + b * cb + t * ct;
    const int half = D >> 1;
    const uint32_t x1 = *reinterpret_cast<const uint32_t *>(x + i);
    const uint32_t x2 = *reinterpret_cast<const uint32_t *>(x + half + i);
    const uint32_t c1 = *reinterpret_cast<const uint32_t *>(c + i);
    const uint32_t c2 = *reinterpret_cast<const uint32_t *>(c + half + i);
    const uint32_t s1 = *reinterpret_cast<const uint32_t *>(s + i);
    const uint32_t s2 = *reinterpret_cast<const uint32_t *>(s + half + i);
    // first half: x1*cos + (-x2)*sin; second half: x2*cos + x1*sin
    const uint32_t lo0 = rope_one<BF16>(x1 & 0xFFFFu, c1 & 0xFFFFu, x2 & 0xFFFFu, true, s1 & 0xFFFFu);
    const uint32_t lo1 = rope_one<BF16>(x1 >> 16, c1 >> 16, x2 >> 16, true, s1 >> 16);
    const uint32_t hi0 = rope_one<BF16>(x2 & 0xFFFFu, c2 & 0xFFFFu, x1 & 0xFFFFu, false, s2 & 0xFFFFu);
    const uint32_t hi1 = rope_one<BF16>(x2 >> 16, c2 >> 16, x1 >> 16, false, s2 >> 16);
    *reinterpret_cast<uint32_t *>(o + i) = lo0 | (lo1 << 16);
    *reinterpret_cast<uint32_t *>(o + half + i) = hi0 | (hi1 << 16);
}

// ---------------------------------------------------------------------------------------------
// softmax(float(logits)*scaling + mask) -> fp16   (llama_adkv.py:266-271)
// ---------------------------------------------------------------------------------------------
constexpr int SM_BLOCK = 256;
constexpr int SM_VEC = 8;                             // fp16 values per 16-byte access
constexpr int SM_NV = 3;                              // such accesses per thread and chunk
constexpr int SM_KEEP = SM_VEC * SM_NV;               // row elements a thread keeps in registers
constexpr int SM_CHUNK = SM_BLOCK * SM_KEEP;          // row elements a 256-thread workgroup holds
constexpr int SM_ROW_MAX = 24576;                     // longest row a single workgroup keeps in registers

template <int NT = SM_BLOCK>
__device__ __forceinline__ float block_reduce(float v, float *sm, bool is_max)
{
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const float o = __shfl_xor(v, m, 64);
        v = is_max ? fmaxf(v, o) : v + o;
    }
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0)
        sm[w] = v;
    __syncthreads();
    float r = sm[0];
#pragma unroll
    for (int i = 1; i < NT / 64; i++)
        r = is_max ? fmaxf(r, sm[i]) : r + sm[i];
    return r;
}

// x[k] = logits*scaling + mask for the SM_KEEP elements of this thread in the chunk that starts at
// `base` (-inf past the end of the row); 16-byte accesses wherever a whole vector lies inside the
// row (rows are only 2-byte aligned: the hardware takes unaligned vector accesses).
template <int NV = SM_NV, int NT = SM_BLOCK>
__device__ __forceinline__ void softmax_load_chunk(const h1 *l, const float *mk, int n, int base,
                                                   float scaling, float *x, float &mx,
                                                   int tid = (int)threadIdx.x)
{
    mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int i0 = base + (v * NT + tid) * SM_VEC;
        float *xv = x + v * SM_VEC;
        if (i0 + SM_VEC <= n) {
            uint4 raw;
            __builtin_memcpy(&raw, l + i0, 16);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const h2 p = as_h2(w[k]);
                xv[2 * k] = (float)p.x * scaling;
                xv[2 * k + 1] = (float)p.y * scaling;
            }
            if (mk) {
                float m8[SM_VEC];
                __builtin_memcpy(m8, mk + i0, 32);
#pragma unroll
                for (int k = 0; k < SM_VEC; k++)
                    xv[k] += m8[k];
            }
        } else {
#pragma unroll
            for (int k = 0; k < SM_VEC; k++) {
                const int i = i0 + k;
                xv[k] = -INFINITY;
                if (i < n) {
                    xv[k] = (float)l[i] * scaling;
                    if (mk)
                        xv[k] += mk[i];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < SM_VEC; k++)
            mx = fmaxf(mx, xv[k]);
    }
}

// w[i] = fp16(x[k] * inv) for the same elements
template <int NV = SM_NV, int NT = SM_BLOCK>
__device__ __forceinline__ void softmax_store_chunk(h1 *w, int n, int base, const float *x, float inv,
                                                    int tid = (int)threadIdx.x)
{
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int i0 = base + (v * NT + tid) * SM_VEC;
        const float *xv = x + v * SM_VEC;
        if (i0 + SM_VEC <= n) {
            uint32_t o[4];
#pragma unroll
            for (int k = 0; k < 4; k++)
                o[k] = as_u32((h2){(h1)(xv[2 * k] * inv), (h1)(xv[2 * k + 1] * inv)});
            const uint4 raw = make_uint4(o[0], o[1], o[2], o[3]);
            __builtin_memcpy(w + i0, &raw, 16);
        } else {
#pragma unroll
            for (int k = 0; k < SM_VEC; k++)
                if (i0 + k < n)
                    w[i0 + k] = (h1)(xv[k] * inv);
        }
    }
}

// Short rows: one wave per row (four rows per workgroup), the row in registers, reductions across
// the wave only.  A workgroup per row would spend most of its time on two barriers for a handful of
// elements per thread; rows of a few hundred tokens are the common decode case.
template <int NV>
__global__ __launch_bounds__(SM_BLOCK) void softmax_wave_kernel(
    const h1 *__restrict__ logits, h1 *__restrict__ weights, const float *__restrict__ mask,
    int rows, int n, long ld, int rows_per_mask_row, float scaling)
{
    const int row = blockIdx.x * (SM_BLOCK / 64) + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const int lane = threadIdx.x & 63;
    const h1 *l = logits + (size_t)row * ld;
    h1 *w = weights + (size_t)row * ld;
    const float *mk = mask ? mask + (size_t)(row / rows_per_mask_row) * n : nullptr;
    float x[NV * SM_VEC], mx;
    softmax_load_chunk<NV, 64>(l, mk, n, 0, scaling, x, mx, lane);
#pragma unroll
    for (int m = 1; m < 64; m <<= 1)
        mx = fmaxf(mx, __shfl_xor(mx, m, 64));
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < NV * SM_VEC; k++) {
        x[k] = __expf(x[k] - mx);
        sum += x[k];
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1)
        sum += __shfl_xor(sum, m, 64);
    softmax_store_chunk<NV, 64>(w, n, 0, x, 1.0f / sum, lane);
}

// One workgroup of NT threads per row.  A row of up to NT * NV * 8 elements is read once and kept
// in registers (the launcher picks NT and NV by the row length, up to 24576 elements); longer rows
// are walked three times (the chunked kernels below avoid that when the caller gives a workspace).
template <int NT, int NV>
__global__ __launch_bounds__(NT) void softmax_kernel(
    const h1 *__restrict__ logits, h1 *__restrict__ weights, const float *__restrict__ mask,
    int n, long ld, int rows_per_mask_row, float scaling)
{
    __shared__ float sm[NT / 64];
    const int row = blockIdx.x;
    const h1 *l = logits + (size_t)row * ld;
    h1 *w = weights + (size_t)row * ld;
    const float *mk = mask ? mask + (size_t)(row / rows_per_mask_row) * n : nullptr;

    if (n <= NT * NV * SM_VEC) {
        float x[NV * SM_VEC], mx;
        softmax_load_chunk<NV, NT>(l, mk, n, 0, scaling, x, mx);
        mx = block_reduce<NT>(mx, sm, true);
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < NV * SM_VEC; k++) {
            x[k] = __expf(x[k] - mx);
            sum += x[k];
        }
        sum = block_reduce<NT>(sum, sm, false);
        softmax_store_chunk<NV, NT>(w, n, 0, x, 1.0f / sum);
        return;
    }
    auto at = [&](int i) {
        float v = (float)l[i] * scaling;
        if (mk)
            v += mk[i];
        return v;
    };
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < n; i += NT)
        mx = fmaxf(mx, at(i));
    mx = block_reduce<NT>(mx, sm, true);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < n; i += NT)
        sum += __expf(at(i) - mx);
    sum = block_reduce<NT>(sum, sm, false);
    const float inv = 1.0f / sum;
    for (int i = threadIdx.x; i < n; i += NT)
        w[i] = (h1)(__expf(at(i) - mx) * inv);
}

// Unmasked rows of up to 1024 * NV * 8 elements (139 264 with NV = 17), one 1024-thread workgroup
// per row: the row stays in registers AS FP16 (NV 16-byte vectors per thread), so it is read once
// and written once; maximum, sum and weights are three walks over registers.  Up to 9 vectors
// per thread two such workgroups fit a CU (64 registers per lane), beyond that one (104 registers
// with 17 vectors); few and very long rows are better cut into chunks.
// scaling must be non-zero: elements past the end of the row are held as the infinity that
// scaling turns into -inf.
constexpr int SM_REG_NV = 17;
constexpr int SM_REG_MAX = 1024 * SM_REG_NV * SM_VEC;
#ifndef ADKV_SM_REG_MIN_ROWS
#define ADKV_SM_REG_MIN_ROWS 128
#endif
constexpr int SM_REG_MIN_ROWS = ADKV_SM_REG_MIN_ROWS;

template <int NV>
__global__ __launch_bounds__(1024) void softmax_regrow_kernel(
    const h1 *__restrict__ logits, h1 *__restrict__ weights, int n, long ld, float scaling)
{
    constexpr int NT = 1024;
    __shared__ float sm[NT / 64];
    const h1 *l = logits + (size_t)blockIdx.x * ld;
    h1 *w = weights + (size_t)blockIdx.x * ld;
    const int tid = threadIdx.x;
    const uint32_t pad = scaling > 0.0f ? 0xFC00FC00u : 0x7C007C00u; // scaling * pad = -inf

    uint4 raw[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int i0 = (v * NT + tid) * SM_VEC;
        if (i0 + SM_VEC <= n) {
            __builtin_memcpy(&raw[v], l + i0, 16); // rows are only 2-byte aligned
        } else {
            uint32_t u[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t lo = i0 + 2 * k < n ? __builtin_bit_cast(uint16_t, l[i0 + 2 * k]) : (pad & 0xFFFFu);
                const uint32_t hi = i0 + 2 * k + 1 < n ? __builtin_bit_cast(uint16_t, l[i0 + 2 * k + 1]) : (pad & 0xFFFFu);
                u[k] = lo | (hi << 16);
            }
            raw[v] = make_uint4(u[0], u[1], u[2], u[3]);
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const uint32_t u[4] = {raw[v].x, raw[v].y, raw[v].z, raw[v].w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const h2 p = as_h2(u[k]);
            mx = fmaxf(mx, fmaxf((float)p.x * scaling, (float)p.y * scaling));
        }
    }
    mx = block_reduce<NT>(mx, sm, true);
    // each walk converts the row again: values carried over from the walk before (which the
    // compiler would otherwise keep, 136 more registers per lane) are cut off here
    auto forget = [&]() {
#pragma unroll
        for (int v = 0; v < NV; v++)
            asm volatile("" : "+v"(raw[v].x), "+v"(raw[v].y), "+v"(raw[v].z), "+v"(raw[v].w));
    };
    forget();
    // exp(x * scaling - mx) = exp2(x * s2 + c2)
    const float s2 = scaling * 1.44269504088896340736f;
    const float c2 = mx == -INFINITY ? 0.0f : -mx * 1.44269504088896340736f;
    float sum = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const uint32_t u[4] = {raw[v].x, raw[v].y, raw[v].z, raw[v].w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const h2 p = as_h2(u[k]);
            sum += __builtin_amdgcn_exp2f(__builtin_fmaf((float)p.x, s2, c2));
            sum += __builtin_amdgcn_exp2f(__builtin_fmaf((float)p.y, s2, c2));
        }
    }
    sum = block_reduce<NT>(sum, sm, false);
    const float inv = 1.0f / sum;
    forget();
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int i0 = (v * NT + tid) * SM_VEC;
        const uint32_t u[4] = {raw[v].x, raw[v].y, raw[v].z, raw[v].w};
        uint32_t o[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const h2 p = as_h2(u[k]);
            o[k] = as_u32((h2){(h1)(__builtin_amdgcn_exp2f(__builtin_fmaf((float)p.x, s2, c2)) * inv),
                               (h1)(__builtin_amdgcn_exp2f(__builtin_fmaf((float)p.y, s2, c2)) * inv)});
        }
        if (i0 + SM_VEC <= n) {
            const uint4 ov = make_uint4(o[0], o[1], o[2], o[3]);
            __builtin_memcpy(w + i0, &ov, 16);
        } else {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const h2 p = as_h2(o[k]);
                if (i0 + 2 * k < n)
                    w[i0 + 2 * k] = p.x;
                if (i0 + 2 * k + 1 < n)
                    w[i0 + 2 * k + 1] = p.y;
            }
        }
    }
}

// Rows longer than one workgroup can hold in registers are cut into chunks of SM_CHUNK elements,
// one workgroup each: the first pass leaves (max, sum of exp(x - max)) per chunk, the second
// combines a row's chunks and normalises.  Each logit is read twice and nothing depends on the
// order in which workgroups run.

// (m, s) with s = sum of exp(x - m) over a set of elements; the pair of the union of two sets.
__device__ __forceinline__ float2 softmax_merge(float2 a, float2 b)
{
    const float m = fmaxf(a.x, b.x);
    if (m == -INFINITY)
        return make_float2(-INFINITY, 0.0f); // both sets empty or fully masked
    return make_float2(m, a.y * __expf(a.x - m) + b.y * __expf(b.x - m));
}

__device__ __forceinline__ float2 softmax_wave_merge(float2 v)
{
#pragma unroll
    for (int k = 1; k < 64; k <<= 1)
        v = softmax_merge(v, make_float2(__shfl_xor(v.x, k, 64), __shfl_xor(v.y, k, 64)));
    return v;
}

// SUB chunks per workgroup.  With SUB > 1 and every chunk inside the row, all of the workgroup's
// loads are issued before anything waits for one (a 256-thread workgroup that fetches 12 KB and
// leaves is mostly launch and latency: 3.0 TB/s over the 512 rows of 131 073 logits of the
// long-context shape; 48 KB per workgroup: see the kernel trace of that shape); the merged pair
// goes to the first chunk's slot and the other slots get the neutral element.
template <int SUB>
__global__ __launch_bounds__(SM_BLOCK) void softmax_part_kernel(
    const h1 *__restrict__ logits, const float *__restrict__ mask, float2 *__restrict__ part,
    int n, long ld, int nchunk, int rows_per_mask_row, float scaling)
{
    __shared__ float2 sm[SM_BLOCK / 64];
    const int row = blockIdx.y, ck0 = blockIdx.x * SUB;
    const h1 *l = logits + (size_t)row * ld;
    const float *mk = mask ? mask + (size_t)(row / rows_per_mask_row) * n : nullptr;
    float mx = -INFINITY, sum = 0.0f;
    if (SUB > 1 && !mk && (ck0 + SUB) * SM_CHUNK <= n) {
        uint4 raw[SUB][SM_NV];
#pragma unroll
        for (int s = 0; s < SUB; s++)
#pragma unroll
            for (int v = 0; v < SM_NV; v++)
                __builtin_memcpy(&raw[s][v], l + (size_t)(ck0 + s) * SM_CHUNK + (v * SM_BLOCK + threadIdx.x) * SM_VEC, 16);
        float x[SUB][SM_KEEP];
#pragma unroll
        for (int s = 0; s < SUB; s++)
#pragma unroll
            for (int v = 0; v < SM_NV; v++) {
                const uint32_t w[4] = {raw[s][v].x, raw[s][v].y, raw[s][v].z, raw[s][v].w};
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const h2 p = as_h2(w[k]);
                    x[s][v * SM_VEC + 2 * k] = (float)p.x * scaling;
                    x[s][v * SM_VEC + 2 * k + 1] = (float)p.y * scaling;
                    mx = fmaxf(mx, fmaxf(x[s][v * SM_VEC + 2 * k], x[s][v * SM_VEC + 2 * k + 1]));
                }
            }
        if (mx > -INFINITY) {
#pragma unroll
            for (int s = 0; s < SUB; s++)
#pragma unroll
                for (int k = 0; k < SM_KEEP; k++)
                    sum += __expf(x[s][k] - mx);
        }
    } else {
        // the generic way, a chunk at a time (chunks past the end of the row are all -inf)
        for (int s = 0; s < SUB; s++) {
            float x[SM_KEEP], m1;
            softmax_load_chunk(l, mk, n, (ck0 + s) * SM_CHUNK, scaling, x, m1);
            float s1 = 0.0f;
            if (m1 > -INFINITY) {
#pragma unroll
                for (int k = 0; k < SM_KEEP; k++)
                    s1 += __expf(x[k] - m1);
            }
            const float2 r = softmax_merge(make_float2(mx, sum), make_float2(m1, s1));
            mx = r.x;
            sum = r.y;
        }
    }
    // the thread's own (max, sum), then ONE reduction of pairs over the workgroup
    const float2 w = softmax_wave_merge(make_float2(mx, sum));
    if ((threadIdx.x & 63) == 0)
        sm[threadIdx.x >> 6] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        float2 r = sm[0];
#pragma unroll
        for (int i = 1; i < SM_BLOCK / 64; i++)
            r = softmax_merge(r, sm[i]);
        part[(size_t)row * nchunk + ck0] = r;
    }
    if (threadIdx.x > 0 && threadIdx.x < SUB && ck0 + (int)threadIdx.x < nchunk)
        part[(size_t)row * nchunk + ck0 + threadIdx.x] = make_float2(-INFINITY, 0.0f);
}

__global__ __launch_bounds__(SM_BLOCK) void softmax_norm_kernel(
    const h1 *__restrict__ logits, h1 *__restrict__ weights, const float *__restrict__ mask,
    const float2 *__restrict__ part, int n, long ld, int nchunk, int rows_per_mask_row, float scaling)
{
    __shared__ float2 row_stats;
    const int row = blockIdx.y, ck = blockIdx.x;
    const h1 *l = logits + (size_t)row * ld;
    h1 *w = weights + (size_t)row * ld;
    const float *mk = mask ? mask + (size_t)(row / rows_per_mask_row) * n : nullptr;
    float x[SM_KEEP], mx;
    softmax_load_chunk(l, mk, n, ck * SM_CHUNK, scaling, x, mx);   // issued first: in flight meanwhile
    if (threadIdx.x < 64) {
        // the row's (max, sum) from its chunks: one wave, a chunk per lane and round
        const float2 *pr = part + (size_t)row * nchunk;
        float2 v = make_float2(-INFINITY, 0.0f);
        for (int k = threadIdx.x; k < nchunk; k += 64)
            v = softmax_merge(v, pr[k]);
        v = softmax_wave_merge(v);
        if (threadIdx.x == 0)
            row_stats = v;
    }
    __syncthreads();
    const float M = row_stats.x, inv = 1.0f / row_stats.y;
#pragma unroll
    for (int k = 0; k < SM_KEEP; k++)
        x[k] = __expf(x[k] - M);
    softmax_store_chunk(w, n, ck * SM_CHUNK, x, inv);
}

} // namespace adkv

// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------
using namespace adkv;

static thread_local int g_last_hip_error = 0;

static int check_launch()
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return ADKV_E_LAUNCH;
    }
    return ADKV_OK;
}

static int check_common(int B, int H, int T, int D, int n_super_cap)
{
    if (B <= 0 || H <= 0 || T < 0 || n_super_cap <= 0)
        return ADKV_E_SHAPE;
    if (D != 128 && D != 256 && D != 512)
        return ADKV_E_DIM;
    if ((int64_t)B * H > (int64_t)INT32_MAX / 64)
        return ADKV_E_SHAPE;
    return ADKV_OK;
}

static inline int lanes_per_head(int D) { return D == 128 ? 32 : 64; }

#include "adkv_gqa_kernels.h"
#include "adkv_ft_kernels.h"

// Waves a SIMD should hold for packed-f16 issue to run near full rate, and SIMDs on the device.
constexpr int WAVES_PER_SIMD_TARGET = 4;
// Compute units of the device the calling thread is on, asked once per device (256 on an MI355X,
// and that is what every measurement behind the plans below was taken on).  Without a device (the
// planning entry points can be called on a host that has none) the MI355X's count is assumed.
static int cus()
{
    constexpr int MAX_DEV = 64, MI355X_CUS = 256;
    static std::atomic<int> cached[MAX_DEV];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) {
        (void)hipGetLastError(); // not this call's error to report
        return MI355X_CUS;
    }
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = MI355X_CUS;
        }
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}
static int n_simd() { return 4 * cus(); }

// Segment plan for a decode launch.  Starting from the fewest segments that give every SIMD its
// target of waves, finer splits are taken when they shorten the launch: 16-wave workgroups run one
// per CU, so a launch is ceil(workgroups / 256) rounds of one segment's length each, and a batch
// whose workgroup count falls just past a multiple of 256 (B = 352: 352 workgroups = 2 rounds for
// 1.4 rounds of work) wastes most of a round unless it is cut finer.
static Seg plan_segments(void *ckpt, int n_ckpt_cap, int ckpt_interval, int BH, int T, int D, int lanes = 0)
{
    Seg s;
    s.ckpt = (h1 *)ckpt;
    s.n_ckpt_cap = n_ckpt_cap;
    s.ckpt_interval = ckpt ? ckpt_interval : 0;
    s.seg_tokens = T > 0 ? T : 1;
    s.nseg = 1;
    s.row_pitch = T + 1;
    s.act_bf16 = 0;
    s.combine = 0;
    s.groups = 0;
    s.intervals = 0;
    s.phys_per_head = 0;
    s.skew = 0;
    if (!ckpt || ckpt_interval <= 0 || T <= ckpt_interval)
        return s;
    const int avail = (T + ckpt_interval - 1) / ckpt_interval;               // finest split
    const int lph = lanes ? lanes : lanes_per_head(D); // lanes: 16 for the two-pass per-head-table kernels
    const long units_target = (long)n_simd() * WAVES_PER_SIMD_TARGET * (64 / lph);
    long want = (units_target + BH - 1) / BH;
    if (want < 1)
        want = 1;
    if (want > avail)
        want = avail;
    const int m0 = (int)((avail + want - 1) / want);                          // intervals per segment
    // every segment start s*m*interval needs checkpoint s*m-1 < n_ckpt_cap
    auto valid = [&](int m) { return m >= avail || ((avail - 1) / m) * m - 1 < n_ckpt_cap; };
    // launch length in units of one checkpoint interval
    auto cost = [&](int m) {
        const int nseg = (avail + m - 1) / m;
        const long threads = (lph == 16 ? padded_units<16>(BH, nseg) : lph == 32 ? padded_units<32>(BH, nseg) : padded_units<64>(BH, nseg)) * lph;
        if (D == 512 || threads < 1024L * cus())
            return (double)m;                        // small workgroups: no round structure to model
        const long wgs = (threads + 1023) / 1024;
        return (double)((wgs + cus() - 1) / cus()) * m;
    };
    int best = -1;
    double best_cost = 0.0;
    for (int m = avail; m >= 1; m--) {
        if (m > m0 && m < avail)
            continue;                                // between "one segment" and the occupancy target: skip
        if (!valid(m))
            continue;
        const double c = cost(m);
        if (best < 0 || c < 0.97 * best_cost) {      // a finer split has to pay for its overheads
            best = m;
            best_cost = c;
        }
    }
    // the occupancy target comes first: one segment is only kept when no split is possible
    if (best >= avail && m0 < avail && valid(m0))
        best = m0;
    if (best < 0 || best >= avail)
        return s;
    s.seg_tokens = best * ckpt_interval;
    s.nseg = (T + s.seg_tokens - 1) / s.seg_tokens;
    return s;
}

template <typename F256, typename FBIG>
static void launch_units(long threads, int big, F256 f256, FBIG fbig)
{
    // 16-wave workgroups share one lookup table and let a CU hold 4 waves per SIMD; small launches
    // use 4-wave workgroups so that they still spread over the CUs
    if (big > 256 && threads >= (long)big * cus())
        fbig(dim3((unsigned)((threads + big - 1) / big)), dim3(big));
    else
        f256(dim3((unsigned)((threads + 255) / 256)), dim3(256));
}

#define ADKV_LAUNCH(KERNEL, DD, CC, BIG, ...)                                                   \
    launch_units(                                                                               \
        padded_units<DD / CC>(BH, seg.nseg) * (DD / CC), BIG,                                                  \
        [&](dim3 g, dim3 b) { hipLaunchKernelGGL((KERNEL<DD, CC, 256>), g, b, 0, st, __VA_ARGS__); }, \
        [&](dim3 g, dim3 b) { hipLaunchKernelGGL((KERNEL<DD, CC, BIG>), g, b, 0, st, __VA_ARGS__); })

// Head dim 128 has a second shape, two channels per lane (a head per wave): twice the waves, each
// with half the instruction stream per token.  It pays when every wave has a SIMD to itself and
// the launch is bound by the length of that stream (small batches, or no checkpoints to cut the
// context with); with more waves per SIMD the four-channel lanes do less work in total.
#define ADKV_DISPATCH_D(KERNEL, ...)                  \
    switch (D) {                                      \
    case 128:                                         \
        if (padded_units<32>(BH, seg.nseg) / 2 <= n_simd()) \
            ADKV_LAUNCH(KERNEL, 128, 2, 256, __VA_ARGS__); \
        else                                          \
            ADKV_LAUNCH(KERNEL, 128, 4, 1024, __VA_ARGS__); \
        break;                                        \
    case 256:                                         \
        ADKV_LAUNCH(KERNEL, 256, 4, 1024, __VA_ARGS__); \
        break;                                        \
    default:                                          \
        ADKV_LAUNCH(KERNEL, 512, 8, 256, __VA_ARGS__); \
        break;                                        \
    }

// Matrix-core kernels (head dim 128): 16-wave workgroups for big launches, 8-wave ones otherwise
// (their LDS tile leaves room for one workgroup per CU either way).  Eight query heads per KV head
// need ~138 registers per lane, more than the 128 a 16-wave workgroup leaves: qk_gqa_kernel still
// gains from four waves per SIMD with a dozen cold values spilled (cfg5 KV shape, 64 query heads:
// 563 -> 530 us with 4-bit codes, 518 -> 425 us with 2-bit ones), ov_gqa_kernel spills
// accumulators and loses (421 -> 533 us, 346 -> 747 us), so BIG8 says which of the two this is.
#define ADKV_LAUNCH_GQA(KERNEL, BIG8, BB, GQV, ...)                                                \
    do {                                                                                            \
        const long threads = padded_units<32>(BH, seg.nseg) * 32;                                   \
        constexpr int GBIG = (GQV <= 4 || BIG8) ? GQV : 1; /* unused instantiation otherwise */     \
        if ((GQV <= 4 || BIG8) && threads >= 1024L * cus())                                         \
            hipLaunchKernelGGL((KERNEL<BB, GBIG, 1024>), dim3((unsigned)((threads + 1023) / 1024)), \
                               dim3(1024), 0, st, __VA_ARGS__);                                     \
        else                                                                                        \
            hipLaunchKernelGGL((KERNEL<BB, GQV, 512>), dim3((unsigned)((threads + 511) / 512)),     \
                               dim3(512), 0, st, __VA_ARGS__);                                      \
    } while (0)

#define ADKV_DISPATCH_GQ_BITS(KERNEL, BIG8, BB, ...)                                               \
    switch (GQ) {                                                                                   \
    case 1: ADKV_LAUNCH_GQA(KERNEL, BIG8, BB, 1, __VA_ARGS__); break;                               \
    case 2: ADKV_LAUNCH_GQA(KERNEL, BIG8, BB, 2, __VA_ARGS__); break;                               \
    case 4: ADKV_LAUNCH_GQA(KERNEL, BIG8, BB, 4, __VA_ARGS__); break;                               \
    case 8: ADKV_LAUNCH_GQA(KERNEL, BIG8, BB, 8, __VA_ARGS__); break;                               \
    default: return ADKV_E_UNSUPPORTED;                                                             \
    }

#define ADKV_DISPATCH_GQ(KERNEL, BIG8, ...)                                                        \
    if (bits == 4) {                                                                                \
        ADKV_DISPATCH_GQ_BITS(KERNEL, BIG8, 4, __VA_ARGS__)                                         \
    } else {                                                                                        \
        ADKV_DISPATCH_GQ_BITS(KERNEL, BIG8, 2, __VA_ARGS__)                                         \
    }

// Whether single-query-head launches (GQ == 1, head dim 128) also take the matrix-core kernels:
// the built-in choice, overridden by ADKV_MFMA=0/1 in the environment, overridden by
// adkv_set_mha_kernel().
// The environment is read once, when the first launch asks; the override is an atomic so that
// launches from several host threads never see a torn value.
static std::atomic<int> g_mha_kernel{-1};
static int mha_kernel_default()
{
    static const int from_env = [] {
        const char *e = getenv("ADKV_MFMA");
        return (e ? atoi(e) : 0) != 0 ? 1 : 0;
    }();
    return from_env;
}
static bool mfma_for_mha()
{
    const int v = g_mha_kernel.load(std::memory_order_relaxed);
    return (v < 0 ? mha_kernel_default() : v) == 1;
}

// Whether a launch with one query head per KV head takes the kernels with a per-head table
// (adkv_ft_kernels.h).  They need head dim 128 and 4-bit codes.  By default the choice follows a
// model of the two launches, both bound by vector issue: the per-head-table kernels run 16-wave
// workgroups, one per CU, in ceil(workgroups / 256) rounds of one segment each (every head's
// waves padded to whole workgroups), at 0.93 of the shared-table kernels' time per wave; the
// shared-table kernels run the same rounds when the launch is big enough for 16-wave workgroups,
// and otherwise spread 4-wave workgroups over the SIMDs, where the fullest SIMD sets the time
// (its waves / 4 rounds).  Measured (B x 32 heads, ctx; per-head table against shared table):
// 128 x 4096: 587 / 624 us per layer-step, 34 x 3000: 155 / 181, 40 x 1500: 89 / 107, 24 x 3000:
// 141 / 141, 20 x 8192 (288 workgroups, two rounds): 369 / 255.  adkv_set_mha_kernel(2) takes them whenever they can run (3: with 16 lanes per head, 4: with 32), (0) never.
static bool use_head_table(int B, int H, int GQ, int bits, int D, const Seg &seg)
{
    if (D != 128 || bits != 4 || GQ != 1)
        return false;
    const int v = g_mha_kernel.load(std::memory_order_relaxed);
    if (v >= 2)
        return true;
    if (v >= 0 || mha_kernel_default() == 1)
        return false;
    const long BH = (long)B * H;
    const long padded = padded_units<32>((int)BH, seg.nseg);
    const long waves_shared = padded / 2;
    if (waves_shared <= n_simd())
        return false;                                 // every wave a SIMD to itself: two-channel lanes
    const long wgs_ft = (long)H * ft_wgs_per_head(B, seg.nseg, 2);
    const double t_ft = 0.93 * (double)((wgs_ft + cus() - 1) / cus());
    double t_shared;
    if (padded * 32 >= (long)FT_BLK * cus())
        t_shared = (double)(((padded * 32 + FT_BLK - 1) / FT_BLK + cus() - 1) / cus());
    else
        t_shared = (double)((waves_shared + n_simd() - 1) / n_simd()) / WAVES_PER_SIMD_TARGET;
    return t_ft <= t_shared;
}

// The plan of a launch that takes the per-head-table kernels.
//
// A SIMD issues from its OLDEST resident wave whenever that wave has an instruction ready (wave
// priorities set by the program do not change that on this chip), and one wave alone keeps the
// vector pipe only about half busy.  Four waves with equal shares of work therefore finish one
// after the other (measured at B=128, 32 heads, 4096 tokens in two even segments: the four waves of
// a SIMD are done after 131, 188, 261 and 327 us) and the pipe idles more and more towards the end.
// So the shares are made UNEVEN, in the proportions in which the four slots of a SIMD actually
// progress while all are resident (FT_SKEW, oldest first): a workgroup's waves 4k..4k+3 are slot k
// of its four SIMDs, interleave_segment gives quad k of a workgroup segment k of a group of four,
// and the context of every sequence is cut into groups of four such segments, at checkpoints.
//
// That needs four segments where the even plan has one or two, hence more workgroups than CUs;
// a second round of workgroups costs a table build, a launch gap and a second ragged end (12 % at
// the shape above).  Instead each launched workgroup walks through several VIRTUAL workgroups of
// its head one after the other (phys_per_head apart) with no barrier between them.
//
// Measured at B=128, 32 heads, 4096 tokens, checkpoints every 256 (medians of interleaved runs on
// one device, us): forward_qk 300-303 with two even segments, 297 with four even ones walked as
// two virtual workgroups, 280-285 with shares 7:5:2:2 (8:4:2:2 and 6:6:3:1 within 3 us of that,
// 9:4:2:1 302); forward_ov 261 with two even segments added inside the workgroup, 262-266 with the
// best uneven shares (6:5:3:2, 7:5:2:2) plus the 4 us kernel that then adds the partial sums: no
// gain, so forward_ov takes uneven shares only where one group of four segments fills the device and
// the four are added inside the workgroup (plan_ft_ov): with 16 lanes per head at that shape, 259
// even, 250 with 6:5:3:2 (8:4:2:2 251, 7:5:2:2 252, 6:4:3:3 and 5:5:3:3 257).
// Shares of a SIMD's work given to its four wave slots, oldest first, in sixteenths of a group's
// checkpoint intervals: measured on the headline shape, one setting per kernel.
constexpr unsigned FT_SKEW_QK = pack_skew(7, 5, 2, 2);
constexpr unsigned FT_SKEW_OV = pack_skew(6, 5, 3, 2);
// matrix-core kernels in 16-wave workgroups, measured on B=16, 32 query heads over 8 KV heads, 131072
// tokens of 2-bit codes (64 segments, us): forward_qk 320 even, 299 with 6:5:3:2 (305 with 7:5:2:2,
// 318 with 6:6:3:1, 330 with 8:4:2:2); forward_ov 265 even, 252 with 6:5:3:2 / 6:6:3:1 / 8:5:2:1
constexpr unsigned GQA_SKEW_QK = pack_skew(6, 5, 3, 2);
constexpr unsigned GQA_SKEW_OV = pack_skew(6, 5, 3, 2);
constexpr bool FT16_QK = true, FT16_OV = true; // whether forward_qk / forward_ov may take 16 lanes per head
constexpr int FT_MIN_GROUP = 8;  // checkpoint intervals a group needs for its shares to differ
constexpr int FT_MAX_GROUPS = 16;

// Longest segment of an uneven cut, in checkpoint intervals (the oldest wave slot's of the group
// that got the most intervals).
static int uneven_longest(int groups, int intervals, unsigned skew)
{
    int longest = 0;
    for (int g = 0; g < groups; g++) {
        const int n = uneven_cut(4 * g + 4, groups, intervals, skew) - uneven_cut(4 * g + 3, groups, intervals, skew);
        if (n > longest)
            longest = n;
    }
    return longest;
}

// What a unit (one wave's segment) costs besides its tokens, in tokens: parameters, checkpoint,
// the first loads' latency, the first lookups, the last reduction.
constexpr int FT_UNIT_OVERHEAD_TOKENS = 32;

// Groups and workgroups per head are chosen together, for the shortest launch by the model
//   rounds of workgroups on the CUs x virtual workgroups walked through by each x longest segment.
// (Groups by occupancy alone, then workgroups, left awkward batches on two thirds of the CUs:
// 40 sequences x 32 heads x 8192 tokens took two groups and 160 workgroups of two virtual ones
// where three groups fill 256.)  Ties go to fewer groups, then fewer workgroups.  virtual_ok =
// false (forward_ov, whose kernel runs one virtual workgroup per workgroup) only considers plans
// with as many workgroups as virtual ones.
static void plan_head_table(Seg &seg, int B, int H, int T, unsigned skew, int upw, bool virtual_ok = true)
{
    seg.groups = 0;
    seg.skew = skew;
    seg.phys_per_head = ft_wgs_per_head(B, seg.nseg, upw);
    if (!seg.ckpt || seg.ckpt_interval <= 0 || skew == 0)
        return;
    const int iv = seg.ckpt_interval;
    const int avail = (T + iv - 1) / iv;
    int gmax = avail / FT_MIN_GROUP; // FT_MIN_GROUP intervals or more per group
    if (gmax > FT_MAX_GROUPS)
        gmax = FT_MAX_GROUPS;
    int best_g = 0, best_p = 0;
    double best_cost = -1.0;
    for (int G = 1; G <= gmax; G++) {
        // segment s > 0 starts from checkpoint cut(s) - 1
        if (uneven_cut(4 * G - 1, G, avail, skew) - 1 >= seg.n_ckpt_cap)
            continue;
        const int W = ft_wgs_per_head(B, 4 * G, upw);
        const double unit = (double)uneven_longest(G, avail, skew) * iv + FT_UNIT_OVERHEAD_TOKENS;
        for (int P = virtual_ok ? 1 : W; P <= W; P++) {
            const double cost = (double)(((long)H * P + cus() - 1) / cus()) * ((W + P - 1) / P) * unit;
            if (best_cost < 0.0 || cost < 0.999 * best_cost) {
                best_g = G;
                best_p = P;
                best_cost = cost;
            }
        }
    }
    if (best_g == 0)
        return;
    seg.groups = best_g;
    seg.intervals = avail;
    seg.nseg = 4 * best_g;
    seg.seg_tokens = iv; // not read by the kernels of an uneven plan
    seg.phys_per_head = best_p;
}

// Length of a launch under a per-head-table plan, in tokens of a 32-lane wave's work: rounds of
// workgroups on the CUs x virtual workgroups walked through by each x the longest segment (the
// oldest wave slot's), x 1.86 for a head over 16 lanes (eight channels per lane at 0.93 of the
// instructions per channel).
static double ft_plan_cost(const Seg &s, int B, int H, int T, int upw)
{
    const int W = ft_wgs_per_head(B, s.nseg, upw);
    const int P = s.phys_per_head > 0 ? s.phys_per_head : W;
    const long rounds = ((long)H * P + cus() - 1) / cus();
    const int virt = (W + P - 1) / P;
    const int longest = s.groups ? uneven_longest(s.groups, s.intervals, s.skew) * s.ckpt_interval
                                 : (s.seg_tokens < T ? s.seg_tokens : T);
    return (double)rounds * virt * (longest + FT_UNIT_OVERHEAD_TOKENS) * (upw == 4 ? 1.86 : 1.0);
}

// Lanes per head of the per-head-table kernels for a launch, and its plan (`seg` comes in as the
// launch's even plan for 32 lanes and goes out as the plan to run).  Sixteen lanes per head (four
// sequences per wave, two passes over every supergroup) spend 5-7 % fewer instructions per channel
// but need twice the segments for the same number of waves.  They are taken when their plan is
// uneven with groups of at least FT16_MIN_GROUP checkpoint intervals (so that the four shares keep
// their proportions and the shortest segment its length) and shorter than the 32-lane plan by
// ft_plan_cost; 32 lanes otherwise.  Measured, 32 heads, checkpoints every 256 tokens, layer-step
// with 32 / 16 lanes in us (each with the plan the model picks for it): B x ctx 128 x 4096
// 581 / 552, 100 x 4096 528 / 475, 200 x 4096 1014 / 948, 352 x 4096 1667 / 1563, 16 x 32768
// 570 / 537 (16 lanes shorter by the model); 24 x 16384 463 / 495, 40 x 8192 406 / 473, 96 x 4096
// 466 / 481, 8 x 65536 569 / 714 (32 lanes shorter: the 16-lane plans leave padding waves or CUs
// idle); 64 x 4096 303 / 304, 128 x 2048 290 / 304 (groups of 8); 128 x 640 106 / 131 (even plans).
constexpr int FT16_MIN_GROUP = 16;
static int plan_ft(Seg &seg, int B, int H, int T, unsigned skew, bool sixteen_ok, bool virtual_ok = true)
{
    const int forced = g_mha_kernel.load(std::memory_order_relaxed); // 3: sixteen lanes, 4: thirty-two
    Seg s32 = seg;
    plan_head_table(s32, B, H, T, skew, 2, virtual_ok);
    if (sixteen_ok && forced != 4) {
        Seg s16 = plan_segments(seg.ckpt, seg.n_ckpt_cap, seg.ckpt_interval, B * H, T, 128, 16);
        s16.row_pitch = seg.row_pitch;
        s16.act_bf16 = seg.act_bf16;
        plan_head_table(s16, B, H, T, skew, 4, virtual_ok);
        const bool long_groups = s16.groups > 0 && s16.intervals / s16.groups >= FT16_MIN_GROUP;
        if (forced == 3 ||
            (long_groups && ft_plan_cost(s16, B, H, T, 4) < 0.97 * ft_plan_cost(s32, B, H, T, 2))) {
            seg = s16;
            return 16;
        }
    }
    seg = s32;
    return 32;
}

// forward_ov's plan: ov_ft_kernel runs one virtual workgroup per workgroup and adds two or four
// segments of a sequence inside the workgroup; whatever else it leaves in the workspace costs a
// second kernel of some 5 us.  Uneven shares pay with a head over 16 lanes (measured at 16-lane
// shapes: 128 x 4096 266 -> 249 us added in the workgroup; 16 x 32768, 64 x 8192, 32 x 16384
// 262 -> 242 us through the workspace) and not with a head over 32 (64 x 4096: 127.5 either way;
// 8 x 65536: 250 even, 258 uneven): they are taken when the uneven plan has 16 lanes per head and
// needs no virtual workgroups, the even plan for 32 lanes otherwise.
static int plan_ft_ov(Seg &seg, int B, int H, int T)
{
    Seg un = seg;
    const int lanes_un = plan_ft(un, B, H, T, FT_SKEW_OV, FT16_OV, false);
    if (lanes_un == 16 && un.groups >= 1 && un.phys_per_head == ft_wgs_per_head(B, un.nseg, 4)) {
        seg = un;
        return 16;
    }
    return plan_ft(seg, B, H, T, 0, FT16_OV);
}
static bool ft_ov_combines(const Seg &seg, int B, int lanes)
{
    return (seg.nseg == 2 || seg.nseg == 4) && seg.phys_per_head == ft_wgs_per_head(B, seg.nseg, 64 / lanes);
}

// The same uneven shares for the kernels without virtual workgroups (matrix-core and shared-table
// kernels in 16-wave workgroups, where a workgroup's quads of waves are the four slots of its
// SIMDs as well): the even plan's segments, when their number is a multiple of four, are re-cut
// in groups of four.  The segment count, and with it the workgroup count, stays what it was.
static void plan_uneven(Seg &seg, int T, long threads, unsigned skew)
{
    seg.groups = 0;
    seg.skew = skew;
    if (skew == 0 || !seg.ckpt || seg.ckpt_interval <= 0 || threads < 1024L * cus() || seg.nseg < 4 || (seg.nseg & 3))
        return;
    const int avail = (T + seg.ckpt_interval - 1) / seg.ckpt_interval;
    const int G = seg.nseg / 4;
    if (G > FT_MAX_GROUPS || avail / G < FT_MIN_GROUP)
        return;
    if (uneven_cut(4 * G - 1, G, avail, skew) - 1 >= seg.n_ckpt_cap)
        return;
    seg.groups = G;
    seg.intervals = avail;
}

// How many segments the forward_ov partial sums of a launch can have under either plan (what a
// workspace must be sized for: the kernel family can be switched between sizing and launch).
static int max_plan_segments(void *ckpt, int n_ckpt_cap, int ckpt_interval, int B, int H, int T, int D)
{
    Seg seg = plan_segments(ckpt, n_ckpt_cap, ckpt_interval, B * H, T, D);
    int n = seg.nseg;
    if (D == 128) {
        Seg a = seg, b = seg, c = seg;
        plan_head_table(a, B, H, T, FT_SKEW_QK, 2);
        plan_ft(b, B, H, T, FT_SKEW_QK, true);
        plan_ft_ov(c, B, H, T);
        n = std::max(std::max(n, a.nseg), std::max(b.nseg, c.nseg));
    }
    return n;
}

// Whether adkv_decode_step may run its three stages as ONE launch (decode_ft_kernel): off unless
// adkv_set_fused_step(1) asks for it.  Measured at B=128, 32 heads, 4096 tokens (builds alternating
// in one process): 545 us per layer-step in one launch against 543 us in three.  The launch gaps
// and the softmax kernel that the fused launch saves (some 40 us of device idle time per step) buy
// nothing: the device then runs the same instructions at a lower clock.
static std::atomic<int> g_fused_step{0};

// The plans of a fused step, or 0: per-head-table kernels, forward_qk and forward_ov both on four
// segments per sequence with the same lane width and as many workgroups as virtual ones (then the
// four quads of a workgroup hold the four segments of the same sequences).  Returns the lanes
// per head.
static int fused_step_plan(Seg &ka, Seg &va, int B, int Hq, int H, int T, int D, int bits, void *k_ckpt,
                           void *v_ckpt, int n_ckpt_cap, int ckpt_interval)
{
    if (g_fused_step.load(std::memory_order_relaxed) == 0 || Hq != H || D != 128 || bits != 4 || T < 1 ||
        T + 1 > FT_SOFTMAX_MAX_ROW || !k_ckpt || !v_ckpt)
        return 0;
    ka = plan_segments(k_ckpt, n_ckpt_cap, ckpt_interval, B * H, T, D);
    if (mfma_for_mha() || !use_head_table(B, H, 1, bits, D, ka))
        return 0;
    va = plan_segments(v_ckpt, n_ckpt_cap, ckpt_interval, B * H, T, D);
    const int lanes = plan_ft(ka, B, H, T, FT_SKEW_QK, FT16_QK);
    const int lanes_v = plan_ft_ov(va, B, H, T);
    const int W = ft_wgs_per_head(B, 4, 64 / lanes);
    if (lanes != lanes_v || ka.nseg != 4 || va.nseg != 4 || ka.phys_per_head != W || va.phys_per_head != W)
        return 0;
    return lanes;
}

static int check_ckpt(const void *ckpt, int n_ckpt_cap, int ckpt_interval, int bits = 4)
{
    if (!ckpt)
        return ADKV_OK;
    // a checkpoint sits on a supergroup boundary: 8 tokens with 4-bit codes, 16 with 2-bit ones
    if (n_ckpt_cap <= 0 || ckpt_interval <= 0 || (ckpt_interval % (32 / bits)))
        return ADKV_E_SHAPE;
    if ((uintptr_t)ckpt & 3)
        return ADKV_E_ALIGN;
    return ADKV_OK;
}

extern "C" {

int adkv_abi_version(void) { return 16; }

void adkv_set_fused_step(int mode) { g_fused_step.store(mode > 0 ? 1 : 0, std::memory_order_relaxed); }

int adkv_decode_step_is_fused(int B, int Hq, int H, int T, int D, int bits, int n_ckpt_cap, int ckpt_interval,
                              int masked)
{
    int dummy = 0;
    Seg ka, va;
    void *ck = n_ckpt_cap > 0 && ckpt_interval > 0 ? &dummy : nullptr;
    if (masked || B <= 0 || H <= 0 || Hq <= 0 || T < 0)
        return 0;
    return fused_step_plan(ka, va, B, Hq, H, T, D, bits, ck, ck, n_ckpt_cap, ckpt_interval) ? 1 : 0;
}

void adkv_set_mha_kernel(int use_matrix_cores)
{
    g_mha_kernel.store(use_matrix_cores < 0 ? -1 : (use_matrix_cores > 4 ? 1 : use_matrix_cores),
                       std::memory_order_relaxed);
}

int adkv_last_hip_error(void) { return g_last_hip_error; }

const char *adkv_strerror(int code)
{
    switch (code) {
    case ADKV_OK: return "ok";
    case ADKV_E_NULL: return "required pointer is NULL";
    case ADKV_E_DIM: return "DIM must be 128, 256 or 512";
    case ADKV_E_SHAPE: return "invalid shape";
    case ADKV_E_CAPACITY: return "cache capacity too small";
    case ADKV_E_ALIGN: return "pointer not sufficiently aligned";
    case ADKV_E_UNSUPPORTED: return "unsupported configuration";
    case ADKV_E_WORKSPACE: return "workspace too small";
    case ADKV_E_SCRATCH_LIMIT:
        return "launch needs more scratch than the library's static buffer holds (adkv_static_scratch_bytes)";
    case ADKV_E_DEVICE: return "HIP device query failed";
    case ADKV_E_LAUNCH: return "HIP launch failed";
    default: return "unknown error";
    }
}

// One tensor, or two of the same shape (v_cache != NULL) in one launch.
static int encode_common(void *cache, const void *kv_new,
                         const void *zp, const void *sc, const void *alpha, const void *beta,
                         const void *tgt,
                         int B, int H, int T0, int T, int D, int n_super_cap,
                         const void *state_in, void *state_out, void *ckpt_out, int n_ckpt_cap,
                         int ckpt_interval, void *stream, int bits = 4,
                         const EncTensor *second = nullptr, const RowStrides *first_strides = nullptr,
                         bool bf16 = false)
{
    if (!cache || !kv_new || !zp || !sc || !alpha || !beta || !tgt)
        return ADKV_E_NULL;
    if (second && (!second->cache || !second->kv_new || !second->zp || !second->sc || !second->al ||
                   !second->be || !second->tg))
        return ADKV_E_NULL;
    if (bits != 2 && bits != 4)
        return ADKV_E_UNSUPPORTED;
    int rc = check_common(B, H, T, D, n_super_cap);
    if (rc)
        return rc;
    if (T0 < 0 || T0 > T)
        return ADKV_E_SHAPE;
    if (T0 > 0 && (!state_in || (second && !second->state_in)))
        return ADKV_E_NULL;
    const int tpw = 32 / bits;
    if ((T + tpw - 1) / tpw > n_super_cap)
        return ADKV_E_CAPACITY;
    if (((uintptr_t)cache & 15) || ((uintptr_t)kv_new & 3))
        return ADKV_E_ALIGN;
    if (second && (((uintptr_t)second->cache & 15) || ((uintptr_t)second->kv_new & 3)))
        return ADKV_E_ALIGN;
    if (second && (ckpt_out == nullptr) != (second->ckpt == nullptr))
        return ADKV_E_NULL; // both tensors keep checkpoints or neither does
    const RowStrides packed = {(long)H * (T - T0) * D, (long)(T - T0) * D, (long)D};
    const RowStrides xs1 = first_strides ? *first_strides : packed;
    for (const RowStrides *xs : {&xs1, second ? &second->xs : &xs1}) {
        // rows are read as aligned 32-bit words
        if (xs->b < 0 || xs->h < 0 || xs->t < D || (xs->b | xs->h | xs->t) & 1)
            return ADKV_E_SHAPE;
    }
    if ((rc = check_ckpt(ckpt_out, n_ckpt_cap, ckpt_interval, bits)))
        return rc;
    if (T == T0 && !second && (state_out == nullptr || state_out == state_in))
        return ADKV_OK;
    const int BH = B * H;
    hipStream_t st = (hipStream_t)stream;
    Seg seg;
    seg.ckpt = (h1 *)ckpt_out;
    seg.n_ckpt_cap = n_ckpt_cap;
    seg.ckpt_interval = ckpt_out ? ckpt_interval : 0;
    seg.seg_tokens = T > 0 ? T : 1;
    seg.nseg = 1;
    seg.row_pitch = T + 1;
    seg.act_bf16 = 0;
    seg.combine = 0;
    seg.groups = 0;
    seg.intervals = 0;
    seg.phys_per_head = 0;
    seg.skew = 0;
    // Lane width, measured on an MI355X (4096 tokens, ms for 65 536 / 131 072 / 196 608 / 262 144 /
    // 524 288 channels): one channel per lane 0.29 / 0.44 / 0.60 / 0.74 / 1.38, two 0.43 / 0.44 /
    // 0.55 / 0.60 / 1.17, four 0.78 / 0.78 / 0.78 / 0.79 / 1.18.  Up to two waves per SIMD the
    // one-channel lanes win (each wave is paced by its own dependent chain, and only they run the
    // branch-free speculative form); beyond that two channels share the packed fp16 updates.
    // Four channels per lane never win and are not instantiated.
    const long channels = (long)BH * D;
    const long tensors = second ? 2 : 1;
    int cpl = tensors * channels > 2L * 64 * n_simd() + 32768 ? 2 : 1;
    const long lanes = channels / cpl;
    const dim3 grid((unsigned)((lanes + 255) / 256), (unsigned)tensors), block(256);
    EncTensor first;
    first.cache = (uint32_t *)cache;
    first.kv_new = (const h1 *)kv_new;
    first.zp = (const h1 *)zp;
    first.sc = (const h1 *)sc;
    first.al = (const h1 *)alpha;
    first.be = (const h1 *)beta;
    first.tg = (const h1 *)tgt;
    first.state_in = (const h1 *)state_in;
    first.state_out = (h1 *)state_out;
    first.ckpt = (h1 *)ckpt_out;
    first.xs = xs1;
#define ADKV_ENC(BB, C)                                                                          \
    do {                                                                                         \
        if (second && bf16)                                                                      \
            hipLaunchKernelGGL((encode_pair_kernel<BB, C, 256, true>), grid, block, 0, st,       \
                               first, *second, BH, H, T0, T, D, n_super_cap, seg);               \
        else if (second)                                                                         \
            hipLaunchKernelGGL((encode_pair_kernel<BB, C, 256, false>), grid, block, 0, st,      \
                               first, *second, BH, H, T0, T, D, n_super_cap, seg);               \
        else                                                                                     \
            hipLaunchKernelGGL((encode_kernel<BB, C, 256>), grid, block, 0, st, first.cache,     \
                               first.kv_new, first.zp, first.sc, first.al, first.be, first.tg,   \
                               BH, H, T0, T, D, n_super_cap, first.state_in, first.state_out,    \
                               seg);                                                             \
    } while (0)
#define ADKV_ENC_CPL(BB)                                                                         \
    do {                                                                                         \
        if (cpl == 2)                                                                            \
            ADKV_ENC(BB, 2);                                                                     \
        else                                                                                     \
            ADKV_ENC(BB, 1);                                                                     \
    } while (0)
    if (bits == 4)
        ADKV_ENC_CPL(4);
    else
        ADKV_ENC_CPL(2);
#undef ADKV_ENC_CPL
#undef ADKV_ENC
    return check_launch();
}

int adkv_encode_kv_ex(void *cache, const void *kv_new,
                      const void *zp, const void *sc, const void *alpha, const void *beta,
                      const void *tgt,
                      int B, int H, int T, int D, int n_super_cap,
                      void *state_out, void *ckpt_out, int n_ckpt_cap, int ckpt_interval,
                      void *stream)
{
    return encode_common(cache, kv_new, zp, sc, alpha, beta, tgt, B, H, 0, T, D, n_super_cap,
                         nullptr, state_out, ckpt_out, n_ckpt_cap, ckpt_interval, stream);
}

int adkv_append_kv(void *cache, const void *kv_new,
                   const void *zp, const void *sc, const void *alpha, const void *beta,
                   const void *tgt,
                   int B, int H, int T0, int n_new, int D, int n_super_cap, int bits,
                   void *state_io, void *ckpt, int n_ckpt_cap, int ckpt_interval, void *stream)
{
    if (!state_io)
        return ADKV_E_NULL;
    if (n_new < 0)
        return ADKV_E_SHAPE;
    if (n_new == 0)
        return ADKV_OK; // nothing to quantise; state_io already is the answer
    return encode_common(cache, kv_new, zp, sc, alpha, beta, tgt, B, H, T0, T0 + n_new, D,
                         n_super_cap, state_io, state_io, ckpt, n_ckpt_cap, ckpt_interval, stream,
                         bits);
}

int adkv_append_kv_pair(void *k_cache, void *v_cache, const void *k_new, const void *v_new,
                        int kv_dtype, const int64_t *k_strides, const int64_t *v_strides,
                        const void *const *k_params, const void *const *v_params,
                        int B, int H, int T0, int n_new, int D, int n_super_cap, int bits,
                        void *k_state_io, void *v_state_io, void *k_ckpt, void *v_ckpt,
                        int n_ckpt_cap, int ckpt_interval, void *stream)
{
    if (!k_params || !v_params || !k_state_io || !v_state_io)
        return ADKV_E_NULL;
    if (kv_dtype != ADKV_DT_F16 && kv_dtype != ADKV_DT_BF16)
        return ADKV_E_UNSUPPORTED;
    if (n_new < 0)
        return ADKV_E_SHAPE;
    if (n_new == 0)
        return ADKV_OK;
    const RowStrides packed = {(long)H * n_new * D, (long)n_new * D, (long)D};
    const RowStrides ks = k_strides ? RowStrides{(long)k_strides[0], (long)k_strides[1], (long)k_strides[2]} : packed;
    EncTensor v;
    v.cache = (uint32_t *)v_cache;
    v.kv_new = (const h1 *)v_new;
    v.zp = (const h1 *)v_params[0];
    v.sc = (const h1 *)v_params[1];
    v.al = (const h1 *)v_params[2];
    v.be = (const h1 *)v_params[3];
    v.tg = (const h1 *)v_params[4];
    v.state_in = (const h1 *)v_state_io;
    v.state_out = (h1 *)v_state_io;
    v.ckpt = (h1 *)v_ckpt;
    v.xs = v_strides ? RowStrides{(long)v_strides[0], (long)v_strides[1], (long)v_strides[2]} : packed;
    return encode_common(k_cache, k_new, k_params[0], k_params[1], k_params[2], k_params[3],
                         k_params[4], B, H, T0, T0 + n_new, D, n_super_cap, k_state_io, k_state_io,
                         k_ckpt, n_ckpt_cap, ckpt_interval, stream, bits, &v, &ks,
                         kv_dtype == ADKV_DT_BF16);
}

int adkv_encode_kv(void *cache, const void *kv_new,
                   const void *zp, const void *sc, const void *alpha, const void *beta,
                   const void *tgt,
                   int B, int H, int T, int D, int n_super_cap,
                   float, float, void *state_out, void *stream)
{
    return adkv_encode_kv_ex(cache, kv_new, zp, sc, alpha, beta, tgt, B, H, T, D, n_super_cap,
                             state_out, nullptr, 0, 0, stream);
}

} // extern "C"

// Which decode kernel family and shape a launch of these sizes takes (the dispatch below, as text).
static const char *decode_kernel_name(int B, int Hq, int H, int T, int D, int bits, int n_ckpt_cap,
                                      int ckpt_interval)
{
    if (B <= 0 || H <= 0 || Hq <= 0 || Hq % H || T < 0 || (D != 128 && D != 256 && D != 512) ||
        (bits != 2 && bits != 4))
        return "invalid";
    const int GQ = Hq / H;
    if ((GQ > 1 || bits != 4) && D != 128)
        return "invalid";
    int dummy = 0;
    const Seg seg = plan_segments(n_ckpt_cap > 0 && ckpt_interval > 0 ? &dummy : nullptr, n_ckpt_cap,
                                  ckpt_interval, B * H, T, D);
    if (D == 128 && (GQ > 1 || bits != 4 || mfma_for_mha())) {
        const long threads = padded_units<32>(B * H, seg.nseg) * 32;
        return threads >= 1024L * cus() ? "gqa_kernel, 16-wave workgroups (matrix cores)"
                                      : "gqa_kernel, 8-wave workgroups (matrix cores)";
    }
    if (use_head_table(B, H, GQ, bits, D, seg)) {
        Seg s2 = seg;
        const int lanes = plan_ft(s2, B, H, T, FT_SKEW_QK, FT16_QK);
        if (lanes == 16)
            return s2.groups ? "ft_kernel (per-head table, 16 lanes per head, 16-wave workgroups, uneven segments)"
                             : "ft_kernel (per-head table, 16 lanes per head, 16-wave workgroups)";
        return s2.groups ? "ft_kernel (per-head table, 16-wave workgroups, uneven segments)"
                         : "ft_kernel (per-head table, 16-wave workgroups)";
    }
    if (D == 128) {
        const long units = padded_units<32>(B * H, seg.nseg);
        if (units / 2 <= n_simd())
            return "kernel<128,2,256> (shared table, two channels per lane)";
        return units * 32 >= 1024L * cus() ? "kernel<128,4,1024> (shared table)" : "kernel<128,4,256> (shared table)";
    }
    return D == 256 ? "kernel<256,4,*> (shared table)" : "kernel<512,8,256> (shared table)";
}

// act_bf16: q, k_new / v_new and the output are bfloat16 (only adkv_decode_step asks for it)
static int forward_qk_impl(const void *q, void *k_cache, const void *k_new, void *logits,
                           const void *zp, const void *sc, const void *alpha, const void *beta,
                           const void *tgt,
                           int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                           void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                           void *stream, int act_bf16)
{
    if (ld != 0 && ld < (int64_t)T + 1)
        return ADKV_E_SHAPE;
    if (!q || !k_cache || !k_new || !logits || !zp || !sc || !alpha || !beta || !tgt)
        return ADKV_E_NULL;
    if (bits != 2 && bits != 4)
        return ADKV_E_UNSUPPORTED;
    int rc = check_common(B, H, T, D, n_super_cap);
    if (rc)
        return rc;
    if (Hq <= 0 || Hq % H)
        return ADKV_E_SHAPE;
    const int GQ = Hq / H;
    if ((GQ > 1 || bits != 4) && D != 128)
        return ADKV_E_UNSUPPORTED;
    if (T / (32 / bits) >= n_super_cap)
        return ADKV_E_CAPACITY;
    if (((uintptr_t)k_cache & 15) || ((uintptr_t)q & 7) || ((uintptr_t)k_new & 3))
        return ADKV_E_ALIGN;
    if ((rc = check_ckpt(ckpt, n_ckpt_cap, ckpt_interval, bits)))
        return rc;
    const int BH = B * H;
    hipStream_t st = (hipStream_t)stream;
    Seg seg = plan_segments(ckpt, n_ckpt_cap, ckpt_interval, BH, T, D);
    seg.act_bf16 = act_bf16;
    if (ld)
        seg.row_pitch = ld;
    if (D == 128 && (GQ > 1 || bits != 4 || mfma_for_mha())) {
        if (GQ <= 4) // eight query heads per KV head may fall back to 8-wave workgroups
            plan_uneven(seg, T, padded_units<32>(BH, seg.nseg) * 32, GQA_SKEW_QK);
        ADKV_DISPATCH_GQ(qk_gqa_kernel, true, (const h1 *)q, (uint4 *)k_cache, (const h1 *)k_new,
                         (h1 *)logits, (const h1 *)zp, (const h1 *)sc, (const h1 *)alpha,
                         (const h1 *)beta, (const h1 *)tgt, BH, H, T, n_super_cap, (h1 *)state_out,
                         seg);
        return check_launch();
    }
    if (use_head_table(B, H, GQ, bits, D, seg)) {
        const int lanes = plan_ft(seg, B, H, T, FT_SKEW_QK, FT16_QK);
        const auto kernel = lanes == 16 ? qk_ft_kernel<16> : qk_ft_kernel<32>;
        hipLaunchKernelGGL(kernel, dim3((unsigned)(H * seg.phys_per_head)), dim3(FT_BLK), 0, st,
                           (const h1 *)q, (uint4 *)k_cache, (const h1 *)k_new, (h1 *)logits,
                           (const h1 *)zp, (const h1 *)sc, (const h1 *)alpha, (const h1 *)beta,
                           (const h1 *)tgt, B, H, T, n_super_cap, (h1 *)state_out, seg);
        return check_launch();
    }
    ADKV_DISPATCH_D(qk_kernel, (const h1 *)q, (uint4 *)k_cache, (const h1 *)k_new, (h1 *)logits,
                    (const h1 *)zp, (const h1 *)sc, (const h1 *)alpha, (const h1 *)beta,
                    (const h1 *)tgt, BH, H, T, n_super_cap, (h1 *)state_out, seg);
    return check_launch();
}

extern "C" {

const char *adkv_decode_kernel_name(int B, int Hq, int H, int T, int D, int bits, int n_ckpt_cap,
                                    int ckpt_interval)
{
    return decode_kernel_name(B, Hq, H, T, D, bits, n_ckpt_cap, ckpt_interval);
}

int adkv_decode_segments(int B, int Hq, int H, int T, int D, int bits, int n_ckpt_cap,
                         int ckpt_interval, int *bounds, int max_bounds, int *info)
{
    if (B <= 0 || H <= 0 || Hq <= 0 || Hq % H || T < 0 || (D != 128 && D != 256 && D != 512) ||
        (bits != 2 && bits != 4))
        return -1;
    const int GQ = Hq / H;
    if ((GQ > 1 || bits != 4) && D != 128)
        return -1;
    int dummy = 0;
    Seg seg = plan_segments(n_ckpt_cap > 0 && ckpt_interval > 0 ? &dummy : nullptr, n_ckpt_cap,
                            ckpt_interval, B * H, T, D);
    const bool matrix_cores = D == 128 && (GQ > 1 || bits != 4 || mfma_for_mha());
    const bool head_table = !matrix_cores && use_head_table(B, H, GQ, bits, D, seg);
    long wgs = 0;
    int virt = 1;
    if (matrix_cores && GQ <= 4)
        plan_uneven(seg, T, padded_units<32>(B * H, seg.nseg) * 32, GQA_SKEW_QK);
    if (head_table) {
        const int lanes = plan_ft(seg, B, H, T, FT_SKEW_QK, FT16_QK);
        const int W = ft_wgs_per_head(B, seg.nseg, 64 / lanes);
        wgs = (long)H * seg.phys_per_head;
        virt = (W + seg.phys_per_head - 1) / seg.phys_per_head;
    }
    if (bounds != nullptr && max_bounds > seg.nseg) {
        for (int s = 0; s < seg.nseg; s++)
            bounds[s] = seg.groups ? uneven_cut(s, seg.groups, seg.intervals, seg.skew) * seg.ckpt_interval
                                   : s * seg.seg_tokens; // in time order
        bounds[seg.nseg] = T;
    }
    if (info != nullptr) {
        info[0] = (int)wgs; // 0: not a per-head-table launch (workgroup count follows the kernel's shape)
        info[1] = virt;
    }
    return seg.nseg;
}

int adkv_forward_qk_gqa(const void *q, void *k_cache, const void *k_new, void *logits,
                        const void *zp, const void *sc, const void *alpha, const void *beta,
                        const void *tgt,
                        int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                        void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                        void *stream)
{
    return forward_qk_impl(q, k_cache, k_new, logits, zp, sc, alpha, beta, tgt, B, Hq, H, T, D,
                           n_super_cap, bits, ld, state_out, ckpt, n_ckpt_cap, ckpt_interval, stream, 0);
}

int adkv_forward_qk_ex(const void *q, void *k_cache, const void *k_new, void *logits,
                       const void *zp, const void *sc, const void *alpha, const void *beta,
                       const void *tgt,
                       int B, int H, int T, int D, int n_super_cap,
                       void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                       void *stream)
{
    return adkv_forward_qk_gqa(q, k_cache, k_new, logits, zp, sc, alpha, beta, tgt, B, H, H, T, D,
                               n_super_cap, 4, 0, state_out, ckpt, n_ckpt_cap, ckpt_interval, stream);
}

int adkv_forward_qk(const void *q, void *k_cache, const void *k_new, void *logits,
                    const void *zp, const void *sc, const void *alpha, const void *beta,
                    const void *tgt,
                    int B, int H, int T, int D, int n_super_cap,
                    float, float, void *state_out, void *stream)
{
    return adkv_forward_qk_ex(q, k_cache, k_new, logits, zp, sc, alpha, beta, tgt, B, H, T, D,
                              n_super_cap, state_out, nullptr, 0, 0, stream);
}

int64_t adkv_forward_ov_workspace_bytes(int B, int H, int T, int D, int n_ckpt_cap, int ckpt_interval)
{
    if (B <= 0 || H <= 0 || T < 0 || n_ckpt_cap <= 0 || ckpt_interval <= 0)
        return 0;
    int dummy = 0;
    const int nseg = max_plan_segments(&dummy, n_ckpt_cap, ckpt_interval, B, H, T, D);
    return nseg > 1 ? (int64_t)nseg * B * H * D * 4 : 0;
}

} // extern "C"

static int forward_ov_impl(const void *attn, void *v_cache, const void *v_new, void *out,
                           const void *zp, const void *sc, const void *alpha, const void *beta,
                           const void *tgt,
                           int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                           void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                           void *workspace, int64_t workspace_bytes, void *stream, int act_bf16)
{
    if (ld != 0 && ld < (int64_t)T + 1)
        return ADKV_E_SHAPE;
    if (!attn || !v_cache || !v_new || !out || !zp || !sc || !alpha || !beta || !tgt)
        return ADKV_E_NULL;
    if (bits != 2 && bits != 4)
        return ADKV_E_UNSUPPORTED;
    int rc = check_common(B, H, T, D, n_super_cap);
    if (rc)
        return rc;
    if (Hq <= 0 || Hq % H)
        return ADKV_E_SHAPE;
    const int GQ = Hq / H;
    if ((GQ > 1 || bits != 4) && D != 128)
        return ADKV_E_UNSUPPORTED;
    if (T / (32 / bits) >= n_super_cap)
        return ADKV_E_CAPACITY;
    if (((uintptr_t)v_cache & 15) || ((uintptr_t)out & 3) || ((uintptr_t)v_new & 3))
        return ADKV_E_ALIGN;
    if ((rc = check_ckpt(ckpt, n_ckpt_cap, ckpt_interval, bits)))
        return rc;
    const int BH = B * H;
    hipStream_t st = (hipStream_t)stream;
    Seg seg = plan_segments(ckpt, n_ckpt_cap, ckpt_interval, BH, T, D);
    seg.act_bf16 = act_bf16;
    if (ld)
        seg.row_pitch = ld;
    const bool matrix_cores = D == 128 && (GQ > 1 || bits != 4 || mfma_for_mha());
    const bool head_table = !matrix_cores && use_head_table(B, H, GQ, bits, D, seg);
    const int ft_lanes = head_table ? plan_ft_ov(seg, B, H, T) : 32;
    // per-head table, two or four segments, one virtual workgroup per workgroup: the waves of one
    // sequence pair sit in the same workgroup (interleave_segment) and add their partial outputs
    // there; no second launch and nothing in the workspace
    seg.combine = (head_table && ft_ov_combines(seg, B, ft_lanes)) ? 1 : 0;
    if (seg.nseg > 1 && !seg.combine) {
        if (!workspace || workspace_bytes < (int64_t)seg.nseg * BH * GQ * D * 4)
            return ADKV_E_WORKSPACE;
        if ((uintptr_t)workspace & 15)
            return ADKV_E_ALIGN;
    }
    if (matrix_cores) {
        if (GQ <= 4)
            plan_uneven(seg, T, padded_units<32>(BH, seg.nseg) * 32, GQA_SKEW_OV);
        ADKV_DISPATCH_GQ(ov_gqa_kernel, false, (const h1 *)attn, (uint4 *)v_cache, (const h1 *)v_new,
                         (h1 *)out, (float *)workspace, (const h1 *)zp, (const h1 *)sc,
                         (const h1 *)alpha, (const h1 *)beta, (const h1 *)tgt, BH, H, T, n_super_cap,
                         (h1 *)state_out, seg);
    } else if (head_table) {
        const auto kernel = ft_lanes == 16 ? ov_ft_kernel<16> : ov_ft_kernel<32>;
        hipLaunchKernelGGL(kernel, dim3((unsigned)(H * ft_wgs_per_head(B, seg.nseg, 64 / ft_lanes))),
                           dim3(FT_BLK), 0, st, (const h1 *)attn, (uint4 *)v_cache, (const h1 *)v_new, (h1 *)out,
                           (float *)workspace, (const h1 *)zp, (const h1 *)sc, (const h1 *)alpha,
                           (const h1 *)beta, (const h1 *)tgt, B, H, T, n_super_cap, (h1 *)state_out, seg);
    } else {
        ADKV_DISPATCH_D(ov_kernel, (const h1 *)attn, (uint4 *)v_cache, (const h1 *)v_new, (h1 *)out,
                        (float *)workspace, (const h1 *)zp, (const h1 *)sc, (const h1 *)alpha,
                        (const h1 *)beta, (const h1 *)tgt, BH, H, T, n_super_cap, (h1 *)state_out,
                        seg);
    }
    if ((rc = check_launch()))
        return rc;
    if (seg.nseg > 1 && !seg.combine) {
        const long n = (long)BH * GQ * D;
        if (seg.nseg > 8)
            hipLaunchKernelGGL(ov_finalize_wide_kernel, dim3((unsigned)((n + 63) / 64)), dim3(256), 0, st,
                               (const float *)workspace, (h1 *)out, n, seg.nseg, seg.act_bf16);
        else
            hipLaunchKernelGGL(ov_finalize_kernel, dim3((unsigned)((n + 511) / 512)), dim3(256), 0, st,
                               (const float *)workspace, (h1 *)out, n, seg.nseg, seg.act_bf16);
        rc = check_launch();
    }
    return rc;
}

// ---------------------------------------------------------------------------------------------
// Static scratch for callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc): the fp32 partial sums of a segmented forward_ov live in a
// device array that is part of the code object, one copy per GPU, held until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; the device address it
// yields (a different one on every GPU) is what launches are given.
// ---------------------------------------------------------------------------------------------
constexpr int64_t STATIC_SCRATCH_FLOATS = (int64_t)8 << 20; // 32 MiB
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
static std::atomic<float *> g_scratch_ptr[MAX_DEVICES];
static std::mutex g_scratch_mu;

// Device address of `scratch` on the current device, resolved once per device.
static int static_scratch(float **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return ADKV_E_DEVICE;
    }
    if (dev < 0 || dev >= MAX_DEVICES)
        return ADKV_E_UNSUPPORTED;
    float *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        std::lock_guard<std::mutex> lock(g_scratch_mu);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (p == nullptr) {
            void *addr = nullptr;
            e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
            if (e != hipSuccess || addr == nullptr) {
                g_last_hip_error = (int)e;
                return ADKV_E_DEVICE;
            }
            p = (float *)addr;
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return ADKV_OK;
}

extern "C" {

int64_t adkv_static_scratch_bytes(void) { return STATIC_SCRATCH_FLOATS * 4; }

int adkv_init(void)
{
    float *p = nullptr;
    return static_scratch(&p);
}

int adkv_forward_ov_noalloc(const void *attn, void *v_cache, const void *v_new, void *out,
                            const void *zp, const void *sc, const void *alpha, const void *beta,
                            const void *tgt,
                            int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                            void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                            void *stream)
{
    // what the segment plan of this launch needs, priced before anything touches the device
    // (nothing when the kernel adds its two or four segments inside the workgroup)
    int64_t need = 0;
    if (ckpt != nullptr && B > 0 && H > 0 && Hq > 0 && Hq % H == 0 && T >= 0 && n_ckpt_cap > 0 &&
        ckpt_interval > 0 && (D == 128 || D == 256 || D == 512)) {
        int dummy = 0;
        Seg seg = plan_segments(&dummy, n_ckpt_cap, ckpt_interval, B * H, T, D);
        const int GQ = Hq / H;
        const bool matrix_cores = D == 128 && (GQ > 1 || bits != 4 || mfma_for_mha());
        bool in_workgroup = false;
        if (!matrix_cores && use_head_table(B, H, GQ, bits, D, seg)) {
            const int lanes = plan_ft_ov(seg, B, H, T);
            in_workgroup = ft_ov_combines(seg, B, lanes);
        }
        if (seg.nseg > 1 && !in_workgroup)
            need = (int64_t)seg.nseg * B * Hq * D * 4;
    }
    if (need > adkv_static_scratch_bytes())
        return ADKV_E_SCRATCH_LIMIT;
    float *ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc)
        return rc;
    // Every partial a launch reads was written by the same launch (each segment stores its whole
    // [B*Hq, D] slice before the summing kernel runs), so nothing has to start at zero.
    return forward_ov_impl(attn, v_cache, v_new, out, zp, sc, alpha, beta, tgt, B, Hq, H, T, D,
                           n_super_cap, bits, ld, state_out, ckpt, n_ckpt_cap, ckpt_interval, ws,
                           adkv_static_scratch_bytes(), stream, 0);
}

int adkv_forward_ov_gqa(const void *attn, void *v_cache, const void *v_new, void *out,
                        const void *zp, const void *sc, const void *alpha, const void *beta,
                        const void *tgt,
                        int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int64_t ld,
                        void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                        void *workspace, int64_t workspace_bytes, void *stream)
{
    return forward_ov_impl(attn, v_cache, v_new, out, zp, sc, alpha, beta, tgt, B, Hq, H, T, D,
                           n_super_cap, bits, ld, state_out, ckpt, n_ckpt_cap, ckpt_interval, workspace,
                           workspace_bytes, stream, 0);
}

int adkv_forward_ov_ex(const void *attn, void *v_cache, const void *v_new, void *out,
                       const void *zp, const void *sc, const void *alpha, const void *beta,
                       const void *tgt,
                       int B, int H, int T, int D, int n_super_cap,
                       void *state_out, void *ckpt, int n_ckpt_cap, int ckpt_interval,
                       void *workspace, int64_t workspace_bytes, void *stream)
{
    return adkv_forward_ov_gqa(attn, v_cache, v_new, out, zp, sc, alpha, beta, tgt, B, H, H, T, D,
                               n_super_cap, 4, 0, state_out, ckpt, n_ckpt_cap, ckpt_interval, workspace,
                               workspace_bytes, stream);
}

int adkv_forward_ov(const void *attn, void *v_cache, const void *v_new, void *out,
                    const void *zp, const void *sc, const void *alpha, const void *beta,
                    const void *tgt,
                    int B, int H, int T, int D, int n_super_cap,
                    float, float, void *state_out, void *stream)
{
    return adkv_forward_ov_ex(attn, v_cache, v_new, out, zp, sc, alpha, beta, tgt, B, H, T, D,
                              n_super_cap, state_out, nullptr, 0, 0, nullptr, 0, stream);
}

int64_t adkv_softmax_workspace_bytes(int rows, int n)
{
    if (rows <= 0 || n <= SM_ROW_MAX)
        return 0;
    return (int64_t)rows * ((n + SM_CHUNK - 1) / SM_CHUNK) * 8;
}

int64_t adkv_row_pitch(int n)
{
    // smallest odd multiple of 128 elements (256 bytes) that holds n: consecutive rows then start
    // in different memory channels even when n itself is a power of two
    int64_t k = ((int64_t)n + 127) / 128;
    if (!(k & 1))
        k++;
    return k * 128;
}

int adkv_softmax_ex(const void *logits, void *weights, const void *mask,
                    int rows, int n, int64_t ld, int rows_per_mask_row, float scaling,
                    void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!logits || !weights)
        return ADKV_E_NULL;
    if (rows <= 0 || n <= 0 || (mask && rows_per_mask_row <= 0) || (ld != 0 && ld < n))
        return ADKV_E_SHAPE;
    if (ld == 0)
        ld = n;
    if (n <= 64 * SM_VEC * 4) {
        // short rows: a wave per row, the row in 8, 16 or 32 registers per lane (longer rows were
        // measured slower this way: 27 us against 22 us for 4096 rows of 4097 elements)
        const dim3 grid((unsigned)((rows + SM_BLOCK / 64 - 1) / (SM_BLOCK / 64)));
#define ADKV_SM_WAVE(NVW)                                                                           \
    hipLaunchKernelGGL(softmax_wave_kernel<NVW>, grid, dim3(SM_BLOCK), 0, (hipStream_t)stream,      \
                       (const h1 *)logits, (h1 *)weights, (const float *)mask, rows, n, (long)ld,   \
                       mask ? rows_per_mask_row : 1, scaling)
        if (n <= 64 * SM_VEC)
            ADKV_SM_WAVE(1);
        else if (n <= 64 * SM_VEC * 2)
            ADKV_SM_WAVE(2);
        else
            ADKV_SM_WAVE(4);
#undef ADKV_SM_WAVE
        return check_launch();
    }
    const int reg_nv = (n + 1024 * SM_VEC - 1) / (1024 * SM_VEC); // 16-byte vectors per thread
    if (n > SM_ROW_MAX && !mask && n <= SM_REG_MAX && (rows >= SM_REG_MIN_ROWS || reg_nv <= 9) &&
        scaling != 0.0f && scaling == scaling) {
        // long unmasked rows stay in registers, unless they are few and very long (32 rows of
        // 131 073: 14.6 us cut into chunks, 19.8 us this way; 128 rows: 28.1 and 24.8; 512 rows:
        // 74.8 and 56.7; 64 rows of 32 769: 11.4 and 9.4; 4096 rows of 24 577: 148 and 80)
#define ADKV_SM_REG(NV)                                                                             \
    case NV:                                                                                        \
        hipLaunchKernelGGL(softmax_regrow_kernel<NV>, dim3((unsigned)rows), dim3(1024), 0,          \
                           (hipStream_t)stream, (const h1 *)logits, (h1 *)weights, n, (long)ld,     \
                           scaling);                                                                \
        break
        switch (reg_nv) {
            ADKV_SM_REG(4); ADKV_SM_REG(5); ADKV_SM_REG(6); ADKV_SM_REG(7); ADKV_SM_REG(8);
            ADKV_SM_REG(9); ADKV_SM_REG(10); ADKV_SM_REG(11); ADKV_SM_REG(12); ADKV_SM_REG(13);
            ADKV_SM_REG(14); ADKV_SM_REG(15); ADKV_SM_REG(16);
        default:
            ADKV_SM_REG(17);
        }
#undef ADKV_SM_REG
        return check_launch();
    }
    const int64_t need = adkv_softmax_workspace_bytes(rows, n);
    if (need == 0 || !workspace || rows > 65535) {
        // one workgroup per row, sized so that the row stays in its registers (read once, written
        // once); rows beyond 24576 elements without a workspace are read three times
#define ADKV_SM_ROW(NT, NV)                                                                         \
    hipLaunchKernelGGL((softmax_kernel<NT, NV>), dim3((unsigned)rows), dim3(NT), 0,                 \
                       (hipStream_t)stream, (const h1 *)logits, (h1 *)weights, (const float *)mask, \
                       n, (long)ld, mask ? rows_per_mask_row : 1, scaling)
        // (threads, 16-byte vectors per thread) per row length, measured on 4096 rows: 4097 elements
        // 18.4 us with 256 x 3 and 16.7 with 320 x 2; 8192: 35.5 with 512 x 3, 24.3 with 512 x 2;
        // 10000: 36.9 with 512 x 3, 33.0 with 256 x 6; 16384: 76.5 with 1024 x 3, 46.9 with 1024 x 2;
        // 2048 rows of 24576: 42.1 with 1024 x 3, 37.4 with 512 x 6
        if (n <= 5120)
            ADKV_SM_ROW(320, 2);
        else if (n <= SM_CHUNK || n > SM_ROW_MAX)
            ADKV_SM_ROW(SM_BLOCK, SM_NV);
        else if (n <= 8192)
            ADKV_SM_ROW(512, 2);
        else if (n <= 12288)
            ADKV_SM_ROW(256, 6);
        else if (n <= 16384)
            ADKV_SM_ROW(1024, 2);
        else
            ADKV_SM_ROW(512, 6);
#undef ADKV_SM_ROW
        return check_launch();
    }
    if (workspace_bytes < need)
        return ADKV_E_WORKSPACE;
    if ((uintptr_t)workspace & 7)
        return ADKV_E_ALIGN;
    const int nchunk = (n + SM_CHUNK - 1) / SM_CHUNK;
    const dim3 grid((unsigned)nchunk, (unsigned)rows);
    if (nchunk >= 8 && !mask) {
        // long rows: four chunks per workgroup in the first pass
        const dim3 grid4((unsigned)((nchunk + 3) / 4), (unsigned)rows);
        hipLaunchKernelGGL(softmax_part_kernel<4>, grid4, dim3(SM_BLOCK), 0, (hipStream_t)stream,
                           (const h1 *)logits, (const float *)mask, (float2 *)workspace, n, (long)ld, nchunk,
                           1, scaling);
    } else {
        hipLaunchKernelGGL(softmax_part_kernel<1>, grid, dim3(SM_BLOCK), 0, (hipStream_t)stream,
                           (const h1 *)logits, (const float *)mask, (float2 *)workspace, n, (long)ld, nchunk,
                           mask ? rows_per_mask_row : 1, scaling);
    }
    hipLaunchKernelGGL(softmax_norm_kernel, grid, dim3(SM_BLOCK), 0, (hipStream_t)stream,
                       (const h1 *)logits, (h1 *)weights, (const float *)mask,
                       (const float2 *)workspace, n, (long)ld, nchunk, mask ? rows_per_mask_row : 1,
                       scaling);
    return check_launch();
}

int adkv_softmax(const void *logits, void *weights, const void *mask,
                 int rows, int n, int rows_per_mask_row, float scaling, void *stream)
{
    return adkv_softmax_ex(logits, weights, mask, rows, n, 0, rows_per_mask_row, scaling, nullptr, 0,
                           stream);
}

int adkv_rope_qk(const void *q, const void *k, const void *cos, const void *sin, void *q_out, void *k_out,
                 int B, int Hq, int H, int T, int D,
                 int64_t q_sb, int64_t q_sh, int64_t q_st, int64_t k_sb, int64_t k_sh, int64_t k_st,
                 int64_t cs_sb, int64_t cs_st, int bf16, void *stream)
{
    if (!q || !k || !cos || !sin || !q_out || !k_out)
        return ADKV_E_NULL;
    if (B <= 0 || Hq <= 0 || H <= 0 || T <= 0 || D <= 0 || (D & 3))
        return ADKV_E_SHAPE;
    // 4-byte accesses: every base and every stride a multiple of two elements
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)cos | (uintptr_t)sin | (uintptr_t)q_out | (uintptr_t)k_out) & 3)
        return ADKV_E_ALIGN;
    if ((q_sb | q_sh | q_st | k_sb | k_sh | k_st | cs_sb | cs_st) & 1)
        return ADKV_E_ALIGN;
    if ((long)(Hq + H) * (D >> 2) > (long)INT32_MAX)
        return ADKV_E_SHAPE;
    const RopeSide qs = {(const uint16_t *)q, (uint16_t *)q_out, (long)q_sb, (long)q_sh, (long)q_st, Hq};
    const RopeSide ks = {(const uint16_t *)k, (uint16_t *)k_out, (long)k_sb, (long)k_sh, (long)k_st, H};
    const unsigned gx = (unsigned)(((long)(Hq + H) * (D >> 2) + 255) / 256);
    constexpr int GMAX = 65535; // grid limit of the token and batch axes: longer ones take several launches
    for (int b0 = 0; b0 < B; b0 += GMAX)
        for (int t0 = 0; t0 < T; t0 += GMAX) {
            const dim3 grid(gx, (unsigned)min(T - t0, GMAX), (unsigned)min(B - b0, GMAX));
            if (bf16)
                hipLaunchKernelGGL(rope_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, qs, ks,
                                   (const uint16_t *)cos, (const uint16_t *)sin, (long)cs_sb, (long)cs_st, T, D,
                                   t0, b0);
            else
                hipLaunchKernelGGL(rope_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, qs, ks,
                                   (const uint16_t *)cos, (const uint16_t *)sin, (long)cs_sb, (long)cs_st, T, D,
                                   t0, b0);
        }
    return check_launch();
}

static int64_t pad256(int64_t n) { return (n + 255) & ~(int64_t)255; }

// Events adkv_decode_step records around its stages in this thread (a measurement hook).
static thread_local hipEvent_t g_stage_events[4] = {nullptr, nullptr, nullptr, nullptr};

void adkv_set_stage_events(void *const *events)
{
    for (int i = 0; i < 4; i++)
        g_stage_events[i] = events ? (hipEvent_t)events[i] : nullptr;
}

static int stage_mark(int i, void *stream)
{
    if (g_stage_events[i] == nullptr)
        return ADKV_OK;
    const hipError_t e = hipEventRecord(g_stage_events[i], (hipStream_t)stream);
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return ADKV_E_LAUNCH;
    }
    return ADKV_OK;
}

int64_t adkv_forward_ov_gqa_workspace_bytes(int B, int Hq, int H, int T, int D, int n_ckpt_cap,
                                            int ckpt_interval)
{
    if (H <= 0 || Hq <= 0 || Hq % H)
        return 0;
    return adkv_forward_ov_workspace_bytes(B, H, T, D, n_ckpt_cap, ckpt_interval) * (Hq / H);
}

int64_t adkv_decode_step_workspace_bytes(int B, int Hq, int H, int T, int D, int n_ckpt_cap,
                                          int ckpt_interval)
{
    if (B <= 0 || H <= 0 || Hq <= 0 || T < 0)
        return 0;
    const int64_t mat = pad256((int64_t)B * Hq * adkv_row_pitch(T + 1) * 2);
    return 2 * mat + pad256(adkv_softmax_workspace_bytes(B * Hq, T + 1)) +
           adkv_forward_ov_gqa_workspace_bytes(B, Hq, H, T, D, n_ckpt_cap, ckpt_interval);
}

int adkv_decode_step(const void *q, void *k_cache, void *v_cache, const void *k_new, const void *v_new,
                      const void *const *k_params, const void *const *v_params,
                      const void *mask, int rows_per_mask_row, float scaling,
                      void *out, void *weights_out, int64_t weights_ld,
                      int B, int Hq, int H, int T, int D, int n_super_cap, int bits, int act_dtype,
                      void *k_ckpt, void *v_ckpt, int n_ckpt_cap, int ckpt_interval,
                      void *workspace, int64_t workspace_bytes, void *stream)
{
    if (!k_params || !v_params || !workspace)
        return workspace ? ADKV_E_NULL : ADKV_E_WORKSPACE;
    if (act_dtype != ADKV_DT_F16 && act_dtype != ADKV_DT_BF16)
        return ADKV_E_UNSUPPORTED;
    const int act_bf16 = act_dtype == ADKV_DT_BF16;
    if (B <= 0 || H <= 0 || Hq <= 0 || Hq % H || T < 0)
        return ADKV_E_SHAPE;
    if (workspace_bytes < adkv_decode_step_workspace_bytes(B, Hq, H, T, D, n_ckpt_cap, ckpt_interval))
        return ADKV_E_WORKSPACE;
    if ((uintptr_t)workspace & 255)
        return ADKV_E_ALIGN;
    // The logits live in the workspace with padded rows.  The weights do too unless the caller
    // wants them; the softmax writes them with the logits' pitch, so a caller-provided matrix
    // must use that pitch as well (weights_ld == adkv_row_pitch(T + 1)) or be avoided.
    const int64_t ld = adkv_row_pitch(T + 1);
    if (weights_out && weights_ld != ld)
        return ADKV_E_SHAPE;
    const int64_t mat = pad256((int64_t)B * Hq * ld * 2);
    char *ws = (char *)workspace;
    void *logits = ws;
    void *weights = weights_out ? weights_out : (void *)(ws + mat);
    int rc = stage_mark(0, stream);
    if (rc)
        return rc;
    {
        // one launch for the whole step where the plans allow it (decode_ft_kernel)
        Seg ka, va;
        const int lanes = mask ? 0 : fused_step_plan(ka, va, B, Hq, H, T, D, bits, k_ckpt, v_ckpt, n_ckpt_cap, ckpt_interval);
        if (lanes) {
            if ((rc = check_common(B, H, T, D, n_super_cap)))
                return rc;
            if (T / 8 >= n_super_cap)
                return ADKV_E_CAPACITY;
            if (!q || !k_cache || !v_cache || !k_new || !v_new || !out)
                return ADKV_E_NULL;
            for (int i = 0; i < 5; i++)
                if (!k_params[i] || !v_params[i])
                    return ADKV_E_NULL;
            if (((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15) || ((uintptr_t)q & 7) || ((uintptr_t)k_new & 3) ||
                ((uintptr_t)v_new & 3) || ((uintptr_t)out & 3) || ((uintptr_t)weights & 1))
                return ADKV_E_ALIGN;
            if ((rc = check_ckpt(k_ckpt, n_ckpt_cap, ckpt_interval, bits)) || (rc = check_ckpt(v_ckpt, n_ckpt_cap, ckpt_interval, bits)))
                return rc;
            ka.row_pitch = va.row_pitch = ld;
            ka.act_bf16 = va.act_bf16 = act_bf16;
            va.combine = 1;
            const FtParams kp = {(const h1 *)k_params[0], (const h1 *)k_params[1], (const h1 *)k_params[2],
                                 (const h1 *)k_params[3], (const h1 *)k_params[4]};
            const FtParams vp = {(const h1 *)v_params[0], (const h1 *)v_params[1], (const h1 *)v_params[2],
                                 (const h1 *)v_params[3], (const h1 *)v_params[4]};
            const auto kernel = lanes == 16 ? decode_ft_kernel<16> : decode_ft_kernel<32>;
            hipLaunchKernelGGL(kernel, dim3((unsigned)(H * ka.phys_per_head)), dim3(FT_BLK), 0, (hipStream_t)stream,
                               (const h1 *)q, (uint4 *)k_cache, (const h1 *)k_new, (uint4 *)v_cache, (const h1 *)v_new,
                               (h1 *)logits, (h1 *)weights, (h1 *)out, kp, vp, B, H, T, n_super_cap, scaling, ka, va);
            if ((rc = check_launch()))
                return rc;
            for (int i = 1; i <= 3; i++)
                if ((rc = stage_mark(i, stream)))
                    return rc;
            return ADKV_OK;
        }
    }
    rc = forward_qk_impl(q, k_cache, k_new, logits, k_params[0], k_params[1], k_params[2],
                         k_params[3], k_params[4], B, Hq, H, T, D, n_super_cap, bits, ld,
                         nullptr, k_ckpt, n_ckpt_cap, ckpt_interval, stream, act_bf16);
    if (rc || (rc = stage_mark(1, stream)))
        return rc;
    const int64_t smb = pad256(adkv_softmax_workspace_bytes(B * Hq, T + 1));
    rc = adkv_softmax_ex(logits, weights, mask, B * Hq, T + 1, ld, rows_per_mask_row, scaling,
                         smb ? ws + 2 * mat : nullptr, smb, stream);
    if (rc || (rc = stage_mark(2, stream)))
        return rc;
    rc = forward_ov_impl(weights, v_cache, v_new, out, v_params[0], v_params[1], v_params[2],
                         v_params[3], v_params[4], B, Hq, H, T, D, n_super_cap, bits, ld,
                         nullptr, v_ckpt, n_ckpt_cap, ckpt_interval, ws + 2 * mat + smb,
                         workspace_bytes - 2 * mat - smb, stream, act_bf16);
    if (rc)
        return rc;
    return stage_mark(3, stream);
}

} // extern "C"
