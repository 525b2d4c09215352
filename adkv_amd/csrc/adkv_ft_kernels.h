// Vector decode kernels with a PER-HEAD lookup table (head dim 128, 4-bit codes, one query head
// per KV head, big launches).  Included by adkv_kernels.hip after the shared device helpers.
//
// The replay is bound by vector-instruction issue, so every instruction per (channel pair, token)
// counts.  The scale multiplier f = r16(beta*|q| + omt) (gemv.cu:163) depends only on the code and
// on two per-channel constants, never on the state: it can come out of a table.  The shared table
// of qk_kernel / ov_kernel returns (q, |q|) for a code byte and leaves the fused multiply-add to
// the lane; here the table is built per KV head and returns (q, f) for (code byte, channel pair),
// which removes one of the six packed instructions per pair and token.
//
//   * 256 code bytes x 64 channel pairs x 8 bytes = 128 KB of the CU's 160 KB of LDS, as two
//     64 KB tables; with a head over 32 lanes (four channels per lane) entry (pair j, byte b, lane)
//     sits at j*64 KB + b*256 + lane*8, so the 32 lanes of a head read 32 distinct 8-byte slots of
//     one 256-byte row whatever their codes are, and the address is still ONE v_perm_b32:
//     [0, table, code byte, lane*8].
//   * A head over 16 lanes (eight channels per lane, two passes of four over every supergroup,
//     four sequences per wave) pays the logit reduction, the store and the loop overhead once per
//     eight channels: 7 % fewer instructions in forward_qk, 4 % in forward_ov.  Its table is
//     [pass][byte][pair j][lane]: the 16 lanes of a head on the 16 slots of one half row.  The
//     launchers take it for big launches whose segments stay long (plan_ft).
//   * All units of a workgroup must belong to the SAME head: units are ordered head-major (for one
//     head: a wave per two or four sequences and segment, consecutive quads of waves on different
//     segments, interleave_segment), and every head's run of waves is padded to whole 16-wave
//     workgroups.
//   * No LDS is left for the logit transpose of qk_kernel, and none is needed: the 8 per-lane
//     partials are reduced and scattered over the head's lanes with bank-masked DPP adds (8 + 4
//     instructions), then one row swap and two quad permutes (32 lanes) or two selects and two
//     quad permutes (16 lanes).
#pragma once

namespace adkv {

constexpr int FT_BLK = 1024;
constexpr int FT_WAVES = FT_BLK / 64;
constexpr int FT_TABLE_WORDS64 = 2 * LUT_ENTRIES * 32; // uint2 elements: 2 x 64 KB

// A head is spread over LPH lanes of a wave: 32 lanes with four channels each, or 16 lanes that
// make two passes of four channels (channels 4*lane.. in the first, 64 + 4*lane.. in the second)
// over every supergroup.  A wave then holds upw = 64 / LPH sequences of one segment.
// host and device: how the (head, segment, sequence) units of a launch are laid out
__host__ __device__ inline int ft_waves_per_seg(int B, int upw) { return (B + upw - 1) / upw; }
__host__ __device__ inline int ft_wgs_per_head(int B, int nseg, int upw)
{
    return (nseg * pad4(ft_waves_per_seg(B, upw)) + FT_WAVES - 1) / FT_WAVES;
}

template <int LPH>
struct FtUnit {
    int seg, bx, lh, c0;
    bool active, wave_active;
    // h: KV head; vw: virtual workgroup within the head (16 waves' worth of the head's units)
    __device__ __forceinline__ FtUnit(int B, int H, int nseg, int h, int vw)
    {
        constexpr int UPW = 64 / LPH;
        const int wps = ft_waves_per_seg(B, UPW);
        const int w = __builtin_amdgcn_readfirstlane(vw * FT_WAVES + (int)(threadIdx.x >> 6)); // wave within the head
        int sg, wis;
        interleave_segment(w, nseg, sg, wis);
        const int lane = threadIdx.x & 63;
        const int b = wis * UPW + lane / LPH;
        lh = lane % LPH;
        c0 = lh * 4;
        wave_active = wis < wps;
        active = wave_active && b < B;
        seg = sg;
        bx = (b < B ? b : B - 1) * H + h;
    }
};

// 32 lanes: table[j][code byte][lane] = (q pair, f pair) for channels 4*lane + 2j, 4*lane + 2j + 1
// of head h.  16 lanes: table[pass][code byte][j][lane] for channels 64*pass + 4*lane + 2j, + 1: the
// 16 lanes of a head read the 16 slots of one half of a 256-byte row, again whatever their codes.
template <int LPH>
__device__ __forceinline__ void ft_fill(uint2 *tab, const h1 *be, const h1 *tg, int h)
{
    const int tid = threadIdx.x;
    const int cg = tid >> 6; // 16 code bytes each
    const int lh = tid & (LPH - 1);
    const int j = LPH == 32 ? (tid >> 5) & 1 : (tid >> 4) & 1;
    const int pass = LPH == 32 ? 0 : (tid >> 5) & 1;
    const int pi = h * 128 + 64 * pass + 4 * lh + 2 * j;
    const int slot = LPH == 32 ? j * (LUT_ENTRIES * 32) + lh : pass * (LUT_ENTRIES * 32) + j * 16 + lh;
    const h2 b2 = *reinterpret_cast<const h2 *>(be + pi);
    const h2 t2 = *reinterpret_cast<const h2 *>(tg + pi);
    const h2 bt = b2 * t2;
    const h2 omt = splat((h1)1.0f) - bt; // gemv.cu:220-221
#pragma unroll
    for (int i = 0; i < LUT_ENTRIES / FT_WAVES; i++) {
        const int code = cg * (LUT_ENTRIES / FT_WAVES) + i;
        const h2 q = (h2){(h1)((code & 15) - 8), (h1)((code >> 4) - 8)};
        const h2 f = pk_fma(b2, pk_abs(q), omt); // gemv.cu:163, first half
        tab[slot + code * 32] = make_uint2(as_u32(q), as_u32(f));
    }
}

// The per-lane constant the table address is permuted from.
template <int LPH>
__device__ __forceinline__ uint32_t ft_lane_copy(int lh)
{
    return LPH == 32 ? 0x100u | ((uint32_t)lh * 8u)
                     : 0x10000u | ((128u + (uint32_t)lh * 8u) << 8) | ((uint32_t)lh * 8u);
}

// Entry of byte k (0..3) of `bytes` for pair j (0 / 1) of pass `pass`; k, j and pass must be
// compile-time constants after unrolling (the selector becomes a literal).
template <int LPH>
__device__ __forceinline__ uint2 ft_get(const uint2 *tab, uint32_t bytes, uint32_t lane_copy, int k, int j, int pass)
{
    // selector bytes 0-3 pick from lane_copy, 4-7 from bytes, 0x0C is zero
    //   32 lanes: [0, j, bytes.byte[k], lane*8]
    //   16 lanes: [0, pass, bytes.byte[k], j*128 + lane*8]
    const uint32_t sel = LPH == 32 ? (j ? 0x0C010000u : 0x0C0C0000u) | ((4u + (uint32_t)k) << 8)
                                   : (pass ? 0x0C020000u : 0x0C0C0000u) | ((4u + (uint32_t)k) << 8) | (j ? 1u : 0u);
    const uint32_t addr = __builtin_amdgcn_perm(bytes, lane_copy, sel);
    return *reinterpret_cast<const uint2 *>(reinterpret_cast<const char *>(tab) + addr);
}

// The main loop needs zp, sc and alpha only (the table holds what beta and the target give); the
// handful of tokens after it (ragged tail, appended token) use the plain update and load them then.
__device__ __forceinline__ void ft_init_pairs(Pair *st, const h1 *zp, const h1 *sc, const h1 *al, int h,
                                              int bx, int c0, int seg, const Seg &sa)
{
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const int pi = h * 128 + c0 + 2 * p;
        st[p].zp = *reinterpret_cast<const h2 *>(zp + pi);
        st[p].sc = *reinterpret_cast<const h2 *>(sc + pi);
        st[p].al = *reinterpret_cast<const h2 *>(al + pi);
    }
    if (seg_begin(sa, seg) > 0) {
        const int j = seg_begin(sa, seg) / sa.ckpt_interval - 1;
        load_state<4>(sa.ckpt + (((size_t)bx * sa.n_ckpt_cap + j) * 128 + c0) * 2, st);
    }
}

__device__ __forceinline__ void ft_load_beta(Pair *st, const h1 *be, const h1 *tg, int h, int c0)
{
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const int pi = h * 128 + c0 + 2 * p;
        st[p].be = *reinterpret_cast<const h2 *>(be + pi);
        const h2 bt = st[p].be * *reinterpret_cast<const h2 *>(tg + pi);
        st[p].omt = splat((h1)1.0f) - bt;
    }
}

// State update with the tabulated multiplier: zp <- r16(alpha*qs + zp), sc <- r16(sc*f).
__device__ __forceinline__ void update_pair_f(Pair &p, h2 f, h2 qs)
{
    p.zp = pk_fma(p.al, qs, p.zp);
    p.sc = p.sc * f;
}

// ---------------------------------------------------------------------------------------------
// forward_qk  (gemv.cu:435-815), per-head table
// ---------------------------------------------------------------------------------------------
//
// A workgroup serves one head and walks through one or more VIRTUAL workgroups of that head
// (sa.phys_per_head apart), each 16 waves' worth of (sequences, segment) units, without a
// barrier between them: the table is built once, and a wave that finishes its unit goes straight
// on to its unit of the next virtual workgroup.
//
// LPH = 16: a lane makes two passes over every supergroup (32 + 32 channel-pair tokens), so the
// reduction of the eight partial logits, the store and the loop overhead are paid once per eight
// channels instead of once per four.
// One unit of forward_qk: this wave's sequences of head h over its segment of virtual workgroup
// vw, with the head's table in `tab`.
template <int LPH>
__device__ __forceinline__ void qk_ft_unit(
    const uint2 *tab, const h1 *__restrict__ q, uint4 *__restrict__ cache, const h1 *__restrict__ k_new,
    h1 *__restrict__ out,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int B, int H, int T, int n_super_cap, h1 *__restrict__ state_out, const Seg &sa, int h, int vw)
{
    constexpr int D = 128, CPL = 4; // per pass
    using G = Geo<D, CPL>;
    constexpr int NPASS = 32 / LPH;
    constexpr int PFQ = PF / NPASS; // supergroups in flight: the same bytes per lane either way
    const int lane = threadIdx.x & 63;
    const int tk = LPH == 32 ? token_of_lane(lane) : token_of_lane16(lane);
    {
        const FtUnit<LPH> un(B, H, sa.nseg, h, vw);
        const uint32_t lane_copy = ft_lane_copy<LPH>(un.lh);
        const int bx = un.bx, lh = un.lh, c0 = un.c0;
        const bool active = un.active;
        const bool last = seg_is_last(sa, un.seg);

        Pair st[NPASS * G::NP];
        h2 qv[NPASS * G::NP];
#pragma unroll
        for (int ps = 0; ps < NPASS; ps++) {
            ft_init_pairs(st + ps * G::NP, zp, sc, al, h, bx, c0 + 64 * ps, un.seg, sa);
#pragma unroll
            for (int p = 0; p < G::NP; p++)
                qv[ps * G::NP + p] = load_act2(q + (size_t)bx * D + c0 + 64 * ps + 2 * p, sa.act_bf16);
        }

        const int t0 = seg_begin(sa, un.seg);
        const int t1 = last ? T : seg_end(sa, un.seg);
        uint4 *cbh = cache + (size_t)bx * n_super_cap * G::VPS + lh; // pass ps: vector lh + LPH*ps
        const uint4 *cb = cbh + (size_t)(t0 >> 3) * G::VPS;
        h1 *ob = out + (size_t)bx * sa.row_pitch + t0;
        const int nfull = (t1 - t0) >> 3;
        const bool storer = active && (LPH == 32 ? (lane & 3) == 0 : (lane & 1) == 0);

        // (padding waves have valid, clamped addresses and simply drop what they loaded)
        uint4 buf[PFQ][NPASS];
#pragma unroll
        for (int i = 0; i < PFQ; i++)
#pragma unroll
            for (int ps = 0; ps < NPASS; ps++)
                buf[i][ps] = (i < nfull) ? load_codes(cb + (size_t)i * G::VPS + LPH * ps) : make_uint4(0, 0, 0, 0);
        if (!un.wave_active)
            return; // padding waves of the head's last virtual workgroup

        auto finish = [&](const float *part, int sg, int ntok) {
            const float s = LPH == 32 ? reduce8_head32(part) : reduce8_head16(part);
            if (storer && tk < ntok)
                ob[sg * 8 + tk] = (h1)s;
        };

        // one token of the current pass, then the lookups of the same slot of the next pass
        auto token = [&](int t, auto pc, uint2 (*e)[8], const uint32_t (*nb)[2], float &out_t) {
            constexpr int ps = decltype(pc)::value;
            float acc = out_t;
#pragma unroll
            for (int p = 0; p < G::NP; p++) {
                Pair &s = st[ps * G::NP + p];
                const h2 qs = as_h2(e[p][t].x) * s.sc;
                const h2 kh = qs + s.zp;
                if (ps == 0 && p == 0)
                    acc = dot2_from_zero(qv[p], kh);
                else
                    acc = __builtin_amdgcn_fdot2(qv[ps * G::NP + p], kh, acc, false);
                update_pair_f(s, as_h2(e[p][t].y), qs);
            }
            out_t = acc;
#pragma unroll
            for (int p = 0; p < G::NP; p++)
                e[p][t] = ft_get<LPH>(tab, nb[p][t & 1], lane_copy, t >> 1, p, (ps + 1) % NPASS);
            __builtin_amdgcn_sched_barrier(0);
        };

        uint2 lk[G::NP][8];
        uint32_t nb[G::NP][2];
        float part[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (nfull > 0) {
            pair_bytes_of<D, CPL>(&buf[0][0], nb);
#pragma unroll
            for (int t = 0; t < 8; t++)
#pragma unroll
                for (int p = 0; p < G::NP; p++)
                    lk[p][t] = ft_get<LPH>(tab, nb[p][t & 1], lane_copy, t >> 1, p, 0);
        }
        // One supergroup; i = its buffer in the rotation.  Nothing conditional: the trip count is
        // wave-uniform, the prefetch index is clamped to the segment's last supergroup (the load is
        // unconditional; a load inside a branch makes the next wait cover every load in flight), and the reduction of the previous supergroup
        // (done here, between the lookups' issue and their first use) stores nothing for sg == 0.
        auto body = [&](int sg, auto ic) {
            constexpr int i = decltype(ic)::value;
            static_for<NPASS>([&](auto pc) {
                constexpr int ps = decltype(pc)::value;
                // the code bytes of the pass after this one: same supergroup, or the next one's first
                if (ps + 1 < NPASS)
                    pair_bytes_of<D, CPL>(&buf[i][(ps + 1) % NPASS], nb);
                else
                    pair_bytes_of<D, CPL>(&buf[(i + 1) % PFQ][0], nb);
                buf[i][ps] = load_codes(cb + (size_t)min(sg + PFQ, nfull - 1) * G::VPS + LPH * ps);
                __builtin_amdgcn_sched_barrier(0);
                if (ps == 0) {
                    finish(part, sg - 1, sg > 0 ? 8 : 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int t = 0; t < 8; t++)
                    token(t, pc, lk, nb, part[t]);
            });
        };
        rotate_over<PFQ>(nfull, body);
        if (nfull > 0)
            finish(part, nfull - 1, 8);
        if (!last)
            return;

        // ragged tail: T % 8 tokens of the last supergroup (gemv.cu:648-654); plain arithmetic
        const int ntail = (t1 - t0) & 7;
        float tp[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int ps = 0; ps < NPASS; ps++) {
            ft_load_beta(st + ps * G::NP, be, tg, h, c0 + 64 * ps);
            if (ntail) {
                uint32_t w[4];
                vec_words(cb[(size_t)nfull * G::VPS + LPH * ps], w);
#pragma unroll
                for (int pp = 0; pp < 2; pp++) {
                    Pair &s = st[ps * G::NP + pp];
                    for (int tt = 0; tt < ntail; tt++) {
                        const h2 qc = extract_pair<4>(w[2 * pp], w[2 * pp + 1], tt);
                        const h2 qs = qc * s.sc;
                        const float d = __builtin_amdgcn_fdot2(qv[ps * G::NP + pp], qs + s.zp, 0.0f, false);
#pragma unroll
                        for (int k = 0; k < 8; k++)
                            tp[k] += (k == tt) ? d : 0.0f;
                        update_pair(s, qc, qs);
                    }
                }
            }
        }
        if (ntail)
            finish(tp, nfull, ntail);

        float self = 0.0f;
#pragma unroll
        for (int ps = 0; ps < NPASS; ps++) {
            if (active)
                publish_state<D, CPL>(st + ps * G::NP, state_out, sa, bx, c0 + 64 * ps, T);
            h2 deq[G::NP];
            append_new_token<D, CPL>(cbh + LPH * ps, T, k_new + (size_t)bx * D + c0 + 64 * ps, st + ps * G::NP, deq,
                                     active, sa.act_bf16);
#pragma unroll
            for (int p = 0; p < G::NP; p++)
                self = __builtin_amdgcn_fdot2(qv[ps * G::NP + p], deq[p], self, false);
        }
        self = head_allreduce<LPH>(self);
        if (active && lh == 0)
            out[(size_t)bx * sa.row_pitch + T] = (h1)self;
    }
}

template <int LPH>
__global__ __launch_bounds__(FT_BLK) void qk_ft_kernel(
    const h1 *__restrict__ q, uint4 *__restrict__ cache, const h1 *__restrict__ k_new,
    h1 *__restrict__ out,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int B, int H, int T, int n_super_cap, h1 *__restrict__ state_out, Seg sa)
{
    __shared__ uint2 tab[FT_TABLE_WORDS64]; // the only LDS object: sits at offset 0
    const int h = (int)blockIdx.x / sa.phys_per_head;
    const int pw = (int)blockIdx.x % sa.phys_per_head;
    const int wph = ft_wgs_per_head(B, sa.nseg, 64 / LPH);
    // The table is built before the loop: a barrier under a condition inside it, even a uniform
    // one, costs the loop body some twenty registers and spills.
    ft_fill<LPH>(tab, be, tg, h);
    __syncthreads();
    for (int vw = pw; vw < wph; vw += sa.phys_per_head)
        qk_ft_unit<LPH>(tab, q, cache, k_new, out, zp, sc, al, be, tg, B, H, T, n_super_cap, state_out, sa, h, vw);
}

// ---------------------------------------------------------------------------------------------
// forward_ov  (gemv.cu:946-1178), per-head table
// ---------------------------------------------------------------------------------------------
//
// The contraction runs on the matrix cores.  v_mfma_f32_4x4x4_16B_f16 multiplies, in each group of
// four lanes, the 4x4 matrix whose row i is lane i's A operand with the matrix whose column r is
// lane r's B operand, and lane r receives column r of the product.  With
//   B of lane r = (x_A[t], x_B[t], x_A[t+1], x_B[t+1])   the lane's channel pair at two tokens, which
//                                                        is two consecutive registers as they are,
//   A of lane 0 = (w[t], 0, w[t+1], 0),  A of lane 1 = (0, w[t], 0, w[t+1]),  A of lanes 2, 3 = 0,
// element 0 of the lane's result is sum w*x_A and element 1 is sum w*x_B: the lane's own two
// outputs, nothing crosses lanes, products exact and sums in fp32 as in the vector form.  One
// instruction per (pair, two tokens) replaces four mixed-precision multiply-adds; a matrix
// instruction takes one issue slot and then runs beside the vector pipe.  The weights reach the A
// layout with two v_perm_b32 per token pair and per-lane selectors.  x = r16(q*sc + zp), the
// reference's dequantised value (gemv.cu:1085-1086).  (The product is linear, so contracting q*sc
// and zp separately would save the packed add; the outputs would then lack that rounding, up to
// half an fp16 ulp of the largest value, for 1 % of the kernel's time: not done.)
// A non-finite cached value makes both outputs of its channel PAIR non-finite (0 * inf inside the
// product); the vector form of ov_kernel's two-channel lanes confines it to its own channel.
//
// One virtual workgroup per workgroup (forward_ov's plans never need more).  sa.combine: the two
// or four segments of a wave's sequences sit in the same workgroup and are added there; otherwise
// every segment stores its fp32 partial sums for ov_finalize_kernel.
// The whole of forward_ov for one workgroup: builds head h's table in `tab` (which no wave may
// still be reading), then this wave's unit of virtual workgroup vw.  Every wave of the workgroup
// must call it (barriers).
template <int LPH>
__device__ __forceinline__ void ov_ft_unit(
    uint2 *tab, const h1 *__restrict__ attn, uint4 *__restrict__ cache, const h1 *__restrict__ v_new,
    h1 *__restrict__ out, float *__restrict__ partial,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int B, int H, int T, int n_super_cap, h1 *__restrict__ state_out, const Seg &sa, int h, int vw)
{
    constexpr int D = 128, CPL = 4; // per pass
    using G = Geo<D, CPL>;
    constexpr int NPASS = 32 / LPH;
    constexpr int PFQ = PF / NPASS;
    const int BH = B * H;
    // selectors that turn the word (w[t], w[t+1]) into this lane's two A registers
    const int role = threadIdx.x & 3;
    const uint32_t sel_a0 = role == 0 ? 0x0C0C0100u : role == 1 ? 0x01000C0Cu : 0x0C0C0C0Cu;
    const uint32_t sel_a1 = role == 0 ? 0x0C0C0302u : role == 1 ? 0x03020C0Cu : 0x0C0C0C0Cu;
    {
        const FtUnit<LPH> un(B, H, sa.nseg, h, vw);
        const uint32_t lane_copy = ft_lane_copy<LPH>(un.lh);
        const int bx = un.bx, lh = un.lh, c0 = un.c0;
        const bool active = un.active;
        const bool last = seg_is_last(sa, un.seg);

        Pair st[NPASS * G::NP];
        float acc[NPASS * CPL];
        f4v acc4[NPASS * G::NP];
#pragma unroll
        for (int ps = 0; ps < NPASS; ps++)
            ft_init_pairs(st + ps * G::NP, zp, sc, al, h, bx, c0 + 64 * ps, un.seg, sa);
#pragma unroll
        for (int p = 0; p < NPASS * G::NP; p++)
            acc4[p] = (f4v){0.0f, 0.0f, 0.0f, 0.0f};

        const int t0 = seg_begin(sa, un.seg);
        const int t1 = last ? T : seg_end(sa, un.seg);
        uint4 *cbh = cache + (size_t)bx * n_super_cap * G::VPS + lh; // pass ps: vector lh + LPH*ps
        const uint4 *cb = cbh + (size_t)(t0 >> 3) * G::VPS;
        const h1 *wrow = attn + (size_t)bx * sa.row_pitch;
        const h1 *wb = wrow + t0;
        const int nfull = (t1 - t0) >> 3;

        auto load_w = [&](int sg) {
            uint4 r;
            __builtin_memcpy(&r, wb + (size_t)sg * 8, 16); // row base is only 2-byte aligned
            return r;
        };
        // the first code words and weights, like the parameters above, are requested before the
        // table is built, so that their latency runs beside the fill instead of after it
        uint4 buf[PFQ][NPASS];
        uint4 wbuf[PFQ];
#pragma unroll
        for (int i = 0; i < PFQ; i++) {
#pragma unroll
            for (int ps = 0; ps < NPASS; ps++)
                buf[i][ps] = (i < nfull) ? load_codes(cb + (size_t)i * G::VPS + LPH * ps) : make_uint4(0, 0, 0, 0);
            wbuf[i] = (i < nfull) ? load_w(i) : make_uint4(0, 0, 0, 0);
        }
        ft_fill<LPH>(tab, be, tg, h);
        __syncthreads();
        if (!un.wave_active) {
            if (sa.combine) { // the two barriers of the in-workgroup sum below
                __syncthreads();
                __syncthreads();
            }
            return;
        }

        // two tokens of the current pass on the matrix cores, then the lookups of the same two
        // slots of the next pass.  The A operands are built in the first pass and kept for the second.
        h4v aop[4];
        auto token2 = [&](int t, auto pc, uint2 (*e)[8], const uint32_t (*nb)[2], const uint4 wv) {
            constexpr int ps = decltype(pc)::value;
            if (ps == 0) {
                const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
                const uint32_t w2 = ww[t >> 1];
                aop[t >> 1] = as_h4(__builtin_amdgcn_perm(w2, w2, sel_a0), __builtin_amdgcn_perm(w2, w2, sel_a1));
            }
            const h4v a = aop[t >> 1];
            uint32_t vd[G::NP][2];
#pragma unroll
            for (int k = 0; k < 2; k++)
#pragma unroll
                for (int p = 0; p < G::NP; p++) {
                    Pair &s = st[ps * G::NP + p];
                    const h2 qs = as_h2(e[p][t + k].x) * s.sc;
                    vd[p][k] = as_u32(qs + s.zp);
                    update_pair_f(s, as_h2(e[p][t + k].y), qs);
                }
#pragma unroll
            for (int p = 0; p < G::NP; p++)
                acc4[ps * G::NP + p] = __builtin_amdgcn_mfma_f32_4x4x4f16(a, as_h4(vd[p][0], vd[p][1]),
                                                                          acc4[ps * G::NP + p], 0, 0, 0);
#pragma unroll
            for (int k = 0; k < 2; k++)
#pragma unroll
                for (int p = 0; p < G::NP; p++)
                    e[p][t + k] = ft_get<LPH>(tab, nb[p][(t + k) & 1], lane_copy, (t + k) >> 1, p, (ps + 1) % NPASS);
            __builtin_amdgcn_sched_barrier(0);
        };

        uint2 lk[G::NP][8];
        uint32_t nb[G::NP][2];
        if (nfull > 0) {
            pair_bytes_of<D, CPL>(&buf[0][0], nb);
#pragma unroll
            for (int t = 0; t < 8; t++)
#pragma unroll
                for (int p = 0; p < G::NP; p++)
                    lk[p][t] = ft_get<LPH>(tab, nb[p][t & 1], lane_copy, t >> 1, p, 0);
        }
        auto body = [&](int sg, auto ic) {
            constexpr int i = decltype(ic)::value;
            const int sgp = min(sg + PFQ, nfull - 1);
            static_for<NPASS>([&](auto pc) {
                constexpr int ps = decltype(pc)::value;
                if (ps + 1 < NPASS)
                    pair_bytes_of<D, CPL>(&buf[i][(ps + 1) % NPASS], nb);
                else
                    pair_bytes_of<D, CPL>(&buf[(i + 1) % PFQ][0], nb);
                buf[i][ps] = load_codes(cb + (size_t)sgp * G::VPS + LPH * ps);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < 8; t += 2)
                    token2(t, pc, lk, nb, wbuf[i]);
            });
            wbuf[i] = load_w(sgp); // reloaded once its last token is done (see ov_kernel)
        };
        rotate_over<PFQ>(nfull, body);
#pragma unroll
        for (int p = 0; p < NPASS * G::NP; p++) {
            acc[2 * p] = acc4[p].x;
            acc[2 * p + 1] = acc4[p].y;
        }

        if (last) {
            const int ntail = (t1 - t0) & 7;
            const float wT = (float)wrow[T];
#pragma unroll
            for (int ps = 0; ps < NPASS; ps++) {
                Pair *sp = st + ps * G::NP;
                float *ap = acc + ps * CPL;
                ft_load_beta(sp, be, tg, h, c0 + 64 * ps);
                if (ntail) {
                    uint32_t w[4];
                    vec_words(cb[(size_t)nfull * G::VPS + LPH * ps], w);
#pragma unroll
                    for (int pp = 0; pp < 2; pp++) {
                        Pair &s = sp[pp];
                        for (int tt = 0; tt < ntail; tt++) {
                            const h2 qc = extract_pair<4>(w[2 * pp], w[2 * pp + 1], tt);
                            const h2 qs = qc * s.sc;
                            const h2 vd = qs + s.zp;
                            const float wt = (float)wb[nfull * 8 + tt];
                            ap[2 * pp] = __builtin_fmaf(wt, (float)vd.x, ap[2 * pp]);
                            ap[2 * pp + 1] = __builtin_fmaf(wt, (float)vd.y, ap[2 * pp + 1]);
                            update_pair(s, qc, qs);
                        }
                    }
                }
                if (active)
                    publish_state<D, CPL>(sp, state_out, sa, bx, c0 + 64 * ps, T);
                h2 deq[G::NP];
                append_new_token<D, CPL>(cbh + LPH * ps, T, v_new + (size_t)bx * D + c0 + 64 * ps, sp, deq, active,
                                         sa.act_bf16);
#pragma unroll
                for (int p = 0; p < G::NP; p++) {
                    ap[2 * p] = __builtin_fmaf(wT, (float)deq[p].x, ap[2 * p]);
                    ap[2 * p + 1] = __builtin_fmaf(wT, (float)deq[p].y, ap[2 * p + 1]);
                }
            }
        }
        if (sa.combine) {
            // nseg is 2 or 4: the waves holding
            // the other segments of these sequences are 4, 8, 12 waves away (interleave_segment:
            // quad q takes segment q mod nseg).  The table is finished with once every wave is
            // here; its first 16 KB per pass take the partial sums, and the wave of segment 0 adds
            // them in segment order (what ov_finalize_kernel does).
            __syncthreads();
            float4 *red = reinterpret_cast<float4 *>(tab);
            const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
            for (int ps = 0; ps < NPASS; ps++)
                red[(ps * FT_WAVES + wv) * 64 + lane] =
                    make_float4(acc[4 * ps], acc[4 * ps + 1], acc[4 * ps + 2], acc[4 * ps + 3]);
            __syncthreads();
            if (un.seg != 0 || !active)
                return;
            for (int s = 1; s < sa.nseg; s++)
#pragma unroll
                for (int ps = 0; ps < NPASS; ps++) {
                    const float4 p = red[(ps * FT_WAVES + wv + 4 * s) * 64 + lane];
                    acc[4 * ps] += p.x;
                    acc[4 * ps + 1] += p.y;
                    acc[4 * ps + 2] += p.z;
                    acc[4 * ps + 3] += p.w;
                }
        }
        if (!active)
            return;
#pragma unroll
        for (int ps = 0; ps < NPASS; ps++) {
            if (sa.nseg == 1 || sa.combine) {
                h1 *o = out + (size_t)bx * D + c0 + 64 * ps;
#pragma unroll
                for (int p = 0; p < G::NP; p++)
                    store_act2(o + 2 * p, acc[4 * ps + 2 * p], acc[4 * ps + 2 * p + 1], sa.act_bf16);
            } else {
                float2 *o = reinterpret_cast<float2 *>(partial + ((size_t)un.seg * BH + bx) * D + c0 + 64 * ps);
#pragma unroll
                for (int p = 0; p < G::NP; p++)
                    o[p] = make_float2(acc[4 * ps + 2 * p], acc[4 * ps + 2 * p + 1]);
            }
        }
    }
}

template <int LPH>
__global__ __launch_bounds__(FT_BLK) void ov_ft_kernel(
    const h1 *__restrict__ attn, uint4 *__restrict__ cache, const h1 *__restrict__ v_new,
    h1 *__restrict__ out, float *__restrict__ partial,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int B, int H, int T, int n_super_cap, h1 *__restrict__ state_out, Seg sa)
{
    __shared__ uint2 tab[FT_TABLE_WORDS64];
    const int wph = ft_wgs_per_head(B, sa.nseg, 64 / LPH);
    ov_ft_unit<LPH>(tab, attn, cache, v_new, out, partial, zp, sc, al, be, tg, B, H, T, n_super_cap, state_out, sa,
                    (int)blockIdx.x / wph, (int)blockIdx.x % wph);
}

// ---------------------------------------------------------------------------------------------
// One launch per decode step  (llama_adkv.py:264-274: forward_qk, softmax, forward_ov)
// ---------------------------------------------------------------------------------------------
//
// When both forward_qk and forward_ov cut every sequence into FOUR segments and run one virtual
// workgroup per workgroup, the four quads of a workgroup hold the four segments of the same
// sequences: a workgroup sees whole rows of logits, and the three stages need no launch between
// them, only barriers.  forward_qk's unit writes the logits; once every wave of the workgroup is
// done, wave (quad k, j) turns row k of wave j's sequences into weights (the arithmetic of
// softmax_kernel: scaled logit, maximum, __expf, sum, reciprocal, one rounding to fp16; sums in a
// fixed order, so replays agree bit for bit; rows of up to FT_SOFTMAX_MAX_ROW elements, longer
// contexts take three launches); then the table is rebuilt for V and
// forward_ov's unit runs, adding its four segments inside the workgroup.  Saved: two launch gaps
// with their cache write-backs and the softmax kernel's own launch, and a workgroup whose waves
// finish early no longer waits for the slowest workgroup of the launch before it goes on.
// One row of n <= NV * 512 logits -> weights by one wave: the row is read once, 16 bytes per lane
// and load, all loads issued before the first use, and kept in registers as fp16.
constexpr int FT_SOFTMAX_MAX_NV = 17;
constexpr int FT_SOFTMAX_MAX_ROW = FT_SOFTMAX_MAX_NV * 512;

template <int NV>
__device__ __forceinline__ void ft_softmax_row(const h1 *l, h1 *w, int n, float scaling, int lane)
{
    h1 x[NV][8];
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int i0 = (v * 64 + lane) * 8;
        if (i0 + 8 <= n) {
            __builtin_memcpy(x[v], l + i0, 16); // rows may be only 2-byte aligned
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++)
                x[v][k] = i0 + k < n ? l[i0 + k] : (h1)0.0f;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < NV; v++)
#pragma unroll
        for (int k = 0; k < 8; k++)
            if ((v * 64 + lane) * 8 + k < n)
                mx = fmaxf(mx, (float)x[v][k] * scaling);
#pragma unroll
    for (int m = 1; m < 64; m <<= 1)
        mx = fmaxf(mx, __shfl_xor(mx, m, 64));
    float sum = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; v++)
#pragma unroll
        for (int k = 0; k < 8; k++)
            if ((v * 64 + lane) * 8 + k < n)
                sum += __expf((float)x[v][k] * scaling - mx);
#pragma unroll
    for (int m = 1; m < 64; m <<= 1)
        sum += __shfl_xor(sum, m, 64);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int i0 = (v * 64 + lane) * 8;
        h1 o[8];
#pragma unroll
        for (int k = 0; k < 8; k++)
            o[k] = (h1)(__expf((float)x[v][k] * scaling - mx) * inv);
        if (i0 + 8 <= n) {
            __builtin_memcpy(w + i0, o, 16);
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (i0 + k < n)
                    w[i0 + k] = o[k];
        }
    }
}

template <int LPH>
__device__ __forceinline__ void ft_softmax_rows(const h1 *logits, h1 *weights, long pitch, int B, int H, int T,
                                                int h, int vw, float scaling)
{
    constexpr int UPW = 64 / LPH;
    const int wave = threadIdx.x >> 6, k = wave >> 2, j = wave & 3, lane = threadIdx.x & 63;
    const int b = (vw * 4 + j) * UPW + k; // FtUnit with four segments: wave j of a quad holds these sequences
    if (k >= UPW || b >= B)
        return;
    const h1 *l = logits + (size_t)(b * H + h) * pitch;
    h1 *w = weights + (size_t)(b * H + h) * pitch;
    const int n = T + 1;
    if (n <= 9 * 512)
        ft_softmax_row<9>(l, w, n, scaling, lane);
    else
        ft_softmax_row<FT_SOFTMAX_MAX_NV>(l, w, n, scaling, lane);
}

struct FtParams {
    const h1 *zp, *sc, *al, *be, *tg;
};

template <int LPH>
__global__ __launch_bounds__(FT_BLK) void decode_ft_kernel(
    const h1 *q, uint4 *k_cache, const h1 *k_new, uint4 *v_cache, const h1 *v_new,
    h1 *logits, h1 *weights, h1 *out, FtParams kp, FtParams vp,
    int B, int H, int T, int n_super_cap, float scaling, Seg ka, Seg va)
{
    __shared__ uint2 tab[FT_TABLE_WORDS64];
    const int wph = ft_wgs_per_head(B, ka.nseg, 64 / LPH); // == ka.phys_per_head, and the same for va
    const int h = (int)blockIdx.x / wph, vw = (int)blockIdx.x % wph;
    ft_fill<LPH>(tab, kp.be, kp.tg, h);
    __syncthreads();
    qk_ft_unit<LPH>(tab, q, k_cache, k_new, logits, kp.zp, kp.sc, kp.al, kp.be, kp.tg, B, H, T, n_super_cap,
                    nullptr, ka, h, vw);
    __syncthreads(); // the workgroup's rows of logits are complete and visible to all its waves
    ft_softmax_rows<LPH>(logits, weights, ka.row_pitch, B, H, T, h, vw, scaling);
    __syncthreads(); // weights written; nobody reads the K table any more
    ov_ft_unit<LPH>(tab, weights, v_cache, v_new, out, nullptr, vp.zp, vp.sc, vp.al, vp.be, vp.tg, B, H, T,
                    n_super_cap, nullptr, va, h, vw);
}

} // namespace adkv
