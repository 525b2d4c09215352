// Decode kernels for head dim 128 that put the contraction on the matrix cores, for GQ >= 1 query
// heads per KV head and for 4-bit or 2-bit codes.  Included by adkv_kernels.hip after
// the shared device helpers.
//
// The fp16 replay of the filter state (the dominant cost) is the same per-lane arithmetic as in
// qk_kernel / ov_kernel and runs once per KV head; only what happens to the dequantised value
// differs.  v_mfma_f32_4x4x4_16B_f16 multiplies sixteen independent 4x4 blocks per instruction:
// lane 4b+r supplies row r of A and column r of B of block b (four fp16 each) and receives column
// r of D (four fp32, one per row).
//
//   QK:  D[token][head] += A[token][4 channels] * B[4 channels][head]
//        The dequantised keys of 8 tokens x 2 heads x 128 channels go through a wave-private LDS
//        tile; a block is (KV head, 4 tokens, a quarter of the channels), eight instructions walk
//        the quarter, two DPP rotations add the quarters.  No cross-lane reduction of per-lane
//        partial dot products is left.
//   OV:  D[head][channel] += A[head][4 tokens] * B[4 tokens][channel]
//        B is the lane's own channel over four consecutive tokens (two v_perm_b32 per channel pair
//        repack token-major pairs), A the attention weights of the block's heads: every lane gets
//        the outputs of all GQ heads for its own channels, with no data leaving the lane.
//
// The time axis is walked in units of 8 tokens: one unit per supergroup with 4-bit codes, two with
// 2-bit codes (16 tokens per channel word).  Table lookups for the next unit are issued between
// the tokens of the current one, into the register slots they vacate.
#pragma once

namespace adkv {


constexpr int GQA_D = 128;
constexpr int GQA_CPL = 4;
// The key tile of a wave: 8 token rows of 8-byte words (a lane's two channel pairs).  The LDS
// serves an 8-byte access of 16 lanes per clock from 32 four-byte banks, so a group of 16 lanes has
// to touch 16 different 8-byte slots modulo 16.  Writes: lane L of a head goes to column
// tile_col(L) of its head's 36 columns, 16 consecutive lanes to 16 consecutive words.  Reads of the
// matrix operands: lane (row r of 4, quarter qd of 4) reads word m of its quarter from token row
// r, eight times; the second half of a head sits 4 words further (columns 20-35), so that the
// quarters start at 0, 8, 20, 28 = 0, 8, 4, 12 modulo 16, and a row stride of 73 = 9 modulo 16
// spreads the four rows over 0, 9, 2, 11: all 16 (row, quarter) slots differ.  (With 32 columns per
// head and a stride of 65 quarters 0 and 2 met in the same banks: SQ_LDS_BANK_CONFLICT was a
// quarter of the LDS's busy cycles, and this kernel keeps the LDS busier than the vector pipe.)
constexpr int TILE_HEAD64 = 36;              // columns per head
constexpr int TILE_ROW64 = 73;               // 8-byte words per token row: 2 heads x 36 columns + 1
constexpr int TILE_WORDS64 = 8 * TILE_ROW64; // per wave
__device__ __forceinline__ int tile_col(int lane_in_head) { return lane_in_head + 4 * (lane_in_head >> 4); }

// d: a lane's partial logits of four tokens over its quarter of the channels, fresh from the matrix
// cores; the other quarters are in the lanes that differ in bits 2 and 3 (qd).  Lane qd gets the
// total of token qd, in six masked DPP adds: a masked add writes only the banks of its mask
//   banks 0,1 | 2,3 (bit 3): keep tokens 0,1 | 2,3, add the partner's (rotate by 8)
//   banks 0,2 | 1,3 (bit 2): keep the first | second of those, add lane+4's | lane-4's.
// The leading wait states cover the matrix cores' write of d (up to five are required before a
// vector instruction reads it), the inner ones a DPP operand written by the two instructions before.
__device__ __forceinline__ float quarter_sum(f4v d)
{
    float s0, s1, r;
    asm volatile(
        "s_nop 7\n\t"
        "v_add_f32_dpp %0, %3, %3 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %1, %4, %4 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %0, %5, %5 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %1, %6, %6 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %2, %0, %0 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %2, %1, %1 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "s_nop 0"
        : "=&v"(s0), "=&v"(s1), "=&v"(r)
        : "v"(d.x), "v"(d.y), "v"(d.z), "v"(d.w));
    return r;
}


// The code words of one supergroup -> the per-pair byte streams the table is indexed with.
template <int BITS>
__device__ __forceinline__ void code_bytes(const uint4 &u, uint32_t (*nb)[2])
{
    if (BITS == 4) {
        pair_bytes(u.x, u.y, nb[0][0], nb[0][1]);
        pair_bytes(u.z, u.w, nb[1][0], nb[1][1]);
    } else {
        pair_bytes2(u.x, u.y, nb[0][0], nb[0][1]);
        pair_bytes2(u.z, u.w, nb[1][0], nb[1][1]);
    }
}

// Table entries of one 8-token unit held in registers, and how a token finds its (q, |q|):
//   4-bit: slot t, 8 bytes.   2-bit: slot 2*(t/4) + (t&1), 16 bytes, second half for t&2.
template <int BITS>
struct Lookups {
    static constexpr int SLOTS = BITS == 4 ? 8 : 4;
    using Entry = typename std::conditional<BITS == 4, uint2, uint4>::type;
    Entry e[2][SLOTS];

    // all lookups of unit `half` (0 or 1 within the supergroup) of the words `nb`
    __device__ __forceinline__ void fill(const uint2 *lut, const uint32_t (*nb)[2], uint32_t lane_copy, int half)
    {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            if constexpr (BITS == 4) {
#pragma unroll
                for (int t = 0; t < 8; t++)
                    e[p][t] = lut_get(lut, nb[p][t & 1], lane_copy, t >> 1);
            } else {
#pragma unroll
                for (int s = 0; s < 4; s++)
                    e[p][s] = lut2_get(lut, nb[p][s & 1], lane_copy, 2 * half + (s >> 1));
            }
        }
    }
    __device__ __forceinline__ void get(int p, int t, h2 &q, h2 &qabs) const
    {
        if constexpr (BITS == 4) {
            q = as_h2(e[p][t].x);
            qabs = as_h2(e[p][t].y);
        } else {
            const uint4 v = e[p][2 * (t >> 2) + (t & 1)];
            q = as_h2((t & 2) ? v.z : v.x);
            qabs = as_h2((t & 2) ? v.w : v.y);
        }
    }
    // after token t: refill the slot it has just finished with, for the unit `next_half` of `nb`
    __device__ __forceinline__ void refill(const uint2 *lut, const uint32_t (*nb)[2], uint32_t lane_copy,
                                           int t, int next_half)
    {
        if constexpr (BITS == 4) {
#pragma unroll
            for (int p = 0; p < 2; p++)
                e[p][t] = lut_get(lut, nb[p][t & 1], lane_copy, t >> 1);
        } else {
            if (t & 2) {
#pragma unroll
                for (int p = 0; p < 2; p++)
                    e[p][2 * (t >> 2) + (t & 1)] = lut2_get(lut, nb[p][t & 1], lane_copy, 2 * next_half + (t >> 2));
            }
        }
    }
};

template <int BITS>
__device__ __forceinline__ void fill_table(uint2 *lut, int tid, int nthreads)
{
    if (BITS == 4)
        lut_fill(lut, tid, nthreads);
    else
        lut2_fill(lut, tid, nthreads);
}

template <int BITS>
__device__ __forceinline__ uint32_t table_lane_offset(int lane)
{
    return BITS == 4 ? (uint32_t)(lane & (LUT_COPIES - 1)) * 8u : (uint32_t)(lane & (LUT2_COPIES - 1)) * 16u;
}

// ---------------------------------------------------------------------------------------------
// forward_qk with GQ query heads per KV head
// ---------------------------------------------------------------------------------------------
template <int BITS, int GQ, int BLK>
__global__ __launch_bounds__(BLK) void qk_gqa_kernel(
    const h1 *__restrict__ q, uint4 *__restrict__ cache, const h1 *__restrict__ k_new,
    h1 *__restrict__ out,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int BH, int H, int T, int n_super_cap, h1 *__restrict__ state_out, Seg sa)
{
    constexpr int D = GQA_D, CPL = GQA_CPL;
    constexpr int NB = (GQ + 3) / 4; // column sets of four heads
    constexpr int TPW = Code<BITS>::TPW, UPS = TPW / 8;
    // supergroups in flight per lane: fewer where a supergroup is 16 tokens or registers are short
    constexpr int GPF = (BITS == 2 || NB > 1) ? 2 : PF;
    using G = Geo<D, CPL>;
    __shared__ uint2 smem[LUT_WORDS64 + (BLK / 64) * TILE_WORDS64];
    const uint2 *lut = smem;
    fill_table<BITS>(smem, threadIdx.x, BLK);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const uint32_t lane_copy = table_lane_offset<BITS>(lane);
    uint2 *tile = smem + LUT_WORDS64 + (threadIdx.x >> 6) * TILE_WORDS64;

    const Unit<D, CPL, BLK> un(BH, sa.nseg);
    if (!un.wave_active)
        return; // padding waves
    const int bx = un.bx, lh = un.lh, c0 = un.c0;
    const bool active = un.active;
    const bool last = seg_is_last(sa, un.seg);
    const int h = bx % H;

    Pair st[G::NP];
    init_pairs<D, CPL>(st, zp, sc, al, be, tg, h, bx, c0, un.seg, sa);

    // matrix-core roles of this lane: block (hh, tg4, qd), row/column r
    const int r = lane & 3, qd = (lane >> 2) & 3, tg4 = (lane >> 4) & 1;
    // B operands: q of head r (+4 per column set), channels of quarter qd, four per instruction
    uint2 qb[NB][8];
#pragma unroll
    for (int n = 0; n < NB; n++) {
        const int g = 4 * n + r;
        const h1 *src = q + ((size_t)bx * GQ + (g < GQ ? g : 0)) * D + qd * 32;
#pragma unroll
        for (int m = 0; m < 8; m++) {
            const uint2 four = make_uint2(as_u32(load_act2(src + 4 * m, sa.act_bf16)),
                                          as_u32(load_act2(src + 4 * m + 2, sa.act_bf16)));
            qb[n][m] = (g < GQ) ? four : make_uint2(0u, 0u);
        }
    }
    const uint2 *arow = tile + (tg4 * 4 + r) * TILE_ROW64 + (lane >> 5) * TILE_HEAD64 + tile_col(qd * 8);
    const int wcol = (lane >> 5) * TILE_HEAD64 + tile_col(lane & 31); // where this lane's values go in a row

    const int t0 = seg_begin(sa, un.seg);
    const int t1 = last ? T : seg_end(sa, un.seg);
    uint4 *cbh = cache + (size_t)bx * n_super_cap * G::VPS + lh * G::NV;
    const uint4 *cb = cbh + (size_t)(t0 / TPW) * G::VPS;
    const int nfull = (t1 - t0) / TPW;

    // logits of the tile's tokens: read the A operands, run the instructions, add the quarters,
    // lane (.., qd, r) stores token tg4*4+qd of head r.  `unit` counts 8-token units from t0.
    auto emit_read = [&](uint2 *a) {
#pragma unroll
        for (int m = 0; m < 8; m++)
            a[m] = arow[m];
    };
    auto emit_finish = [&](const uint2 *a, int unit, int ntok) {
#pragma unroll
        for (int n = 0; n < NB; n++) {
            f4v d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int m = 0; m < 8; m++)
                d = __builtin_amdgcn_mfma_f32_4x4x4f16(as_h4(a[m].x, a[m].y), as_h4(qb[n][m].x, qb[n][m].y),
                                                       d, 0, 0, 0);
            const float mine = quarter_sum(d);
            const int tok = tg4 * 4 + qd, g = 4 * n + r;
            if (active && g < GQ && tok < ntok)
                out[((size_t)bx * GQ + g) * sa.row_pitch + t0 + unit * 8 + tok] = (h1)mine;
        }
    };

    Lookups<BITS> lk;
    // token t of the current unit; then the lookups that reuse its slot for the unit after it
    auto token = [&](int t, const uint32_t (*nbnext)[2], int next_half) {
        uint32_t kh[G::NP];
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            Pair &s = st[p];
            h2 qc, qa;
            lk.get(p, t, qc, qa);
            const h2 qs = qc * s.sc;
            kh[p] = as_u32(qs + s.zp);
            update_pair_abs(s, qa, qs);
        }
        tile[t * TILE_ROW64 + wcol] = make_uint2(kh[0], kh[1]);
        lk.refill(lut, nbnext, lane_copy, t, next_half);
        __builtin_amdgcn_sched_barrier(0);
    };

    uint4 buf[GPF];
    uint32_t nbc[G::NP][2], nbn[G::NP][2]; // byte streams of the current / the next supergroup
    uint2 areg[8] = {}; // read (and discarded) once before the first unit has filled it
#pragma unroll
    for (int i = 0; i < GPF; i++)
        buf[i] = (i < nfull) ? load_codes(cb + (size_t)i * G::VPS) : make_uint4(0, 0, 0, 0);
    if (nfull > 0) {
        code_bytes<BITS>(buf[0], nbc);
        lk.fill(lut, nbc, lane_copy, 0);
    }
    // one supergroup, nothing conditional in it; i = its buffer in the rotation
    auto body = [&](int sg, auto ic) {
        constexpr int i = decltype(ic)::value;
        // bytes of supergroup sg+1 (stale data past the end: looked up, never used)
        code_bytes<BITS>(buf[(i + 1) % GPF], nbn);
        // unconditional, clamped to the segment's last supergroup: a load inside a branch makes
        // the next wait cover every load in flight, this one included
        buf[i] = load_codes(cb + (size_t)min(sg + GPF, nfull - 1) * G::VPS);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int hf = 0; hf < UPS; hf++) {
            const int unit = sg * UPS + hf;
            const bool into_next_sg = hf == UPS - 1;
#pragma unroll
            for (int t = 0; t < 3; t++)
                token(t, into_next_sg ? nbn : nbc, into_next_sg ? 0 : hf + 1);
            // the tile reads of the previous unit were issued before these three tokens overwrote
            // its first rows (LDS operations of a wave execute in order); nothing is stored for
            // the unit before the first
            emit_finish(areg, unit - 1, unit > 0 ? 8 : 0);
#pragma unroll
            for (int t = 3; t < 8; t++)
                token(t, into_next_sg ? nbn : nbc, into_next_sg ? 0 : hf + 1);
            emit_read(areg);
        }
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            nbc[p][0] = nbn[p][0];
            nbc[p][1] = nbn[p][1];
        }
    };
    rotate_over<GPF>(nfull, body);
    if (nfull > 0)
        emit_finish(areg, nfull * UPS - 1, 8);
    if (!last)
        return;

    // ragged tail (fewer than a supergroup of tokens, gemv.cu:648-654) and the appended token
    const int ntail = (t1 - t0) % TPW;
    int unit = nfull * UPS, row = 0;
    if (ntail) {
        const uint4 u = cb[(size_t)nfull * G::VPS];
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
        for (int tt = 0; tt < ntail; tt++) {
            uint32_t kh[2];
#pragma unroll
            for (int pp = 0; pp < 2; pp++) {
                Pair &s = st[pp];
                const h2 qc = extract_pair<BITS>(w[2 * pp], w[2 * pp + 1], tt);
                const h2 qs = qc * s.sc;
                kh[pp] = as_u32(qs + s.zp);
                update_pair(s, qc, qs);
            }
            tile[row * TILE_ROW64 + wcol] = make_uint2(kh[0], kh[1]);
            if (++row == 8) {
                emit_read(areg);
                emit_finish(areg, unit, 8);
                unit++;
                row = 0;
            }
        }
    }
    if (active)
        publish_state<D, CPL>(st, state_out, sa, bx, c0, T);
    h2 deq[G::NP];
    append_new_token<D, CPL, BITS>(cbh, T, k_new + (size_t)bx * D + c0, st, deq, active, sa.act_bf16);
    tile[row * TILE_ROW64 + wcol] = make_uint2(as_u32(deq[0]), as_u32(deq[1]));
    emit_read(areg);
    emit_finish(areg, unit, row + 1);
}

// ---------------------------------------------------------------------------------------------
// forward_ov with GQ query heads per KV head
// ---------------------------------------------------------------------------------------------
template <int BITS, int GQ, int BLK>
__global__ __launch_bounds__(BLK) void ov_gqa_kernel(
    const h1 *__restrict__ attn, uint4 *__restrict__ cache, const h1 *__restrict__ v_new,
    h1 *__restrict__ out, float *__restrict__ partial,
    const h1 *__restrict__ zp, const h1 *__restrict__ sc, const h1 *__restrict__ al,
    const h1 *__restrict__ be, const h1 *__restrict__ tg,
    int BH, int H, int T, int n_super_cap, h1 *__restrict__ state_out, Seg sa)
{
    constexpr int D = GQA_D, CPL = GQA_CPL;
    constexpr int NB = (GQ + 3) / 4;
    constexpr int TPW = Code<BITS>::TPW, UPS = TPW / 8;
    constexpr int GPF = (BITS == 2 || NB > 1) ? 2 : PF;    // supergroups in flight per lane
    constexpr int WPF = 2;                                 // weight vectors (8 tokens each) in flight
    static_assert((GPF * UPS) % WPF == 0, "weight ring must line up with the unrolled loop");
    using G = Geo<D, CPL>;
    __shared__ uint2 lut[LUT_WORDS64];
    fill_table<BITS>(lut, threadIdx.x, BLK);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const uint32_t lane_copy = table_lane_offset<BITS>(lane);

    const Unit<D, CPL, BLK> un(BH, sa.nseg);
    if (!un.wave_active)
        return; // padding waves
    const int bx = un.bx, lh = un.lh, c0 = un.c0;
    const bool active = un.active;
    const bool last = seg_is_last(sa, un.seg);
    const int h = bx % H;
    const int r = lane & 3;

    Pair st[G::NP];
    init_pairs<D, CPL>(st, zp, sc, al, be, tg, h, bx, c0, un.seg, sa);
    f4v acc[NB][CPL]; // [column set][channel of this lane], element i = head 4n+i
#pragma unroll
    for (int n = 0; n < NB; n++)
#pragma unroll
        for (int c = 0; c < CPL; c++)
            acc[n][c] = (f4v){0.0f, 0.0f, 0.0f, 0.0f};

    const int t0 = seg_begin(sa, un.seg);
    const int t1 = last ? T : seg_end(sa, un.seg);
    uint4 *cbh = cache + (size_t)bx * n_super_cap * G::VPS + lh * G::NV;
    const uint4 *cb = cbh + (size_t)(t0 / TPW) * G::VPS;
    const int nfull = (t1 - t0) / TPW;
    const int nunits = nfull * UPS;
    // A operand rows: the weights of head r (+4 per column set) of this lane's KV head
    const h1 *wb[NB];
    bool wok[NB];
#pragma unroll
    for (int n = 0; n < NB; n++) {
        wok[n] = 4 * n + r < GQ;
        wb[n] = attn + ((size_t)bx * GQ + (wok[n] ? 4 * n + r : 0)) * sa.row_pitch + t0;
    }
    auto load_w = [&](int n, int unit) {
        uint4 v;
        __builtin_memcpy(&v, wb[n] + (size_t)unit * 8, 16); // rows are only 2-byte aligned
        return wok[n] ? v : make_uint4(0u, 0u, 0u, 0u);
    };

    // four tokens of dequantised values, token-major pairs -> per-channel h4 -> four instructions
    auto contract = [&](const uint32_t (*kh)[4], const uint4 *wv, int half) {
        uint32_t b[CPL][2];
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            b[2 * p][0] = __builtin_amdgcn_perm(kh[p][1], kh[p][0], 0x05040100u);
            b[2 * p][1] = __builtin_amdgcn_perm(kh[p][3], kh[p][2], 0x05040100u);
            b[2 * p + 1][0] = __builtin_amdgcn_perm(kh[p][1], kh[p][0], 0x07060302u);
            b[2 * p + 1][1] = __builtin_amdgcn_perm(kh[p][3], kh[p][2], 0x07060302u);
        }
#pragma unroll
        for (int n = 0; n < NB; n++) {
            const h4v a = half ? as_h4(wv[n].z, wv[n].w) : as_h4(wv[n].x, wv[n].y);
#pragma unroll
            for (int c = 0; c < CPL; c++)
                acc[n][c] = __builtin_amdgcn_mfma_f32_4x4x4f16(a, as_h4(b[c][0], b[c][1]), acc[n][c], 0, 0, 0);
        }
    };
    uint32_t kh[G::NP][4];
    Lookups<BITS> lk;
    auto token = [&](int t, const uint32_t (*nbnext)[2], int next_half) {
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            Pair &s = st[p];
            h2 qc, qa;
            lk.get(p, t, qc, qa);
            const h2 qs = qc * s.sc;
            kh[p][t & 3] = as_u32(qs + s.zp);
            update_pair_abs(s, qa, qs);
        }
        lk.refill(lut, nbnext, lane_copy, t, next_half);
        __builtin_amdgcn_sched_barrier(0);
    };

    uint4 buf[GPF];
    uint4 wbuf[WPF][NB];
    uint32_t nbc[G::NP][2], nbn[G::NP][2];
#pragma unroll
    for (int i = 0; i < GPF; i++)
        buf[i] = (i < nfull) ? load_codes(cb + (size_t)i * G::VPS) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < WPF; i++)
#pragma unroll
        for (int n = 0; n < NB; n++)
            wbuf[i][n] = (i < nunits) ? load_w(n, i) : make_uint4(0, 0, 0, 0);
    if (nfull > 0) {
        code_bytes<BITS>(buf[0], nbc);
        lk.fill(lut, nbc, lane_copy, 0);
    }
    // one supergroup, nothing conditional in it; i = its buffer in the rotation
    auto body = [&](int sg, auto ic) {
        constexpr int i = decltype(ic)::value;
        code_bytes<BITS>(buf[(i + 1) % GPF], nbn);
        buf[i] = load_codes(cb + (size_t)min(sg + GPF, nfull - 1) * G::VPS); // unconditional: see qk_gqa_kernel
#pragma unroll
        for (int hf = 0; hf < UPS; hf++) {
            const int unit = sg * UPS + hf;
            const int ws = (i * UPS + hf) % WPF; // compile-time after unrolling
            __builtin_amdgcn_sched_barrier(0);
            const bool into_next_sg = hf == UPS - 1;
#pragma unroll
            for (int t = 0; t < 4; t++)
                token(t, into_next_sg ? nbn : nbc, into_next_sg ? 0 : hf + 1);
            contract(kh, wbuf[ws], 0);
#pragma unroll
            for (int t = 4; t < 8; t++)
                token(t, into_next_sg ? nbn : nbc, into_next_sg ? 0 : hf + 1);
            contract(kh, wbuf[ws], 1);
            // reloaded once used: an earlier load into a second register set costs copies at the
            // loop edge, which wait for the load they move
#pragma unroll
            for (int n = 0; n < NB; n++)
                wbuf[ws][n] = load_w(n, min(unit + WPF, nunits - 1));
        }
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            nbc[p][0] = nbn[p][0];
            nbc[p][1] = nbn[p][1];
        }
    };
    rotate_over<GPF>(nfull, body);

    if (last) {
        // ragged tail, then the appended token: a handful of tokens, plain fp32 multiply-adds
        auto add_token = [&](const h2 *vd, int t) {
#pragma unroll
            for (int g = 0; g < GQ; g++) {
                const float wt = (float)attn[((size_t)bx * GQ + g) * sa.row_pitch + t];
#pragma unroll
                for (int p = 0; p < G::NP; p++) {
                    acc[g >> 2][2 * p][g & 3] = __builtin_fmaf(wt, (float)vd[p].x, acc[g >> 2][2 * p][g & 3]);
                    acc[g >> 2][2 * p + 1][g & 3] =
                        __builtin_fmaf(wt, (float)vd[p].y, acc[g >> 2][2 * p + 1][g & 3]);
                }
            }
        };
        const int ntail = (t1 - t0) % TPW;
        if (ntail) {
            const uint4 u = cb[(size_t)nfull * G::VPS];
            const uint32_t w[4] = {u.x, u.y, u.z, u.w};
            for (int tt = 0; tt < ntail; tt++) {
                h2 vd[2];
#pragma unroll
                for (int pp = 0; pp < 2; pp++) {
                    Pair &s = st[pp];
                    const h2 qc = extract_pair<BITS>(w[2 * pp], w[2 * pp + 1], tt);
                    const h2 qs = qc * s.sc;
                    vd[pp] = qs + s.zp;
                    update_pair(s, qc, qs);
                }
                add_token(vd, t0 + nfull * TPW + tt);
            }
        }
        if (active)
            publish_state<D, CPL>(st, state_out, sa, bx, c0, T);
        h2 deq[G::NP];
        append_new_token<D, CPL, BITS>(cbh, T, v_new + (size_t)bx * D + c0, st, deq, active, sa.act_bf16);
        add_token(deq, T);
    }
    if (!active)
        return;
#pragma unroll
    for (int g = 0; g < GQ; g++) {
        const size_t row = (size_t)bx * GQ + g;
        const float o0 = acc[g >> 2][0][g & 3], o1 = acc[g >> 2][1][g & 3];
        const float o2 = acc[g >> 2][2][g & 3], o3 = acc[g >> 2][3][g & 3];
        if (sa.nseg == 1) {
            store_act2(out + row * D + c0, o0, o1, sa.act_bf16);
            store_act2(out + row * D + c0 + 2, o2, o3, sa.act_bf16);
        } else {
            *reinterpret_cast<float4 *>(partial + ((size_t)un.seg * BH * GQ + row) * D + c0) =
                make_float4(o0, o1, o2, o3);
        }
    }
}

} // namespace adkv
