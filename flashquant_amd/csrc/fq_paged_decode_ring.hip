// Split-K paged decode, ring form: groups of 8 KV heads of dimension 128, TQ4 pages, gfx950.
//
// Operator and page layout as in fq_paged_decode.hip (paged_decode_reference,
// src/flashquant/kernels/cpu_reference.py:230-368; token row
// [K idx H*64 | K norm H*4 | V idx H*64 | V norm H*4], src/flashquant/vllm/impl.py:132-138).
//
// One workgroup of 16 wavefronts per (sequence, split, group of 8 KV heads).  All 16 compute:
// wavefront w works on KV head w % 8 and on the 16-token block w / 8 of every 32 tokens, so a
// SIMD holds four wavefronts whose dependent chains (operand bytes -> table lookups -> MFMA ->
// softmax -> lookups -> MFMA) overlap each other.  No wavefront copies through registers:
// the token rows go from the cache straight into LDS with global_load_lds_dwordx4, every
// wavefront issuing its share (two or three 1 KB requests per 32 tokens), into a ring of five
// 16-token stages (three stages on their way while two are worked on).  A wavefront waits for
// its own requests by count (s_waitcnt vmcnt) and the workgroup meets at one barrier per 32
// tokens; nothing else synchronises.
//
// LDS image of a stage: the 16 token rows of the group as they lie in the cache (1088 bytes
// each), cut into 1 KB blocks; inside a block the 16-byte chunk p sits at p ^ ((p >> 3) & 3).
// A direct-to-LDS request writes 64 consecutive chunks (lane l -> chunk l of the block), so the
// swizzle is applied on the source side: lane l fetches chunk l ^ ((l >> 3) & 3) of the block's
// 1 KB of cache, which is still eight whole 128-byte lines per request.  With it the K operand
// reads (16 bytes of row n, quarter g), the V operand reads (dword n of rows 4g + i) and the
// norm reads are free of bank conflicts for every head.
//
// Arithmetic per 16-token block as in the staged kernel, on half the tile: scores
// S^T = K (16 tokens x 128) . Q^T (128 x 16 columns) on v_mfma_f32_16x16x32_f16, the 16 columns
// carrying (query head, copy); a lane keeps the scores of its copy's tokens, so all lanes own
// distinct (head, token) pairs; weights w * |v| in fp16 as the A operand of
// v_mfma_f32_16x16x16_f16 against V (tokens x coordinates) dequantised with one lookup per
// byte after a 2x2 nibble transpose of token pairs.  The two wavefronts of a KV head merge
// their partial results through LDS at the end and publish one partial per split.

#include <cstdio>
#include <cstdlib>

#include "fq_paged_decode.hpp"

namespace fq {

constexpr int kRingRowBytes = 1088;                 // 8 KV heads x 136
constexpr int kRingStageBytes = 16 * kRingRowBytes;   // 17408 = 17 blocks of 1 KB

// LDS byte offset, inside a stage, of byte `byte` of token row `row`.
__host__ __device__ constexpr int ring_off(int row, int byte) {
    const int L = row * kRingRowBytes + byte;
    const int c = L >> 4, pos = c & 63;
    return ((c >> 6) << 10) | ((pos ^ ((pos >> 3) & 3)) << 4) | (L & 15);
}

// Byte offset, from the base of the stage's first page, of chunk `cc` (0 .. 1087) of the 16 rows
// that head group `hgrp` sees: with 8 KV heads the rows themselves, with more the group's slices
// of the four sections of each row laid end to end.  RPP = rows of a stage that lie in one page
// (16, or 8 with 8-token pages: the stage's second half comes from the next page, `second`).
template <int RPP>
__device__ __forceinline__ uint32_t ring_src_offset(int cc, int H, int hgrp, bool& second) {
    const int r = cc / 68, ci = cc - r * 68;
    second = r >= RPP;
    const int rr = r >= RPP ? r - RPP : r;
    int off;
    if (ci < 32) off = 512 * hgrp + 16 * ci;                               // K indices
    else if (ci < 34) off = H * 64 + 32 * hgrp + 16 * (ci - 32);           // K norms
    else if (ci < 66) off = H * 68 + 512 * hgrp + 16 * (ci - 34);          // V indices
    else off = H * 132 + 32 * hgrp + 16 * (ci - 66);                       // V norms
    return uint32_t(rr * (H * 136) + off);
}

// The 64 KB pair table (K in the lower, V in the upper 128 bytes of every 256-byte row, 32 copies
// each) filled by 16 wavefronts: wavefront w writes the rows of the bytes 16 i + w.
__device__ __forceinline__ void fill_pair_tables16(uint32_t* table, float mine_k, float mine_v, int wave, int lane) {
    const int hk = int(__builtin_bit_cast(uint16_t, _Float16(mine_k)));
    const int hv = int(__builtin_bit_cast(uint16_t, _Float16(mine_v)));
    // the low nibble of this wavefront's bytes is `wave`: the high half of every entry
    const uint32_t klo = uint32_t(__builtin_amdgcn_readlane(hk, wave)) << 16;
    const uint32_t vlo = uint32_t(__builtin_amdgcn_readlane(hv, wave)) << 16;
    uint32_t* mine = table + lane + 64 * wave;
#pragma unroll
    for (int hi = 0; hi < 16; ++hi) {
        const uint32_t ke = uint32_t(__builtin_amdgcn_readlane(hk, hi)) | klo;
        const uint32_t ve = uint32_t(__builtin_amdgcn_readlane(hv, hi)) | vlo;
        mine[64 * 16 * hi] = lane < 32 ? ke : ve;
    }
}

// One codebook for keys and values: a single table of 128-byte rows (32 copies of the entry of a byte),
// 32 KB, which leaves LDS for seven stages instead of five.  The address of a lookup is then
// (byte << 7) | copy offset: a bit-field extract and a shift-or instead of the one v_perm_b32 that
// splices whole bytes.  Wavefront `wave` of `waves` (8 or 16) fills the rows of its share of the bytes,
// two rows per store (lanes 0..31 one byte, lanes 32..63 the next).
__device__ __forceinline__ void fill_shared_table(uint32_t* table, float mine, int wave, int waves, int lane) {
    const int hc = int(__builtin_bit_cast(uint16_t, _Float16(mine)));   // lane l: fp16 centroid l % 16
    // bytes whose low nibble is `wave` (and `wave` + 8 when 8 wavefronts fill): the entry's high half is
    // that nibble's centroid, a scalar; the high nibble 2i / 2i + 1 goes by lane half
    uint32_t* mine_row = table + (lane & 31) + 32 * 16 * (lane >> 5);
    for (int lo = wave; lo < 16; lo += waves) {
        const uint32_t hi_half = uint32_t(__builtin_amdgcn_readlane(hc, lo)) << 16;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t a = uint32_t(__builtin_amdgcn_readlane(hc, 2 * i)), b = uint32_t(__builtin_amdgcn_readlane(hc, 2 * i + 1));
            mine_row[(32 * i + lo) * 32] = (lane < 32 ? a : b) | hi_half;     // byte = 16 (2i + lane / 32) + lo
        }
    }
}
template <int K>
__device__ __forceinline__ uint32_t lut_addr_shared(uint32_t w, uint32_t lane_off) {
    return (__builtin_amdgcn_ubfe(w, 8 * K, 8) << 7) | lane_off;
}

// RING = stages of the ring: 7 with the shared 32 KB table, 5 with the 64 KB pair of tables.
template <int BSL, int GP, int DT, int PVR, int RING>
__global__ __launch_bounds__(1024) void paged_decode_ring_kernel(const DecodeParams p) {
    constexpr bool kShared = RING == 7;
    constexpr int kRingStages = RING;
    constexpr int BS = 1 << BSL;
    constexpr int D = 128;
    constexpr int KS = 4;                 // k-steps of the score product
    constexpr int DPL = 8;                // V coordinates per lane
    constexpr int NSC = GP / 4;           // scores a lane keeps per 16-token block
    constexpr int STAGE = kRingStageBytes;
    constexpr int RPP = BS >= 16 ? 16 : 8;   // rows of a stage that lie in one page

    __shared__ __attribute__((aligned(256))) uint32_t lut[kShared ? kLutWords / 2 : kLutWords];
    extern __shared__ __attribute__((aligned(1024))) uint8_t ring[];   // kRingStages stages

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = wv & 7;                 // KV head inside the group
    const int half = wv >> 3;             // which 16 tokens of every 32
    const int n = lane & 15;
    const int g = lane >> 4;
    const int hd = n % GP;                // query head inside the GQA group
    const int cls = n / GP;               // copy of the head among the 16 columns
    int seq = blockIdx.x;
    int split = blockIdx.y;
    const int hgrp = blockIdx.z;
    const int HQG = 8 * p.G;              // query heads of the group
    const int hq0 = hgrp * HQG;
    const int row_bytes = p.H_KV * 136;

    // Timing instrumentation, compiled in with -DFQ_RING_TIMING only: `dbg` is then a bit set given
    // with the launch (1: no arithmetic, 2: no requests in the loop, 4: time stamps of the
    // prologue, 8: of the iterations), otherwise a constant 0 that removes all of it.
#ifdef FQ_RING_TIMING
    const int dbg = p.spin_limit;
#else
    constexpr int dbg = 0;
#endif
    unsigned long long stamps[12];
    auto stamp = [&](int k) { if (dbg & 4) stamps[k] = wall_clock64(); };
    stamp(0);
    // ---- loads that depend on nothing ------------------------------------------------------
    // Wavefronts 8..15 rotate the query heads (wavefront 8 + h: columns 16h .. 16h + 15 of every
    // head) and ask for the matrix and the first 32 heads before anything else; wavefronts 0..7,
    // which are launched first, have their sequence length and page ids in the memory pipeline by
    // then.  The matrix loads (64 KB per workgroup, 16 bytes per lane) keep the pipeline busy for
    // over a microsecond: whatever is asked for behind them waits that long, so the wavefronts
    // that make the first token requests must not be the ones that queue up behind them.
    const bool rotates = p.rotation != nullptr && half == 1;
    // Which 16 columns this wavefront produces changes from workgroup to workgroup: the workgroups
    // that share an L2 (every eighth one) would otherwise all walk the matrix in the same order at
    // the same time and queue up at one L2 channel after the other.
    const int cb = (h + ((int(blockIdx.x) + int(gridDim.x) * int(blockIdx.y)) >> 3)) & 7;
    float rot_b[4][8];
    uint4v q_pre[2][4];
    if (rotates && p.balance_slots == 0) {
        const int HQG0 = 8 * p.G;
        const uint16_t* qs0 = reinterpret_cast<const uint16_t*>(p.q_rot) + (int64_t(blockIdx.x) * p.H_Q + int(blockIdx.z) * HQG0) * 128;
        load_rotation_any<128>(p.rotation, p.rot_col_major != 0, true, 16 * cb, n, g, rot_b);
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            const int row = 16 * rb + n < HQG0 ? 16 * rb + n : HQG0 - 1;
#pragma unroll
            for (int j = 0; j < 4; ++j) q_pre[rb][j] = *reinterpret_cast<const uint4v*>(qs0 + row * 128 + 32 * j + 8 * g);
        }
    }
    const float cent_k_mine = p.centroids_k[lane & 15];
    const float cent_v_mine = p.centroids_v[lane & 15];
    const uint8_t* lut_k = reinterpret_cast<const uint8_t*>(lut);
    const uint32_t lane_off = 4u * (lane & 31);
    const uint32_t lane_off_v = kShared ? lane_off : 128u + lane_off;

    const int NS = p.num_splits;
    const bool rowwide = p.max_blocks <= 64 * PVR;
    int chunk = (((p.max_blocks * BS + NS - 1) / NS) + 63) & ~63;
    int L_known = -1;
    if (p.balance_slots > 0) {
        balance_chunks<PVR, BS, 1>(p, lane, NS, rowwide, chunk, seq, split, L_known);
        // the same in every lane: kept in scalar registers from here on
        chunk = __builtin_amdgcn_readfirstlane(chunk);
        seq = __builtin_amdgcn_readfirstlane(seq);
        split = __builtin_amdgcn_readfirstlane(split);
        L_known = __builtin_amdgcn_readfirstlane(L_known);
    }

    const int32_t* bt = p.block_table + int64_t(seq) * p.max_blocks;
    int pv[PVR];
#pragma unroll
    for (int r = 0; r < PVR; ++r) pv[r] = 0;
    if (rowwide) {
#pragma unroll
        for (int r = 0; r < PVR; ++r) {
            const int idx = 64 * r + lane < p.max_blocks ? 64 * r + lane : p.max_blocks - 1;
            pv[r] = bt[idx];
        }
    }
    int L = L_known;
    if (L_known < 0) L = p.seq_lens[seq];

    const uint16_t* qseq = reinterpret_cast<const uint16_t*>(p.q_rot) + (int64_t(seq) * p.H_Q + hq0) * D;
    if (rotates && p.balance_slots != 0) {
        // (the sequence of a rebalanced workgroup is known only now)
        load_rotation_any<D>(p.rotation, p.rot_col_major != 0, true, 16 * cb, n, g, rot_b);
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            const int row = 16 * rb + n < HQG ? 16 * rb + n : HQG - 1;
#pragma unroll
            for (int j = 0; j < 4; ++j) q_pre[rb][j] = *reinterpret_cast<const uint4v*>(qseq + row * D + 32 * j + 8 * g);
        }
    }

    // ---- lane constants (worked out while the loads are on their way) ---------------------------
    // source of this wavefront's requests: blocks wv (first stage of a pair), (wv + 15) % 16 (second
    // stage), and block 16 of the first stage for wavefront 0, of the second for wavefront 1
    const int blk_a = wv, blk_b = (wv + 15) & 15;
    const int swz = lane ^ ((lane >> 3) & 3);
    uint32_t src_a, src_b, src_x, src_p;
    bool sec_a, sec_b, sec_x, sec_p;
    src_a = ring_src_offset<RPP>(64 * blk_a + swz, p.H_KV, hgrp, sec_a);
    src_b = ring_src_offset<RPP>(64 * blk_b + swz, p.H_KV, hgrp, sec_b);
    src_x = ring_src_offset<RPP>(64 * 16 + swz, p.H_KV, hgrp, sec_x);
    src_p = ring_src_offset<RPP>(64 * (h + 8) + swz, p.H_KV, hgrp, sec_p);   // first requests: blocks h, h + 8
    // operand reads inside a stage
    const int k_rd = ring_off(n, 64 * h + 16 * g);
    int v_rd[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v_rd[i] = ring_off(4 * g + i, 544 + 64 * h + 4 * n);
    int sc_row[NSC], kn_rd[NSC], vn_rd[NSC];
#pragma unroll
    for (int e = 0; e < NSC; ++e) {
        sc_row[e] = 4 * g + (GP == 4 ? cls : (GP == 8 ? 2 * cls + e : e));
        kn_rd[e] = ring_off(sc_row[e], 512 + 4 * h);
        vn_rd[e] = ring_off(sc_row[e], 1056 + 4 * h);
    }
    // (each offset is one register: the compiler is not to keep its pieces apart and add them per use)
    int k_rd_v = k_rd;
    asm volatile("" : "+v"(k_rd_v));
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(v_rd[i]));
#pragma unroll
    for (int e = 0; e < NSC; ++e) {
        asm volatile("" : "+v"(kn_rd[e]));
        asm volatile("" : "+v"(vn_rd[e]));
    }
    // the P operand holds the weights of tokens 4g .. 4g + 3 for column n: this lane's copy owns
    // token cls (GP = 4), tokens 2 cls, 2 cls + 1 (GP = 8), all four (GP = 16)
    uint32_t pa_mask[2];
    if (GP == 4) {
        pa_mask[0] = cls == 0 ? 0x0000ffffu : (cls == 1 ? 0xffff0000u : 0u);
        pa_mask[1] = cls == 2 ? 0x0000ffffu : (cls == 3 ? 0xffff0000u : 0u);
    } else if (GP == 8) {
        pa_mask[0] = cls == 0 ? 0xffffffffu : 0u;
        pa_mask[1] = cls == 1 ? 0xffffffffu : 0u;
    } else {
        pa_mask[0] = pa_mask[1] = 0xffffffffu;
    }

    __builtin_amdgcn_sched_barrier(0);
    L = __builtin_amdgcn_readfirstlane(L);   // one value per workgroup: everything derived from it is scalar
    L = L < 0 ? 0 : L;
    L = L > p.max_blocks * BS ? p.max_blocks * BS : L;
    const int begin = split * chunk;
    const int end = L < begin + chunk ? L : begin + chunk;
    const int hq_lane = h * p.G + n;
    if (begin >= end) {   // uniform over the workgroup
        if (half == 0 && g == 0 && n < p.G) {
            const int64_t o = (int64_t(seq) * p.H_Q + hq0 + hq_lane) * NS + split;
            p.part_m[o] = -__builtin_inff();
            p.part_l[o] = 0.0f;
        }
        return;
    }
    stamp(1);
    const int last_page_idx = (L - 1) >> BSL;
    const int max_page = p.num_blocks - 1;
    const uint8_t* cache = p.cache;
    const int64_t page_bytes = int64_t(BS) * row_bytes;

    const int split_p0 = rowwide ? 0 : begin >> BSL;   // page index held by lane 0 of pv[0]
    if (!rowwide) {
#pragma unroll
        for (int r = 0; r < PVR; ++r) {
            int idx = split_p0 + 64 * r + lane;
            idx = idx > last_page_idx ? last_page_idx : idx;
            pv[r] = bt[idx];
        }
    }
    auto page_id = [&](int rel) -> int {
        int v = __builtin_amdgcn_readlane(pv[0], rel & 63);
#pragma unroll
        for (int r = 1; r < PVR; ++r) {
            const int vr = __builtin_amdgcn_readlane(pv[r], rel & 63);
            v = (rel >> 6) == r ? vr : v;
        }
        return v;
    };
    // the tables are filled while the page ids are on their way: by all 16 wavefronts, or by
    // wavefronts 8..15 where the first eight have the rotation to do
    if constexpr (kShared) {
        if (p.rotation == nullptr) fill_shared_table(lut, cent_k_mine, wv, 16, lane);
        else if (half == 0) fill_shared_table(lut, cent_k_mine, h, 8, lane);
    } else {
        if (p.rotation == nullptr) fill_pair_tables16(lut, cent_k_mine, cent_v_mine, wv, lane);
        else if (half == 0) fill_pair_tables<8>(lut, cent_k_mine, cent_v_mine, 15, h, lane);
    }
#pragma unroll
    for (int r = 0; r < PVR; ++r) pv[r] = pv[r] < 0 ? 0 : (pv[r] > max_page ? max_page : pv[r]);

    // ---- requests ---------------------------------------------------------------------------
    const int nstages = (end - begin + 15) >> 4;
    // one 1 KB block of stage `st` (0-based inside the split) into its ring slot
    auto request = [&](int st, int blk, uint32_t src, bool second) {
        const int t0 = begin + 16 * st;
        const int p0 = (t0 >> BSL) - split_p0;
        const uint8_t* base = cache + int64_t(page_id(p0)) * page_bytes + (BS == 32 ? (t0 & 16) * row_bytes : 0);
        const uint8_t* g_src = base + src;
        if constexpr (BS == 8) {
            // the second page of a stage past the sequence's last page is never read: its rows are masked
            int p1 = p0 + 1;
            p1 = p1 + split_p0 > last_page_idx ? p0 : p1;
            const uint8_t* base1 = cache + int64_t(page_id(p1)) * page_bytes;
            g_src = second ? base1 + src : g_src;
        }
        uint8_t* dst = ring + (st % kRingStages) * STAGE + blk * 1024;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g_src,
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    };
    // first stage of a pair: block wv, and block 16 from wavefront 0; second stage: block
    // (wv + 15) % 16, and block 16 from wavefront 1.  Stages past the split's end are not asked for.
    auto request_first = [&](int st) {
        if (st < nstages) {
            request(st, blk_a, src_a, sec_a);
            if (wv == 0) request(st, 16, src_x, sec_x);
        }
    };
    auto request_second = [&](int st) {
        if (st < nstages) {
            request(st, blk_b, src_b, sec_b);
            if (wv == 1) request(st, 16, src_x, sec_x);
        }
    };
    // The first stages are asked for by wavefronts 0..7 alone (blocks h and h + 8, block 16 from
    // wavefront 0), which know the page ids first; in the tile loop all 16 share the requests.  With
    // at most 32 query heads the rotated heads are exchanged beside the ring and all five stages
    // are asked for now; with more they pass through the last two stages, which are asked for in
    // the first iteration.
    constexpr bool kAllUpfront = false;
    constexpr int kFirstStages = kAllUpfront ? kRingStages : kRingStages - 2;
    stamp(2);
    if (half == 0) {
#pragma unroll
        for (int st = 0; st < kFirstStages; ++st) {
            if (st < nstages) {
                request(st, h, src_a, sec_a);
                request(st, h + 8, src_p, sec_p);
                if (wv == 0) request(st, 16, src_x, sec_x);
            }
        }
    }
    stamp(3);

    // ---- query operand ------------------------------------------------------------------------
    // With a rotation matrix the workgroup first rotates all query heads of its group: wavefront
    // (h, half) produces columns 16h .. 16h + 15 of q_rot = (q @ R.T) for the heads of the row blocks
    // half, half + 2, ..., rounded to the query dtype as the reference rounds it, and the heads are
    // exchanged through the last two ring stages, which receive no tokens before the first barrier
    // of the tile loop.
    half8 qh[KS];
    float qscale;
    {
        float qf[KS][8];
        float mx = 0.0f;
        const bool live = hd < p.G;
        uint4v qraw[KS];
        if (p.rotation != nullptr) {
            uint16_t* qs = reinterpret_cast<uint16_t*>(ring + (kAllUpfront ? kRingStages : kRingStages - 2) * STAGE);
            if (rotates) {
                constexpr bool kRawBf16 = DT == FQ_BF16;
                half8 rot_hi[KS], rot_lo[KS];
                bf16v8 rot_t[3][KS];
                if constexpr (kRawBf16) split_rotation_block_bf16_packed<D>(rot_b, rot_t);
                else split_rotation_block<D>(rot_b, rot_hi, rot_lo);
                stamp(7);
                auto rotate_rows = [&](int rb, const uint4v (&raw)[KS]) {
                    float4v acc;
                    float up = 1.0f;
                    if constexpr (kRawBf16) {
                        bf16v8 a[KS];
#pragma unroll
                        for (int j = 0; j < KS; ++j) a[j] = __builtin_bit_cast(bf16v8, raw[j]);
                        acc = rotate_block_bf16<D>(a, rot_t);
                    } else {
                        half8 a[KS];
                        rows_as_f16<D, DT>(raw, a, up);
                        acc = rotate_block_f16<D>(a, rot_hi, rot_lo);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int head = 16 * rb + 4 * g + i;
                        if (head < HQG) qs[head * D + 16 * cb + n] = store_elem<DT>(acc[i] * up);
                    }
                };
                // the first two row blocks outside the loop: their operands were asked for before the
                // token rows, and straight-line code lets the wait for them leave the token requests
                // on their way
                rotate_rows(0, q_pre[0]);
                stamp(8);
                if (16 < HQG) rotate_rows(1, q_pre[1]);
                stamp(9);
                for (int rb = 2; 16 * rb < HQG; ++rb) {
                    const int row = 16 * rb + n < HQG ? 16 * rb + n : HQG - 1;
                    uint4v raw[KS];
#pragma unroll
                    for (int j = 0; j < KS; ++j) raw[j] = *reinterpret_cast<const uint4v*>(qseq + row * D + 32 * j + 8 * g);
                    rotate_rows(rb, raw);
                }
            }
            // (a barrier that waits for this wavefront's LDS stores only: the token requests stay in flight)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            stamp(10);
            __builtin_amdgcn_s_barrier();
            stamp(11);
            asm volatile("" ::: "memory");
            // (read here, through a pointer that is known to be LDS: one load site for both sources would
            // be a generic load, and its wait would take in the token requests)
            typedef const __attribute__((address_space(3))) uint4v* lds_u4;
            const uint16_t* src = qs + (h * p.G + (live ? hd : 0)) * D + g * (D / 4);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) qraw[ks] = *(lds_u4)(src + 8 * ks);
            // (waited for inside the branch, as LDS reads)
            asm volatile("" : "+v"(qraw[0]), "+v"(qraw[1]), "+v"(qraw[2]), "+v"(qraw[3]));
        } else {
            const uint16_t* src = qseq + (h * p.G + (live ? hd : 0)) * D + g * (D / 4);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) qraw[ks] = *reinterpret_cast<const uint4v*>(src + 8 * ks);
            asm volatile("" : "+v"(qraw[0]), "+v"(qraw[1]), "+v"(qraw[2]), "+v"(qraw[3]));
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint4v raw = qraw[ks];
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qf[ks][2 * i] = live ? load_elem<DT>(uint16_t(w[i] & 0xffffu)) : 0.0f;
                qf[ks][2 * i + 1] = live ? load_elem<DT>(uint16_t(w[i] >> 16)) : 0.0f;
                mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(qf[ks][2 * i]), __builtin_fabsf(qf[ks][2 * i + 1])));
            }
        }
        mx = max_xor32(max_xor16(mx));
        int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
        if (ex < -100 || ex > 100) ex = 0;
        const float down = bits_to_float(uint32_t(127 - ex) << 23);
        qscale = p.scale_log2e * bits_to_float(uint32_t(127 + ex) << 23);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) qh[ks][e] = _Float16(qf[ks][e] * down);
    }

    stamp(4);
    // ---- running state ---------------------------------------------------------------------
    float4v O[DPL];
#pragma unroll
    for (int db = 0; db < DPL; ++db) O[db] = float4v{0.f, 0.f, 0.f, 0.f};
    float M = -__builtin_inff();
    float lsum = 0.0f;

    // operands of this lane as they lie in the stage: everything a block's arithmetic reads from it
    uint4v kraw;
    uint32_t vraw[4];
    float kn[NSC], vn[NSC];
    auto read_operands = [&](const uint8_t* stage) {
        kraw = *reinterpret_cast<const uint4v*>(stage + k_rd_v);
#pragma unroll
        for (int i = 0; i < 4; ++i) vraw[i] = *reinterpret_cast<const uint32_t*>(stage + v_rd[i]);
#pragma unroll
        for (int e = 0; e < NSC; ++e) {
            kn[e] = *reinterpret_cast<const float*>(stage + kn_rd[e]);
            vn[e] = *reinterpret_cast<const float*>(stage + vn_rd[e]);
        }
    };
    auto compute_block = [&](int t0) {
        // ---- scores ------------------------------------------------------------------------------
        uint4v ka[KS];
        const uint32_t kw[4] = {kraw.x, kraw.y, kraw.z, kraw.w};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if constexpr (kShared) {
                ka[ks].x = lds_word(lut_k, lut_addr_shared<0>(kw[ks], lane_off));
                ka[ks].y = lds_word(lut_k, lut_addr_shared<1>(kw[ks], lane_off));
                ka[ks].z = lds_word(lut_k, lut_addr_shared<2>(kw[ks], lane_off));
                ka[ks].w = lds_word(lut_k, lut_addr_shared<3>(kw[ks], lane_off));
            } else {
                ka[ks] = lookup_word(lut_k, kw[ks], lane_off);
            }
        }
        // nibble transposes of the V token pairs (rows 4g, 4g + 1) and (4g + 2, 4g + 3)
        uint32_t X[2], Y[2];
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            const uint32_t A = vraw[2 * jp], B = vraw[2 * jp + 1];
            X[jp] = (A & 0xF0F0F0F0u) | ((B >> 4) & 0x0F0F0F0Fu);
            Y[jp] = ((A << 4) & 0xF0F0F0F0u) | (B & 0x0F0F0F0Fu);
        }
        uint2v vb[DPL];
        auto v_lookup = [&](int db) {
            const int bi = db >> 1;
            const uint32_t (&s2)[2] = (db & 1) ? Y : X;
            uint2v r;
            auto addr = [&](uint32_t w) {
                if constexpr (kShared)
                    return bi == 0 ? lut_addr_shared<0>(w, lane_off_v) : bi == 1 ? lut_addr_shared<1>(w, lane_off_v)
                         : bi == 2 ? lut_addr_shared<2>(w, lane_off_v) : lut_addr_shared<3>(w, lane_off_v);
                else
                    return bi == 0 ? lut_addr<0>(w, lane_off_v) : bi == 1 ? lut_addr<1>(w, lane_off_v)
                         : bi == 2 ? lut_addr<2>(w, lane_off_v) : lut_addr<3>(w, lane_off_v);
            };
            r.x = lds_word(lut_k, addr(s2[0]));
            r.y = lds_word(lut_k, addr(s2[1]));
            return r;
        };
#pragma unroll
        for (int db = 0; db < DPL; ++db) vb[db] = v_lookup(db);

        float4v acc = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ka[ks]), qh[ks], acc, 0, 0, 0);

        // ---- this lane's scores ------------------------------------------------------------------
        float a_[NSC], rv[NSC];
#pragma unroll
        for (int e = 0; e < NSC; ++e) {
            float s;
            if (GP == 4) {
                const float s01 = (cls & 1) ? acc[1] : acc[0];
                const float s23 = (cls & 1) ? acc[3] : acc[2];
                s = (cls >> 1) ? s23 : s01;
            } else if (GP == 8) {
                s = cls ? acc[2 + e] : acc[e];
            } else {
                s = acc[e];
            }
            // (the products are formed whether the token is live or not: the norm reads then stay up
            // with the operand reads instead of moving behind a branch that follows the MFMAs)
            float sc = s * kn[e] * qscale;
            float vnv = vn[e];
            asm volatile("" : "+v"(sc), "+v"(vnv));
            const bool live = t0 + sc_row[e] < end;
            rv[e] = live ? vnv : 0.0f;
            a_[e] = live ? sc : -__builtin_inff();
        }
        // Weights relative to the reference M the head already has.  M is not the exact running
        // maximum: it moves only when a score leads it by more than 2^16 or a weighted value norm
        // w * |v| would not fit fp16 (the P operand), which one vote over the wavefront finds out.
        // Any reference gives the same softmax as long as numerator and denominator share it.
        float wgt[NSC];
        float psum = 0.0f;
        bool redo = false;
#pragma unroll
        for (int e = 0; e < NSC; ++e) {
            const float d = a_[e] - M;
            const float w = __builtin_amdgcn_exp2f(d);
            psum += w;
            wgt[e] = w * rv[e];
            // (a block may hold no live token for this lane while M is still -inf: -inf - -inf is NaN,
            // and the vote must then send the block through the safe path)
            redo = redo || !(d <= kMaxLead) || wgt[e] > kHalfSafe;
        }
        if (__any(redo)) {
            // The reference moves to max(M, max over the block of (score + bias)), where the bias of a
            // token is the number of binary orders its value norm lies above 2^10: weights then stay
            // below 1 / 2^bias and w * |v| below 2^11 whatever the norms are.
            float tmax = -__builtin_inff();
#pragma unroll
            for (int e = 0; e < NSC; ++e) tmax = __builtin_fmaxf(tmax, a_[e] + norm_bias(rv[e]));
            tmax = max_same_head<GP>(tmax);
            const float Mnew = __builtin_fmaxf(M, tmax);
            const float Ms = Mnew == -__builtin_inff() ? 0.0f : Mnew;
            const float alpha = __builtin_amdgcn_exp2f(M - Ms);   // M = -inf (first block): 0
            M = Mnew;
            psum = 0.0f;
#pragma unroll
            for (int e = 0; e < NSC; ++e) {
                const float w = __builtin_amdgcn_exp2f(a_[e] - Ms);
                psum += w;
                wgt[e] = __builtin_fminf(w * rv[e], kHalfMax);     // only a norm of Inf still reaches the bound
            }
            lsum *= alpha;
            float ar[4];
            if (GP == 4) {
                ar[0] = dpp_mov<0x00>(alpha);
                ar[1] = dpp_mov<0x55>(alpha);
                ar[2] = dpp_mov<0xAA>(alpha);
                ar[3] = dpp_mov<0xFF>(alpha);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) ar[i] = __shfl(alpha, 4 * g + i, kWave);
            }
#pragma unroll
            for (int db = 0; db < DPL; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) O[db][i] *= ar[i];
        }
        lsum += psum;

        // ---- weights as the A operand: slot i <-> token 4g + i --------------------------------------
        uint2v pa_w;
        if (GP == 4) {
            const half2v h2 = {_Float16(wgt[0]), _Float16(wgt[0])};
            const uint32_t pk = __builtin_bit_cast(uint32_t, h2);
            pa_w = uint2v{pk & pa_mask[0], pk & pa_mask[1]};
        } else if (GP == 8) {
            const half2v h2 = {_Float16(wgt[0]), _Float16(wgt[1 % NSC])};
            const uint32_t pk = __builtin_bit_cast(uint32_t, h2);
            pa_w = uint2v{pk & pa_mask[0], pk & pa_mask[1]};
        } else {
            const half2v h01 = {_Float16(wgt[0]), _Float16(wgt[1 % NSC])};
            const half2v h23 = {_Float16(wgt[2 % NSC]), _Float16(wgt[3 % NSC])};
            pa_w = uint2v{__builtin_bit_cast(uint32_t, h01), __builtin_bit_cast(uint32_t, h23)};
        }
        const half4 pa = __builtin_bit_cast(half4, pa_w);
#pragma unroll
        for (int db = 0; db < DPL; ++db)
            O[db] = __builtin_amdgcn_mfma_f32_16x16x16f16(pa, __builtin_bit_cast(half4, vb[db]), O[db], 0, 0, 0);
    };

    // ---- tiles of 32 tokens: stages 2j (wavefronts 0..7) and 2j + 1 (wavefronts 8..15) ---------------
    // One barrier per iteration: behind it the two stages are complete (every wavefront has waited
    // for its own requests by count), and the stages of the iteration before, whose operands have
    // long been read, are asked for again: stage 2j + 3 (block wv, and block 16 from wavefront 0)
    // and stage 2j + 4 (block (wv + 15) % 16, and block 16 from wavefront 1).  At the top of
    // iteration j the requests that may still be on their way are those of the stages from 2j + 2
    // on: of the first stages (two or three per stage, wavefronts 0..7 only) while they last, then
    // the one or two of stage 2j + 2.
    const int iters = (nstages + 1) >> 1;
    const int n_first = half == 0 ? (wv == 0 ? 3 : 2) : 0;
    const int n_odd = wv == 0 ? 2 : 1, n_even = wv == 1 ? 2 : 1;
    int slot = half;                      // ring slot of stage 2j + half
    for (int j = 0; j < iters; ++j) {
        // (the common case first, in two scalar branches: the three, or the one, stages ahead are all
        // pairs of earlier iterations and all exist)
        if (2 * j + 2 >= kFirstStages && 2 * j + kRingStages - 3 <= nstages - 1) {
            if constexpr (kRingStages == 7) {
                if (wv == 0) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
                else if (wv == 1) asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
            } else {
                if (wv == 1) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(1) lgkmcnt(0)" ::: "memory");
            }
        } else {
            // asked for so far: the first stages, and the pairs of the iterations before this one
            int top = j > 0 ? 2 * j + kRingStages - 3 : -1;
            top = top < kFirstStages - 1 ? kFirstStages - 1 : top;
            top = top < nstages - 1 ? top : nstages - 1;
            int allowed = 0;
            for (int st = 2 * j + 2; st <= top; ++st) allowed += st < kFirstStages ? n_first : ((st & 1) ? n_odd : n_even);
#define FQ_WAIT_CASE(N) case N: asm volatile("s_waitcnt vmcnt(" #N ") lgkmcnt(0)" ::: "memory"); break;
            switch (allowed) {
                FQ_WAIT_CASE(0) FQ_WAIT_CASE(1) FQ_WAIT_CASE(2) FQ_WAIT_CASE(3) FQ_WAIT_CASE(4) FQ_WAIT_CASE(5)
                FQ_WAIT_CASE(6) FQ_WAIT_CASE(7) FQ_WAIT_CASE(8) FQ_WAIT_CASE(9) FQ_WAIT_CASE(10) FQ_WAIT_CASE(11)
                FQ_WAIT_CASE(12) FQ_WAIT_CASE(13) FQ_WAIT_CASE(14) FQ_WAIT_CASE(15)
                default: asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); break;
            }
#undef FQ_WAIT_CASE
        }
        if ((dbg & 8) && lane == 0 && j < 32)
            reinterpret_cast<unsigned long long*>(ring + kRingStages * STAGE)[(wv * 32 + j) * 3] = wall_clock64();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if ((dbg & 8) && lane == 0 && j < 32)
            reinterpret_cast<unsigned long long*>(ring + kRingStages * STAGE)[(wv * 32 + j) * 3 + 1] = wall_clock64();
        // the requests of this iteration: the stages of the iteration before, which every wavefront
        // left before the barrier above, asked for again
        if (!(dbg & 2) && 2 * j + kRingStages - 2 >= kFirstStages) {
            request_first(2 * j + kRingStages - 2);
            request_second(2 * j + kRingStages - 1);
        }
        const int st = 2 * j + half;
        if (st < nstages && !(dbg & 1)) {
            read_operands(ring + slot * STAGE);
            compute_block(begin + 16 * st);
        }
        if ((dbg & 8) && lane == 0 && j < 32)
            reinterpret_cast<unsigned long long*>(ring + kRingStages * STAGE)[(wv * 32 + j) * 3 + 2] = wall_clock64();
        slot += 2;
        slot = slot >= kRingStages ? slot - kRingStages : slot;
    }

    stamp(5);
    if ((dbg & 8) && (wv == 0 || wv == 8) && lane < 48) {
        const unsigned long long* src = reinterpret_cast<const unsigned long long*>(ring + kRingStages * STAGE) + wv * 96;
        unsigned long long* dst = reinterpret_cast<unsigned long long*>(const_cast<float*>(p.sketch)) + 65536 +
                                  ((blockIdx.x + gridDim.x * blockIdx.y) * 2 + half) * 96;
        dst[lane] = src[lane];
        dst[lane + 48] = src[lane + 48];
    }
    // ---- publish the partial of this split ---------------------------------------------------------
    // A wavefront's accumulators are 16 rows (query head, copy) of 128 coordinates.  All 16
    // wavefronts write theirs to LDS (the tables and the ring are free now: 128 KB from LDS address
    // 0), with the reference and the denominator of each of their heads, and the workgroup then
    // adds up, per (KV head, query head, coordinate), the copies of both wavefronts of the head,
    // each wavefront's share scaled to the common reference: no sums across lanes.
    auto sum_xor = [](float v, int mask) {
        return mask == 16 ? sum_xor16(v) : (mask == 32 ? sum_xor32(v) : v + xor_shuffle(v, mask));
    };
#pragma unroll
    for (int mask = GP; mask < 64; mask <<= 1) lsum = sum_xor(lsum, mask);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();         // every wavefront is done with the tables and the ring
    asm volatile("" ::: "memory");
    float* obuf = reinterpret_cast<float*>(lut);                 // [16 wavefronts][16 rows][128]
    float* mlbuf = obuf + 16 * 16 * D;                           // [16 wavefronts][16 heads][2]
    {
        float* mine = obuf + (wv * 16 + 4 * g) * D + n * DPL;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int q4 = 0; q4 < 2; ++q4)
                *reinterpret_cast<float4v*>(mine + i * D + 4 * q4) =
                    float4v{O[4 * q4][i], O[4 * q4 + 1][i], O[4 * q4 + 2][i], O[4 * q4 + 3][i]};
        if (g == 0 && n < GP) {
            mlbuf[(wv * 16 + n) * 2] = M;
            mlbuf[(wv * 16 + n) * 2 + 1] = lsum;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    stamp(6);
    if ((dbg & 4) && lane == 0) {
        unsigned long long* dbg = reinterpret_cast<unsigned long long*>(const_cast<float*>(p.sketch)) +
                                  ((blockIdx.x + gridDim.x * blockIdx.y) * 16 + wv) * 12;
        for (int k = 0; k < 12; ++k) dbg[k] = stamps[k];
    }
    const int items = 8 * p.G * (D / 4);  // (KV head, query head of its group, four coordinates)
    for (int item = tid; item < items; item += 1024) {
        const int c4 = item & 31;
        const int hq = item >> 5;         // KV head * G + query head
        const int kvh = hq / p.G, qhd = hq - kvh * p.G;
        float mh[2], lh[2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            mh[hf] = mlbuf[((kvh + 8 * hf) * 16 + qhd) * 2];
            lh[hf] = mlbuf[((kvh + 8 * hf) * 16 + qhd) * 2 + 1];
        }
        const float Mstar = __builtin_fmaxf(mh[0], mh[1]);
        const float Ms = Mstar == -__builtin_inff() ? 0.0f : Mstar;
        float4v acc = {0.f, 0.f, 0.f, 0.f};
        float den = 0.0f;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const float w = __builtin_amdgcn_exp2f(mh[hf] - Ms);      // -inf -> 0
            float4v part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < 16 / GP; ++c)
                part += *reinterpret_cast<const float4v*>(obuf + ((kvh + 8 * hf) * 16 + qhd + GP * c) * D + 4 * c4);
            acc += part * w;
            den += lh[hf] * w;
        }
        const int64_t o = (int64_t(seq) * p.H_Q + hq0 + hq) * NS + split;
        *reinterpret_cast<float4v*>(p.part_acc + o * D + 4 * c4) = acc;
        if (c4 == 0) {
            p.part_m[o] = Mstar;
            p.part_l[o] = den;
        }
    }
}

template <int DT>
static int launch_ring_dt(const DecodeParams& p, int S, int BS, bool wide, hipStream_t stream) {
    // One codebook for keys and values (the reference's serving path, src/flashquant/vllm/impl.py:380-393):
    // the 32 KB table and seven stages.  Behind the ring, the 8 KB through which at most 32 rotated
    // query heads are exchanged.
    // (seven stages measured slower than five on 32 x 4096 tokens: the extra vector instruction per
    // lookup of the 32 KB table costs more than the deeper ring gains; kept for bit 16 of the timing switch)
    const bool shared = p.two_tables == 0 && (p.spin_limit & 16);
    const size_t lds = size_t(shared ? 7 : 5) * kRingStageBytes + (p.G <= 4 ? 8192 : 0);
    const dim3 grid(S, p.num_splits, p.H_KV / 8), block(1024);
#define FQ_RING_PV(BSL, GPV, PVRV)                                                                             \
    return shared ? launch_with_lds(paged_decode_ring_kernel<BSL, GPV, DT, PVRV, 7>, p, grid, block, lds, stream) \
                  : launch_with_lds(paged_decode_ring_kernel<BSL, GPV, DT, PVRV, 5>, p, grid, block, lds, stream)
#define FQ_RING_GP(BSL, GPV)                \
    do {                                    \
        if (wide) { FQ_RING_PV(BSL, GPV, 4); } \
        else { FQ_RING_PV(BSL, GPV, 1); }   \
    } while (0)
#define FQ_RING_BS(BSL)                         \
    do {                                        \
        if (p.G <= 4) { FQ_RING_GP(BSL, 4); }   \
        else if (p.G <= 8) { FQ_RING_GP(BSL, 8); } \
        else { FQ_RING_GP(BSL, 16); }           \
    } while (0)
    switch (BS) {
        case 8: FQ_RING_BS(3); break;
        case 16: FQ_RING_BS(4); break;
        default: FQ_RING_BS(5); break;
    }
#undef FQ_RING_BS
#undef FQ_RING_GP
#undef FQ_RING_PV
    return FQ_ERR_UNSUPPORTED_BLOCK;
}

int launch_ring(const DecodeParams& p0, int num_seqs, int block_size, bool wide, int dtype, hipStream_t stream) {
    DecodeParams p = p0;
    p.spin_limit = 0;
#ifdef FQ_RING_TIMING
    const char* dbg = std::getenv("FQ_RING_DEBUG");
    p.spin_limit = dbg ? std::atoi(dbg) : 0;
    if (p.spin_limit & 12) {
        static void* buf = nullptr;
        if (!buf) (void)hipMalloc(&buf, 2 << 20);
        p.sketch = static_cast<const float*>(buf);
        std::fprintf(stderr, "ring debug buffer %p\n", buf);
    }
#endif
    return dtype == FQ_F16 ? launch_ring_dt<FQ_F16>(p, num_seqs, block_size, wide, stream)
                           : launch_ring_dt<FQ_BF16>(p, num_seqs, block_size, wide, stream);
}

}  // namespace fq
