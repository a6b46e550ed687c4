// Block-sparse Summary-Attention prefill forward for gfx950.
//
// Replaces, for the forward pass, what the reference reaches through
//   summary_attn wheel, summary_attn/interface.py:70-91   (SummaryAttnFunc.forward)
//   flash_attn_cute wheel, flash_attn/cute/flash_fwd.py:1162-2480 (FlashAttentionForwardSm90)
//   flash_attn_cute wheel, flash_attn/cute/block_sparse_utils.py:134-476 (tile walk)
//   flash_attn_cute wheel, flash_attn/cute/softmax.py:52-146 (online soft-max)
// and keeps its numerics: 16-bit inputs, fp32 scores and soft-max state, exp2 with
// the scale folded in, probabilities rounded to 16 bit before the second product,
// fp32 output accumulator, one reciprocal per row at the end.
//
// A workgroup owns a 128-row query tile of one or two query heads of a kv group (shapes:
// `PrefillShape`); a wave owns 32 (or 64) of those rows for one head.  It walks the tile's
// non-empty key tiles (64 keys each) taken from the block index.  K and V tiles go from
// global memory straight into LDS (global_load_lds, two buffers each, row-major with the
// 16-byte chunks of every row XOR-permuted against bank conflicts); V is transposed on the
// way out of LDS by ds_read_b64_tr_b16 (operand layouts: ksa_tile.h).  The summary prefix of
// the key axis is read in place from the in-line summary rows (or, with `phys_prefix`, from
// the first P rows of K/V), never concatenated.
//
// The loop is software-pipelined: the score MFMAs of tile i+1 are interleaved with the
// soft-max of tile i, one MFMA and one pair of probabilities per time slot, so that matrix
// and vector work of one wave overlap; K therefore runs one tile ahead of V through LDS.
// All MFMA operands that come from LDS pass through a small rolling queue of fragments that
// is refilled right behind each MFMA and runs across the steps; the one workgroup barrier of a
// step stands in front of the last MFMAs of its second product, which then cover the reads of
// the next step's first fragments.
//
// Masking.  The walk has two phases that are uniform for the workgroup.  Phase A holds
// the tiles that need no per-element mask: the leading partial tiles below every text
// row's old-summary bound (there a row is visible as a whole iff it is a text row), the
// in-line tiles that lie inside every text row's window and below every row's diagonal and
// in front of the own chunk of the tile's summary rows (again a row is visible iff it is a
// text row; the one 8-aligned group of summary columns such a tile may hold is wiped for all
// rows at once: four registers of the score layout), and the full tiles.  Phase B holds the
// remaining partial tiles, masked per element from a 64-bit visibility word per query row.
//
// Soft-max reference.  The first walk is optimistic: a row's reference exponent comes from
// the unmasked scores of the first tile and is never moved (no row maximum is computed);
// the walk only records whether an exponent left the safe range.  If that ever happens
// the workgroup repeats the walk with the textbook online soft-max.
#include <hip/hip_runtime.h>
#include <math.h>

#include <type_traits>

#include "ksa_api_internal.h"
#include "ksa_mask.h"
#include "ksa_tile.h"

// This source is compiled as five translation units, so that the instantiations of the kernel
// compile side by side: unit 0 holds head_dim 64 and 128 and the entry point; units 1 to 4 (files
// that include this one with KSA_PREFILL_UNIT set) hold one kernel of head_dim 256 each - bf16 /
// fp16, regular / general tile addressing - because each of those takes over a minute to compile.
#ifndef KSA_PREFILL_UNIT
#define KSA_PREFILL_UNIT 0
#endif
// which of the two addressing variants a unit instantiates in launch_shape: 0 both, 1 regular, 2 general
#if KSA_PREFILL_UNIT == 1 || KSA_PREFILL_UNIT == 3
#define KSA_PREFILL_VARIANTS 1
#elif KSA_PREFILL_UNIT == 2 || KSA_PREFILL_UNIT == 4
#define KSA_PREFILL_VARIANTS 2
#else
#define KSA_PREFILL_VARIANTS 0
#endif

namespace {

struct PrefillParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    float* lse;  // may be null
    const int32_t* mask_cnt;
    const int32_t* mask_idx;
    const int32_t* full_cnt;
    const int32_t* full_idx;
    int idx_stride;  // N
    int M, Hq, Hkv, g;
    int phys_prefix;            // K/V rows are [P prefix rows | Sq in-line rows]
    int64_t q_bs, q_rs, q_hs;   // element strides: batch, row, head
    int64_t kv_bs, kv_rs, kv_hs;
    int64_t o_bs, o_rs, o_hs;
    int64_t lse_bs, lse_hs;
    KsaMask mk;
    float scale;
    float scale_log2;
    int shape;  // 2: two heads on 8 waves; 32: one head per workgroup; 64: two heads, 64 query rows per wave
    // Work items (batch element, m tile, head (pair), kv head) are numbered heavy first; workgroup
    // i takes item i while i < n_static.  The workgroups behind that take the remaining (light)
    // items from eight queues in device memory, one per XCD (queue = item number modulo 8, which is
    // also the XCD a workgroup of that number runs on and the kv head whose K/V that XCD's cache
    // holds): first from the queue of their own XCD, then from the others.  The XCDs of one chip
    // run at clocks a few per cent apart; with a fixed split the launch ends when the slowest one
    // is done, with the queues the faster ones take over part of its tail.  sched == null: all
    // workgroups take the item of their own number.
    int32_t* sched;   // eight counters, zeroed in front of the launch
    int n_items;      // items per batch element
    int total;        // items in all
    int n_static;     // multiple of 8
};

constexpr int kTileM = 128;
constexpr int kTileN = 64;

// Visible key set of one query row in key coordinates, fixed for the whole tile walk:
//   [0, xa)    (in-line mode: summary columns only)
//   [blo, bhi) (text rows: text columns only)
struct RowVis {
    int xa, blo, bhi;
    bool b_text;
};

__device__ __forceinline__ RowVis ksa_row_vis(const KsaMask& mk, int q) {
    const int B = mk.C + mk.S;
    const int c = q / B, o = q % B;
    RowVis r;
    if (o >= mk.C) {  // summary row: own chunk, causal, every column kind
        r.xa = 0;
        r.blo = mk.P + c * B;
        r.bhi = mk.P + q + 1;
        r.b_text = false;
        return r;
    }
    const int w0 = c > mk.W ? c - mk.W : 0;
    r.b_text = true;
    r.bhi = mk.P + q + 1;
    if (mk.P > 0) {
        r.xa = mk.skip_old ? 0 : w0 * mk.S;
        r.blo = max(mk.P + w0 * B, r.xa);
    } else {
        r.xa = mk.skip_old ? 0 : w0 * B;
        r.blo = w0 * B;
    }
    return r;
}

// kRegular: every listed key tile lies entirely in the summary prefix or entirely in the
// in-line region and inside the key axis (P and Sk multiples of 64), and in-place prefix
// rows of one thread differ by a uniform step; then tile addressing is branch-free.
//
// RB: 32-row query blocks per wave.  RB = 1: one query head per workgroup, wave w owns rows
// 32w..32w+31, two workgroups per CU.  RB = 2: two query heads of one kv group per workgroup,
// waves {0,1} / {2,3} own rows 0..63 / 64..127 of the first / second head, one workgroup per
// CU with up to 512 registers per lane; every K and V fragment read from LDS then feeds two
// MFMAs, which halves the LDS traffic per MFMA (at one fragment per MFMA the four SIMDs ask
// for more than the LDS delivers).
//
// HW: query heads (of one kv group) per workgroup.  The workgroup has 4 HW / RB waves; with
// HW = 2, RB = 1 (8 waves, two per SIMD) one K/V tile in LDS serves twice the MFMA work, which
// halves the fill traffic into LDS per MFMA.
template <int RB, int HW>
struct PrefillShape {
    static constexpr int kWaves = 4 * HW / RB;
    static constexpr int kThreads = 64 * kWaves;
};

template <typename T, int D, bool kRegular, int RB, int HW>
__global__ __launch_bounds__((PrefillShape<RB, HW>::kThreads), (RB == 1 && D <= 128 ? 2 : 1)) void ksa_prefill_kernel(
    const PrefillParams p) {
    constexpr int kThreads = PrefillShape<RB, HW>::kThreads;
    using Ops = KsaOps<T>;
    constexpr int KS = D / 16;       // contraction steps of K Q^T
    constexpr int DB = D / 32;       // 32-row blocks of O^T
    constexpr int CPR = D / 8;       // 16-byte chunks per K/V row
    constexpr int ROWB = 2 * D;      // LDS row of K / V in bytes (unpadded, XOR-swizzled chunks)
    constexpr int KLD = (kTileN * CPR) / kThreads;  // K (and V) loads per thread
    constexpr int RSTEP = kThreads / CPR;           // row distance between a thread's loads
    constexpr float kTau = 8.f;      // lazy rescale: exponents stay below 2^kTau

    // K and V tiles travel global -> LDS directly (global_load_lds), 1 KB per wave
    // instruction, so LDS rows cannot be padded; bank conflicts are avoided by permuting the
    // 16-byte chunks inside each row instead:
    //   K: chunk c of tile row r sits at position c ^ ksw(r)  (the 16 lanes of a b128 read
    //      phase hold 16 consecutive rows and the same chunk)
    //   V: 64-byte segment s of row r sits at segment s ^ vsw(r)  (a transposing b64 read
    //      phase covers 4 consecutive rows and one segment)
    // Four separate arrays (not one [2][..]) so that the compiler can tell the buffer being
    // filled from the one being read and does not wait for the fill before unrelated reads.
    __shared__ __attribute__((aligned(1024))) uint16_t Ks0[kTileN * D];
    __shared__ __attribute__((aligned(1024))) uint16_t Ks1[kTileN * D];
    __shared__ __attribute__((aligned(1024))) uint16_t Vs0[kTileN * D];
    __shared__ __attribute__((aligned(1024))) uint16_t Vs1[kTileN * D];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lq = lane & 31;
    const int lh = lane >> 5;

    // workgroup -> (kv head, query head (pair) in group, m tile); kv head fastest so that
    // the workgroups sharing K/V land on one XCD; heavy (late) m tiles first.
    int item = blockIdx.x;
    if (p.sched != nullptr && item >= p.n_static) {
        __shared__ int s_item;
        if (tid == 0) {
            int got = -1;
            for (int k = 0; k < 8 && got < 0; ++k) {
                const int y = (item + k) & 7;
                const int cand = p.n_static + y + 8 * atomicAdd(&p.sched[y], 1);
                if (cand < p.total) got = cand;
            }
            s_item = got;
        }
        __syncthreads();
        item = s_item;
        if (item < 0) return;  // every queue is empty: a spare workgroup
    }
    const int bz = item / p.n_items;
    const int id = item - bz * p.n_items;
    const int kvh = id % p.Hkv;
    const int rest = id / p.Hkv;
    constexpr int kWavesPerHead = 4 / RB;

    const int gper = p.g / HW;
    const int gi = rest % gper;
    const int mt = p.M - 1 - rest / gper;
    const int head = kvh * p.g + HW * gi + wave / kWavesPerHead;
    const int row0 = mt * kTileM + (wave % kWavesPerHead) * 32 * RB;
    const KsaMask mk = p.mk;
    const bool prefix_mode = mk.P > 0;
    const bool phys = p.phys_prefix != 0;
    const int Bblk = mk.C + mk.S;

    int qrow[RB];
    RowVis rv[RB];
    // Q as B operand, resident in registers for the whole tile walk
    u32x4 qf[RB][KS];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        qrow[r] = row0 + 32 * r + lq;
        const int qrow_c = min(qrow[r], mk.Sq - 1);
        rv[r] = ksa_row_vis(mk, qrow_c);
        const uint16_t* qp = p.q + bz * p.q_bs + (int64_t)qrow_c * p.q_rs + head * p.q_hs + 8 * lh;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[r][s] = *reinterpret_cast<const u32x4*>(qp + 16 * s);
    }

    // ---- K/V addressing: uniform base + uniform tile offset + 32-bit thread offset ----
    const char* kbase = reinterpret_cast<const char*>(p.k + bz * p.kv_bs + kvh * p.kv_hs);
    const char* vbase = reinterpret_cast<const char*>(p.v + bz * p.kv_bs + kvh * p.kv_hs);
    const uint32_t rb = (uint32_t)p.kv_rs * 2u;  // row pitch in bytes
    const int ld_row = tid / CPR;                // first tile row this thread loads
    auto ksw = [](int r) { return D >= 128 ? (r & 15) : ((r >> 1) & 7); };
    auto vsw = [](int r) { return D >= 128 ? (r & 3) : ((r >> 1) & 1); };
    // this thread fills chunk position tid % CPR of its rows: the source chunk is the position
    // with the row's permutation undone.  Rows of one thread differ by multiples of RSTEP: 16 or 32
    // (the permutation is then the same for all of them), or 8 at head_dim 256, where K's permutation
    // of a thread's odd loads differs in bit 3 of the chunk number (kKOdd, in bytes).
    constexpr uint32_t kKOdd = (D >= 128 && RSTEP % 16 != 0) ? 128u : 0u;
    static_assert(RSTEP % 8 == 0, "a thread's rows differ by multiples of eight");
    const uint32_t kcol = (uint32_t)((tid % CPR) ^ ksw(ld_row)) * 16u;
    const uint32_t vcol = (uint32_t)((tid % CPR) ^ (vsw(ld_row) << 2)) * 16u;
    const uint32_t thr_main = (uint32_t)ld_row * rb;
    // in-place prefix: prefix row j lives at in-line row (j / S) * B + C + j % S; when S
    // divides the per-thread row step the rows of one thread differ by a uniform amount
    const bool s_fast = !phys && (RSTEP % mk.S == 0);
    const uint32_t thr_pre =
        s_fast ? (uint32_t)((ld_row / mk.S) * Bblk + mk.C + ld_row % mk.S) * rb : 0u;
    const uint32_t step_main = RSTEP * rb;
    const uint32_t step_pre = s_fast ? (uint32_t)(RSTEP / mk.S) * Bblk * rb : 0u;

    auto src_row = [&](int kv) -> uint32_t {  // generic key column -> K/V row
        kv = min(kv, mk.Sk - 1);
        if (phys || kv >= mk.P) return (uint32_t)(phys ? kv : kv - mk.P);
        return (uint32_t)((kv / mk.S) * Bblk + mk.C + kv % mk.S);
    };

    // tile, load i -> (uniform byte offset, uniform per-load step, this thread's byte offset for load i)
    auto tile_src = [&](int n0, int i, uint32_t& ubase, uint32_t& ustep, uint32_t& voff) {
        const bool in_main = (phys || n0 >= mk.P) && n0 + kTileN <= mk.Sk;
        if (in_main) {
            ubase = (uint32_t)(phys ? n0 : n0 - mk.P) * rb;
            ustep = step_main;
            voff = thr_main;
        } else if (s_fast && n0 + kTileN <= mk.P) {
            ubase = (uint32_t)(n0 / mk.S) * Bblk * rb;
            ustep = step_pre;
            voff = thr_pre;
        } else {
            ubase = 0;
            ustep = 0;
            voff = src_row(n0 + ld_row + RSTEP * i) * rb;
        }
    };

    // Regular tiles: uniform offset word = byte offset of the tile's first row | 1 if the
    // tile lies in the in-line region (computed per lane when the walk order is fetched).
    auto tile_word = [&](int n) -> uint32_t {
        const int n0 = n * kTileN;
        const bool in_main = phys || n0 >= mk.P;
        return in_main ? ((uint32_t)(phys ? n0 : n0 - mk.P) * rb) | 1u
                       : (uint32_t)(n0 / mk.S) * Bblk * rb;
    };
    // one 1 KB piece (load i of KLD) of tile n into an LDS tile; `col` = kcol or vcol
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto fill1 = [&](const char* base, uint16_t* tile, uint32_t col, int n, uint32_t word, int i, uint32_t odd_xor) {
        uint32_t ub, us, vo;
        if constexpr (kRegular) {
            const bool in_main = word & 1u;
            ub = word & ~1u;
            us = in_main ? step_main : step_pre;
            vo = in_main ? thr_main : thr_pre;
        } else {
            tile_src(n * kTileN, i, ub, us, vo);
        }
        typedef __attribute__((address_space(3))) char* lptr;
        char* dst = reinterpret_cast<char*>(tile) + (RSTEP * i + wave_u * (64 / CPR)) * ROWB;
        // Uniform 64-bit base + one 32-bit lane offset (the scalar-base addressing form); M0
        // carries the LDS address of the wave's 1 KB piece, lane l lands at + 16 l.  Written as
        // assembly so that the compiler does not track the fill: it would otherwise make LDS
        // reads wait for fills it cannot tell apart; which fills must have landed before a
        // barrier is decided by fills_done.
        uint64_t ubase = reinterpret_cast<uint64_t>(base + (ub + us * i));
        const uint32_t loff = vo + (col ^ ((i & 1) ? odd_xor : 0u));
        uint32_t lds_addr = (uint32_t)(uintptr_t)(lptr)dst;
        if constexpr (D > 128) {
            // (both are the same in every lane; at this size the compiler no longer proves it and
            // would hand the statement below vector registers)
            lds_addr = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr);
            ubase = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)ubase) |
                    ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(ubase >> 32)) << 32);
        }
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // M0 is reserved; nothing else in this kernel uses it
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(loff), "s"(ubase)
                     : "memory", "m0");
#pragma clang diagnostic pop
    };
    auto fill = [&](const char* base, uint16_t* tile, uint32_t col, int n, uint32_t word, uint32_t odd_xor) {
#pragma unroll
        for (int i = 0; i < KLD; ++i) fill1(base, tile, col, n, word, i, odd_xor);
    };
    // all of this wave's fills have landed (the barrier that follows publishes them)
    auto fills_done = []() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
    // Workgroup barrier of the tile loop: a plain s_barrier (the fills that have to be visible
    // are awaited explicitly by fills_done; LDS reads are complete once their data was used).
    auto wg_barrier = []() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // per-lane byte offsets of the MFMA operand reads inside a tile
    uint32_t koff[KS];  // K fragment of contraction step s, key block 0 (block 1: + 32 rows)
#pragma unroll
    for (int sx = 0; sx < KS; ++sx) koff[sx] = (uint32_t)lq * ROWB + (uint32_t)((2 * sx + lh) ^ ksw(lq)) * 16u;
    uint32_t voff[DB];  // V fragment of dim block b, key step 0 (step ks: + 16 ks rows; second half: + 8 rows)
    {
        const int t = lq & 15, r = 4 * lh + (t >> 2);
#pragma unroll
        for (int bx = 0; bx < DB; ++bx)
            voff[bx] = (uint32_t)r * ROWB + (uint32_t)(bx ^ vsw(r)) * 64u + (uint32_t)((lq & 16) + 4 * (t & 3)) * 2u;
    }
    auto read_k = [&](const uint16_t* tile, int j) {  // j = 2 s + kb
        return *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(tile) + koff[j >> 1] + (j & 1) * 32 * ROWB);
    };
    auto read_v = [&](const uint16_t* tile, int j) {  // j = DB ks + b
        typedef __attribute__((address_space(3))) ksa_short4* lds_ptr;
        const char* pv = reinterpret_cast<const char*>(tile) + voff[j % DB] + (j / DB) * 16 * ROWB;
        const u32x2 l2 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(pv)));
        const u32x2 h2 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(pv + 8 * ROWB)));
        u32x4 f;
        f[0] = l2[0];
        f[1] = l2[1];
        f[2] = h2[0];
        f[3] = h2[1];
        return f;
    };

    // ---- walk order ----
    const int npart = p.mask_cnt[mt];
    const int nfull = p.full_cnt[mt];
    const int ntiles = npart + nfull;
    const int32_t* plist = p.mask_idx + (int64_t)mt * p.idx_stride;
    const int32_t* flist = p.full_idx + (int64_t)mt * p.idx_stride;
    int nquick = 0;
    int c0 = 0, c1 = 0;  // entries [c0, c1) of the list of partial tiles: the uniform in-line tiles described below
    {
        const int c_first = (mt * kTileM) / Bblk;
        const int w_first = c_first > mk.W ? c_first - mk.W : 0;
        // every text row of the tile has xa >= w_first * S and blo >= P >= thr
        const int thr = (prefix_mode && !mk.skip_old) ? min(w_first * mk.S, mk.P) : 0;
        const int nlim = thr / kTileN;  // tiles n < nlim end at or below thr
        // number of entries of the ascending list below nlim (at most nlim of them): counted by
        // the whole wave, 128 entries per round of independent loads, instead of a binary search
        // whose dependent loads would cost several microseconds at the start of every workgroup
        // In-line tiles that every text row of this row tile sees in all their text columns and no summary
        // row sees at all (entirely inside every text row's [blo, bhi) and in front of the own chunk of the
        // tile's first summary row): tiles n in [n_c0, n_c1).  They need no per-row mask either - a row is
        // visible iff it is a text row, and the one group of S = 8 summary columns such a tile may hold is
        // wiped for all rows at once (see `step`).  With chunks of C + S columns that are multiples of 8
        // and hold a whole tile, a tile holds at most one such group and the group is 8-aligned in it.
        int n_c0 = 0, n_c1 = 0;
#ifndef KSA_PREFILL_NO_UNIFORM_TILES
        if (mk.S == 8 && mk.C % 8 == 0 && mk.P % 8 == 0 && Bblk >= kTileN + 8) {
            const int R0 = mt * kTileM, R1 = min(R0 + kTileM, mk.Sq) - 1;
            const int q_ft = (R0 % Bblk) < mk.C ? R0 : (R0 / Bblk + 1) * Bblk;            // first text row
            const int q_lt = (R1 % Bblk) < mk.C ? R1 : (R1 / Bblk) * Bblk + mk.C - 1;      // last text row
            const int q_fs = (R0 % Bblk) >= mk.C ? R0 : (R0 / Bblk) * Bblk + mk.C;          // first summary row
            if (q_ft <= R1 && q_lt >= q_ft) {
                const int c_lt = q_lt / Bblk;
                const int lo = mk.P + (c_lt > mk.W ? c_lt - mk.W : 0) * Bblk;
                int hi = mk.P + q_ft + 1;
                if (q_fs <= R1) hi = min(hi, mk.P + (q_fs / Bblk) * Bblk);
                n_c0 = (lo + kTileN - 1) / kTileN;
                n_c1 = max(hi / kTileN, n_c0);
            }
        }
#endif
        // number of entries of the ascending list below nlim (at most nlim of them), below n_c0 and
        // below n_c1: counted by the whole wave, 128 entries per round of independent loads, instead
        // of binary searches whose dependent loads would cost several microseconds at the start of
        // every workgroup
        const int lim = min(npart, max(nlim, n_c1));
        int cnt = 0, cnt0 = 0, cnt1 = 0;
        for (int base = 0; base < lim; base += 128) {
            const int i0 = base + lane, i1 = base + 64 + lane;
            const int e0 = i0 < lim ? plist[i0] : 0x7fffffff;
            const int e1 = i1 < lim ? plist[i1] : 0x7fffffff;
            cnt += __popcll(__ballot(e0 < nlim)) + __popcll(__ballot(e1 < nlim));
            cnt0 += __popcll(__ballot(e0 < n_c0)) + __popcll(__ballot(e1 < n_c0));
            cnt1 += __popcll(__ballot(e0 < n_c1)) + __popcll(__ballot(e1 < n_c1));
        }
        nquick = cnt;
        c0 = max(cnt0, nquick);
        c1 = max(cnt1, c0);
    }
    const bool last_full_cut = nfull > 0 && (flist[nfull - 1] + 1) * kTileN > mk.Sk;
    const int nfull_a = nfull - (last_full_cut ? 1 : 0);
    // Walk order.  Phase A: the leading prefix tiles, the uniform in-line tiles, the full tiles; phase B:
    // the other partial tiles (those in front of the uniform run, those behind it, a cut full tile).
    const int ncheap = c1 - c0;
    const int n_a = nquick + ncheap + nfull_a;
    auto tile_at = [&](int i) {
        if (i < nquick) return plist[i];
        if (i < nquick + ncheap) return plist[c0 + (i - nquick)];
        if (i < n_a) return flist[i - nquick - ncheap];
        int j = i - n_a + nquick;            // entries [nquick, c0), then [c1, npart)
        if (j >= c0) j += ncheap;
        return j < npart ? plist[j] : flist[nfull - 1];
    };
    // The order is kept in registers, 64 entries at a time (lane i holds entry base + i),
    // so the loop never waits on a dependent index load.
    auto seq_chunk = [&](int base) { return base + lane < ntiles ? tile_at(base + lane) : 0; };
    int seq_cur = seq_chunk(0);
    int seq_nxt = seq_chunk(64);
    uint32_t word_cur = kRegular ? tile_word(seq_cur) : 0u;
    uint32_t word_nxt = kRegular ? tile_word(seq_nxt) : 0u;
    // Where a tile's first column stands in the period of C text + S summary columns of the
    // in-line region, (n0 - P) mod (C + S) in [0, C + S): computed with the walk order, one
    // division per lane and 64 tiles, so that the masked steps have none.
    auto tile_phase = [&](int n) {
        const int r = (n * kTileN - mk.P) % Bblk;
        return r < 0 ? r + Bblk : r;
    };
    int phase_cur = tile_phase(seq_cur);
    int phase_nxt = tile_phase(seq_nxt);
    auto seq_phase = [&](int i, int it) {
        const int src = (i >> 6) == (it >> 6) ? phase_cur : phase_nxt;
        return __builtin_amdgcn_readlane(src, i & 63);
    };
    // entry i in {it, .., it+3} while processing tile it
    auto seq = [&](int i, int it) {
        const int src = (i >> 6) == (it >> 6) ? seq_cur : seq_nxt;
        return __builtin_amdgcn_readlane(src, i & 63);
    };
    auto seq_word = [&](int i, int it) {
        const uint32_t src = (i >> 6) == (it >> 6) ? word_cur : word_nxt;
        return (uint32_t)__builtin_amdgcn_readlane((int)src, i & 63);
    };

    floatx16 oacc[RB][DB];
    float m_ref[RB];  // reference of the exponents (raw score units), see `walk` below
    float l_run[RB];  // this lane's half of the row sum
    bool bad = false; // optimistic walk: some exponent left the safe range
    const float c2 = p.scale_log2;

    auto zero16 = []() {
        floatx16 z;
#pragma unroll
        for (int i = 0; i < 16; ++i) z[i] = 0.f;
        return z;
    };

    auto scores = [&](floatx16 (&sacc)[RB][2], const uint16_t* ktile) __attribute__((always_inline)) {  // S^T = K Q^T
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const u32x4 a = read_k(ktile, 2 * s + kb);
#pragma unroll
                for (int r = 0; r < RB; ++r) {
                    if constexpr (RB == 1) {
                        sacc[r][kb] = Ops::mfma(a, qf[r][s], s == 0 ? zero16() : sacc[r][kb]);
                    } else {
                        if (s == 0) sacc[r][kb] = Ops::mfma_v0(a, qf[r][s]);
                        else Ops::mfma_v(sacc[r][kb], a, qf[r][s]);
                    }
                }
            }
        }
        if constexpr (RB != 1) ksa_mfma_settle();
    };

    // MFMA operands that come from LDS travel through a rolling queue of kQueue fragments that
    // runs across the steps: see `step`.
    constexpr int kQueue = 4;
#ifndef KSA_PREFILL_BEHIND
#define KSA_PREFILL_BEHIND 4
#endif
    constexpr int kBehind = KSA_PREFILL_BEHIND;  // MFMAs of the second product behind the step's barrier
    static_assert(kBehind >= 1 && kBehind <= kQueue, "fragments behind the barrier come from the queue");
    u32x4 fq[kQueue];
    // One pipeline step for tile `it` (parity tag = it % 2): its scores are in `scur`; the
    // scores of tile it+1 are produced into `snext`.  On entry K(it+1) and V(it) are in LDS and
    // published (the previous step's barrier, or the prologue's), the first operands of the score
    // product are in the queue, and the other two buffers are free: this step refills them with
    // K(it+2) and V(it+1) while it computes and publishes them with its own barrier near its end.
    // `quick`: a row is visible as a whole iff it is a text row (leading prefix tiles).
    auto step = [&](auto safe_tag, auto general_tag, auto parity_tag, int it, floatx16 (&scur)[RB][2],
                    floatx16 (&snext)[RB][2], bool quick) __attribute__((always_inline)) {
        constexpr bool kSafe = decltype(safe_tag)::value;
        constexpr bool kGeneral = decltype(general_tag)::value;
        constexpr int PAR = decltype(parity_tag)::value;
        const int n0 = seq(it, it) * kTileN;
        // Past the end of the walk the pipeline keeps running on the last tile (fills) and
        // on stale LDS contents (scores); those results are never used.
        // fills: K(it+2) and V(it+1), both issued in the first slots of the score stage
        const int ik = min(it + 2, ntiles - 1), iv = min(it + 1, ntiles - 1);
        const int nk = seq(ik, it), nv = seq(iv, it);
        const uint32_t wk = seq_word(ik, it), wv = seq_word(iv, it);
        bool row_vis[RB];
#pragma unroll
        for (int r = 0; r < RB; ++r) row_vis[r] = quick ? rv[r].b_text : true;

        // MFMA operands that come from LDS travel through a rolling queue of kQueue fragments:
        // the read for operand j + kQueue is issued right behind the MFMAs of operand j, through
        // the score product (K fragments), across its end (the first V fragments), through the
        // second product and across the end of the step (the first K fragments of the next step),
        // so every read has kQueue operands' worth of MFMAs plus the vector work between them to
        // land.  The step's barrier stands in front of the last kQueue MFMAs of the second
        // product: by then every fragment this step takes from LDS is in registers, the barrier
        // publishes the tiles filled during the step, and the MFMAs behind it cover the reads
        // of the next step's first fragments.
        constexpr int NQK = 2 * KS;   // K fragments: contraction step s = j / 2, key block kb = j % 2
        constexpr int NPV = 4 * DB;   // V fragments: key step ks = j / DB, dim block j % DB
        const uint16_t* ksrc = PAR ? Ks0 : Ks1;   // K(it+1)
        const uint16_t* vsrc = PAR ? Vs1 : Vs0;   // V(it)
        uint16_t* kdst = PAR ? Ks1 : Ks0;         // <- K(it+2)
        uint16_t* vdst = PAR ? Vs0 : Vs1;         // <- V(it+1)
        auto kfrag = [&](int j) { return read_k(ksrc, j); };
        auto vfrag = [&](int j) { return read_v(vsrc, j); };
        __builtin_amdgcn_sched_barrier(0);

        if constexpr (!kGeneral) {
            if (quick && it >= nquick) {
                // a uniform in-line tile (see the walk order): if it holds the group of summary columns of a
                // chunk, those eight keys are hidden from every row - in the score layout they are four
                // registers of one 32-key block, the same in every lane
                int rel = mk.C - seq_phase(it, it);
                rel += rel < 0 ? Bblk : 0;
                if (rel < kTileN) {
                    // (one uniform branch per 32-key block, then selects in place on a uniform condition: with
                    // a branch per group the compiler copied the score registers around, cfg 1 -1.3 %;
                    // selects over both blocks cost the dense-causal layer 2.4 %)
                    const int gj = rel >> 3;
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
                        if ((gj >> 2) == kb) {
#pragma unroll
                            for (int qd = 0; qd < 4; ++qd) {
                                const bool hit = (gj & 3) == qd;
#pragma unroll
                                for (int r = 0; r < RB; ++r)
#pragma unroll
                                    for (int e = 0; e < 4; ++e)
                                        scur[r][kb][4 * qd + e] = hit ? -INFINITY : scur[r][kb][4 * qd + e];
                            }
                        }
                }
            }
        }
        if constexpr (kGeneral) {  // 64-bit visibility word per row
            const int kv = n0 + lane;
            const bool in = kv < mk.Sk;
            const uint64_t valid = __ballot(in);
            // text column: its offset in the period is below C.  phase + lane is below two periods
            // when a period holds a tile's 64 columns (any real chunk size).
            int o = seq_phase(it, it) + lane;
            if (Bblk >= kTileN) o -= o >= Bblk ? Bblk : 0;
            else o %= Bblk;
            const uint64_t text = valid & __ballot(kv >= mk.P) & __ballot(o < mk.C);
            const uint64_t fa = prefix_mode ? valid : (valid & ~text);
            // bits [lo, hi) of a 64-bit word, without a branch
            auto range_bits = [](int lo, int hi) {
                lo = max(lo, 0);
                hi = max(hi, 0);
                const uint64_t below_hi = hi >= 64 ? ~0ull : ~(~0ull << hi);
                const uint64_t from_lo = lo >= 64 ? 0ull : (~0ull << lo);
                return below_hi & from_lo;
            };
            // -inf where the word has a 0: one bit-field extract (0 or all ones) and one bit-field
            // insert per element, no compare; a half whose 16 bits are set in every lane that sees
            // anything of the tile is left alone (the 8 summary columns that a tile below the
            // diagonal hides from text rows lie in one half; skipping by groups of 8 keys inside a
            // half as well measured slower: cfg 2 -0.3 %, cfg 1 -1.1 %).
            auto mask_half = [](floatx16& sc, uint32_t w, bool any) {
                if (__ballot(any && (w & 0x0f0f0f0fu) != 0x0f0f0f0fu) == 0ull) return;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t m = (uint32_t)__builtin_amdgcn_sbfe((int)w, 8 * (i / 4) + (i % 4), 1);
                    sc[i] = __uint_as_float((__float_as_uint(sc[i]) & m) | (0xff800000u & ~m));
                }
            };
            // (uniform) a tile of the in-line region behind a prefix: no row's [0, xa) reaches it
            const bool no_xa = prefix_mode && n0 >= mk.P;
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const uint64_t fb = rv[r].b_text ? text : valid;
                uint64_t bits = range_bits(rv[r].blo - n0, rv[r].bhi - n0) & fb;
                if (!no_xa) bits |= range_bits(-n0, rv[r].xa - n0) & fa;
                // a row that sees nothing of the tile loses it through its reference (infinite:
                // every probability 0) and does not keep a half from being skipped
                const bool any = bits != 0ull;
                row_vis[r] = any;
                const uint64_t sh = bits >> (4 * lh);
                mask_half(scur[r][0], (uint32_t)sh, any);
                mask_half(scur[r][1], (uint32_t)(sh >> 32), any);
            }
        }

        // Probabilities relative to the current reference.  The row maximum is computed only
        // in the safe walk; the optimistic walk keeps the reference it has and only watches
        // the tile sums.
        float l_tile[RB];
        u32x4 pf[RB][4];
        float mc[RB];
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            l_tile[r] = 0.f;
            mc[r] = row_vis[r] ? m_ref[r] * c2 : INFINITY;
        }
        // Probability pair cc (row block cc / 16, keys of 16-key group (cc % 16) / 4, word cc % 4)
        // in four dependent stages.  In the interleaved loop below the stages of one pair run
        // in consecutive time slots, so no vector instruction waits for its predecessor.
        float pa[2][2];
        uint32_t pw[2];
        auto stage_a = [&](int cc) {  // exponent arguments
            const int r = cc >> 4, c = cc & 15;
            const int g = c >> 2, kb = g >> 1, i0 = 8 * (g & 1) + 2 * (c & 3);
            pa[cc & 1][0] = fmaf(scur[r][kb][i0], c2, -mc[r]);
            pa[cc & 1][1] = fmaf(scur[r][kb][i0 + 1], c2, -mc[r]);
        };
        auto stage_b = [&](int cc) {
            pa[cc & 1][0] = ksa_exp2(pa[cc & 1][0]);
            pa[cc & 1][1] = ksa_exp2(pa[cc & 1][1]);
        };
        auto stage_c = [&](int cc) { pw[cc & 1] = Ops::pack2(pa[cc & 1][0], pa[cc & 1][1]); };
        auto stage_d = [&](int cc) {
            const int r = cc >> 4, c = cc & 15;
            l_tile[r] = Ops::sum2(pw[cc & 1], l_tile[r]);
            pf[r][c >> 2][c & 3] = pw[cc & 1];
        };
        constexpr int NCH = 16 * RB;
        // time slot vt: stage d of pair vt-3, c of vt-2, b of vt-1, a of vt
        auto prob_slot = [&](int vt) {
            if (vt >= 3 && vt - 3 < NCH) stage_d(vt - 3);
            if (vt >= 2 && vt - 2 < NCH) stage_c(vt - 2);
            if (vt >= 1 && vt - 1 < NCH) stage_b(vt - 1);
            if (vt < NCH) stage_a(vt);
        };
        // move the reference of the rows whose maximum outgrew it (or that have none yet)
        auto rebase = [&]() {
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                float mloc = fmaxf(scur[r][0][0], scur[r][1][0]);
#pragma unroll
                for (int i = 1; i < 16; ++i) mloc = fmaxf(mloc, fmaxf(scur[r][0][i], scur[r][1][i]));
                if (!row_vis[r]) mloc = -INFINITY;
                mloc = ksa_pair_max(mloc);
                const bool bump = (mloc - m_ref[r]) * c2 > kTau;
                if (__any(bump)) {
                    const float m_new = bump ? mloc : m_ref[r];
                    const float alpha = ksa_exp2((m_ref[r] - m_new) * c2);
                    m_ref[r] = m_new;
                    l_run[r] *= alpha;
#pragma unroll
                    for (int b = 0; b < DB; ++b) {
#pragma unroll
                        for (int i = 0; i < 16; ++i) oacc[r][b][i] *= alpha;
                        if constexpr (RB != 1) {
                            // back to its AGPR block before the next one is touched, so that
                            // this rare path never holds more than one block in VGPRs
                            asm volatile("" : "+a"(oacc[r][b]));
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            }
        };
        if constexpr (kSafe) {
            rebase();
#pragma unroll
            for (int r = 0; r < RB; ++r) mc[r] = row_vis[r] ? m_ref[r] * c2 : INFINITY;
        }

        // Score MFMAs of the NEXT tile with the probability pairs of THIS tile between them.
        // The fences pin the order; kLead slots run first and cover the first operand reads.
        // The first slots also issue the fills of the two buffers freed by the barrier.
        constexpr int kLead = 3;
        constexpr int NM = NQK * RB;             // score MFMAs of the step; MFMA m is followed by the
                                                 // probability slots kLead + [m NCH / NM, (m + 1) NCH / NM)
                                                 // (two, one, or one at every second MFMA for head_dim 64, 128, 256)
        static_assert(2 * KLD <= NM, "one fill per MFMA slot at most");
#pragma unroll
        for (int vt = 0; vt < kLead; ++vt) prob_slot(vt);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NQK; ++j) {
            const int kb = j & 1;
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                if constexpr (RB == 1) {
                    snext[r][kb] = Ops::mfma(fq[j % kQueue], qf[r][j >> 1], j < 2 ? zero16() : snext[r][kb]);
                } else {
                    if (j < 2) snext[r][kb] = Ops::mfma_v0(fq[j % kQueue], qf[r][j >> 1]);
                    else Ops::mfma_v(snext[r][kb], fq[j % kQueue], qf[r][j >> 1]);
                }
                if (r == RB - 1)
                    fq[j % kQueue] = (j + kQueue < NQK) ? kfrag(j + kQueue) : vfrag(j + kQueue - NQK);
                const int m = j * RB + r;
#pragma unroll
                for (int vt = kLead + (m * NCH) / NM; vt < kLead + ((m + 1) * NCH) / NM; ++vt) prob_slot(vt);
                if (m < KLD) fill1(kbase, kdst, kcol, nk, wk, m, kKOdd);
                else if (m < 2 * KLD) fill1(vbase, vdst, vcol, nv, wv, m - KLD, 0u);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if constexpr (!kSafe) {
            // 2^24: some exponent exceeded the reference by more than ~19
#pragma unroll
            for (int r = 0; r < RB; ++r) bad = bad || l_tile[r] > 16777216.f;
        }
#pragma unroll
        for (int r = 0; r < RB; ++r) l_run[r] += l_tile[r];

        // O^T += V^T P^T
#pragma unroll
        for (int j = 0; j < NPV; ++j) {
            if (j == NPV - kBehind) {
                fills_done();
                wg_barrier();
                // the next step's fragments whose queue places came free in front of the barrier
#pragma unroll
                for (int t = NPV; t < NPV - kBehind + kQueue; ++t) fq[t % kQueue] = read_k(kdst, t - NPV);
            }
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                if constexpr (RB == 1) oacc[r][j % DB] = Ops::mfma(fq[j % kQueue], pf[r][j / DB], oacc[r][j % DB]);
                else Ops::mfma_a(oacc[r][j % DB], fq[j % kQueue], pf[r][j / DB]);
            }
            if (j + kQueue < NPV) fq[j % kQueue] = vfrag(j + kQueue);
            else if (j >= NPV - kBehind) fq[j % kQueue] = read_k(kdst, j + kQueue - NPV);
            __builtin_amdgcn_sched_barrier(0);
        }
        if ((it & 63) == 63) {  // roll the index chunk
            seq_cur = seq_nxt;
            word_cur = word_nxt;
            phase_cur = phase_nxt;
            seq_nxt = seq_chunk(it + 1 + 64);
            word_nxt = kRegular ? tile_word(seq_nxt) : 0u;
            phase_nxt = tile_phase(seq_nxt);
        }
    };

    // One complete walk over the tile list.  The optimistic walk (kSafe = false) takes each
    // row's reference from the unmasked scores of the first tile and never moves it; it
    // reports when that went wrong -- an exponent far above the reference (tile sum
    // above 2^24) or a row sum so small that the reference was far too high -- and the
    // workgroup then repeats the walk in the safe form, which moves the reference before the
    // probabilities of every tile (the textbook online soft-max, still with the lazy
    // threshold).  Random-like scores never need the second walk.
    floatx16 s0[RB][2], s1[RB][2];
    auto copy_scores = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int i = 0; i < 16; ++i) s0[r][kb][i] = s1[r][kb][i];
    };
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;
    auto walk = [&](auto safe_tag) __attribute__((always_inline)) {
        constexpr bool kSafe = decltype(safe_tag)::value;
        using A = std::false_type;
        using B = std::true_type;
        seq_cur = seq_chunk(0);
        seq_nxt = seq_chunk(64);
        word_cur = kRegular ? tile_word(seq_cur) : 0u;
        word_nxt = kRegular ? tile_word(seq_nxt) : 0u;
        phase_cur = tile_phase(seq_cur);
        phase_nxt = tile_phase(seq_nxt);
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            m_ref[r] = -1e30f;  // finite: the first rescale multiplies the zero accumulators by 0
            l_run[r] = 0.f;
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[r][b][i] = 0.f;
        }
        if (ntiles > 0) {  // prologue: K(0), V(0), K(1) in LDS, scores of tile 0
            const int i1 = min(1, ntiles - 1);
            fill(kbase, Ks0, kcol, seq(0, 0), seq_word(0, 0), kKOdd);
            fill(vbase, Vs0, vcol, seq(0, 0), seq_word(0, 0), 0u);
            fill(kbase, Ks1, kcol, seq(i1, 0), seq_word(i1, 0), kKOdd);
            fills_done();
            __syncthreads();
            scores(s0, Ks0);
#pragma unroll
            for (int j = 0; j < kQueue; ++j) fq[j] = read_k(Ks1, j);  // the first step's first operands
            // the first step refills K(0)'s buffer at once: every wave must be done reading it
            wg_barrier();
            if constexpr (!kSafe) {
#pragma unroll
                for (int r = 0; r < RB; ++r) {
                    float mloc = fmaxf(s0[r][0][0], s0[r][1][0]);
#pragma unroll
                    for (int i = 1; i < 16; ++i) mloc = fmaxf(mloc, fmaxf(s0[r][0][i], s0[r][1][i]));
                    m_ref[r] = ksa_pair_max(mloc);
                }
            }
        }
        int it = 0;
        for (; it + 2 <= n_a; it += 2) {
            step(safe_tag, A{}, Even{}, it, s0, s1, it < nquick + ncheap);
            step(safe_tag, A{}, Odd{}, it + 1, s1, s0, it + 1 < nquick + ncheap);
        }
        if (it < n_a) {
            step(safe_tag, A{}, Even{}, it, s0, s1, it < nquick + ncheap);
            copy_scores();
            ++it;
        }
        if ((it & 1) && it < ntiles) {  // phase B starts on an odd tile: one step to realign
            step(safe_tag, B{}, Odd{}, it, s0, s1, false);
            copy_scores();
            ++it;
        }
        for (; it + 2 <= ntiles; it += 2) {
            step(safe_tag, B{}, Even{}, it, s0, s1, false);
            step(safe_tag, B{}, Odd{}, it + 1, s1, s0, false);
        }
        if (it < ntiles) step(safe_tag, B{}, Even{}, it, s0, s1, false);
    };

    walk(std::false_type{});
    {
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const float l_tot = ksa_pair_sum(l_run[r]);
            // Every row sees at least itself: a small sum means a reference far too high.  How
            // small depends on what the 16-bit probabilities can hold.  bf16 has fp32's exponent
            // range, so only a vanishing sum (below 2^-64) loses anything.  fp16 is exact in
            // relative terms down to 2^-14 and absolute (steps of 2^-24) below: with a row sum
            // of at least 2^-4 the rounding of n probabilities adds up to at most n 2^-25 / 2^-4
            // of the sum (2^-8 for 8192 keys, in practice its square root); below that the row
            // is walked again with exact references.
            constexpr float kMinRowSum = std::is_same<T, KsaF16>::value ? 0.0625f : 5.4e-20f;
            bad = bad || !(l_tot > kMinRowSum);
        }
        if (__syncthreads_or(bad)) {
            walk(std::true_type{});
            __syncthreads();  // the epilogue reuses the tiles' LDS
        }
    }

    // ---- epilogue ----
    // The normalised rows go to global memory through LDS (the K/V tiles are dead by now): in the
    // accumulator layout a lane holds 4-element pieces of its query row, and a store instruction
    // straight from there would touch 32 rows in 16-byte pieces; turned around in LDS, every
    // store instruction writes four whole rows of 2 D bytes (3 us less per workgroup).  A wave's
    // 32-row block has its own LDS region (16-byte chunk c of row r at position c ^ (r % CPR):
    // conflict-free both ways), so waves do not wait for each other.
    if constexpr (RB != 1) ksa_mfma_settle();
    {
        const int q0 = wave_u * RB;  // first region of this wave; two regions per 64-row LDS array
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const float l_tot = ksa_pair_sum(l_run[r]);
            const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
            const int qreg = q0 + r;
            uint16_t* arr = (qreg >> 1) == 0 ? Ks0 : (qreg >> 1) == 1 ? Ks1 : (qreg >> 1) == 2 ? Vs0 : Vs1;
            char* region = reinterpret_cast<char*>(arr) + (qreg & 1) * 32 * ROWB;
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    u32x2 w;
                    w[0] = Ops::pack2(oacc[r][b][4 * j] * inv, oacc[r][b][4 * j + 1] * inv);
                    w[1] = Ops::pack2(oacc[r][b][4 * j + 2] * inv, oacc[r][b][4 * j + 3] * inv);
                    const int pch = (4 * b + j) ^ (lq & (CPR - 1));
                    *reinterpret_cast<u32x2*>(region + lq * ROWB + pch * 16 + 8 * lh) = w;
                }
            ksa_wave_lds_fence();
            const int brow0 = row0 + 32 * r;  // first query row of the block
            uint16_t* ob = p.out + bz * p.o_bs + head * p.o_hs;
#pragma unroll
            for (int i = 0; i < (32 * CPR) / 64; ++i) {
                const int idx = i * 64 + lane;
                const int row = idx / CPR, c = idx % CPR;
                const u32x4 w = *reinterpret_cast<const u32x4*>(region + row * ROWB + ((c ^ (row & (CPR - 1))) * 16));
                if (brow0 + row < mk.Sq)
                    *reinterpret_cast<u32x4*>(ob + (int64_t)(brow0 + row) * p.o_rs + 8 * c) = w;
            }
            if (p.lse && lh == 0 && qrow[r] < mk.Sq)
                p.lse[bz * p.lse_bs + head * p.lse_hs + qrow[r]] =
                    l_tot > 0.f ? m_ref[r] * p.scale + logf(l_tot) : -INFINITY;
        }
    }
}

__global__ void ksa_prefill_zero_queues_kernel(int32_t* sched) {
    if (threadIdx.x < 8) sched[threadIdx.x] = 0;
}

// whether a launch can use the kernel variant with regular tile addressing (see kRegular)
template <int D, int RB, int HW>
bool prefill_regular(const PrefillParams& p) {
    constexpr int RSTEP = PrefillShape<RB, HW>::kThreads / (D / 8);
    const KsaMask& mk = p.mk;
    const bool prefix_ok = mk.P == 0 || p.phys_prefix || (RSTEP % mk.S == 0 && mk.P % kTileN == 0);
    return prefix_ok && mk.Sk % kTileN == 0;
}

template <typename T, int D, int RB, int HW>
int launch_shape(const PrefillParams& p, int batch, hipStream_t stream) {
    constexpr int kThreads = PrefillShape<RB, HW>::kThreads;
    const bool regular = prefill_regular<D, RB, HW>(p);
    if ((KSA_PREFILL_VARIANTS == 1 && !regular) || (KSA_PREFILL_VARIANTS == 2 && regular)) return KSA_ERR_INVALID;
    PrefillParams pp = p;
    pp.n_items = p.M * (p.Hq / HW);
    pp.total = pp.n_items * batch;
    pp.n_static = pp.total;
    int spare = 0;
    // Queues only for long launches (32 workgroups per CU and more; measured at 128k rows: +2.2 %,
    // at 32k rows with 17 per CU: -0.8 %), where the tail they even out is worth the clearing kernel
    // and the atomic in front of the light items: the last 30 % of the items, with a quarter more
    // workgroups than items there (the spare ones find the queues empty and leave).
    if (p.sched != nullptr && (int64_t)pp.total >= 32ll * ksa_cu_count_or(256)) {
        pp.n_static = (int)((int64_t)pp.total * 7 / 10) / 8 * 8;
        spare = ((pp.total - pp.n_static) / 4 + 7) / 8 * 8;
        hipLaunchKernelGGL(ksa_prefill_zero_queues_kernel, dim3(1), dim3(64), 0, stream, p.sched);
    } else {
        pp.sched = nullptr;
    }
    dim3 grid(pp.total + spare);
#if KSA_PREFILL_VARIANTS != 2
    if (regular) hipLaunchKernelGGL((ksa_prefill_kernel<T, D, true, RB, HW>), grid, dim3(kThreads), 0, stream, pp);
#endif
#if KSA_PREFILL_VARIANTS != 1
    if (!regular) hipLaunchKernelGGL((ksa_prefill_kernel<T, D, false, RB, HW>), grid, dim3(kThreads), 0, stream, pp);
#endif
    return ksa_check_launch();
}

template <typename T, int D>
int launch(const PrefillParams& p, int batch, hipStream_t stream) {
    // workgroup shapes with two heads need an even group size and are built for D = 128
    if constexpr (D == 128) {
        if (p.g % 2 == 0) {
            if (p.shape == 64) return launch_shape<T, D, 2, 2>(p, batch, stream);
            if (p.shape == 2) return launch_shape<T, D, 1, 2>(p, batch, stream);
        }
    }
    return launch_shape<T, D, 1, 1>(p, batch, stream);
}

#if KSA_PREFILL_UNIT == 0
bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }
bool stride_ok(int64_t s) { return (s % 8) == 0; }
#endif

}  // namespace

// head_dim 256: one launcher per translation unit (they all see the same PrefillParams)
int ksa_prefill_launch_d256_bf16_regular(const void* params, int batch, void* stream);
int ksa_prefill_launch_d256_bf16_general(const void* params, int batch, void* stream);
int ksa_prefill_launch_d256_f16_regular(const void* params, int batch, void* stream);
int ksa_prefill_launch_d256_f16_general(const void* params, int batch, void* stream);
#if KSA_PREFILL_UNIT == 1
int ksa_prefill_launch_d256_bf16_regular(const void* params, int batch, void* stream) {
    return launch<KsaBf16, 256>(*static_cast<const PrefillParams*>(params), batch, (hipStream_t)stream);
}
#elif KSA_PREFILL_UNIT == 2
int ksa_prefill_launch_d256_bf16_general(const void* params, int batch, void* stream) {
    return launch<KsaBf16, 256>(*static_cast<const PrefillParams*>(params), batch, (hipStream_t)stream);
}
#elif KSA_PREFILL_UNIT == 3
int ksa_prefill_launch_d256_f16_regular(const void* params, int batch, void* stream) {
    return launch<KsaF16, 256>(*static_cast<const PrefillParams*>(params), batch, (hipStream_t)stream);
}
#elif KSA_PREFILL_UNIT == 4
int ksa_prefill_launch_d256_f16_general(const void* params, int batch, void* stream) {
    return launch<KsaF16, 256>(*static_cast<const PrefillParams*>(params), batch, (hipStream_t)stream);
}
#else

extern "C" int ksa_prefill_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                               int batch, int Sq, int Hq, int Hkv, int D, int dtype,
                               const int64_t* q_strides, const int64_t* kv_strides,
                               const int64_t* out_strides, int C, int S, int W, int P,
                               int skip_old, int phys_prefix, const int32_t* mask_cnt,
                               const int32_t* mask_idx, const int32_t* full_cnt,
                               const int32_t* full_idx, int idx_stride, float scale, int shape,
                               int32_t* sched, void* stream) {
    if (!q || !k || !v || !out || !mask_cnt || !mask_idx || !full_cnt || !full_idx) return KSA_ERR_NULL;
    if (!q_strides || !kv_strides || !out_strides) return KSA_ERR_NULL;
    if (batch <= 0 || Sq <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return KSA_ERR_INVALID;
    if (C <= 0 || S <= 0 || W < 0 || P < 0) return KSA_ERR_INVALID;
    if ((int64_t)Sq + P >= (1ll << 30)) return KSA_ERR_INVALID;
    if (dtype != KSA_DTYPE_BF16 && dtype != KSA_DTYPE_F16) return KSA_ERR_UNSUPPORTED;
    if (shape != 0 && shape != 2 && shape != 32 && shape != 64) return KSA_ERR_INVALID;
    const int Sk = Sq + P;
    const int N = (Sk + kTileN - 1) / kTileN;
    if (idx_stride < N) return KSA_ERR_INVALID;
    // K/V rows are addressed with 32-bit byte offsets inside one (batch, head) slice
    const int64_t kv_rows = phys_prefix ? Sk : Sq;
    if (kv_rows * kv_strides[1] * 2 >= (1ll << 32)) return KSA_ERR_INVALID;
    if (!phys_prefix && P > 0) {
        // in-place prefix: row j is in-line row (j/S)*B + C + j%S, which must exist
        const int64_t last = (int64_t)((P - 1) / S) * (C + S) + C + (P - 1) % S;
        if (last >= Sq) return KSA_ERR_INVALID;
    }
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return KSA_ERR_ALIGN;
    for (int i = 0; i < 3; ++i)
        if (!stride_ok(q_strides[i]) || !stride_ok(kv_strides[i]) || !stride_ok(out_strides[i]))
            return KSA_ERR_ALIGN;

    PrefillParams p{};
    p.q = (const uint16_t*)q;
    p.k = (const uint16_t*)k;
    p.v = (const uint16_t*)v;
    p.out = (uint16_t*)out;
    p.lse = lse;
    p.mask_cnt = mask_cnt;
    p.mask_idx = mask_idx;
    p.full_cnt = full_cnt;
    p.full_idx = full_idx;
    p.idx_stride = idx_stride;
    p.M = (Sq + kTileM - 1) / kTileM;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.g = Hq / Hkv;
    p.phys_prefix = phys_prefix ? 1 : 0;
    p.q_bs = q_strides[0], p.q_rs = q_strides[1], p.q_hs = q_strides[2];
    p.kv_bs = kv_strides[0], p.kv_rs = kv_strides[1], p.kv_hs = kv_strides[2];
    p.o_bs = out_strides[0], p.o_rs = out_strides[1], p.o_hs = out_strides[2];
    p.lse_bs = (int64_t)Hq * Sq;
    p.lse_hs = Sq;
    p.mk = KsaMask{C, S, W, P, skip_old ? 1 : 0, Sq, Sk};
    p.scale = scale;
    p.scale_log2 = scale * 1.4426950408889634f;
    p.sched = sched;
    // Workgroup shape (D = 128, even group size; anything else uses one head per workgroup):
    // 2 = two heads on 8 waves; 32 = one head on 4 waves; 64 = two heads on 4 waves with 64 query
    // rows per wave (one wave per SIMD).  Left to the library (0), a short launch (fewer than 16
    // two-head workgroups per CU of the device) takes the one-head shape: two of its workgroups
    // share a CU and hide each other's start and end (8k rows: +9 %, 16k: +4 %, 24k: +1.5 %,
    // 32k rows and up: the same within 1 %); longer launches take two heads on 8 waves.
    p.shape = shape ? shape : ((int64_t)p.M * (Hq / 2) * batch < 16ll * ksa_cu_count_or(256) ? 32 : 2);

    hipStream_t st = (hipStream_t)stream;
    if (dtype == KSA_DTYPE_BF16) {
        if (D == 128) return launch<KsaBf16, 128>(p, batch, st);
        if (D == 64) return launch<KsaBf16, 64>(p, batch, st);
        if (D == 256)
            return prefill_regular<256, 1, 1>(p) ? ksa_prefill_launch_d256_bf16_regular(&p, batch, stream)
                                                 : ksa_prefill_launch_d256_bf16_general(&p, batch, stream);
    } else {
        if (D == 128) return launch<KsaF16, 128>(p, batch, st);
        if (D == 64) return launch<KsaF16, 64>(p, batch, st);
        if (D == 256)
            return prefill_regular<256, 1, 1>(p) ? ksa_prefill_launch_d256_f16_regular(&p, batch, stream)
                                                 : ksa_prefill_launch_d256_f16_general(&p, batch, stream);
    }
    return KSA_ERR_UNSUPPORTED;  // other head dimensions: the caller pads to 64 / 128 / 256
}
#endif  // KSA_PREFILL_UNIT
