// lv_mega.h — the whole decode step of one token as ONE persistent kernel (gfx950, 256 CUs).
//
// Why: at batch 1 a layer is five tiny dependent GEMVs (1-6 us of HBM time each).  Launched one by one
// they spend more time draining, launching and refilling the memory pipeline than streaming weights.
// Here one workgroup per CU stays resident for the whole token; every wavefront walks its own contiguous
// weight stream with a register queue (8 q4_0 tiles or 4 q8_0 tiles deep) of 128-bit loads that keeps running across the phase
// boundaries, so HBM stays busy while the workgroups exchange the small activation vectors.
//
// Phases of a layer (llava_layer.cpp:53-73), each separated by a data hand-over through HBM/L2:
//   A  norm + [Wq;Wk;Wv] x        -> q, new K/V row (fp16 into the cache)
//   B  single-query attention, 8 (or 6) position chunks per head -> partial numerators / denominators
//   B' combine the chunks         -> o
//   C  x += Wo o                  -> x1
//   D  norm + (W3 x1)*silu(W1 x1) -> ff
//   E  x1 += W2 ff                -> x2 (next layer's x)
// then norm + output matrix -> logits.
//
// Hand-over without barriers: every exchanged float lives in a buffer that holds the bit pattern
// 0xFFFFFFFF ("not written yet") until its producer stores the value with a device-scope write-through
// store; consumers poll the data itself with device-scope loads.  No flag, no fence, no wait for store
// acknowledgement.  Two buffer sets alternate between tokens; each token re-arms the other set.
// Every poll loop is bounded: on expiry the kernel raises *status and carries on to its end.
// The vectors every workgroup reads (o, x1, ff, x2) lie in uncached device memory, where such a hand-over between
// XCDs is a third shorter; q, k, v and the partial sums go from a head's producers to that head's own workgroups
// only, which a launch normally places on one XCD: those two hand-overs then go through the XCD's L2 (ld_xcd).
//
// Weight stream: for each (layer, phase, workgroup, wave) the tiles that wave will consume, in order.
// A tile is one matrix row restricted to the wave's 64-block column slab: 64 x 16 B (q4_0) or two planes of 64 x 16 B
// (q8_0: first and second half of every block's codes) + 64 x fp16 scales (1152 B / 2176 B).  Lane l of the wave always owns
// block column 64*slab + l, so the 32 activations of that column sit in registers for the whole phase.  Where a row ends in
// half a slab (D = 5120: 2.5 slabs) the tiles of that half slab carry two rows, 32 blocks of each, so that no lane idles.
#pragma once

#include "lv_device.h"

namespace lv {

constexpr uint32_t kNotReady = 0xFFFFFFFFu;
constexpr int kMegaWGs = 256;
constexpr int kMegaVocabRows = 125;     // output-matrix rows per workgroup the head phase is laid out for (32000 / 256)
// Default bound on the polls of one hand-over (MegaArgs::spin_limit).  A hand-over normally takes one to three polls of
// about 1.3 us; 16384 of them (20 ms) only run out when the workgroups are not all resident, and a token whose every
// hand-over ran out still ends within seconds.
constexpr uint32_t kSpinLimit = 1u << 14;
constexpr int kStatusToken = 2;         // word of the status block that receives the index of the largest logit
constexpr int kStatusXcd = 3;           // word that tells whether workgroup 0 handed over inside its XCD in the last launch
// A consumer reaches a hand-over about when its producers store: a load issued at once samples memory before the
// stores are visible (0.6 us) yet comes back only after the prefetched tiles ahead of it on the CU's return path
// (1-2 us), and the second try pays that again.  Sleeping this many 64-clock units first makes the first try
// succeed; measured optimum, flat between 16 and 32.
constexpr int kPollDelay = 24;

__device__ __forceinline__ uint32_t ld_dev(const uint32_t *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev(float *p, float v)
{
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p), __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Hand-overs inside one XCD.  The workgroups of a launch go to the XCDs in turn (workgroups b and b + 8 run on the same
// XCD; which one workgroup 0 gets depends on what was dispatched before, and launches of other streams dispatched in
// between break the pattern, so every launch looks: see the kernel's first layer), and the CUs of an XCD share its L2.  A plain store is written through the CU's cache into that L2, and a non-temporal load
// does not stop at the CU's cache, so a value stored by one workgroup is seen by another one of the same XCD after one
// L2 round trip: 0.5 us for a flag bounced between two such workgroups, against 1.1 us with the device-scope pair above,
// whose store has to reach memory (measured; a load with only sc0 set keeps hitting the CU's own cache and never sees
// the store).  Across XCDs only the device-scope pair works.
__device__ __forceinline__ uint32_t ld_xcd(const uint32_t *p) { return __builtin_nontemporal_load(p); }

// Where a workgroup stands in the attention phase: the 32 workgroups with one value of b % 8 hold H / 8 heads, for each of them the CPH workgroups that
// take a chunk of the cache each; chunk 0 also combines the chunks.  The same XCD computes the query, key and value rows
// of its heads in phase A, so these two hand-overs stay inside the XCD.
template <class S>
struct MegaPlace {
    int xcd, slot, h, c;
    bool attends;
    __device__ __forceinline__ explicit MegaPlace(int b)
    {
        static_assert(S::H % 8 == 0 && (S::H / 8) * S::CPH <= kMegaWGs / 8, "heads must split over eight XCDs");
        xcd = b & 7; slot = b >> 3;
        const int hl = slot / S::CPH;
        c = slot % S::CPH;
        attends = hl < S::H / 8;
        h = hl * 8 + xcd;
    }
};
// row t of workgroup b in phase A: which of q, k, v (0..2) and which of its D rows
template <class S>
__host__ __device__ __forceinline__ void mega_qkv_row(int b, int t, int &which, int &row)
{
    const int lr = (b >> 3) * S::ROWS_A + t;            // among the 3 R H / 8 rows of the XCD's heads
    const int hl = lr / (3 * S::R), within = lr % (3 * S::R);
    which = within / S::R;
    row = (hl * 8 + (b & 7)) * S::R + within % S::R;
}

// Workgroup barrier that orders LDS traffic only: global loads of the weight queue stay in flight across it
// (__syncthreads would wait for vmcnt(0) and drain the queue at every phase step).
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// A value the compiler has to take as new each time: what is computed from it inside the layer loop (LDS addresses above
// all) is then computed there, a few instructions each, instead of once in front of the loop and kept in registers.  Used
// (OPAQUE) by the shape classes whose kernel would otherwise spill; where registers suffice, keeping the values is faster.
template <bool OPAQUE>
__device__ __forceinline__ int maybe_opaque(int v)
{
    if constexpr (OPAQUE) asm volatile("" : "+v"(v));
    return v;
}

constexpr int cdiv(int a, int b) { return (a + b - 1) / b; }
constexpr int round_up(int a, int b) { return cdiv(a, b) * b; }

// Static shape of one model class.  NW = wavefronts per workgroup.
// SF32_: the tiles carry fp32 block scales (a version-1 file, llava_buffer.cpp:193-224) instead of fp16 ones.
template <int D_, int F_, int H_, int NW_, int QT_, int DEPTH_, bool SF32_>
struct MegaShapeBase {
    static constexpr int D = D_, F = F_, H = H_, NW = NW_, R = 128;
    static constexpr int QT = QT_;                               // 4: q4_0, 8: q8_0
    static constexpr int CODE = QT == 4 ? 16 : 32;               // bytes of codes per block
    static constexpr bool SF32 = SF32_;
    static constexpr int TILE = 64 * CODE + (SF32 ? 256 : 128);  // bytes per tile: 64 blocks of codes, 64 fp16 (or fp32) scales
    static constexpr int DEPTH = DEPTH_ ? DEPTH_ : (QT == 4 ? 4 : 2);   // tiles in flight per wave
    static constexpr int NBD = D / 32, NBF = F / 32;            // blocks per row
    static constexpr int NSD = cdiv(NBD, 64), NSF = cdiv(NBF, 64);  // column slabs
    // D-wide phases (A, C, D, head).  A row of D = 4096 is two full slabs of 64 blocks; a row of D = 5120 is two full slabs and
    // HALF a slab (32 blocks).  Tiles of the half slab carry TWO rows, 32 blocks of each (lanes 0-31 row 2p, lanes 32-63 row
    // 2p + 1; a lane's block column is the same for both), so every lane of every tile works and every queue slot holds a
    // full tile.  The waves are dealt to the slabs by their work: WPF waves to each full slab (one tile per row), WPH to the
    // half slab (one tile per two rows).
    static constexpr int FULLD = NBD / 64, HALFD = NBD % 64 ? 1 : 0;
    static_assert(NBD % 64 == 0 || NBD % 64 == 32, "a row is full slabs plus at most half a slab");
    static constexpr int WPH = HALFD ? (NW + FULLD) / (2 * FULLD + 1) : 0, WPF = (NW - WPH) / FULLD;
    static_assert(WPF >= 1 && (!HALFD || WPH >= 1), "waves for every slab");
    // tiles (queue slots) a wave has in a D-wide phase of `rows` rows, and the tiles a half-slab wave really has of them
    static constexpr int tiles_half(int rows) { return HALFD ? cdiv(cdiv(rows, 2), WPH) : 0; }
    static constexpr int tiles_d(int rows) { return cdiv(rows, WPF) > tiles_half(rows) ? cdiv(rows, WPF) : tiles_half(rows); }
    static constexpr int NRF = NW / NSF;                        // row sets of the F-wide phase (waves sharing a slab split the rows)
    static constexpr int ROWS_A = 3 * D / kMegaWGs, ROWS_C = D / kMegaWGs, ROWS_D = 2 * F / kMegaWGs, ROWS_E = D / kMegaWGs;
    // Down projection (phase E).  Where the waves outnumber the column slabs (7B: six slabs, eight waves) the spare waves take
    // the last E_SPARE_ROWS rows of E_SPARE_SLABS slabs each, so that every wave has the same number of tiles (12 instead of 16
    // for six waves); a spare wave's tile i is row ROWS_E - E_SPARE_ROWS + i % E_SPARE_ROWS of slab (w - NSF) * E_SPARE_SLABS + i / E_SPARE_ROWS.
    static constexpr int E_SPARE = NRF == 1 ? NW - NSF : 0;
    static constexpr bool E_REDEAL = E_SPARE > 0 && (ROWS_E * NSF) % NW == 0 && NSF % E_SPARE == 0 &&
                                     (ROWS_E - ROWS_E * NSF / NW) % 4 == 0 && (ROWS_E * NSF / NW) % 4 == 0 &&
                                     (ROWS_E - ROWS_E * NSF / NW) * (NSF / E_SPARE) == ROWS_E * NSF / NW;
    static constexpr int E_SPARE_SLABS = E_REDEAL ? NSF / E_SPARE : 0, E_SPARE_ROWS = E_REDEAL ? ROWS_E - ROWS_E * NSF / NW : 0;
    // phase E where every working wave owns exactly one column slab (a wave without one idles): each fetches its own part of
    // the input vector (acquire_own_slab).  Where spare waves take rows of several slabs (E_REDEAL) the common fetch by all
    // threads is as fast.
    static constexpr bool OWN_SLAB_E = NRF == 1 && !E_REDEAL;
    static constexpr int TA = tiles_d(ROWS_A), TC = tiles_d(ROWS_C), TD = tiles_d(ROWS_D),
                         TE = E_REDEAL ? ROWS_E * NSF / NW : cdiv(ROWS_E, NRF);
    static constexpr int SEQ_A = 0, SEQ_C = TA, SEQ_D = TA + TC, SEQ_E = TA + TC + TD;
    static constexpr int PER_LAYER = round_up(TA + TC + TD + TE, DEPTH);
    static constexpr int MAX_VOCAB_ROWS = kMegaVocabRows + 3;           // output-matrix rows per workgroup the kernel has room for (vocabularies up to 32768)
    static constexpr int HEAD = round_up(tiles_d(MAX_VOCAB_ROWS), 4);   // head tiles per wave (static upper bound)
    static constexpr int CPH = kMegaWGs / H;                    // position chunks per head
    static constexpr int PART = R + 4;                          // floats per partial (128 numerators, denominator, pad)
    // floats of one layer's hand-over buffers
    // two buffers: what stays inside an XCD (q, k, v, the chunks' partial sums) and what every workgroup reads
    static constexpr int OFF_QKV = 0, OFF_PART = 3 * D, LOCAL_LAYER = OFF_PART + H * CPH * PART;
    static constexpr int OFF_O = 0, OFF_X1 = OFF_O + D, OFF_FF = OFF_X1 + D, OFF_X2 = OFF_FF + F, XCHG_LAYER = OFF_X2 + D;
    static_assert(LOCAL_LAYER % 4 == 0 && XCHG_LAYER % 4 == 0, "re-armed sixteen bytes at a time");
    // after the layers: every workgroup's best logit (value, index), then the XCD every workgroup found itself on
    static constexpr int XCHG_TAIL = 3 * kMegaWGs, OFF_XCC = 2 * kMegaWGs;
    static_assert((3 * D) % kMegaWGs == 0 && (2 * F) % kMegaWGs == 0 && D % kMegaWGs == 0, "rows must split over 256 workgroups");
    static_assert(H * R == D && CPH >= 1 && NRF >= 1, "shape");
    // bytes of the weight stream of one layer
    static constexpr size_t PHASE_A_BYTES = (size_t)kMegaWGs * NW * TA * TILE, PHASE_C_BYTES = (size_t)kMegaWGs * NW * TC * TILE,
                            PHASE_D_BYTES = (size_t)kMegaWGs * NW * TD * TILE, PHASE_E_BYTES = (size_t)kMegaWGs * NW * TE * TILE;
    static constexpr size_t LAYER_BYTES = PHASE_A_BYTES + PHASE_C_BYTES + PHASE_D_BYTES + PHASE_E_BYTES;
    static constexpr size_t HEAD_BYTES = (size_t)kMegaWGs * NW * HEAD * TILE;
};
// the shape classes the kernel is instantiated for: fp16 block scales (file version 3), fp32 ones (version 1)
template <int D_, int F_, int H_, int NW_, int QT_, int DEPTH_ = 0>
struct MegaShape : MegaShapeBase<D_, F_, H_, NW_, QT_, DEPTH_, false> {};
template <int D_, int F_, int H_, int NW_, int QT_, int DEPTH_ = 0>
struct MegaShapeV1 : MegaShapeBase<D_, F_, H_, NW_, QT_, DEPTH_, true> {};

// phase E of a re-dealt shape: row (of the workgroup's ROWS_E) and column slab of tile i of wave w
template <class S>
__host__ __device__ __forceinline__ void mega_e_tile(int w, int i, int &row, int &slab)
{
    constexpr int SR = S::E_SPARE_ROWS > 0 ? S::E_SPARE_ROWS : 1;   // shapes without spare rows never take the second branch
    if (w < S::NSF) { row = i; slab = w; }
    else { row = S::ROWS_E - S::E_SPARE_ROWS + i % SR; slab = (w - S::NSF) * S::E_SPARE_SLABS + i / SR; }
}

struct MegaArgs {
    const uint8_t *wstream;    // [layers] x LAYER_BYTES, then HEAD_BYTES, then one all-zero tile
    const float *norms;        // [layers][2][D] (attention_norm, ffn_norm), then the final norm [D]
    const float *tok_f32;      // embedding table [vocab][D] (fp32)
    uint16_t *kv;              // [layers][2][backlog][D] fp16
    const float2 *trig;        // [backlog][64]
    float *xchg;               // this token's hand-over buffers for the vectors every workgroup reads: [layers] x XCHG_LAYER +
                               // XCHG_TAIL floats, all kNotReady.  Uncached device memory: a flag bounced between two XCDs takes
                               // 0.80 us per round trip there against 1.24 us in ordinary memory (measured)
    float *xchg_rearm;         // the other set, re-armed to kNotReady during this token
    float *xl, *xl_rearm;      // the same for what stays inside an XCD: [layers] x LOCAL_LAYER floats of ordinary memory (ld_xcd)
    float *logits;             // [vocab]
    uint32_t *status;          // host-visible; [0] set non-zero when a poll loop expired, [kStatusToken] = greedy pick
    uint32_t layers, vocab, backlog, pos, token;
    uint32_t spin_limit;       // polls per hand-over before the step is given up (kSpinLimit; tests of the failure path lower it)
    uint32_t xcd_local;        // non-zero: the hand-overs between the workgroups of a head may go through their XCD's L2 (ld_xcd)
                               // where the launch placed all of them on one XCD; zero: device scope everywhere
};

struct MegaTile {
    uint4 c, c2;   // c2: second half of the codes of a q8_0 block (unused for q4_0)
    uint16_t d;    // fp16 scale bits
    uint32_t d32;  // fp32 scale bits (shapes with SF32; the other member is unused then, and this one otherwise)
};

template <class S>
__device__ __forceinline__ void load_tile(MegaTile &t, const uint8_t *p, int lane)
{
    // Non-temporal loads: the weights pass once per token and need no place in the caches, which the cache rows, the norm
    // weights and the hand-over vectors then keep (measured: a pure read stream reaches 6.9 instead of 6.1-6.2 TB/s with
    // them; the 7B q4_0 token takes 3 % less, the q8_0 tokens 6-7 % less).  Every load of a wave covers one contiguous
    // kilobyte: without the CU's cache a second load into the same cache line would be a request of its own.
    if constexpr (S::QT == 4) {
        typedef uint32_t nt_u4v __attribute__((ext_vector_type(4)));
        const nt_u4v v = __builtin_nontemporal_load(reinterpret_cast<const nt_u4v *>(p + lane * S::CODE));
        t.c = make_uint4(v.x, v.y, v.z, v.w);
    } else {
        // q8_0: the two halves of a block's codes lie in two planes of the tile (64 x 16 bytes each), so that either load of
        // a wave covers one contiguous kilobyte
        typedef uint32_t nt_u4v __attribute__((ext_vector_type(4)));
        const nt_u4v v = __builtin_nontemporal_load(reinterpret_cast<const nt_u4v *>(p + lane * 16));
        const nt_u4v v2 = __builtin_nontemporal_load(reinterpret_cast<const nt_u4v *>(p + 1024 + lane * 16));
        t.c = make_uint4(v.x, v.y, v.z, v.w);
        t.c2 = make_uint4(v2.x, v2.y, v2.z, v2.w);
    }
    if constexpr (S::SF32) t.d32 = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p + 64 * S::CODE + lane * 4));
    else t.d = __builtin_nontemporal_load(reinterpret_cast<const uint16_t *>(p + 64 * S::CODE + lane * 2));
}

// one block column of one row: sum over 32 weights of w * x, from the raw codes
template <class S>
__device__ __forceinline__ float tile_dot(const MegaTile &t, const float (&xr)[32], float xsum)
{
    float d;
    if constexpr (S::SF32) d = __uint_as_float(t.d32);
    else d = half_bits_to_float(t.d);
    if constexpr (S::QT == 4) return (q4_block_dot(t.c, xr) - 8.f * xsum) * d;
    else return (q8_block_dot(t.c, t.c2, xr) - 128.f * xsum) * d;
}

// ---- polling helpers ----------------------------------------------------------------------------------------
// N values strided by `stride` elements starting at p; spins until none of them is the not-ready pattern.
template <int N, int SLEEP = 0, bool XCD = false>
__device__ __forceinline__ void poll_values(float (&v)[N], const float *p, int stride, const bool (&want)[N], uint32_t *status,
                                            uint32_t spin_limit, int group_stride = 0 /* when non-zero: element j lives at p[(j/8)*8*group_stride + j%8] */)
{
    uint32_t spins = 0;
    bool pending;
    if constexpr (SLEEP > 0) __builtin_amdgcn_s_sleep(SLEEP);
    do {
        pending = false;
        if constexpr (XCD) asm volatile("" ::: "memory");      // the loads below are ordinary ones: every turn has to issue them again
#pragma unroll
        for (int j = 0; j < N; j++) {
            uint32_t u = 0;
            const size_t off = group_stride ? (size_t)(j / 8) * 8 * group_stride + (j % 8) : (size_t)j * stride;
            if (want[j]) u = XCD ? ld_xcd(reinterpret_cast<const uint32_t *>(p) + off) : ld_dev(reinterpret_cast<const uint32_t *>(p) + off);
            v[j] = __uint_as_float(u);
            pending |= (u == kNotReady);
        }
    } while (pending && ++spins < spin_limit);
    if (pending) *status = 1u;
}

// The phase's input vector sits in LDS block by block (32 floats = 128 bytes), and lane l of a wave reads block
// 64 * slab + l: in plain order the 64 lanes of a 128-bit read would all fall on the same four banks (measured: 0.8 us
// per phase between the vector's arrival and the first tile).  Inside each block the eight 16-byte groups are therefore
// rotated by the block index, so that eight consecutive lanes cover all 32 banks.
__device__ __forceinline__ int xs_index(int idx)
{
    return (idx & ~31) | ((((idx >> 2) + (idx >> 5)) & 7) << 2) | (idx & 3);
}

// the 32 activations of this lane's block column, from LDS
template <bool OPAQUE = false>
__device__ __forceinline__ void load_slab(float (&xr)[32], float &xsum, const float *xs, int block, bool have)
{
    const int blk = maybe_opaque<OPAQUE>(have ? block : 0);
    const float *src = xs + blk * 32;
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        float4 v = *reinterpret_cast<const float4 *>(src + 4 * ((j + blk) & 7));
        if (!have) v = make_float4(0.f, 0.f, 0.f, 0.f);
        xr[4 * j] = v.x; xr[4 * j + 1] = v.y; xr[4 * j + 2] = v.z; xr[4 * j + 3] = v.w;
        s += (v.x + v.y) + (v.z + v.w);
    }
    xsum = s;
}

// Everything a wave needs to find its tiles.
template <class S>
struct MegaWave {
    const uint8_t *wstream, *dummy /* one all-zero tile after the head */;
    uint32_t layers, vocab_rows /* head rows per workgroup */, vocab;
    int b, w, lane;
    // per phase geometry (column slab, row set, whether the wave works in the phase, whether the lane has a column)
    int sD, rD, sF, rF, blockD /* this lane's block column in the D-wide phases */;
    bool actD, actF, laneF, halfD /* the wave works on the half slab: two rows per tile */;

    __device__ __forceinline__ void init(const MegaArgs &a)
    {
        wstream = a.wstream; layers = a.layers; vocab = a.vocab;
        dummy = a.wstream + (size_t)a.layers * S::LAYER_BYTES + S::HEAD_BYTES;
        vocab_rows = (a.vocab + kMegaWGs - 1) / kMegaWGs;
        // the wave index is uniform: telling the compiler so keeps every tile address in scalar registers
        b = blockIdx.x; w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); lane = threadIdx.x & 63;
        halfD = S::HALFD && w >= S::FULLD * S::WPF && w < S::FULLD * S::WPF + S::WPH;
        actD = w < S::FULLD * S::WPF + S::WPH;
        sD = halfD ? S::FULLD : w % S::FULLD;
        rD = halfD ? w - S::FULLD * S::WPF : w / S::FULLD;
        blockD = halfD ? S::FULLD * 64 + (lane & 31) : sD * 64 + lane;
        sF = w % S::NSF; rF = w / S::NSF; actF = rF < S::NRF; laneF = sF * 64 + lane < S::NBF;
    }

    // Loads sequence slot k (relative to the start of `layer`; k >= PER_LAYER runs into the next layer, or into
    // the head after the last layer).  k is a compile-time constant after unrolling, so whether a slot loads at
    // all is static; every runtime condition (row past the end, lane without a column, last layer) only selects
    // the address: an invalid tile reads the all-zero dummy tile at the end of the stream.  Straight-line loads
    // let the compiler count outstanding loads exactly and wait with vmcnt(N > 0).
    __device__ __forceinline__ void fetch(MegaTile &t, int k, uint32_t layer) const
    {
        const bool wrapped = k >= S::PER_LAYER;
        if (wrapped) { k -= S::PER_LAYER; layer += 1; }
        const bool into_head = wrapped && layer >= layers;  // uniform, runtime
        int i = 0, tiles = 0, rows = 0, rset = 0;
        bool act = false, lane_ok = false, real = true, dwide = true;
        size_t off = 0;
        if (k < S::SEQ_C) { i = k; tiles = S::TA; rows = S::ROWS_A; }
        else if (k < S::SEQ_D) { i = k - S::SEQ_C; tiles = S::TC; rows = S::ROWS_C; off = S::PHASE_A_BYTES; }
        else if (k < S::SEQ_E) { i = k - S::SEQ_D; tiles = S::TD; rows = S::ROWS_D; off = S::PHASE_A_BYTES + S::PHASE_C_BYTES; }
        else if (k < S::SEQ_E + S::TE) {
            dwide = false;
            i = k - S::SEQ_E; tiles = S::TE; rows = S::ROWS_E; act = actF; lane_ok = laneF; rset = rF; off = S::PHASE_A_BYTES + S::PHASE_C_BYTES + S::PHASE_D_BYTES;
            if constexpr (S::E_REDEAL) {
                int row, slab;
                mega_e_tile<S>(w, i, row, slab);
                act = true; rset = 0; rows = S::TE;          // every wave has TE tiles; only the lanes past the last block column have none
                lane_ok = slab * 64 + lane < S::NBF;
            }
        }
        else real = false;                                   // padding slot of the layer sequence
        const bool head_slot = wrapped && k < S::HEAD;  // static
        if (!real && !head_slot) return;                     // static: this slot never loads
        const uint8_t *p = dummy;
        if (real) {
            bool ok;
            if (dwide) ok = !into_head && d_tile_valid(i, tiles, S::tiles_half(rows), rows);
            else ok = !into_head && act && lane_ok && rset * tiles + i < rows;
            const uint8_t *q = wstream + (size_t)layer * S::LAYER_BYTES + off + ((size_t)(b * S::NW + w) * tiles + i) * S::TILE;
            p = ok ? q : p;
        }
        if (head_slot) {
            const uint8_t *q = head_tile(k);
            p = (into_head && q) ? q : p;
        }
        load_tile<S>(t, p, lane);
    }

    // D-wide phases: the row (of the workgroup's `rows`) this lane works on in the wave's tile i, or -1 when it has none.  A
    // full-slab wave takes rows rD * stride + i, stride = the phase's tiles per wave; a half-slab wave takes the row pairs
    // rD * stride_half + i, its lower lanes the first row of a pair, its upper lanes the second.
    __device__ __forceinline__ int d_row(int i, int stride, int stride_half, int rows) const
    {
        if (!actD) return -1;
        if (!halfD) { const int r = rD * stride + i; return i < stride && r < rows ? r : -1; }
        const int r = 2 * (rD * stride_half + i) + (lane >> 5);
        return i < stride_half && r < rows ? r : -1;
    }
    __device__ __forceinline__ bool d_tile_valid(int i, int stride, int stride_half, int rows) const { return d_row(i, stride, stride_half, rows) >= 0; }

    // address of head tile k of this wave, or null when the wave/lane/row has none
    __device__ __forceinline__ const uint8_t *head_tile(int k) const
    {
        const int rows = (int)vocab_rows;
        const int j = d_row(k, cdiv(rows, S::WPF), S::HALFD ? cdiv(cdiv(rows, 2), S::WPH) : 0, rows);
        const bool ok = j >= 0 && (uint32_t)(b * rows + j) < vocab;
        return ok ? wstream + (size_t)layers * S::LAYER_BYTES + ((size_t)(b * S::NW + w) * S::HEAD + k) * S::TILE : nullptr;
    }

    // head phase: slot k of the head sequence (static k)
    __device__ __forceinline__ void fetch_head(MegaTile &t, int k) const
    {
        if (k >= S::HEAD) return;
        const uint8_t *q = head_tile(k);
        const uint8_t *p = q ? q : dummy;
        load_tile<S>(t, p, lane);
    }
};

// One GEMV phase of one wave: consumes NT queue slots starting at sequence index SEQ0, refills each consumed
// slot with the tile S::DEPTH further down the sequence, leaves per-row sums in red[row*NS + slab].
template <class S, int SEQ0, int NT, int NS>
__device__ __forceinline__ void gemv_phase(MegaTile (&q)[S::DEPTH], const MegaWave<S> &mw, uint32_t layer, const float (&xr)[32],
                                           float xsum, int slab, int rset, bool active, int rows, float *red)
{
    constexpr int NT4 = round_up(NT, 4);
    float p[4];
#pragma unroll
    for (int i = 0; i < NT4; i++) {
        if (i < NT) {
            const int slot = (SEQ0 + i) % S::DEPTH;
            const MegaTile t = q[slot];
            p[i & 3] = tile_dot<S>(t, xr, xsum);
            mw.fetch(q[slot], SEQ0 + i + S::DEPTH, layer);
        } else {
            p[i & 3] = 0.f;
        }
        if ((i & 3) == 3) {
            const float s = quad_partials_sum(p[0], p[1], p[2], p[3]);
            const int ii = (i - 3) + quad_partial_of_lane(mw.lane);
            const int row = rset * NT + ii;
            if (active && (mw.lane & 15) == 0 && row < rows && ii < NT) red[row * NS + slab] = s;
        }
    }
}

// A D-wide GEMV phase (input vector of D floats, ROWS rows per workgroup): waves on a full slab take one row per tile, waves
// on the half slab two (MegaShapeBase).  Leaves per-row sums in red[row * NSD + slab].
template <class S, int SEQ0, int ROWS>
__device__ __forceinline__ void gemv_phase_d(MegaTile (&q)[S::DEPTH], const MegaWave<S> &mw, uint32_t layer, const float (&xr)[32],
                                             float xsum, float *red)
{
    constexpr int NT = S::tiles_d(ROWS), TH = S::tiles_half(ROWS), NT4 = round_up(NT, 4), NS = S::NSD;
    float p[4];
#pragma unroll
    for (int i = 0; i < NT4; i++) {
        if (i < NT) {
            const int slot = (SEQ0 + i) % S::DEPTH;
            const MegaTile t = q[slot];
            p[i & 3] = tile_dot<S>(t, xr, xsum);
            mw.fetch(q[slot], SEQ0 + i + S::DEPTH, layer);
        } else {
            p[i & 3] = 0.f;
        }
        if ((i & 3) == 3) {
            // where the sums go is computed here, every time (shapes with a half slab: dozens of addresses kept from in front
            // of the layer loop would spill)
            const int ln = maybe_opaque<S::HALFD != 0>(mw.lane);
            if (S::HALFD && mw.halfD) {          // uniform over the wave
                float s01, s23;
                quad_partials_sum_halves(p[0], p[1], p[2], p[3], s01, s23);
                const int g = ln >> 4;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int ii = (i - 3) + 2 * h + (g >> 1), row = 2 * (mw.rD * TH + ii) + (g & 1);
                    if ((ln & 15) == 0 && ii < TH && row < ROWS) red[row * NS + mw.sD] = h ? s23 : s01;
                }
            } else {
                const float s = quad_partials_sum(p[0], p[1], p[2], p[3]);
                const int ii = (i - 3) + quad_partial_of_lane(ln);
                const int row = mw.rD * NT + ii;
                if (mw.actD && (ln & 15) == 0 && row < ROWS && ii < NT) red[row * NS + mw.sD] = s;
            }
        }
    }
}

template <int NS>
__device__ __forceinline__ float red_row(const float *red, int row)
{
    float t = 0.f;
#pragma unroll
    for (int s = 0; s < NS; s++) t += red[row * NS + s];
    return t;
}

// LDS of the kernel.
template <class S>
struct MegaLds {
    static constexpr int XS = S::F > S::D ? S::F : S::D;
    static constexpr int RED_ROWS = S::ROWS_D > S::MAX_VOCAB_ROWS ? S::ROWS_D : S::MAX_VOCAB_ROWS;
    static constexpr int RED_COLS = S::NSF > S::NSD ? S::NSF : S::NSD;
    float xs[XS];                    // the phase's input vector (during attention: exp(score) of the chunk)
    float red[RED_ROWS * RED_COLS];  // per-row partial sums, one column per slab
    float xown[S::ROWS_C];           // this workgroup's rows of the residual stream
    float scratch[2 * S::NW];        // two halves: the waves' sums of x, then of x^2 (later: best logit and its index)
    float attn_red[S::NW * (S::R + 1)];
    float qkv[3 * S::R];             // query of the workgroup's head, K and V row of the newest position
    float same_xcd;                  // non-zero: the 32 workgroups this one shares heads with all run on its XCD
};

// Brings the N-float vector at `src` (being produced by other workgroups) into LDS.  With NORM the vector is to be
// normalised (normalize.comp:34-64: x * w * rsqrt(mean((x - mean)^2)), no epsilon): LDS gets x * w, and the scale
// rsqrt(variance), the same for every element, is returned for the caller to apply to its row sums.  The waves so
// start on their tiles one barrier after the vector has arrived instead of three; the variance is taken as
// mean(x^2) - mean(x)^2 from one pass over the registers.  The norm weights are requested before the wait, not after.
template <int N, int NW, bool NORM, int SLEEP = 0, bool OPAQUE = false>
__device__ __forceinline__ float acquire_vector(float *xs, const float *src, const float *w, float *scratch, uint32_t *status, uint32_t spin_limit)
{
    constexpr int T = NW * 64, PER = cdiv(N, T);
    const int tx = maybe_opaque<OPAQUE>((int)threadIdx.x);
    float v[PER];
    bool want[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) want[j] = tx + j * T < N;
    float wn[NORM ? PER : 1];
    if constexpr (NORM) {
#pragma unroll
        for (int j = 0; j < PER; j++) wn[j] = want[j] ? w[tx + j * T] : 0.f;
    }
    poll_values<PER, SLEEP>(v, src + tx, T, want, status, spin_limit);
    float inv = 1.f;
    if constexpr (NORM) {
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            const float x = want[j] ? v[j] : 0.f;
            s1 += x;
            s2 = fmaf(x, x, s2);
            if (want[j]) xs[xs_index(tx + j * T)] = x * wn[j];
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        if ((tx & 63) == 0) { scratch[tx >> 6] = s1; scratch[NW + (tx >> 6)] = s2; }
        lds_barrier();
        float t1 = 0.f, t2 = 0.f;
#pragma unroll
        for (int i = 0; i < NW; i++) { t1 += scratch[i]; t2 += scratch[NW + i]; }
        const float mean = t1 / (float)N;
        inv = rsqrtf(t2 / (float)N - mean * mean);
    } else {
#pragma unroll
        for (int j = 0; j < PER; j++)
            if (want[j]) xs[xs_index(tx + j * T)] = v[j];
        lds_barrier();
    }
    return inv;
}

// The same for a long vector without normalisation (the down projection's input): 16 bytes a thread and load, a quarter of
// the load instructions per poll (a buffer load with sc1 = device scope; past the end of the vector it returns zeros).
typedef uint32_t mega_u4v __attribute__((ext_vector_type(4)));
template <int N, int NW, int SLEEP>
__device__ __forceinline__ void acquire_vector_wide(float *xs, const float *src, uint32_t *status, uint32_t spin_limit)
{
    constexpr int T = NW * 64, PER = cdiv(N, 4 * T);
    static_assert(N % 4 == 0, "whole 16-byte groups");
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(src), 0, N * 4, 0x00020000);
    mega_u4v v[PER];
    uint32_t spins = 0;
    bool pending;
    if constexpr (SLEEP > 0) __builtin_amdgcn_s_sleep(SLEEP);
    do {
        pending = false;
        asm volatile("" ::: "memory");      // every turn issues the loads again
#pragma unroll
        for (int j = 0; j < PER; j++) {
            v[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, 16 * ((int)threadIdx.x + j * T), 0, 16 /* sc1 */);
            pending |= (v[j].x == kNotReady) | (v[j].y == kNotReady) | (v[j].z == kNotReady) | (v[j].w == kNotReady);
        }
    } while (pending && ++spins < spin_limit);
    if (pending) *status = 1u;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int idx = 4 * ((int)threadIdx.x + j * T);
        if (idx < N) *reinterpret_cast<mega_u4v *>(xs + xs_index(idx)) = v[j];
    }
    lds_barrier();
}

// Phase E, where every working wave owns one column slab (S::NRF == 1): a wave fetches the 2048 floats of its own slab and
// nothing else, 16 bytes a lane and load, at device scope; it starts on its tiles when the producers of that slab have
// stored, without a workgroup barrier, and the workgroup no longer moves the whole F-float vector with every thread.
// The slab passes through the wave's own part of LDS to reach the block-per-lane order of load_slab.
template <class S, int SLEEP>
__device__ __forceinline__ void acquire_own_slab(float (&xr)[32], float &xsum, float *xs, const float *src, int slab, int lane, bool active,
                                                 bool lane_has, uint32_t *status, uint32_t spin_limit)
{
    static_assert(S::NRF == 1 && S::F % 4 == 0, "one wave per slab");
    if (active) {
        // loads past the end of the vector return zero (the last slab is not full)
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(src), 0, S::F * 4, 0x00020000);
        const int base = slab * 2048;
        mega_u4v v[8];
        uint32_t spins = 0;
        bool pending;
        if constexpr (SLEEP > 0) __builtin_amdgcn_s_sleep(SLEEP);
        do {
            pending = false;
            asm volatile("" ::: "memory");      // every turn issues the loads again
#pragma unroll
            for (int j = 0; j < 8; j++) {
                v[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (base + (j * 64 + lane) * 4) * 4, 0, 16 /* sc1: device scope */);
                pending |= (v[j].x == kNotReady) | (v[j].y == kNotReady) | (v[j].z == kNotReady) | (v[j].w == kNotReady);
            }
        } while (pending && ++spins < spin_limit);
        if (pending) *status = 1u;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int idx = base + (j * 64 + lane) * 4;
            if (idx < S::F) *reinterpret_cast<mega_u4v *>(xs + xs_index(idx)) = v[j];
        }
    }
    load_slab(xr, xsum, xs, slab * 64 + lane, active && lane_has);
}

template <class S>
__global__ __launch_bounds__(S::NW * 64, 1) void mega_decode_kernel(MegaArgs a)
{
    constexpr int D = S::D, F = S::F, R = S::R, NW = S::NW, T = NW * 64;
    __shared__ __attribute__((aligned(16))) MegaLds<S> l;
    float *xs = l.xs, *red = l.red, *xown = l.xown, *scratch = l.scratch;
    MegaWave<S> mw;
    mw.init(a);
    const int b = mw.b, w = mw.w, lane = mw.lane;
    const int st = threadIdx.x;
    uint32_t *status = a.status;
    const uint32_t spin_limit = a.spin_limit;
    const MegaPlace<S> place(b);
    // Every workgroup says which XCD it runs on; before its first hand-over inside a head a workgroup reads what the 32
    // workgroups it shares heads with have said (below, layer 0) and takes the path through the XCD's L2 only if all of
    // them are where it is.  All 32 read the same words, so they decide alike.
    uint32_t my_xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(my_xcc));
    my_xcc &= 0xfu;
    float *const xcc_table = a.xchg + (size_t)a.layers * S::XCHG_LAYER + S::OFF_XCC;
    if (threadIdx.x == 0) st_dev(xcc_table + b, __uint_as_float(my_xcc));
    bool xcd_local = false;

    // ---- start the weight stream ------------------------------------------------------------------------------
    MegaTile q[S::DEPTH];
#pragma unroll
    for (int k = 0; k < S::DEPTH; k++) mw.fetch(q[k], k, 0);

    // ---- re-arm the other buffer set for the next token ---------------------------------------------------------
    {
        const size_t n4 = ((size_t)a.layers * S::XCHG_LAYER + S::XCHG_TAIL) / 4, m4 = (size_t)a.layers * S::LOCAL_LAYER / 4;
        uint4 *dst = reinterpret_cast<uint4 *>(a.xchg_rearm), *dl = reinterpret_cast<uint4 *>(a.xl_rearm);
        for (size_t i = (size_t)b * T + threadIdx.x; i < n4; i += (size_t)kMegaWGs * T)
            dst[i] = make_uint4(kNotReady, kNotReady, kNotReady, kNotReady);
        for (size_t i = (size_t)b * T + threadIdx.x; i < m4; i += (size_t)kMegaWGs * T)
            dl[i] = make_uint4(kNotReady, kNotReady, kNotReady, kNotReady);
    }

    const uint32_t pos = a.pos;
    const float *x_src = a.tok_f32 + (size_t)a.token * D;  // layer 0 reads the embedding row directly (constant data)
    if (threadIdx.x < S::ROWS_C) xown[threadIdx.x] = x_src[b * S::ROWS_C + threadIdx.x];

    float xr[32];
    float xsum;

    for (uint32_t layer = 0; layer < a.layers; layer++) {
        float *xc = a.xchg + (size_t)layer * S::XCHG_LAYER, *xlc = a.xl + (size_t)layer * S::LOCAL_LAYER;
        const float *norm_w = a.norms + (size_t)layer * 2 * D;
        uint16_t *kc = a.kv + (size_t)layer * 2 * a.backlog * D, *vc = kc + (size_t)a.backlog * D;

        // ================= A: norm + QKV ====================================================================
        const float inv_a = acquire_vector<D, NW, true, kPollDelay, S::HALFD != 0>(xs, x_src, norm_w, scratch, status, spin_limit);
        load_slab<S::HALFD != 0>(xr, xsum, xs, mw.blockD, mw.actD);
        gemv_phase_d<S, S::SEQ_A, S::ROWS_A>(q, mw, layer, xr, xsum, red);
        if (layer == 0 && a.xcd_local && w == 0) {
            // lane j asks for workgroup (b % 8) + 8 j; the words were stored when the kernel started
            float got[1];
            const bool want1[1] = {lane < kMegaWGs / 8};
            poll_values<1, 0>(got, xcc_table + (b & 7) + 8 * (lane & 31), 1, want1, status, spin_limit);
            const bool same = !want1[0] || __float_as_uint(got[0]) == my_xcc;
            if (lane == 0) l.same_xcd = __builtin_amdgcn_ballot_w64(!same) == 0 ? 1.f : 0.f;
        }
        lds_barrier();
        if (layer == 0) {
            xcd_local = a.xcd_local && l.same_xcd != 0.f;
            if (b == 0 && threadIdx.x == 0) status[kStatusXcd] = xcd_local ? 1u : 0u;      // what workgroup 0's 32 decided
        }
        if (threadIdx.x < S::ROWS_A) {
            const float v = red_row<S::NSD>(red, threadIdx.x) * inv_a;
            int which, col;
            mega_qkv_row<S>(b, threadIdx.x, which, col);
            float out = v;
            if (which != 0) {
                // copy_to_cache.comp:35: the cache keeps fp16; attention of this very step reads the rounded value too
                const uint16_t hbits = float_to_half_bits(v);
                (which == 1 ? kc : vc)[(size_t)pos * D + col] = hbits;
                out = half_bits_to_float(hbits);
            }
            // read by the chunk workgroups of the row's head, which run on this XCD
            if (xcd_local) xlc[S::OFF_QKV + which * D + col] = out;
            else st_dev(xlc + S::OFF_QKV + which * D + col, out);
        }

        // ================= B: attention chunk (head h, chunk c) ================================================
        {
            const int h = place.h, c = place.c;
            if (place.attends) {
                const uint32_t n_valid = pos + 1;
                uint32_t chunk = (n_valid + S::CPH - 1) / S::CPH;
                chunk = (chunk + 3) & ~3u;
                const uint32_t p_begin = min((uint32_t)c * chunk, n_valid), p_end = min(p_begin + chunk, n_valid);
                const int sub = lane & 15, rsel = w * 4 + (lane >> 4);
                constexpr int RPR = NW * 4;   // cache rows per round of the workgroup
                constexpr int PRE = 2;        // rounds of K, V and rotation rows in flight (3 and 4 measured: no faster)
                const size_t row_off = (size_t)h * R + sub * 8;
                auto unpack8 = [](float (&f)[8], const uint4 &raw) {
                    const uint32_t wv[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        f[2 * i] = half_bits_to_float((uint16_t)(wv[i] & 0xffffu));
                        f[2 * i + 1] = half_bits_to_float((uint16_t)(wv[i] >> 16));
                    }
                };
                // Rows older than this token do not depend on it: ask for the first rounds, then wait for q.  The
                // rounds form a queue PRE deep: a slot is refilled with the round PRE further on as soon as it is
                // used (rounds past the end of the chunk read row 0 and are masked).
                uint4 kpre[PRE], vpre[PRE];
                float4 tpre[PRE][2];
                auto request_round = [&](int slot, uint32_t p0) {
                    const uint32_t p = p0 + rsel;
                    const uint32_t pc = (p < p_end && p != pos) ? p : 0;  // any valid row; unused when masked
                    kpre[slot] = *reinterpret_cast<const uint4 *>(kc + (size_t)pc * D + row_off);
                    vpre[slot] = *reinterpret_cast<const uint4 *>(vc + (size_t)pc * D + row_off);
                    const float4 *tp = reinterpret_cast<const float4 *>(a.trig + (size_t)(p < p_end ? pos - p : 0) * (R / 2) + sub * 4);
                    tpre[slot][0] = tp[0];
                    tpre[slot][1] = tp[1];
                };
#pragma unroll
                for (int r = 0; r < PRE; r++) request_round(r, p_begin + r * RPR);
                // The query of this head and, where the chunk holds the newest position, that position's K and V row (all
                // three still on their way from phase A): waves 0, 1 and 2 fetch one of them each, two floats a lane, and
                // pass them on through LDS (every 16-lane group polling the same 512 bytes for itself cost 32 times the
                // requests).  The polls travel behind the cache rows requested above: that is the time the producers'
                // stores need to become visible, so no sleep in front of them.
                const bool holds_new = pos >= p_begin && pos < p_end;          // uniform over the workgroup
                if (w < 3 && (w == 0 || holds_new)) {
                    float pv[2];
                    const bool want2[2] = {true, true};
                    if (xcd_local) poll_values<2, 0, true>(pv, xlc + S::OFF_QKV + w * D + h * R + lane * 2, 1, want2, status, spin_limit);
                    else poll_values<2, 0>(pv, xlc + S::OFF_QKV + w * D + h * R + lane * 2, 1, want2, status, spin_limit);
                    l.qkv[w * R + lane * 2] = pv[0];
                    l.qkv[w * R + lane * 2 + 1] = pv[1];
                }
                lds_barrier();
                const bool newest = holds_new && ((pos - p_begin) % RPR) == (uint32_t)rsel;
                float qkv[24];
                {
                    const float4 *qs = reinterpret_cast<const float4 *>(l.qkv + sub * 8);
                    const float4 q0 = qs[0], q1 = qs[1];
                    qkv[0] = q0.x; qkv[1] = q0.y; qkv[2] = q0.z; qkv[3] = q0.w; qkv[4] = q1.x; qkv[5] = q1.y; qkv[6] = q1.z; qkv[7] = q1.w;
#pragma unroll
                    for (int i = 8; i < 24; i++) qkv[i] = 0.f;
                    if (newest) {
#pragma unroll
                        for (int i = 0; i < 8; i++) { qkv[8 + i] = l.qkv[R + sub * 8 + i]; qkv[16 + i] = l.qkv[2 * R + sub * 8 + i]; }
                    }
                }
                const float scale = rsqrtf((float)R);
                float den = 0.f;
                // exp(score / sqrt(R)) of cache row p for this 16-lane group's query head; every lane of the group gets it
                auto weight_of = [&](uint32_t p, const uint4 &kraw, const float4 &t0, const float4 &t1) -> float {
                    float s = 0.f;
                    if (p < p_end) {
                        float kf[8];
                        unpack8(kf, kraw);
                        if (p == pos) {
#pragma unroll
                            for (int i = 0; i < 8; i++) kf[i] = qkv[8 + i];
                        }
                        const float ct[4] = {t0.x, t0.z, t1.x, t1.z}, stn[4] = {t0.y, t0.w, t1.y, t1.w};
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float kx = kf[2 * i], ky = kf[2 * i + 1], qx = qkv[2 * i], qy = qkv[2 * i + 1];
                            const float dotp = fmaf(qy, ky, qx * kx);
                            const float crs = fmaf(qx, ky, -(qy * kx));
                            s = fmaf(ct[i], dotp, s);
                            s = fmaf(stn[i], crs, s);
                        }
                    }
                    s = group16_sum(s);   // the same bits in all 16 lanes
                    const float e = p < p_end ? __expf(s * scale) : 0.f;
                    den += (sub == 0) ? e : 0.f;
                    return e;
                };
                float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                auto add_row = [&](uint32_t p, float e, const uint4 &vraw) {
                    if (p < p_end) {
                        float vf[8];
                        unpack8(vf, vraw);
                        if (p == pos) {
#pragma unroll
                            for (int i = 0; i < 8; i++) vf[i] = qkv[16 + i];
                        }
#pragma unroll
                        for (int i = 0; i < 8; i++) acc[i] = fmaf(e, vf[i], acc[i]);
                    }
                };
                // a row's weight is computed and used by the same 16 lanes: no exchange through LDS, no barrier
                for (uint32_t p0 = p_begin; p0 < p_end; p0 += PRE * RPR) {
#pragma unroll
                    for (int r = 0; r < PRE; r++) {
                        const uint32_t p = p0 + r * RPR + rsel;
                        add_row(p, weight_of(p, kpre[r], tpre[r][0], tpre[r][1]), vpre[r]);
                        if (p0 + (r + PRE) * RPR < p_end) request_round(r, p0 + (r + PRE) * RPR);   // uniform condition
                    }
                }
#pragma unroll
                for (int off = 16; off < 64; off <<= 1) {
#pragma unroll
                    for (int i = 0; i < 8; i++) acc[i] += __shfl_xor(acc[i], off, kWave);
                    den += __shfl_xor(den, off, kWave);
                }
                if (lane < 16) {
#pragma unroll
                    for (int i = 0; i < 8; i++) l.attn_red[w * (R + 1) + lane * 8 + i] = acc[i];
                    if (lane == 0) l.attn_red[w * (R + 1) + R] = den;
                }
                lds_barrier();
                if (st <= R) {
                    float t = 0.f;
#pragma unroll
                    for (int i = 0; i < NW; i++) t += l.attn_red[i * (R + 1) + st];
                    // read by chunk 0 of this head, on this XCD
                    if (xcd_local) xlc[S::OFF_PART + (h * S::CPH + c) * S::PART + st] = t;
                    else st_dev(xlc + S::OFF_PART + (h * S::CPH + c) * S::PART + st, t);
                }
            }
        }

        // ================= B': combine the chunks of head b (one wait for numerators and denominators) ==========
        if (place.attends && place.c == 0 && st < R) {
            float nd[2 * S::CPH];
            const uint32_t *hp = reinterpret_cast<const uint32_t *>(xlc + S::OFF_PART + (size_t)place.h * S::CPH * S::PART);
            uint32_t spins = 0;
            bool pending;
            do {
                pending = false;
                if (xcd_local) asm volatile("" ::: "memory");      // ordinary loads: every turn has to issue them again
#pragma unroll
                for (int c = 0; c < S::CPH; c++) {
                    const uint32_t un = xcd_local ? ld_xcd(hp + c * S::PART + st) : ld_dev(hp + c * S::PART + st);
                    const uint32_t ud = xcd_local ? ld_xcd(hp + c * S::PART + R) : ld_dev(hp + c * S::PART + R);
                    nd[c] = __uint_as_float(un);
                    nd[S::CPH + c] = __uint_as_float(ud);
                    pending |= (un == kNotReady) | (ud == kNotReady);
                }
            } while (pending && ++spins < spin_limit);
            if (pending) *status = 1u;
            float n = 0.f, d = 0.f;
#pragma unroll
            for (int c = 0; c < S::CPH; c++) { n += nd[c]; d += nd[S::CPH + c]; }
            st_dev(xc + S::OFF_O + place.h * R + st, n / d);       // every workgroup of the device reads this one
        }

        // ================= C: x += Wo o ============================================================================
        acquire_vector<D, NW, false, kPollDelay, S::HALFD != 0>(xs, xc + S::OFF_O, nullptr, scratch, status, spin_limit);
        load_slab<S::HALFD != 0>(xr, xsum, xs, mw.blockD, mw.actD);
        gemv_phase_d<S, S::SEQ_C, S::ROWS_C>(q, mw, layer, xr, xsum, red);
        lds_barrier();
        if (st < S::ROWS_C) {
            const float v = xown[st] + red_row<S::NSD>(red, st);
            xown[st] = v;
            st_dev(xc + S::OFF_X1 + b * S::ROWS_C + st, v);
        }

        // ================= D: norm + SwiGLU ========================================================================
        const float inv_d = acquire_vector<D, NW, true, kPollDelay, S::HALFD != 0>(xs, xc + S::OFF_X1, norm_w + D, scratch, status, spin_limit);
        load_slab<S::HALFD != 0>(xr, xsum, xs, mw.blockD, mw.actD);
        gemv_phase_d<S, S::SEQ_D, S::ROWS_D>(q, mw, layer, xr, xsum, red);
        lds_barrier();
        if (st < S::ROWS_D / 2) {
            // rows alternate W3 row k, W1 row k (matmul_silu_ff.comp:96: result1 * result2 / (exp(-result2) + 1))
            const float r1 = red_row<S::NSD>(red, 2 * st) * inv_d, r2 = red_row<S::NSD>(red, 2 * st + 1) * inv_d;
            st_dev(xc + S::OFF_FF + b * (S::ROWS_D / 2) + st, r1 * r2 / (__expf(-r2) + 1.f));
        }

        // ================= E: x += W2 ff ===========================================================================
        if constexpr (S::OWN_SLAB_E) {
            acquire_own_slab<S, kPollDelay>(xr, xsum, xs, xc + S::OFF_FF, mw.sF, lane, mw.actF, mw.laneF, status, spin_limit);
        } else {
            acquire_vector_wide<F, NW, kPollDelay>(xs, xc + S::OFF_FF, status, spin_limit);
            if constexpr (S::E_REDEAL) {
                int row0, slab0;
                mega_e_tile<S>(w, 0, row0, slab0);
                load_slab(xr, xsum, xs, slab0 * 64 + lane, slab0 * 64 + lane < S::NBF);
            } else {
                load_slab(xr, xsum, xs, mw.sF * 64 + lane, mw.laneF);
            }
        }
        if constexpr (S::E_REDEAL) {
            // every wave TE tiles; the spare waves change their column slab every E_SPARE_ROWS tiles and fetch its activations anew
            float p[4];
#pragma unroll
            for (int i = 0; i < S::TE; i++) {
                int row, slab;
                mega_e_tile<S>(w, i, row, slab);
                if (i > 0 && i % S::E_SPARE_ROWS == 0 && w >= S::NSF) load_slab(xr, xsum, xs, slab * 64 + lane, slab * 64 + lane < S::NBF);
                const int slot = (S::SEQ_E + i) % S::DEPTH;
                const MegaTile t = q[slot];
                p[i & 3] = tile_dot<S>(t, xr, xsum);
                mw.fetch(q[slot], S::SEQ_E + i + S::DEPTH, layer);
                if ((i & 3) == 3) {
                    const float sum4 = quad_partials_sum(p[0], p[1], p[2], p[3]);
                    int r0, sl;
                    mega_e_tile<S>(w, i - 3, r0, sl);       // the four tiles are four consecutive rows of one slab
                    if ((lane & 15) == 0) red[(r0 + quad_partial_of_lane(lane)) * S::NSF + sl] = sum4;
                }
            }
        } else {
            gemv_phase<S, S::SEQ_E, S::TE, S::NSF>(q, mw, layer, xr, xsum, mw.sF, mw.rF, mw.actF, S::ROWS_E, red);
        }
        // padding slots of the layer's sequence carry no tile, but the slot S::DEPTH ahead of them does
#pragma unroll
        for (int k = S::SEQ_E + S::TE; k < S::PER_LAYER; k++) mw.fetch(q[k % S::DEPTH], k + S::DEPTH, layer);
        lds_barrier();
        if (st < S::ROWS_E) {
            const float v = xown[st] + red_row<S::NSF>(red, st);
            xown[st] = v;
            st_dev(xc + S::OFF_X2 + b * S::ROWS_E + st, v);
        }
        x_src = xc + S::OFF_X2;
    }

    // ================= head: norm + output matrix ====================================================================
    {
        const float inv_h = acquire_vector<D, NW, true, kPollDelay, S::HALFD != 0>(xs, x_src, a.norms + (size_t)a.layers * 2 * D, scratch, status, spin_limit);
        load_slab<S::HALFD != 0>(xr, xsum, xs, mw.blockD, mw.actD);
        const int rows = (int)mw.vocab_rows, per_set = cdiv(rows, S::WPF), per_half = S::HALFD ? cdiv(cdiv(rows, 2), S::WPH) : 0;
        // the head's slots are numbered from 0; tiles beyond per_set read the dummy tile
        float p[4];
#pragma unroll
        for (int i = 0; i < S::HEAD; i++) {
            const int slot = i % S::DEPTH;
            const MegaTile t = q[slot];
            p[i & 3] = tile_dot<S>(t, xr, xsum);
            mw.fetch_head(q[slot], i + S::DEPTH);
            if ((i & 3) == 3) {
                if (S::HALFD && mw.halfD) {      // uniform over the wave: two rows per tile
                    float s01, s23;
                    quad_partials_sum_halves(p[0], p[1], p[2], p[3], s01, s23);
                    const int g = lane >> 4;
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const int ii = (i - 3) + 2 * h + (g >> 1), row = 2 * (mw.rD * per_half + ii) + (g & 1);
                        if ((lane & 15) == 0 && ii < per_half && row < rows) red[row * S::NSD + mw.sD] = h ? s23 : s01;
                    }
                } else {
                    const float s = quad_partials_sum(p[0], p[1], p[2], p[3]);
                    const int ii = (i - 3) + quad_partial_of_lane(lane);
                    const int row = mw.rD * per_set + ii;
                    if (mw.actD && (lane & 15) == 0 && ii < per_set && row < rows) red[row * S::NSD + mw.sD] = s;
                }
            }
        }
        lds_barrier();
        // logits out; on the way the greedy pick (llava_session.cpp:144-152: index of the first strict maximum):
        // every workgroup hands its best (value, index) to workgroup 0 like any other hand-over
        float bv = -INFINITY;
        uint32_t bi = kNotReady;
        auto better = [](float ov, uint32_t oi, float mv, uint32_t mi) {
            return oi != kNotReady && (mi == kNotReady || ov > mv || (ov == mv && oi < mi));
        };
        for (int j = st; j < rows; j += T) {
            const uint32_t n = (uint32_t)b * rows + j;
            if (n < a.vocab) {
                const float v = red_row<S::NSD>(red, j) * inv_h;
                a.logits[n] = v;
                if (better(v, n, bv, bi)) { bv = v; bi = n; }
            }
        }
        auto block_best = [&]() {          // result in thread 0
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ov = __shfl_xor(bv, off, kWave);
                const uint32_t oi = __shfl_xor(bi, off, kWave);
                if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
            }
            if (lane == 0) { scratch[w] = bv; scratch[NW + w] = __uint_as_float(bi); }
            lds_barrier();
            if (st == 0) {
#pragma unroll
                for (int i = 1; i < NW; i++) {
                    const float ov = scratch[i];
                    const uint32_t oi = __float_as_uint(scratch[NW + i]);
                    if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
                }
            }
        };
        block_best();
        float *cand = a.xchg + (size_t)a.layers * S::XCHG_LAYER;
        if (st == 0) {
            // neither word may look like "not written yet": an all-ones NaN becomes the default NaN, a workgroup
            // without rows reports index 0xFFFFFFFE
            st_dev(cand + 2 * b, __float_as_uint(bv) == kNotReady ? __uint_as_float(0x7fc00000u) : bv);
            st_dev(cand + 2 * b + 1, __uint_as_float(bi == kNotReady ? kNotReady - 1 : bi));
        }
        if (b == 0) {
            lds_barrier();                 // thread 0 has read the scratch words of the first reduction
            bv = -INFINITY;
            bi = kNotReady;
            if (st < kMegaWGs) {
                float pair[2];
                const bool want2[2] = {true, true};
                poll_values<2, kPollDelay>(pair, cand + 2 * st, 1, want2, status, spin_limit);
                const uint32_t oi = __float_as_uint(pair[1]);
                if (oi < kNotReady - 1) { bv = pair[0]; bi = oi; }
            }
            block_best();
            if (st == 0) status[kStatusToken] = bi == kNotReady ? 0u : bi;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// Builds the weight stream from the row-major split layout (runs once at upload).
// One thread per (tile, lane).  phase: 0 A, 1 C, 2 D, 3 E, 4 head.
// ---------------------------------------------------------------------------------------------------------
struct MegaPackSrc {
    MatView m[3];  // A: wq, wk, wv;  C: wo;  D: w3, w1;  E: w2;  head: output
};

template <class S>
__global__ void mega_pack_kernel(uint8_t *dst /* start of the phase region */, MegaPackSrc src, int phase, uint32_t vocab)
{
    const int tiles = phase == 0 ? S::TA : phase == 1 ? S::TC : phase == 2 ? S::TD : phase == 3 ? S::TE : S::HEAD;
    const bool dwide = phase != 3;
    const int nb = dwide ? S::NBD : S::NBF;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)kMegaWGs * S::NW * tiles * 64;
    if (idx >= total) return;
    const int lane = idx % 64;
    const size_t tile = idx / 64;
    const int i = tile % tiles;
    const int w = (tile / tiles) % S::NW;
    const int b = tile / tiles / S::NW;
    uint8_t *out = dst + tile * S::TILE;
    uint4 codes = make_uint4(0, 0, 0, 0), codes2 = codes;
    uint16_t scale = 0;
    float scale32 = 0.f;
    // which row of the workgroup's rows and which block column this lane of this tile holds (-1: none) -- the same rules as
    // MegaWave::init / d_row for the D-wide phases, as MegaWave::fetch for phase E
    int j = -1, blk = 0;
    const int rows = phase == 0 ? S::ROWS_A : phase == 1 ? S::ROWS_C : phase == 2 ? S::ROWS_D : phase == 3 ? S::ROWS_E : (int)((vocab + kMegaWGs - 1) / kMegaWGs);
    if (dwide) {
        const bool half = S::HALFD && w >= S::FULLD * S::WPF && w < S::FULLD * S::WPF + S::WPH;
        const bool act = w < S::FULLD * S::WPF + S::WPH;
        const int stride = phase == 4 ? cdiv(rows, S::WPF) : tiles;
        const int stride_half = S::HALFD ? cdiv(cdiv(rows, 2), S::WPH) : 0;
        if (act && !half) {
            const int rset = w / S::FULLD, r = rset * stride + i;
            blk = (w % S::FULLD) * 64 + lane;
            if (i < stride && r < rows) j = r;
        } else if (act) {
            const int rset = w - S::FULLD * S::WPF, r = 2 * (rset * stride_half + i) + (lane >> 5);
            blk = S::FULLD * 64 + (lane & 31);
            if (i < stride_half && r < rows) j = r;
        }
    } else {
        int slab = w % S::NSF, rset = w / S::NSF, r = rset * tiles + i;
        if (S::E_REDEAL) { mega_e_tile<S>(w, i, r, slab); rset = 0; }
        blk = slab * 64 + lane;
        if (rset < S::NRF && blk < nb && r < rows) j = r;
    }
    bool ok = j >= 0;
    const MatView *mv = nullptr;
    uint32_t row = 0;
    if (ok) {
        const int g = b * rows + j;
        if (phase == 4) {
            ok = (uint32_t)g < vocab;
            row = g;
            mv = &src.m[0];
        } else if (phase == 0) {
            int which = 0, r = 0;
            mega_qkv_row<S>(b, j, which, r);
            mv = &src.m[which];
            row = r;
        }
        else if (phase == 2) { mv = &src.m[g & 1]; row = g >> 1; }
        else { mv = &src.m[0]; row = g; }
    }
    if (ok) {
        const size_t sb = (size_t)row * nb + blk;
        if constexpr (S::QT == 4) {
            codes = mv->codes[sb];
        } else {
            codes = mv->codes[2 * sb];
            codes2 = mv->codes[2 * sb + 1];
        }
        if constexpr (S::SF32) scale32 = mv->scales_f32[sb];
        else scale = mv->scales[sb];
    }
    if constexpr (S::QT == 8) {
        *reinterpret_cast<uint4 *>(out + lane * 16) = codes;
        *reinterpret_cast<uint4 *>(out + 1024 + lane * 16) = codes2;
    } else {
        *reinterpret_cast<uint4 *>(out + lane * S::CODE) = codes;
    }
    if constexpr (S::SF32) *reinterpret_cast<float *>(out + 64 * S::CODE + lane * 4) = scale32;
    else *reinterpret_cast<uint16_t *>(out + 64 * S::CODE + lane * 2) = scale;
}

}  // namespace lv
