// Device-side building blocks shared by the forward kernels (gfx950 / CDNA4 only).
//
// Tile geometry used throughout:
//   * a workgroup is 4 wavefronts (256 threads) and owns BLOCK_M = 128 query rows, 32 per wavefront;
//   * keys are consumed in blocks of 128 or 64 (per kernel and head_dim), each handled as sub-tiles of 32 keys;
//   * the score tile is computed TRANSPOSED, S^T = K Q^T, with v_mfma_i32_32x32x32_i8: a lane then holds one
//     query column (lane % 32) and 16 keys, so row max / row sum are in-lane reductions plus one exchange
//     between lane l and lane l^32, and the accumulator registers run along the key axis - the contraction
//     axis of P V - which lets P be packed to int8 in-lane and fed straight back as an MFMA B operand.
//
// MFMA register layouts relied on (verified on hardware against a CPU matmul):
//   v_mfma_i32_32x32x32_i8   A: lane (m = l%32, h = l/32) holds bytes k = 16h .. 16h+15 of row m
//                            B: lane (n = l%32, h)        holds bytes k = 16h .. 16h+15 of column n
//                            D: lane (n = l%32, h) register r holds row m = 8*(r/4) + 4*h + r%4
//   v_mfma_f32_32x32x16_f16  same with 8 halves per lane, k = 8h .. 8h+7
//   ds_read_b64_tr_b8        inside each group of 16 lanes, result lane i byte j = byte (i%8) of the 8 bytes
//                            addressed by lane (2j + i/8) of the group
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace intfa {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));

#define INTFA_LDS(p) ((__attribute__((address_space(3))) void*)(p))
// compile-time switch passed as a lambda argument (selects the LDS buffer or the masked code instance of a pipeline step)
template <bool V> struct BoolTag { static constexpr bool value = V; };
#define INTFA_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

constexpr int kBlockM = 128;
constexpr int kThreads = 256;
constexpr float kLog2_127 = 6.98868468677f;   // log2(127)
// floor(n / d) for 0 <= n < 2^31 and a divisor d fixed per launch: (n * m) >> s with s = 31 + ceil(log2 d) and
// m = ceil(2^s / d) < 2^32 computed on the host (Granlund & Montgomery, "Division by invariant integers using
// multiplication").  For a wave-uniform n that is three scalar instructions; a run-time integer division expands to some
// forty dependent vector instructions, and the mapping of a workgroup to its work needs a dozen of them.
struct FastDiv { uint32_t m, s; };
__host__ __device__ __forceinline__ int fast_div(int n, FastDiv d) { return (int)(((uint64_t)(uint32_t)n * d.m) >> d.s); }

// Kernel-side parameter block (byte strides, resolved pointers).
struct KParams {
    const char* q; const char* k; const char* v; char* out;
    const char* q_scale; const char* k_scale; const char* v_scale;
    float* lse;
    const int32_t* seqlens_k;              // optional [batch]: number of keys per batch entry (<= seqlen_k)
    int32_t* s_dump;                       // debug: int32 S [B,H,N,N]
    float* o_part; float* lse_part;        // split-KV partials [S,B,H,N,D] fp32 / [S,B,H,N]
    int64_t q_sb, q_sh, q_sn;              // bytes
    int64_t k_sb, k_sh, k_sn;
    int64_t v_sb, v_sh, v_sn;
    int64_t o_sb, o_sh, o_sn;
    int64_t qs_sb, qs_sh, qs_sn;           // elements
    int64_t ks_sb, ks_sh, ks_sn;
    int64_t vs_sb, vs_sh;
    int64_t vs_sblk;                       // blocked V scales: elements between the scale rows of consecutive key ranges
    int32_t batch, heads, seqlen, head_dim;  // seqlen = number of query rows
    int32_t seqlen_k;                      // number of keys (= seqlen unless the caller passes separate lengths)
    int32_t scale_dtype, causal, num_splits, blocks_per_split;
    int32_t kv_group;                      // query heads per K/V head (1 = every query head has its own K/V)
    int32_t pair_mblocks;                  // causal single-pass launches: one workgroup takes query blocks i and n-1-i
    int32_t vs_g;                          // blocked V scales: key blocks of the kernel per scale row (0 = scalar V scale)
    int32_t vs_sub;                        // blocked V scales: 2 when a scale row covers 64 keys, half of the 128-key block
    int32_t causal_rows;                   // decode kernel: query positions per folded query head (0 = the row is the position)
    float qk_scale_log2;                   // sm_scale * log2(e)
    // workgroup -> work mapping of this launch (set by finish_mapping() in intfa_launch.h from the grid size)
    int32_t per_head;                      // workgroups per query head
    int32_t heads_kv;                      // heads / kv_group
    int32_t xcd_whole_wgs;                 // workgroups of the K/V heads that are dealt whole to the 8 XCDs (a multiple of 8)
    int32_t xcd_rem_chunk;                 // the remaining heads: consecutive workgroups per XCD (0: dealt one by one)
    FastDiv d_per_kv, d_heads_kv, d_per_head, d_n_split, d_heads, d_kv_group;
};

// The kernel's own argument block as the epilogues re-read it: the pointer keeps the constant address space, so its
// fields arrive through scalar loads (a generic pointer would make them vector loads that a vmcnt wait has to cover).
typedef const __attribute__((address_space(4))) KParams* KernargPtr;
__device__ __forceinline__ KernargPtr kernarg_block() {
    KernargPtr pe = (KernargPtr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(pe));       // opaque: the fields are loaded where they are used, not held since the prologue
    return pe;
}
__device__ __forceinline__ float load_scale(const char* base, int64_t idx, int dtype) {
    if (dtype == 0) return (float)((const _Float16*)base)[idx];
    if (dtype == 1) return __builtin_bit_cast(float, ((uint32_t)((const uint16_t*)base)[idx]) << 16);
    return ((const float*)base)[idx];
}

// ---- What every forward kernel does before its main loop: which (batch, head, query block, split) the workgroup
// works on, which key blocks it visits, its Q fragments and scales.  One copy, shared by the four kernels.

// blockIdx.x -> (batch * heads + head, index among the head's `per_head` workgroups).  Workgroups are dealt round-robin to
// the 8 XCDs, each with its own L2: every XCD gets whole K/V heads, so the K/V tiles of a head are re-read from one L2.
// With grouped K/V heads (kv_group query heads share one K/V head) the unit dealt to an XCD is the K/V head: all query
// heads of a group run on the XCD whose L2 holds their K/V.
// When the number of (batch, K/V head) pairs is no multiple of 8, the first 8 * floor(pairs / 8) are dealt whole as above and
// the workgroups of the remaining pairs, taken in head order, are cut into 8 equal runs, one per XCD: a remaining head's
// K/V then reaches two or three L2s instead of all eight.
// (All divisors are fixed per launch: fast_div.)
struct WorkgroupJob { int b, h, hk, rem; };      // batch entry, query head, K/V head, index among the head's workgroups
__device__ __forceinline__ WorkgroupJob deal_workgroup(const KParams& p, int bid) {
    const int kv_group = p.kv_group;
    const int per_head = p.per_head;
    const int per_kv = per_head * kv_group;              // workgroups per K/V head
    int kv_lin, r;
    if (bid < p.xcd_whole_wgs) {
        const int xcd = bid & 7, slot = bid >> 3;
        const int q = fast_div(slot, p.d_per_kv);
        kv_lin = q * 8 + xcd;
        r = slot - q * per_kv;
    } else {
        const int j = bid - p.xcd_whole_wgs;                        // (xcd_whole_wgs is a multiple of 8: j & 7 is the XCD)
        const int idx = p.xcd_rem_chunk ? (j & 7) * p.xcd_rem_chunk + (j >> 3) : j;
        const int q = fast_div(idx, p.d_per_kv);
        kv_lin = fast_div(p.xcd_whole_wgs, p.d_per_kv) + q;
        r = idx - q * per_kv;
    }
    const int bb = fast_div(kv_lin, p.d_heads_kv), hk = kv_lin - bb * p.heads_kv;
    const int hq = fast_div(r, p.d_per_head);            // query head inside the group
    return {bb, hk * kv_group + hq, hk, r - hq * per_head};
}

// Number of keys of batch entry b: one length for all, or per batch (a cache filled to different lengths), clamped to
// [0, seqlen_k] so that rows past the allocation are never addressed.
__device__ __forceinline__ int keys_of_batch(const KParams& p, int b) {
    int seqlen_k = p.seqlen_k;
    if (p.seqlens_k != nullptr) {
        const int n = p.seqlens_k[b];
        seqlen_k = n < 0 ? 0 : (n < seqlen_k ? n : seqlen_k);
    }
    return seqlen_k;
}

// Key blocks [begin, end) of BN keys that a workgroup visits.  `visible_end` is the end of the range before a split
// narrows it (the blocks that hold a key visible to some row of the workgroup).
//   causal: the mask is aligned to the bottom right corner (csrc/mask.h:53,172 of the reference's CUDA tree): the row at
//           position i sees keys 0 .. i + causal_off, causal_off = seqlen_k - (number of positions); pos_end is one past the
//           workgroup's largest position.
//   split_on: with deal_visible the VISIBLE blocks are dealt evenly to the splits (no split of a query block is empty or
//           short); otherwise the blocks of the whole sequence are, blocks_per_split each (csrc/flash_fwd_kernel.h:503-511).
struct KeyBlocks { int total, begin, end, visible_end; };
template <int BN>
__device__ __forceinline__ KeyBlocks key_block_range(int seqlen_k, bool causal, int pos_end, int causal_off, bool split_on, int n_split,
                                                     int split, bool deal_visible, int blocks_per_split) {
    KeyBlocks r;
    r.total = (seqlen_k + BN - 1) / BN;
    r.begin = 0;
    r.end = r.total;
    if (causal) {
        const int e = (pos_end + causal_off + BN - 1) / BN;
        r.end = e < 0 ? 0 : (e < r.total ? e : r.total);
    }
    r.visible_end = r.end;
    if (split_on) {
        const int per = deal_visible ? (r.end + n_split - 1) / n_split : blocks_per_split;
        r.begin = split * per;
        const int e = r.begin + per;
        r.end = e < r.end ? e : r.end;
    }
    return r;
}

// int8 Q fragments of query row q_ld (B operand of S^T = K Q^T): 16 bytes per k-step of 32, the half lh of the lane.
template <int KS>
__device__ __forceinline__ void load_q8_fragments(v4i (&qreg)[KS], const KParams& p, int b, int h, int q_ld, int lh) {
    const char* qrow = p.q + b * p.q_sb + h * p.q_sh + (int64_t)q_ld * p.q_sn;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qreg[ks] = *(const v4i*)(qrow + ks * 32 + lh * 16);
}
// q_scale of query row q_ld times sm_scale * log2(e): the factor between S * k_scale and the exponent of exp2.
__device__ __forceinline__ float load_q_scale_log2(const KParams& p, int b, int h, int q_ld) {
    return load_scale(p.q_scale, b * p.qs_sb + h * p.qs_sh + (int64_t)q_ld * p.qs_sn, p.scale_dtype) * p.qk_scale_log2;
}

// k_scale of the keys of one (batch, K/V head): fetched as raw bits (one key per thread, ahead of the block that uses
// them) and converted to fp32 when stored to LDS.  Keys past the end read the last key's scale; they are masked later.
struct KScaleSource {
    const char* base;
    int stride, dtype, seqlen_k;
    __device__ __forceinline__ KScaleSource(const KParams& p, int b, int hk, int seqlen_k_) {
        const int esize = p.scale_dtype == 2 ? 4 : 2;
        base = p.k_scale + (b * p.ks_sb + hk * p.ks_sh) * esize;
        stride = (int)(p.ks_sn * esize);
        dtype = p.scale_dtype;
        seqlen_k = seqlen_k_;
    }
    __device__ __forceinline__ uint32_t load(int key) const {
        key = key < seqlen_k ? key : seqlen_k - 1;
        const char* src = base + (int64_t)key * stride;
        if (dtype == 2) return *(const uint32_t*)src;
        return (uint32_t)*(const uint16_t*)src;
    }
    __device__ __forceinline__ float cvt(uint32_t raw) const {
        if (dtype == 0) return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
        if (dtype == 1) return __builtin_bit_cast(float, raw << 16);
        return __builtin_bit_cast(float, raw);
    }
};

// ---- LDS swizzles.  A tile row is ROW_BYTES bytes; its 16-byte chunks are XOR-permuted with a function of the
// row so that the rows touched together by one LDS access cycle (64 banks x 4 bytes = 256 bytes: 16 lanes of a
// 16-byte read, 32 lanes of an 8-byte read) fall into different bank groups.  Every function depends on the low
// four bits of the row only.
enum { SWZ_K = 0, SWZ_V8 = 1, SWZ_V16 = 2 };
// K / Q style rows: 16 consecutive lanes read the same chunk of 16 consecutive rows.
template <int ROW_BYTES> __device__ __forceinline__ int swz_k(int row) {
    if (ROW_BYTES >= 256) return row & 15;                           // every row starts at bank 0
    if (ROW_BYTES == 128) return (row & 7) ^ ((row >> 3) & 1);       // rows r, r+8 share banks: flip bit 0
    return (row >> 2) & 3;                                           // 64-byte rows: rows r, r+4, r+8, r+12 share banks
}
// int8 V rows read by ds_read_b64_tr_b8: a 16-lane group touches rows {0,1,2,3,8,9,10,11} + 4h of a sub-tile.
template <int ROW_BYTES> __device__ __forceinline__ int swz_v8(int row) {
    // 256-byte rows all start at bank 0, and the two 16-lane groups served together read neighbouring chunks (2 dt and
    // 2 dt + 1) of eight rows each: even flips keep the groups in the even and the odd chunks respectively
    if (ROW_BYTES >= 256) return 2 * ((row & 3) | ((row >> 1) & 4));
    if (ROW_BYTES >= 128) return (row & 3) | ((row >> 1) & 4);
    return ((row >> 1) & 1) | ((row >> 2) & 2);
}
// 16-bit V rows read by ds_read_b64_tr_b16: 32 lanes touch 4 consecutive rows x 64 contiguous bytes.
template <int ROW_BYTES> __device__ __forceinline__ int swz_v16(int row) {
    if (ROW_BYTES >= 256) return (row & 3) << 2;
    return ((row >> 1) & 1) << 2;                                    // 128-byte rows: rows r, r+1 differ by half
}
template <int ROW_BYTES, int SWZ> __device__ __forceinline__ int swz(int row) {
    return SWZ == SWZ_K ? swz_k<ROW_BYTES>(row) : (SWZ == SWZ_V8 ? swz_v8<ROW_BYTES>(row) : swz_v16<ROW_BYTES>(row));
}

// Asynchronous copy of one ROWS-row tile (ROW_BYTES bytes per row) from global memory straight into LDS with
// buffer_load_dwordx4 ... lds: every wave instruction moves 64 x 16 bytes into 1 KiB of consecutive LDS, so the
// swizzle is applied on the GLOBAL side (which chunk a lane fetches).  The four waves split the instructions.
// Addressing is split into a wave-uniform part (SGPRs) and a per-lane 32-bit offset.  The swizzle of a row depends
// on the row's low four bits only; wave w issues instructions w, w+4, w+8, ... whose first rows differ by
// multiples of 4*RPI rows, so a lane needs one offset when 4*RPI >= 16 and 16/(4*RPI) otherwise.
template <int ROW_BYTES, int SWZ, int ROWS> struct TileLoadLane {
    static constexpr int CH = ROW_BYTES / 16;        // 16-byte chunks per row
    static constexpr int RPI = 64 / CH;              // rows per wave instruction
    static constexpr int NINST = ROWS * CH / 64;     // wave instructions per tile
    static constexpr int NV = (4 * RPI >= 16) ? 1 : 16 / (4 * RPI);
    static_assert(CH >= 4 && CH <= 32 && NINST % 4 == 0, "unsupported tile geometry");
    uint32_t off[NV];
};
template <int ROW_BYTES, int SWZ, int ROWS>
__device__ __forceinline__ TileLoadLane<ROW_BYTES, SWZ, ROWS> tile_load_lane(uint32_t row_stride, int wave, int lane) {
    using T = TileLoadLane<ROW_BYTES, SWZ, ROWS>;
    const int rsub = lane / T::CH, cp = lane % T::CH;
    T t;
#pragma unroll
    for (int v = 0; v < T::NV; ++v) {
        const int row = (v * 4 + wave) * T::RPI + rsub;
        const int f = swz<ROW_BYTES, SWZ>(row) & (T::CH - 1);
        t.off[v] = (uint32_t)rsub * row_stride + (uint32_t)((cp ^ f) << 4);
    }
    return t;
}
// The global side is addressed through a buffer resource (base pointer of the (batch, head) slice, SGPRs) plus a
// wave-uniform byte offset (SGPR) plus the lane's 32-bit offset: no 64-bit per-lane pointers.  The copy itself is
// written as inline assembly (M0 = LDS destination of the wave's 1 KiB, then buffer_load_dwordx4 ... lds) so that
// the compiler does not serialise later LDS reads of the OTHER buffer behind it; completion is awaited explicitly
// with s_waitcnt vmcnt(0) before the workgroup barrier that publishes the tile.
__device__ __forceinline__ v4i make_rsrc(const void* base, uint32_t bytes) {
    const uint64_t a = (uint64_t)base;
    v4i r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu));   // stride 0: raw buffer
    r[2] = __builtin_amdgcn_readfirstlane((int)bytes);                              // num_records, bounds-checked
    r[3] = 0x00020000;
    return r;
}
// Issues wave instruction number `it` (0 .. NINST/4 - 1) of this wave's share of one tile copy.
// The statement overwrites M0 and cannot say so: the compiler keeps M0 reserved on this target, warns about a clobber
// entry for it and ignores it.  Nothing the compiler generates in these kernels reads M0 (no LDS-DMA builtins, GWS,
// relative moves or interpolation), and every copy sets it afresh.  tile_off and row_stride must be wave-uniform values
// the compiler can see as such (kernel arguments, readfirstlane results): they end up in scalar operands.
template <int ROW_BYTES, int SWZ, int ROWS>
__device__ __forceinline__ void issue_tile_part(v4i rsrc, uint32_t tile_off, uint32_t row_stride, uint32_t lds_tile,
                                                int wave, const TileLoadLane<ROW_BYTES, SWZ, ROWS>& ln, int it) {
    using T = TileLoadLane<ROW_BYTES, SWZ, ROWS>;
    const int i = it * 4 + wave;                     // wave-uniform instruction index
    const uint32_t m0v = lds_tile + (uint32_t)i * 1024u;
    const uint32_t soff = tile_off + (uint32_t)(i * T::RPI) * row_stride;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(m0v), "v"(ln.off[it % T::NV]), "s"(rsrc), "s"(soff) : "memory");
}
template <int ROW_BYTES, int SWZ, int ROWS>
__device__ __forceinline__ void issue_tile_load(v4i rsrc, uint32_t tile_off, uint32_t row_stride, uint32_t lds_tile,
                                                int wave, const TileLoadLane<ROW_BYTES, SWZ, ROWS>& ln) {
    using T = TileLoadLane<ROW_BYTES, SWZ, ROWS>;
#pragma unroll
    for (int it = 0; it < T::NINST / 4; ++it) issue_tile_part<ROW_BYTES, SWZ, ROWS>(rsrc, tile_off, row_stride, lds_tile, wave, ln, it);
}

// ---- 16-bit output rows through LDS.  In the accumulator layout a lane holds four consecutive columns of ONE row per
// register quad, so a direct store writes 8-byte pieces of 32 different rows per instruction and every 64-byte line
// of the output is touched by several partial writes.  Each wave therefore stages its 32 rows x NCOL columns in a
// private LDS region (rows of NCOL * 2 bytes, 16-byte chunks XOR-permuted by the row so that neither the 8-byte
// writes nor the 16-byte reads meet in a bank) and writes them out with 16 bytes per lane: a row's NCOL * 2 bytes are
// contiguous in one store instruction.  The region must be dead tile memory: a workgroup barrier lies between the last
// tile read of any wave and the first out_stage_put.
template <int NCOL> struct OutStage {
    static constexpr int RS = NCOL * 2;                  // bytes per staged row
    static constexpr int CH = RS / 16;                   // 16-byte chunks per row
    static constexpr int RPB = RS >= 256 ? 1 : 256 / RS; // rows per 256 bytes (one pass over the banks)
    static constexpr int BYTES = 32 * RS;                // per wave
    static constexpr int LPR = RS / 16, RPI = 64 / LPR;  // lanes per row / rows per store instruction
    static_assert(NCOL == 64 || NCOL == 128, "staging is laid out for 128- and 256-byte rows");
    static __device__ __forceinline__ int key(int row) { return (row / RPB) & (CH - 1); }
};
// four 16-bit values (columns d0 .. d0 + 3, d0 a multiple of 4) of the wave's row `row`
template <int NCOL>
__device__ __forceinline__ void out_stage_put(char* stage, int row, int d0, v2i bits) {
    using S = OutStage<NCOL>;
    *(v2i*)(stage + row * S::RS + ((((d0 * 2) >> 4) ^ S::key(row)) << 4) + ((d0 * 2) & 15)) = bits;
}
// g_row0: global address of the wave's first row (column offset applied); rows_valid: how many of the 32 rows exist
template <int NCOL>
__device__ __forceinline__ void out_stage_flush(const char* stage, char* g_row0, int64_t row_stride, int rows_valid, int lane) {
    using S = OutStage<NCOL>;
    const int sub = lane / S::LPR, ch = lane % S::LPR;
#pragma unroll
    for (int j = 0; j < 32 / S::RPI; ++j) {
        const int row = j * S::RPI + sub;
        const v4i x = *(const v4i*)(stage + row * S::RS + ((ch ^ S::key(row)) << 4));
        if (row < rows_valid) *(v4i*)(g_row0 + row * row_stride + ch * 16) = x;
    }
}

// fp32 -> bf16 in hardware (v_cvt_pk_bf16_f32 converts two values per instruction, round-to-nearest-even): what the
// attention kernels use for P and for the output.  (The quantisers keep the integer form below: they reproduce another
// library's results bit for bit, NaN patterns included.)
__device__ __forceinline__ short f32_to_bf16(float f) { return __builtin_bit_cast(short, (__bf16)f); }
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {   // round-to-nearest-even
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

// Reductions across the two lanes that share a query column (lane l and lane l ^ 32): v_permlane32_swap turns
// one register into (lower halves, upper halves), so one swap plus one max/add serves all 64 lanes.
__device__ __forceinline__ float half_pair_max(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float half_pair_sum(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// v for a visible key, -inf for a hidden one (key index k_r past the lane's last visible index `last`), without a
// compare and select: min with a threshold that is +inf or -inf by the sign of last - k_r.  No condition registers,
// so the statement cannot be merged with a wave-uniform test around it into a select per element.
__device__ __forceinline__ float hide_past(float v, int last, int k_r) {
    const uint32_t t = (uint32_t)(last - k_r);
    return __builtin_fminf(v, __builtin_bit_cast(float, (t & 0x80000000u) | 0x7f800000u));
}

// The reference's requantisation of P (flash_atten_full_int8.py:49-51) for the 16 probabilities a lane holds of one 32-key
// sub-tile, in the reference's own fp16 operations: fp16(p) (round to nearest even) * 127 -> fp16, + 0.5 -> fp16,
// truncating conversion to an integer.  The multiply and the add are the packed fp16 instructions (two values each; kept
// apart: a fused multiply-add would skip the rounding of the product).  The sixteen truncating conversions write their
// byte straight into the four packed words (SDWA destination select).  A write with a destination select needs one wait
// state before the next vector instruction touches that register, and the compiler places wait states for its own
// instructions only: the conversions are therefore issued word-interleaved (bytes 0 of the four words, then bytes 1, ...),
// so that three other conversions lie between two writes to one word, each round as ONE asm statement so that nothing can
// be scheduled into it, and a single s_nop closes the last round before the words can be consumed.
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ v4i requant_p_reference16(const float (&p)[16]) {
    unsigned hb[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        v2h h = __builtin_convertvector((v2f){p[2 * i], p[2 * i + 1]}, v2h);
        {
#pragma clang fp contract(off)
            h = h * (v2h){(_Float16)127.0f, (_Float16)127.0f};
            h = h + (v2h){(_Float16)0.5f, (_Float16)0.5f};
        }
        hb[i] = __builtin_bit_cast(unsigned, h);
    }
    unsigned w0, w1, w2, w3;
    asm volatile("v_cvt_u16_f16_sdwa %0, %4 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:WORD_0\n\t"
                 "v_cvt_u16_f16_sdwa %1, %5 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:WORD_0\n\t"
                 "v_cvt_u16_f16_sdwa %2, %6 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:WORD_0\n\t"
                 "v_cvt_u16_f16_sdwa %3, %7 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:WORD_0"
                 : "=&v"(w0), "=&v"(w1), "=&v"(w2), "=&v"(w3) : "v"(hb[0]), "v"(hb[2]), "v"(hb[4]), "v"(hb[6]));
    asm volatile("v_cvt_u16_f16_sdwa %0, %4 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"
                 "v_cvt_u16_f16_sdwa %1, %5 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"
                 "v_cvt_u16_f16_sdwa %2, %6 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"
                 "v_cvt_u16_f16_sdwa %3, %7 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1"
                 : "+v"(w0), "+v"(w1), "+v"(w2), "+v"(w3) : "v"(hb[0]), "v"(hb[2]), "v"(hb[4]), "v"(hb[6]));
    asm volatile("v_cvt_u16_f16_sdwa %0, %4 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0\n\t"
                 "v_cvt_u16_f16_sdwa %1, %5 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0\n\t"
                 "v_cvt_u16_f16_sdwa %2, %6 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0\n\t"
                 "v_cvt_u16_f16_sdwa %3, %7 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0"
                 : "+v"(w0), "+v"(w1), "+v"(w2), "+v"(w3) : "v"(hb[1]), "v"(hb[3]), "v"(hb[5]), "v"(hb[7]));
    asm volatile("v_cvt_u16_f16_sdwa %0, %4 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"
                 "v_cvt_u16_f16_sdwa %1, %5 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"
                 "v_cvt_u16_f16_sdwa %2, %6 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"
                 "v_cvt_u16_f16_sdwa %3, %7 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n\t"
                 "s_nop 0"
                 : "+v"(w0), "+v"(w1), "+v"(w2), "+v"(w3) : "v"(hb[1]), "v"(hb[3]), "v"(hb[5]), "v"(hb[7]));
    return (v4i){(int)w0, (int)w1, (int)w2, (int)w3};
}

}  // namespace intfa
