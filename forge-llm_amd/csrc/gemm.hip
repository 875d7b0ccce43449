// Batched-prefill quantised GEMM (matmul_mat_q8_0_KxN / matmul_mat_q4_0_KxN, emit.rs:2108-2302,
// 3667-3817):  y[m][n] = sum_b (a_s[m][b] * w_s[n][b]) * f32(isum[m][n][b]).
//
// Both products of the formula run on the matrix unit:
//   * v_mfma_i32_32x32x32_i8 has K = 32 = exactly one quant block, so each MFMA result is a 32x32 tile
//     of exact int32 block sums;
//   * the scale products a_s[m]*w_s[n] of that tile are a rank-1 outer product of fp16 values, exact in
//     f32 (11-bit x 11-bit significands): one v_mfma_f32_32x32x16_f16 with the scales in k = 0 and zeros
//     elsewhere (fp16 subnormal scales included; the unit does not flush them).
// The scaling itself is elementwise in (m, n, b) and has to be done on the VALU.  In exact mode that is
// int->float, multiply, add per element: bit for bit the reference's `r += (a_scale*w_scale) * f32(isum)` in
// block order.  That VALU work, not the matrix unit, bounds the kernel (32 VALU instructions = 128 cycles per
// 64 cycles of MFMA), so the fast mode halves it by never converting: the integer MFMA starts from
// C = 0x4B400000 in every element, which makes its int32 result, read as f32, the number 12582912 + isum
// exactly (|isum| <= 516128 < 2^22), and one FMA per element adds S * (12582912 + isum).  To keep the
// accumulators near their true size the bias alternates in sign: in odd blocks the activation codes come
// negated (the quantising kernels store them so for this kernel: no work here) and the weight scale carries a
// minus sign, which adds S * (isum - 12582912).  What
// is left of the bias after 8 blocks, 12582912 * sum_b (+-)S_b, is itself a product of the scales: one more
// f16 MFMA (k = the 8 blocks) gives it, and one FMA per element takes it out.  Block sums stay exact; the
// f32 accumulation carries a rounding error of about 2e-5 of the typical output (measured; 1e-7 in the
// cvt + FMA form), inside the 1e-3 the fast mode is held to.
//
// Tiling: 256 threads = 4 waves (2x2), workgroup tile 128 (m) x 128 (n), wave tile 64x64 = 2x2 MFMA
// tiles, K step 128 (4 blocks).  Activations are the MFMA A operand (rows), weights the B operand
// (columns): a lane's 16 results share one weight row n, stores are contiguous in n.
// Two waves per SIMD (<= 256 VGPRs) so that MFMA results land in ordinary VGPRs, not AccVGPRs.
//
// Data movement: int8 operand tiles go from global memory straight into LDS (buffer loads with the LDS
// destination; Q4_0 weights pass through registers to have their nibbles expanded), into one of two
// buffers, so that a stage needs one barrier and the loads of stage s+1 fly under the arithmetic of
// stage s.  LDS rows are 128 B, unpadded; the 16-byte chunk c of row r sits at position
// c ^ ((r >> 1) & 7), which makes the fragment reads (32 rows x one chunk) free of bank conflicts.
// All global accesses go through buffer descriptors: rows past the end of a matrix read as zero and
// stores past the end are dropped by the hardware's range check, so the loops carry no predication.
// A K tail (K % 128) reads whatever follows in the row-major matrix; those blocks get scale 0.
#include <type_traits>

#include "common.h"
#include "device_utils.h"

namespace fh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int BM = 128, BN = 128, BK = 128;   // BK in elements (= bytes of int8)
constexpr int KB = BK / 32;                   // quant blocks per stage
constexpr int TILE_BYTES = BM * BK;           // one operand tile of one stage in LDS
// LDS map: A tiles [2], B tiles [2], A scales [2][128 rows][4] fp16, B scales likewise, 512 zero bytes
// scale tables: [4 stage slots][128 rows][4 blocks] fp16, slot = stage & 3 (rows 8 bytes apart: 32 rows, 32 banks)
constexpr int SC_ROW = KB * 2, SC_SLOT = BM * SC_ROW;
constexpr int LDS_A = 0, LDS_B = 2 * TILE_BYTES, LDS_ASC = 4 * TILE_BYTES, LDS_BSC = LDS_ASC + 4 * SC_SLOT,
              LDS_ZERO = LDS_BSC + 4 * SC_SLOT, GEMM_LDS_BYTES = LDS_ZERO + 512;
constexpr uint32_t MAGIC_BITS = 0x4B400000u;  // 12582912.0f = 1.5 * 2^23: ulp 1, room for +-2^22
// The fast mode's bias removal multiplies the activation scales by 2^SCALE_A_LOG2 and the weight scales by
// 2^(23 - SCALE_A_LOG2) (and half of that) on their way into an f16 MFMA.  The factors themselves (256, 32768) and the
// products are exact fp16 numbers while a_s < 2^(16 - SCALE_A_LOG2) = 256 (a block's largest activation below 32 512) and
// w_s < 2 (Q8_0 weights below 254, Q4_0 weights below 16 in magnitude).
constexpr int SCALE_A_LOG2 = 8;
static_assert(23 - SCALE_A_LOG2 <= 15, "2^16 is not an fp16 number");
constexpr uint32_t RSRC_FLAGS = 0x00020000;   // raw buffer, 32-bit data format
constexpr uint32_t OOB = 0x80000000u;         // an offset no descriptor here covers
constexpr uint32_t GEMM_SPLIT_MAX_ITEMS = 256; // K ranges one launch may park in the split workspace (64 KB each)

#define FH_LDS3(p) ((__attribute__((address_space(3))) void*)(p))

// (c - 8) for each of four nibble codes c held in the low nibbles of the four bytes.
__device__ __forceinline__ uint32_t nib_minus8(uint32_t x) {
    return ((x | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

// EXACT: multiply then add per block (bit-identical to the CPU path); otherwise one FMA per block.
// TM: 32-row tiles per wave along m.  2 = the 128-row workgroup tile; 1 = a 64-row tile for problems so small that even
// twice the workgroups leave CUs idle (a workgroup's time per K stage halves with its tile).
// SPLIT (fast mode only): a one-dimensional grid of work items.  The first `full_tiles` output tiles (row-major over the
// tile grid) are worked over the whole of K by one workgroup each, as in the other variants; each of the remaining tiles
// is cut into `split` ranges of `stages_per_part` K stages, one workgroup per range, whose partial tiles go to
// `partials`; the workgroup that finishes a tile's last range adds the ranges in range order (so the result does not
// depend on who came last) and stores the tile.  The launch code uses it when the tiles fill the CUs once and a fraction:
// the fraction is what gets cut, so that every CU ends up with the same amount of work.
// SILU (fast mode only): the matrix is a fused [gate; up] pair of `inter` rows each (emit.rs:5390-5420 computes both from
// the same normalised row).  A workgroup's 128 columns are then 64 consecutive inter indices: each wave's first 32-column
// tile holds gate rows i0 .. i0 + 32, its second the up rows of the same indices, so a lane ends up with gate and up of
// one (row, index) pair and the epilogue is silu(gate) * up (emit.rs:380-386, hardware exp) and the activation quantiser
// (emit.rs:1410-1440: the 32 indices of a tile are exactly one block, spread over 32 lanes) -- the down projection's
// input, codes and scales, instead of 2 * inter floats per row written and read back.
struct GemmSplit {
    uint32_t full_tiles, split, stages_per_part;
    float* partials;        // [tiles - full_tiles][split][tile elements]
    uint32_t* counters;     // [tiles - full_tiles], zero between launches
    int8_t* silu_q;         // SILU: [M][inter] codes (odd blocks negated, as the fast GEMM takes its activations)
    uint16_t* silu_sc;      // SILU: [M][inter / 32] fp16 scales
    uint32_t inter;
    const float* mt_a;      // MINT: [M][K / 32] slots of 4 bytes (a hi | lo pair of fp16 numbers), one per activation block
    const float* mt_w;      // MINT: [N][K / 32] slots likewise, one per weight block
};

// MINT: the tile additionally receives sum_b mt_a[m][b] * mt_w[n][b], a matmul of depth K / 32 on the f16 matrix unit (operands
// as hi | lo pairs of fp16 numbers) in front of the epilogue (the minimum term of a Q4_K matrix: activation block sums times a coefficient per weight block,
// kquant_prefill.hip) -- so that it costs no pass over the result and may precede the SiLU epilogue.
template <bool Q4, bool DUMP, bool EXACT, int TM, bool SPLIT = false, bool SILU = false, bool MINT = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
void gemm_q_kernel(const uint8_t* __restrict__ wq, const uint16_t* __restrict__ wsc, const int8_t* __restrict__ aq,
                   const uint16_t* __restrict__ asc, float* __restrict__ y, int32_t* __restrict__ isums, uint32_t M,
                   uint32_t N, uint32_t K, uint32_t ldy, int accumulate, GemmSplit sp) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr bool MAGIC = !EXACT;               // DUMP && !EXACT: the fast arithmetic, with its block sums written out too
    static_assert(!SPLIT || (MAGIC && !DUMP), "K ranges change the order of the block sum: fast mode only");
    static_assert(!SILU || (MAGIC && !DUMP), "the fused SiLU epilogue belongs to the fast mode");
    static_assert(!MINT || (MAGIC && !DUMP && !Q4), "the extra f32 term belongs to the fast mode on Q8_0-layout matrices (no 1/16 pending)");

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));   // uniform: the compiler keeps it scalar
    const uint32_t wm = wave >> 1, wn = wave & 1;
    constexpr int WM = 32 * TM;                  // rows of a wave's tile
    const uint32_t stages = (K + BK - 1) / BK;
    uint32_t tile_x = blockIdx.x, tile_y = blockIdx.y, s_begin = 0, s_end = stages;
    bool ranged = false;                         // this workgroup holds one K range of its tile
    uint32_t range_tile = 0;                     // index of the tile among the cut ones
    if (SPLIT) {
        const uint32_t gx = (N + BN - 1) / BN;
        uint32_t tile = blockIdx.x;
        if (tile >= sp.full_tiles) {
            const uint32_t r = tile - sp.full_tiles;
            range_tile = r / sp.split;
            tile = sp.full_tiles + range_tile;
            s_begin = (r % sp.split) * sp.stages_per_part;       // even: the bias is taken out per pair of stages
            s_end = s_begin + sp.stages_per_part < stages ? s_begin + sp.stages_per_part : stages;
            ranged = true;
        }
        tile_x = tile % gx; tile_y = tile / gx;
    }
    const uint32_t m0 = tile_y * (2 * WM), n0 = tile_x * BN;
    const uint32_t nblk = K / 32;
    const uint32_t lrow = lane & 31, lhalf = lane >> 5;
    const uint32_t wrow = Q4 ? K / 2 : K;   // bytes of one weight row

    const __amdgpu_buffer_rsrc_t rdump = __builtin_amdgcn_make_buffer_rsrc((void*)isums, 0, DUMP ? M * N * nblk * 4 : 0, RSRC_FLAGS);

    // ---- loader mapping: load i of wave w fills LDS rows (4i + w) * 8 .. + 8 of a tile, lane -> (row, position)
    const uint32_t ld_row = wave * 8 + (lane >> 3);                        // + 32 i
    const uint32_t ld_chunk = (lane & 7) ^ ((ld_row >> 1) & 7);            // global chunk for LDS position lane & 7
    const uint32_t a_voff = (m0 + ld_row) * K + ld_chunk * 16;             // + 32 i K + k0
    // SILU: tile row j is weight row i0 + (j / 64) * 32 + j % 32 (+ inter for the up half, (j / 32) odd), i0 = 64 tile_x
    const uint32_t s_inter = SILU ? sp.inter : 0u, si0 = tile_x * 64;
    const uint32_t w_voff = (SILU ? si0 + ld_row : n0 + ld_row) * K + ld_chunk * 16;     // Q8_0 only; load i: + w_step[i]
    // Q4_0: piece idx = tid + 256 i: row = idx / 4, block = idx % 4 (16 packed bytes -> 32 codes)
    const uint32_t q4_row = tid >> 2, q4_blk = tid & 3;                    // + 64 i
    const uint32_t q4_wrow = SILU ? si0 + (q4_row & 31) + (q4_row >> 5) * s_inter : n0 + q4_row;
    const uint32_t q4_voff = (q4_wrow * nblk + q4_blk) * 16;               // + q4_step i + (k0/32) 16
    // scales: threads 0..127 take activation row tid, threads 128..255 weight row tid - 128
    const bool sc_is_a = wave < 2;
    const uint32_t sc_row = tid & 127;
    const uint32_t sc_wrow = SILU ? si0 + (sc_row >> 6) * 32 + (sc_row & 31) + ((sc_row >> 5) & 1) * s_inter : n0 + sc_row;
    const uint32_t sc_voff = (sc_is_a ? m0 + sc_row : sc_wrow) * nblk * 2;
    // uniform steps from load to load (rows 32 i further on; SILU: 32 (i / 2) further on, odd loads in the up half)
    const uint32_t w_step[4] = {0u, SILU ? s_inter * K : 32 * K, SILU ? 32 * K : 64 * K, SILU ? 32 * K + s_inter * K : 96 * K};
    const uint32_t q4_step = (SILU ? 32u : 64u) * nblk * 16;

    v4i rb[2];
    uint32_t rs[KB];

    // The K position of a stage moves the descriptors (scalar work: base + k0, records - k0), not the lanes' offsets: the
    // range check still sees the whole offset (a scalar offset operand would be left out of it), and the per-lane
    // offsets stay the same from stage to stage.
    // part: which of the stage's loads to issue (1: activation tile, 2: weight tile, 4: scales; 7: all)
    auto issue_stage = [&](uint32_t k0, uint32_t buf, int part = 7) {
        const uint32_t kq = Q4 ? k0 / 2 : k0, ks = (k0 / 32) * 2;
        // 0 records: every access is out of range.  (readfirstlane: the value is uniform, and a descriptor word in a
        // vector register would cost a loop over its values around every load.)
        auto left = [](uint32_t total, uint32_t skip) {
            return (uint32_t)__builtin_amdgcn_readfirstlane((int)(total > skip ? total - skip : 0u));
        };
        const __amdgpu_buffer_rsrc_t ra_k = __builtin_amdgcn_make_buffer_rsrc((void*)(aq + k0), 0, left(M * K, k0), RSRC_FLAGS);
        const __amdgpu_buffer_rsrc_t rw_k = __builtin_amdgcn_make_buffer_rsrc((void*)(wq + kq), 0, left(N * wrow, kq), RSRC_FLAGS);
        const __amdgpu_buffer_rsrc_t ras_k = __builtin_amdgcn_make_buffer_rsrc((void*)((const uint8_t*)asc + ks), 0, left(M * nblk * 2, ks), RSRC_FLAGS);
        const __amdgpu_buffer_rsrc_t rws_k = __builtin_amdgcn_make_buffer_rsrc((void*)((const uint8_t*)wsc + ks), 0, left(N * nblk * 2, ks), RSRC_FLAGS);
        if (part & 1) {
#pragma unroll
            for (int i = 0; i < 2 * TM; i++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ra_k, FH_LDS3(lds + LDS_A + buf * TILE_BYTES + (i * 4 + wave) * 1024), 16,
                                                         a_voff + i * 32 * K, 0, 0, 0);
        }
        if ((part & 2) && Q4) {
#pragma unroll
            for (int i = 0; i < 2; i++) rb[i] = __builtin_amdgcn_raw_buffer_load_b128(rw_k, q4_voff + i * q4_step, 0, 0);
        } else if (part & 2) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rw_k, FH_LDS3(lds + LDS_B + buf * TILE_BYTES + (i * 4 + wave) * 1024), 16,
                                                         w_voff + w_step[i], 0, 0, 0);
        }
        if (part & 4) {
#pragma unroll
            for (int b = 0; b < KB; b++) {
                const uint32_t v = sc_is_a ? __builtin_amdgcn_raw_buffer_load_b16(ras_k, sc_voff + b * 2, 0, 0)
                                           : __builtin_amdgcn_raw_buffer_load_b16(rws_k, sc_voff + b * 2, 0, 0);
                rs[b] = v;          // looked at only when the stage is committed: nothing at the start of a stage waits for it
            }
        }
    };

    // what passes through registers: expanded Q4_0 codes and the scales
    auto commit_stage = [&](uint32_t buf, uint32_t slot, uint32_t blk0) {
        if (Q4) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint32_t row = q4_row + 64 * i, sw = (row >> 1) & 7;
                const v4i p = rb[i];
                const uint32_t m = 0x0F0F0F0Fu;
                v4i lo, hi;
                if (MAGIC) {
                    // 16 (c - 8) per byte: the biased accumulation resolves sums in units of 1 against a bias of 2^23,
                    // and 4-bit codes leave 4 bits of headroom (|16 isum| <= 520192); the epilogue divides by 16
                    const uint32_t h = 0xF0F0F0F0u, b = 0x80808080u;
                    lo.x = (int)((((uint32_t)p.x & m) << 4) ^ b); lo.y = (int)((((uint32_t)p.y & m) << 4) ^ b);
                    lo.z = (int)((((uint32_t)p.z & m) << 4) ^ b); lo.w = (int)((((uint32_t)p.w & m) << 4) ^ b);
                    hi.x = (int)(((uint32_t)p.x & h) ^ b); hi.y = (int)(((uint32_t)p.y & h) ^ b);
                    hi.z = (int)(((uint32_t)p.z & h) ^ b); hi.w = (int)(((uint32_t)p.w & h) ^ b);
                } else {
                lo.x = nib_minus8((uint32_t)p.x & m); lo.y = nib_minus8((uint32_t)p.y & m);
                lo.z = nib_minus8((uint32_t)p.z & m); lo.w = nib_minus8((uint32_t)p.w & m);
                hi.x = nib_minus8(((uint32_t)p.x >> 4) & m); hi.y = nib_minus8(((uint32_t)p.y >> 4) & m);
                hi.z = nib_minus8(((uint32_t)p.z >> 4) & m); hi.w = nib_minus8(((uint32_t)p.w >> 4) & m);
                }
                uint8_t* base = lds + LDS_B + buf * TILE_BYTES + row * BK;
                *reinterpret_cast<v4i*>(base + ((q4_blk * 2) ^ sw) * 16) = lo;       // elements 0..15 of the block
                *reinterpret_cast<v4i*>(base + ((q4_blk * 2 + 1) ^ sw) * 16) = hi;   // elements 16..31
            }
        }
        // blocks past the end of K (they hold the next row's scales) count with scale 0
        uint32_t sc4[KB];
#pragma unroll
        for (int b = 0; b < KB; b++) sc4[b] = (blk0 + b < nblk) ? (rs[b] & 0xFFFFu) : 0u;
        uint2 pk;
        pk.x = sc4[0] | (sc4[1] << 16);
        pk.y = sc4[2] | (sc4[3] << 16);
        if (MAGIC && !sc_is_a) { pk.x ^= 0x80000000u; pk.y ^= 0x80000000u; }   // odd blocks: minus sign on the weight scale
        *reinterpret_cast<uint2*>(lds + (sc_is_a ? LDS_ASC : LDS_BSC) + slot * SC_SLOT + sc_row * SC_ROW) = pk;
    };

    // ---- fragment addresses (bytes from the start of a tile / of a scale table)
    const uint32_t f_sw = (lrow >> 1) & 7;
    const uint32_t fa_off = (wm * WM + lrow) * BK + ((lhalf ^ f_sw) * 16);          // chunk of block kb: ^ (kb * 32)
    const uint32_t fb_off = (wn * 64 + lrow) * BK + ((lhalf ^ f_sw) * 16);
    // scale operand of the rank-1 product: lanes 0..31 hold k = 0 (the scale), lanes 32..63 read zeros
    const uint32_t sa_off = lhalf ? (uint32_t)LDS_ZERO : LDS_ASC + (wm * WM + lrow) * SC_ROW;
    const uint32_t sb_off = lhalf ? (uint32_t)LDS_ZERO : LDS_BSC + (wn * 64 + lrow) * SC_ROW;
    const uint32_t s_slot_stride = lhalf ? 0u : (uint32_t)SC_SLOT;
    const uint32_t s_t_stride = lhalf ? 0u : (uint32_t)(32 * SC_ROW);

    float acc[TM][2][16];
#pragma unroll
    for (int a = 0; a < TM; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    if (tid < 128) reinterpret_cast<uint32_t*>(lds + LDS_ZERO)[tid] = 0u;

    struct Frag {
        v4i af[TM], bf[2];
        uint32_t sa[TM], sb[2];
    };
    auto read_frag = [&](Frag& f, uint32_t buf, uint32_t slot, int kb) {
        const uint8_t* A = lds + LDS_A + buf * TILE_BYTES;
        const uint8_t* B = lds + LDS_B + buf * TILE_BYTES;
#pragma unroll
        for (int t = 0; t < 2; t++) {
            f.bf[t] = *reinterpret_cast<const v4i*>(B + ((fb_off ^ (kb * 32)) + t * 32 * BK));
            f.sb[t] = *reinterpret_cast<const uint16_t*>(lds + sb_off + slot * s_slot_stride + t * s_t_stride + kb * 2);
        }
#pragma unroll
        for (int t = 0; t < TM; t++) {
            f.af[t] = *reinterpret_cast<const v4i*>(A + ((fa_off ^ (kb * 32)) + t * 32 * BK));
            f.sa[t] = *reinterpret_cast<const uint16_t*>(lds + sa_off + slot * s_slot_stride + t * s_t_stride + kb * 2);
        }
    };
    // operand of the rank-1 product: the scale in k = 0, zeros in the other slots (the K = 8 form of the MFMA: two registers
    // per operand, one of them the zero, where the K = 16 form needs three zero registers beside every scale)
    typedef _Float16 v4s __attribute__((ext_vector_type(4)));
    auto scale_operand = [](uint32_t bits) {
        const _Float16 z = (_Float16)0.0f;
        return (v4s){__builtin_bit_cast(_Float16, (uint16_t)bits), z, z, z};
    };

    const v16i zero_i = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const v16f zero_f = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    v16i c_in = zero_i;                 // C operand of the integer MFMA: zeros, or the bias that makes the result a float
    if (MAGIC) {
#pragma unroll
        for (int r = 0; r < 16; r++) c_in[r] = (int)MAGIC_BITS;
    }

    issue_stage(s_begin * BK, 0);
    commit_stage(0, s_begin & 3, s_begin * KB);
    __builtin_amdgcn_s_waitcnt(0);      // vmcnt(0): the tiles of stage 0 are in LDS
    __syncthreads();

    // One stage: 4 blocks out of LDS buffer `buf` while the next stage's tiles fly into the other one.
    auto run_stage = [&](uint32_t s, uint32_t buf) {
        const uint32_t slot = s & 3;
        // unconditionally: past the last stage this fetches blocks that do not exist (zeros or the next row's
        // bytes, with scale 0), which keeps the loop body one straight block of code.  The next stage's loads go out in
        // three portions, the activation tile here, the weight tile and the scales behind the first and the second block:
        // a wave that issues all twelve at once sits in their issue for a fifth to a third of the stage (time stamps),
        // longer the fuller the memory pipeline is
        issue_stage((s + 1) * BK, buf ^ 1, 1);

        Frag fr[2];
        read_frag(fr[0], buf, slot, 0);
        v16i isum = __builtin_amdgcn_mfma_i32_32x32x32_i8(fr[0].af[0], fr[0].bf[0], c_in, 0, 0, 0);
        v16f S = __builtin_amdgcn_mfma_f32_32x32x8f16(scale_operand(fr[0].sa[0]), scale_operand(fr[0].sb[0]), zero_f, 0, 0, 0);
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            Frag& f = fr[kb & 1];
            Frag& fnext = fr[(kb + 1) & 1];
            if (kb + 1 < KB) read_frag(fnext, buf, slot, kb + 1);
            // four tiles, software-pipelined by one (across blocks too): the MFMAs of the next tile are issued
            // before this one is combined, so the matrix unit works while the VALU scales
            constexpr int NT = 2 * TM;           // MFMA tiles of a wave
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int tm = t >> 1, tn = t & 1;
                // next tile's two MFMAs, with this tile's combine split between them: the second MFMA would
                // otherwise wait (in order, blocking the FMAs behind it) for the first to clear the matrix pipe
                const bool has_next = t < NT - 1 || kb + 1 < KB;
                const Frag& fn = t < NT - 1 ? f : fnext;
                const int tm2 = t < NT - 1 ? (t + 1) >> 1 : 0, tn2 = t < NT - 1 ? (t + 1) & 1 : 0;
                v16i isum_n = zero_i;
                v16f S_n = zero_f;
                if (has_next) isum_n = __builtin_amdgcn_mfma_i32_32x32x32_i8(fn.af[tm2], fn.bf[tn2], c_in, 0, 0, 0);
                // pin each MFMA where it is written: left alone, the scheduler sinks it below the FMAs of its region, right in
                // front of its own first reader, and pays the matrix pipe's latency in wait states every tile
                __builtin_amdgcn_sched_barrier(0);
                const v16f biased = __builtin_bit_cast(v16f, isum);   // fast mode: 12582912 +- isum, exactly
                auto combine = [&](int r) {
                    if (MAGIC) {
                        acc[tm][tn][r] = fmaf(S[r], biased[r], acc[tm][tn][r]);
                    } else {
                        const float fl = (float)isum[r];
                        if (EXACT) acc[tm][tn][r] = acc[tm][tn][r] + S[r] * fl;
                        else acc[tm][tn][r] = fmaf(S[r], fl, acc[tm][tn][r]);
                    }
                };
#pragma unroll
                for (int r = 0; r < 8; r++) combine(r);
                __builtin_amdgcn_sched_barrier(0);
                if (has_next)
                    S_n = __builtin_amdgcn_mfma_f32_32x32x8f16(scale_operand(fn.sa[tm2]), scale_operand(fn.sb[tn2]), zero_f, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 8; r < 16; r++) combine(r);
                if (DUMP) {
                    const uint32_t b = s * KB + kb;
                    const uint32_t n = n0 + wn * 64 + tn * 32 + lrow;
                    const uint32_t mb = m0 + wm * WM + tm * 32 + 4 * lhalf;
                    const uint32_t base = (n < N && b < nblk) ? ((mb * N + n) * nblk + b) * 4 : OOB;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        int32_t v = isum[r];
                        if (MAGIC) {                 // what the biased accumulator holds, turned back into the block sum
                            v -= (int32_t)MAGIC_BITS;
                            if (kb & 1) v = -v;      // odd blocks ran on negated activation codes
                            if (Q4) v >>= 4;         // nibble codes were fed as 16 (c - 8)
                        }
                        __builtin_amdgcn_raw_buffer_store_b32((uint32_t)v, rdump, base + (8 * (r >> 2) + (r & 3)) * N * nblk * 4, 0, 0);
                    }
                }
                isum = isum_n;
                S = S_n;
                __builtin_amdgcn_sched_barrier(0);   // keep the tiles in this order: one tile of temporaries ahead, no more
            }
            if (kb == 0) { issue_stage((s + 1) * BK, buf ^ 1, 2); __builtin_amdgcn_sched_barrier(0); }
            if (kb == 1) { issue_stage((s + 1) * BK, buf ^ 1, 4); __builtin_amdgcn_sched_barrier(0); }
        }
        commit_stage(buf ^ 1, (s + 1) & 3, (s + 1) * KB);
        __builtin_amdgcn_s_waitcnt(0);   // this wave's share of stage s+1 has landed
        __syncthreads();
    };

    // Stages go in pairs (an odd count runs one stage of zero scales).  After a pair the fast mode removes what the 8
    // blocks left of the bias, 1.5 * 2^23 * sum_b a_s[m][b] * (+-w_s[n][b]).  That is sum_b (2^8 a_s[b]) * (2^15 w[b] +
    // 2^14 w[b]), sixteen products of fp16 numbers, so one f16 MFMA subtracts it from the accumulators directly: the
    // activation side holds 2^8 a_s[b] in both halves of the wave, the weight side -2^15 w[b] in the lanes of the lower
    // half (k = 0..7) and -2^14 w[b] in the upper half (k = 8..15).  (Before: the sum from the MFMA and one FMA per
    // element to apply it, 64 VALU instructions per wave and stage pair instead of 16 packed multiplies.)
    const uint32_t ta_off = LDS_ASC + (wm * WM + lrow) * SC_ROW;
    const uint32_t tb_off = LDS_BSC + (wn * 64 + lrow) * SC_ROW;
    for (uint32_t s = s_begin; s < s_end; s += 2) {
        run_stage(s, 0);
        run_stage(s + 1, 1);
        if (MAGIC) {
            const uint32_t pair = (s & 2u) * (uint32_t)SC_SLOT;      // slots {0,1} or {2,3}
            typedef _Float16 v4h __attribute__((ext_vector_type(4)));
            const _Float16 bf = lhalf ? (_Float16)(-(float)(1 << (22 - SCALE_A_LOG2))) : (_Float16)(-(float)(1 << (23 - SCALE_A_LOG2)));
            const _Float16 af = (_Float16)(float)(1 << SCALE_A_LOG2);
            const v8h bfv = (v8h){bf, bf, bf, bf, bf, bf, bf, bf}, afv = (v8h){af, af, af, af, af, af, af, af};
            v8h ta[TM], tb[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const v4h b0 = *reinterpret_cast<const v4h*>(lds + tb_off + pair + t * (32 * SC_ROW));
                const v4h b1 = *reinterpret_cast<const v4h*>(lds + tb_off + pair + SC_SLOT + t * (32 * SC_ROW));
                tb[t] = (v8h){b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]} * bfv;
            }
#pragma unroll
            for (int t = 0; t < TM; t++) {
                const v4h a0 = *reinterpret_cast<const v4h*>(lds + ta_off + pair + t * (32 * SC_ROW));
                const v4h a1 = *reinterpret_cast<const v4h*>(lds + ta_off + pair + SC_SLOT + t * (32 * SC_ROW));
                ta[t] = (v8h){a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]} * afv;
            }
#pragma unroll
            for (int t = 0; t < 2 * TM; t++) {
                const int tm = t >> 1, tn = t & 1;
                v16f c;
#pragma unroll
                for (int r = 0; r < 16; r++) c[r] = acc[tm][tn][r];
                c = __builtin_amdgcn_mfma_f32_32x32x16_f16(ta[tm], tb[tn], c, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) acc[tm][tn][r] = c[r];
            }
        }
    }

    if (SPLIT && ranged) {
        // Park this range's tile (thread-major: element e of thread t at [e][t], the same mapping in every workgroup).
        // Partial tiles cross between CUs whose L2 caches do not see each other's lines, so they travel as device-scope
        // (write-through / cache-bypassing) stores and loads rather than behind device-scope fences, which would write
        // back and invalidate a whole L2 per workgroup: the stores are waited for, then counted, and the workgroup that
        // counts last reads them all.
        constexpr uint32_t TILE_ELEMS = TM * 2 * 16 * 256;
        float* mine = sp.partials + ((size_t)range_tile * sp.split + s_begin / sp.stages_per_part) * TILE_ELEMS;
#pragma unroll
        for (int e = 0; e < TM * 2 * 16; e++)
            __hip_atomic_store(mine + e * 256 + tid, acc[e / 32][(e / 16) & 1][e & 15], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");   // for the compiler: the stores stay above this line
        __builtin_amdgcn_s_waitcnt(0);                           // vmcnt(0): they have been acknowledged
        __syncthreads();
        __shared__ uint32_t arrived;
        if (tid == 0) arrived = __hip_atomic_fetch_add(sp.counters + range_tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (arrived != sp.split - 1) return;      // whole workgroup: not the last range of this tile
        const float* all = sp.partials + (size_t)range_tile * sp.split * TILE_ELEMS;
        // ranges in K order, whoever arrived last; a whole range's loads in flight at a time
        for (uint32_t p = 0; p < sp.split; p++) {
            float part[TM * 2 * 16];
#pragma unroll
            for (int e = 0; e < TM * 2 * 16; e++)
                part[e] = __hip_atomic_load(all + (size_t)p * TILE_ELEMS + e * 256 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int e = 0; e < TM * 2 * 16; e++) {
                float& dst = acc[e / 32][(e / 16) & 1][e & 15];
                dst = p == 0 ? part[e] : dst + part[e];
            }
        }
        if (tid == 0) __hip_atomic_store(sp.counters + range_tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch (stream order)
    }

    if (MINT) {
        // On the f16 matrix unit, sixteen b per step: every operand arrives as a hi | lo pair of fp16 numbers in a 4-byte slot
        // (kquant_prefill.hip: hi = fp16(x), lo = fp16(x - hi), x scaled by a power of two that cancels between the sides) and the
        // three products hi*hi + hi*lo + lo*hi carry it to 2^-22 relative -- a sixteenth of the f32 MFMA's time, which for
        // K = 2048 was as long as the tile's whole int8 loop.
        // A: lane = (row lrow of the tile, b = 8 lhalf .. + 8 of each group of sixteen), B: lane = (column lrow, the same b).
        auto split = [](const float4& x0, const float4& x1, v8h& hi, v8h& lo) {
            const uint32_t p[8] = {__float_as_uint(x0.x), __float_as_uint(x0.y), __float_as_uint(x0.z), __float_as_uint(x0.w),
                                   __float_as_uint(x1.x), __float_as_uint(x1.y), __float_as_uint(x1.z), __float_as_uint(x1.w)};
            uint32_t h[4], l[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                h[i] = __builtin_amdgcn_perm(p[2 * i + 1], p[2 * i], 0x05040100u);      // the two low halves
                l[i] = __builtin_amdgcn_perm(p[2 * i + 1], p[2 * i], 0x07060302u);      // the two high halves
            }
            hi = __builtin_bit_cast(v8h, make_uint4(h[0], h[1], h[2], h[3]));
            lo = __builtin_bit_cast(v8h, make_uint4(l[0], l[1], l[2], l[3]));
        };
        // The operand rows (256 bytes per 64 blocks) come through LDS, which the main loop no longer needs: a lane that fetched its
        // own row from memory touched one cache line per lane and load, and the term cost as much as a third of the tile.
        // Chunks of 64 blocks; rows 272 bytes apart (a row's 32-byte fragments of neighbouring rows on different banks).
        constexpr uint32_t MT_ROW = 272, MT_B = 128 * MT_ROW;          // the B rows start behind 128 A rows
        static_assert(2 * 128 * 272 <= GEMM_LDS_BYTES, "the minimum term's operand rows fit the kernel's LDS");
        for (uint32_t b0 = 0; b0 < nblk; b0 += 64) {
            const uint32_t nb = min(64u, nblk - b0);                   // a multiple of 8
            __syncthreads();                                           // the previous chunk (or the main loop) is done with LDS
            // thread: 16-byte piece (tid % 16) of rows tid / 16, + 16, ...
            const uint32_t piece = tid & 15, r0 = tid >> 4;
            if (piece * 4 < nb) {
#pragma unroll
                for (uint32_t r = r0; r < 2 * WM; r += 16) {
                    const uint32_t mrow = min(m0 + r, M - 1);
                    *reinterpret_cast<float4*>(lds + r * MT_ROW + piece * 16) = *reinterpret_cast<const float4*>(sp.mt_a + (size_t)mrow * nblk + b0 + piece * 4);
                }
#pragma unroll
                for (uint32_t c = r0; c < 128; c += 16) {
                    const uint32_t cwn = c >> 6, ctn = (c >> 5) & 1, clr = c & 31;
                    const uint32_t nrow = SILU ? si0 + 32 * cwn + clr + ctn * s_inter : min(n0 + c, N - 1);
                    *reinterpret_cast<float4*>(lds + MT_B + c * MT_ROW + piece * 16) = *reinterpret_cast<const float4*>(sp.mt_w + (size_t)nrow * nblk + b0 + piece * 4);
                }
            }
            __syncthreads();
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int tn = 0; tn < 2; tn++) {
                    const uint8_t* ap = lds + (wm * WM + tm * 32 + lrow) * MT_ROW + lhalf * 32;
                    const uint8_t* bp = lds + MT_B + (wn * 64 + tn * 32 + lrow) * MT_ROW + lhalf * 32;
                    v16f c;
#pragma unroll
                    for (int r = 0; r < 16; r++) c[r] = acc[tm][tn][r];
                    for (uint32_t g = 0; g < nb; g += 16) {
                        // the upper half-wave of a last, half group reads the group's first half again and multiplies it by zeros
                        const bool in = g + 8 * lhalf < nb;
                        const uint32_t go = (in ? g : g - 8 * lhalf) * 4;
                        const float4 a0 = *reinterpret_cast<const float4*>(ap + go), a1 = *reinterpret_cast<const float4*>(ap + go + 16);
                        float4 b0v = *reinterpret_cast<const float4*>(bp + go), b1v = *reinterpret_cast<const float4*>(bp + go + 16);
                        if (!in) { b0v = make_float4(0.f, 0.f, 0.f, 0.f); b1v = b0v; }
                        v8h ah, al, bh, bl;
                        split(a0, a1, ah, al);
                        split(b0v, b1v, bh, bl);
                        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, c, 0, 0, 0);
                        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl, c, 0, 0, 0);
                        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh, c, 0, 0, 0);
                    }
#pragma unroll
                    for (int r = 0; r < 16; r++) acc[tm][tn][r] = c[r];
                }
        }
    }

    if (SILU) {
        // lane: inter index i0 + 32 wn + lrow, gate in the first column tile, up in the second; rows as below
        const uint32_t inter = sp.inter, blk = tile_x * 2 + wn;           // the quant block this wave's 32 indices are
        const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc((void*)sp.silu_q, 0, M * inter, RSRC_FLAGS);
        const __amdgpu_buffer_rsrc_t rsc = __builtin_amdgcn_make_buffer_rsrc((void*)sp.silu_sc, 0, M * (inter / 32) * 2, RSRC_FLAGS);
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float g = acc[tm][0][r], u = acc[tm][1][r];
                if (Q4) { g *= 0.0625f; u *= 0.0625f; }
                // fast mode: reciprocals instead of divisions (1 ulp), round-to-nearest-even instead of half-away (they part
                // on exact ties only); |o * inv| <= 127 up to rounding, so the conversion needs no clamp
                const float o = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
                const float amax = half_wave_max(fabsf(o));               // the 32 lanes that share lhalf: one block of one row
                const float scl = amax * (1.0f / 127.0f);                 // an all-zero block: scale 0 (see quantize_block_part)
                float inv = amax > 0.f ? 127.0f * __builtin_amdgcn_rcpf(amax) : 0.f;
                if (blk & 1u) inv = -inv;                                 // odd blocks negated for the GEMM that reads them
                const uint32_t code = (uint32_t)(int)__builtin_rintf(o * inv) & 0xFFu;
                const uint32_t pk = quad_broadcast<0>(code) | (quad_broadcast<1>(code) << 8) | (quad_broadcast<2>(code) << 16) |
                                    (quad_broadcast<3>(code) << 24);
                const uint32_t m = m0 + wm * WM + tm * 32 + 4 * lhalf + 8 * (r >> 2) + (r & 3);
                // rows >= M lie past the end of the descriptors and are dropped
                if ((lrow & 3u) == 0) __builtin_amdgcn_raw_buffer_store_b32(pk, rq, m * inter + blk * 32 + lrow, 0, 0);
                if (lrow == 0) __builtin_amdgcn_raw_buffer_store_b16((uint16_t)f32_to_f16_bits(scl), rsc, (m * (inter / 32) + blk) * 2, 0, 0);
            }
        return;
    }

    // epilogue: lane holds column n = lrow, rows 8g + 4*lhalf + (r&3); the descriptor drops rows >= M.
    // y += ...: all of a lane's old values are requested before the first is used (a load, its wait, the add and the
    // store per element would be 64 memory round trips one after the other: every wait also waits for the store before it)
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc((void*)y, 0, M * ldy * 4, RSRC_FLAGS);
    auto offset_of = [&](int tm, int tn, int r) {
        const uint32_t n = n0 + wn * 64 + tn * 32 + lrow;
        const uint32_t mb = m0 + wm * WM + tm * 32 + 4 * lhalf;
        const uint32_t base = n < N ? (mb * ldy + n) * 4 : OOB;
        return base + (8 * (r >> 2) + (r & 3)) * ldy * 4;
    };
    if (accumulate) {
        float old[TM][2][16];
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int tn = 0; tn < 2; tn++)
#pragma unroll
                for (int r = 0; r < 16; r++) old[tm][tn][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ry, offset_of(tm, tn, r), 0, 0));
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int tn = 0; tn < 2; tn++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float v = acc[tm][tn][r];
                    if (MAGIC && Q4) v *= 0.0625f;
                    acc[tm][tn][r] = old[tm][tn][r] + v;
                }
    } else if (MAGIC && Q4) {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int tn = 0; tn < 2; tn++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[tm][tn][r] *= 0.0625f;
    }
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
        for (int tn = 0; tn < 2; tn++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, acc[tm][tn][r]), ry, offset_of(tm, tn, r), 0, 0);
}

// The kernel addresses each matrix with 32-bit byte offsets below 2^31: larger problems are cut into
// row ranges of the activations and of the weights, one launch each.
size_t gemm_split_workspace_bytes() { return (size_t)GEMM_SPLIT_MAX_ITEMS * BM * BN * sizeof(float) + GEMM_SPLIT_MAX_ITEMS * sizeof(uint32_t); }

// Whether launch_gemm's fused SiLU epilogue covers a fused [gate; up] matrix of 2 * inter rows for M activation rows.
bool gemm_silu_supported(const QWeight& w, uint32_t inter, uint32_t M) {
    const uint64_t LIMIT = 0x7FFFFFFFull - 2 * BK;
    return w.N == 2 * (uint64_t)inter && inter % 64 == 0 && (uint64_t)M * std::max<uint64_t>(w.K, inter) <= LIMIT &&
           (uint64_t)w.N * std::max<uint64_t>(w.qs_row_bytes(), (uint64_t)(w.K / 32) * 2) <= LIMIT;
}

void launch_gemm(const QWeight& w, const int8_t* aq, const uint16_t* as, uint32_t M, float* y, uint32_t ldy,
                 bool accumulate, bool exact, int32_t* isums, hipStream_t s, void* split_ws, int8_t* silu_q, uint16_t* silu_sc,
                 const float* mt_a, const float* mt_w) {
    if (M == 0 || w.N == 0) return;
    const bool silu = silu_q != nullptr;      // caller: gemm_silu_supported, fast mode, no block-sum dump
    const int accf = accumulate ? 1 : 0;
    const bool q4 = w.wdtype == FORGE_HIP_Q4_0;
    const uint64_t LIMIT = 0x7FFFFFFFull - 2 * BK;
    const uint64_t nblk = w.K / 32;
    const uint64_t per_m = std::max<uint64_t>(w.K, (uint64_t)ldy * 4);
    const uint64_t per_n = std::max<uint64_t>(w.qs_row_bytes(), nblk * 2);
    // a whole dimension in one launch when it fits, else steps of whole tiles
    const uint64_t m_fit = LIMIT / per_m, n_fit = LIMIT / per_n;
    const uint32_t m_step = M <= m_fit ? M : (uint32_t)std::max<uint64_t>(BM, m_fit / BM * BM);
    const uint32_t n_step = w.N <= n_fit ? w.N : (uint32_t)std::max<uint64_t>(BN, n_fit / BN * BN);
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 256;
        return n > 0 ? n : 256;
    }();
#define FH_GEMM_LAUNCH_TM(Q4_, DUMP_, EXACT_, TM_)                                                                        \
    do {                                                                                                                \
        static const hipError_t lds_ok = hipFuncSetAttribute((const void*)gemm_q_kernel<Q4_, DUMP_, EXACT_, TM_>,      \
                                                             hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS_BYTES); \
        (void)lds_ok;                                                                                                   \
        dim3 grid((nc + BN - 1) / BN, (mc + 64 * TM_ - 1) / (64 * TM_));                                                \
        fh::launch(gemm_q_kernel<Q4_, DUMP_, EXACT_, TM_>, grid, 256, GEMM_LDS_BYTES, s, wq, wsc, aq_c, as_c, y_c, is_c, \
                   mc, nc, w.K, ldy, accf, GemmSplit{});                                                                \
    } while (0)
#define FH_GEMM_LAUNCH(Q4_, DUMP_, EXACT_)                         \
    do {                                                           \
        if (tm == 1) FH_GEMM_LAUNCH_TM(Q4_, DUMP_, EXACT_, 1);     \
        else FH_GEMM_LAUNCH_TM(Q4_, DUMP_, EXACT_, 2);             \
    } while (0)
    for (uint32_t mlo = 0; mlo < M; mlo += m_step)
        for (uint32_t nlo = 0; nlo < w.N; nlo += n_step) {
            const uint32_t mc = std::min(m_step, M - mlo), nc = std::min(n_step, w.N - nlo);
            const uint8_t* wq = w.qs + (size_t)nlo * w.qs_row_bytes();
            const uint16_t* wsc = w.scales + (size_t)nlo * nblk;
            const int8_t* aq_c = aq + (size_t)mlo * w.K;
            const uint16_t* as_c = as + (size_t)mlo * nblk;
            float* y_c = y + (size_t)mlo * ldy + nlo;
            // block sums of a sub-problem are laid out [mc][nc][nblk]: only whole problems are dumped
            int32_t* is_c = isums;
            // 64-row tiles when even those leave no CU with more than one workgroup: a workgroup's time per K stage
            // halves with its tile, and a larger tile would only leave more CUs idle
            const uint64_t tiles64 = (uint64_t)((nc + BN - 1) / BN) * ((mc + 63) / 64);
            const bool small_tiles = tiles64 <= (uint64_t)cus && mc > 64;
            int tm = small_tiles ? 1 : 2;
            // Fast mode with a workspace from the caller: tiles that fill the CUs a few times and a fraction have the tiles of
            // the fraction cut along K, so that they spread over all CUs; a problem with fewer tiles than half the CUs is
            // all fraction.  Which tile height then fills the CUs best is decided by a small cost model (microseconds per K
            // stage of a workgroup that has a CU to itself, measured: 1.3 for a 128-row tile, 1.1 for a 64-row one).
            GemmSplit fsp{};
            uint32_t items = 0;
            if (split_ws && !exact && !isums && mc == M && nc == w.N) {
                struct Plan { int tm; GemmSplit sp; uint32_t items; double cost; };
                const uint32_t stages = (w.K + BK - 1) / BK;
                auto plan = [&](int tm_) {
                    const uint32_t tile_rows = 64 * tm_, tiles = ((nc + BN - 1) / BN) * ((mc + tile_rows - 1) / tile_rows);
                    const double t_stage = tm_ == 1 ? 1.1 : 1.3;
                    Plan p{tm_, GemmSplit{}, 0, (double)((tiles + cus - 1) / cus) * stages * t_stage};   // items 0: not cut
                    const uint32_t rem = tiles % (uint32_t)cus;
                    const uint32_t split = rem ? std::min<uint32_t>({(uint32_t)cus / rem, 8u, stages / 2, GEMM_SPLIT_MAX_ITEMS / rem}) : 0;
                    if (tiles / (uint32_t)cus < 4 && split >= 2) {
                        GemmSplit sp{};
                        sp.stages_per_part = ((stages + split - 1) / split + 1) & ~1u;
                        sp.split = (stages + sp.stages_per_part - 1) / sp.stages_per_part;
                        sp.full_tiles = tiles - rem;
                        sp.partials = reinterpret_cast<float*>(split_ws);
                        sp.counters = reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(split_ws) + (size_t)GEMM_SPLIT_MAX_ITEMS * BM * BN * sizeof(float));
                        // parking, counting and adding partial tiles: 12 us (64-row tiles) to 18 us (128-row tiles) end to end
                        // when every workgroup does it at the same moment, 5 when whole tiles are still being worked beside it
                        const double cost = ((double)(sp.full_tiles / cus) * stages + sp.stages_per_part) * t_stage +
                                            (sp.full_tiles ? 5.0 : tm_ == 1 ? 12.0 : 18.0);
                        if (sp.split >= 2 && cost < p.cost) { p.sp = sp; p.items = sp.full_tiles + rem * sp.split; p.cost = cost; }
                    }
                    return p;
                };
                Plan best = plan(tm);
                if (tm == 1) { const Plan other = plan(2); if (other.cost < best.cost) best = other; }
                tm = best.tm;
                if (best.items) { fsp = best.sp; items = best.items; }
            }
            if (items || silu || mt_a) {
                // the fast kernel's variants: tiles cut along K, the SiLU epilogue, the extra f32 term
                if (silu) { fsp.silu_q = silu_q; fsp.silu_sc = silu_sc; fsp.inter = w.N / 2; }
                if (mt_a) { fsp.mt_a = mt_a + (size_t)mlo * nblk; fsp.mt_w = mt_w + (size_t)nlo * nblk; }
                const dim3 grid = items ? dim3(items) : dim3((nc + BN - 1) / BN, (mc + 64 * tm - 1) / (64 * tm));
                auto go = [&](auto q4_, auto tm_, auto split_, auto silu_, auto mint_) {
                    constexpr bool Q4_ = decltype(q4_)::value, SPLIT_ = decltype(split_)::value, SILU_ = decltype(silu_)::value,
                                   MINT_ = decltype(mint_)::value;
                    constexpr int TM_ = decltype(tm_)::value;
                    static const hipError_t lds_ok = hipFuncSetAttribute((const void*)gemm_q_kernel<Q4_, false, false, TM_, SPLIT_, SILU_, MINT_>,
                                                                         hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS_BYTES);
                    (void)lds_ok;
                    fh::launch(gemm_q_kernel<Q4_, false, false, TM_, SPLIT_, SILU_, MINT_>, grid, 256, GEMM_LDS_BYTES, s, wq, wsc, aq_c, as_c,
                               y_c, is_c, mc, nc, w.K, ldy, accf, fsp);
                };
                using T = std::true_type;
                using F = std::false_type;
                using One = std::integral_constant<int, 1>;
                using Two = std::integral_constant<int, 2>;
                auto by_tm = [&](auto q4_, auto split_, auto silu_, auto mint_) {
                    if (tm == 1) go(q4_, One{}, split_, silu_, mint_);
                    else go(q4_, Two{}, split_, silu_, mint_);
                };
                auto by_shape = [&](auto q4_, auto mint_) {
                    if (items && silu) by_tm(q4_, T{}, T{}, mint_);
                    else if (items) by_tm(q4_, T{}, F{}, mint_);
                    else if (silu) by_tm(q4_, F{}, T{}, mint_);
                    else by_tm(q4_, F{}, F{}, mint_);
                };
                if (mt_a) by_shape(F{}, T{});          // caller: a Q8_0-layout matrix
                else if (q4) by_shape(T{}, F{});
                else by_shape(F{}, F{});
                continue;
            }
            if (q4) {
                if (isums && exact) FH_GEMM_LAUNCH(true, true, true);
                else if (isums) FH_GEMM_LAUNCH(true, true, false);
                else if (exact) FH_GEMM_LAUNCH(true, false, true);
                else FH_GEMM_LAUNCH(true, false, false);
            } else {
                if (isums && exact) FH_GEMM_LAUNCH(false, true, true);
                else if (isums) FH_GEMM_LAUNCH(false, true, false);
                else if (exact) FH_GEMM_LAUNCH(false, false, true);
                else FH_GEMM_LAUNCH(false, false, false);
            }
        }
#undef FH_GEMM_LAUNCH
#undef FH_GEMM_LAUNCH_TM
}

}  // namespace fh
