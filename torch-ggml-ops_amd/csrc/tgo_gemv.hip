// Decode-regime forward kernels (a few activation rows per expert): HBM-bound.
//
// Same algebra as the MFMA kernel (q8_1 activations, int8 weight operand, fp32 block scales), laid out
// for bandwidth: a workgroup streams 16 consecutive weight rows (one contiguous run of packed bytes) into
// LDS with coalesced loads, each wave takes four of the rows, and the 64 lanes of a wave split a row's K
// dimension in 16-value units.  A lane keeps the q8_1 values and scales of its units for the task's activation
// rows (the code exists for 1, 2, 4 and 8 of them) in registers, forms exact integer dot products with
// v_dot4, scales them, and the wave reduces the per-lane partial sums with cross-lane shuffles at the end.
// Q4_K / Q5_K tasks of three or more rows use the matrix cores for the dot products instead (gemv_task_k45_mfma).
// With K of at most four super-blocks several weight rows share a pass (FOLD).  Dense calls of more rows than a
// task holds are walked in chunks by kernel instantiations of their own.
#include <algorithm>
#include <type_traits>

#include "tgo_device.h"
#include "tgo_launch.h"

namespace tgo {

constexpr int GEMV_ROWS = GEMV_ROW_TILE;   // activation rows per task
constexpr int GEMV_GN = 16;                // weight rows per workgroup
constexpr int GEMV_THREADS = 256;
constexpr int GEMV_WAVE_ROWS = GEMV_GN / (GEMV_THREADS / 64);
constexpr int GEMV_CHUNK = 8;              // super-blocks of K per pass: 128 units = 2 per lane
// LDS bytes per activation row of a pass in the matrix-core variant: 8 super-blocks of values plus 32, so that
// the rows start eight banks apart (the four lanes of a row read eight consecutive words)
constexpr int GEMV_X_PITCH = GEMV_CHUNK * QK_K + 32;
// floats per row of its block-scale and block-sum copies (64 per pass), and per super-block of its scale and
// min tables (two groups of 16 weight rows); both padded so that the lanes of one read spread over the banks
constexpr int GEMV_XD_PITCH = GEMV_CHUNK * 8 + 4;
constexpr int GEMV_K45_KB_SCALES = 2 * GEMV_GN + 8;

struct GemvArgs {
    const uint8_t * packed;
    const uint8_t * packed_second;   // second projection of a pair, or nullptr
    int64_t bytes_per_expert;
    int64_t row_bytes;
    const int8_t * qx;
    const float * dx;
    const float * sx;
    uint16_t * y;
    uint16_t * y_second;
    const int32_t * task_count;   // nullptr: dense, all rows (at most GEMV_DENSE_ROWS, taken GEMV_ROWS or 16 at a time)
    const int32_t * task_expert;
    const int32_t * task_row_start;
    const int32_t * task_row_end;
    int rows;
    int rows_padded;
    int in_features;
    int out_features;
    int n_groups;   // workgroups per task and projection: groups of GEMV_GN (long) weight rows
    int projections;   // 1, or 2 for a pair
    int unit_staging;  // 2-byte aligned formats: the tensors may be read in whole aligned 16-byte units (wide_stage_ok)
    // Fused calls (kernel instances with FUSED set): the activations arrive as bf16 and every workgroup quantizes the
    // rows of its task itself, so that a call is one launch; qx, dx, sx and the task arrays are not used.
    const uint16_t * x;              // [input_rows or rows, in_features] bf16
    const int64_t * gather;          // row r of the call is row gather[r] of x (absent when outside [0, input_rows)), or nullptr
    int64_t input_rows;
    const int64_t * expert_indices;  // grouped fused calls: the groups themselves (a workgroup finds its task in them)
    const int32_t * expert_offsets;
    int num_experts;
    int num_groups;
};

// LDS of a fused workgroup's activations: ROWS rows of a pass's int8 values, then ROWS x 64 block scales.
template <int ROWS>
constexpr int gemv_fused_x_bytes() {
    return ROWS * GEMV_CHUNK * QK_K + ROWS * GEMV_CHUNK * 8 * 4;
}

// LDS slot of super-block `kb` of a pass for weight row `row`.  Row-major, so that the lanes of a wave, which
// differ in kb, hit slots one RAW_PITCH (an odd number of words) apart and spread over the banks; with the
// super-blocks outermost the stride is 16 pitches, an even number of words, and the lanes' reads of one
// instruction pile up eight deep on a few banks.
TGO_DEVICE int gemv_slot(int kb, int row) { return row * GEMV_CHUNK + kb; }
// bytes per slot: the format's padded block, or the larger slot of the aligned-unit staging (gemv_stage_units)
template <int TYPE>
constexpr int gemv_slot_bytes() {
    return Format<TYPE>::BLOCK_BYTES % 16 == 0 || Format<TYPE>::RAW_PITCH > WideStage<TYPE>::PITCH ? Format<TYPE>::RAW_PITCH
                                                                                                  : WideStage<TYPE>::PITCH;
}
// The matrix-core variant's lanes differ in the weight row instead, and take the other order for the same reason
// (byte offset of the slot, given its pitch).  Sixteen slots are a multiple of 16 words, and the staging writes of
// consecutive lanes, 4 words apart within a block, would meet the same eight banks again in the next
// super-block: every super-block is therefore shifted one more word (GEMV_CHUNK words of slack at the end).
TGO_DEVICE int gemv_kb_major_offset(int kb, int row, int pitch) { return (kb * GEMV_GN + row) * pitch + kb * 4; }

TGO_DEVICE int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), c, false);
}

// Copies `chunk_blocks` super-block columns (starting at `kb0`) of the workgroup's 16 weight rows into
// their LDS slots.  All loads of a batch are issued before the first store, so a thread waits for memory
// once per batch instead of once per load.
template <int TYPE>
TGO_DEVICE void gemv_stage(uint8_t * raw, const uint8_t * weights, int64_t row_bytes, int n0, int row_limit,
                           int kb0, int chunk_blocks, int tid) {
    using F = Format<TYPE>;
    constexpr bool WIDE = F::BLOCK_BYTES % 16 == 0;
    constexpr int PIECE = WIDE ? 16 : 2;
    constexpr int UNITS = F::BLOCK_BYTES / PIECE;
    constexpr int BATCH = WIDE ? 6 : 12;
    typedef typename std::conditional<WIDE, uint4, uint16_t>::type piece_t;
    const int total = chunk_blocks * GEMV_GN * UNITS;
    for (int base = tid; base < total; base += GEMV_THREADS * BATCH) {
        piece_t value[BATCH];
        int slot[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int id = min(base + b * GEMV_THREADS, total - 1);
            const int unit = id % UNITS;
            const int row = (id / UNITS) % GEMV_GN;
            const int kb = id / (UNITS * GEMV_GN);
            int src_row = n0 + row;
            src_row = src_row < row_limit ? src_row : row_limit - 1;
            value[b] = *reinterpret_cast<const piece_t *>(
                weights + src_row * row_bytes + static_cast<int64_t>(kb0 + kb) * F::BLOCK_BYTES + unit * PIECE);
            slot[b] = gemv_slot(kb, row) * F::RAW_PITCH + (WIDE ? 0 : F::RAW_SHIFT) + unit * PIECE;
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            if (base + b * GEMV_THREADS < total) {
                if constexpr (WIDE) {
                    uint32_t * dst = reinterpret_cast<uint32_t *>(raw + slot[b]);
                    dst[0] = value[b].x; dst[1] = value[b].y; dst[2] = value[b].z; dst[3] = value[b].w;
                } else {
                    *reinterpret_cast<uint16_t *>(raw + slot[b]) = value[b];
                }
            }
        }
    }
}

// Staging for the formats whose blocks are only 2-byte aligned, when the rows themselves start on G-byte
// boundaries (G = 16 or 4: row_bytes is a multiple of G, and a pass starts a multiple of 8 blocks into the
// row).  Sixteen threads walk one weight row's bytes of the pass in G-byte pieces, so a pass is one batch of
// wide loads instead of several batches of 2-byte loads; each piece is then dealt out to the LDS slots of the
// one or two blocks it covers, two bytes at a time (the slots keep every block 4-byte aligned, which the
// global layout does not).
template <int TYPE, int G>
TGO_DEVICE void gemv_stage_pieces(uint8_t * raw, const uint8_t * weights, int64_t row_bytes, int n0, int row_limit,
                                  int kb0, int chunk_blocks, int tid) {
    using F = Format<TYPE>;
    constexpr int B = F::BLOCK_BYTES;
    constexpr int BATCH = G == 16 ? 4 : 8;
    constexpr int HALFWORDS = G / 2;
    typedef typename std::conditional<G == 16, uint4, uint32_t>::type piece_t;
    static_assert(GEMV_THREADS / 16 == GEMV_GN && G < B, "sixteen threads per weight row; a piece spans at most two blocks");
    const int row = tid >> 4;
    const int member = tid & 15;
    const int pieces = chunk_blocks * B / G;
    const int src_row = min(n0 + row, row_limit - 1);
    const uint8_t * src = weights + src_row * row_bytes + static_cast<int64_t>(kb0) * B;
    for (int first = member; first < pieces; first += 16 * BATCH) {
        piece_t value[BATCH];
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            value[b] = *reinterpret_cast<const piece_t *>(src + min(first + 16 * b, pieces - 1) * G);
        }
#pragma unroll
        for (int b = 0; b < BATCH; ++b) {
            const int piece = first + 16 * b;
            if (piece < pieces) {
                int block = piece * G / B;
                int within = piece * G - block * B;
                uint32_t words[G / 4];
                if constexpr (G == 16) {
                    words[0] = value[b].x; words[1] = value[b].y; words[2] = value[b].z; words[3] = value[b].w;
                } else {
                    words[0] = value[b];
                }
#pragma unroll
                for (int h = 0; h < HALFWORDS; ++h) {
                    if (within >= B) {
                        within -= B;
                        block += 1;
                    }
                    *reinterpret_cast<uint16_t *>(raw + gemv_slot(block, row) * F::RAW_PITCH + F::RAW_SHIFT + within) =
                        static_cast<uint16_t>(words[h >> 1] >> (16 * (h & 1)));
                    within += 2;
                }
            }
        }
    }
}

// The same pass as aligned 16-byte units (the 2-byte aligned formats, tensors that start and end on a unit boundary:
// wide_stage_ok): every (weight row, super-block) is covered by WideStage::UNITS aligned units, each loaded whole
// and written to the block's slot with four 4-byte stores, shifted by the block's misalignment on the way
// (v_alignbyte for the odd halfword, the store position for the rest), so that the block starts at
// WideStage::FRONT of its slot.  A third of the vector instructions of dealing out 2-byte pieces.  Slots are
// WideStage::PITCH bytes here.  `tile`: first byte of (long) weight row n0 (wave-uniform).
template <int TYPE>
struct GemvUnits {
    using W = WideStage<TYPE>;
    static constexpr int TOTAL = GEMV_GN * GEMV_CHUNK * W::UNITS;
    static constexpr int REGS = (TOTAL + GEMV_THREADS - 1) / GEMV_THREADS;
    static constexpr int RECIPROCAL = (65536 + W::UNITS - 1) / W::UNITS;   // id -> id / UNITS, exact below 3000
    static_assert(TOTAL < 3000, "range of the reciprocal");
};
template <int TYPE>
struct GemvUnitRegs {
    u32x4_t unit_value[GemvUnits<TYPE>::REGS];
    uint32_t next_value[GemvUnits<TYPE>::REGS];
    uint32_t place[GemvUnits<TYPE>::REGS];   // LDS byte offset of the unit's first word | halfword shift << 16
};
// (requests the units; gemv_units_park writes them to LDS, so that a caller can put work of its own between the two)
template <int TYPE>
TGO_DEVICE void gemv_units_fetch(GemvUnitRegs<TYPE> & regs, const uint8_t * tile, int64_t row_bytes, int rows_valid,
                                 int kb0, int chunk_blocks, int tid) {
    using U = GemvUnits<TYPE>;
    using W = WideStage<TYPE>;
    const uint32_t tile_m = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(tile)) & 15u;
    const uint8_t * const aligned = tile - tile_m;
#pragma unroll
    for (int i = 0; i < U::REGS; ++i) {
        // ids past the pass repeat its last unit: no lane branches around a load
        const int id = min(tid + GEMV_THREADS * i, U::TOTAL - 1);
        const int slot = static_cast<int>(__umul24(id, U::RECIPROCAL) >> 16);   // gemv_slot(kb, row) = row * GEMV_CHUNK + kb
        int unit = id - slot * W::UNITS;
        const int row = min(slot / GEMV_CHUNK, rows_valid - 1);
        const int kb = min(slot % GEMV_CHUNK, chunk_blocks - 1);
        // (a pass of 16 rows spans less than 2^31 bytes: the host checks row_bytes)
        const uint32_t first = tile_m + static_cast<uint32_t>(row) * static_cast<uint32_t>(row_bytes) +
                               static_cast<uint32_t>(kb0 + kb) * W::BLOCK;
        const int reach = static_cast<int>(first & 15u) + W::BLOCK;   // block end, from its first unit
        const bool carries = 16 * (unit + 1) < reach;                 // the following unit still holds bytes of the block
        const int source_unit = 16 * unit < reach ? unit : 0;         // (units past the block re-read its first one)
        const uint32_t offset = (first & ~15u) + 16u * source_unit;
        regs.unit_value[i] = *reinterpret_cast<const u32x4_t *>(aligned + offset);
        regs.next_value[i] = *reinterpret_cast<const uint32_t *>(aligned + offset + (carries ? 16u : 0u));
        const uint32_t m = first & 15u;
        // rows and super-blocks the pass does not have are parked in their own slots (never read)
        regs.place[i] = static_cast<uint32_t>(slot * W::PITCH + W::FRONT + 16 * unit) - (m & 12u) + ((m & 2u) << 16);
    }
}
template <int TYPE>
TGO_DEVICE void gemv_units_park(uint8_t * raw, const GemvUnitRegs<TYPE> & regs) {
#pragma unroll
    for (int i = 0; i < GemvUnits<TYPE>::REGS; ++i) {
        const uint32_t shift = regs.place[i] >> 16;
        const u32x4_t d = regs.unit_value[i];
        uint32_t * dst = reinterpret_cast<uint32_t *>(raw + (regs.place[i] & 0xffffu));
        dst[0] = __builtin_amdgcn_alignbyte(d.y, d.x, shift);
        dst[1] = __builtin_amdgcn_alignbyte(d.z, d.y, shift);
        dst[2] = __builtin_amdgcn_alignbyte(d.w, d.z, shift);
        dst[3] = __builtin_amdgcn_alignbyte(regs.next_value[i], d.w, shift);
    }
}
template <int TYPE>
TGO_DEVICE void gemv_stage_units(uint8_t * raw, const uint8_t * tile, int64_t row_bytes, int rows_valid, int kb0,
                                 int chunk_blocks, int tid) {
    GemvUnitRegs<TYPE> regs;
    gemv_units_fetch<TYPE>(regs, tile, row_bytes, rows_valid, kb0, chunk_blocks, tid);
    gemv_units_park<TYPE>(raw, regs);
}

// Register-staged copy for the formats whose blocks are whole 16-byte units: the loads of a pass are issued into
// registers one pass ahead (gemv_fetch) and written to LDS when their pass begins (gemv_park), so that the
// memory system keeps working while the workgroup computes.  Without this every workgroup of a launch alternates
// between waiting for memory and computing, in step with all the others, and the memory sits idle half the time.
// A thread's units run along a weight row (a pass of a row is one contiguous run of chunk_blocks blocks).
template <int TYPE>
struct GemvWide {
    using F = Format<TYPE>;
    static constexpr int UNITS = F::BLOCK_BYTES / 16;
    static constexpr int REGS = (GEMV_GN * GEMV_CHUNK * UNITS + GEMV_THREADS - 1) / GEMV_THREADS;
};

template <int TYPE>
TGO_DEVICE void gemv_fetch(uint4 (&regs)[GemvWide<TYPE>::REGS], const uint8_t * weights, int64_t row_bytes, int n0,
                           int row_limit, int kb0, int chunk_blocks, int tid) {
    using F = Format<TYPE>;
    constexpr int UNITS = GemvWide<TYPE>::UNITS;
    const int run = chunk_blocks * UNITS;       // 16-byte units of one row in this pass
    const int total = GEMV_GN * run;
#pragma unroll
    for (int i = 0; i < GemvWide<TYPE>::REGS; ++i) {
        const int id = min(tid + i * GEMV_THREADS, total - 1);
        const int row = id / run;
        const int unit = id - row * run;
        int src_row = n0 + row;
        src_row = src_row < row_limit ? src_row : row_limit - 1;
        regs[i] = *reinterpret_cast<const uint4 *>(
            weights + src_row * row_bytes + static_cast<int64_t>(kb0) * F::BLOCK_BYTES + unit * 16);
    }
}

template <int TYPE, bool KB_MAJOR = false>
TGO_DEVICE void gemv_park(uint8_t * raw, const uint4 (&regs)[GemvWide<TYPE>::REGS], int chunk_blocks, int tid) {
    using F = Format<TYPE>;
    constexpr int UNITS = GemvWide<TYPE>::UNITS;
    const int run = chunk_blocks * UNITS;
    const int total = GEMV_GN * run;
#pragma unroll
    for (int i = 0; i < GemvWide<TYPE>::REGS; ++i) {
        const int id = tid + i * GEMV_THREADS;
        if (id < total) {
            const int row = id / run;
            const int unit_in_row = id - row * run;
            const int kb = unit_in_row / UNITS;
            const int unit = unit_in_row - kb * UNITS;
            const int offset = KB_MAJOR ? gemv_kb_major_offset(kb, row, F::RAW_PITCH) : gemv_slot(kb, row) * F::RAW_PITCH;
            uint32_t * dst = reinterpret_cast<uint32_t *>(raw + offset + unit * 16);
            dst[0] = regs[i].x; dst[1] = regs[i].y; dst[2] = regs[i].z; dst[3] = regs[i].w;
        }
    }
}

// Sums COUNT values per lane over aligned groups of WIDTH lanes (powers of two, COUNT <= WIDTH).  Reducing every
// value with its own chain of shuffles costs COUNT * log2(WIDTH) of them; here each step first halves the number
// of values a lane is responsible for -- the lane keeps the half chosen by one bit of its number and hands the
// other half to the partner that keeps it -- so the steps cost COUNT/2, COUNT/4, ... 1, 1, ... shuffles.  A lane
// ends up with the total of value butterfly_index(lane); lanes that differ only in the bits below WIDTH / COUNT
// hold the same total.  The order of the additions is fixed.
template <int COUNT, int WIDTH>
TGO_DEVICE int butterfly_index(int lane) {
    int index = 0;
    int offset = WIDTH / 2;
#pragma unroll
    for (int count = COUNT; count > 1; count >>= 1, offset >>= 1) {
        index += (lane & offset) ? count / 2 : 0;
    }
    return index;
}

// (one step per template instance, so that every array index is a constant)
template <int COUNT, int OFFSET>
TGO_DEVICE float butterfly_step(const float (&v)[COUNT], int lane) {
    if constexpr (COUNT == 1) {
        float total = v[0];
#pragma unroll
        for (int rest = OFFSET; rest > 0; rest >>= 1) {
            total += __shfl_xor(total, rest);
        }
        return total;
    } else {
        constexpr int HALF = COUNT / 2;
        const bool upper = (lane & OFFSET) != 0;
        float next[HALF];
#pragma unroll
        for (int k = 0; k < HALF; ++k) {
            const float keep = upper ? v[k + HALF] : v[k];
            const float send = upper ? v[k] : v[k + HALF];
            next[k] = keep + __shfl_xor(send, OFFSET);
        }
        return butterfly_step<HALF, OFFSET / 2>(next, lane);
    }
}

template <int COUNT, int WIDTH>
TGO_DEVICE float butterfly_sum(const float (&v)[COUNT], int lane) {
    static_assert(COUNT >= 1 && COUNT <= WIDTH && (COUNT & (COUNT - 1)) == 0 && (WIDTH & (WIDTH - 1)) == 0, "powers of two");
    return butterfly_step<COUNT, WIDTH / 2>(v, lane);
}

// One 16-value unit of a Q3_K / Q6_K / IQ2_S block as four words of packed bytes: the weight behind byte b is
// (b - bias) * scale, with the integer sub-scale of the unit already inside `scale`.  Everything happens four
// values per 32-bit operation; the constant bias (32 for Q6_K's 6-bit values, 4 for Q3_K's 3-bit values) is
// taken out of the dot product afterwards with the sum of the unit's activations, which is shared by all
// weight rows.  IQ2_S carries signs: a nibble of sign bits is spread to one bit per byte with a multiply,
// widened to byte masks, and (m ^ mask) + bit negates the chosen bytes (the magnitudes are never 0).
template <int TYPE>
TGO_DEVICE void gemv_unit(const uint8_t * blk, int u, const uint2 * grid, uint32_t (&w)[4], float & scale, int & bias) {
    static_assert(TYPE == Q3_K || TYPE == Q6_K || TYPE == IQ2_S, "formats without a dedicated GEMV routine");
    if constexpr (TYPE == Q6_K) {
        const int chunk = u >> 3;
        const int rem = (16 * u) & 127;
        const uint8_t * ql = blk + chunk * 64 + (rem & 63);
        const uint8_t * qh = blk + 128 + chunk * 32 + ((16 * u) & 31);
        const int shift_l = 4 * (rem >> 6);
        const int shift_h = 2 * ((rem >> 5) & 3);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t low = lds_u32(ql + 4 * t) >> shift_l;
            const uint32_t high = lds_u32(qh + 4 * t) >> shift_h;
            w[t] = (low & 0x0f0f0f0fu) | ((high & 0x03030303u) << 4);
        }
        scale = half_bits_to_float(lds_u16(blk + 208)) * static_cast<float>(static_cast<int8_t>(blk[192 + u]));
        bias = 32;
    } else if constexpr (TYPE == Q3_K) {
        const int i0 = 16 * u;
        const uint8_t * qs = blk + 32 + (i0 >> 7) * 32 + (i0 & 31);
        const uint8_t * hm = blk + (i0 & 31);
        const int shift_l = 2 * ((i0 & 127) >> 5);
        const int shift_h = i0 >> 5;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t low = lds_u32(qs + 4 * t) >> shift_l;
            const uint32_t high = lds_u32(hm + 4 * t) >> shift_h;
            w[t] = (low & 0x03030303u) | ((high & 0x01010101u) << 2);
        }
        const uint8_t * scales = blk + 96;
        const int low = u < 8 ? scales[u] : scales[u - 8] >> 4;
        const int high = scales[8 + (u & 3)] >> (2 * (u >> 2));
        const int sub = ((low & 0x0f) | ((high & 3) << 4)) - 32;
        scale = half_bits_to_float(lds_u16(blk + 108)) * static_cast<float>(sub);
        bias = 4;
    } else {
        const uint8_t * qs = blk + 2;
        const uint32_t idx_pair = lds_u16(qs + 2 * u);
        const uint32_t sign_pair = lds_u16(qs + 32 + 2 * u);
        const uint32_t qh = blk[66 + (u >> 1)] >> (4 * (u & 1));
#pragma unroll
        for (int gsel = 0; gsel < 2; ++gsel) {
            const uint32_t index = ((idx_pair >> (8 * gsel)) & 0xffu) | (((qh >> (2 * gsel)) & 3u) << 8);
            const uint2 magnitudes = grid[index];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t nibble = (sign_pair >> (8 * gsel + 4 * h)) & 0xfu;
                const uint32_t bits = __umul24(nibble, 0x00204081u) & 0x01010101u;   // sign bit e -> bit 0 of byte e (a 24-bit multiply: full rate)
                const uint32_t mask = (bits << 8) - bits;                      // 0xff in the bytes to negate
                w[2 * gsel + h] = ((h == 0 ? magnitudes.x : magnitudes.y) ^ mask) + bits;
            }
        }
        const int sub = (blk[74 + (u >> 1)] >> (4 * (u & 1))) & 0x0f;
        scale = half_bits_to_float(lds_u16(blk)) * 0.125f * static_cast<float>(2 * sub + 1);
        bias = 0;
    }
}

// Everything after the task lookup, for a task of at most ROWS activation rows (ROWS is 1, 2, 4 or 8: the
// arithmetic per weight unit grows with it, and single-token decoding should not pay for eight rows).
//
// FOLD: with K of at most four (two) super-blocks a pass of eight would leave half (three quarters) of the lanes
// without a unit.  FOLD = 2 (4) consecutive weight rows are then treated as one "long row": they are contiguous in
// memory, so staging does not change at all, and the workgroup covers 16 * FOLD weight rows.  Only the lane's view
// differs: its unit belongs to weight row `sub` of the long row (FOLD 2: the slot; FOLD 4: slot and half of the
// wave), the activations repeat with the real K, and the partial sums are kept per slot and reduced over the lanes
// that share a weight row.  n0 counts long rows; out_features must be a multiple of FOLD.
//
// FUSED: the activations are bf16 in memory; before a pass's weights are staged every thread requests eight values of
// each of the task's rows, and while the weights travel it quantizes them (quantize_eight, the quantizer kernels'
// arithmetic, so the results are the same bit for bit) into x_lds, where the pass reads them after its barrier.
template <int TYPE, int ROWS, int FOLD, bool FUSED>
TGO_DEVICE void gemv_task(const GemvArgs & a, uint8_t * raw, uint8_t * x_lds, const uint2 * grid, const uint8_t * weights,
                          uint16_t * y, int n0, int row_start, int nrows, int tid) {
    using F = Format<TYPE>;
    static_assert(FOLD == 1 || FOLD == 2 || FOLD == 4, "long rows of one, two or four weight rows");
    constexpr int ACCS = FOLD > 1 ? 2 : 1;   // partial sums per slot when the slots belong to different weight rows
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int blocks_per_row = a.in_features / 32;
    const int super_blocks = a.in_features / QK_K;
    const int long_blocks = super_blocks * FOLD;            // super-blocks per long row (at most 8 when FOLD > 1)
    const int64_t long_row_bytes = a.row_bytes * FOLD;
    const int long_rows = a.out_features / FOLD;
    const int lane_kb = FOLD == 1 ? 0 : FOLD == 2 ? lane >> 4 : (lane >> 4) & 1;   // FOLD > 1: the lane's super-block
    // staging by aligned units (gemv_stage_units) when the expert's tensor starts and ends on a unit boundary
    const bool unit_staging = a.unit_staging != 0;
    const int slot_pitch = unit_staging ? WideStage<TYPE>::PITCH : F::RAW_PITCH;
    const int slot_front = unit_staging ? WideStage<TYPE>::FRONT : F::RAW_SHIFT;

    float acc[ACCS][GEMV_WAVE_ROWS][ROWS];
#pragma unroll
    for (int s = 0; s < ACCS; ++s)
#pragma unroll
        for (int i = 0; i < GEMV_WAVE_ROWS; ++i)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[s][i][r] = 0.0f;

    // q8_1 values and scales of a lane's 16-value unit `slot` of a pass for the task's activation rows.  Tasks
    // of one or two rows request both units before the pass's weights are staged, so that everything travels
    // together; with more rows the registers are needed elsewhere and a unit's activations are fetched when its
    // turn comes.
    constexpr bool EARLY = ROWS <= 2 && !FUSED;
    struct Activations {
        uint4 q[ROWS];
        float d[ROWS];
    };
    int8_t * const xq_lds = reinterpret_cast<int8_t *>(x_lds);
    float * const xd_lds = reinterpret_cast<float *>(x_lds + ROWS * GEMV_CHUNK * QK_K);
    auto load_activations = [&](int kb0, int slot, Activations & x) {
        const int unit_in_chunk = lane + 64 * slot;
        // lanes past the end repeat the last block
        const int kb = min(FOLD == 1 ? kb0 + (unit_in_chunk >> 4) : lane_kb, super_blocks - 1);
        const int unit = unit_in_chunk & 15;
        const int block = kb * 8 + (unit >> 1);      // 32-value activation block
        const int half = unit & 1;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            if constexpr (FUSED) {
                // (the pass's copy in LDS starts at super-block kb0; rows the task does not have were written as zeros)
                const int local = block - kb0 * 8;
                x.q[r] = *reinterpret_cast<const uint4 *>(xq_lds + r * GEMV_CHUNK * QK_K + local * 32 + half * 16);
                x.d[r] = xd_lds[r * GEMV_CHUNK * 8 + local];
            } else {
                const int row = row_start + (r < nrows ? r : nrows - 1);
                x.q[r] = *reinterpret_cast<const uint4 *>(
                    a.qx + static_cast<int64_t>(row) * a.in_features + block * 32 + half * 16);
                x.d[r] = a.dx[static_cast<int64_t>(row) * blocks_per_row + block];
            }
        }
    };
    // FUSED: where the task's rows are in x (nullptr: a gathered row that does not exist, quantized as zeros)
    const uint16_t * x_row[FUSED ? ROWS : 1];
    if constexpr (FUSED) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int row = row_start + (r < nrows ? r : nrows - 1);
            int64_t source = row;
            bool present = true;
            if (a.gather != nullptr) {
                source = a.gather[row];
                present = source >= 0 && source < a.input_rows;
            }
            x_row[r] = present ? a.x + source * a.in_features : nullptr;
        }
    }

    for (int kb0 = 0; kb0 < long_blocks; kb0 += GEMV_CHUNK) {
        const int chunk_blocks = min(GEMV_CHUNK, long_blocks - kb0);
        Activations early[EARLY ? 2 : 1];
        if constexpr (EARLY) {
            load_activations(kb0, 0, early[0]);
            load_activations(kb0, 1, early[1]);
        }
        // FUSED: this thread's eight values of the pass for every row (a pass covers the real K once, also for long
        // rows), requested ahead of the weights
        const int x_k = (FOLD == 1 ? kb0 * QK_K : 0) + tid * 8;
        const bool x_mine = tid * 8 < (FOLD == 1 ? chunk_blocks : super_blocks) * QK_K;   // (whole blocks of four lanes)
        uint4 x_bits[FUSED ? ROWS : 1];
        if constexpr (FUSED) {
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                x_bits[r] = make_uint4(0, 0, 0, 0);
                if (r < nrows && x_mine && x_row[r] != nullptr) {
                    x_bits[r] = *reinterpret_cast<const uint4 *>(x_row[r] + x_k);
                }
            }
        }
        __syncthreads();   // the previous pass is done with `raw` (and with the activations in LDS)
        const auto quantize_rows = [&]() __attribute__((always_inline)) {
            if (x_mine) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    // (rows past the task's last are all zeros: d = 0 and q = 0, no arithmetic needed)
                    uint32_t packed[2] = {0u, 0u};
                    float d = 0.0f;
                    if (r < nrows) {   // uniform
                        float x[8], total;
                        uint32_t halves[4];
                        int magnitude[8];
                        unpack_bf16x8(x_bits[r], x);
                        quantize_eight(x_bits[r], x, packed, d, total, halves, magnitude);
                    }
                    *reinterpret_cast<uint2 *>(xq_lds + r * GEMV_CHUNK * QK_K + tid * 8) = make_uint2(packed[0], packed[1]);
                    if ((tid & 3) == 0) {
                        xd_lds[r * GEMV_CHUNK * 8 + (tid >> 2)] = d;
                    }
                }
            }
        };
        if (unit_staging) {
            // (the activations were requested first and are quantized while the weights travel)
            GemvUnitRegs<TYPE> units;
            gemv_units_fetch<TYPE>(units, weights + static_cast<int64_t>(n0) * long_row_bytes, long_row_bytes,
                                   min(GEMV_GN, long_rows - n0), kb0, chunk_blocks, tid);
            if constexpr (FUSED) {
                quantize_rows();
            }
            gemv_units_park<TYPE>(raw, units);
        } else if ((long_row_bytes & 15) == 0) {
            gemv_stage_pieces<TYPE, 16>(raw, weights, long_row_bytes, n0, long_rows, kb0, chunk_blocks, tid);
        } else if ((long_row_bytes & 3) == 0) {
            gemv_stage_pieces<TYPE, 4>(raw, weights, long_row_bytes, n0, long_rows, kb0, chunk_blocks, tid);
        } else {
            gemv_stage<TYPE>(raw, weights, long_row_bytes, n0, long_rows, kb0, chunk_blocks, tid);
        }
        if constexpr (FUSED) {
            if (!unit_staging) {
                quantize_rows();
            }
        }
        __syncthreads();

#pragma unroll
        for (int slot = 0; slot < 2; ++slot) {
            const int unit_in_chunk = lane + 64 * slot;          // 16-value unit inside this pass
            int kb;                                              // super-block of the long row
            if constexpr (FOLD == 1) {
                if (unit_in_chunk >= chunk_blocks * 16) {
                    continue;
                }
                kb = unit_in_chunk >> 4;
            } else {
                if (lane_kb >= super_blocks) {
                    continue;
                }
                const int sub = FOLD == 2 ? slot : 2 * slot + (lane >> 5);
                kb = sub * super_blocks + lane_kb;
            }
            const int unit = unit_in_chunk & 15;
            Activations late;
            if constexpr (!EARLY) {
                load_activations(kb0, slot, late);
            }
            const Activations & x = EARLY ? early[slot] : late;
            const uint4 (&xq)[ROWS] = x.q;
            const float (&dxv)[ROWS] = x.d;
            int xsum[ROWS];   // sum of the unit's sixteen activation values
            if constexpr (TYPE != IQ2_S) {
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    xsum[r] = dot4(0x01010101u, xq[r].x, 0);
                    xsum[r] = dot4(0x01010101u, xq[r].y, xsum[r]);
                    xsum[r] = dot4(0x01010101u, xq[r].z, xsum[r]);
                    xsum[r] = dot4(0x01010101u, xq[r].w, xsum[r]);
                }
            }
#pragma unroll
            for (int i = 0; i < GEMV_WAVE_ROWS; ++i) {
                const int n_local = wave * GEMV_WAVE_ROWS + i;
                const uint8_t * blk = raw + gemv_slot(kb, n_local) * slot_pitch + slot_front;
                uint32_t w[4];
                float scale;
                int bias;
                gemv_unit<TYPE>(blk, unit, grid, w, scale, bias);
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    int dot = dot4(w[0], xq[r].x, 0);
                    dot = dot4(w[1], xq[r].y, dot);
                    dot = dot4(w[2], xq[r].z, dot);
                    dot = dot4(w[3], xq[r].w, dot);
                    if constexpr (TYPE != IQ2_S) {
                        dot -= bias * xsum[r];
                    }
                    float & sum = acc[FOLD > 1 ? slot : 0][i][r];
                    sum = fmaf(scale * dxv[r], static_cast<float>(dot), sum);
                }
            }
        }
    }

    // reduction of the per-lane partial sums over the lanes that share a weight row (the wave, or half of it for
    // FOLD 4): all 4 * ROWS sums of a slot at once, after which the first lane of every run of equal totals writes
    // the (weight row, activation row) its total belongs to
    constexpr int WIDTH = FOLD == 4 ? 32 : 64;
    constexpr int COUNT = GEMV_WAVE_ROWS * ROWS;
    const int index = butterfly_index<COUNT, WIDTH>(lane);
    const int i = index / ROWS, r = index % ROWS;
#pragma unroll
    for (int s = 0; s < ACCS; ++s) {
        float sums[COUNT];
#pragma unroll
        for (int k = 0; k < COUNT; ++k) {
            sums[k] = acc[s][k / ROWS][k % ROWS];
        }
        const float total = butterfly_sum<COUNT, WIDTH>(sums, lane);
        const int sub = FOLD == 1 ? 0 : FOLD == 2 ? s : 2 * s + (lane >> 5);
        const int n = (n0 + wave * GEMV_WAVE_ROWS + i) * FOLD + sub;
        if ((lane & (WIDTH / COUNT - 1)) == 0 && r < nrows && n < a.out_features) {
            y[static_cast<int64_t>(row_start + r) * a.out_features + n] = to_bf16_bits(total);
        }
    }
}

// Q4_K / Q5_K variant of gemv_task.  A lane takes whole 32-value blocks, so a block's scale and min are
// derived once per 32 weights instead of once per 16 and the quants are handled four per 32-bit operation
// straight from the packed words.  Two lane layouts:
//   PAIRS (tasks of one or two activation rows, where unpacking dominates): lane = (row half, super-block,
//     group pair); it reads the 32 bytes that hold the two groups' nibbles once and splits them with one
//     shift and two masks per word, derives both groups' 6-bit scales with 16-bit-wide masks, and does this
//     for two of the wave's four weight rows.  The activations of the next pass are requested a pass ahead.
//   otherwise: lane = (super-block, group), one block for each of the wave's four weight rows.
// (Fetching the blocks straight from global memory instead of staging them in LDS was tried and is slower.)
template <int TYPE, int ROWS, int FOLD>
TGO_DEVICE void gemv_task_k45(const GemvArgs & a, uint8_t * raw, const uint8_t * weights, uint16_t * y, int n0,
                              int row_start, int nrows, int tid) {
    using F = Format<TYPE>;
    static_assert(TYPE == Q4_K || TYPE == Q5_K, "K-quants with 32-value groups and a min term");
    constexpr int QS = TYPE == Q4_K ? 16 : 48;
    constexpr bool PAIRS = ROWS <= 2;
    static_assert(FOLD == 1 || (PAIRS && (FOLD == 2 || FOLD == 4)), "long rows exist in the two-group layout only");
    constexpr int LANE_BLOCKS = PAIRS ? 2 : 1;                       // consecutive blocks of K per lane
    constexpr int LANE_ROWS = PAIRS ? GEMV_WAVE_ROWS / 2 : GEMV_WAVE_ROWS;   // weight rows per lane
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int blocks_per_row = a.in_features / 32;
    const int super_blocks = a.in_features / QK_K;
    // FOLD > 1 (short K, see gemv_task): the upper bits of the lane's super-block number select one of the FOLD
    // weight rows of a long row instead
    const int lane_kb = PAIRS ? (lane >> 2) & 7 : lane >> 3;
    const int kb = FOLD == 1 ? lane_kb : FOLD == 2 ? lane_kb & 3 : lane_kb & 1;     // super-block inside the pass
    const int sub = FOLD == 1 ? 0 : FOLD == 2 ? lane_kb >> 2 : lane_kb >> 1;         // weight row of the long row
    const int long_blocks = super_blocks * FOLD;
    const int64_t long_row_bytes = a.row_bytes * FOLD;
    const int long_rows = a.out_features / FOLD;
    const int slot_kb = sub * super_blocks + kb;
    const int group = PAIRS ? 2 * (lane & 3) : lane & 7;    // (first) 32-value group inside it
    const int row_half = PAIRS ? lane >> 5 : 0;

    float acc[LANE_ROWS][ROWS];
#pragma unroll
    for (int i = 0; i < LANE_ROWS; ++i)
#pragma unroll
        for (int r = 0; r < ROWS; ++r) acc[i][r] = 0.0f;

    // Where a thread's units of a whole pass come from and go to does not change from pass to pass, so both
    // offsets are worked out once; only a last, shorter pass takes the general route.
    constexpr int REGS = GemvWide<TYPE>::REGS;
    constexpr int RUN = GEMV_CHUNK * GemvWide<TYPE>::UNITS;
    int64_t unit_source[REGS];
    int unit_slot[REGS];
#pragma unroll
    for (int i = 0; i < REGS; ++i) {
        const int id = min(tid + i * GEMV_THREADS, GEMV_GN * RUN - 1);
        const int row = id / RUN;
        const int unit_in_row = id - row * RUN;
        const int unit_kb = unit_in_row / GemvWide<TYPE>::UNITS;
        const int unit = unit_in_row - unit_kb * GemvWide<TYPE>::UNITS;
        const int src_row = min(n0 + row, long_rows - 1);
        unit_source[i] = src_row * long_row_bytes + unit_in_row * 16;
        unit_slot[i] = gemv_slot(unit_kb, row) * F::RAW_PITCH + unit * 16;
    }
    uint4 staged[REGS];
    auto fetch = [&](int first_block) {
        const int blocks = min(GEMV_CHUNK, long_blocks - first_block);
        if (blocks == GEMV_CHUNK) {
            const uint8_t * origin = weights + static_cast<int64_t>(first_block) * F::BLOCK_BYTES;
#pragma unroll
            for (int i = 0; i < REGS; ++i) {
                staged[i] = *reinterpret_cast<const uint4 *>(origin + unit_source[i]);
            }
        } else {
            gemv_fetch<TYPE>(staged, weights, long_row_bytes, n0, long_rows, first_block, blocks, tid);
        }
    };

    // q8_1 values, scale and sum of this lane's block(s) for the task's activation rows
    struct Activations {
        uint4 q[ROWS][LANE_BLOCKS][2];
        float d[ROWS][LANE_BLOCKS], sum[ROWS][LANE_BLOCKS];
    };
    auto load_activations = [&](int first_block, Activations & x) {
        // lanes past the end of K repeat the last super-block (their results are not used)
        const int block = min(first_block + kb, super_blocks - 1) * 8 + group;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int row = row_start + (r < nrows ? r : nrows - 1);
#pragma unroll
            for (int j = 0; j < LANE_BLOCKS; ++j) {
                const int8_t * values = a.qx + static_cast<int64_t>(row) * a.in_features + (block + j) * 32;
                x.q[r][j][0] = *reinterpret_cast<const uint4 *>(values);
                x.q[r][j][1] = *reinterpret_cast<const uint4 *>(values + 16);
                x.d[r][j] = a.dx[static_cast<int64_t>(row) * blocks_per_row + block + j];
                x.sum[r][j] = a.sx[static_cast<int64_t>(row) * blocks_per_row + block + j];
            }
        }
    };
    auto dot32 = [&](const uint32_t (&q)[8], const uint4 (&x)[2]) {
        int dot = dot4(q[0], x[0].x, 0);
        dot = dot4(q[1], x[0].y, dot);
        dot = dot4(q[2], x[0].z, dot);
        dot = dot4(q[3], x[0].w, dot);
        dot = dot4(q[4], x[1].x, dot);
        dot = dot4(q[5], x[1].y, dot);
        dot = dot4(q[6], x[1].z, dot);
        return dot4(q[7], x[1].w, dot);
    };

    fetch(0);
    Activations ahead;
    if constexpr (PAIRS) {
        load_activations(0, ahead);
    }
    for (int kb0 = 0; kb0 < long_blocks; kb0 += GEMV_CHUNK) {
        const int chunk_blocks = min(GEMV_CHUNK, long_blocks - kb0);
        __syncthreads();   // the previous pass is done with `raw`
        if (chunk_blocks == GEMV_CHUNK) {
#pragma unroll
            for (int i = 0; i < REGS; ++i) {
                if (tid + i * GEMV_THREADS < GEMV_GN * RUN) {
                    uint32_t * dst = reinterpret_cast<uint32_t *>(raw + unit_slot[i]);
                    dst[0] = staged[i].x; dst[1] = staged[i].y; dst[2] = staged[i].z; dst[3] = staged[i].w;
                }
            }
        } else {
            gemv_park<TYPE>(raw, staged, chunk_blocks, tid);
        }
        const bool more = kb0 + GEMV_CHUNK < long_blocks;
        if (more) {   // the next pass travels while this one is computed
            fetch(kb0 + GEMV_CHUNK);
        }
        Activations x;
        if constexpr (PAIRS) {
            x = ahead;
            if (more) {
                load_activations(kb0 + GEMV_CHUNK, ahead);
            }
        } else {
            // requested before the barrier so that they travel while the staged weights settle
            load_activations(kb0, x);
        }
        __syncthreads();
        if (FOLD == 1 ? kb < chunk_blocks : kb < super_blocks) {
#pragma unroll
            for (int i = 0; i < LANE_ROWS; ++i) {
                const int n_local = wave * GEMV_WAVE_ROWS + (PAIRS ? 2 * i + row_half : i);
                const uint8_t * blk = raw + gemv_slot(slot_kb, n_local) * F::RAW_PITCH;
                const uint32_t d_dmin = lds_u32(blk);
                const float d = half_bits_to_float(d_dmin & 0xffffu), dmin = half_bits_to_float(d_dmin >> 16);
                if constexpr (PAIRS) {
                    // 6-bit scales and mins of groups `group` and `group + 1`, two bytes at a time
                    const int shift = 8 * (group & 3);
                    const uint32_t low = lds_u32(blk + 4) >> shift, mid = lds_u32(blk + 8) >> shift,
                                   high = lds_u32(blk + 12) >> shift;
                    const uint32_t sc = group < 4 ? (low & 0x3f3fu) : ((high & 0x0f0fu) | ((low >> 2) & 0x3030u));
                    const uint32_t mn =
                        group < 4 ? (mid & 0x3f3fu) : (((high >> 4) & 0x0f0fu) | ((mid >> 2) & 0x3030u));
                    const float scale[2] = {d * static_cast<float>(sc & 0xffu), d * static_cast<float>((sc >> 8) & 0xffu)};
                    const float minimum[2] = {dmin * static_cast<float>(mn & 0xffu),
                                              dmin * static_cast<float>((mn >> 8) & 0xffu)};
                    // both nibbles of the 32 bytes that hold the two groups
                    const uint8_t * qs = blk + QS + (group >> 1) * 32;
                    uint32_t q[2][8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const uint32_t word = lds_u32(qs + 4 * t);
                        q[0][t] = word & 0x0f0f0f0fu;
                        q[1][t] = (word >> 4) & 0x0f0f0f0fu;
                        if constexpr (TYPE == Q5_K) {
                            const uint32_t bits = lds_u32(blk + 16 + 4 * t) >> group;
                            q[0][t] |= (bits & 0x01010101u) << 4;
                            q[1][t] |= ((bits >> 1) & 0x01010101u) << 4;
                        }
                    }
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) {
#pragma unroll
                        for (int j = 0; j < 2; ++j) {
                            const int dot = dot32(q[j], x.q[r][j]);
                            acc[i][r] = fmaf(scale[j] * x.d[r][j], static_cast<float>(dot), acc[i][r]);
                            acc[i][r] = fmaf(-minimum[j], x.sum[r][j], acc[i][r]);
                        }
                    }
                } else {
                    // 6-bit scale and min of the group from the 12 packed bytes after d and dmin
                    const int shift = 8 * (group & 3);
                    const uint32_t b0 = (lds_u32(blk + 4) >> shift) & 0xffu, b1 = (lds_u32(blk + 8) >> shift) & 0xffu,
                                   b2 = (lds_u32(blk + 12) >> shift) & 0xffu;
                    const uint32_t sc = group < 4 ? (b0 & 63u) : ((b2 & 15u) | ((b0 >> 6) << 4));
                    const uint32_t mn = group < 4 ? (b1 & 63u) : ((b2 >> 4) | ((b1 >> 6) << 4));
                    const float scale = d * static_cast<float>(sc);
                    const float minimum = dmin * static_cast<float>(mn);
                    // the group's 32 quants: one nibble of 32 consecutive bytes (plus one bit plane of qh for Q5_K)
                    const uint8_t * qs = blk + QS + (group >> 1) * 32;
                    const int nibble = 4 * (group & 1);
                    uint32_t q[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        q[t] = (lds_u32(qs + 4 * t) >> nibble) & 0x0f0f0f0fu;
                        if constexpr (TYPE == Q5_K) {
                            q[t] |= ((lds_u32(blk + 16 + 4 * t) >> group) & 0x01010101u) << 4;
                        }
                    }
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) {
                        const int dot = dot32(q, x.q[r][0]);
                        acc[i][r] = fmaf(scale * x.d[r][0], static_cast<float>(dot), acc[i][r]);
                        acc[i][r] = fmaf(-minimum, x.sum[r][0], acc[i][r]);
                    }
                }
            }
        }
    }

    // Reduction of the per-lane partial sums over the lanes that share a weight row (all 64, or one half of the
    // wave for PAIRS, or the 16 / 8 lanes of one weight row of a long row), then lane r of that set writes
    // activation row r.
    constexpr int SHARE = !PAIRS ? 64 : 32 / FOLD;
#pragma unroll
    for (int i = 0; i < LANE_ROWS; ++i) {
        const int n = (n0 + wave * GEMV_WAVE_ROWS + (PAIRS ? 2 * i + row_half : i)) * FOLD + sub;
        const int member = lane & (SHARE - 1);
        float mine = 0.0f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            float value = acc[i][r];
#pragma unroll
            for (int offset = SHARE / 2; offset > 0; offset >>= 1) {
                value += __shfl_xor(value, offset);
            }
            if (member == r) {
                mine = value;
            }
        }
        if (member < nrows && n < a.out_features) {
            y[static_cast<int64_t>(row_start + member) * a.out_features + n] = to_bf16_bits(mine);
        }
    }
}

// Single-row tasks of Q4_K / Q5_K without LDS: a lane fetches the header and the 32 (+32) bytes of its two
// groups straight from global memory, one pass ahead, for two of the wave's four weight rows.  Same lane layout
// and arithmetic as the two-group variant above; no staging, no barrier, the four waves run independently.  The
// four lanes of a super-block fetch its header separately (the line is in the vector cache after the first).
template <int TYPE, int FOLD>
TGO_DEVICE void gemv_task_k45_direct(const GemvArgs & a, const uint8_t * weights, uint16_t * y, int n0,
                                     int row_start, int tid) {
    using F = Format<TYPE>;
    static_assert(TYPE == Q4_K || TYPE == Q5_K, "K-quants with 32-value groups and a min term");
    constexpr int QS = TYPE == Q4_K ? 16 : 48;
    constexpr int PLANE_REGS = TYPE == Q5_K ? 2 : 0;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int blocks_per_row = a.in_features / 32;
    const int super_blocks = a.in_features / QK_K;
    // (FOLD > 1, short K: the upper bits of the super-block number select the weight row of a long row, see
    // gemv_task; n0 counts long rows)
    const int lane_kb = (lane >> 2) & 7;
    const int kb = FOLD == 1 ? lane_kb : FOLD == 2 ? lane_kb & 3 : lane_kb & 1;      // super-block inside the pass
    const int sub = FOLD == 1 ? 0 : FOLD == 2 ? lane_kb >> 2 : lane_kb >> 1;
    const int pair = lane & 3;           // groups 2 * pair and 2 * pair + 1
    const int group = 2 * pair;
    const int row_half = lane >> 5;

    struct Packed {
        uint4 header, quants[2], planes[PLANE_REGS > 0 ? PLANE_REGS : 1];
    };
    struct Activations {
        uint4 q[2][2];
        float d[2], sum[2];
    };
    // byte offsets of this lane's two weight rows (rows past the end repeat the last one; never stored)
    uint32_t row_offset[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int n = min((n0 + wave * GEMV_WAVE_ROWS + 2 * i + row_half) * FOLD + sub, a.out_features - 1);
        row_offset[i] = static_cast<uint32_t>(n - n0 * FOLD) * static_cast<uint32_t>(a.row_bytes);
    }
    const uint8_t * const tile = weights + static_cast<int64_t>(n0) * FOLD * a.row_bytes;
    auto fetch = [&](int first_block, Packed (&w)[2], Activations & x) {
        const int block_kb = min(first_block + kb, super_blocks - 1);   // lanes past the end repeat the last block
        const uint8_t * base = tile + static_cast<int64_t>(block_kb) * F::BLOCK_BYTES;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint8_t * blk = base + row_offset[i];
            w[i].header = *reinterpret_cast<const uint4 *>(blk);
            w[i].quants[0] = *reinterpret_cast<const uint4 *>(blk + QS + pair * 32);
            w[i].quants[1] = *reinterpret_cast<const uint4 *>(blk + QS + pair * 32 + 16);
            if constexpr (TYPE == Q5_K) {
                w[i].planes[0] = *reinterpret_cast<const uint4 *>(blk + 16);
                w[i].planes[1] = *reinterpret_cast<const uint4 *>(blk + 32);
            }
        }
        const int block = block_kb * 8 + group;
        const int8_t * values = a.qx + static_cast<int64_t>(row_start) * a.in_features + block * 32;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            x.q[j][0] = *reinterpret_cast<const uint4 *>(values + 32 * j);
            x.q[j][1] = *reinterpret_cast<const uint4 *>(values + 32 * j + 16);
            x.d[j] = a.dx[static_cast<int64_t>(row_start) * blocks_per_row + block + j];
            x.sum[j] = a.sx[static_cast<int64_t>(row_start) * blocks_per_row + block + j];
        }
    };

    float acc[2] = {0.0f, 0.0f};
    Packed ahead[2];
    Activations x_ahead;
    fetch(0, ahead, x_ahead);
    for (int kb0 = 0; kb0 < super_blocks; kb0 += GEMV_CHUNK) {
        Packed w[2] = {ahead[0], ahead[1]};
        const Activations x = x_ahead;
        if (kb0 + GEMV_CHUNK < super_blocks) {
            fetch(kb0 + GEMV_CHUNK, ahead, x_ahead);
        }
        if (kb0 + kb < super_blocks) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint32_t d_dmin = w[i].header.x;
                const float d = half_bits_to_float(d_dmin & 0xffffu), dmin = half_bits_to_float(d_dmin >> 16);
                const int shift = 8 * (group & 3);
                const uint32_t low = w[i].header.y >> shift, mid = w[i].header.z >> shift, high = w[i].header.w >> shift;
                const uint32_t sc = group < 4 ? (low & 0x3f3fu) : ((high & 0x0f0fu) | ((low >> 2) & 0x3030u));
                const uint32_t mn = group < 4 ? (mid & 0x3f3fu) : (((high >> 4) & 0x0f0fu) | ((mid >> 2) & 0x3030u));
                const float scale[2] = {d * static_cast<float>(sc & 0xffu), d * static_cast<float>((sc >> 8) & 0xffu)};
                const float minimum[2] = {dmin * static_cast<float>(mn & 0xffu), dmin * static_cast<float>((mn >> 8) & 0xffu)};
                const uint32_t words[8] = {w[i].quants[0].x, w[i].quants[0].y, w[i].quants[0].z, w[i].quants[0].w,
                                           w[i].quants[1].x, w[i].quants[1].y, w[i].quants[1].z, w[i].quants[1].w};
                uint32_t q[2][8];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    q[0][t] = words[t] & 0x0f0f0f0fu;
                    q[1][t] = (words[t] >> 4) & 0x0f0f0f0fu;
                    if constexpr (TYPE == Q5_K) {
                        const uint4 & plane = w[i].planes[t >> 2];
                        const uint32_t bits = (t % 4 == 0 ? plane.x : t % 4 == 1 ? plane.y : t % 4 == 2 ? plane.z : plane.w) >> group;
                        q[0][t] |= (bits & 0x01010101u) << 4;
                        q[1][t] |= ((bits >> 1) & 0x01010101u) << 4;
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    int dot = dot4(q[j][0], x.q[j][0].x, 0);
                    dot = dot4(q[j][1], x.q[j][0].y, dot);
                    dot = dot4(q[j][2], x.q[j][0].z, dot);
                    dot = dot4(q[j][3], x.q[j][0].w, dot);
                    dot = dot4(q[j][4], x.q[j][1].x, dot);
                    dot = dot4(q[j][5], x.q[j][1].y, dot);
                    dot = dot4(q[j][6], x.q[j][1].z, dot);
                    dot = dot4(q[j][7], x.q[j][1].w, dot);
                    acc[i] = fmaf(scale[j] * x.d[j], static_cast<float>(dot), acc[i]);
                    acc[i] = fmaf(-minimum[j], x.sum[j], acc[i]);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int n = (n0 + wave * GEMV_WAVE_ROWS + 2 * i + row_half) * FOLD + sub;
        float value = acc[i];
#pragma unroll
        for (int offset = 16 / FOLD; offset > 0; offset >>= 1) {
            value += __shfl_xor(value, offset);
        }
        if ((lane & (32 / FOLD - 1)) == 0 && n < a.out_features) {
            y[static_cast<int64_t>(row_start) * a.out_features + n] = to_bf16_bits(value);
        }
    }
}

// Q4_K / Q5_K tasks of three to sixteen activation rows: the per-row arithmetic of the routines above (a dozen
// vector instructions per 32-value block and activation row) would outgrow the memory time, so the integer dot
// products go to the matrix cores.  One v_mfma_i32_16x16x32_i8 multiplies a 32-value group of the workgroup's 16
// weight rows (A: lane = (weight row, 8 consecutive values)) with the same group of up to 16 activation rows
// (B: lane = (activation row, the same 8 values); rows the task does not have are zero), and leaves four weight
// rows of one activation row in each lane, which takes three vector instructions per result to scale and
// accumulate -- whatever the number of activation rows.  Wave w owns groups 2w and 2w + 1 of every super-block
// (the two nibbles of the same 32 bytes), so the four waves share every pass evenly for any K.  The min term
// sum_g min[n][g] * sum[m][g] is itself a small matrix product and runs as v_mfma_f32_16x16x4_f32 over four
// groups at a time.  The per-wave partial results meet in LDS at the end and are summed in wave order.
template <int TYPE, int XROWS>
TGO_DEVICE void gemv_task_k45_mfma(const GemvArgs & a, uint8_t * raw, float * scale_lds, uint8_t * x_lds,
                                   const uint8_t * weights, uint16_t * y, int n0, int row_start, int nrows, int tid) {
    using F = Format<TYPE>;
    static_assert(TYPE == Q4_K || TYPE == Q5_K, "K-quants with 32-value groups and a min term");
    typedef int v4i __attribute__((ext_vector_type(4)));
    typedef float v4f __attribute__((ext_vector_type(4)));
    constexpr int QS = TYPE == Q4_K ? 16 : 48;
    constexpr int KB_SCALES = GEMV_K45_KB_SCALES;                // floats per super-block, wave and table
    constexpr int WAVE_SCALES = GEMV_CHUNK * KB_SCALES;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15;      // weight row (A, scale tables) or activation row (B, results)
    const int part = lane >> 4;     // which 8 of a group's 32 values (A, B); which four weight rows (results)
    const int blocks_per_row = a.in_features / 32;
    const int super_blocks = a.in_features / QK_K;
    float * const scale_table = scale_lds + wave * WAVE_SCALES;                      // [kb][j][weight row]
    float * const min_table = scale_lds + (GEMV_THREADS / 64 + wave) * WAVE_SCALES;   // the same for the mins

    constexpr int REGS = GemvWide<TYPE>::REGS;
    constexpr int RUN = GEMV_CHUNK * GemvWide<TYPE>::UNITS;
    uint32_t unit_source[REGS];
    int unit_slot[REGS];
#pragma unroll
    for (int i = 0; i < REGS; ++i) {
        const int id = min(tid + i * GEMV_THREADS, GEMV_GN * RUN - 1);
        const int row = id / RUN;
        const int unit_in_row = id - row * RUN;
        const int unit_kb = unit_in_row / GemvWide<TYPE>::UNITS;
        const int unit = unit_in_row - unit_kb * GemvWide<TYPE>::UNITS;
        const int src_row = min(n0 + row, a.out_features - 1);
        unit_source[i] = static_cast<uint32_t>(src_row - n0) * static_cast<uint32_t>(a.row_bytes) + unit_in_row * 16;
        unit_slot[i] = gemv_kb_major_offset(unit_kb, row, F::RAW_PITCH) + unit * 16;
    }
    const uint8_t * const tile = weights + static_cast<int64_t>(n0) * a.row_bytes;
    uint4 staged[REGS];
    auto fetch = [&](int first_block) {
        const int blocks = min(GEMV_CHUNK, super_blocks - first_block);
        if (blocks == GEMV_CHUNK) {
            const uint8_t * origin = tile + static_cast<int64_t>(first_block) * F::BLOCK_BYTES;
#pragma unroll
            for (int i = 0; i < REGS; ++i) {
                staged[i] = *reinterpret_cast<const uint4 *>(origin + unit_source[i]);
            }
        } else {
            gemv_fetch<TYPE>(staged, weights, a.row_bytes, n0, a.out_features, first_block, blocks, tid);
        }
    };

    // The activations of a pass (the rows' q8_1 values of 8 super-blocks, their block scales and block sums) are
    // copied to LDS by the whole workgroup with 16-byte loads along the rows: a lane of the matrix instruction
    // needs 8 bytes of one row at a time, and fetched that way from global memory every load instruction would
    // touch as many cache lines as the task has rows and use a quarter of each.  Like the weights they are
    // requested a pass ahead.  Rows the task does not have stay zero.
    //   x_lds: [XROWS][GEMV_X_PITCH] values, then [XROWS][XD_PITCH] scales, then [XROWS][XD_PITCH] sums
    // XROWS (8 or 16) is the most rows a call of the routine can have: the LDS it needs, and with it how many
    // workgroups share a CU, follows from it.
    static_assert(XROWS == 8 || XROWS == 16, "half or all of the matrix instruction's 16 columns");
    constexpr int X_LOADS = XROWS * GEMV_CHUNK * QK_K / 16 / GEMV_THREADS;   // 16-byte pieces per thread
    constexpr int SCALE_LOADS = XROWS / 8;                                   // pieces of 4 scales or sums per thread
    constexpr int XD_PITCH = GEMV_XD_PITCH;
    float * const xd_lds = reinterpret_cast<float *>(x_lds + XROWS * GEMV_X_PITCH);
    const int piece_row = tid >> 7, piece = tid & 127;               // value pieces: two rows per instruction
    // scale / sum pieces: 16 per row, all scale rows first, then all sum rows
    const int scale_piece = tid & 15;
    const float * scale_source[SCALE_LOADS];
    int scale_row[SCALE_LOADS], scale_slot[SCALE_LOADS];
#pragma unroll
    for (int l = 0; l < SCALE_LOADS; ++l) {
        const int id = (tid >> 4) + 16 * l;          // 0 .. 2 * XROWS - 1
        scale_row[l] = id & (XROWS - 1);
        scale_slot[l] = id * XD_PITCH + scale_piece * 4;
        scale_source[l] = (id < XROWS ? a.dx : a.sx) +
            static_cast<int64_t>(row_start + min(scale_row[l], nrows - 1)) * blocks_per_row + scale_piece * 4;
    }
    const int8_t * const x_source = a.qx + static_cast<int64_t>(row_start) * a.in_features + piece * 16;
    uint32_t x_row_offset[X_LOADS];   // a task's rows span less than 2^27 bytes
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) {
        x_row_offset[i] = static_cast<uint32_t>(2 * i + piece_row) * static_cast<uint32_t>(a.in_features);
    }
    uint4 x_staged[X_LOADS];
    float4 scale_staged[SCALE_LOADS];
    auto fetch_activations = [&](int first_block) {
        const int blocks = min(GEMV_CHUNK, super_blocks - first_block);
        const int8_t * const origin = x_source + static_cast<int64_t>(first_block) * QK_K;
#pragma unroll
        for (int i = 0; i < X_LOADS; ++i) {
            x_staged[i] = make_uint4(0u, 0u, 0u, 0u);
            if (2 * i + piece_row < nrows && piece * 16 < blocks * QK_K) {
                x_staged[i] = *reinterpret_cast<const uint4 *>(origin + x_row_offset[i]);
            }
        }
#pragma unroll
        for (int l = 0; l < SCALE_LOADS; ++l) {
            scale_staged[l] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (scale_row[l] < nrows && scale_piece * 4 < blocks * 8) {
                scale_staged[l] = *reinterpret_cast<const float4 *>(scale_source[l] + first_block * 8);
            }
        }
    };
    auto park_activations = [&]() {
#pragma unroll
        for (int i = 0; i < X_LOADS; ++i) {
            *reinterpret_cast<uint4 *>(x_lds + (2 * i + piece_row) * GEMV_X_PITCH + piece * 16) = x_staged[i];
        }
#pragma unroll
        for (int l = 0; l < SCALE_LOADS; ++l) {
            *reinterpret_cast<float4 *>(xd_lds + scale_slot[l]) = scale_staged[l];
        }
    };
    const uint8_t * const x_lane = x_lds + (col & (XROWS - 1)) * GEMV_X_PITCH + wave * 64 + part * 8;
    const float * const xd_lane = xd_lds + (col & (XROWS - 1)) * XD_PITCH + wave * 2;
    const float * const xsum_lane =
        xd_lds + (XROWS + (col & (XROWS - 1))) * XD_PITCH + wave * 2 + (part >> 1) * 8 + (part & 1);

    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
    v4f acc_min = {0.0f, 0.0f, 0.0f, 0.0f};
    // One pass from LDS.  A whole pass (FULL) is straight-line code, so that the LDS reads, matrix instructions
    // and scaling of its eight super-blocks can be interleaved; a last, shorter pass checks every super-block.
    auto compute = [&](auto full, int chunk_blocks) {
        constexpr bool FULL = decltype(full)::value;
        // scales and mins of this wave's two groups as floats: lane = (weight row, super-blocks part and part + 4)
        {
            const int shift = 16 * (wave & 1);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int kb = part + 4 * h;
                if (FULL || kb < chunk_blocks) {
                    const uint8_t * blk = raw + gemv_kb_major_offset(kb, col, F::RAW_PITCH);
                    const uint32_t d_dmin = lds_u32(blk);
                    const float d = half_bits_to_float(d_dmin & 0xffffu), dmin = half_bits_to_float(d_dmin >> 16);
                    const uint32_t low = lds_u32(blk + 4) >> shift, mid = lds_u32(blk + 8) >> shift,
                                   high = lds_u32(blk + 12) >> shift;
                    const uint32_t sc = wave < 2 ? (low & 0x3f3fu) : ((high & 0x0f0fu) | ((low >> 2) & 0x3030u));
                    const uint32_t mn = wave < 2 ? (mid & 0x3f3fu) : (((high >> 4) & 0x0f0fu) | ((mid >> 2) & 0x3030u));
                    scale_table[kb * KB_SCALES + col] = d * static_cast<float>(sc & 0xffu);
                    scale_table[kb * KB_SCALES + GEMV_GN + col] = d * static_cast<float>((sc >> 8) & 0xffu);
                    min_table[kb * KB_SCALES + col] = dmin * static_cast<float>(mn & 0xffu);
                    min_table[kb * KB_SCALES + GEMV_GN + col] = dmin * static_cast<float>((mn >> 8) & 0xffu);
                }
            }
        }
        // the tables are private to the wave, whose LDS operations complete in order: no barrier, but the
        // compiler must not move the reads below across the writes above
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // (activation rows the task does not have, and lanes 8..15 of every 16, which repeat rows 0..7, produce
        // result columns that are never stored)
#pragma unroll
        for (int kb = 0; kb < GEMV_CHUNK; ++kb) {
            if (FULL || kb < chunk_blocks) {
                const uint8_t * blk = raw + gemv_kb_major_offset(kb, col, F::RAW_PITCH);
                const uint32_t a0 = lds_u32(blk + QS + wave * 32 + part * 8);
                const uint32_t a1 = lds_u32(blk + QS + wave * 32 + part * 8 + 4);
                uint32_t lo0 = a0 & 0x0f0f0f0fu, lo1 = a1 & 0x0f0f0f0fu;
                uint32_t hi0 = (a0 >> 4) & 0x0f0f0f0fu, hi1 = (a1 >> 4) & 0x0f0f0f0fu;
                if constexpr (TYPE == Q5_K) {
                    const uint32_t h0 = lds_u32(blk + 16 + part * 8) >> (2 * wave);
                    const uint32_t h1 = lds_u32(blk + 16 + part * 8 + 4) >> (2 * wave);
                    lo0 |= (h0 & 0x01010101u) << 4;
                    lo1 |= (h1 & 0x01010101u) << 4;
                    hi0 |= ((h0 >> 1) & 0x01010101u) << 4;
                    hi1 |= ((h1 >> 1) & 0x01010101u) << 4;
                }
                const long a_lo = static_cast<long>(static_cast<uint64_t>(lo1) << 32 | lo0);
                const long a_hi = static_cast<long>(static_cast<uint64_t>(hi1) << 32 | hi0);
                const uint2 x_lo = *reinterpret_cast<const uint2 *>(x_lane + kb * QK_K);
                const uint2 x_hi = *reinterpret_cast<const uint2 *>(x_lane + kb * QK_K + 32);
                const float2 xd = *reinterpret_cast<const float2 *>(xd_lane + kb * 8);
                const long b_lo = static_cast<long>(static_cast<uint64_t>(x_lo.y) << 32 | x_lo.x);
                const long b_hi = static_cast<long>(static_cast<uint64_t>(x_hi.y) << 32 | x_hi.x);
                const v4i zero = {0, 0, 0, 0};
                const v4i dot_lo = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_lo, b_lo, zero, 0, 0, 0);
                const v4i dot_hi = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_hi, b_hi, zero, 0, 0, 0);
                const v4f scale_lo = *reinterpret_cast<const v4f *>(scale_table + kb * KB_SCALES + part * 4);
                const v4f scale_hi = *reinterpret_cast<const v4f *>(scale_table + kb * KB_SCALES + GEMV_GN + part * 4);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    acc[v] = fmaf(static_cast<float>(dot_lo[v]) * xd.x, scale_lo[v], acc[v]);
                    acc[v] = fmaf(static_cast<float>(dot_hi[v]) * xd.y, scale_hi[v], acc[v]);
                }
            }
        }
        // min term: four groups per instruction, (kb, j) = (2i + part / 2, part % 2)
#pragma unroll
        for (int i = 0; i < GEMV_CHUNK / 2; ++i) {
            if (FULL || 2 * i < chunk_blocks) {
                const int kb = 2 * i + (part >> 1);
                float minimum = 0.0f, block_sum = 0.0f;
                if (FULL || kb < chunk_blocks) {
                    minimum = min_table[kb * KB_SCALES + (part & 1) * GEMV_GN + col];
                    block_sum = xsum_lane[2 * i * 8];
                }
                acc_min = __builtin_amdgcn_mfma_f32_16x16x4f32(minimum, block_sum, acc_min, 0, 0, 0);
            }
        }
    };

    fetch(0);
    fetch_activations(0);
    for (int kb0 = 0; kb0 < super_blocks; kb0 += GEMV_CHUNK) {
        const int chunk_blocks = min(GEMV_CHUNK, super_blocks - kb0);
        __syncthreads();   // the previous pass is done with `raw` and `x_lds`
        if (chunk_blocks == GEMV_CHUNK) {
#pragma unroll
            for (int i = 0; i < REGS; ++i) {
                if (tid + i * GEMV_THREADS < GEMV_GN * RUN) {
                    uint32_t * dst = reinterpret_cast<uint32_t *>(raw + unit_slot[i]);
                    dst[0] = staged[i].x; dst[1] = staged[i].y; dst[2] = staged[i].z; dst[3] = staged[i].w;
                }
            }
        } else {
            gemv_park<TYPE, true>(raw, staged, chunk_blocks, tid);
        }
        park_activations();
        if (kb0 + GEMV_CHUNK < super_blocks) {   // the next pass travels while this one is computed
            fetch(kb0 + GEMV_CHUNK);
            fetch_activations(kb0 + GEMV_CHUNK);
        }
        __syncthreads();

        if (chunk_blocks == GEMV_CHUNK) {
            compute(std::true_type(), chunk_blocks);
        } else {
            compute(std::false_type(), chunk_blocks);
        }
    }

    // lane (col, part) holds activation row `col`, weight rows 4 * part .. + 3 of this wave's share of K
    __syncthreads();   // everyone is done with `raw`, which now carries the partial results: [wave][m][n]
    float * const partial = reinterpret_cast<float *>(raw);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        partial[(wave * 16 + col) * GEMV_GN + part * 4 + v] = acc[v] - acc_min[v];
    }
    __syncthreads();
    {
        const int n = tid & 15, m = tid >> 4;
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < GEMV_THREADS / 64; ++w) {
            total += partial[(w * 16 + m) * GEMV_GN + n];
        }
        if (m < nrows && n0 + n < a.out_features) {
            y[static_cast<int64_t>(row_start + m) * a.out_features + n0 + n] = to_bf16_bits(total);
        }
    }
}

template <int TYPE, int ROWS, int FOLD, bool FUSED>
TGO_DEVICE void gemv_rows(const GemvArgs & a, uint8_t * raw, float * scale_lds, uint8_t * x_lds, const uint2 * grid,
                          const uint8_t * weights, uint16_t * y, int n0, int row_start, int nrows, int tid) {
    static_assert(!FUSED || (TYPE != Q4_K && TYPE != Q5_K), "the Q4_K / Q5_K routines read quantized activations");
    if constexpr ((TYPE == Q4_K || TYPE == Q5_K) && ROWS > 2) {
        // (no long rows in the matrix-core routine: it takes the 16 * FOLD weight rows 16 at a time)
        if constexpr (FOLD == 1) {
            gemv_task_k45_mfma<TYPE, GEMV_ROWS>(a, raw, scale_lds, x_lds, weights, y, n0, row_start, nrows, tid);
        } else {
#pragma unroll 1
            for (int part = 0; part < FOLD; ++part) {
                const int first = n0 * FOLD + part * GEMV_GN;
                if (first < a.out_features) {   // (the routine addresses its rows relative to a first row that exists)
                    gemv_task_k45_mfma<TYPE, GEMV_ROWS>(a, raw, scale_lds, x_lds, weights, y, first, row_start, nrows, tid);
                }
            }
        }
        return;
    }
    if constexpr ((TYPE == Q4_K || TYPE == Q5_K) && ROWS == 1) {
        if (static_cast<int64_t>(GEMV_GN) * FOLD * a.row_bytes < (int64_t{1} << 32)) {   // 32-bit row offsets
            gemv_task_k45_direct<TYPE, FOLD>(a, weights, y, n0, row_start, tid);
            return;
        }
    }
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        gemv_task_k45<TYPE, ROWS <= 2 ? ROWS : 1, FOLD>(a, raw, weights, y, n0, row_start, nrows, tid);
    } else {
        gemv_task<TYPE, ROWS, FOLD, FUSED>(a, raw, x_lds, grid, weights, y, n0, row_start, nrows, tid);
    }
}

// Fused grouped calls: task `task` of the list that build_tasks would write for row tiles of GEMV_ROWS (group g covers
// rows [offsets[g - 1], offsets[g]) of expert indices[g]; groups with an expert out of range, no rows or rows outside
// the input are dropped; every other group is cut into tasks of at most GEMV_ROWS rows, in group order), found by the
// workgroup itself: 256 groups per round, a prefix sum of their task counts, and the thread whose group holds the
// task publishes it.  All threads of the workgroup call this; false when the list has no such task.
TGO_DEVICE bool gemv_find_task(const GemvArgs & a, int task, int tid, int * shared, int & expert, int & row_start,
                               int & row_end) {
    const int lane = tid & 63;
    const int wave = tid >> 6;
    if (tid == 0) {
        shared[4] = -1;
    }
    int running = 0;   // tasks of the groups of earlier rounds (the same on every thread)
    for (int base = 0; base < a.num_groups; base += GEMV_THREADS) {
        const int group = base + tid;
        int begin = 0, end = 0, group_expert = -1, count = 0;
        if (group < a.num_groups) {
            begin = group == 0 ? 0 : a.expert_offsets[group - 1];
            end = a.expert_offsets[group];
            const int64_t expert64 = a.expert_indices[group];
            if (expert64 >= 0 && expert64 < a.num_experts && begin >= 0 && end > begin && end <= a.rows) {
                group_expert = static_cast<int>(expert64);
                count = (end - begin + GEMV_ROWS - 1) / GEMV_ROWS;
            }
        }
        int inclusive = count;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const int below = __shfl_up(inclusive, offset);
            inclusive += lane >= offset ? below : 0;
        }
        __syncthreads();   // (the previous round's wave totals have been read)
        if (lane == 63) {
            shared[wave] = inclusive;
        }
        __syncthreads();
        int before = running;
#pragma unroll
        for (int w = 0; w < GEMV_THREADS / 64; ++w) {
            const int total = shared[w];
            before += w < wave ? total : 0;
            running += total;
        }
        const int first = before + inclusive - count;
        if (task >= first && task < first + count) {
            shared[4] = group_expert;
            shared[5] = begin + (task - first) * GEMV_ROWS;
            shared[6] = end;
        }
        if (running > task) {   // uniform
            break;
        }
    }
    __syncthreads();
    expert = shared[4];
    row_start = shared[5];
    row_end = min(row_start + GEMV_ROWS, shared[6]);
    return expert >= 0;
}

// MAX_ROWS (1, 2, 4 or 8) bounds the rows of any task of the launch: the register budget, and with it how
// many workgroups a CU can keep in flight to cover memory latency, follows the largest variant compiled in.
// FOLD: weight rows per long row, see gemv_task; n_groups then counts groups of 16 long rows.
// WALK: a dense call of more than GEMV_ROWS rows, taken GEMV_ROWS at a time.  Its own instantiation: around that
// loop the compiler keeps the routines' per-thread constants in registers, which costs the single-pass kernels
// (every grouped call, every dense call of up to GEMV_ROWS rows) a wave per SIMD if they share the code.
// FUSED: bf16 activations, quantized by the workgroups themselves (gemv_task), and, for grouped calls, the task looked
// up in the group list instead of a task list (gemv_find_task): the whole call is this one launch.
// Three workgroups per CU are asked of the compiler for the instances of more than two rows whose eight-row routine
// alone would take 180 to 250 registers and leave room for two, where it spills little to get there (IQ2_S 28 and, fused,
// 116 bytes of scratch per lane, Q5_K 36, Q6_K 52, all inside the routines for five to eight rows, which few tasks of a
// decode batch take): the tasks of one to four rows gain the third workgroup.  The other instances (Q3_K, the fused
// Q6_K ones, long rows) spill three times as much under the same bound and measured slower with it; Q4_K fits as it is.
template <int TYPE, int MAX_ROWS, int FOLD, bool WALK = false, bool FUSED = false>
__global__ __launch_bounds__(GEMV_THREADS, (MAX_ROWS > 2 && FOLD == 1 && !WALK && (TYPE == IQ2_S || (!FUSED && (TYPE == Q5_K || TYPE == Q6_K)))) ? 3 : 1)
void mmq_gemv_kernel(const GemvArgs a) {
    static_assert(!WALK || MAX_ROWS == GEMV_ROWS, "a walked call has full chunks");
    using F = Format<TYPE>;
    __shared__ __attribute__((aligned(16))) uint8_t raw[GEMV_GN * GEMV_CHUNK * gemv_slot_bytes<TYPE>() + GEMV_CHUNK * 4];
    __shared__ uint2 grid[TYPE == IQ2_S ? TGO_IQ2S_GRID_ENTRIES : 1];
    // float scale and min tables of the matrix-core variant: [scales, mins][wave][super-block][group of the wave's two][weight row]
    constexpr bool TABLES = (TYPE == Q4_K || TYPE == Q5_K) && MAX_ROWS > 2;
    __shared__ __attribute__((aligned(16))) float scale_lds[TABLES ? 2 * (GEMV_THREADS / 64) * GEMV_CHUNK * GEMV_K45_KB_SCALES : 4];
    // its copy of a pass's activations: q8_1 values, block scales, block sums
    __shared__ __attribute__((aligned(16))) uint8_t x_lds[TABLES  ? GEMV_ROWS * GEMV_X_PITCH + 2 * GEMV_ROWS * GEMV_XD_PITCH * 4
                                                          : FUSED ? gemv_fused_x_bytes<MAX_ROWS>()
                                                                  : 16];
    __shared__ int found_task[8];

    const int tid = threadIdx.x;
    int n_group = blockIdx.x % (a.n_groups * a.projections);
    const int task = blockIdx.x / (a.n_groups * a.projections);
    const bool second = n_group >= a.n_groups;
    n_group -= second ? a.n_groups : 0;

    // the codebook's packed entries travel while the task is looked up
    constexpr int GRID_PER_THREAD = TGO_IQ2S_GRID_ENTRIES / GEMV_THREADS;
    uint32_t packed_grid[TYPE == IQ2_S ? GRID_PER_THREAD : 1];
    if constexpr (TYPE == IQ2_S) {
        request_iq2s_grid<GRID_PER_THREAD>(packed_grid, tid);
    }
    int expert = 0, row_start = 0, row_end = a.rows;
    if constexpr (FUSED) {
        if (a.expert_offsets != nullptr && !gemv_find_task(a, task, tid, found_task, expert, row_start, row_end)) {
            return;
        }
    } else if (a.task_count != nullptr) {
        // all four loads go out together (slot `task` exists in the list's arrays whatever the count says)
        const int count = a.task_count[0];
        expert = a.task_expert[task];
        row_start = a.task_row_start[task];
        row_end = a.task_row_end[task];
        if (task >= count) {
            return;
        }
    }
    const uint8_t * weights = (second ? a.packed_second : a.packed) + static_cast<int64_t>(expert) * a.bytes_per_expert;
    uint16_t * const y = second ? a.y_second : a.y;
    const int n0 = n_group * GEMV_GN;

    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_grid<GRID_PER_THREAD>(grid, packed_grid, tid);
    }
    // a task has 1..GEMV_ROWS rows; a walked dense call has more (every routine starts with a barrier before it
    // touches LDS again)
    auto run = [&](int first, int nrows) {
        if (MAX_ROWS == 1 || nrows == 1) {
            gemv_rows<TYPE, 1, FOLD, FUSED>(a, raw, scale_lds, x_lds, grid, weights, y, n0, first, nrows, tid);
        } else if (MAX_ROWS == 2 || nrows == 2) {
            gemv_rows<TYPE, MAX_ROWS >= 2 ? 2 : 1, FOLD, FUSED>(a, raw, scale_lds, x_lds, grid, weights, y, n0, first, nrows, tid);
        } else if (MAX_ROWS == 4 || nrows <= 4) {
            gemv_rows<TYPE, MAX_ROWS >= 4 ? 4 : 1, FOLD, FUSED>(a, raw, scale_lds, x_lds, grid, weights, y, n0, first, nrows, tid);
        } else {
            gemv_rows<TYPE, MAX_ROWS >= 8 ? GEMV_ROWS : 1, FOLD, FUSED>(a, raw, scale_lds, x_lds, grid, weights, y, n0, first, nrows, tid);
        }
    };
    if constexpr (WALK) {
#pragma unroll 1
        for (int first = row_start; first < row_end; first += GEMV_ROWS) {
            run(first, min(GEMV_ROWS, row_end - first));
        }
    } else {
        run(row_start, row_end - row_start);
    }
}

// The matrix-core routine alone, for launches whose tasks all take it (dense calls of three or more rows): without
// the other routines' registers more workgroups fit a CU.
template <int TYPE, int XROWS>
__global__ __launch_bounds__(GEMV_THREADS) void mmq_gemv_mfma_kernel(const GemvArgs a) {
    using F = Format<TYPE>;
    __shared__ __attribute__((aligned(16))) uint8_t raw[GEMV_GN * GEMV_CHUNK * gemv_slot_bytes<TYPE>() + GEMV_CHUNK * 4];
    __shared__ __attribute__((aligned(16))) float scale_lds[2 * (GEMV_THREADS / 64) * GEMV_CHUNK * GEMV_K45_KB_SCALES];
    __shared__ __attribute__((aligned(16))) uint8_t x_lds[XROWS * GEMV_X_PITCH + 2 * XROWS * GEMV_XD_PITCH * 4];
    const int n_group = blockIdx.x % a.n_groups;
    const bool second = blockIdx.x >= a.n_groups;
    const uint8_t * const weights = second ? a.packed_second : a.packed;
    uint16_t * const y = second ? a.y_second : a.y;
    if constexpr (XROWS == GEMV_ROWS) {
        // calls of up to eight rows: one pass over the matrix (kept free of the loop below, around which the
        // compiler holds the routine's per-thread constants in registers: 185 instead of 142, one wave per SIMD less)
        gemv_task_k45_mfma<TYPE, XROWS>(a, raw, scale_lds, x_lds, weights, y, n_group * GEMV_GN, 0, a.rows, threadIdx.x);
    } else {
#pragma unroll 1
        for (int first = 0; first < a.rows; first += XROWS) {   // calls of up to GEMV_DENSE_ROWS rows, 16 at a time
            gemv_task_k45_mfma<TYPE, XROWS>(a, raw, scale_lds, x_lds, weights, y, n_group * GEMV_GN, first,
                                            min(XROWS, a.rows - first), threadIdx.x);
        }
    }
}

static bool gemv_grouped(const GemvArgs & args) { return args.task_count != nullptr || args.expert_offsets != nullptr; }

template <int TYPE, int FOLD, bool FUSED>
static hipError_t launch_gemv_folded(const GemvArgs & args, int max_rows, unsigned grid, hipStream_t stream) {
    if (max_rows <= 1) {
        mmq_gemv_kernel<TYPE, 1, FOLD, false, FUSED><<<grid, GEMV_THREADS, 0, stream>>>(args);
    } else if (max_rows <= 2) {
        mmq_gemv_kernel<TYPE, 2, FOLD, false, FUSED><<<grid, GEMV_THREADS, 0, stream>>>(args);
    } else if (max_rows <= 4) {
        mmq_gemv_kernel<TYPE, 4, FOLD, false, FUSED><<<grid, GEMV_THREADS, 0, stream>>>(args);
    } else if (gemv_grouped(args) || args.rows <= GEMV_ROWS) {
        mmq_gemv_kernel<TYPE, GEMV_ROWS, FOLD, false, FUSED><<<grid, GEMV_THREADS, 0, stream>>>(args);
    } else if constexpr (TYPE != Q4_K && TYPE != Q5_K && !FUSED) {
        // (dense Q4_K / Q5_K calls of that size take the matrix-core kernel; fused dense calls are one task)
        mmq_gemv_kernel<TYPE, GEMV_ROWS, FOLD, true, false><<<grid, GEMV_THREADS, 0, stream>>>(args);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <int TYPE>
static hipError_t launch_gemv_typed(GemvArgs args, int task_slots, hipStream_t stream) {
    // no task has more rows than the call (dense: the call is the task)
    const int max_rows = args.rows < GEMV_ROWS ? args.rows : GEMV_ROWS;
    const bool matrix_cores_only = (TYPE == Q4_K || TYPE == Q5_K) && !gemv_grouped(args) && max_rows > 2;
    // short K: 2 or 4 consecutive weight rows form one long row, see gemv_task
    int fold = 1;
    const int super_blocks = args.in_features / QK_K;
    if (!matrix_cores_only) {
        if (super_blocks <= 2 && args.out_features % 4 == 0) {
            fold = 4;
        } else if (super_blocks <= 4 && args.out_features % 2 == 0) {
            fold = 2;
        }
    }
    args.n_groups = (args.out_features / fold + GEMV_GN - 1) / GEMV_GN;
    const int64_t total = static_cast<int64_t>(args.n_groups) * args.projections * task_slots;
    if (total <= 0 || total > 0x7fffffffLL) {
        return hipErrorInvalidValue;
    }
    const unsigned grid = static_cast<unsigned>(total);
    const ProfileScope scope(5, stream);
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        if (args.x != nullptr) {
            return hipErrorInvalidValue;   // (gemv_fuses is false for these formats)
        }
        if (matrix_cores_only) {
            if (args.rows <= GEMV_ROWS) {
                mmq_gemv_mfma_kernel<TYPE, GEMV_ROWS><<<grid, GEMV_THREADS, 0, stream>>>(args);
            } else {
                mmq_gemv_mfma_kernel<TYPE, 16><<<grid, GEMV_THREADS, 0, stream>>>(args);
            }
            return hipGetLastError();
        }
    } else if (args.x != nullptr) {
        switch (fold) {
            case 4: return launch_gemv_folded<TYPE, 4, true>(args, max_rows, grid, stream);
            case 2: return launch_gemv_folded<TYPE, 2, true>(args, max_rows, grid, stream);
            default: return launch_gemv_folded<TYPE, 1, true>(args, max_rows, grid, stream);
        }
    }
    switch (fold) {
        case 4: return launch_gemv_folded<TYPE, 4, false>(args, max_rows, grid, stream);
        case 2: return launch_gemv_folded<TYPE, 2, false>(args, max_rows, grid, stream);
        default: return launch_gemv_folded<TYPE, 1, false>(args, max_rows, grid, stream);
    }
}

static hipError_t launch_gemv_by_type(const GemvArgs & args, int task_slots, int quant_type, hipStream_t stream) {
    switch (quant_type) {
        case Q3_K: return launch_gemv_typed<Q3_K>(args, task_slots, stream);
        case Q4_K: return launch_gemv_typed<Q4_K>(args, task_slots, stream);
        case Q5_K: return launch_gemv_typed<Q5_K>(args, task_slots, stream);
        case Q6_K: return launch_gemv_typed<Q6_K>(args, task_slots, stream);
        case IQ2_S: return launch_gemv_typed<IQ2_S>(args, task_slots, stream);
        default: return hipErrorInvalidValue;
    }
}

// What both kinds of call share: the weights, the results, the shape.
static GemvArgs gemv_common_args(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                                 uint16_t * output, uint16_t * output_second, int rows, int in_features,
                                 int out_features, int quant_type) {
    GemvArgs args = {};
    args.packed = packed;
    args.packed_second = packed_second;
    args.y = output;
    args.y_second = output_second;
    args.projections = packed_second != nullptr ? 2 : 1;
    args.bytes_per_expert = bytes_per_expert;
    args.row_bytes = static_cast<int64_t>(in_features / QK_K) * block_bytes(quant_type);
    args.rows = rows;
    args.in_features = in_features;
    args.out_features = out_features;
    args.n_groups = (out_features + GEMV_GN - 1) / GEMV_GN;
    // (a dense call has one "expert": the whole weight)
    const int64_t weight_bytes = static_cast<int64_t>(out_features) * args.row_bytes;
    args.unit_staging = block_bytes(quant_type) % 16 != 0 && wide_stage_ok(packed, weight_bytes) &&
                                (packed_second == nullptr || wide_stage_ok(packed_second, weight_bytes)) &&
                                args.row_bytes < (1 << 24)
                            ? 1 : 0;
    return args;
}

hipError_t launch_mmq_gemv_fused(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                                 const uint16_t * input, const int64_t * gather, int64_t input_rows,
                                 const int64_t * expert_indices, const int32_t * expert_offsets, int num_experts,
                                 int num_groups, uint16_t * output, uint16_t * output_second, int rows, int in_features,
                                 int out_features, int quant_type, hipStream_t stream) {
    if (!gemv_fuses(quant_type, rows, expert_offsets != nullptr ? num_groups : 0)) {
        return hipErrorInvalidValue;
    }
    GemvArgs args = gemv_common_args(packed, packed_second, bytes_per_expert, output, output_second, rows, in_features,
                                     out_features, quant_type);
    args.x = input;
    args.gather = gather;
    args.input_rows = input_rows;
    args.rows_padded = rows;
    int task_slots = 1;
    if (expert_offsets != nullptr) {
        args.expert_indices = expert_indices;
        args.expert_offsets = expert_offsets;
        args.num_experts = num_experts;
        args.num_groups = num_groups;
        // (every task holds at least one row of its own, so a call of few rows over many listed groups -- a router
        // that lists every expert -- has no more tasks than rows: each slot costs its workgroups a task lookup)
        task_slots = std::min(max_tasks_for(rows, num_groups, GEMV_ROWS), rows);
    }
    return launch_gemv_by_type(args, task_slots, quant_type, stream);
}

hipError_t launch_mmq_gemv(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                           const Q8Workspace & ws, uint16_t * output, uint16_t * output_second,
                           const TaskList * tasks, int rows, int in_features, int out_features,
                           int quant_type, hipStream_t stream) {
    if (!ws.by_rows()) {
        return hipErrorInvalidValue;   // these kernels read the row-major activation layout
    }
    GemvArgs args = gemv_common_args(packed, packed_second, bytes_per_expert, output, output_second, rows, in_features,
                                     out_features, quant_type);
    args.qx = ws.q;
    args.dx = ws.d;
    args.sx = ws.sum;
    args.rows_padded = static_cast<int>(ws.rows_padded);
    int task_slots = 1;
    if (tasks != nullptr) {
        args.task_count = tasks->count;
        args.task_expert = tasks->expert;
        args.task_row_start = tasks->row_start;
        args.task_row_end = tasks->row_end;
        task_slots = tasks->max_tasks;
    } else {
        if (rows > GEMV_DENSE_ROWS) {
            return hipErrorInvalidValue;
        }
        args.task_count = nullptr;
        args.task_expert = nullptr;
        args.task_row_start = nullptr;
        args.task_row_end = nullptr;
    }
    return launch_gemv_by_type(args, task_slots, quant_type, stream);
}

}  // namespace tgo
