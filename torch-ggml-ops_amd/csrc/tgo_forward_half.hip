// Forward kernels with exact-integer fp16 matrix operands: q8_1 activations x packed GGUF weights on gfx950.
//
// y[r, n] = sum over super-blocks of  d[n] * (sum over its 32-value blocks b of dx[r, b] * I_b(r, n))  -  wm[n, b] * sx[r, b]
// where I_b is the integer dot product of the block's quantized activations with the weight operand
// v = integer sub-scale x quant (decode16_half; exact in fp16).  v_mfma_f32_32x32x16_f16 returns I_b exactly
// and already as a float (two instructions per 32-value block, the second accumulating onto the first), so what is
// left per result and block is ONE multiply-add with the activation scale; the weight scale d is one number per
// weight row and super-block and is applied once per stage.  The int8 matrix instruction delivers int32 and cannot
// take the 11- to 13-bit operand v, which costs its kernels (tgo_forward.hip) a second and third vector instruction
// per result; the vector pipe, not the matrix pipe, bounds either family.
//
// Work split.  A workgroup (4 waves) owns 128 weight rows x 128 activation rows; wave w owns activation rows
// [32w, 32w + 32) and all 128 weight rows (1 x 4 tiles, 64 accumulator registers).  The matrix instructions run
// with the weights as the A operand: a lane then holds one activation row (its block scales are lane scalars) and
// 16 weight rows per tile.  A super-block is processed in stages of 128 values (64 for Q6_K, whose operand needs
// two fp16 numbers): the packed blocks of the 128 weight rows wait in LDS, each stage unpacks its share into a
// 32 KiB fp16 tile in fragment order, all waves multiply from it.  Two workgroups share a CU, so one's barriers
// and unpack phases overlap the other's multiply phases.
//
// Latency.  Nothing is loaded where it is used: the packed blocks of the next super-block are requested at the
// start of the current one's last stage and parked in LDS after it; a wave's activation fragments, scales and sums
// of the next stage are requested as the current stage's multiply phase frees their registers, and arrive during the
// unpack phase in between.
#include <type_traits>

#include "tgo_device.h"
#include "tgo_forward_args.h"
#include "tgo_launch.h"

namespace tgo {

typedef float v16f __attribute__((ext_vector_type(16)));

// WAVES = 4: 128 activation rows per workgroup, two workgroups per CU; every stage has an unpack phase and a multiply
// phase with a barrier after each.  WAVES = 8 (half_forward_waves in tgo_launch.h): 256 rows, one workgroup per CU,
// operand tile, packed blocks and scales double-buffered in LDS; every wave multiplies stage g and then unpacks its
// share of stage g + 1 before the one barrier of the stage, so the unpack work per activation row halves and a
// stage costs one barrier instead of two.
template <int TYPE>
struct HalfShape {
    static constexpr int WAVES = half_forward_waves(TYPE);
    static constexpr bool PIPE = WAVES == 8;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int PLANES = TYPE == Q6_K ? 2 : 1;     // fp16 numbers per weight value
    static constexpr int STAGE_BLOCKS = 4 / PLANES;         // 32-value blocks per stage
    static constexpr int STAGES = 8 / STAGE_BLOCKS;
    static constexpr int PLANE_BYTES = FWD_TN * STAGE_BLOCKS * 32 * 2;
    static constexpr int BUFFERS = PIPE ? 2 : 1;
};

template <int TYPE>
struct HalfLds {
    static constexpr int RAW_SLOT = Format<TYPE>::BLOCK_BYTES % 16 == 0 || Format<TYPE>::RAW_PITCH > WideStage<TYPE>::PITCH
                                        ? Format<TYPE>::RAW_PITCH : WideStage<TYPE>::PITCH;
    static constexpr int BUFFERS = HalfShape<TYPE>::BUFFERS;
    alignas(16) uint8_t raw[BUFFERS][FWD_TN * RAW_SLOT];                                   // packed blocks of a super-block column
    alignas(16) uint8_t wq[BUFFERS][HalfShape<TYPE>::PLANES][HalfShape<TYPE>::PLANE_BYTES];   // fp16 operand of a stage, fragment order
    alignas(16) float ws[BUFFERS][FWD_TN];                                                 // weight scale of the super-block
    alignas(16) float wm[BUFFERS][Format<TYPE>::HAS_MIN ? 8 : 1][FWD_TN];                  // block minima
    std::conditional_t<TYPE == IQ2_S, Iq2sSelectors, uint2> codebook;   // IQ2_S: the selector table of decode16_half
};

// NARROW: a task of at most 32 rows; every wave takes the same 32 activation rows and weight tile number `wave`.
template <int TYPE, bool NARROW, bool WIDE>
TGO_DEVICE void forward_half_task(const ForwardArgs & a, HalfLds<TYPE> & lds, int n_tile, bool second, int expert,
                                  int row_start, int row_end) {
    using F = Format<TYPE>;
    using S = HalfShape<TYPE>;
    constexpr int PLANES = S::PLANES;
    constexpr int SB = S::STAGE_BLOCKS;
    constexpr int STAGES = S::STAGES;
    constexpr int THREADS = S::THREADS;
    constexpr bool PIPE = S::PIPE;
    auto & raw = lds.raw;
    auto & wq = lds.wq;
    auto & ws = lds.ws;
    auto & wm = lds.wm;
    const auto * const grid = &lds.codebook;
    // (the thread id is made opaque so that a caller running two passes in a loop gets each pass compiled
    // like a lone one: nothing derived from it can be computed once and kept alive across both passes)
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;

    const uint8_t * weights = (second ? a.packed_second : a.packed) + static_cast<int64_t>(expert) * a.bytes_per_expert;
    uint16_t * const y = second ? a.y_second : a.y;
    const bool fuse = a.swiglu != 0 && second;   // the gate tile of this workgroup's first pass is in a.y
    const int n0 = n_tile * FWD_TN;
    const int blocks_per_row = a.in_features / 32;
    const int super_blocks = a.in_features / QK_K;

    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_selectors(lds.codebook, tid, THREADS);
    }

    const int granule = NARROW ? 0 : wave;
    const int wave_row = row_start + granule * 32;
    const bool wave_active = wave_row < row_end && (!NARROW || wave < FWD_NT);   // (a narrow task has four tiles)
    int lane_row = wave_row + l32;
    lane_row = lane_row < a.rows_padded ? lane_row : a.rows_padded - 1;
    // Every global address below is a uniform 64-bit base, advanced with scalar arithmetic, plus a 32-bit lane
    // offset.  The host checks that the offsets fit (row_bytes and rows_padded below 2^24).
    const int first_tile = row_start >> 5;
    const uint8_t * const qx_task = reinterpret_cast<const uint8_t *>(a.qx) + static_cast<int64_t>(first_tile) * blocks_per_row * 2048;
    const uint32_t x_lane_offset = static_cast<uint32_t>((lane_row >> 5) - first_tile) * blocks_per_row * 2048u +
                                   static_cast<uint32_t>(((lane_row & 31) + 32 * half) * 16);
    const uint32_t dx_lane_offset = static_cast<uint32_t>(lane_row) * 4u;
    const uint32_t sum_lane_offset = (__umul24(half, a.rows_padded) + lane_row) * 4u;
    const uint8_t * const tile_weights = weights + static_cast<int64_t>(n0) * a.row_bytes;
    const int tile_rows = min(FWD_TN, a.out_features - n0);   // weight rows of this tile that exist

    // ---- packed blocks: global -> registers -> LDS ------------------------------------------------
    constexpr bool RAW_IN_REGS = F::BLOCK_BYTES % 16 == 0;
    constexpr int RAW_UNITS = RAW_IN_REGS ? F::BLOCK_BYTES / 16 : 1;
    constexpr int RAW_REGS = RAW_IN_REGS ? (FWD_TN * RAW_UNITS + THREADS - 1) / THREADS : 1;
    uint4 raw_next[RAW_REGS];
    static_assert(!(WIDE && RAW_IN_REGS), "the wide copy is for the 2-byte aligned formats");
    using W = WideStage<TYPE>;
    constexpr int WIDE_REGS = WIDE ? W::template regs<FWD_TN, THREADS>() : 1;
    WideRegs<WIDE_REGS> wide_next;
    constexpr int SLOT_PITCH = WIDE ? W::PITCH : F::RAW_PITCH;
    constexpr int SLOT_FRONT = WIDE ? W::FRONT : F::RAW_SHIFT;
    constexpr int UNIT_RECIPROCAL = (65536 + RAW_UNITS - 1) / RAW_UNITS;
    static_assert(!RAW_IN_REGS || FWD_TN * RAW_UNITS < 3000, "range of the reciprocal trick");
    auto load_raw = [&](int kb, int t) {
        if constexpr (RAW_IN_REGS) {
            const uint8_t * base = tile_weights + static_cast<int64_t>(kb) * F::BLOCK_BYTES;
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                // ids past the tile repeat its last unit, so no lane branches around a load
                const int id = min(t + THREADS * i, FWD_TN * RAW_UNITS - 1);
                const int row = static_cast<int>(__umul24(id, UNIT_RECIPROCAL) >> 16);
                const int unit = id - row * RAW_UNITS;
                const uint32_t offset = __umul24(min(row, tile_rows - 1), static_cast<uint32_t>(a.row_bytes)) + unit * 16;
                raw_next[i] = *reinterpret_cast<const uint4 *>(base + offset);
            }
        } else if constexpr (WIDE) {
            wide_fetch<TYPE, FWD_TN, THREADS, WIDE_REGS>(wide_next, tile_weights, static_cast<int>(a.row_bytes), tile_rows, kb, t);
        }
    };
    auto park_raw = [&](int kb, int t, int buffer) {
        uint8_t * const raw_slot = &raw[buffer][0];
        if constexpr (RAW_IN_REGS) {
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = min(t + THREADS * i, FWD_TN * RAW_UNITS - 1);
                const int row = static_cast<int>(__umul24(id, UNIT_RECIPROCAL) >> 16);
                const int unit = id - row * RAW_UNITS;
                uint32_t * dst = reinterpret_cast<uint32_t *>(raw_slot + row * F::RAW_PITCH + unit * 16);
                dst[0] = raw_next[i].x; dst[1] = raw_next[i].y; dst[2] = raw_next[i].z; dst[3] = raw_next[i].w;
            }
        } else if constexpr (WIDE) {
            wide_park<TYPE, FWD_TN, THREADS, WIDE_REGS>(raw_slot, wide_next, tile_weights, static_cast<int>(a.row_bytes), tile_rows, kb, t);
        } else {
            stage_blocks<TYPE>(raw_slot, weights, a.row_bytes, n0, a.out_features, kb, FWD_TN, t, THREADS);
        }
    };

    // ---- this wave's activations: fragments, block scales, block sums of one stage ----------------
    // (requested at the end of a stage's multiply phase for the next stage: they arrive during the unpack phase in
    // between; a second set of registers requested a whole stage earlier measured no faster)
    half8_t x[SB][2];
    float dxb[SB];
    float sums[F::HAS_MIN ? SB / 2 : 1];
    auto load_stage = [&](int first_block) {   // first_block: global number of the stage's first block
#pragma unroll
        for (int b = 0; b < SB; ++b) {
            const int block = first_block + b < blocks_per_row ? first_block + b : blocks_per_row - 1;
            const uint8_t * base = qx_task + static_cast<int64_t>(block) * 2048;
            x[b][0] = *reinterpret_cast<const half8_t *>(base + x_lane_offset);
            x[b][1] = *reinterpret_cast<const half8_t *>(base + 1024 + x_lane_offset);
            const float * scales = a.dx + static_cast<int64_t>(block) * a.rows_padded;
            dxb[b] = *reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(scales) + dx_lane_offset);
        }
        if constexpr (F::HAS_MIN) {
#pragma unroll
            for (int j = 0; j < SB / 2; ++j) {
                const int block = first_block + 2 * j < blocks_per_row ? first_block + 2 * j : blocks_per_row - 2;
                const float * base = a.sx + static_cast<int64_t>(block) * a.rows_padded;
                sums[j] = *reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(base) + sum_lane_offset);
            }
        }
    };

    load_raw(0, tid);
    if (wave_active) {
        load_stage(0);
    }

    constexpr int CT = NARROW ? 1 : FWD_NT;   // weight tiles per wave
    v16f acc[CT];
#pragma unroll
    for (int nt = 0; nt < CT; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nt][v] = 0.0f;
    const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    // ---- unpack of one stage: raw blocks -> fp16 operand tile -----------------------------------------
    // A thread keeps its weight row and takes 16-value units of the stage's 32-value blocks, all of the same k-half,
    // so consecutive lanes write consecutive 16-byte fragment slots.  `share` = t / 128 is wave-uniform.
    // `source`: buffer of the packed blocks and the scales; `target`: operand tile buffer.
    constexpr int SHARES = THREADS / FWD_TN;   // 2 or 4 threads per weight row
    auto unpack = [&](auto stage_tag, int t, int source, int target) {
        constexpr int s = decltype(stage_tag)::value;
        const uint32_t row = static_cast<uint32_t>(t) & (FWD_TN - 1);
        const uint32_t share = (static_cast<uint32_t>(t) / FWD_TN) & (SHARES - 1);
        const uint32_t fu = share & 1u;   // k-half of the thread's units
        const uint8_t * blk = &raw[source][0] + row * SLOT_PITCH + SLOT_FRONT;
        // slot of (tile, block b, k-half h, lane = 32 * eighth + row in tile): (((tile * SB + b) * 2 + h) * 64 + lane) * 16
        uint8_t * const out = &wq[target][0][0] + (row >> 5) * (SB * 2048) + (row & 31) * 16 + fu * 1024;
        if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
            constexpr int QS = TYPE == Q4_K ? 16 : 48;
            const uint8_t * half_blk = blk + 16 * fu;
            uint32_t planes[4] = {0, 0, 0, 0};
            if constexpr (TYPE == Q5_K) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    planes[w] = lds_u32(half_blk + 16 + 4 * w);
                }
            }
            const float dmin = half_bits_to_float(lds_u16(blk + 2));
            // 32 bytes of nibbles: low nibbles are group g, high nibbles group g + 1; a stage has two such chunks,
            // which a thread takes both (two shares per row) or one of (four shares)
            static_assert(SB == 4, "two nibble chunks per stage");
            auto chunk = [&](int p) {
                const int g = 4 * s + 2 * p;
                int sc_low, mn_low, sc_high, mn_high;
                if constexpr (s == 0) {   // groups 0..3
                    sc_low = blk[4 + g] & 0x3f; mn_low = blk[8 + g] & 0x3f;
                    sc_high = blk[5 + g] & 0x3f; mn_high = blk[9 + g] & 0x3f;
                } else {                  // groups 4..7
                    const int j = g - 4;
                    sc_low = (blk[12 + j] & 0x0f) | ((blk[4 + j] >> 2) & 0x30);
                    mn_low = (blk[12 + j] >> 4) | ((blk[8 + j] >> 2) & 0x30);
                    sc_high = (blk[13 + j] & 0x0f) | ((blk[5 + j] >> 2) & 0x30);
                    mn_high = (blk[13 + j] >> 4) | ((blk[9 + j] >> 2) & 0x30);
                }
                const HalfScale scale_low = half_scale(sc_low);
                const HalfScale scale_high = half_scale(sc_high);
                uint32_t low[8], high[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t word = lds_u32(half_blk + QS + (g >> 1) * 32 + 4 * w);
                    uint32_t bytes_low = word & 0x0f0f0f0fu;
                    uint32_t bytes_high = (word >> 4) & 0x0f0f0f0fu;
                    if constexpr (TYPE == Q5_K) {
                        // the fifth bit of group g is bit g of the plane byte: moved to bit 4
                        if constexpr (s == 0) {   // g in {0, 2}
                            bytes_low |= (planes[w] << (4 - g)) & 0x10101010u;
                            bytes_high |= (planes[w] << (3 - g)) & 0x10101010u;
                        } else {                  // g in {4, 6}
                            bytes_low |= (planes[w] >> (g - 4)) & 0x10101010u;
                            bytes_high |= (planes[w] >> (g - 3)) & 0x10101010u;
                        }
                    }
                    scaled_halves(bytes_low, scale_low, low[2 * w], low[2 * w + 1]);
                    scaled_halves(bytes_high, scale_high, high[2 * w], high[2 * w + 1]);
                }
                uint8_t * dst = out + (2 * p) * 2048;
                *reinterpret_cast<uint4 *>(dst) = make_uint4(low[0], low[1], low[2], low[3]);
                *reinterpret_cast<uint4 *>(dst + 512) = make_uint4(low[4], low[5], low[6], low[7]);
                *reinterpret_cast<uint4 *>(dst + 2048) = make_uint4(high[0], high[1], high[2], high[3]);
                *reinterpret_cast<uint4 *>(dst + 2048 + 512) = make_uint4(high[4], high[5], high[6], high[7]);
                return make_float2(dmin * static_cast<float>(mn_low), dmin * static_cast<float>(mn_high));
            };
            if constexpr (SHARES == 4) {
                const int p = static_cast<int>(share >> 1);
                const float2 minima = chunk(p);
                if (fu == 0) {   // uniform
                    wm[source][4 * s + 2 * p][row] = minima.x;
                    wm[source][4 * s + 2 * p + 1][row] = minima.y;
                }
            } else {
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    const float2 minima = chunk(p);
                    if (fu == static_cast<uint32_t>(p)) {   // uniform: each half of the workgroup writes two of the four minima
                        wm[source][4 * s + 2 * p][row] = minima.x;
                        wm[source][4 * s + 2 * p + 1][row] = minima.y;
                    }
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 2 * SB / SHARES; ++j) {
                const uint32_t local = share + SHARES * j;         // unit within the stage: block local / 2, k-half local % 2
                const uint32_t unit = 2 * SB * s + local;
                uint32_t first[8], second_plane[8];
                decode16_half<TYPE>(blk, unit, grid, first, second_plane);
                uint8_t * dst = out + (local >> 1) * 2048;
                *reinterpret_cast<uint4 *>(dst) = make_uint4(first[0], first[1], first[2], first[3]);
                *reinterpret_cast<uint4 *>(dst + 512) = make_uint4(first[4], first[5], first[6], first[7]);
                if constexpr (PLANES == 2) {
                    *reinterpret_cast<uint4 *>(dst + S::PLANE_BYTES) = make_uint4(second_plane[0], second_plane[1], second_plane[2], second_plane[3]);
                    *reinterpret_cast<uint4 *>(dst + S::PLANE_BYTES + 512) = make_uint4(second_plane[4], second_plane[5], second_plane[6], second_plane[7]);
                }
            }
        }
        if constexpr (s == 0) {
            if (share == 0) {
                ws[source][row] = half_weight_scale<TYPE>(blk);
            }
        }
    };

    // ---- multiply phase of one stage ---------------------------------------------------------------
    auto tile_of = [&](int index) { return NARROW ? wave : index; };
    auto multiply = [&](auto stage_tag, int kb, int source, int tile) {   // buffers of the scales and of the operand tile
        constexpr int s = decltype(stage_tag)::value;
        // Software pipeline over the CT x SB (tile, block) steps: the fragments of step t + 2 are read from LDS and
        // the matrix instructions of step t + 1 issued before the 16 vector instructions of step t.
        constexpr int STEPS = CT * SB;
        constexpr int RING = 3;   // fragment sets in flight: read two steps before their matrix instructions are issued (three: no faster)
        half8_t w[RING][PLANES][2];
        v16f dot[2];
        v16f within;
        auto read_step = [&](int t) {
            const int nt = tile_of(t / SB), b = t % SB;
            const int slot = ((nt * SB + b) * 2 * 64 + lane) * 16;
#pragma unroll
            for (int p = 0; p < PLANES; ++p) {
                w[t % RING][p][0] = *reinterpret_cast<const half8_t *>(&wq[tile][p][slot]);
                w[t % RING][p][1] = *reinterpret_cast<const half8_t *>(&wq[tile][p][slot + 1024]);
            }
        };
        // The matrix instructions of a step depend on one another (they accumulate into the same result), and a wave
        // issues in order: the next one is placed after a share of the step's vector instructions, which then run
        // while the previous one is in the matrix pipe instead of waiting behind its successor.
        constexpr int PARTS = 2 * PLANES;   // matrix instructions per step
        auto multiply_part = [&](int t, int part) {
            const int b = t % SB;
            const int p = part / 2, h = part % 2;
            if (part == 0) {
                dot[t & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(w[t % RING][0][0], x[b][0], zero, 0, 0, 0);
            } else {
                dot[t & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(w[t % RING][p][h], x[b][h], dot[t & 1], 0, 0, 0);
            }
        };
#pragma unroll
        for (int t = 0; t < RING - 1; ++t) {
            if (t < STEPS) {
                read_step(t);
            }
        }
#pragma unroll
        for (int part = 0; part < PARTS; ++part) {
            multiply_part(0, part);
        }
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const int nt = t / SB, b = t % SB;
            if (t + RING - 1 < STEPS) {
                read_step(t + RING - 1);
            }
#pragma unroll
            for (int part = 0; part < PARTS; ++part) {
                if (t + 1 < STEPS) {
                    multiply_part(t + 1, part);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int v = part * (16 / PARTS); v < (part + 1) * (16 / PARTS); ++v) {
                    within[v] = b == 0 ? dot[t & 1][v] * dxb[0] : __builtin_fmaf(dot[t & 1][v], dxb[b], within[v]);
                }
                // (the vector instructions above have no ordering of their own against the scheduling barriers, and
                // instruction selection may otherwise place them a whole phase later, with every matrix result kept
                // alive until then: an empty statement that "uses" them holds them here)
                asm volatile("" : "+v"(within));
                if (part + 1 < PARTS) {
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (b == SB - 1) {
                // the tile's share of the stage is complete: apply the weight scales (weight rows 8j + 4*half + 0..3)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float4 d4 = *reinterpret_cast<const float4 *>(&ws[source][tile_of(nt) * 32 + 8 * j + 4 * half]);
                    acc[nt][4 * j + 0] = __builtin_fmaf(within[4 * j + 0], d4.x, acc[nt][4 * j + 0]);
                    acc[nt][4 * j + 1] = __builtin_fmaf(within[4 * j + 1], d4.y, acc[nt][4 * j + 1]);
                    acc[nt][4 * j + 2] = __builtin_fmaf(within[4 * j + 2], d4.z, acc[nt][4 * j + 2]);
                    acc[nt][4 * j + 3] = __builtin_fmaf(within[4 * j + 3], d4.w, acc[nt][4 * j + 3]);
                }
                asm volatile("" : "+v"(acc[nt]));   // (held here like the instructions above)
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (F::HAS_MIN) {
            // acc[n][r] -= sum_b wm[n][b] * sx[r][b]: a pair of blocks per fp32 matrix instruction of depth 2
#pragma unroll
            for (int j = 0; j < SB / 2; ++j) {
                const float minus_sum = -sums[j];
#pragma unroll
                for (int nt = 0; nt < CT; ++nt) {
                    acc[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                        wm[source][s * SB + 2 * j + half][tile_of(nt) * 32 + l32], minus_sum, acc[nt], 0, 0, 0);
                }
            }
        }
        load_stage(kb * 8 + s * SB + SB);   // the following stage (block numbers are clamped)
    };

    // The loop exists once per kind of wave (with rows, without) instead of branching around the multiply phase
    // inside one loop: with a branch in the body the compiler's wait-count bookkeeping merges both paths and ends up
    // waiting for every outstanding load, prefetches included, once per round.
    // mode 0: no rows for this wave; 1: multiplies
    auto main_loop = [&](auto mode_tag) {
        constexpr bool ACTIVE = decltype(mode_tag)::value != 0;
        if constexpr (!PIPE) {
#pragma unroll 1
            for (int kb = 0; kb < super_blocks; ++kb) {
                int t = tid;
                asm volatile("" : "+v"(t));
                // (every wave has left the previous round's last unpack phase, the last reader of `raw`)
                park_raw(kb, t, 0);
                const int kb_next = kb + 1 < super_blocks ? kb + 1 : kb;   // the last round re-fetches its own blocks
                auto stage = [&](auto stage_tag) {
                    constexpr int s = decltype(stage_tag)::value;
                    __syncthreads();   // the blocks are parked; nobody still reads the previous stage's operand tile
                    if constexpr (s == STAGES - 1) {
                        load_raw(kb_next, t);
                    }
                    unpack(stage_tag, t, 0, 0);
                    __syncthreads();
                    if constexpr (ACTIVE) {
                        multiply(stage_tag, kb, 0, 0);
                    }
                };
                stage(std::integral_constant<int, 0>{});
                stage(std::integral_constant<int, 1>{});
                if constexpr (STAGES == 4) {
                    stage(std::integral_constant<int, 2>{});
                    stage(std::integral_constant<int, 3>{});
                }
            }
        } else {
            // Stage g is multiplied from operand tile g % 2 while stage g + 1 is unpacked into the other one; the
            // packed blocks of super-block kb + 1 are requested at the start of kb's last stage but one, parked at
            // its end in raw[(kb + 1) % 2], and first read one barrier later, by the unpack of (kb + 1, stage 0)
            // during kb's last stage.  Scales and minima follow the super-block's parity like the packed blocks.
            {
                int t = tid;
                asm volatile("" : "+v"(t));
                park_raw(0, t, 0);
                __syncthreads();
                unpack(std::integral_constant<int, 0>{}, t, 0, 0);
                __syncthreads();
            }
#pragma unroll 1
            for (int kb = 0; kb < super_blocks; ++kb) {
                int t = tid;
                asm volatile("" : "+v"(t));
                const int parity = kb & 1;
                const int kb_next = kb + 1 < super_blocks ? kb + 1 : kb;   // the last round re-fetches its own blocks
                auto stage = [&](auto stage_tag) {
                    constexpr int s = decltype(stage_tag)::value;
                    if constexpr (s == STAGES - 2) {
                        load_raw(kb_next, t);
                    }
                    if constexpr (ACTIVE) {
                        multiply(stage_tag, kb, parity, s & 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);   // the phases stay apart: mixed, their registers do not fit
                    if constexpr (s + 1 < STAGES) {
                        unpack(std::integral_constant<int, s + 1>{}, t, parity, (s + 1) & 1);
                    } else {
                        unpack(std::integral_constant<int, 0>{}, t, parity ^ 1, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (s == STAGES - 2) {
                        park_raw(kb_next, t, parity ^ 1);
                    }
                    __syncthreads();
                };
                stage(std::integral_constant<int, 0>{});
                stage(std::integral_constant<int, 1>{});
                if constexpr (STAGES == 4) {
                    stage(std::integral_constant<int, 2>{});
                    stage(std::integral_constant<int, 3>{});
                }
            }
        }
    };
    static_assert((STAGES == 2 || STAGES == 4) && STAGES % 2 == 0, "stages are written out above; operand tiles alternate");
    if (wave_active) {
        main_loop(std::integral_constant<int, 1>{});
    } else {
        main_loop(std::integral_constant<int, 0>{});
    }
    __syncthreads();

    // The LDS of the packed blocks and the operand tile is free now: the results, which the swapped operands left
    // transposed in the registers, pass through it (rows padded to 136) and leave as whole 256-byte rows.
    constexpr int STAGE_PITCH = 136;
    static_assert(offsetof(HalfLds<TYPE>, wq) == sizeof(raw), "the operand tiles follow the packed blocks");
    static_assert(sizeof(raw) + sizeof(wq) >= S::WAVES * 32 * STAGE_PITCH * sizeof(uint16_t), "the staging area fits");
    uint16_t * const stage_base = reinterpret_cast<uint16_t *>(&raw[0][0]);
    if constexpr (NARROW) {
        if (wave < FWD_NT) {
            stage_tile_32x32<STAGE_PITCH, true>(stage_base, acc[0], wave * 32, lane);
        }
        __syncthreads();
        const int64_t origin = static_cast<int64_t>(row_start) * a.out_features + n0;
        store_staged_rows<STAGE_PITCH>(stage_base, y + origin, a.out_features, row_end - row_start, a.out_features - n0, tid,
                                       THREADS, fuse ? a.y + origin : nullptr);
    } else {
        if (wave_active) {
            const int64_t origin = static_cast<int64_t>(wave_row) * a.out_features + n0;
            store_rows_32x128<STAGE_PITCH, false, true>(stage_base + wave * (32 * STAGE_PITCH), acc, y + origin, a.out_features,
                                                        row_end - wave_row, a.out_features - n0, lane,
                                                        fuse ? a.y + origin : nullptr);
        }
    }
}

template <int TYPE>
TGO_DEVICE void forward_half_any_task(const ForwardArgs & a, HalfLds<TYPE> & lds, int n_tile, bool second, int expert,
                                      int row_start, int row_end) {
    const bool narrow = row_end - row_start <= 32;
    if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
        if (a.wide != 0) {
            if (narrow) {
                forward_half_task<TYPE, true, true>(a, lds, n_tile, second, expert, row_start, row_end);
            } else {
                forward_half_task<TYPE, false, true>(a, lds, n_tile, second, expert, row_start, row_end);
            }
            return;
        }
    }
    if (narrow) {
        forward_half_task<TYPE, true, false>(a, lds, n_tile, second, expert, row_start, row_end);
    } else {
        forward_half_task<TYPE, false, false>(a, lds, n_tile, second, expert, row_start, row_end);
    }
}

template <int TYPE>
__global__ __launch_bounds__(HalfShape<TYPE>::THREADS, 2) void mmq_forward_half_kernel(const ForwardArgs a) {
    __shared__ HalfLds<TYPE> lds;
    int n_tile, expert, row_start, row_end;
    bool second;
    if (!forward_pick(a, n_tile, second, expert, row_start, row_end)) {
        return;
    }
    forward_half_any_task<TYPE>(a, lds, n_tile, second, expert, row_start, row_end);
}

// Fused SwiGLU: the gate tile goes to a.y as usual; the up pass of the same workgroup reads it back in its epilogue,
// element for element by the thread that stored it, and writes swiglu(gate, up) to a.y_second.  A thread's own
// stores and loads of one address stay ordered once the stores have left the wave (the release fence waits for
// that), and the CU's vector cache is coherent for its own waves.
template <int TYPE>
__global__ __launch_bounds__(HalfShape<TYPE>::THREADS, 2) void mmq_forward_half_swiglu_kernel(const ForwardArgs a) {
    __shared__ HalfLds<TYPE> lds;
    int n_tile, expert, row_start, row_end;
    bool second;
    if (!forward_pick(a, n_tile, second, expert, row_start, row_end)) {
        return;
    }
#pragma unroll 1
    for (int pass = 0; pass < 2; ++pass) {
        forward_half_any_task<TYPE>(a, lds, n_tile, pass == 1, expert, row_start, row_end);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
    }
}

template <int TYPE>
static hipError_t launch_forward_half_typed(const ForwardArgs & args, hipStream_t stream) {
    const int64_t total = static_cast<int64_t>(args.n_tiles) * args.projections *
                          (args.task_count != nullptr ? xcd_chunk_slots(args.task_slots) : pad_task_slots(args.task_slots, FWD_XCD_RUN));
    if (total <= 0 || total > 0x7fffffffLL) {
        return hipErrorInvalidValue;
    }
    const ProfileScope scope(2, stream);
    if (args.swiglu != 0) {
        mmq_forward_half_swiglu_kernel<TYPE><<<static_cast<unsigned>(total), HalfShape<TYPE>::THREADS, 0, stream>>>(args);
    } else {
        mmq_forward_half_kernel<TYPE><<<static_cast<unsigned>(total), HalfShape<TYPE>::THREADS, 0, stream>>>(args);
    }
    return hipGetLastError();
}

hipError_t launch_forward_half(const ForwardArgs & args, int quant_type, hipStream_t stream) {
    switch (quant_type) {
        case Q3_K: return launch_forward_half_typed<Q3_K>(args, stream);
        case Q4_K: return launch_forward_half_typed<Q4_K>(args, stream);
        case Q5_K: return launch_forward_half_typed<Q5_K>(args, stream);
        case Q6_K: return launch_forward_half_typed<Q6_K>(args, stream);
        case IQ2_S: return launch_forward_half_typed<IQ2_S>(args, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace tgo
