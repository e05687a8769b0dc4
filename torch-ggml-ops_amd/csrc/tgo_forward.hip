// Forward kernels: q8_1 activations x packed GGUF weights on gfx950 int8 MFMA.
//
// y[r, n] = sum over 32-value blocks b of  ws[n, b] * dx[r, b] * dot_b(qx[r], v[n]) - wm[n, b] * sx[r, b]
// where v is the int8 weight operand (decode16_int8), ws/wm its fp32 block scale/min
// (forward_block_scale), qx/dx/sx the q8_1 activation block.  One v_mfma_i32_32x32x32_i8 is exactly one
// 32-value block for a 32(r) x 32(n) output tile, so every MFMA result is scaled and added to the fp32
// accumulators right away; that scaling (two VALU operations per output and block), not the MFMA, bounds
// the kernel.
//
// Work split.  A workgroup owns 128 weight rows and 32 activation rows per wave; wave w owns activation
// rows [32w, 32w+32) and all 128 weight rows (1 x 4 MFMA tiles, 64 accumulator registers).  Weights: each
// super-block column of the 128 rows is staged in LDS as raw bytes, unpacked once into int8 in MFMA
// fragment order and shared by the waves.  Activations: the quantizer already wrote them in fragment order,
// so each lane fetches its 16 bytes per block straight from global memory with a fully coalesced load and
// reuses them for four MFMAs.  The activations are the A operand: a lane then owns one weight row per tile
// (scale and min are lane scalars, one 4-byte LDS read each) and 16 activation rows, whose scales come
// from an LDS copy with four 16-byte reads per block, reused by the four tiles.
//
// Latency.  A global load takes microseconds here while a wave spends about 0.2 us per block, so nothing
// is loaded where it is used: every load is issued a whole super-block ahead into registers that stay
// allocated (no spills: a scratch reload would wait on the same counter as the prefetches and serialise
// them), which is why a wave may use up to 256 registers and a SIMD holds two waves.
#include <type_traits>

#include "tgo_device.h"
#include "tgo_forward_args.h"
#include "tgo_launch.h"

namespace tgo {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// Waves per workgroup; each owns 32 activation rows.  Single-plane formats need about 72 KiB of LDS, so two
// 4-wave workgroups share a CU; two-plane formats need about 100 KiB and run one 8-wave workgroup per CU.
// Either way a SIMD holds two waves of up to 256 registers.
template <int TYPE>
struct ForwardShape {
    static constexpr int WAVES = Format<TYPE>::PLANES == 1 ? 4 : 8;
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int ROWS = 32 * WAVES;
    static constexpr int DX_PITCH = ROWS + 4;  // floats per block row of the activation-scale copy
};

// LDS of one workgroup.
template <int TYPE>
struct ForwardLds {
    static constexpr int RAW_SLOT = Format<TYPE>::BLOCK_BYTES % 16 == 0 || Format<TYPE>::RAW_PITCH > WideStage<TYPE>::PITCH
                                        ? Format<TYPE>::RAW_PITCH : WideStage<TYPE>::PITCH;
    alignas(16) uint8_t raw[FWD_TN * RAW_SLOT];                        // packed blocks of one super-block column
    alignas(16) uint8_t wq[Format<TYPE>::PLANES][FWD_TN * 256];        // int8 weight operand in fragment order
    alignas(16) float ws[8][FWD_TN];                                   // block scales
    alignas(16) float wm[Format<TYPE>::HAS_MIN ? 8 : 1][FWD_TN];       // block minima
    alignas(16) float dxs[2][8][ForwardShape<TYPE>::DX_PITCH];         // activation scales, two copies
    uint2 grid[TYPE == IQ2_S ? TGO_IQ2S_GRID_ENTRIES : 1];
};

// WIDE (formats whose blocks are not multiples of 16 bytes): the packed blocks are prefetched into registers as
// aligned units like those of Q4_K / Q5_K (wide_fetch) instead of being copied two bytes at a time when needed.
template <int TYPE, bool NARROW, bool WIDE>
TGO_DEVICE void forward_task(const ForwardArgs & a, ForwardLds<TYPE> & lds, int n_tile, bool second, int expert,
                             int row_start, int row_end) {
    using F = Format<TYPE>;
    using S = ForwardShape<TYPE>;
    constexpr int PLANES = F::PLANES;
    constexpr int THREADS = S::THREADS;
    auto & raw = lds.raw;
    auto & wq = lds.wq;
    auto & ws = lds.ws;
    auto & wm = lds.wm;
    auto & dxs = lds.dxs;
    auto & grid = lds.grid;
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
        expand_iq2s_grid(grid, tid, THREADS);
    }

    // this wave's 32 activation rows (NARROW: every wave takes the task's only 32 rows and weight tile number
    // `wave`); loads of rows past the padded workspace are clamped (their results are never stored)
    constexpr bool narrow = NARROW;
    const int granule = narrow ? 0 : wave;
    const int wave_row = row_start + granule * 32;
    const bool wave_active = wave_row < row_end;
    int lane_row = wave_row + l32;
    lane_row = lane_row < a.rows_padded ? lane_row : a.rows_padded - 1;
    // Every global address below is a uniform 64-bit base, advanced with scalar arithmetic, plus a 32-bit lane
    // offset: the loads then take the base from scalar registers and no 64-bit (quarter-rate) vector arithmetic
    // is left in the loop.  The host checks that the offsets fit (row_bytes and rows_padded below 2^24).
    const int first_tile = row_start >> 5;
    const int8_t * const qx_task = a.qx + static_cast<int64_t>(first_tile) * blocks_per_row * 1024;
    const uint32_t x_lane_offset = static_cast<uint32_t>((lane_row >> 5) - first_tile) * blocks_per_row * 1024u +
                                   static_cast<uint32_t>(((lane_row & 31) + 32 * half) * 16);
    const uint32_t sum_lane_offset = (__umul24(half, a.rows_padded) + lane_row) * 4u;
    const uint8_t * const tile_weights = weights + static_cast<int64_t>(n0) * a.row_bytes;
    const int tile_rows = min(FWD_TN, a.out_features - n0);   // weight rows of this tile that exist

    // Everything that comes from global memory is fetched one super-block (eight MFMA steps, several
    // microseconds) before it is needed and parked in registers: the packed weights and activation scales
    // the workgroup stages in LDS, and this wave's activation fragments and sums.
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
    // (`t` is the thread id: the main loop passes a copy the compiler cannot see through, so that the small
    // address computations below are redone per round instead of being kept alive, and spilled, across it)
    // (unit id -> weight row by a 24-bit multiply and a shift, exact for the few thousand ids of a tile)
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
    auto store_raw = [&](int kb, int t) {
        if constexpr (RAW_IN_REGS) {
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = min(t + THREADS * i, FWD_TN * RAW_UNITS - 1);
                const int row = static_cast<int>(__umul24(id, UNIT_RECIPROCAL) >> 16);
                const int unit = id - row * RAW_UNITS;
                uint32_t * dst = reinterpret_cast<uint32_t *>(raw + row * F::RAW_PITCH + unit * 16);
                dst[0] = raw_next[i].x; dst[1] = raw_next[i].y; dst[2] = raw_next[i].z; dst[3] = raw_next[i].w;
            }
        } else if constexpr (WIDE) {
            wide_park<TYPE, FWD_TN, THREADS, WIDE_REGS>(raw, wide_next, tile_weights, static_cast<int>(a.row_bytes), tile_rows, kb, t);
        } else {
            stage_blocks<TYPE>(raw, weights, a.row_bytes, n0, a.out_features, kb, FWD_TN, t, THREADS);
        }
    };

    // activation scales: one thread covers four consecutive rows of one of the eight blocks
    float dx_next[4];
    auto load_dx = [&](int kb, int t) {
        const int dx_block = t / (S::ROWS / 4);
        const int dx_row = (t - dx_block * (S::ROWS / 4)) * 4;
        const float * base = a.dx + static_cast<int64_t>(kb) * 8 * a.rows_padded;
        const uint32_t block_offset = __umul24(dx_block, a.rows_padded);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = min(row_start + dx_row + e, a.rows_padded - 1);
            dx_next[e] = *reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(base) + (block_offset + row) * 4u);
        }
    };

    // activation fragments: block i of the row lives in x[i % X_AHEAD] and is fetched X_AHEAD blocks ahead
    constexpr int X_AHEAD = PLANES == 1 ? 4 : 8;
    v4i x[X_AHEAD];
    float sum_next[4];
    auto load_x = [&](int block) {
        const int clamped = block < blocks_per_row ? block : blocks_per_row - 1;
        x[block % X_AHEAD] = *reinterpret_cast<const v4i *>(qx_task + static_cast<int64_t>(clamped) * 1024 + x_lane_offset);
    };
    auto load_sums = [&](int kb) {
        if constexpr (F::HAS_MIN) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float * base = a.sx + static_cast<int64_t>(kb * 8 + 2 * j) * a.rows_padded;
                sum_next[j] = *reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(base) + sum_lane_offset);
            }
        }
    };

    load_raw(0, tid);
    load_dx(0, tid);
    if (wave_active) {
        load_sums(0);
#pragma unroll
        for (int b = 0; b < X_AHEAD; ++b) {
            load_x(b);
        }
    }

    v16f acc[FWD_NT];
#pragma unroll
    for (int nt = 0; nt < FWD_NT; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[nt][v] = 0.0f;

    // Int-to-float without a convert: the MFMA adds the dot product to the bit pattern of 1.5 * 2^23, whose
    // float value is then exactly BIAS + dot (|dot| < 2^22 for the single-plane types).  The weight scale
    // ws = d * sc (or +-d) has at most 17 significant bits, so BIAS * ws is exact and
    // fma(BIAS + dot, ws, -BIAS * ws) = dot * ws rounded once.
    constexpr bool BIASED = PLANES == 1;
    constexpr float BIAS = 12582912.0f;
    const int seed = BIASED ? 0x4b400000 : 0;
    const v16i dot_init = {seed, seed, seed, seed, seed, seed, seed, seed, seed, seed, seed, seed, seed, seed, seed, seed};

    // The loop exists twice, for waves with and without activation rows, instead of branching around the
    // MFMA part inside one loop: with a branch in the body the compiler's wait-count bookkeeping merges
    // both paths and ends up waiting for every outstanding load, prefetches included, once per round.
    // mode 0: no rows for this wave; 1: four weight tiles per wave; 2: narrow, weight tile number `wave` only
    auto main_loop = [&](auto mode_tag) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr bool ACTIVE = MODE != 0;
    constexpr int TILES = MODE == 2 ? 1 : FWD_NT;
    auto tile_of = [&](int index) { return MODE == 2 ? wave : index; };
#pragma unroll 1
    for (int kb = 0; kb < super_blocks; ++kb) {
        // Two barriers per super-block.  `raw` is rewritten here while no wave can still be unpacking it
        // (all passed the second barrier of the previous round); the activation scales alternate between
        // two copies because slower waves may still be reading the previous one.
        const int buffer = kb & 1;
        int t = tid;
        asm volatile("" : "+v"(t));
        store_raw(kb, t);
        *reinterpret_cast<float4 *>(&dxs[buffer][t / (S::ROWS / 4)][(t % (S::ROWS / 4)) * 4]) =
            make_float4(dx_next[0], dx_next[1], dx_next[2], dx_next[3]);
        __syncthreads();
        // The unpack below is a chain of LDS round trips with little arithmetic; the other workgroup of the CU is
        // usually in its scaling loop, which would fill every issue slot.  The chain's waves go first (measured:
        // Q5_K forward 2.5 % faster, Q6_K 2.4 %, nothing for the other formats).
        __builtin_amdgcn_s_setprio(3);

        // the last round re-fetches its own super-block instead of branching around the prefetch
        const int kb_next = kb + 1 < super_blocks ? kb + 1 : kb;
        load_raw(kb_next, t);
        load_dx(kb_next, t);

        // unpack: 128 rows x 16 units; consecutive lanes take consecutive rows of one unit, so the
        // 16-byte stores of a half-wave fill one contiguous 512-byte fragment slab.  A thread keeps its weight
        // row and walks the units in steps of THREADS / 128, so that the row's LDS address, the unit's parity
        // and, with the loop unrolled, most shift counts of the decoders are fixed.
        {
            constexpr int UNIT_STEP = THREADS / FWD_TN;
            const uint32_t row = static_cast<uint32_t>(t) & (FWD_TN - 1);
            // (masked so that the compiler knows the range: unit numbers first_unit + UNIT_STEP * j then split into a
            // run-time part and constants, and most of the decoders' offset arithmetic folds away)
            const uint32_t first_unit = (static_cast<uint32_t>(t) / FWD_TN) & (UNIT_STEP - 1);
            const uint8_t * blk = raw + row * SLOT_PITCH + SLOT_FRONT;
            const uint32_t row_slot = ((row >> 5) * 8 * 64 + (row & 31)) * 16;
            if constexpr ((TYPE == Q4_K || TYPE == Q5_K) && UNIT_STEP == 2) {
                // The thread's units are the same 16-value half (first_unit) of all eight 32-value groups, so
                // the group number is the loop counter: nibble select and bit-plane shift are immediates, the
                // 16 bytes of Q5_K's fifth bits are read once for all groups.
                constexpr int QS = TYPE == Q4_K ? 16 : 48;
                const uint8_t * half_blk = blk + 16 * first_unit;
                const uint32_t half_slot = row_slot + 32 * 16 * first_unit;
                uint32_t planes[4] = {0, 0, 0, 0};
                if constexpr (TYPE == Q5_K) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        planes[w] = lds_u32(half_blk + 16 + 4 * w);
                    }
                }
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    uint32_t lo[4];
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        lo[w] = (lds_u32(half_blk + QS + (g >> 1) * 32 + 4 * w) >> (4 * (g & 1))) & 0x0f0f0f0fu;
                        if constexpr (TYPE == Q5_K) {
                            lo[w] |= ((planes[w] >> g) & 0x01010101u) << 4;
                        }
                    }
                    *reinterpret_cast<uint4 *>(&wq[0][half_slot + g * 64 * 16]) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 16 / UNIT_STEP; ++j) {
                    const uint32_t unit = first_unit + UNIT_STEP * j;
                    uint32_t lo[4], hi[4];
                    decode16_int8<TYPE>(blk, unit, grid, lo, hi);
                    const uint32_t slot = row_slot + ((unit >> 1) * 64 + 32 * (unit & 1)) * 16;
                    *reinterpret_cast<uint4 *>(&wq[0][slot]) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                    if constexpr (PLANES == 2) {
                        *reinterpret_cast<uint4 *>(&wq[1][slot]) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 8 / UNIT_STEP; ++j) {
                const uint32_t b = first_unit + UNIT_STEP * j;
                float scale, minimum;
                forward_block_scale<TYPE>(blk, b, scale, minimum);
                ws[b][row] = scale;
                if constexpr (F::HAS_MIN) {
                    wm[b][row] = minimum;
                }
            }
        }
        __builtin_amdgcn_s_setprio(0);
        __syncthreads();

        if constexpr (ACTIVE) {
            if constexpr (F::HAS_MIN) {
                // acc[r][n] -= sum_b sx[r][b] * wm[n][b]: eight blocks = four fp32 MFMAs of depth 2 per tile
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float minus_sum = -sum_next[j];
#pragma unroll
                    for (int nt = 0; nt < TILES; ++nt) {
                        acc[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            minus_sum, wm[2 * j + half][tile_of(nt) * 32 + l32], acc[nt], 0, 0, 0);
                    }
                }
                load_sums(kb_next);
            }

            if constexpr (PLANES == 1) {
                // Software pipeline over the 8 x TILES (block, tile) steps of the super-block.  The LDS reads of
                // step t + 2 and the MFMA of step t + 1 are issued ahead of the 33 vector operations that
                // consume step t, so that neither an LDS round trip nor the MFMA latency sits between a
                // wave's vector operations; the scheduling barriers keep the stages where they are written.
                v4i w_frag[3];
                float w_scale[3];
                float dxv[3][16];   // scales of the 16 activation rows of this lane's results, by block number mod 3
                                    // (read two steps ahead, and a block may last a single step)
                v16i dot[2];
                constexpr int STEPS = 8 * TILES;
                auto read_step = [&](int t) {
                    const int b = t / TILES, nt = tile_of(t % TILES);
                    w_frag[t % 3] = *reinterpret_cast<const v4i *>(&wq[0][((nt * 8 + b) * 64 + lane) * 16]);
                    w_scale[t % 3] = ws[b][nt * 32 + l32];
                    if (t % TILES == 0) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {   // rows 8j + 4*half + (0..3) of the wave's granule
                            const float4 d4 =
                                *reinterpret_cast<const float4 *>(&dxs[buffer][b][granule * 32 + 8 * j + 4 * half]);
                            dxv[b % 3][4 * j + 0] = d4.x; dxv[b % 3][4 * j + 1] = d4.y;
                            dxv[b % 3][4 * j + 2] = d4.z; dxv[b % 3][4 * j + 3] = d4.w;
                        }
                    }
                };
                read_step(0);
                read_step(1);
                dot[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x[0], w_frag[0], dot_init, 0, 0, 0);
                const int block0 = kb * 8;
#pragma unroll
                for (int t = 0; t < STEPS; ++t) {
                    if (t + 2 < STEPS) {
                        read_step(t + 2);
                    }
                    if (t + 1 < STEPS) {
                        dot[(t + 1) & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(
                            x[((t + 1) / TILES) % X_AHEAD], w_frag[(t + 1) % 3], dot_init, 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    const float scale = w_scale[t % 3];
                    const float bias_scale = -BIAS * scale;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const float scaled = fmaf(__int_as_float(dot[t & 1][v]), scale, bias_scale);
                        acc[t % TILES][v] = fmaf(scaled, dxv[(t / TILES) % 3][v], acc[t % TILES][v]);
                    }
                    if (t % TILES == TILES - 1) {
                        // block t / TILES is done (its last MFMA has been issued): its registers take the
                        // block X_AHEAD further on
                        load_x(block0 + t / TILES + X_AHEAD);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                // Two planes: the weight scale is one number per weight row and super-block (the integer sub-scales
                // are inside the int8 planes), so it is applied once per super-block instead of once per block.  For
                // that the matrix instructions run with the operands swapped: a lane then holds one activation row
                // (its eight block scales are eight registers) and 16 weight rows per tile, and per result and block
                // three vector instructions are left: combine the planes, convert, multiply-add with the
                // activation scale.
                float dxb[8];
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    dxb[b] = dxs[buffer][b][wave * 32 + l32];
                }
                // The 32 (tile, block) steps as a software pipeline, like the single-plane loop: the two fragments of
                // step t + 2 are read from LDS and the two matrix instructions of step t + 1 issued before the 48
                // vector instructions of step t, so that neither an LDS round trip nor the matrix latency sits
                // between a wave's vector instructions.
                constexpr int STEPS = 8 * FWD_NT;
                constexpr int RING = 3;   // fragment sets: of the step being read, the one being multiplied and the one being scaled
                v4i w_lo[RING], w_hi[RING];
                v16i dot_lo[2], dot_hi[2];
                v16f within;
                auto read_step = [&](int step) {
                    const int nt = step / 8, b = step % 8;
                    const int slot = ((nt * 8 + b) * 64 + lane) * 16;
                    w_lo[step % RING] = *reinterpret_cast<const v4i *>(&wq[0][slot]);
                    w_hi[step % RING] = *reinterpret_cast<const v4i *>(&wq[PLANES - 1][slot]);
                };
                auto multiply_step = [&](int step) {
                    dot_lo[step & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w_lo[step % RING], x[step % 8], dot_init, 0, 0, 0);
                    dot_hi[step & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w_hi[step % RING], x[step % 8], dot_init, 0, 0, 0);
                };
                read_step(0);
                read_step(1);
                multiply_step(0);
#pragma unroll
                for (int step = 0; step < STEPS; ++step) {
                    const int nt = step / 8, b = step % 8;
                    if (step + 2 < STEPS) {
                        read_step(step + 2);
                    }
                    if (step + 1 < STEPS) {
                        multiply_step(step + 1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (b == 0) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) within[v] = 0.0f;
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        within[v] = fmaf(static_cast<float>(dot_lo[step & 1][v] + (dot_hi[step & 1][v] << 7)), dxb[b], within[v]);
                    }
                    if (b == 7) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {   // weight rows 8j + 4*half + (0..3) of this tile
                            const float4 d4 = *reinterpret_cast<const float4 *>(&ws[0][nt * 32 + 8 * j + 4 * half]);
                            acc[nt][4 * j + 0] = fmaf(within[4 * j + 0], d4.x, acc[nt][4 * j + 0]);
                            acc[nt][4 * j + 1] = fmaf(within[4 * j + 1], d4.y, acc[nt][4 * j + 1]);
                            acc[nt][4 * j + 2] = fmaf(within[4 * j + 2], d4.z, acc[nt][4 * j + 2]);
                            acc[nt][4 * j + 3] = fmaf(within[4 * j + 3], d4.w, acc[nt][4 * j + 3]);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // the super-block is done: fetch the next one's activation fragments
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    load_x(kb * 8 + b + X_AHEAD);
                }
            }
        }
    }
    };
    if constexpr (narrow) {
        main_loop(std::integral_constant<int, 2>{});
    } else {
        if (wave_active) {
            main_loop(std::integral_constant<int, 1>{});
        } else {
            main_loop(std::integral_constant<int, 0>{});
        }
    }
    __syncthreads();
    if constexpr (narrow) {
        // the four tiles of the task's 32 x 128 block meet in LDS and leave as whole rows
        uint16_t * block = reinterpret_cast<uint16_t *>(&wq[0][0]);
        stage_tile_32x32<128>(block, acc[0], wave * 32, lane);
        __syncthreads();
        const int64_t origin = static_cast<int64_t>(row_start) * a.out_features + n0;
        store_staged_rows<128>(block, y + origin, a.out_features, row_end - row_start, a.out_features - n0, tid,
                               THREADS, fuse ? a.y + origin : nullptr);
        return;
    } else {

    // The weight tile is free now: the waves transpose their 32 x 128 results through it (8 KiB each, four
    // waves at a time) so that the output is written in whole 256-byte rows.
    // (the two-plane formats hold transposed results, which need padded rows in the staging area: their weight
    // tile has a second plane's worth of room)
    constexpr bool TRANSPOSED = PLANES == 2;
    constexpr int STAGE_PITCH = TRANSPOSED ? 136 : 128;
    static_assert(FWD_TN == 128 && sizeof(wq) >= 4 * 32 * STAGE_PITCH * sizeof(uint16_t), "stage fits the weight tile");
    uint16_t * stage = reinterpret_cast<uint16_t *>(&wq[0][0]) + (wave & 3) * (32 * STAGE_PITCH);
#pragma unroll
    for (int round = 0; round < S::WAVES / 4; ++round) {
        if ((wave >> 2) == round && wave_active) {
            const int64_t origin = static_cast<int64_t>(wave_row) * a.out_features + n0;
            store_rows_32x128<STAGE_PITCH, false, TRANSPOSED>(stage, acc, y + origin, a.out_features, row_end - wave_row,
                                                             a.out_features - n0, lane, fuse ? a.y + origin : nullptr);
        }
        if (round + 1 < S::WAVES / 4) {
            __syncthreads();
        }
    }
    }
}

// A task of at most 32 rows has work for one wave only in the usual split (a wave = 32 rows x 128 weight
// rows).  Such tasks are common under skewed routing, so for them the four waves of a single-plane
// workgroup take one of the four 32-row weight tiles each instead.  The variants are separate
// instantiations of the task body so that neither's registers weigh on the other.
template <int TYPE>
TGO_DEVICE void forward_any_task(const ForwardArgs & a, ForwardLds<TYPE> & lds, int n_tile, bool second, int expert,
                                 int row_start, int row_end) {
    constexpr bool SINGLE = Format<TYPE>::PLANES == 1;
    const bool narrow = SINGLE && row_end - row_start <= 32;
    if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
        if (a.wide != 0) {
            if (narrow) {
                forward_task<TYPE, SINGLE, true>(a, lds, n_tile, second, expert, row_start, row_end);
            } else {
                forward_task<TYPE, false, true>(a, lds, n_tile, second, expert, row_start, row_end);
            }
            return;
        }
    }
    if (narrow) {
        forward_task<TYPE, SINGLE, false>(a, lds, n_tile, second, expert, row_start, row_end);
    } else {
        forward_task<TYPE, false, false>(a, lds, n_tile, second, expert, row_start, row_end);
    }
}

template <int TYPE>
__global__ __launch_bounds__(ForwardShape<TYPE>::THREADS, 2) void mmq_forward_kernel(const ForwardArgs a) {
    using F = Format<TYPE>;
    using S = ForwardShape<TYPE>;
    constexpr int PLANES = F::PLANES;
    static_assert(S::ROWS == forward_row_tile(TYPE, OPERAND_INT8), "task rows match the workgroup");
    __shared__ ForwardLds<TYPE> lds;

    int n_tile, expert, row_start, row_end;
    bool second;
    if (!forward_pick(a, n_tile, second, expert, row_start, row_end)) {
        return;
    }
    forward_any_task<TYPE>(a, lds, n_tile, second, expert, row_start, row_end);
}

// Fused SwiGLU, its own kernel so that the plain forward's register allocation is untouched.  The gate tile
// goes to a.y as usual; the up pass of the same workgroup reads it back in its epilogue, element for element
// by the thread that stored it, and writes swiglu(gate, up) to a.y_second.  A thread's own stores and loads of
// one address stay ordered once the stores have left the wave (the release fence waits for that), and the
// CU's vector cache is coherent for its own waves.
template <int TYPE>
__global__ __launch_bounds__(ForwardShape<TYPE>::THREADS, 2) void mmq_forward_swiglu_kernel(const ForwardArgs a) {
    constexpr int PLANES = Format<TYPE>::PLANES;
    __shared__ ForwardLds<TYPE> lds;

    int n_tile, expert, row_start, row_end;
    bool second;
    if (!forward_pick(a, n_tile, second, expert, row_start, row_end)) {
        return;
    }
#pragma unroll 1
    for (int pass = 0; pass < 2; ++pass) {
        forward_any_task<TYPE>(a, lds, n_tile, pass == 1, expert, row_start, row_end);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
    }
}

template <int TYPE>
static hipError_t launch_forward_typed(const ForwardArgs & args, hipStream_t stream) {
    const int64_t total = static_cast<int64_t>(args.n_tiles) * args.projections *
                          (args.task_count != nullptr ? xcd_chunk_slots(args.task_slots) : pad_task_slots(args.task_slots, FWD_XCD_RUN));
    if (total <= 0 || total > 0x7fffffffLL) {
        return hipErrorInvalidValue;
    }
    const ProfileScope scope(2, stream);
    if (args.swiglu != 0) {
        mmq_forward_swiglu_kernel<TYPE><<<static_cast<unsigned>(total), ForwardShape<TYPE>::THREADS, 0, stream>>>(args);
    } else {
        mmq_forward_kernel<TYPE><<<static_cast<unsigned>(total), ForwardShape<TYPE>::THREADS, 0, stream>>>(args);
    }
    return hipGetLastError();
}

static hipError_t launch_forward(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                                 const Q8Workspace & ws, uint16_t * output, uint16_t * output_second,
                                 const TaskList * tasks, int rows, int in_features, int out_features,
                                 int quant_type, hipStream_t stream, bool swiglu) {
    if (ws.by_rows()) {
        return hipErrorInvalidValue;   // this kernel reads the tile-ordered activation layout
    }
    if (ws.rows_padded >= (1 << 24) || in_features >= (1 << 24)) {
        return hipErrorInvalidValue;   // lane offsets are formed with 24-bit multiplies
    }
    ForwardArgs args = {};
    args.packed = packed;
    args.packed_second = packed_second;
    args.y_second = output_second;
    args.swiglu = swiglu && packed_second != nullptr ? 1 : 0;
    args.projections = packed_second != nullptr && args.swiglu == 0 ? 2 : 1;
    args.bytes_per_expert = bytes_per_expert;
    args.row_bytes = static_cast<int64_t>(in_features / QK_K) * block_bytes(quant_type);
    // (a dense call has one "expert": the whole weight)
    const int64_t weight_bytes = static_cast<int64_t>(out_features) * args.row_bytes;
    args.wide = wide_stage_ok(packed, weight_bytes) && (packed_second == nullptr || wide_stage_ok(packed_second, weight_bytes)) ? 1 : 0;
    args.qx = ws.q;
    args.dx = ws.d;
    args.sx = ws.sum;
    args.power = ws.power;
    args.row_power = ws.row_power;
    args.block_sums = ws.block_sums;
    args.y = output;
    args.rows = rows;
    args.rows_padded = static_cast<int>(ws.rows_padded);
    args.in_features = in_features;
    args.out_features = out_features;
    args.n_tiles = (out_features + FWD_TN - 1) / FWD_TN;
    if (tasks != nullptr) {
        args.task_count = tasks->count;
        args.task_early = tasks->early;
        args.task_cursor = tasks->cursor;
        args.task_expert = tasks->expert;
        args.task_row_start = tasks->row_start;
        args.task_row_end = tasks->row_end;
        args.task_slots = tasks->max_tasks;
        args.dense_row_tile = forward_row_tile(quant_type, ws.operand_kind());
    } else {
        args.task_count = nullptr;
        args.task_early = nullptr;
        args.task_cursor = nullptr;
        args.task_expert = nullptr;
        args.task_row_start = nullptr;
        args.task_row_end = nullptr;
        // A dense call whose full tiles would not even give every second CU a workgroup runs as smaller tiles.
        // Single-plane formats: 32 rows, i.e. the kernel's narrow variant, whose four waves split the weight rows
        // (four times the workgroups, each about a third as long).  The two-plane formats have no narrow variant,
        // but their eight waves own 32 rows each: with tiles of 128, 64 or 32 rows only 4, 2 or 1 of them multiply
        // (the others still help to unpack), the vector work of a tile no longer queues two waves deep on every
        // SIMD, and there are 2, 4 or 8 times the workgroups; the largest tile that yields 128 workgroups is taken.
        int row_tile = forward_row_tile(quant_type, ws.operand_kind());
        const auto tiles = [&](int tile) { return static_cast<int64_t>(args.n_tiles) * ((rows + tile - 1) / tile); };
        if (row_tile == 128) {
            if (tiles(128) <= 128) {
                row_tile = 32;
            }
        } else {
            while (row_tile > 32 && tiles(row_tile) < 128) {
                row_tile /= 2;
            }
        }
        args.dense_row_tile = row_tile;
        args.task_slots = (rows + row_tile - 1) / row_tile;
    }
    if (ws.scaled_tiles()) {
        return launch_forward_scaled(args, quant_type, stream);
    }
    if (ws.half_tiles()) {
        return launch_forward_half(args, quant_type, stream);
    }
    switch (quant_type) {
        case Q3_K: return launch_forward_typed<Q3_K>(args, stream);
        case Q4_K: return launch_forward_typed<Q4_K>(args, stream);
        case Q5_K: return launch_forward_typed<Q5_K>(args, stream);
        case Q6_K: return launch_forward_typed<Q6_K>(args, stream);
        case IQ2_S: return launch_forward_typed<IQ2_S>(args, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_mmq_forward(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                              const Q8Workspace & ws, uint16_t * output, uint16_t * output_second,
                              const TaskList * tasks, int rows, int in_features, int out_features,
                              int quant_type, hipStream_t stream) {
    return launch_forward(packed, packed_second, bytes_per_expert, ws, output, output_second, tasks, rows,
                          in_features, out_features, quant_type, stream, false);
}

hipError_t launch_mmq_forward_swiglu(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                                     const Q8Workspace & ws, uint16_t * output, uint16_t * output_second,
                                     const TaskList * tasks, int rows, int in_features, int out_features,
                                     int quant_type, hipStream_t stream) {
    if (packed_second == nullptr || output_second == nullptr) {
        return hipErrorInvalidValue;
    }
    return launch_forward(packed, packed_second, bytes_per_expert, ws, output, output_second, tasks, rows,
                          in_features, out_features, quant_type, stream, true);
}

}  // namespace tgo
