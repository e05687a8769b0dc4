// Forward kernel with scaled fp16 operands: q8_1 activations x packed GGUF weights as one fp16 matrix product per
// task, bounded by the matrix pipe instead of the vector pipe.
//
//   y[r, n] = 2^(E[r] + S[n]) * sum over k of  w[n, k] * h[r, k]      (v_mfma_f32_32x32x16_f16, fp32 accumulation)
//   h[r, k] = fp16(dx * qx * 2^-e[r, s]) * 2^(e[r, s] - E[r])   the dequantized q8_1 activation, rounded once after a
//             normalisation per row and super-block s, then brought to the row's common exponent (exact)
//   w[n, k] = fp16(v[n, k] * fp16(scale * 2^-S[n]))   the integer operand v = sub-scale x quant (exact in fp16) times
//             the weight scale of its group, normalised per weight row
// Q4_K/Q5_K: v = q, scale = d * sc, and the minimum term -dmin * m * (block sum) is one more reduction step per
// super-block whose operands are fp16(-dmin * m * 2^-S[n]) and the block sum treated like h.  The quantizer writes
// the normalised values and block sums, 2^(e - E) and 2^E (quantize_q8_1_scaled_kernel, scaled_row_power_kernel);
// S[n] comes from a scan of the weight row's super-block scales.
// The algebra is the q8_1 one (same quants, block scales and sums as the int8 kernels of tgo_forward.hip); what
// differs is that both operands carry their scales into the matrix instruction, each rounded to fp16 once (relative
// 2^-11: the reference keeps its own scale products d * sc and dmin * m as halves too,
// csrc/vendor/llama_cpp/mmq-load-targets.cuh:190-195), so that no vector instruction touches a result between the
// first and the last reduction step.  The int8 kernels spend two or three vector operations per result on every 32
// values, which bounds them at a quarter of the matrix pipe's rate.
//
// Work split: role-split workgroup of twelve waves, one per CU.  Waves 0-7 multiply: wave w owns activation rows
// [32w, 32w + 32) of the task and all 128 weight rows of the column tile (1 x 4 tiles of 32 x 32, 64 accumulator
// registers; the weights are the A operand, so a lane holds one activation row and 16 weight rows per tile).
// Waves 8-11 unpack: wave 8 + t owns weight rows [32t, 32t + 32) from the global load of their packed blocks to
// their fp16 operand tile (packed blocks RAW_DEPTH super-blocks ahead in registers, parked in the wave's own LDS
// slot; LDS executes a wave's accesses in order, so these steps need no workgroup barrier).  Each SIMD then holds two
// waves that feed the matrix pipe and one that keeps the vector pipe busy.  A super-block is two stages of 128
// values; the operand tile of a stage (32 KiB, fragment order) goes through a ring of three buffers.  No workgroup
// barrier hands a buffer over: every unpacking wave counts the stages it has written and every multiplying wave the
// stages it has read, in LDS; a multiplier starts stage g when all four unpackers have counted g + 1, an unpacker
// overwrites the buffer of stage g - 3 when all eight multipliers have counted g - 2.  (A barrier per stage makes
// every stage as long as its slowest wave: twelve waves with memory latencies of their own then wait a quarter of
// the time.)  LDS executes a wave's accesses in issue order, so a counter written after the data, or after the
// last read, needs no wait of its own.
//
// A workgroup is persistent: it owns every n-th (task, column tile) item of the launch, n being the number of role-split
// workgroups (one per CU), and runs their super-blocks as one stream, so an item's first loads (task description, packed blocks, the scan of its scales,
// activation fragments) are requested while the item before it is still being multiplied, and its results are
// stored while the unpackers already work on the next one.  With one item per workgroup those latencies and the
// epilogue, none of them overlapped by anything on a CU that holds a single workgroup, were 40 % of the kernel's time.
//
// Grouped calls keep their groups of at most 32 rows out of these workgroups: the launch ends in workgroups that run
// short_group_items() on them instead (below), and which the CUs take up as their role-split workgroup runs out of
// items: the last round of role-split items occupies a fraction of the CUs only.
#include <type_traits>

#include "tgo_device.h"
#include "tgo_forward_args.h"
#include "tgo_launch.h"

namespace tgo {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int FSC_MULTIPLIERS = 8;                         // multiplying waves, 32 activation rows each
constexpr int FSC_THREADS = 64 * (FSC_MULTIPLIERS + 4);
constexpr int FSC_STEPS = 8;                                // 16-value reduction steps per stage
constexpr int FSC_TILE_BYTES = FWD_NT * FSC_STEPS * 1024;   // fp16 operand of a stage: [tile][step][64 lanes][16 bytes]
constexpr int FSC_ROWS = 256;                               // activation rows per task
static_assert(FSC_ROWS == forward_row_tile(12, OPERAND_SCALED), "task rows match the workgroup");
constexpr int FSC_W_AHEAD = 1;                               // reduction steps a weight fragment is read ahead of its matrix instructions

constexpr int FSC_MAX_ITEMS = 64;      // items per workgroup (one wave builds the table)
constexpr int FSC_GRID = 256;          // one workgroup per CU
constexpr int FSC_BUFFERS = 3;         // operand tiles in flight between the unpacking and the multiplying waves
constexpr int FSC_SPIN_LIMIT = 1 << 20;   // polls of a stage counter before a wave gives up waiting (a few hundred ms)

struct ScaledItem {
    int expert, row_start, row_end, tile;   // tile: column tile + n_tiles * projection
};

template <int TYPE>
struct ScaledLds {
    static constexpr bool K45 = TYPE == Q4_K || TYPE == Q5_K;
    // slot of one packed block: Q4_K/Q5_K blocks are whole 16-byte units and lie back to back (16-byte reads of 32
    // consecutive rows then cover all banks); the other formats take the larger of their two staging pitches
    static constexpr int RAW_SLOT = K45 ? Format<TYPE>::BLOCK_BYTES
                                        : (Format<TYPE>::RAW_PITCH > WideStage<TYPE>::PITCH ? Format<TYPE>::RAW_PITCH
                                                                                             : WideStage<TYPE>::PITCH);
    alignas(16) uint8_t wq[FSC_BUFFERS][FSC_TILE_BYTES];       // ring of operand tiles, one stage each
    alignas(16) uint8_t raw[4][2][32 * RAW_SLOT];              // per unpacking wave: packed blocks of two super-blocks
    // fp16(-dmin * m * 2^-S): [tile][32 rows][8 blocks], beside the operand tile of the super-block's first stage
    alignas(16) uint8_t mins[FSC_BUFFERS][K45 ? FWD_NT * 512 : 16];
    // 2^S of the tile's weight rows by item & 3 (the unpackers open at most the second item after the one whose
    // results are being stored)
    alignas(16) float row_power[4][FWD_TN];
    alignas(16) int produced[4];                               // stages written, per unpacking wave
    alignas(16) int consumed[FSC_MULTIPLIERS];                 // stages read, per multiplying wave
    ScaledItem items[FSC_MAX_ITEMS];
    int item_count;
    std::conditional_t<TYPE == IQ2_S, Iq2sSelectors, uint2> codebook;
};

// 6-bit scale and minimum of 32-value group G of a Q4_K/Q5_K block from its 12 scale bytes (three words)
template <int G>
TGO_DEVICE void k45_group_scale_min(uint32_t w1, uint32_t w2, uint32_t w3, int & sc, int & mn) {
    if constexpr (G < 4) {
        sc = static_cast<int>((w1 >> (8 * G)) & 63u);
        mn = static_cast<int>((w2 >> (8 * G)) & 63u);
    } else {
        constexpr int J = G - 4;
        sc = static_cast<int>(((w3 >> (8 * J)) & 15u) | (((w1 >> (8 * J + 6)) & 3u) << 4));
        mn = static_cast<int>(((w3 >> (8 * J + 4)) & 15u) | (((w2 >> (8 * J + 6)) & 3u) << 4));
    }
}

// (1024 + byte) pairs times an fp16 multiplier h, minus the bias: fma(1024 + b, h, -1024 h) is evaluated with one
// rounding and -1024 h is a power-of-two multiple of h, so the result is fp16(b * h).
TGO_DEVICE HalfScale half_scale_of(float value) {
    const _Float16 h = static_cast<_Float16>(value);
    const _Float16 offset = static_cast<_Float16>(-1024.0f) * h;
    return HalfScale{half2_t{h, h}, half2_t{offset, offset}};
}

// Largest magnitude a weight of the format can take per unit of its super-block scale d.
template <int TYPE>
constexpr float weight_reach() {
    return TYPE == Q4_K ? 63.0f * 15.0f : TYPE == Q5_K ? 63.0f * 31.0f : TYPE == Q3_K ? 32.0f * 4.0f
           : TYPE == Q6_K ? 128.0f * 32.0f : 31.0f * 43.0f / 8.0f;
}

// Byte offset of the fp16 super-block scale d inside a block (Q4_K/Q5_K: d, then dmin).
template <int TYPE>
constexpr int scale_offset() { return TYPE == Q3_K ? 108 : TYPE == Q6_K ? 208 : 0; }


// Stores the wave's 32 rows x (32 * TILES) columns of results, which the matrix instructions left transposed (weights as the
// A operand: the lane holds row l32 and, as element v of tile t, column 32 t + 8 (v / 4) + 4 (lane / 32) + v % 4), as
// bf16.  The two half-waves exchange runs of four columns, after which a lane holds eight neighbouring columns and
// stores 16 bytes; a row gets 32 contiguous bytes per instruction.  `dst` points at row 0, column 0; rows >=
// valid_rows and columns >= valid_cols are skipped.  The 16-byte path needs row_stride % 8 == 0 (dst is then 16-byte
// aligned: the tensor is, and column tiles start at multiples of 128).
// The lane's number computed from nothing, and opaque: what is derived from it is derived where it is used instead of
// being kept in a register through a loop (where such a register is spilled, its reload waits for every load in flight).
TGO_DEVICE int lane_afresh() {
    int lane = static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
    asm volatile("" : "+v"(lane));
    return lane;
}

template <int TILES>
TGO_DEVICE void store_rows_32xn(const v16f * tiles, uint16_t * dst, int64_t row_stride, int valid_rows, int valid_cols, int lane) {
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const bool wide = (row_stride & 7) == 0;
    uint16_t * const row = dst + l32 * row_stride;
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            // runs 2m and 2m + 1 of the tile: the lower half-wave keeps its run 2m and takes the upper one's,
            // the upper half-wave keeps its run 2m + 1 and takes the lower one's
            const uint32_t p0 = pack_bf16x2(tiles[t][8 * m + 0], tiles[t][8 * m + 1]);
            const uint32_t p1 = pack_bf16x2(tiles[t][8 * m + 2], tiles[t][8 * m + 3]);
            const uint32_t q0 = pack_bf16x2(tiles[t][8 * m + 4], tiles[t][8 * m + 5]);
            const uint32_t q1 = pack_bf16x2(tiles[t][8 * m + 6], tiles[t][8 * m + 7]);
            const auto s0 = __builtin_amdgcn_permlane32_swap(p0, q0, false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(p1, q1, false, false);
            const uint32_t words[4] = {s0[0], s1[0], s0[1], s1[1]};
            const int c = 32 * t + 16 * m + 8 * half;
            if (l32 < valid_rows && c < valid_cols) {
                if (wide && c + 8 <= valid_cols) {
                    *reinterpret_cast<uint4 *>(row + c) = make_uint4(words[0], words[1], words[2], words[3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (c + e < valid_cols) {
                            row[c + e] = static_cast<uint16_t>(words[e >> 1] >> (16 * (e & 1)));
                        }
                    }
                }
            }
        }
    }
}

// ---- groups of at most 32 rows ---------------------------------------------------------------------------------
// A task of a few rows costs the role-split workgroups below what a full one costs their unpacking waves, while seven of
// their eight multiplying waves have nothing to do: on a routing with many small groups a third of the time went into
// 1.5 % of the rows.  Such tasks (the list keeps whole groups of at most 32 rows behind the others) go to workgroups of
// the same launch that run this routine instead, in which every wave unpacks: a wave owns 32 weight rows of the task's column tile and the task's one 32-row activation
// tile, from the packed blocks to the stored results, and never meets another wave.  Its fp16 weights stay in
// registers: the lane that unpacks k-half h of a 32-value block of weight row n holds exactly the two matrix-instruction
// fragments of reduction step 2 * block + h, and one exchange between the half-waves (v_permlane32_swap) per register
// puts them where the instruction wants them.  Three such groups of four waves make a workgroup, so that twelve waves keep
// the vector pipe busy where four did.  The algebra is that of the role-split routine except for the weight normalisation,
// which is per super-block here (see below): the two agree to fp32 rounding of that last step, not bit for bit.
constexpr int FSS_WAVES = 4;

template <int TYPE>
struct ShortLds {
    static constexpr int RAW_SLOT = ScaledLds<TYPE>::RAW_SLOT;
    alignas(16) uint8_t raw[FSS_WAVES][32 * RAW_SLOT];   // per wave: the packed blocks of one super-block
    alignas(16) uint8_t x[16 * 1024];                    // the task's activation fragments of one super-block
    alignas(16) float column_power[FSS_WAVES][32];       // 2^s of the wave's weight rows in the current super-block
    alignas(16) int arrived[FSS_WAVES];                  // barriers of the group that each of its waves has reached
    int next_item;                                       // the chunk of items that the group has taken from the list
    std::conditional_t<TYPE == IQ2_S, Iq2sSelectors, uint2> codebook;
};

// `tid`: the thread's index in its group of FSS_WAVES waves; `group`: which of the groups that share the workgroup
// this is; `blocks` workgroups run short items.  The groups of a workgroup run side by side like workgroups of their
// own: what one waits for (its packed blocks, its barrier) the others cover with their unpacking, which they could not
// if the workgroup's barrier held them in step.  So a group synchronises its four waves through counters in LDS (LDS
// executes a wave's accesses in issue order: a count written after the data, or after the last read, needs no wait of
// its own), and takes its items from the list's cursor by itself.  Three groups that unpack side by side on a CU each
// take more than twice as long as one that is alone there, so towards the end of the list the later groups stop
// taking items and the last ones are spread over the CUs.  Workgroups that start late, on the CUs of the role-split
// workgroups that ran longest, simply take fewer.
// Without TRAILING the routine is a workgroup's whole program (one group: the workgroup's barrier serves) and the items
// go round the `blocks` workgroups of a launch of its own: for rows of fewer than four super-blocks, whose items are too
// short to pay for an item taken from a cursor (two dependent round trips to memory each).
template <int TYPE, bool WIDE, bool TRAILING>
TGO_DEVICE void short_group_items(const ForwardArgs & a, ShortLds<TYPE> & lds, const int tid, const int group, const int blocks) {
    using F = Format<TYPE>;
    constexpr bool K45 = TYPE == Q4_K || TYPE == Q5_K;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;
    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_selectors(lds.codebook, tid, 64 * FSS_WAVES);
    }
    if (tid < FSS_WAVES) {
        lds.arrived[tid] = 0;
    }
    __syncthreads();   // (of the whole workgroup: its groups are still in step here, and part ways behind it)
    static_assert(FSS_WAVES == 4, "one 16-byte read covers the group's counters");
    typedef int i32x4_t __attribute__((ext_vector_type(4)));
    int barriers_passed = 0;
    auto group_barrier = [&]() __attribute__((always_inline)) {
        ++barriers_passed;
        if constexpr (!TRAILING) {
            __syncthreads();
            return;
        }
        asm volatile("" ::: "memory");   // (the data accesses stay before the count)
        if (lane == 0) {
            *(volatile __attribute__((address_space(3))) int *)&lds.arrived[wave] = barriers_passed;
        }
        for (int polls = 0; polls < FSC_SPIN_LIMIT; ++polls) {
            const i32x4_t v = *(const volatile __attribute__((address_space(3))) i32x4_t *)&lds.arrived[0];
            if (__builtin_amdgcn_readfirstlane(min(min(v.x, v.y), min(v.z, v.w))) >= barriers_passed) {
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        asm volatile("" ::: "memory");   // (the data accesses stay after the count)
    };
    // The number of short tasks is known on the device only (one round trip to read it).
    const int inner = a.n_tiles * a.projections;
    const int tasks = a.task_count[0];
    const int first_short = min(a.task_early[0], tasks);
    const int items = (tasks - first_short) * inner;
    // Items are taken in chunks of at least four super-blocks of work, from TASK_CURSORS lists: chunk j belongs to list
    // j % TASK_CURSORS, whose cursor counts the chunks taken from it.  (Atomic operations on one address complete one
    // after the other, at some tens of nanoseconds each: a thousand items through one cursor cost more than they saved.)
    // A group starts with the list of its workgroup's number and goes on to the others when that is used up.
    const int chunk_items = max(1, 4 / (a.in_features / QK_K));
    const int chunks = (items + chunk_items - 1) / chunk_items;
    const int home = static_cast<int>(blockIdx.x) % TASK_CURSORS;
    const int blocks_per_list = max(1, blocks / TASK_CURSORS);
    int item = TRAILING ? 0 : static_cast<int>(blockIdx.x) - blocks + 1, item_end = 0;
#pragma unroll 1
    for (;;) {
    if constexpr (!TRAILING) {
        item += blocks - 1;   // (with the increment at the end of an item: every blocks-th item, from the workgroup's number)
        if (item >= items) {
            break;
        }
    } else if (item == item_end) {
        if (tid == 0) {
            int chunk = -1;
            for (int k = 0; k < TASK_CURSORS && chunk < 0; ++k) {
                const int list = (home + k) % TASK_CURSORS;
                int32_t * const cursor = a.task_cursor + list * TASK_CURSOR_STRIDE;
                const int in_list = (chunks - list + TASK_CURSORS - 1) / TASK_CURSORS;   // chunks j = list (mod TASK_CURSORS)
                // (an estimate of what is left decides whether this group still takes part; the count itself is exact)
                const int left = in_list - __hip_atomic_load(cursor, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // (a group's first chunk: while any is left -- the groups that started with it are all busy as long;
                // later: only if the groups before it, one more chunk each, would not finish the list)
                if (left > (barriers_passed == 0 ? 0 : group * blocks_per_list)) {
                    const int taken = atomicAdd(cursor, 1);
                    if (taken < in_list) {
                        chunk = taken * TASK_CURSORS + list;
                    }
                }
            }
            *(volatile __attribute__((address_space(3))) int *)&lds.next_item = chunk;
        }
        group_barrier();
        const int chunk = __builtin_amdgcn_readfirstlane(*(const volatile __attribute__((address_space(3))) int *)&lds.next_item);
        if (chunk < 0) {
            break;
        }
        item = chunk * chunk_items;
        item_end = min(item + chunk_items, items);
    }
    const int task = first_short + item / inner;
    int tile = item % inner;
    const bool second = tile >= a.n_tiles;
    tile -= second ? a.n_tiles : 0;
    // (a wave whose weight rows lie past the end of the matrix repeats the last row and stores nothing: the
    // workgroup's barriers need it)
    const int n0 = tile * FWD_TN + 32 * wave;
    const int expert = a.task_expert[task];
    const int row_start = a.task_row_start[task];
    const int row_end = a.task_row_end[task];
    const int super_blocks = a.in_features / QK_K;
    const int blocks_per_row = a.in_features / 32;
    const uint8_t * const weights = (second ? a.packed_second : a.packed) + static_cast<int64_t>(expert) * a.bytes_per_expert;
    const int rows_valid = max(1, min(32, a.out_features - n0));   // weight rows past the end repeat the last one (never stored)
    const uint8_t * const rows = weights + static_cast<int64_t>(min(n0, a.out_features - 1)) * a.row_bytes;

    // ---- the packed blocks: one super-block ahead in registers, the current one in the wave's LDS slot
    constexpr int RAW_UNITS = K45 ? F::BLOCK_BYTES / 16 : 1;
    constexpr int RAW_REGS = K45 ? (32 * RAW_UNITS + 63) / 64 : 1;
    using W = WideStage<TYPE>;
    constexpr int WIDE_REGS = WIDE ? W::template regs<32, 64>() : 1;
    constexpr int SLOT_PITCH = K45 ? F::BLOCK_BYTES : (WIDE ? W::PITCH : F::RAW_PITCH);
    constexpr int SLOT_FRONT = K45 ? 0 : (WIDE ? W::FRONT : F::RAW_SHIFT);
    uint8_t * const slot = lds.raw[wave];
    struct RawSet {
        u32x4_t units[RAW_REGS];
        WideRegs<WIDE_REGS> wide;
    };
    RawSet pending;
    auto request = [&](int kb) __attribute__((always_inline)) {
        kb = min(kb, super_blocks - 1);
        if constexpr (K45) {
            const uint8_t * base = rows + static_cast<int64_t>(kb) * F::BLOCK_BYTES;
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = min(lane + 64 * i, 32 * RAW_UNITS - 1);
                const int row = id / RAW_UNITS;
                const int unit = id - row * RAW_UNITS;
                const uint32_t offset = __umul24(min(row, rows_valid - 1), static_cast<uint32_t>(a.row_bytes)) + unit * 16;
                pending.units[i] = *reinterpret_cast<const u32x4_t *>(base + offset);
            }
        } else if constexpr (WIDE) {
            wide_fetch<TYPE, 32, 64, WIDE_REGS>(pending.wide, rows, static_cast<int>(a.row_bytes), rows_valid, kb, lane);
        }
    };
    auto park = [&](int kb) __attribute__((always_inline)) {
        kb = min(kb, super_blocks - 1);
        // (the slot is written as words and read as bytes, halves and words: without these the compiler may move the
        // writes across reads of another type; the hardware runs a wave's LDS accesses in order)
        asm volatile("" ::: "memory");
        if constexpr (K45) {
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = min(lane + 64 * i, 32 * RAW_UNITS - 1);
                *reinterpret_cast<u32x4_t *>(slot + id * 16) = pending.units[i];
            }
        } else if constexpr (WIDE) {
            wide_park<TYPE, 32, 64, WIDE_REGS>(slot, pending.wide, rows, static_cast<int>(a.row_bytes), rows_valid, kb, lane);
        } else {
            stage_blocks<TYPE>(slot, weights, a.row_bytes, min(n0, a.out_features - 1), a.out_features, kb, 32, lane, 64);
        }
        asm volatile("" ::: "memory");
    };
    request(0);

    // ---- the weight normalisation: per weight row AND super-block here (2^s: the largest magnitude of the
    // super-block's weights goes to [2^8, 2^9)), applied when a super-block's sum joins the row's: a scan of the row's
    // scales ahead of the first block, as the kernel above does, would fetch a line of every block for four bytes of
    // it, all waves at once, and the few waves of a short task have nothing to cover that with
    auto block_power = [&](float reach, float & shrink) __attribute__((always_inline)) {
        int exponent = static_cast<int>(__float_as_uint(reach) >> 23);   // biased
        exponent = min(max(exponent, 9), 254);
        if (half == 0) {
            lds.column_power[wave][l32] = __uint_as_float(static_cast<uint32_t>(exponent - 8) << 23);   // 2^s
        }
        shrink = __uint_as_float(static_cast<uint32_t>(262 - exponent) << 23);   // 2^-s
    };

    // ---- the activation rows (at most 32, from row_start: they may straddle two 32-row tiles of the workspace)
    const int first_tile = row_start >> 5;
    const uint8_t * const x_base = reinterpret_cast<const uint8_t *>(a.qx) + static_cast<int64_t>(first_tile) * blocks_per_row * 2048;
    const uint8_t * const sums_base = reinterpret_cast<const uint8_t *>(a.block_sums) + static_cast<int64_t>(first_tile) * super_blocks * 512;
    int lane_row = row_start + l32;
    lane_row = lane_row < a.rows_padded ? lane_row : a.rows_padded - 1;
    // 2^E of the lane's row, for the epilogue (requested here: asked for there, the whole item would wait for it, and
    // for every load still in flight in front of it)
    const float row_power = a.row_power[lane_row];
    const uint32_t x_lane = static_cast<uint32_t>((lane_row >> 5) - first_tile) * blocks_per_row * 2048u +
                            static_cast<uint32_t>(((lane_row & 31) + 32 * half) * 16);
    const uint32_t sums_lane = static_cast<uint32_t>((lane_row >> 5) - first_tile) * super_blocks * 512u +
                               static_cast<uint32_t>((lane_row & 31) * 16);
    // Everything a super-block needs from memory is requested while the one before it is unpacked and multiplied, and
    // awaited once, at its end: the packed blocks (this wave's), the wave's quarter of the task's activation fragments
    // (which go to LDS for all four waves), the row's 2^(e - E) and block sums.  Loads return in order, so waiting
    // for an activation fragment from the L2 in the middle of a super-block would also wait for the packed blocks
    // behind which it was requested, and those come from HBM.
    struct Incoming {
        half8_t x[4];
        float ratio;
        uint4 sums;
    };
    Incoming incoming;
    auto request_rows = [&](int kb) __attribute__((always_inline)) {
        kb = min(kb, super_blocks - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            incoming.x[i] = *reinterpret_cast<const half8_t *>(x_base + static_cast<int64_t>(kb * 16 + 4 * wave + i) * 1024 + x_lane);
        }
        incoming.ratio = a.power[static_cast<int64_t>(kb) * a.rows_padded + lane_row];
        incoming.sums = make_uint4(0, 0, 0, 0);
        if constexpr (K45) {
            incoming.sums = *reinterpret_cast<const uint4 *>(sums_base + static_cast<int64_t>(kb) * 512 + sums_lane);
        }
    };
    auto publish_rows = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<half8_t *>(&lds.x[(4 * wave + i) * 1024 + lane * 16]) = incoming.x[i];
        }
    };

    const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v16f acc = zero;     // of the super-block
    v16f total = zero;   // of the row: sum over super-blocks of 2^s * acc
    // The lane's 16 values of a block (k-half `half`: registers 0-3 hold its first eight, 4-7 the other eight) are the
    // two fragments of reduction step 2 * block + half; the half-waves exchange what the other one multiplies, then
    // `first` is step 2 * block and `other` step 2 * block + 1.
    auto rescale = [&](half8_t fragment, half2_t ratio) __attribute__((always_inline)) {
        const uint4 words = __builtin_bit_cast(uint4, fragment);
        const uint4 scaled = make_uint4(half2_mul(words.x, ratio), half2_mul(words.y, ratio), half2_mul(words.z, ratio),
                                        half2_mul(words.w, ratio));
        return __builtin_bit_cast(half8_t, scaled);
    };
    // `step`: of the super-block (0..15); `fragments`: the super-block's activation fragments in LDS.  (Applying the
    // row's 2^(e - E) to the super-block's sums instead of its fragments would save these multiplications; the
    // compiler then schedules the fragment reads far ahead and spills what the wave has unpacked: measured slower.)
    auto multiply_block = [&](uint32_t (&values)[8], int step, half2_t ratio, const uint8_t * fragments) __attribute__((always_inline)) {
        uint32_t first[4], other[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const auto swapped = __builtin_amdgcn_permlane32_swap(values[i], values[4 + i], false, false);
            first[i] = swapped[0];
            other[i] = swapped[1];
        }
        const half8_t x0 = *reinterpret_cast<const half8_t *>(fragments + step * 1024 + lane * 16);
        const half8_t x1 = *reinterpret_cast<const half8_t *>(fragments + (step + 1) * 1024 + lane * 16);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, make_uint4(first[0], first[1], first[2], first[3])),
                                                     rescale(x0, ratio), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, make_uint4(other[0], other[1], other[2], other[3])),
                                                     rescale(x1, ratio), acc, 0, 0, 0);
    };

    const uint8_t * const blk = slot + l32 * SLOT_PITCH + SLOT_FRONT;
    request_rows(0);
    park(0);
    publish_rows();
    group_barrier();
#pragma unroll 1
    for (int kb = 0; kb < super_blocks; ++kb) {
        const half2_t ratio = {static_cast<_Float16>(incoming.ratio), static_cast<_Float16>(incoming.ratio)};
        const uint4 sums = incoming.sums;
        const uint8_t * const fragments = lds.x;
        request(kb + 1);
        request_rows(kb + 1);
        if constexpr (K45) {
            constexpr int QS = TYPE == Q4_K ? 16 : 48;
            const u32x4_t header = *reinterpret_cast<const u32x4_t *>(blk);
            u32x4_t planes = {0, 0, 0, 0};
            if constexpr (TYPE == Q5_K) {
                planes = *reinterpret_cast<const u32x4_t *>(blk + 16 + 16 * half);
            }
            const uint32_t plane_word[4] = {planes.x, planes.y, planes.z, planes.w};
            float shrink;
            block_power(fmaxf(fabsf(half_bits_to_float(header.x & 0xffffu)) * weight_reach<TYPE>(),
                              fabsf(half_bits_to_float(header.x >> 16)) * 63.0f), shrink);
            const float d = half_bits_to_float(header.x & 0xffffu) * shrink;
            auto chunk = [&](auto stage_tag, auto pair_tag) __attribute__((always_inline)) {
                constexpr int S = decltype(stage_tag)::value;
                constexpr int P = decltype(pair_tag)::value;
                // (read where it is used: the other waves of the SIMD cover the LDS round trip, and the registers
                // that an early read would hold are what keeps a stage of activation fragments in flight)
                const u32x4_t nibbles = *reinterpret_cast<const u32x4_t *>(blk + QS + (2 * S + P) * 32 + 16 * half);
                constexpr int G = 4 * S + 2 * P;   // low nibbles: group G, high nibbles: group G + 1
                int sc_low, sc_high, unused;
                k45_group_scale_min<G>(header.y, header.z, header.w, sc_low, unused);
                k45_group_scale_min<G + 1>(header.y, header.z, header.w, sc_high, unused);
                const HalfScale scale_low = half_scale_of(d * static_cast<float>(sc_low));
                const HalfScale scale_high = half_scale_of(d * static_cast<float>(sc_high));
                const uint32_t word[4] = {nibbles.x, nibbles.y, nibbles.z, nibbles.w};
                uint32_t low[8], high[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    uint32_t bytes_low = word[w] & 0x0f0f0f0fu;
                    uint32_t bytes_high = (word[w] >> 4) & 0x0f0f0f0fu;
                    if constexpr (TYPE == Q5_K) {
                        if constexpr (G <= 3) {
                            bytes_low |= (plane_word[w] << (4 - G)) & 0x10101010u;
                            bytes_high |= (plane_word[w] << (3 - G)) & 0x10101010u;
                        } else {
                            bytes_low |= (plane_word[w] >> (G - 4)) & 0x10101010u;
                            bytes_high |= (plane_word[w] >> (G - 3)) & 0x10101010u;
                        }
                    }
                    scaled_halves(bytes_low, scale_low, low[2 * w], low[2 * w + 1]);
                    scaled_halves(bytes_high, scale_high, high[2 * w], high[2 * w + 1]);
                }
                multiply_block(low, 8 * S + 4 * P, ratio, fragments);
                multiply_block(high, 8 * S + 4 * P + 2, ratio, fragments);
            };
            chunk(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
            chunk(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
            {   // the super-block's extra reduction step: block minima x block sums
                int sc, mn[8];
                k45_group_scale_min<0>(header.y, header.z, header.w, sc, mn[0]);
                k45_group_scale_min<1>(header.y, header.z, header.w, sc, mn[1]);
                k45_group_scale_min<2>(header.y, header.z, header.w, sc, mn[2]);
                k45_group_scale_min<3>(header.y, header.z, header.w, sc, mn[3]);
                k45_group_scale_min<4>(header.y, header.z, header.w, sc, mn[4]);
                k45_group_scale_min<5>(header.y, header.z, header.w, sc, mn[5]);
                k45_group_scale_min<6>(header.y, header.z, header.w, sc, mn[6]);
                k45_group_scale_min<7>(header.y, header.z, header.w, sc, mn[7]);
                const float minus = -half_bits_to_float(header.x >> 16) * shrink;
                uint32_t packed[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const half2_t pair = {static_cast<_Float16>(minus * static_cast<float>(mn[2 * i])),
                                          static_cast<_Float16>(minus * static_cast<float>(mn[2 * i + 1]))};
                    packed[i] = half != 0 ? 0u : __builtin_bit_cast(uint32_t, pair);
                }
                const half8_t block_sums = rescale(__builtin_bit_cast(half8_t, half != 0 ? make_uint4(0, 0, 0, 0) : sums), ratio);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                    __builtin_bit_cast(half8_t, make_uint4(packed[0], packed[1], packed[2], packed[3])), block_sums, acc, 0, 0, 0);
            }
            chunk(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
            chunk(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
        } else {
            const auto * const grid = &lds.codebook;
            float shrink;
            block_power(fabsf(half_bits_to_float(lds_u16(blk + scale_offset<TYPE>()))) * weight_reach<TYPE>(), shrink);
            const _Float16 h = static_cast<_Float16>(half_weight_scale<TYPE>(blk) * shrink);
            const half2_t scale = {h, h};
#pragma unroll
            for (int b = 0; b < 8; ++b) {
                uint32_t first[8], fine[8];
                decode16_half<TYPE>(blk, 2 * b + half, grid, first, fine);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if constexpr (TYPE == Q6_K) {
                        first[i] = half2_fma(first[i], scale, __builtin_bit_cast(half2_t, half2_mul(fine[i], scale)));
                    } else {
                        first[i] = half2_mul(first[i], scale);
                    }
                }
                multiply_block(first, 2 * b, ratio, fragments);
            }
        }
        // (everything of this super-block has been read from the slot: the next one goes there; the next fragments
        // replace this super-block's once every wave is done with them.  A second fragment buffer would save this
        // barrier and cost the third workgroup per CU.)
        park(kb + 1);
        group_barrier();
        publish_rows();
        // the super-block's sums join the row's, each column with the power of two its weights were divided by
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 column_power = *reinterpret_cast<const float4 *>(&lds.column_power[wave][8 * j + 4 * half]);
            total[4 * j + 0] = __builtin_fmaf(acc[4 * j + 0], column_power.x, total[4 * j + 0]);
            total[4 * j + 1] = __builtin_fmaf(acc[4 * j + 1], column_power.y, total[4 * j + 1]);
            total[4 * j + 2] = __builtin_fmaf(acc[4 * j + 2], column_power.z, total[4 * j + 2]);
            total[4 * j + 3] = __builtin_fmaf(acc[4 * j + 3], column_power.w, total[4 * j + 3]);
        }
        acc = zero;
        group_barrier();
    }

    // ---- epilogue: scale by 2^(E[r] + S[n]) and store 32 rows x 32 columns
    {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            acc[v] = total[v] * row_power;
        }
        uint16_t * const y = (second ? a.y_second : a.y) + static_cast<int64_t>(row_start) * a.out_features + n0;
        // (recomputing the lane's share here is cheaper than keeping it alive through the loop: kept, it is spilled, and
        // its reload waits for every load in flight)
        const int lane_here = lane_afresh();
        store_rows_32xn<1>(&acc, y, a.out_features, row_end - row_start, a.out_features - n0, lane_here);
    }
    group_barrier();   // (the next item reuses the LDS buffers)
    ++item;
    }
}


// The short groups in a launch of their own (three workgroups of four waves per CU share the items).
template <int TYPE, bool WIDE>
__global__ __launch_bounds__(64 * FSS_WAVES, 3) void mmq_forward_scaled_short_kernel(const ForwardArgs a) {
    __shared__ ShortLds<TYPE> lds;
    short_group_items<TYPE, WIDE, false>(a, lds, threadIdx.x, 0, gridDim.x);
}

template <int TYPE, bool WIDE>
__global__ __launch_bounds__(FSC_THREADS, 3) void mmq_forward_scaled_kernel(const ForwardArgs a, const int total_slots,
                                                                            const int main_blocks) {
    using F = Format<TYPE>;
    using L = ScaledLds<TYPE>;
    constexpr bool K45 = L::K45;
    constexpr int SHORT_GROUPS = FSC_THREADS / (64 * FSS_WAVES);
    union Shared {
        L role_split;
        ShortLds<TYPE> short_groups[SHORT_GROUPS];
    };
    __shared__ Shared shared;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;

    // The workgroups behind the role-split ones run the groups of at most 32 rows.  Workgroups start in the order of
    // their numbers and one fills a CU, so these start on the CUs whose role-split workgroup has run out of items while
    // the last round of items still occupies the others.
    if (static_cast<int>(blockIdx.x) >= main_blocks) {
        const int group = __builtin_amdgcn_readfirstlane(tid / (64 * FSS_WAVES));
        short_group_items<TYPE, WIDE, true>(a, shared.short_groups[group], tid % (64 * FSS_WAVES), group,
                                            static_cast<int>(gridDim.x) - main_blocks);
        return;
    }
    L & lds = shared.role_split;

    // item table: slot i of this workgroup is position blockIdx.x + i * main_blocks of the launch order (main_blocks is
    // a multiple of the XCD count, so all of them map to this workgroup's XCD); empty slots are squeezed out
    if (wave == 0) {
        ScaledItem item = {0, 0, 0, -1};
        const int64_t linear = blockIdx.x + static_cast<int64_t>(lane) * main_blocks;
        if (linear < total_slots) {
            int n_tile, expert, row_start, row_end;
            bool second;
            if (forward_pick_linear(a, static_cast<int>(linear), n_tile, second, expert, row_start, row_end)) {
                item = ScaledItem{expert, row_start, row_end, n_tile + (second ? a.n_tiles : 0)};
            }
        }
        const bool valid = item.tile >= 0;
        const unsigned long long mask = __ballot(valid);
        if (valid) {
            lds.items[__popcll(mask & ((1ull << lane) - 1ull))] = item;
        }
        if (lane == 0) {
            lds.item_count = __popcll(mask);
        }
        if (lane < 4) {
            lds.produced[lane] = 0;
        }
        if (lane < FSC_MULTIPLIERS) {
            lds.consumed[lane] = 0;
        }
    }
    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_selectors(lds.codebook, tid, FSC_THREADS);
    }
    __syncthreads();
    const int n_items = lds.item_count;
    if (n_items == 0) {
        return;
    }
    const int super_blocks = a.in_features / QK_K;
    const int total = n_items * super_blocks;   // super-blocks of this workgroup's stream
    auto item_field = [&](int item, int field) {
        return __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(&lds.items[item])[field]);
    };

    // Stage counters.  Every lane polls the same words (a broadcast read); a wave that has polled FSC_SPIN_LIMIT times
    // stops waiting, so that a lost count ends in wrong results rather than in a workgroup that never finishes.
    typedef int i32x4_t __attribute__((ext_vector_type(4)));
    using SharedCounters = const volatile __attribute__((address_space(3))) i32x4_t *;
    using SharedCounter = volatile __attribute__((address_space(3))) int *;
    auto publish = [&](int * counter, int value) __attribute__((always_inline)) {
        asm volatile("" ::: "memory");   // (the data accesses stay before the count)
        if (lane == 0) {
            *(SharedCounter)counter = value;
        }
    };
    // (counts only grow: what a poll has seen serves every later wait that it already satisfies, without touching LDS,
    // whose queue a poll has to drain first)
    int seen_produced = 0, seen_consumed = 0;
    auto wait_produced = [&](int need) __attribute__((always_inline)) {
        if (seen_produced < need) {
            for (int polls = 0; polls < FSC_SPIN_LIMIT; ++polls) {
                const i32x4_t v = *(SharedCounters)&lds.produced[0];
                seen_produced = __builtin_amdgcn_readfirstlane(min(min(v.x, v.y), min(v.z, v.w)));
                if (seen_produced >= need) {
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        asm volatile("" ::: "memory");   // (the data accesses stay after the count)
    };
    auto wait_consumed = [&](int need) __attribute__((always_inline)) {
        static_assert(FSC_MULTIPLIERS == 8, "two 16-byte reads cover the multipliers' counters");
        if (seen_consumed < need) {
            for (int polls = 0; polls < FSC_SPIN_LIMIT; ++polls) {
                const i32x4_t v = *(SharedCounters)&lds.consumed[0];
                const i32x4_t u = *(SharedCounters)&lds.consumed[4];
                const int least = min(min(min(v.x, v.y), min(v.z, v.w)), min(min(u.x, u.y), min(u.z, u.w)));
                seen_consumed = __builtin_amdgcn_readfirstlane(least);
                if (seen_consumed >= need) {
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        asm volatile("" ::: "memory");
    };
    auto next_buffer = [](int buffer) { return buffer + 1 == FSC_BUFFERS ? 0 : buffer + 1; };

    if (wave >= FSC_MULTIPLIERS) {
        // ---------------- unpacking wave ----------------
        const int dw = wave - FSC_MULTIPLIERS;
        constexpr int RAW_UNITS = K45 ? F::BLOCK_BYTES / 16 : 1;
        constexpr int RAW_REGS = K45 ? (32 * RAW_UNITS + 63) / 64 : 1;
        using W = WideStage<TYPE>;
        constexpr int WIDE_REGS = WIDE ? W::template regs<32, 64>() : 1;
        // super-blocks of packed blocks in flight in registers (Q6_K's 14 aligned units per block leave room for two)
        constexpr int RAW_DEPTH = TYPE == Q6_K ? 2 : 3;
        constexpr int SLOT_PITCH = K45 ? F::BLOCK_BYTES : (WIDE ? W::PITCH : F::RAW_PITCH);
        constexpr int SLOT_FRONT = K45 ? 0 : (WIDE ? W::FRONT : F::RAW_SHIFT);

        // Position of one stage of this wave's pipeline in the stream, with what it needs to know about the item:
        // the wave's 32 weight rows (rows past the end of the weight matrix repeat its last row; their results are
        // never stored).  A cursor at the last super-block stays there: stages that look past the end repeat it.
        struct Cursor {
            int item, kb;
            const uint8_t * weights;   // of the item's expert and projection
            const uint8_t * rows;      // first of the wave's weight rows
            int n0, rows_valid;
        };
        auto open_item = [&](Cursor & c, int item) {
            c.item = item;
            c.kb = 0;
            const int tile = item_field(item, 3);
            const bool second = tile >= a.n_tiles;
            c.weights = (second ? a.packed_second : a.packed) + static_cast<int64_t>(item_field(item, 0)) * a.bytes_per_expert;
            c.n0 = (second ? tile - a.n_tiles : tile) * FWD_TN;
            const int tile_rows = min(FWD_TN, a.out_features - c.n0);
            c.rows_valid = max(1, min(32, tile_rows - 32 * dw));
            c.rows = c.weights + static_cast<int64_t>(c.n0 + min(32 * dw, tile_rows - 1)) * a.row_bytes;
        };
        auto step = [&](Cursor & c) {
            if (c.kb + 1 < super_blocks) {
                ++c.kb;
            } else if (c.item + 1 < n_items) {
                open_item(c, c.item + 1);
            }
        };

        // ---- S of this lane's weight row: the largest weight magnitude over the row's super-blocks goes to
        // [2^8, 2^9).  The scale words of the first eight super-blocks are requested an item ahead.
        constexpr int SCAN_REGS = 4;
        auto scan_request = [&](const Cursor & c, uint32_t (&words)[SCAN_REGS]) {
            const uint8_t * blocks = c.rows + static_cast<int64_t>(min(l32, c.rows_valid - 1)) * a.row_bytes;
#pragma unroll
            for (int i = 0; i < SCAN_REGS; ++i) {
                const int kb = min(half + 2 * i, super_blocks - 1);
                const uint8_t * blk = blocks + static_cast<int64_t>(kb) * F::BLOCK_BYTES;
                if constexpr (K45) {
                    words[i] = *reinterpret_cast<const uint32_t *>(blk);
                } else {
                    words[i] = *reinterpret_cast<const uint16_t *>(blk + scale_offset<TYPE>());
                }
            }
        };
        auto scan_word = [&](uint32_t word) {
            float reach = fabsf(half_bits_to_float(word & 0xffffu)) * weight_reach<TYPE>();
            if constexpr (K45) {
                reach = fmaxf(reach, fabsf(half_bits_to_float(word >> 16)) * 63.0f);
            }
            return reach;
        };
        // returns 2^-S and leaves 2^S for the multiplying waves
        auto scan_finish = [&](const Cursor & c, const uint32_t (&words)[SCAN_REGS]) {
            float reach = 0.0f;
#pragma unroll
            for (int i = 0; i < SCAN_REGS; ++i) {
                reach = fmaxf(reach, scan_word(words[i]));
            }
            if (super_blocks > 2 * SCAN_REGS) {   // long rows: the rest, read here
                const uint8_t * blocks = c.rows + static_cast<int64_t>(min(l32, c.rows_valid - 1)) * a.row_bytes;
                for (int kb = 2 * SCAN_REGS + half; kb < super_blocks; kb += 2) {
                    const uint8_t * blk = blocks + static_cast<int64_t>(kb) * F::BLOCK_BYTES;
                    if constexpr (K45) {
                        reach = fmaxf(reach, scan_word(*reinterpret_cast<const uint32_t *>(blk)));
                    } else {
                        reach = fmaxf(reach, scan_word(*reinterpret_cast<const uint16_t *>(blk + scale_offset<TYPE>())));
                    }
                }
            }
            reach = fmaxf(reach, __shfl_xor(reach, 32));
            int exponent = static_cast<int>(__float_as_uint(reach) >> 23);   // biased
            exponent = min(max(exponent, 9), 254);
            if (half == 0) {
                lds.row_power[c.item & 3][32 * dw + l32] = __uint_as_float(static_cast<uint32_t>(exponent - 8) << 23);   // 2^S
            }
            return __uint_as_float(static_cast<uint32_t>(262 - exponent) << 23);   // 2^-S
        };

        // Packed blocks of RAW_DEPTH super-blocks are in flight in registers: a lone request per super-block would
        // leave the wave waiting for memory once per super-block.
        struct RawSet {
            u32x4_t units[RAW_REGS];
            WideRegs<WIDE_REGS> wide;
        };
        RawSet ring[RAW_DEPTH];
        auto request = [&](const Cursor & c, RawSet & set) {
            if constexpr (K45) {
                const uint8_t * base = c.rows + static_cast<int64_t>(c.kb) * F::BLOCK_BYTES;
#pragma unroll
                for (int i = 0; i < RAW_REGS; ++i) {
                    // ids past the wave's blocks repeat the last unit, so no lane branches around a load
                    const int id = min(lane + 64 * i, 32 * RAW_UNITS - 1);
                    const int row = id / RAW_UNITS;
                    const int unit = id - row * RAW_UNITS;
                    const uint32_t offset = __umul24(min(row, c.rows_valid - 1), static_cast<uint32_t>(a.row_bytes)) + unit * 16;
                    set.units[i] = *reinterpret_cast<const u32x4_t *>(base + offset);
                }
            } else if constexpr (WIDE) {
                wide_fetch<TYPE, 32, 64, WIDE_REGS>(set.wide, c.rows, static_cast<int>(a.row_bytes), c.rows_valid, c.kb, lane);
            }
        };
        // `c`: the super-block the registers were requested for; `slot_parity`: where it goes
        auto park = [&](const Cursor & c, int slot_parity, const RawSet & set) {
            uint8_t * const slot = lds.raw[dw][slot_parity];
            if constexpr (K45) {
#pragma unroll
                for (int i = 0; i < RAW_REGS; ++i) {
                    const int id = min(lane + 64 * i, 32 * RAW_UNITS - 1);
                    *reinterpret_cast<u32x4_t *>(slot + id * 16) = set.units[i];   // (slots lie back to back: row * BLOCK_BYTES + unit * 16)
                }
            } else if constexpr (WIDE) {
                wide_park<TYPE, 32, 64, WIDE_REGS>(slot, set.wide, c.rows, static_cast<int>(a.row_bytes), c.rows_valid, c.kb, lane);
            } else {
                stage_blocks<TYPE>(slot, c.weights, a.row_bytes, c.n0 + 32 * dw, a.out_features, c.kb, 32, lane, 64);
            }
        };
        // A lane keeps weight row `l32` of the wave's 32 and takes k-half `half` of every 32-value block.
        const uint32_t out_lane = static_cast<uint32_t>(dw * (FSC_STEPS * 1024) + half * 1024 + l32 * 16);
        auto block_of = [&](int parity) { return lds.raw[dw][parity] + l32 * SLOT_PITCH + SLOT_FRONT; };
        // Q4_K/Q5_K: what a stage's unpack reads from the parked block, fetched a phase before it is used (a lone
        // wave has nothing else to cover an LDS round trip with): the 16-byte header (d, dmin, 12 bytes of 6-bit
        // scales and minima), this k-half's fifth-bit bytes, and its 16 bytes of each of the stage's two nibble chunks.
        struct StageInputs {
            u32x4_t header, planes, nibbles[2];
        };
        auto fetch_inputs = [&](int stage_of_block, int parity) {
            constexpr int QS = TYPE == Q4_K ? 16 : 48;
            const uint8_t * blk = block_of(parity);
            StageInputs in;
            in.header = *reinterpret_cast<const u32x4_t *>(blk);
            in.planes = u32x4_t{0, 0, 0, 0};
            if constexpr (TYPE == Q5_K) {
                in.planes = *reinterpret_cast<const u32x4_t *>(blk + 16 + 16 * half);
            }
            in.nibbles[0] = *reinterpret_cast<const u32x4_t *>(blk + QS + (2 * stage_of_block) * 32 + 16 * half);
            in.nibbles[1] = *reinterpret_cast<const u32x4_t *>(blk + QS + (2 * stage_of_block + 1) * 32 + 16 * half);
            return in;
        };
        float shrink = 1.0f;   // 2^-S of the lane's weight row in the item being unpacked
        // the eight block minima of a Q4_K/Q5_K super-block as the operand of its extra reduction step
        auto minima_from_header = [&](int buffer, const u32x4_t header) {
            int sc, mn[8];
            k45_group_scale_min<0>(header.y, header.z, header.w, sc, mn[0]);
            k45_group_scale_min<1>(header.y, header.z, header.w, sc, mn[1]);
            k45_group_scale_min<2>(header.y, header.z, header.w, sc, mn[2]);
            k45_group_scale_min<3>(header.y, header.z, header.w, sc, mn[3]);
            k45_group_scale_min<4>(header.y, header.z, header.w, sc, mn[4]);
            k45_group_scale_min<5>(header.y, header.z, header.w, sc, mn[5]);
            k45_group_scale_min<6>(header.y, header.z, header.w, sc, mn[6]);
            k45_group_scale_min<7>(header.y, header.z, header.w, sc, mn[7]);
            if (half == 0) {
                const float minus = -half_bits_to_float(header.x >> 16) * shrink;
                uint32_t packed[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const half2_t pair = {static_cast<_Float16>(minus * static_cast<float>(mn[2 * i])),
                                          static_cast<_Float16>(minus * static_cast<float>(mn[2 * i + 1]))};
                    packed[i] = __builtin_bit_cast(uint32_t, pair);
                }
                *reinterpret_cast<uint4 *>(&lds.mins[buffer][dw * 512 + l32 * 16]) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
            }
        };
        // stage S (0, 1) of a Q4_K/Q5_K super-block from its fetched inputs -> operand tile `target`
        auto finish_stage = [&](auto stage_tag, const StageInputs & in, int target) {
            constexpr int S = decltype(stage_tag)::value;
            uint8_t * const out = &lds.wq[target][0] + out_lane;
            const uint32_t plane_word[4] = {in.planes.x, in.planes.y, in.planes.z, in.planes.w};
            const float d = half_bits_to_float(in.header.x & 0xffffu) * shrink;
            auto chunk = [&](auto pair_tag) {
                constexpr int P = decltype(pair_tag)::value;
                constexpr int G = 4 * S + 2 * P;   // low nibbles: group G, high nibbles: group G + 1
                int sc_low, sc_high, unused;
                k45_group_scale_min<G>(in.header.y, in.header.z, in.header.w, sc_low, unused);
                k45_group_scale_min<G + 1>(in.header.y, in.header.z, in.header.w, sc_high, unused);
                const HalfScale scale_low = half_scale_of(d * static_cast<float>(sc_low));
                const HalfScale scale_high = half_scale_of(d * static_cast<float>(sc_high));
                const uint32_t word[4] = {in.nibbles[P].x, in.nibbles[P].y, in.nibbles[P].z, in.nibbles[P].w};
                uint32_t low[8], high[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    uint32_t bytes_low = word[w] & 0x0f0f0f0fu;
                    uint32_t bytes_high = (word[w] >> 4) & 0x0f0f0f0fu;
                    if constexpr (TYPE == Q5_K) {
                        // the fifth bit of group g is bit g of the plane byte: moved to bit 4
                        if constexpr (G <= 3) {
                            bytes_low |= (plane_word[w] << (4 - G)) & 0x10101010u;
                            bytes_high |= (plane_word[w] << (3 - G)) & 0x10101010u;
                        } else {
                            bytes_low |= (plane_word[w] >> (G - 4)) & 0x10101010u;
                            bytes_high |= (plane_word[w] >> (G - 3)) & 0x10101010u;
                        }
                    }
                    scaled_halves(bytes_low, scale_low, low[2 * w], low[2 * w + 1]);
                    scaled_halves(bytes_high, scale_high, high[2 * w], high[2 * w + 1]);
                }
                // block 2P of the stage is reduction steps 4P and 4P + 1 (this lane: 4P + half), block 2P + 1 the next two
                uint8_t * dst = out + (4 * P) * 1024;
                *reinterpret_cast<uint4 *>(dst) = make_uint4(low[0], low[1], low[2], low[3]);
                *reinterpret_cast<uint4 *>(dst + 512) = make_uint4(low[4], low[5], low[6], low[7]);
                *reinterpret_cast<uint4 *>(dst + 2048) = make_uint4(high[0], high[1], high[2], high[3]);
                *reinterpret_cast<uint4 *>(dst + 2048 + 512) = make_uint4(high[4], high[5], high[6], high[7]);
            };
            chunk(std::integral_constant<int, 0>{});
            chunk(std::integral_constant<int, 1>{});
        };
        // the other formats: stage S of the super-block parked in slot `parity`
        auto unpack = [&](auto stage_tag, int parity, int target) {
            constexpr int S = decltype(stage_tag)::value;
            if constexpr (!K45) {
                const uint8_t * blk = block_of(parity);
                uint8_t * const out = &lds.wq[target][0] + out_lane;
                const auto * const grid = &lds.codebook;
                const _Float16 h = static_cast<_Float16>(half_weight_scale<TYPE>(blk) * shrink);
                const half2_t scale = {h, h};
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int unit = 2 * (4 * S + b) + half;
                    uint32_t first[8], fine[8];
                    decode16_half<TYPE>(blk, unit, grid, first, fine);
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        if constexpr (TYPE == Q6_K) {   // sc * q in two parts that share the sign of sc
                            first[i] = half2_fma(first[i], scale, __builtin_bit_cast(half2_t, half2_mul(fine[i], scale)));
                        } else {
                            first[i] = half2_mul(first[i], scale);
                        }
                    }
                    uint8_t * dst = out + (2 * b) * 1024;
                    *reinterpret_cast<uint4 *>(dst) = make_uint4(first[0], first[1], first[2], first[3]);
                    *reinterpret_cast<uint4 *>(dst + 512) = make_uint4(first[4], first[5], first[6], first[7]);
                }
            }
        };


        // c_request walks RAW_DEPTH super-blocks ahead of c_park, which is two ahead of the super-block the
        // multipliers work on; c_scan is the item whose scale words are in flight.
        Cursor c_request, c_park, c_scan;
        open_item(c_request, 0);
        open_item(c_park, 0);
        open_item(c_scan, 0);
#pragma unroll
        for (int ahead = 0; ahead < RAW_DEPTH; ++ahead) {
            request(c_request, ring[ahead]);
            step(c_request);
        }
        uint32_t scan_words[SCAN_REGS];
        scan_request(c_scan, scan_words);
        shrink = scan_finish(c_scan, scan_words);
        if (n_items > 1) {
            open_item(c_scan, 1);
        }
        scan_request(c_scan, scan_words);
        // the oldest set goes to LDS, the others move up, the newest is requested
        auto advance = [&](int slot_parity) {
            park(c_park, slot_parity, ring[0]);
            step(c_park);
#pragma unroll
            for (int ahead = 0; ahead + 1 < RAW_DEPTH; ++ahead) {
                ring[ahead] = ring[ahead + 1];
            }
            request(c_request, ring[RAW_DEPTH - 1]);
            step(c_request);
        };
        advance(0);
        advance(1);
        // stage g goes to buffer g % FSC_BUFFERS once the multipliers have read stage g - FSC_BUFFERS
        int written = 0, buffer = 0;
        StageInputs inputs = {};
        if constexpr (K45) {
            inputs = fetch_inputs(0, 0);
            minima_from_header(0, inputs.header);
            finish_stage(std::integral_constant<int, 0>{}, inputs, 0);
            inputs = fetch_inputs(1, 0);
        } else {
            unpack(std::integral_constant<int, 0>{}, 0, 0);
        }
        publish(&lds.produced[dw], ++written);
        buffer = next_buffer(buffer);
        int kb = 0;   // of super-block q within its item
#pragma unroll 1
        for (int q = 0; q < total; ++q) {
            const int parity = q & 1;
            // (past the last super-block the wave works on a repeat of it: nobody reads what that writes)
            // stage 1 of q
            wait_consumed(written + 1 - FSC_BUFFERS);
            if constexpr (K45) {
                finish_stage(std::integral_constant<int, 1>{}, inputs, buffer);
            } else {
                unpack(std::integral_constant<int, 1>{}, parity, buffer);
            }
            publish(&lds.produced[dw], ++written);
            buffer = next_buffer(buffer);
            if constexpr (K45) {
                inputs = fetch_inputs(0, parity ^ 1);
            }
            // stage 0 of q + 1, which may open the next item
            if (kb + 1 == super_blocks) {
                kb = 0;
                if (q + 1 < total) {
                    shrink = scan_finish(c_scan, scan_words);
                    if (c_scan.item + 1 < n_items) {
                        open_item(c_scan, c_scan.item + 1);
                    }
                    scan_request(c_scan, scan_words);
                }
            } else {
                ++kb;
            }
            wait_consumed(written + 1 - FSC_BUFFERS);
            if constexpr (K45) {
                minima_from_header(buffer, inputs.header);
                finish_stage(std::integral_constant<int, 0>{}, inputs, buffer);
                inputs = fetch_inputs(1, parity ^ 1);
            } else {
                unpack(std::integral_constant<int, 0>{}, parity ^ 1, buffer);
            }
            publish(&lds.produced[dw], ++written);
            buffer = next_buffer(buffer);
            // slot `parity` is free (Q4_K/Q5_K: its last inputs are in registers; the others: stage 1 is done):
            // super-block q + 2 goes there
            advance(parity);
        }
        return;
    }

    // ---------------- multiplying wave ----------------
    // Two of these share a SIMD.  Back-to-back matrix instructions alone issue every 32 cycles from a single wave, but
    // with the fragment reads and activation requests of this loop in between a lone wave managed one per 42 to 46;
    // two waves cover each other's waits.
    // Every global address is a uniform 64-bit base, advanced with scalar arithmetic, plus a 32-bit lane offset.
    const int blocks_per_row = a.in_features / 32;
    // Where this wave's 32 activation rows of an item are: a wave without rows in the item reads the workspace's last
    // rows instead and multiplies zeros (no branch around the matrix instructions; nothing of it is stored).
    struct Rows {
        const uint8_t * x;      // fragment slabs of the item's first 32-row tile
        const uint8_t * sums;   // block sums of the same tile
        uint32_t x_lane, sums_lane, power_lane;
    };
    auto rows_of = [&](int item) {
        Rows r;
        const int row_start = item_field(item, 1);
        const int first_tile = row_start >> 5;
        r.x = reinterpret_cast<const uint8_t *>(a.qx) + static_cast<int64_t>(first_tile) * blocks_per_row * 2048;
        r.sums = reinterpret_cast<const uint8_t *>(a.block_sums) + static_cast<int64_t>(first_tile) * super_blocks * 512;
        int lane_row = row_start + wave * 32 + l32;
        lane_row = lane_row < a.rows_padded ? lane_row : a.rows_padded - 1;
        r.x_lane = static_cast<uint32_t>((lane_row >> 5) - first_tile) * blocks_per_row * 2048u +
                   static_cast<uint32_t>(((lane_row & 31) + 32 * half) * 16);
        r.sums_lane = static_cast<uint32_t>((lane_row >> 5) - first_tile) * super_blocks * 512u +
                      static_cast<uint32_t>((lane_row & 31) * 16);
        r.power_lane = static_cast<uint32_t>(lane_row) * 4u;
        return r;
    };
    // reduction step `step` (16 values) of the rows: one 1 KiB slab per 32-row tile
    auto load_x = [&](const Rows & r, int step) {
        return *reinterpret_cast<const half8_t *>(r.x + static_cast<int64_t>(step) * 1024 + r.x_lane);
    };
    // 2^(e - E) of the lane's row in super-block kb: what brings the super-block's fragments, which the quantizer
    // normalised by themselves, to the row's common exponent (a power of two: exact; a super-block more than 2^24
    // below the row's largest one vanishes)
    auto load_ratio = [&](const Rows & r, int kb) {
        const uint8_t * base = reinterpret_cast<const uint8_t *>(a.power + static_cast<int64_t>(kb) * a.rows_padded);
        return *reinterpret_cast<const float *>(base + r.power_lane);
    };
    auto rescale = [&](half8_t fragment, half2_t ratio) {
        const uint4 words = __builtin_bit_cast(uint4, fragment);
        const uint4 scaled = make_uint4(half2_mul(words.x, ratio), half2_mul(words.y, ratio), half2_mul(words.z, ratio),
                                        half2_mul(words.w, ratio));
        return __builtin_bit_cast(half8_t, scaled);
    };
    auto load_sums = [&](const Rows & r, int kb) {
        return *reinterpret_cast<const uint4 *>(r.sums + static_cast<int64_t>(kb) * 512 + r.sums_lane);
    };

    // activation fragments are requested a whole stage (FSC_STEPS reduction steps) before their matrix instructions
    Rows rows_next = rows_of(0);   // of the stage being requested
    half8_t x[FSC_STEPS];
#pragma unroll
    for (int i = 0; i < FSC_STEPS; ++i) {
        x[i] = load_x(rows_next, i);
    }

    v16f acc[FWD_NT];
    const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int nt = 0; nt < FWD_NT; ++nt) acc[nt] = zero;

    // weight fragments are read FSC_W_AHEAD reduction steps before their matrix instructions
    constexpr int RING = FSC_W_AHEAD + 1;
    half8_t w[RING][FWD_NT];
    auto read_step = [&](int buffer, int step, half8_t (&out)[FWD_NT]) __attribute__((always_inline)) {
#pragma unroll
        for (int nt = 0; nt < FWD_NT; ++nt) {
            out[nt] = *reinterpret_cast<const half8_t *>(&lds.wq[buffer][((nt * FSC_STEPS + step) * 64 + lane) * 16]);
        }
    };
    // one stage: eight reduction steps from operand tile `buffer` (its first FSC_W_AHEAD steps have been read); every
    // step's activation register is refilled with the same step of the following stage (`next_step` of `rows_next`)
    auto stage_as = [&](auto active_tag, int buffer, int next_step, half2_t ratio) __attribute__((always_inline)) {
        constexpr bool ACTIVE = decltype(active_tag)::value;
#pragma unroll
        for (int s = 0; s < FSC_STEPS; ++s) {
            if constexpr (ACTIVE) {
                if (s + FSC_W_AHEAD < FSC_STEPS) {
                    read_step(buffer, s + FSC_W_AHEAD, w[(s + FSC_W_AHEAD) % RING]);
                }
            }
            const half8_t fragment = rescale(x[s], ratio);
            if constexpr (ACTIVE)
#pragma unroll
            for (int nt = 0; nt < FWD_NT; ++nt) {
                // (weights as the A operand: the lane ends up with one activation row and runs of four neighbouring columns)
                acc[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(w[s % RING][nt], fragment, acc[nt], 0, 0, 0);
            }
            x[s] = load_x(rows_next, next_step + s);
            // (the requests stay where they are written: moved to the end of the stage, as the scheduler would have
            // them, they leave the next stage waiting for memory)
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // (a wave without rows in the item keeps requesting activations, which may be the next item's, but leaves the matrix
    // pipe and the operand tile to the others)
    auto stage = [&](int buffer, int next_step, half2_t ratio, bool active) __attribute__((always_inline)) {
        if (active) {
#pragma unroll
            for (int s = 0; s < FSC_W_AHEAD; ++s) {
                read_step(buffer, s, w[s]);
            }
            stage_as(std::true_type{}, buffer, next_step, ratio);
        } else {
            stage_as(std::false_type{}, buffer, next_step, ratio);
        }
    };
    int item = 0, kb = 0;
    int read = 0, buffer = 0;   // stages read so far; stage g is in buffer g % FSC_BUFFERS
    float ratio_next = load_ratio(rows_next, 0);
#pragma unroll 1
    for (int q = 0; q < total; ++q) {
        // (rows_next: still the rows of this super-block's item, whose stage 0 was requested with them)
        uint4 sums = make_uint4(0, 0, 0, 0);
        if constexpr (K45) {
            sums = load_sums(rows_next, kb);
        }
        // 2^E of the lane's row, for the epilogue (requested with every super-block: one that ends an item has it at hand)
        const float row_power = *reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(a.row_power) + rows_next.power_lane);
        const float ratio_f32 = ratio_next;   // (requested a stage ago: needed at once)
        const bool active = item_field(item, 1) + wave * 32 < item_field(item, 2);
        const half2_t ratio = {static_cast<_Float16>(ratio_f32), static_cast<_Float16>(ratio_f32)};
        // stage 0; requests stage 1 of the same super-block
        wait_produced(read + 1);
        stage(buffer, kb * 16 + 8, ratio, active);
        if constexpr (K45) {
            // the super-block's extra reduction step: block minima x block sums (slots 8..15 of the instruction are
            // empty); the minima lie beside the operand tile of the super-block's first stage
            const half8_t block_sums = rescale(__builtin_bit_cast(half8_t, half != 0 ? make_uint4(0, 0, 0, 0) : sums), ratio);
            if (active)
#pragma unroll
            for (int nt = 0; nt < FWD_NT; ++nt) {
                uint4 minima = *reinterpret_cast<const uint4 *>(&lds.mins[buffer][nt * 512 + l32 * 16]);
                if (half != 0) {
                    minima = make_uint4(0, 0, 0, 0);
                }
                acc[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, minima), block_sums, acc[nt], 0, 0, 0);
            }
        }
        publish(&lds.consumed[wave], ++read);
        buffer = next_buffer(buffer);
        // stage 1; requests stage 0 of the following super-block, which may belong to the next item
        const bool last_of_item = kb + 1 == super_blocks;
        const int item_next = last_of_item ? min(item + 1, n_items - 1) : item;
        const int kb_next = last_of_item ? 0 : kb + 1;
        rows_next = rows_of(item_next);
        ratio_next = load_ratio(rows_next, kb_next);
        wait_produced(read + 1);
        stage(buffer, kb_next * 16, ratio, active);
        publish(&lds.consumed[wave], ++read);
        buffer = next_buffer(buffer);
        if (last_of_item) {
            // The item is complete: scale by 2^(E[r] + S[n]) and store, while the unpacking waves work on the next item.
            const int row_start = item_field(item, 1);
            const int row_end = item_field(item, 2);
            const int tile = item_field(item, 3);
            const bool second = tile >= a.n_tiles;
            const int n0 = (second ? tile - a.n_tiles : tile) * FWD_TN;
            uint16_t * const y = second ? a.y_second : a.y;
            const int r0 = row_start + wave * 32;
            // recomputing the lane's share here is cheaper than keeping it alive through the loop
            const int lane_here = lane_afresh();
            const int l32_here = lane_here & 31, half_here = lane_here >> 5;
            if (r0 < row_end) {
                // one column tile at a time, its powers read when they are needed: read for all four tiles ahead of the
                // stores they no longer fit the registers, and a reload from scratch waits for every store before it
#pragma unroll
                for (int nt = 0; nt < FWD_NT; ++nt) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float4 column_power =
                            *reinterpret_cast<const float4 *>(&lds.row_power[item & 3][nt * 32 + 8 * j + 4 * half_here]);
                        acc[nt][4 * j + 0] *= row_power * column_power.x;
                        acc[nt][4 * j + 1] *= row_power * column_power.y;
                        acc[nt][4 * j + 2] *= row_power * column_power.z;
                        acc[nt][4 * j + 3] *= row_power * column_power.w;
                    }
                    store_rows_32xn<1>(&acc[nt], y + static_cast<int64_t>(r0) * a.out_features + n0 + 32 * nt, a.out_features,
                                       row_end - r0, a.out_features - n0 - 32 * nt, lane_here);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int nt = 0; nt < FWD_NT; ++nt) acc[nt] = zero;
            ++item;
            kb = 0;
        } else {
            ++kb;
        }
    }
}

template <int TYPE>
static hipError_t launch_forward_scaled_typed(const ForwardArgs & call, hipStream_t stream) {
    ForwardArgs args = call;
    const int64_t total = static_cast<int64_t>(args.n_tiles) * args.projections *
                          (args.task_count != nullptr ? xcd_chunk_slots(args.task_slots) : pad_task_slots(args.task_slots, FWD_XCD_RUN));
    // grouped calls: whole groups of at most 32 rows are listed behind the other tasks and go to workgroups of their own,
    // each of which runs up to three such items at a time (one per CU suffices: its groups take items until none is left)
    constexpr int SHORT_GROUPS = FSC_THREADS / (64 * FSS_WAVES);
    const int64_t short_items = args.task_count != nullptr ? static_cast<int64_t>(args.task_slots) * args.n_tiles * args.projections : 0;
    const int64_t short_units = (short_items + SHORT_GROUPS - 1) / SHORT_GROUPS;
    // (rows of fewer than four super-blocks: the short groups get a launch of their own, see short_group_items)
    const bool trailing = args.in_features / QK_K >= 4;
    const int64_t short_blocks = !trailing ? 0 : short_units < FSC_GRID ? short_units : FSC_GRID;
    const int64_t short_grid = trailing ? 0 : short_items < 3 * FSC_GRID ? short_items : 3 * FSC_GRID;
    if (total <= 0 || total > 0x7fffffffLL || args.swiglu != 0 || args.in_features > (1 << 22)) {
        return hipErrorInvalidValue;
    }
    args.early_only = args.task_count != nullptr ? 1 : 0;
    // one role-split workgroup per CU; more when a workgroup's table would not hold its share (a multiple of the XCD
    // count either way, so that a workgroup's items stay on its XCD)
    int64_t grid = FSC_GRID;
    if (total > grid * FSC_MAX_ITEMS) {
        grid = ((total + FSC_MAX_ITEMS - 1) / FSC_MAX_ITEMS + XCDS - 1) / XCDS * XCDS;
    }
    if (total < grid) {
        grid = total;
    }
    const ProfileScope scope(2, stream);
    bool wide = false;
    if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
        wide = args.wide != 0;
    }
    const unsigned blocks = static_cast<unsigned>(grid + short_blocks);
    if (wide) {
        if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
            mmq_forward_scaled_kernel<TYPE, true><<<blocks, FSC_THREADS, 0, stream>>>(args, static_cast<int>(total), static_cast<int>(grid));
        }
    } else {
        mmq_forward_scaled_kernel<TYPE, false><<<blocks, FSC_THREADS, 0, stream>>>(args, static_cast<int>(total), static_cast<int>(grid));
    }
    hipError_t status = hipGetLastError();
    if (status != hipSuccess || short_grid == 0) {
        return status;
    }
    if (wide) {
        if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
            mmq_forward_scaled_short_kernel<TYPE, true><<<static_cast<unsigned>(short_grid), 64 * FSS_WAVES, 0, stream>>>(args);
        }
    } else {
        mmq_forward_scaled_short_kernel<TYPE, false><<<static_cast<unsigned>(short_grid), 64 * FSS_WAVES, 0, stream>>>(args);
    }
    return hipGetLastError();
}

hipError_t launch_forward_scaled(const ForwardArgs & args, int quant_type, hipStream_t stream) {
    switch (quant_type) {
        case Q3_K: return launch_forward_scaled_typed<Q3_K>(args, stream);
        case Q4_K: return launch_forward_scaled_typed<Q4_K>(args, stream);
        case Q5_K: return launch_forward_scaled_typed<Q5_K>(args, stream);
        case Q6_K: return launch_forward_scaled_typed<Q6_K>(args, stream);
        case IQ2_S: return launch_forward_scaled_typed<IQ2_S>(args, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace tgo
