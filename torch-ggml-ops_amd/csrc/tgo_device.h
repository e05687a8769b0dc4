// Device-side building blocks shared by the gfx950 kernels: GGUF super-block geometry, staging of
// packed blocks into LDS, and the per-16-value unpackers that feed the int8 (forward) and bf16
// (grad-input, dequant) operand tiles.  Wave64 throughout.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "iq2s_codebook.h"
#include "tgo_launch.h"

#define TGO_DEVICE static __device__ __forceinline__

namespace tgo {

constexpr int QK_K = 256;

enum QuantType : int {
    Q3_K = 11,
    Q4_K = 12,
    Q5_K = 13,
    Q6_K = 14,
    IQ2_S = 22,
};

// Geometry of one super-block and of its copy in LDS.
//   BLOCK_BYTES  size in the weight tensor (reference: csrc/vendor/llama_cpp/common.cuh:78-127)
//   RAW_SHIFT    byte offset of the copy inside its LDS slot, chosen so that every field the
//                unpackers read as 32-bit words is 4-byte aligned (IQ2_S fields start at +2)
//   RAW_PITCH    LDS slot size per row: 4 * odd, so that rows land on different banks
//   PLANES       int8 planes of the forward weight tile (2 = value split as 128*hi + lo)
//   HAS_MIN      type carries a per-32 minimum (Q4_K, Q5_K)
template <int TYPE> struct Format;
template <> struct Format<Q3_K> { static constexpr int BLOCK_BYTES = 110, RAW_SHIFT = 0, RAW_PITCH = 116, PLANES = 1; static constexpr bool HAS_MIN = false; };
template <> struct Format<Q4_K> { static constexpr int BLOCK_BYTES = 144, RAW_SHIFT = 0, RAW_PITCH = 148, PLANES = 1; static constexpr bool HAS_MIN = true; };
template <> struct Format<Q5_K> { static constexpr int BLOCK_BYTES = 176, RAW_SHIFT = 0, RAW_PITCH = 180, PLANES = 1; static constexpr bool HAS_MIN = true; };
template <> struct Format<Q6_K> { static constexpr int BLOCK_BYTES = 210, RAW_SHIFT = 0, RAW_PITCH = 212, PLANES = 2; static constexpr bool HAS_MIN = false; };
template <> struct Format<IQ2_S> { static constexpr int BLOCK_BYTES = 82, RAW_SHIFT = 2, RAW_PITCH = 84, PLANES = 2; static constexpr bool HAS_MIN = false; };

static inline __host__ __device__ int block_bytes(int quant_type) {
    switch (quant_type) {
        case Q3_K: return 110;
        case Q4_K: return 144;
        case Q5_K: return 176;
        case Q6_K: return 210;
        case IQ2_S: return 82;
        default: return 0;
    }
}

TGO_DEVICE float half_bits_to_float(uint32_t bits16) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(bits16)));
}

TGO_DEVICE uint32_t pack_bf16x2(float lo, float hi) {
    typedef float float2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const float2_t pair = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2_t));
}

TGO_DEVICE uint16_t to_bf16_bits(float value) {
    return static_cast<uint16_t>(pack_bf16x2(value, 0.0f) & 0xffffu);
}

TGO_DEVICE float bf16_bits_to_float(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}

// Hardware workgroups are dealt round-robin to the 8 XCDs (each with its own L2) by linear id.  The
// workgroups of one task (its `inner` column tiles, which share activation rows) are therefore given
// linear ids that are 8 apart, so they run on one XCD, while eight consecutive tasks spread over the
// eight XCDs.  The grid holds inner * task_slots workgroups with task_slots a multiple of 8.
constexpr int XCDS = 8;

// With fewer tasks than XCDs that grouping would leave whole XCDs idle (a dense call of up to one row tile would
// run on an eighth of the chip), so then the tiles of a task are dealt out in plain order, i.e. across the XCDs.
// RUN: consecutive tasks that share an XCD.  (Dense calls and the short tasks of the grad-input; grouped launches,
// where consecutive tasks are row tiles of the same expert, i.e. of the same weights, take xcd_chunk below.)
template <int RUN = 1>
TGO_DEVICE void xcd_tile(int linear, int inner, int tasks, int & inner_id, int & task) {
    if (tasks < XCDS) {
        task = linear / inner;
        inner_id = linear - task * inner;
        return;
    }
    // (with only a few runs' worth of tasks, whole runs per XCD would leave XCDs idle: single tasks then)
    const int run = tasks >= 2 * XCDS * RUN ? RUN : 1;
    const int span = XCDS * inner * run;
    const int group = linear / span;
    const int within = linear - group * span;
    const int slot = within / XCDS;        // position on this XCD: `run` tasks of `inner` tiles each, task by task
    const int run_task = slot / inner;
    task = (group * XCDS + (within % XCDS)) * run + run_task;
    inner_id = slot - run_task * inner;
}

// Grouped launches: consecutive tasks of the list are row tiles of the same expert, i.e. of the same weights, so
// XCD x takes the x-th eighth of the list as one contiguous chunk and an expert's weights are fetched into one L2
// (two where a chunk boundary cuts through it).  The chunks differ by at most one task.  A list may put cheap
// tasks behind the others (`early` = number of ordinary ones): both parts are dealt out that way, so every XCD gets
// its share of either kind and ends with the cheap ones.  The grid holds inner * xcd_chunk_slots(task slots)
// workgroups; a slot past its XCD's chunks returns task = tasks.
TGO_DEVICE void xcd_chunk(int linear, int inner, int tasks, int early, int & inner_id, int & task) {
    if (tasks < XCDS) {
        task = linear / inner;
        inner_id = linear - task * inner;
        return;
    }
    const int xcd = linear % XCDS;
    const int slot = linear / XCDS;
    int t = slot / inner;
    inner_id = slot - t * inner;
    const int late = tasks - early;
    const int early_first = xcd * early / XCDS, early_end = (xcd + 1) * early / XCDS;   // (task counts stay far below 2^28)
    const int late_first = xcd * late / XCDS, late_end = (xcd + 1) * late / XCDS;
    if (t < early_end - early_first) {
        task = early_first + t;
        return;
    }
    t -= early_end - early_first;
    task = t < late_end - late_first ? early + late_first + t : tasks;
}

static inline int xcd_chunk_slots(int slots) { return ((slots + XCDS - 1) / XCDS + 1) * XCDS; }

static inline int pad_task_slots(int slots, int run = 1) { return (slots + XCDS * run - 1) / (XCDS * run) * (XCDS * run); }

// Tile tasks of the grouped operators.  Group g covers rows [offsets[g-1], offsets[g]) of expert indices[g].
// Every valid group is cut into tasks of at most `row_tile` rows; groups with an out-of-range expert, no rows
// or rows outside the input are dropped, as the reference kernels do (csrc/mmq_core.cuh:466-476, :516-571).
// One workgroup of 256 threads (all of them call this) scans the groups 256 at a time, so any group count works
// and no host round trip is needed.  The kernels that consume the list run later in the same stream.
TGO_DEVICE void build_tasks(const TaskBuild & b, int tid) {
    __shared__ int scan[256], scan_late[256];
    __shared__ int running, running_late;
    // Tasks of at most b.late_rows rows (a group's remainder) cost their workgroups a fraction of a full
    // task's time; they go behind all the others so that the grid's last wave of workgroups is made of the
    // short ones.  First sweep: how many tasks come before them.
    // (late_whole_groups: only when that remainder is the whole group; the remainder of a larger group then stays
    // behind the group's other tasks, where xcd_chunk keeps it on the XCD that already holds the expert's weights)
    const auto listed_late = [&](int size) {
        const int rest = size % b.row_tile;
        return rest > 0 && rest <= b.late_rows && (b.late_whole_groups == 0 || size <= b.late_rows) ? 1 : 0;
    };
    int early_total = 0;
    if (b.late_rows > 0) {
        int mine = 0;
        for (int group = tid; group < b.num_groups; group += 256) {
            const int row_begin = group == 0 ? 0 : b.expert_offsets[group - 1];
            const int row_end = b.expert_offsets[group];
            const int64_t expert64 = b.expert_indices[group];
            if (expert64 >= 0 && expert64 < b.num_experts && row_begin >= 0 && row_end > row_begin && row_end <= b.rows) {
                const int size = row_end - row_begin;
                mine += (size + b.row_tile - 1) / b.row_tile - listed_late(size);
            }
        }
        scan[tid] = mine;
        __syncthreads();
        for (int offset = 128; offset > 0; offset >>= 1) {
            if (tid < offset) {
                scan[tid] += scan[tid + offset];
            }
            __syncthreads();
        }
        early_total = scan[0];
        __syncthreads();
    }
    if (tid == 0) {
        running = 0;
        running_late = 0;
    }
    __syncthreads();
    for (int base = 0; base < b.num_groups; base += 256) {
        const int group = base + tid;
        int row_begin = 0, row_end = 0, expert = -1, count = 0, late = 0;
        if (group < b.num_groups) {
            row_begin = group == 0 ? 0 : b.expert_offsets[group - 1];
            row_end = b.expert_offsets[group];
            const int64_t expert64 = b.expert_indices[group];
            if (expert64 >= 0 && expert64 < b.num_experts && row_begin >= 0 && row_end > row_begin && row_end <= b.rows) {
                expert = static_cast<int>(expert64);
                const int size = row_end - row_begin;
                count = (size + b.row_tile - 1) / b.row_tile;
                late = listed_late(size);
            }
        }
        scan[tid] = count - late;
        scan_late[tid] = late;
        __syncthreads();
        for (int offset = 1; offset < 256; offset <<= 1) {
            const int add = tid >= offset ? scan[tid - offset] : 0;
            const int add_late = tid >= offset ? scan_late[tid - offset] : 0;
            __syncthreads();
            scan[tid] += add;
            scan_late[tid] += add_late;
            __syncthreads();
        }
        const int first = running + scan[tid] - (count - late);
        const int first_late = early_total + running_late + scan_late[tid] - late;
        for (int t = 0; t < count; ++t) {
            const int index = t == count - 1 && late ? first_late : first + t;
            if (index < b.tasks.max_tasks) {
                const int start = row_begin + t * b.row_tile;
                b.tasks.expert[index] = expert;
                b.tasks.row_start[index] = start;
                b.tasks.row_end[index] = min(start + b.row_tile, row_end);
            }
        }
        __syncthreads();
        if (tid == 255) {
            running += scan[255];
            running_late += scan_late[255];
        }
        __syncthreads();
    }
    if (tid == 0) {
        b.tasks.count[0] = min(running + running_late, b.tasks.max_tasks);
        b.tasks.early[0] = min(running, b.tasks.max_tasks);
    }
    if (tid < TASK_CURSORS) {
        b.tasks.cursor[tid * TASK_CURSOR_STRIDE] = 0;
    }
}

// Expands the 2-bit codebook into 1024 64-bit words of LDS (8 KiB).  All threads of the block call it.
TGO_DEVICE void expand_iq2s_grid(uint2 * grid_lds, int tid, int nthreads) {
    for (int i = tid; i < TGO_IQ2S_GRID_ENTRIES; i += nthreads) {
        const uint32_t packed = tgo_iq2s_packed[i];
        uint32_t words[2];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t digit = (packed >> (2 * (4 * w + e))) & 3u;
                // {8, 25, 43}[digit] = 8 + 17*digit + (digit >> 1)
                word |= (8u + 17u * digit + (digit >> 1)) << (8 * e);
            }
            words[w] = word;
        }
        grid_lds[i] = make_uint2(words[0], words[1]);
    }
}

// The same in two steps for kernels that have other memory round trips to start first: the packed entries are
// requested early (ENTRIES_PER_THREAD = 1024 / threads of the block) and expanded once the other requests are out.
template <int ENTRIES_PER_THREAD>
TGO_DEVICE void request_iq2s_grid(uint32_t (&packed)[ENTRIES_PER_THREAD], int tid) {
#pragma unroll
    for (int j = 0; j < ENTRIES_PER_THREAD; ++j) {
        packed[j] = tgo_iq2s_packed[tid + j * (TGO_IQ2S_GRID_ENTRIES / ENTRIES_PER_THREAD)];
    }
}
template <int ENTRIES_PER_THREAD>
TGO_DEVICE void expand_iq2s_grid(uint2 * grid_lds, const uint32_t (&packed)[ENTRIES_PER_THREAD], int tid) {
#pragma unroll
    for (int j = 0; j < ENTRIES_PER_THREAD; ++j) {
        uint32_t words[2];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t digit = (packed[j] >> (2 * (4 * w + e))) & 3u;
                word |= (8u + 17u * digit + (digit >> 1)) << (8 * e);
            }
            words[w] = word;
        }
        grid_lds[tid + j * (TGO_IQ2S_GRID_ENTRIES / ENTRIES_PER_THREAD)] = make_uint2(words[0], words[1]);
    }
}

// Copies `nrows` super-blocks (block column `kb` of consecutive weight rows starting at `row0`) into
// LDS slots of RAW_PITCH bytes.  Rows past `row_limit - 1` re-read the last valid row; callers mask
// what they compute from them.
template <int TYPE>
TGO_DEVICE void stage_blocks(uint8_t * raw, const uint8_t * weights, int64_t row_bytes, int row0,
                             int row_limit, int kb, int nrows, int tid, int nthreads) {
    using F = Format<TYPE>;
    // All loads of a batch are issued before the first store, so a thread waits for memory once per batch
    // instead of once per load.
    if constexpr (F::BLOCK_BYTES % 16 == 0) {
        constexpr int UNITS = F::BLOCK_BYTES / 16;
        constexpr int BATCH = 4;
        const int total = nrows * UNITS;
        for (int base = tid; base < total; base += nthreads * BATCH) {
            uint4 value[BATCH];
            int slot[BATCH];
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const int id = min(base + b * nthreads, total - 1);
                const int row = id / UNITS;
                const int unit = id - row * UNITS;
                int src_row = row0 + row;
                src_row = src_row < row_limit ? src_row : row_limit - 1;
                value[b] = *reinterpret_cast<const uint4 *>(
                    weights + src_row * row_bytes + static_cast<int64_t>(kb) * F::BLOCK_BYTES + unit * 16);
                slot[b] = row * F::RAW_PITCH + unit * 16;
            }
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                if (base + b * nthreads < total) {
                    uint32_t * dst = reinterpret_cast<uint32_t *>(raw + slot[b]);
                    dst[0] = value[b].x; dst[1] = value[b].y; dst[2] = value[b].z; dst[3] = value[b].w;
                }
            }
        }
    } else {
        constexpr int UNITS = F::BLOCK_BYTES / 2;
        constexpr int BATCH = 16;
        const int total = nrows * UNITS;
        for (int base = tid; base < total; base += nthreads * BATCH) {
            uint16_t value[BATCH];
            int slot[BATCH];
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const int id = min(base + b * nthreads, total - 1);
                const int row = id / UNITS;
                const int unit = id - row * UNITS;
                int src_row = row0 + row;
                src_row = src_row < row_limit ? src_row : row_limit - 1;
                value[b] = *reinterpret_cast<const uint16_t *>(
                    weights + src_row * row_bytes + static_cast<int64_t>(kb) * F::BLOCK_BYTES + unit * 2);
                slot[b] = row * F::RAW_PITCH + F::RAW_SHIFT + unit * 2;
            }
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                if (base + b * nthreads < total) {
                    *reinterpret_cast<uint16_t *>(raw + slot[b]) = value[b];
                }
            }
        }
    }
}

// ---- register-staged copy for the formats whose blocks are only 2-byte aligned (Q3_K, Q6_K, IQ2_S) ------------
// stage_blocks moves such blocks two bytes per load, issued where the data is needed.  A block can instead be
// fetched as the 16-byte aligned units of memory that cover it, a whole reduction step ahead, into registers.  A
// block then starts m = (its address) % 16 bytes into its first unit, an even number that differs from row to
// row.  On the way to LDS the odd part of that (m & 2) is taken out with a byte alignment of neighbouring words
// (each unit carries the first word of the next one for this), the rest (m & 12) by where the words are
// written, so that the block's first byte lands on the 4-byte aligned position FRONT of its slot and every field
// the unpackers read as words is aligned.  The up to 12 bytes in front of a block and the bytes behind it that
// come along land in the slot's own padding.  Units that lie entirely behind the block are not fetched (the lane
// repeats unit 0).  The first unit starts at or after the 16-byte aligned start of the weight tensor and the
// last one ends at or before its end rounded up to 16: wide_stage_ok() says when both lie inside the tensor.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <int TYPE>
struct WideStage {
    static constexpr int BLOCK = Format<TYPE>::BLOCK_BYTES;
    static constexpr int UNITS = (BLOCK + 14 + 15) / 16;       // units that cover a block at any even misalignment
    static constexpr int FRONT = 12;                           // slot offset of the block's first byte
    static constexpr int SPAN = FRONT + 16 * UNITS;            // bytes a slot may receive
    static constexpr int PITCH = (SPAN / 4) % 2 == 1 ? SPAN : SPAN + 4;   // 4 * odd: rows spread over the banks
    static constexpr int RECIPROCAL = (65536 + UNITS - 1) / UNITS;        // id -> id / UNITS, exact below 3000
    template <int NROWS, int THREADS>
    static constexpr int regs() { return (NROWS * UNITS + THREADS - 1) / THREADS; }
};

// Whether the tensor of one expert may be read in whole aligned units: its first and last byte are unit
// boundaries (the bytes of an expert end where the next expert's begin, so this covers stacked experts).
static __host__ __device__ inline bool wide_stage_ok(const void * packed, int64_t bytes_per_expert) {
    return (reinterpret_cast<uintptr_t>(packed) & 15) == 0 && (bytes_per_expert & 15) == 0;
}

template <int REGS>
struct WideRegs {
    u32x4_t unit[REGS];
    uint32_t next[REGS];   // first word of the following unit
};

// `tile`: first byte of weight row 0 of the tile (wave-uniform); rows past rows_valid - 1 repeat the last valid
// row.  (rows_valid * row_bytes + the bytes of a row) must stay below 2^31.
template <int TYPE, int NROWS, int THREADS, int REGS>
TGO_DEVICE void wide_fetch(WideRegs<REGS> & regs, const uint8_t * tile, int row_bytes, int rows_valid, int kb, int t) {
    using W = WideStage<TYPE>;
    static_assert(NROWS * W::UNITS < 3000, "range of the reciprocal");
    const uint32_t tile_m = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(tile)) & 15u;
    const uint8_t * const aligned = tile - tile_m;
    const uint32_t column = tile_m + static_cast<uint32_t>(kb) * W::BLOCK;
#pragma unroll
    for (int i = 0; i < REGS; ++i) {
        const int id = min(t + THREADS * i, NROWS * W::UNITS - 1);
        const int row = static_cast<int>(__umul24(id, W::RECIPROCAL) >> 16);
        int unit = id - row * W::UNITS;
        const uint32_t first = __umul24(min(row, rows_valid - 1), row_bytes) + column;   // of the block, from `aligned`
        const int reach = static_cast<int>(first & 15u) + W::BLOCK;                      // block end, from its first unit
        const bool carries = 16 * (unit + 1) < reach;   // the following unit still holds bytes of the block
        unit = 16 * unit < reach ? unit : 0;
        const uint32_t offset = (first & ~15u) + 16u * unit;
        regs.unit[i] = *reinterpret_cast<const u32x4_t *>(aligned + offset);
        // (where nothing of the block follows, the word is never looked at: the lane re-reads its own unit
        // rather than branching around the load)
        regs.next[i] = *reinterpret_cast<const uint32_t *>(aligned + offset + (carries ? 16u : 0u));
    }
}

// Writes what wide_fetch brought (same arguments) into slots of WideStage::PITCH bytes; the block of row r then
// starts at raw + r * PITCH + FRONT.
template <int TYPE, int NROWS, int THREADS, int REGS>
TGO_DEVICE void wide_park(uint8_t * raw, const WideRegs<REGS> & regs, const uint8_t * tile, int row_bytes,
                          int rows_valid, int kb, int t) {
    using W = WideStage<TYPE>;
    const uint32_t column = (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(tile)) & 15u) + static_cast<uint32_t>(kb) * W::BLOCK;
#pragma unroll
    for (int i = 0; i < REGS; ++i) {
        // (ids past the tile repeated its last unit in wide_fetch: they write the same words to the same place)
        const int id = min(t + THREADS * i, NROWS * W::UNITS - 1);
        const int row = static_cast<int>(__umul24(id, W::RECIPROCAL) >> 16);
        const int unit = id - row * W::UNITS;
        const uint32_t m = (__umul24(min(row, rows_valid - 1), row_bytes) + column) & 15u;
        const uint32_t shift = m & 2u;
        const u32x4_t d = regs.unit[i];
        uint32_t * dst = reinterpret_cast<uint32_t *>(raw + row * W::PITCH + W::FRONT - (m & 12u) + 16 * unit);
        dst[0] = __builtin_amdgcn_alignbyte(d.y, d.x, shift);
        dst[1] = __builtin_amdgcn_alignbyte(d.z, d.y, shift);
        dst[2] = __builtin_amdgcn_alignbyte(d.w, d.z, shift);
        dst[3] = __builtin_amdgcn_alignbyte(regs.next[i], d.w, shift);
    }
}

TGO_DEVICE uint32_t lds_u32(const uint8_t * p) { return *reinterpret_cast<const uint32_t *>(p); }
TGO_DEVICE uint32_t lds_u16(const uint8_t * p) { return *reinterpret_cast<const uint16_t *>(p); }

// 6-bit scale and min of 32-value group `g` of a Q4_K/Q5_K block (12 bytes at blk+4).
TGO_DEVICE void k_scale_min(const uint8_t * scales, int g, int & sc, int & mn) {
    if (g < 4) {
        sc = scales[g] & 0x3f;
        mn = scales[4 + g] & 0x3f;
    } else {
        const int j = g - 4;
        sc = (scales[8 + j] & 0x0f) | ((scales[j] >> 2) & 0x30);
        mn = (scales[8 + j] >> 4) | ((scales[4 + j] >> 2) & 0x30);
    }
}

// Integer view of 16 consecutive weights (unit u = values 16u .. 16u+15 of a super-block):
//   q[16]   signed integer quants
//   sub     integer scale shared by the 16 values (Q4_K/Q5_K: 6-bit scale of the 32-group,
//           Q3_K: sc-32, Q6_K: int8 scale, IQ2_S: the 4-bit s)
//   mn      6-bit min of the 32-group (Q4_K/Q5_K), else 0
// `blk` points at the block's first byte inside its LDS slot (slot base + RAW_SHIFT).
// Follows the value definition of the reference's scalar decoder (csrc/ck/gguf_decode.cuh:54-149).
template <int TYPE>
TGO_DEVICE void unpack16(const uint8_t * blk, int u, const uint2 * grid, int (&q)[16], int & sub, int & mn) {
    mn = 0;
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        const int g = u >> 1;
        const int h = u & 1;
        constexpr int QS = TYPE == Q4_K ? 16 : 48;
        const uint8_t * qs = blk + QS + (g >> 1) * 32 + 16 * h;
        const int shift = 4 * (g & 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t word = lds_u32(qs + 4 * t) >> shift;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                q[4 * t + e] = (word >> (8 * e)) & 0x0f;
            }
        }
        if constexpr (TYPE == Q5_K) {
            const uint8_t * qh = blk + 16 + 16 * h;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t word = lds_u32(qh + 4 * t) >> g;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    q[4 * t + e] |= ((word >> (8 * e)) & 1) << 4;
                }
            }
        }
        k_scale_min(blk + 4, g, sub, mn);
    } else if constexpr (TYPE == Q6_K) {
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
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                q[4 * t + e] = static_cast<int>(((low >> (8 * e)) & 0x0f) | (((high >> (8 * e)) & 3) << 4)) - 32;
            }
        }
        sub = static_cast<int8_t>(blk[192 + u]);
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
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int lo2 = (low >> (8 * e)) & 3;
                const int keep = (high >> (8 * e)) & 1;
                q[4 * t + e] = lo2 - ((keep ^ 1) << 2);
            }
        }
        const uint8_t * scales = blk + 96;
        const int low = scales[u & 7] >> (4 * (u >> 3));
        const int high = scales[8 + (u & 3)] >> (2 * (u >> 2));
        sub = ((low & 0x0f) | ((high & 3) << 4)) - 32;
    } else {  // IQ2_S
        const uint8_t * qs = blk + 2;
        const uint32_t idx_pair = lds_u16(qs + 2 * u);
        const uint32_t sign_pair = lds_u16(qs + 32 + 2 * u);
        const uint32_t qh = blk[66 + (u >> 1)] >> (4 * (u & 1));
#pragma unroll
        for (int gsel = 0; gsel < 2; ++gsel) {
            const uint32_t index = ((idx_pair >> (8 * gsel)) & 0xff) | (((qh >> (2 * gsel)) & 3) << 8);
            const uint2 word = grid[index];
            const uint32_t signs = (sign_pair >> (8 * gsel)) & 0xff;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int magnitude = ((e < 4 ? word.x : word.y) >> (8 * (e & 3))) & 0xff;
                q[8 * gsel + e] = ((signs >> e) & 1) ? -magnitude : magnitude;
            }
        }
        sub = (blk[74 + (u >> 1)] >> (4 * (u & 1))) & 0x0f;
    }
}

// IQ2_S has only three magnitudes (8, 25, 43), so a 16-value unit, whose values share one fp32 factor t, takes only
// six different bf16 numbers: +-bf16(t * 8), +-bf16(t * 25), +-bf16(t * 43).  The dequantizing kernels therefore
// round three products per unit and let every value pick its number with a byte permute instead of converting and
// multiplying each value: the table below holds, per codebook entry, the permute selectors of its eight values
// (two values per selector word; a value's two selector bytes are 2 * digit and 2 * digit + 1, which address
// the pair (bf16(t*8), bf16(t*25)) and, as bytes 4 and 5, bf16(t*43)).  16 KiB of LDS.
struct Iq2sSelectors {
    uint4 entry[TGO_IQ2S_GRID_ENTRIES];
};
TGO_DEVICE void expand_iq2s_selectors(Iq2sSelectors & table, int tid, int nthreads) {
    for (int i = tid; i < TGO_IQ2S_GRID_ENTRIES; i += nthreads) {
        const uint32_t packed = tgo_iq2s_packed[i];
        uint32_t words[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const uint32_t first = (packed >> (4 * p)) & 3u, second = (packed >> (4 * p + 2)) & 3u;
            words[p] = 0x01000100u + first * 0x0202u + second * 0x02020000u;
        }
        table.entry[i] = make_uint4(words[0], words[1], words[2], words[3]);
    }
}

// fp32 value of 16 consecutive weights, operation order of the reference decoder:
//   Q4_K/Q5_K (d*sc)*q - dmin*m ; Q3_K/Q6_K (d*sc)*q ; IQ2_S ((d*(0.5+s))*0.25)*q
template <int TYPE>
TGO_DEVICE void decode16_f32(const uint8_t * blk, int u, const uint2 * grid, float (&w)[16]) {
    if constexpr (TYPE == Q3_K || TYPE == Q6_K) {
        // Four quants per 32-bit operation as unsigned bytes b = q + BIAS (BIAS = 4 resp. 32), then a
        // byte-to-float conversion, an exact subtraction and the reference's multiplication (d * sc) * q per
        // value.  (A fused scale * b - BIAS * scale would round identically but turn the reference's -0.0, for
        // q = 0 under a negative scale, into +0.0.)
        constexpr int BIAS = TYPE == Q3_K ? 4 : 32;
        uint32_t words[4];
        int sub;
        float d;
        if constexpr (TYPE == Q3_K) {
            const int i0 = 16 * u;
            const uint8_t * qs = blk + 32 + (i0 >> 7) * 32 + (i0 & 31);
            const uint8_t * hm = blk + (i0 & 31);
            const int shift_l = 2 * ((i0 & 127) >> 5);
            const int shift_h = i0 >> 5;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t low = lds_u32(qs + 4 * t) >> shift_l;
                const uint32_t high = lds_u32(hm + 4 * t) >> shift_h;
                words[t] = (low & 0x03030303u) | ((high & 0x01010101u) << 2);
            }
            const uint8_t * scales = blk + 96;
            const int low = scales[u & 7] >> (4 * (u >> 3));
            const int high = scales[8 + (u & 3)] >> (2 * (u >> 2));
            sub = ((low & 0x0f) | ((high & 3) << 4)) - 32;
            d = half_bits_to_float(lds_u16(blk + 108));
        } else {
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
                words[t] = (low & 0x0f0f0f0fu) | ((high & 0x03030303u) << 4);
            }
            sub = static_cast<int8_t>(blk[192 + u]);
            d = half_bits_to_float(lds_u16(blk + 208));
        }
        const float scale = d * static_cast<float>(sub);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float q = static_cast<float>((words[i >> 2] >> (8 * (i & 3))) & 0xffu) - static_cast<float>(BIAS);
            w[i] = scale * q;
        }
        return;
    }
    int q[16];
    int sub, mn;
    unpack16<TYPE>(blk, u, grid, q, sub, mn);
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        const float scale = half_bits_to_float(lds_u16(blk)) * static_cast<float>(sub);
        const float minimum = half_bits_to_float(lds_u16(blk + 2)) * static_cast<float>(mn);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            w[i] = scale * static_cast<float>(q[i]) - minimum;
        }
    } else if constexpr (TYPE == IQ2_S) {
        const float scale = (half_bits_to_float(lds_u16(blk)) * (0.5f + static_cast<float>(sub))) * 0.25f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            w[i] = scale * static_cast<float>(q[i]);
        }
    } else {
        constexpr int D_OFFSET = TYPE == Q3_K ? 108 : 208;
        const float scale = half_bits_to_float(lds_u16(blk + D_OFFSET)) * static_cast<float>(sub);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            w[i] = scale * static_cast<float>(q[i]);
        }
    }
}

// 16 consecutive weights as bf16, two per word (values 2i and 2i + 1 in word i), bit-identical to rounding
// decode16_f32's results.  `codebook`: the magnitude grid, or for IQ2_S the selector table above.
template <int TYPE, typename Codebook>
TGO_DEVICE void decode16_bf16(const uint8_t * blk, int u, const Codebook * codebook, uint32_t (&pairs)[8]) {
    if constexpr (TYPE == IQ2_S && std::is_same_v<Codebook, Iq2sSelectors>) {
        const uint8_t * qs = blk + 2;
        const uint32_t idx_pair = lds_u16(qs + 2 * u);
        const uint32_t sign_pair = lds_u16(qs + 32 + 2 * u);
        const uint32_t qh = blk[66 + (u >> 1)] >> (4 * (u & 1));
        const int sub = (blk[74 + (u >> 1)] >> (4 * (u & 1))) & 0x0f;
        // the reference's ((d * (0.5 + s)) * 0.25) * q with q = +-m: the magnitude of the product does not depend on
        // the signs, and rounding is symmetric, so the three candidates are formed from |t| and every value gets
        // the sign of t xor its own sign bit
        const float t = (half_bits_to_float(lds_u16(blk)) * (0.5f + static_cast<float>(sub))) * 0.25f;
        const float magnitude = __builtin_fabsf(t);
        const uint32_t low_pair = pack_bf16x2(magnitude * 8.0f, magnitude * 25.0f);
        const uint32_t high = pack_bf16x2(magnitude * 43.0f, 0.0f);
        // sign of value 2i at bit 2i, of value 2i + 1 at bit 2i + 16: shifted left by 15 - 2i they are the sign bits of
        // the two halves of word i
        uint32_t spread = (sign_pair & 0x5555u) | ((sign_pair & 0xaaaau) << 15);
        spread ^= static_cast<uint32_t>(static_cast<int>(__builtin_bit_cast(uint32_t, t)) >> 31) & 0x55555555u;
#pragma unroll
        for (int gsel = 0; gsel < 2; ++gsel) {
            const uint32_t index = ((idx_pair >> (8 * gsel)) & 0xff) | (((qh >> (2 * gsel)) & 3) << 8);
            const uint4 selector = codebook->entry[index];
            const uint32_t words[4] = {selector.x, selector.y, selector.z, selector.w};
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int i = 4 * gsel + p;
                const uint32_t picked = __builtin_amdgcn_perm(high, low_pair, words[p]);
                pairs[i] = ((spread << (15 - 2 * i)) & 0x80008000u) | (picked & 0x7fff7fffu);
            }
        }
    } else {
        float w[16];
        decode16_f32<TYPE>(blk, u, codebook, w);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pairs[i] = pack_bf16x2(w[2 * i], w[2 * i + 1]);
        }
    }
}

// int8 operand of the forward dot products for 16 consecutive weights, as 4 dwords per plane.
// The integer sub-scale of the 16-value groups is folded into the int8 values so that one fp32 scale
// per 32 values is left (forward_block_scale):
//   Q4_K/Q5_K  v = q                      (0..31), scale d*sc, min dmin*m
//   Q3_K       v = -(sc-32)*q             in [-128, 124], scale -d
//   Q6_K       v = sc*q  = 128*hi + lo    lo in [-64, 63], scale d
//   IQ2_S      v = (2s+1)*q = 128*hi + lo               , scale d/8
template <int TYPE>
TGO_DEVICE void decode16_int8(const uint8_t * blk, int u, const uint2 * grid, uint32_t (&lo)[4], uint32_t (&hi)[4]) {
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        // four quants per 32-bit operation: nibble select, plus the fifth bit for Q5_K
        const int g = u >> 1;
        const int h = u & 1;
        constexpr int QS = TYPE == Q4_K ? 16 : 48;
        const uint8_t * qs = blk + QS + (g >> 1) * 32 + 16 * h;
        const int shift = 4 * (g & 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            lo[t] = (lds_u32(qs + 4 * t) >> shift) & 0x0f0f0f0fu;
            hi[t] = 0;
            if constexpr (TYPE == Q5_K) {
                lo[t] |= ((lds_u32(blk + 16 + 16 * h + 4 * t) >> g) & 0x01010101u) << 4;
            }
        }
        return;
    }
    if constexpr (TYPE == Q3_K) {
        // Four values per 32-bit operation.  With b = low bits | high bit << 2 (0..7) the quant is b - 4 and the
        // operand byte is -sub * (b - 4), sub = sc - 32.  For sub <= 0 that is s * b - 4 s with s = -sub; for
        // sub > 0 it is s * (b ^ 7) - 3 s with s = sub.  Either way: one multiply of the four packed bytes by s
        // (no byte exceeds 224, so nothing carries into its neighbour) and one byte-wise subtraction of a
        // constant, z = ((x | H) - (y & ~H)) ^ ((x ^ ~y) & H) with H = 0x80 in every byte; the result is the
        // two's-complement byte, which always lies in [-128, 124].
        const int i0 = 16 * u;
        const uint8_t * qs = blk + 32 + (i0 >> 7) * 32 + (i0 & 31);
        const uint8_t * hm = blk + (i0 & 31);
        const int shift_l = 2 * ((i0 & 127) >> 5);
        const int shift_h = i0 >> 5;
        const uint8_t * scales = blk + 96;
        const int low = scales[u & 7] >> (4 * (u >> 3));
        const int high = scales[8 + (u & 3)] >> (2 * (u >> 2));
        const int sub = ((low & 0x0f) | ((high & 3) << 4)) - 32;
        const uint32_t s = static_cast<uint32_t>(sub < 0 ? -sub : sub);
        const uint32_t flip = sub > 0 ? 0x07070707u : 0u;
        const uint32_t y = (sub > 0 ? 3u * s : 4u * s) * 0x01010101u;
        constexpr uint32_t H = 0x80808080u;
        const uint32_t y_low = y & ~H;
        const uint32_t y_not = ~y;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t low_bits = lds_u32(qs + 4 * t) >> shift_l;
            const uint32_t high_bit = lds_u32(hm + 4 * t) >> shift_h;
            const uint32_t b = (low_bits & 0x03030303u) | ((high_bit & 0x01010101u) << 2);
            const uint32_t x = (b ^ flip) * s;
            lo[t] = ((x | H) - y_low) ^ ((x ^ y_not) & H);
            hi[t] = 0;
        }
        return;
    }
    if constexpr (TYPE == Q6_K) {
        // Four values per step, as two pairs of 16-bit lanes (bytes 0 and 2, bytes 1 and 3 of a word).  With
        // b = q + 32 (0..63): t = sc * b + (64 - 32 sc) = sc * q + 64, one packed multiply-add; the low plane is
        // (t & 127) - 64, of which only the low byte is kept, the high plane t >> 7 (arithmetic), since
        // sc * q - low = t - (t & 127).  |sc * q| <= 4096, so nothing leaves its 16-bit lane.
        typedef short pair16 __attribute__((ext_vector_type(2)));
        typedef unsigned short upair16 __attribute__((ext_vector_type(2)));
        const int chunk = u >> 3;
        const int rem = (16 * u) & 127;
        const uint8_t * ql = blk + chunk * 64 + (rem & 63);
        const uint8_t * qh = blk + 128 + chunk * 32 + ((16 * u) & 31);
        const int shift_l = 4 * (rem >> 6);
        const int shift_h = 2 * ((rem >> 5) & 3);
        const short sc = static_cast<int8_t>(blk[192 + u]);
        const short offset = static_cast<short>(64 - 32 * sc);
        const pair16 scale = {sc, sc};
        const pair16 shift = {offset, offset};
        const pair16 mask7 = {127, 127};
        const pair16 rebias = {192, 192};   // -64 modulo 256: only the low byte of a lane is kept
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t low = lds_u32(ql + 4 * t) >> shift_l;
            const uint32_t high = lds_u32(qh + 4 * t) >> shift_h;
            const uint32_t b = (low & 0x0f0f0f0fu) | ((high & 0x03030303u) << 4);
            const pair16 even = __builtin_bit_cast(pair16, b & 0x00ff00ffu);
            const pair16 odd = __builtin_bit_cast(pair16, (b >> 8) & 0x00ff00ffu);
            const pair16 t_even = even * scale + shift;
            const pair16 t_odd = odd * scale + shift;
            const uint32_t low_even = __builtin_bit_cast(uint32_t, (t_even & mask7) + rebias);
            const uint32_t low_odd = __builtin_bit_cast(uint32_t, (t_odd & mask7) + rebias);
            const uint32_t high_even = __builtin_bit_cast(uint32_t, t_even >> 7);
            const uint32_t high_odd = __builtin_bit_cast(uint32_t, t_odd >> 7);
            // bytes (even.0, odd.0, even.2, odd.2)
            lo[t] = __builtin_amdgcn_perm(low_odd, low_even, 0x06020400u);
            hi[t] = __builtin_amdgcn_perm(high_odd, high_even, 0x06020400u);
        }
        return;
    }
    if constexpr (TYPE == IQ2_S) {
        // The same two-lane arithmetic: the codebook word holds four magnitudes m, p = (2 s + 1) * m <= 1333 is one
        // packed multiply, the sign bits become lane masks (0 or -1) that negate p as (p ^ mask) - mask, and
        // t = +-p + 64 splits into the planes as above.
        typedef short pair16 __attribute__((ext_vector_type(2)));
        const uint8_t * qs = blk + 2;
        const uint32_t idx_pair = lds_u16(qs + 2 * u);
        const int sign_pair = static_cast<int>(lds_u16(qs + 32 + 2 * u));
        const uint32_t qh = blk[66 + (u >> 1)] >> (4 * (u & 1));
        const short multiplier = static_cast<short>(2 * ((blk[74 + (u >> 1)] >> (4 * (u & 1))) & 0x0f) + 1);
        const pair16 scale = {multiplier, multiplier};
        const pair16 bias = {64, 64};
        const pair16 mask7 = {127, 127};
        const pair16 rebias = {192, 192};
#pragma unroll
        for (int gsel = 0; gsel < 2; ++gsel) {
            const uint32_t index = ((idx_pair >> (8 * gsel)) & 0xff) | (((qh >> (2 * gsel)) & 3) << 8);
            const uint2 word = grid[index];
#pragma unroll
            for (int part = 0; part < 2; ++part) {
                const uint32_t w = part == 0 ? word.x : word.y;
                const int bit = 8 * gsel + 4 * part;   // sign bit of the word's first value
                const pair16 even = __builtin_bit_cast(pair16, w & 0x00ff00ffu);
                const pair16 odd = __builtin_bit_cast(pair16, (w >> 8) & 0x00ff00ffu);
                // (two sign-extended one-bit fields, low halves side by side)
                const pair16 mask_even = __builtin_bit_cast(pair16, __builtin_amdgcn_perm(
                    static_cast<uint32_t>(__builtin_amdgcn_sbfe(sign_pair, bit + 2, 1)),
                    static_cast<uint32_t>(__builtin_amdgcn_sbfe(sign_pair, bit, 1)), 0x05040100u));
                const pair16 mask_odd = __builtin_bit_cast(pair16, __builtin_amdgcn_perm(
                    static_cast<uint32_t>(__builtin_amdgcn_sbfe(sign_pair, bit + 3, 1)),
                    static_cast<uint32_t>(__builtin_amdgcn_sbfe(sign_pair, bit + 1, 1)), 0x05040100u));
                const pair16 t_even = ((even * scale) ^ mask_even) - mask_even + bias;
                const pair16 t_odd = ((odd * scale) ^ mask_odd) - mask_odd + bias;
                const uint32_t low_even = __builtin_bit_cast(uint32_t, (t_even & mask7) + rebias);
                const uint32_t low_odd = __builtin_bit_cast(uint32_t, (t_odd & mask7) + rebias);
                const uint32_t high_even = __builtin_bit_cast(uint32_t, t_even >> 7);
                const uint32_t high_odd = __builtin_bit_cast(uint32_t, t_odd >> 7);
                lo[2 * gsel + part] = __builtin_amdgcn_perm(low_odd, low_even, 0x06020400u);
                hi[2 * gsel + part] = __builtin_amdgcn_perm(high_odd, high_even, 0x06020400u);
            }
        }
        return;
    }
    int q[16];
    int sub, mn;
    unpack16<TYPE>(blk, u, grid, q, sub, mn);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        lo[t] = 0;
        hi[t] = 0;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        int low, high = 0;
        if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
            low = q[i];
        } else if constexpr (TYPE == Q3_K) {
            low = -(sub * q[i]);
        } else {
            const int value = (TYPE == Q6_K ? sub : 2 * sub + 1) * q[i];
            low = ((value + 64) & 127) - 64;
            high = (value - low) >> 7;
        }
        lo[i >> 2] |= static_cast<uint32_t>(low & 0xff) << (8 * (i & 3));
        hi[i >> 2] |= static_cast<uint32_t>(high & 0xff) << (8 * (i & 3));
    }
}

// ---- exact small integers as fp16 (the forward's matrix operand) --------------------------------
// The forward multiplies integers: quantized activations (|q| <= 127) and weight operands v = integer sub-scale x
// quant.  Both are exactly representable in fp16 when |v| <= 2048 (or has enough trailing zero bits), every
// product is exact in the fp32 accumulator of the matrix instruction, and the sum over a 32-value block stays
// below 2^24, so the fp16 matrix instruction returns the integer dot product without any rounding, already as
// a float.  Operand per format:
//   Q4_K/Q5_K  sc * q            (<= 63 * 31), the weight scale left over is d per super-block
//   Q3_K       (sc - 32) * q     (|.| <= 128), scale d
//   IQ2_S      +-(2 s + 1) * m   (<= 31 * 43), scale d / 8
//   Q6_K       sc * q, |.| <= 4096, as two operands (|sc| & ~15) * q and (|sc| & 15) * q, both with the sign of sc,
//              whose products accumulate in the same fp32 result (4096 * 127 * 32 < 2^24), scale d
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));

// Four unsigned bytes -> two registers of two fp16 each holding 1024 + byte: 0x6400 is 1024.0 and its ten
// mantissa bits count in steps of one, so the byte only has to be placed under the constant.
TGO_DEVICE void bytes_to_biased_halves(uint32_t bytes, uint32_t & first, uint32_t & second) {
    first = __builtin_amdgcn_perm(0x64646464u, bytes, 0x04010400u);    // bytes 0, 1
    second = __builtin_amdgcn_perm(0x64646464u, bytes, 0x04030402u);   // bytes 2, 3
}
TGO_DEVICE uint32_t half2_fma(uint32_t a, half2_t b, half2_t c) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(half2_t, a), b, c));
}
TGO_DEVICE uint32_t half2_add(uint32_t a, half2_t b) {
    return __builtin_bit_cast(uint32_t, static_cast<half2_t>(__builtin_bit_cast(half2_t, a) + b));
}
TGO_DEVICE uint32_t half2_mul(uint32_t a, half2_t b) {
    return __builtin_bit_cast(uint32_t, static_cast<half2_t>(__builtin_bit_cast(half2_t, a) * b));
}
TGO_DEVICE half2_t half2_of(int value) {
    const _Float16 h = static_cast<_Float16>(static_cast<float>(value));
    return half2_t{h, h};
}

// ---- q8_1 quantization of eight activations per lane (the quantizer kernels, and the decode kernels that
// quantize their own activations) ----
// Arithmetic of the reference quantizer (csrc/mmq_core.cuh:151-209): per 32 values amax, d = amax/127,
// q = roundf(x * (127/amax)), and the fp32 sum of the values added in the reference's order (four per
// lane left to right, then a butterfly over eight lanes with offsets 4, 2, 1).  Here a lane holds eight
// consecutive values of a 32-value block, i.e. two of the reference's lanes, and four neighbouring lanes hold the
// block, so the butterfly runs over four lanes on two partial sums; the block's scale and sum come out the same on
// all four lanes.
// round(v) to the nearest integer, halves away from zero (roundf), of a magnitude: the hardware's
// round-to-nearest-with-ties-up conversion of |v| is exactly that for non-negative inputs.
TGO_DEVICE int round_magnitude(float v) {
    int magnitude;
    asm("v_cvt_rpi_i32_f32 %0, |%1|" : "=v"(magnitude) : "v"(v));
    return magnitude;
}

// `bits` are the lane's eight bf16 values as loaded (two per word), `x` the same as floats.  The quants are
// formed as magnitudes, two per register as 16-bit integers, and get their signs from the bf16 words themselves
// (an arithmetic shift of each half by 15 is the sign mask of the value it holds): (m ^ s) - s with packed 16-bit
// operations, then one byte permute per four values.
typedef short short2_t __attribute__((ext_vector_type(2)));
// `halves`: the same quants as fp16 numbers, two per register (1024 + magnitude is the magnitude placed under the
// bits of 1024.0; the sign bit is the one of the bf16 value, which sits at the same place of its half-word).
// `magnitude`: |q| of the eight values (for the scaled layout, which stores d * q instead of q).
TGO_DEVICE void quantize_eight(const uint4 bits, const float (&x)[8], uint32_t (&packed)[2], float & d, float & total,
                               uint32_t (&halves)[4], int (&magnitude)[8]) {
    float amax = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fabsf(x[2]));
    amax = fmaxf(fmaxf(amax, fabsf(x[3])), fabsf(x[4]));
    amax = fmaxf(fmaxf(amax, fabsf(x[5])), fabsf(x[6]));
    amax = fmaxf(amax, fabsf(x[7]));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));

    float even = ((x[0] + x[1]) + x[2]) + x[3];
    float odd = ((x[4] + x[5]) + x[6]) + x[7];
    even = even + __shfl_xor(even, 2);
    odd = odd + __shfl_xor(odd, 2);
    even = even + __shfl_xor(even, 1);
    odd = odd + __shfl_xor(odd, 1);
    total = even + odd;

    d = amax == 0.0f ? 0.0f : amax / 127.0f;
    const float d_inv = amax == 0.0f ? 0.0f : 127.0f / amax;
    const uint32_t words[4] = {bits.x, bits.y, bits.z, bits.w};
    uint32_t signed_pairs[4];
#pragma unroll
    for (int pair = 0; pair < 4; ++pair) {
        magnitude[2 * pair] = round_magnitude(x[2 * pair] * d_inv);
        magnitude[2 * pair + 1] = round_magnitude(x[2 * pair + 1] * d_inv);
        const short2_t magnitudes = __builtin_amdgcn_cvt_pk_i16(magnitude[2 * pair], magnitude[2 * pair + 1]);
        const short2_t sign = __builtin_bit_cast(short2_t, words[pair]) >> 15;
        signed_pairs[pair] = __builtin_bit_cast(uint32_t, static_cast<short2_t>((magnitudes ^ sign) - sign));
        halves[pair] = half2_add(__builtin_bit_cast(uint32_t, magnitudes) | 0x64006400u, half2_of(-1024)) |
                       (words[pair] & 0x80008000u);
    }
    // low byte of each 16-bit half: bytes 0 and 2 of the first word, then of the second
    packed[0] = __builtin_amdgcn_perm(signed_pairs[1], signed_pairs[0], 0x06040200u);
    packed[1] = __builtin_amdgcn_perm(signed_pairs[3], signed_pairs[2], 0x06040200u);
}

TGO_DEVICE void unpack_bf16x8(const uint4 bits, float (&x)[8]) {
    x[0] = bf16_bits_to_float(bits.x & 0xffffu); x[1] = bf16_bits_to_float(bits.x >> 16);
    x[2] = bf16_bits_to_float(bits.y & 0xffffu); x[3] = bf16_bits_to_float(bits.y >> 16);
    x[4] = bf16_bits_to_float(bits.z & 0xffffu); x[5] = bf16_bits_to_float(bits.z >> 16);
    x[6] = bf16_bits_to_float(bits.w & 0xffffu); x[7] = bf16_bits_to_float(bits.w >> 16);
}

// (1024 + byte) pairs times an integer multiplier 0 <= m <= 63, minus the bias: fma(1024 + b, m, -1024 m) is
// evaluated exactly and b * m is representable.
struct HalfScale {
    half2_t multiplier, offset;
};
TGO_DEVICE HalfScale half_scale(int multiplier) {
    return HalfScale{half2_of(multiplier), half2_of(-1024 * multiplier)};
}
TGO_DEVICE void scaled_halves(uint32_t bytes, const HalfScale & scale, uint32_t & first, uint32_t & second) {
    uint32_t a, b;
    bytes_to_biased_halves(bytes, a, b);
    first = half2_fma(a, scale.multiplier, scale.offset);
    second = half2_fma(b, scale.multiplier, scale.offset);
}

// Values 16u .. 16u+15 of a super-block as the forward's fp16 operand: first[i] holds values 2i and 2i + 1;
// `second` is Q6_K's low-scale operand (untouched otherwise).  Q4_K/Q5_K have their own loop in the kernel.
template <int TYPE, typename Codebook>
TGO_DEVICE void decode16_half(const uint8_t * blk, int u, const Codebook * grid, uint32_t (&first)[8], uint32_t (&second)[8]) {
    static_assert(TYPE == Q3_K || TYPE == Q6_K || TYPE == IQ2_S, "formats with 16-value scale groups");
    if constexpr (TYPE == Q3_K) {
        // b = low bits | high bit << 2 in 0..7, quant b - 4, operand (sc - 32) * (b - 4)
        const int i0 = 16 * u;
        const uint8_t * qs = blk + 32 + (i0 >> 7) * 32 + (i0 & 31);
        const uint8_t * hm = blk + (i0 & 31);
        const int shift_l = 2 * ((i0 & 127) >> 5);
        const int shift_h = i0 >> 5;
        const uint8_t * scales = blk + 96;
        const int low = scales[u & 7] >> (4 * (u >> 3));
        const int high = scales[8 + (u & 3)] >> (2 * (u >> 2));
        const int sub = ((low & 0x0f) | ((high & 3) << 4)) - 32;
        const half2_t multiplier = half2_of(sub);
        const half2_t unbias = half2_of(-1028);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t low_bits = lds_u32(qs + 4 * t) >> shift_l;
            const uint32_t high_bit = lds_u32(hm + 4 * t) >> shift_h;
            const uint32_t b = (low_bits & 0x03030303u) | ((high_bit & 0x01010101u) << 2);
            uint32_t p, q;
            bytes_to_biased_halves(b, p, q);
            first[2 * t] = half2_mul(half2_add(p, unbias), multiplier);
            first[2 * t + 1] = half2_mul(half2_add(q, unbias), multiplier);
        }
    } else if constexpr (TYPE == Q6_K) {
        const int chunk = u >> 3;
        const int rem = (16 * u) & 127;
        const uint8_t * ql = blk + chunk * 64 + (rem & 63);
        const uint8_t * qh = blk + 128 + chunk * 32 + ((16 * u) & 31);
        const int shift_l = 4 * (rem >> 6);
        const int shift_h = 2 * ((rem >> 5) & 3);
        const int sc = static_cast<int8_t>(blk[192 + u]);
        // sign-magnitude split, so that both parts have the sign of sc: the absolute values of all products of a
        // block then add up to at most 127 * 32 * 32 * 128 < 2^24 and the sum is exact in any order
        const int magnitude = sc < 0 ? -sc : sc;
        const int coarse_part = magnitude & ~15, fine_part = magnitude & 15;
        const half2_t coarse = half2_of(sc < 0 ? -coarse_part : coarse_part);   // multiple of 16: products up to 4096 are exact
        const half2_t fine = half2_of(sc < 0 ? -fine_part : fine_part);
        const half2_t unbias = half2_of(-1056);      // 1024 + the quant's offset of 32
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t low = lds_u32(ql + 4 * t) >> shift_l;
            const uint32_t high = lds_u32(qh + 4 * t) >> shift_h;
            const uint32_t b = (low & 0x0f0f0f0fu) | ((high & 0x03030303u) << 4);
            uint32_t p, q;
            bytes_to_biased_halves(b, p, q);
            p = half2_add(p, unbias);
            q = half2_add(q, unbias);
            first[2 * t] = half2_mul(p, coarse);
            first[2 * t + 1] = half2_mul(q, coarse);
            second[2 * t] = half2_mul(p, fine);
            second[2 * t + 1] = half2_mul(q, fine);
        }
    } else if constexpr (std::is_same_v<Codebook, Iq2sSelectors>) {
        // (the selector table of decode16_bf16: the unit's values are +-(2 s + 1) times one of three magnitudes, so
        // three products are formed per unit and every pair of values picks its two with one byte permute)
        const uint8_t * qs = blk + 2;
        const uint32_t idx_pair = lds_u16(qs + 2 * u);
        const uint32_t sign_pair = lds_u16(qs + 32 + 2 * u);
        const uint32_t qh = blk[66 + (u >> 1)] >> (4 * (u & 1));
        const half2_t multiplier = half2_of(2 * static_cast<int>((blk[74 + (u >> 1)] >> (4 * (u & 1))) & 0x0f) + 1);
        const uint32_t low_pair = half2_mul(__builtin_bit_cast(uint32_t, multiplier), half2_t{static_cast<_Float16>(8.0f), static_cast<_Float16>(25.0f)});
        const uint32_t high = half2_mul(__builtin_bit_cast(uint32_t, multiplier), half2_t{static_cast<_Float16>(43.0f), static_cast<_Float16>(0.0f)});
        const uint32_t spread = (sign_pair & 0x5555u) | ((sign_pair & 0xaaaau) << 15);
#pragma unroll
        for (int gsel = 0; gsel < 2; ++gsel) {
            const uint32_t index = ((idx_pair >> (8 * gsel)) & 0xff) | (((qh >> (2 * gsel)) & 3) << 8);
            const uint4 selector = grid->entry[index];
            const uint32_t words[4] = {selector.x, selector.y, selector.z, selector.w};
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int i = 4 * gsel + p;
                const uint32_t picked = __builtin_amdgcn_perm(high, low_pair, words[p]);
                first[i] = ((spread << (15 - 2 * i)) & 0x80008000u) | (picked & 0x7fff7fffu);
            }
        }
    } else {
        const uint8_t * qs = blk + 2;
        const uint32_t idx_pair = lds_u16(qs + 2 * u);
        const uint32_t sign_pair = lds_u16(qs + 32 + 2 * u);
        const uint32_t qh = blk[66 + (u >> 1)] >> (4 * (u & 1));
        const HalfScale scale = half_scale(2 * static_cast<int>((blk[74 + (u >> 1)] >> (4 * (u & 1))) & 0x0f) + 1);
        // sign of value 2i at bit 2i, of value 2i + 1 at bit 2i + 16: shifted left by 15 - 2i they are the sign
        // bits of the two halves of register i
        const uint32_t spread = (sign_pair & 0x5555u) | ((sign_pair & 0xaaaau) << 15);
#pragma unroll
        for (int gsel = 0; gsel < 2; ++gsel) {
            const uint32_t index = ((idx_pair >> (8 * gsel)) & 0xff) | (((qh >> (2 * gsel)) & 3) << 8);
            const uint2 word = grid[index];
#pragma unroll
            for (int part = 0; part < 2; ++part) {
                uint32_t p, q;
                scaled_halves(part == 0 ? word.x : word.y, scale, p, q);
                const int i = 4 * gsel + 2 * part;
                first[i] = p | ((spread << (15 - 2 * i)) & 0x80008000u);
                first[i + 1] = q | ((spread << (13 - 2 * i)) & 0x80008000u);
            }
        }
    }
}

// fp32 scale of a super-block's weight operand (decode16_half)
template <int TYPE>
TGO_DEVICE float half_weight_scale(const uint8_t * blk) {
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        return half_bits_to_float(lds_u16(blk));
    } else if constexpr (TYPE == Q3_K) {
        return half_bits_to_float(lds_u16(blk + 108));
    } else if constexpr (TYPE == Q6_K) {
        return half_bits_to_float(lds_u16(blk + 208));
    } else {
        return half_bits_to_float(lds_u16(blk)) * 0.125f;
    }
}

// fp32 scale (and min) of 32-value block b (0..7) of a super-block for the forward algebra.
template <int TYPE>
TGO_DEVICE void forward_block_scale(const uint8_t * blk, int b, float & scale, float & minimum) {
    minimum = 0.0f;
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        int sc, mn;
        k_scale_min(blk + 4, b, sc, mn);
        scale = half_bits_to_float(lds_u16(blk)) * static_cast<float>(sc);
        minimum = half_bits_to_float(lds_u16(blk + 2)) * static_cast<float>(mn);
    } else if constexpr (TYPE == Q3_K) {
        scale = -half_bits_to_float(lds_u16(blk + 108));
    } else if constexpr (TYPE == Q6_K) {
        scale = half_bits_to_float(lds_u16(blk + 208));
    } else {
        scale = half_bits_to_float(lds_u16(blk)) * 0.125f;
    }
}

// SwiGLU of two bf16 values: silu(gate) * up in fp32, rounded once by the caller.
TGO_DEVICE float swiglu(float gate, float up) {
    return gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;
}

TGO_DEVICE uint32_t swiglu_bf16x2(uint32_t gate, uint32_t up) {
    return pack_bf16x2(swiglu(bf16_bits_to_float(gate & 0xffffu), bf16_bits_to_float(up & 0xffffu)),
                       swiglu(bf16_bits_to_float(gate >> 16), bf16_bits_to_float(up >> 16)));
}

TGO_DEVICE uint16_t swiglu_bf16(uint16_t gate, uint16_t up) {
    return to_bf16_bits(swiglu(bf16_bits_to_float(gate), bf16_bits_to_float(up)));
}

TGO_DEVICE uint4 swiglu_bf16x8(const uint4 gate, const uint4 up) {
    return uint4{swiglu_bf16x2(gate.x, up.x), swiglu_bf16x2(gate.y, up.y), swiglu_bf16x2(gate.z, up.z),
                 swiglu_bf16x2(gate.w, up.w)};
}

// Stores a 32-row x 128-column fp32 MFMA result as bf16 rows with whole-line stores.  `tiles` are four
// 32x32 results side by side: a lane holds column lane%32 of each and rows 8*(v/4) + 4*(lane/32) + v%4.
// Storing those directly would take 64 two-byte store instructions per lane; instead the wave transposes
// through `stage` (32 x PITCH bf16 of LDS that only this wave touches) and every lane stores 16-byte
// pieces, four complete 256-byte rows per instruction, eight instructions in all.
// `dst` points at row 0, column 0 of the destination; rows >= valid_rows and columns >= valid_cols are
// skipped.  Needs a 16-byte aligned dst and row_stride % 8 == 0 for the wide path, else stores 2 bytes each.
// WIDE_ONLY drops the 2-byte path for callers whose destination always qualifies.
// With `gate` set (same geometry as dst) the value stored is swiglu(gate element, bf16 of the result).
// TRANSPOSED: the tiles were computed with the operands swapped, so a lane holds row l32 and, as element v of
// tile t, column 32 t + 8 (v / 4) + 4 (lane / 32) + v % 4 (four neighbouring columns per group of four elements).
template <int PITCH, bool WIDE_ONLY = false, bool TRANSPOSED = false, typename V16>
TGO_DEVICE void store_rows_32x128(uint16_t * stage, const V16 (&tiles)[4], uint16_t * dst, int64_t row_stride,
                                  int valid_rows, int valid_cols, int lane, const uint16_t * gate = nullptr) {
    const int l32 = lane & 31;
    const int half = lane >> 5;
    if (!WIDE_ONLY && (row_stride & 7) != 0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int across = 8 * (v >> 2) + 4 * half + (v & 3);
            const int r = TRANSPOSED ? l32 : across;
            if (r < valid_rows) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int c = t * 32 + (TRANSPOSED ? across : l32);
                    if (c < valid_cols) {
                        uint16_t value = to_bf16_bits(tiles[t][v]);
                        if (gate != nullptr) {
                            value = swiglu_bf16(gate[r * row_stride + c], value);
                        }
                        dst[r * row_stride + c] = value;
                    }
                }
            }
        }
        return;
    }
    // the gate pieces are requested first so that their latency passes during the transposition
    uint4 gate_piece[8] = {};
    if (gate != nullptr) {
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int id = lane + 64 * p;
            const int r = id >> 4;
            const int c = (id & 15) * 8;
            if (r < valid_rows && c + 8 <= valid_cols) {
                gate_piece[p] = *reinterpret_cast<const uint4 *>(gate + r * row_stride + c);
            }
        }
    }
    if constexpr (TRANSPOSED) {
        static_assert((PITCH / 2) % 4 == 0 && (PITCH / 2) % 64 != 0, "8-byte aligned rows that do not all start in one bank");
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                *reinterpret_cast<uint2 *>(&stage[l32 * PITCH + t * 32 + 8 * j + 4 * half]) =
                    make_uint2(pack_bf16x2(tiles[t][4 * j], tiles[t][4 * j + 1]), pack_bf16x2(tiles[t][4 * j + 2], tiles[t][4 * j + 3]));
            }
        }
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int r = 8 * (v >> 2) + 4 * half + (v & 3);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                stage[r * PITCH + t * 32 + l32] = to_bf16_bits(tiles[t][v]);
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const int id = lane + 64 * p;
        const int r = id >> 4;
        const int c = (id & 15) * 8;
        if (r < valid_rows && c < valid_cols) {
            uint4 piece = *reinterpret_cast<const uint4 *>(&stage[r * PITCH + c]);
            if (c + 8 <= valid_cols) {
                if (gate != nullptr) {
                    piece = swiglu_bf16x8(gate_piece[p], piece);
                }
                *reinterpret_cast<uint4 *>(dst + r * row_stride + c) = piece;
            } else {
                const uint16_t * values = &stage[r * PITCH + c];
                for (int e = 0; c + e < valid_cols; ++e) {
                    dst[r * row_stride + c + e] =
                        gate != nullptr ? swiglu_bf16(gate[r * row_stride + c + e], values[e]) : values[e];
                }
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// The same in two halves for workgroups whose waves each hold one 32x32 tile of a shared 32-row x 128-column
// block: every wave puts its tile at column `col0` of `stage` (32 x PITCH bf16), and after a barrier
// store_staged_rows writes the block out with all threads, whole rows at a time.
// (TRANSPOSED as in store_rows_32x128: the lane holds row l32 and four neighbouring columns per group of four elements)
template <int PITCH, bool TRANSPOSED = false, typename V16>
TGO_DEVICE void stage_tile_32x32(uint16_t * stage, const V16 & tile, int col0, int lane) {
    const int l32 = lane & 31;
    const int half = lane >> 5;
    if constexpr (TRANSPOSED) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<uint2 *>(&stage[l32 * PITCH + col0 + 8 * j + 4 * half]) =
                make_uint2(pack_bf16x2(tile[4 * j], tile[4 * j + 1]), pack_bf16x2(tile[4 * j + 2], tile[4 * j + 3]));
        }
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int r = 8 * (v >> 2) + 4 * half + (v & 3);
            stage[r * PITCH + col0 + l32] = to_bf16_bits(tile[v]);
        }
    }
}

template <int PITCH>
TGO_DEVICE void store_staged_rows(const uint16_t * stage, uint16_t * dst, int64_t row_stride, int valid_rows,
                                  int valid_cols, int tid, int nthreads, const uint16_t * gate = nullptr) {
    const bool wide = (row_stride & 7) == 0;
    for (int id = tid; id < 32 * 16; id += nthreads) {
        const int r = id >> 4;
        const int c = (id & 15) * 8;
        if (r < valid_rows && c < valid_cols) {
            const uint16_t * values = &stage[r * PITCH + c];
            if (wide && c + 8 <= valid_cols) {
                uint4 piece = *reinterpret_cast<const uint4 *>(values);
                if (gate != nullptr) {
                    piece = swiglu_bf16x8(*reinterpret_cast<const uint4 *>(gate + r * row_stride + c), piece);
                }
                *reinterpret_cast<uint4 *>(dst + r * row_stride + c) = piece;
            } else {
                for (int e = 0; e < 8 && c + e < valid_cols; ++e) {
                    dst[r * row_stride + c + e] =
                        gate != nullptr ? swiglu_bf16(gate[r * row_stride + c + e], values[e]) : values[e];
                }
            }
        }
    }
}

}  // namespace tgo
