// Grad-input kernels: dX[r, k] = bf16( sum_n dY[r, n] * bf16(W[n, k]) ) on gfx950 bf16 MFMA.
//
// The cotangent is not quantized.  Three kernels:
//
// pack_cotangent_kernel copies dY (row-major bf16) into MFMA fragment order, [rows/32][chunks] slabs of 1 KiB
// laid out [half][row 0..31][8 bf16], zero-padded in both directions (columns to a multiple of 64).  One slab
// is the A operand of one v_mfma_f32_32x32x16_bf16, so the main kernels fetch it with one fully coalesced
// 16-byte-per-lane load (a row-major cotangent would cost 32 cache lines per wave load).
//
// mmq_grad_input_kernel (every format): a workgroup (4 waves) owns 256 rows x 128 values of K (half a
// super-block column) and walks the reduction dimension N in steps of 64 weight rows.  Per step the 64 packed
// blocks are copied to LDS, dequantized once to bf16 (bit-exact with the scalar reference decoder) into a
// transposed tile [k][n] whose rows are what a lane needs as its B operand, and shared by the four waves; wave
// w owns rows [64w, 64w+64) and all 128 columns: 2 x 4 MFMA tiles, 32 MFMAs per step.  The tile is double
// buffered and the loop is software pipelined.
//
// mmq_grad_input_split_kernel (Q4_K and Q5_K, what the launcher picks for them): the same tile, with the waves
// of a workgroup specialised into multipliers and decoders; described where it is defined.
//
// The pair variant of both walks a second (dY, W) in the same loop with one fp32 accumulator, so the sum of
// both Jacobian products is rounded to bf16 once.
#include <algorithm>

#include "tgo_device.h"
#include "tgo_launch.h"

namespace tgo {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef u32x4_t u32x4;   // (a native vector type: arrays of the uint4 struct end up in scratch memory)

constexpr int BWD_TR = BACKWARD_ROW_TILE;  // rows per workgroup
constexpr int BWD_TK = 128;                // K columns per workgroup
constexpr int BWD_NS = 64;                 // weight rows per reduction step
constexpr int BWD_PITCH = BWD_NS + 8;      // bf16 per k-row of the tile: +8 keeps 16-byte reads conflict free
constexpr int BWD_THREADS = 256;
constexpr int BWD_XCD_RUN = 4;             // dense calls: consecutive row tasks that share an XCD (grouped calls: xcd_chunk)
static_assert(BWD_TR == 64 * BWD_THREADS / 64, "64 rows per wave");

// ---- cotangent packing ---------------------------------------------------------------------------------
// One workgroup handles 32 rows x 128 columns (8 slabs): coalesced row reads, transpose through LDS,
// one contiguous 8 KiB write.
// With `gather` set (single cotangent only), row r of the cotangent is bf16(scale[r] * grad_first[gather[r], :]):
// the routing-weighted return of a mixture-of-experts layer run backwards, read straight from the per-token
// cotangent (rows whose index lies outside [0, gather_rows) are zeros), so the expert-sorted cotangent that the
// caller would otherwise build (rows x out_features bf16 written and read again) never exists.
TGO_DEVICE uint32_t scale_bf16x2(uint32_t pair, float scale) {
    return pack_bf16x2(scale * bf16_bits_to_float(pair & 0xffffu), scale * bf16_bits_to_float(pair >> 16));
}

__global__ __launch_bounds__(256) void pack_cotangent_kernel(const uint16_t * __restrict__ grad_first,
                                                            const uint16_t * __restrict__ grad_second,
                                                            uint8_t * __restrict__ packed_first,
                                                            uint8_t * __restrict__ packed_second, int rows,
                                                            int out_features, int n_chunks, const TaskBuild build,
                                                            const int64_t * __restrict__ gather,
                                                            const float * __restrict__ scale, int64_t gather_rows) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[8 * 1024];
    if (build.tasks.count != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
        build_tasks(build, threadIdx.x);
    }
    const uint16_t * grad = blockIdx.z == 0 ? grad_first : grad_second;
    uint8_t * packed = blockIdx.z == 0 ? packed_first : packed_second;
    const int tid = threadIdx.x;
    const int row_tile = blockIdx.x;
    const int chunk0 = blockIdx.y * 8;
    const int rr = tid >> 3;            // row inside the tile
    const int c = tid & 7;              // 16-column chunk inside this workgroup
    const int row = row_tile * 32 + rr;
    const int n = (chunk0 + c) * 16;
    uint4 lo = make_uint4(0, 0, 0, 0), hi = make_uint4(0, 0, 0, 0);
    int64_t source_row = row;
    float factor = 1.0f;
    bool present = row < rows && n < out_features;
    if (gather != nullptr && present) {   // (uniform: one launch either gathers or does not)
        source_row = gather[row];
        factor = scale[row];
        present = source_row >= 0 && source_row < gather_rows;
    }
    if (present) {
        const uint16_t * src = grad + source_row * out_features + n;
        if ((out_features & 7) == 0 && n + 16 <= out_features) {
            lo = *reinterpret_cast<const uint4 *>(src);
            hi = *reinterpret_cast<const uint4 *>(src + 8);
        } else {
            uint32_t e[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                e[i] = n + i < out_features ? src[i] : 0u;
            }
            lo = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
            hi = make_uint4(e[8] | (e[9] << 16), e[10] | (e[11] << 16), e[12] | (e[13] << 16), e[14] | (e[15] << 16));
        }
        if (gather != nullptr) {
            lo = make_uint4(scale_bf16x2(lo.x, factor), scale_bf16x2(lo.y, factor), scale_bf16x2(lo.z, factor), scale_bf16x2(lo.w, factor));
            hi = make_uint4(scale_bf16x2(hi.x, factor), scale_bf16x2(hi.y, factor), scale_bf16x2(hi.z, factor), scale_bf16x2(hi.w, factor));
        }
    }
    *reinterpret_cast<uint4 *>(tile + c * 1024 + rr * 16) = lo;
    *reinterpret_cast<uint4 *>(tile + c * 1024 + (32 + rr) * 16) = hi;
    __syncthreads();
    const int chunks_here = min(8, n_chunks - chunk0);
    uint4 * dst = reinterpret_cast<uint4 *>(packed + (static_cast<int64_t>(row_tile) * n_chunks + chunk0) * 1024);
    const uint4 * src4 = reinterpret_cast<const uint4 *>(tile);
    if (tid < chunks_here * 64) {
        dst[tid] = src4[tid];
    }
    if (tid + 256 < chunks_here * 64) {
        dst[tid + 256] = src4[tid + 256];
    }
}

hipError_t launch_pack_cotangent(const uint16_t * grad, const uint16_t * grad_second, uint8_t * packed,
                                 uint8_t * packed_second, int rows, int out_features, hipStream_t stream,
                                 const TaskBuild * build, const int64_t * gather, const float * scale,
                                 int64_t gather_rows) {
    if ((grad_second == nullptr) != (packed_second == nullptr)) {
        return hipErrorInvalidValue;
    }
    if (gather != nullptr && (grad_second != nullptr || scale == nullptr || gather_rows <= 0)) {
        return hipErrorInvalidValue;
    }
    const int n_chunks = cotangent_chunks(out_features);
    const dim3 grid(static_cast<unsigned>((rows + 31) / 32), static_cast<unsigned>((n_chunks + 7) / 8),
                    grad_second != nullptr ? 2 : 1);
    const ProfileScope scope(6, stream);
    pack_cotangent_kernel<<<grid, 256, 0, stream>>>(grad, grad_second, packed, packed_second, rows, out_features,
                                                    n_chunks, build != nullptr ? *build : no_task_build(), gather,
                                                    scale, gather_rows);
    return hipGetLastError();
}

// ---- main kernel ----------------------------------------------------------------------------------------
struct BackwardArgs {
    const uint8_t * cotangent[2];   // fragment-ordered dY, see pack_cotangent_kernel
    const uint8_t * packed[2];
    int64_t bytes_per_expert;
    int64_t row_bytes;
    uint16_t * dx;
    const int32_t * task_count;   // nullptr: dense
    const int32_t * task_early;   // tasks listed before the short ones (at most BACKWARD_SHORT_ROWS rows each)
    const int32_t * task_expert;
    const int32_t * task_row_start;
    const int32_t * task_row_end;
    int segment;        // which tasks of the list a launch runs: 0 all, 1 those before the short ones, 2 the short ones
    int rows;
    int rows_padded;    // rows rounded up to 32: extent of the packed cotangent
    int out_features;   // N, the reduction dimension
    int n_chunks;       // 16-column chunks of the packed cotangent (N rounded up to 64, over 16)
    int in_features;    // K
    int k_tiles;        // K / 128
    int task_slots;
    int short_slots;    // upper bound of the short tasks (one per group at most)
    int sources;        // 1, or 2 for the fused pair
    // Dense calls too small to fill the chip: the reduction over the weight rows is cut into n_splits ranges of
    // steps, blockIdx.y picks one, and the workgroup writes its fp32 sums to partial[split][row][K] instead of
    // dx; reduce_partials_kernel adds them in split order.  n_splits == 1: plain operation.
    float * partial;
    int n_splits;
};

// Q4_K / Q5_K: a thread decodes 8 weight rows x 4 consecutive K positions and stores each K position's
// eight bf16 values with one 16-byte write.  `scale_min` holds (d*sc, dmin*m) per row and 32-value group.
template <int TYPE>
TGO_DEVICE void decode_k45_octet(const uint8_t * raw, const float2 * scale_min, uint16_t * wb, int tid,
                                 int half_block, int n0, int n_total) {
    using F = Format<TYPE>;
    constexpr int QS = TYPE == Q4_K ? 16 : 48;
    const int octet = tid & 7;
    const int word = (tid >> 3) & 15;
    const int nibble = tid >> 7;
    const int chunk = word >> 3;                       // 64-value chunk inside this half block
    const int position = (word & 7) * 4;               // first of 4 positions inside the 32-value group
    const int group_local = 2 * chunk + nibble;        // 32-value group inside this half block
    const int group = 4 * half_block + group_local;
    float w[4][8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int n = 8 * octet + i;
        const uint8_t * blk = raw + n * F::RAW_PITCH;
        uint32_t q = (lds_u32(blk + QS + 64 * half_block + 4 * word) >> (4 * nibble)) & 0x0f0f0f0fu;
        if constexpr (TYPE == Q5_K) {
            q |= ((lds_u32(blk + 16 + position) >> group) & 0x01010101u) << 4;
        }
        const float2 sm = scale_min[group_local * (BWD_NS + 8) + n + (n >> 3)];
        const bool valid = n0 + n < n_total;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float value = sm.x * static_cast<float>((q >> (8 * e)) & 0xffu) - sm.y;
            w[e][i] = valid ? value : 0.0f;
        }
    }
    const int k_local = 32 * group_local + position;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint4 packed = make_uint4(pack_bf16x2(w[e][0], w[e][1]), pack_bf16x2(w[e][2], w[e][3]),
                                        pack_bf16x2(w[e][4], w[e][5]), pack_bf16x2(w[e][6], w[e][7]));
        *reinterpret_cast<uint4 *>(&wb[(k_local + e) * BWD_PITCH + 8 * octet]) = packed;
    }
}

// First task and number of tasks of the list's segment that a launch runs.
// `ordinary`: how many of them come before the short ones (all of them in a segment of one kind).
TGO_DEVICE void task_segment(const BackwardArgs & a, int & first, int & tasks, int & ordinary) {
    const int count = a.task_count[0];
    const int early = min(a.task_early[0], count);
    first = a.segment == 2 ? early : 0;
    tasks = a.segment == 2 ? count - early : a.segment == 1 ? early : count;
    ordinary = a.segment == 0 ? early : tasks;
}
TGO_DEVICE void task_segment(const BackwardArgs & a, int & first, int & tasks) {
    int ordinary;
    task_segment(a, first, tasks, ordinary);
}

// SHORT: the variant for tasks of at most BACKWARD_SHORT_ROWS rows.  Dequantizing a step's weights costs the same
// however few rows multiply them, so for these tasks it is nearly all of the work: every wave takes the task's 64
// rows and one 32-column slice of the tile (8 instead of 32 matrix instructions per step, spread over all four
// SIMDs, 32 accumulator registers instead of 128), and with the smaller register footprint three workgroups share
// a CU, so that one's barriers and memory waits are covered by another's decoding.
// WIDE (formats whose blocks are not multiples of 16 bytes, when wide_stage_ok holds): a step's packed blocks are
// requested as aligned 16-byte units while the previous step multiplies, like those of Q4_K / Q5_K, instead of
// being copied two bytes at a time between the multiplications and the decoding.
template <int TYPE, bool SHORT, bool WIDE>
__global__ __launch_bounds__(BWD_THREADS, SHORT ? 3 : 2) void mmq_grad_input_kernel(const BackwardArgs a) {
    using F = Format<TYPE>;
    constexpr int KT = SHORT ? 1 : 4;   // 32-column tiles per wave
    constexpr bool FAST_K45 = TYPE == Q4_K || TYPE == Q5_K;
    constexpr int RAW_UNITS = F::BLOCK_BYTES / 16;                              // 16-byte units per block (fast types)
    constexpr int RAW_REGS = (BWD_NS * RAW_UNITS + BWD_THREADS - 1) / BWD_THREADS;  // units in flight per thread
    static_assert(!(WIDE && FAST_K45), "the wide copy is for the 2-byte aligned formats");
    using W = WideStage<TYPE>;
    constexpr int WIDE_REGS = WIDE ? W::template regs<BWD_NS, BWD_THREADS>() : 1;
    constexpr int SLOT_PITCH = WIDE ? W::PITCH : F::RAW_PITCH;
    constexpr int SLOT_FRONT = WIDE ? W::FRONT : F::RAW_SHIFT;
    constexpr bool AHEAD = FAST_K45 || WIDE;   // the packed blocks of the next step travel through registers
    __shared__ __attribute__((aligned(16))) uint8_t raw[BWD_NS * SLOT_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t raw_odd[WIDE ? BWD_NS * SLOT_PITCH : 16];   // second slot of the WIDE pipeline
    __shared__ __attribute__((aligned(16))) uint16_t wb[2][BWD_TK * BWD_PITCH];
    __shared__ float2 scale_min[FAST_K45 ? 4 * (BWD_NS + 8) : 1];
    // (IQ2_S: the selector table of decode16_bf16; the other formats have no codebook)
    using Codebook = std::conditional_t<TYPE == IQ2_S, Iq2sSelectors, uint2>;
    __shared__ Codebook codebook_storage;
    const Codebook * const grid = &codebook_storage;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;

    int k_tile, task, first_task = 0, ordinary = 0;
    int tasks = (a.rows + BWD_TR - 1) / BWD_TR;
    if (a.task_count != nullptr) {
        task_segment(a, first_task, tasks, ordinary);
    }
    // (short tasks are remainders of different experts: nothing to gain from keeping neighbours on one XCD)
    if (!SHORT && a.task_count != nullptr) {
        xcd_chunk(blockIdx.x, a.k_tiles, tasks, ordinary, k_tile, task);
    } else {
        xcd_tile<SHORT ? 1 : BWD_XCD_RUN>(blockIdx.x, a.k_tiles, tasks, k_tile, task);
    }
    const int kb = k_tile >> 1;          // super-block column
    const int half_block = k_tile & 1;   // which 128 values of it

    int expert = 0, row_start, row_end;
    if (a.task_count != nullptr) {
        if (task >= tasks) {
            return;
        }
        task += first_task;
        expert = a.task_expert[task];
        row_start = a.task_row_start[task];
        row_end = a.task_row_end[task];
    } else {
        row_start = task * BWD_TR;
        if (row_start >= a.rows) {
            return;
        }
        row_end = min(a.rows, row_start + BWD_TR);
    }
    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_selectors(codebook_storage, tid, BWD_THREADS);
    }

    const int wave_row = SHORT ? row_start : row_start + wave * 64;
    const bool wave_active = SHORT || wave_row < row_end;
    const int row_tiles = SHORT ? (row_end - row_start + 31) / 32 : 2;   // 32-row tiles this wave multiplies
    const int n_total = a.out_features;
    const int steps_per_source = (n_total + BWD_NS - 1) / BWD_NS;
    const int steps = steps_per_source * a.sources;
    const int split = blockIdx.y;
    const int step_begin = steps * split / a.n_splits;        // (n_splits <= steps: no range is empty)
    const int step_end = steps * (split + 1) / a.n_splits;

    // byte offset of this lane's fragment piece inside the packed cotangent, per 32-row tile of the wave
    int64_t lane_offset[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        int r = wave_row + rt * 32 + l32;
        r = r < a.rows_padded ? r : a.rows_padded - 1;
        lane_offset[rt] = static_cast<int64_t>(r >> 5) * a.n_chunks * 1024 + ((r & 31) + 32 * half) * 16;
    }

    v16f acc[2][KT];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rt][kt][v] = 0.0f;

    uint4 afrag[2][4] = {};     // cotangent fragments of the step about to be multiplied
    u32x4 raw_regs[FAST_K45 ? RAW_REGS : 1];   // (a native vector type: arrays of the uint4 struct end up in scratch memory)
    WideRegs<WIDE_REGS> wide_regs;

    // requests the cotangent fragments of a step: chunk s covers columns n0 + 16 s .. + 16
    auto load_cotangent = [&](int step) __attribute__((always_inline)) {
        const int source = step / steps_per_source;
        const int n0 = (step - source * steps_per_source) * BWD_NS;
        const uint8_t * base = a.cotangent[source];
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            if (SHORT && rt >= row_tiles) {
                break;
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int chunk = (n0 >> 4) + s;
                afrag[rt][s] = chunk < a.n_chunks
                    ? *reinterpret_cast<const uint4 *>(base + lane_offset[rt] + static_cast<int64_t>(chunk) * 1024)
                    : make_uint4(0, 0, 0, 0);
            }
        }
    };
    // requests / stores the packed blocks of a step (16-byte aligned types travel through registers)
    auto load_raw = [&](int step) __attribute__((always_inline)) {
        const int source = step / steps_per_source;
        const int n0 = (step - source * steps_per_source) * BWD_NS;
        const uint8_t * weights = a.packed[source] + static_cast<int64_t>(expert) * a.bytes_per_expert;
        if constexpr (FAST_K45) {
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = tid + BWD_THREADS * i;
                const int row = id / RAW_UNITS;
                const int unit = id - row * RAW_UNITS;
                if (row < BWD_NS) {
                    int src_row = n0 + row;
                    src_row = src_row < n_total ? src_row : n_total - 1;
                    raw_regs[i] = *reinterpret_cast<const u32x4 *>(
                        weights + src_row * a.row_bytes + static_cast<int64_t>(kb) * F::BLOCK_BYTES + unit * 16);
                }
            }
        } else if constexpr (WIDE) {
            wide_fetch<TYPE, BWD_NS, BWD_THREADS, WIDE_REGS>(wide_regs, weights + n0 * a.row_bytes, static_cast<int>(a.row_bytes),
                                                             min(BWD_NS, n_total - n0), kb, tid);
        } else {
            stage_blocks<TYPE>(raw, weights, a.row_bytes, n0, n_total, kb, BWD_NS, tid, BWD_THREADS);
        }
    };
    auto store_raw = [&](int step) __attribute__((always_inline)) {
        if constexpr (WIDE) {
            const int source = step / steps_per_source;
            const int n0 = (step - source * steps_per_source) * BWD_NS;
            const uint8_t * weights = a.packed[source] + static_cast<int64_t>(expert) * a.bytes_per_expert;
            wide_park<TYPE, BWD_NS, BWD_THREADS, WIDE_REGS>(raw, wide_regs, weights + n0 * a.row_bytes, static_cast<int>(a.row_bytes),
                                                            min(BWD_NS, n_total - n0), kb, tid);
        }
        if constexpr (FAST_K45) {
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = tid + BWD_THREADS * i;
                const int row = id / RAW_UNITS;
                const int unit = id - row * RAW_UNITS;
                if (row < BWD_NS) {
                    *reinterpret_cast<u32x4 *>(raw + row * F::RAW_PITCH + unit * 16) = raw_regs[i];
                }
            }
        }
    };
    // dequantizes the staged blocks of a step into one of the two bf16 tiles (ends with the tile visible)
    auto decode = [&](int step, uint16_t * tile) __attribute__((always_inline)) {
        const int source = step / steps_per_source;
        const int n0 = (step - source * steps_per_source) * BWD_NS;
        __syncthreads();   // staged blocks visible
        if constexpr (FAST_K45) {
            const int n = tid & 63;
            const int group_local = tid >> 6;
            const uint8_t * blk = raw + n * F::RAW_PITCH;
            int sc, mn;
            k_scale_min(blk + 4, 4 * half_block + group_local, sc, mn);
            scale_min[group_local * (BWD_NS + 8) + n + (n >> 3)] =
                make_float2(half_bits_to_float(lds_u16(blk)) * static_cast<float>(sc),
                            half_bits_to_float(lds_u16(blk + 2)) * static_cast<float>(mn));
            __syncthreads();
            decode_k45_octet<TYPE>(raw, scale_min, tile, tid, half_block, n0, n_total);
        } else {
            // 64 rows x 8 units of 16 values; a half-wave writes 32 consecutive n of one k
#pragma unroll 1
            for (int pass = 0; pass < 2; ++pass) {
                const int id = tid + BWD_THREADS * pass;
                const int n = id & 63;
                const int unit = id >> 6;
                uint32_t pairs[8];
                decode16_bf16<TYPE>(raw + n * SLOT_PITCH + SLOT_FRONT, 8 * half_block + unit, grid, pairs);
                const bool valid = n0 + n < n_total;
                // Neighbouring lanes hold neighbouring weight rows of the same 16 values of K.  They swap pairs of
                // bf16 values so that the even lane writes both rows of an even k and the odd lane both rows of the
                // odd k, 4 bytes at a time: half the LDS writes of one 2-byte write per value.
                const uint32_t selector = (lane & 1) != 0 ? 0x03020706u : 0x05040100u;
                uint32_t * const pair_row = reinterpret_cast<uint32_t *>(&tile[(unit * 16 + (lane & 1)) * BWD_PITCH + (n & ~1)]);
#pragma unroll
                for (int j = 0; j < 16; j += 2) {
                    const uint32_t own = valid ? pairs[j / 2] : 0u;
                    const uint32_t other = static_cast<uint32_t>(
                        __builtin_amdgcn_mov_dpp(static_cast<int>(own), 0xB1, 0xf, 0xf, true));   // lane ^ 1
                    pair_row[j * (BWD_PITCH / 2)] = __builtin_amdgcn_perm(other, own, selector);
                }
            }
        }
        __syncthreads();   // tile visible
    };

    if constexpr (SHORT && FAST_K45) {
        // The multiplications of a step are too short here to cover a memory round trip, so the packed blocks travel
        // DEPTH steps ahead through a ring of register sets and the cotangent fragments two steps ahead; steps past
        // the end repeat the last one (harmless re-reads instead of branches around loads).
        constexpr int DEPTH = 1;
        const int last = step_end - 1;
        u32x4 ring[DEPTH][RAW_REGS];
        u32x4 cot[2][2][4] = {};
        auto request_raw = [&](int step, u32x4 (&regs)[RAW_REGS]) {
            step = min(step, last);
            const int source = step / steps_per_source;
            const int n0 = (step - source * steps_per_source) * BWD_NS;
            const uint8_t * weights = a.packed[source] + static_cast<int64_t>(expert) * a.bytes_per_expert +
                                      static_cast<int64_t>(kb) * F::BLOCK_BYTES;
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = min(tid + BWD_THREADS * i, BWD_NS * RAW_UNITS - 1);
                const int row = id / RAW_UNITS;
                const int unit = id - row * RAW_UNITS;
                const int src_row = min(n0 + row, n_total - 1);
                regs[i] = *reinterpret_cast<const u32x4 *>(weights + src_row * a.row_bytes + unit * 16);
            }
        };
        auto park_raw = [&](const u32x4 (&regs)[RAW_REGS]) {
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = tid + BWD_THREADS * i;
                const int row = id / RAW_UNITS;
                const int unit = id - row * RAW_UNITS;
                if (row < BWD_NS) {
                    *reinterpret_cast<u32x4 *>(raw + row * F::RAW_PITCH + unit * 16) = regs[i];
                }
            }
        };
        auto request_cotangent = [&](int step, u32x4 (&regs)[2][4]) {
            step = min(step, last);
            const int source = step / steps_per_source;
            const int n0 = (step - source * steps_per_source) * BWD_NS;
            const uint8_t * base = a.cotangent[source];
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                if (rt < row_tiles) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        // (the packed cotangent is zero padded to whole steps of 64 columns)
                        regs[rt][c] = *reinterpret_cast<const u32x4 *>(
                            base + lane_offset[rt] + static_cast<int64_t>((n0 >> 4) + c) * 1024);
                    }
                }
            }
        };
        auto multiply = [&](const uint16_t * tile, const u32x4 (&regs)[2][4]) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint4 bits = *reinterpret_cast<const uint4 *>(&tile[(wave * 32 + l32) * BWD_PITCH + 16 * c + 8 * half]);
                const v8bf bfrag = __builtin_bit_cast(v8bf, bits);
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    if (rt < row_tiles) {
                        acc[rt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, regs[rt][c]), bfrag,
                                                                             acc[rt][0], 0, 0, 0);
                    }
                }
            }
        };
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            request_raw(step_begin + d, ring[d]);
        }
        request_cotangent(step_begin, cot[0]);
        request_cotangent(step_begin + 1, cot[1]);
        park_raw(ring[0]);
        request_raw(step_begin + DEPTH, ring[0]);
        decode(step_begin, wb[0]);
#pragma unroll 1
        for (int first = step_begin; first < step_end; first += DEPTH) {
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                const int step = first + u;
                if (step < step_end) {
                    multiply(wb[u & 1], cot[u & 1]);
                    request_cotangent(step + 2, cot[u & 1]);
                    if (step + 1 < step_end) {
                        park_raw(ring[(u + 1) % DEPTH]);
                        request_raw(step + 1 + DEPTH, ring[(u + 1) % DEPTH]);
                        decode(step + 1, wb[(u + 1) & 1]);
                    }
                }
            }
        }
    } else if constexpr (WIDE) {
        // One barrier per step, and every wave both multiplies and dequantizes between two barriers: while the matrix
        // instructions of step i run on tile i % 2, the same wave's vector instructions decode step i + 1 from its
        // parked blocks into the other tile (the two kinds of instruction issue independently, so inside one block
        // of code they overlap), the blocks of step i + 2 go from registers to the raw slot that step i was decoded
        // from, those of step i + 3 are requested, and each quarter of the cotangent fragments is re-requested for
        // step i + 1 as soon as the matrix instructions of step i that read it have been issued.  Steps past the
        // end repeat the last one where that avoids a branch around a load.
        const int last = step_end - 1;
        auto blocks_of = [&](int step, const uint8_t *& tile_rows, int & rows_valid) __attribute__((always_inline)) {
            step = min(step, last);
            const int source = step / steps_per_source;
            const int n0 = (step - source * steps_per_source) * BWD_NS;
            tile_rows = a.packed[source] + static_cast<int64_t>(expert) * a.bytes_per_expert + n0 * a.row_bytes;
            rows_valid = min(BWD_NS, n_total - n0);
        };
        auto request = [&](int step) __attribute__((always_inline)) {
            const uint8_t * tile_rows;
            int rows_valid;
            blocks_of(step, tile_rows, rows_valid);
            wide_fetch<TYPE, BWD_NS, BWD_THREADS, WIDE_REGS>(wide_regs, tile_rows, static_cast<int>(a.row_bytes), rows_valid, kb, tid);
        };
        auto park = [&](int step, uint8_t * slot) __attribute__((always_inline)) {
            const uint8_t * tile_rows;
            int rows_valid;
            blocks_of(step, tile_rows, rows_valid);
            wide_park<TYPE, BWD_NS, BWD_THREADS, WIDE_REGS>(slot, wide_regs, tile_rows, static_cast<int>(a.row_bytes), rows_valid, kb, tid);
        };
        // half of a step's 64 rows x 8 units of 16 values; a half-wave writes 32 consecutive n of one k
        auto decode_pass = [&](int step, int pass, const uint8_t * slot, uint16_t * tile) __attribute__((always_inline)) {
            const int source = step / steps_per_source;
            const int n0 = (step - source * steps_per_source) * BWD_NS;
            const int n = lane;
            const int unit = wave + 4 * pass;   // (wave-uniform: the unit's shifts and offsets are scalars)
            uint32_t pairs[8];
            decode16_bf16<TYPE>(slot + n * SLOT_PITCH + SLOT_FRONT, 8 * half_block + unit, grid, pairs);
            // rows past the end of the weight matrix become zeros (a mask the compiler cannot see through: a visible
            // condition ends up as a branch around part of the arithmetic, which splits the block of code that the
            // matrix and vector instructions are meant to share)
            uint32_t keep = n0 + n < n_total ? 0xffffffffu : 0u;
            asm volatile("" : "+v"(keep));
            // (pairs of lanes swap halves so that each writes both rows of one k: see the two-barrier loop's decode)
            const uint32_t selector = (lane & 1) != 0 ? 0x03020706u : 0x05040100u;
            uint32_t * const pair_row = reinterpret_cast<uint32_t *>(&tile[(unit * 16 + (lane & 1)) * BWD_PITCH + (n & ~1)]);
#pragma unroll
            for (int j = 0; j < 16; j += 2) {
                const uint32_t own = pairs[j / 2] & keep;
                const uint32_t other = static_cast<uint32_t>(
                    __builtin_amdgcn_mov_dpp(static_cast<int>(own), 0xB1, 0xf, 0xf, true));   // lane ^ 1
                pair_row[j * (BWD_PITCH / 2)] = __builtin_amdgcn_perm(other, own, selector);
            }
        };
        auto request_cotangent = [&](int step, int s) __attribute__((always_inline)) {
            const int source = step / steps_per_source;
            const int n0 = (step - source * steps_per_source) * BWD_NS;
            const uint8_t * base = a.cotangent[source];
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                if (!SHORT || rt < row_tiles) {
                    // (the packed cotangent is zero padded to whole steps of 64 columns)
                    afrag[rt][s] = *reinterpret_cast<const uint4 *>(
                        base + lane_offset[rt] + static_cast<int64_t>((n0 >> 4) + s) * 1024);
                }
            }
        };
        // the weight fragments of chunk s of a tile (one per 32-column tile of the wave), and the chunk's multiplications
        uint4 fragment[2][KT];
        auto read_fragments = [&](const uint16_t * tile, int s) __attribute__((always_inline)) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const int k = (SHORT ? wave : kt) * 32 + l32;
                fragment[s & 1][kt] = *reinterpret_cast<const uint4 *>(&tile[k * BWD_PITCH + 16 * s + 8 * half]);
            }
        };
        auto multiply = [&](int s) __attribute__((always_inline)) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const v8bf bfrag = __builtin_bit_cast(v8bf, fragment[s & 1][kt]);
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    if (!SHORT || rt < row_tiles) {
                        // (full-size tasks swap the operands: the lane then holds one task row and runs of four
                        // neighbouring columns, which the epilogue stages with 8-byte LDS writes)
                        acc[rt][kt] = SHORT ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                                  __builtin_bit_cast(v8bf, afrag[rt][s]), bfrag, acc[rt][kt], 0, 0, 0)
                                            : __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                                  bfrag, __builtin_bit_cast(v8bf, afrag[rt][s]), acc[rt][kt], 0, 0, 0);
                    }
                }
            }
        };
        request(step_begin);
        park(step_begin, raw);
        request(step_begin + 1);
        __syncthreads();
        decode_pass(step_begin, 0, raw, wb[0]);
        decode_pass(step_begin, 1, raw, wb[0]);
        if (wave_active) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                request_cotangent(step_begin, s);
            }
        }
        park(step_begin + 1, raw_odd);
        request(step_begin + 2);
        __syncthreads();
        auto run = [&](auto active_tag) __attribute__((always_inline)) {
            constexpr bool ACTIVE = decltype(active_tag)::value;
            // vector instructions scheduled behind each matrix instruction of a step (12: measured best of 0..16)
            constexpr int INTERLEAVED_VALU = 12;
#pragma unroll 1
            for (int step = step_begin; step < last; ++step) {
                const int parity = (step - step_begin) & 1;
                const uint16_t * tile = wb[parity];
                uint16_t * next_tile = wb[parity ^ 1];
                const uint8_t * next_raw = parity != 0 ? raw : raw_odd;
                if constexpr (ACTIVE) {
                    read_fragments(tile, 0);
                }
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    if constexpr (ACTIVE) {
                        if (s + 1 < 4) {
                            read_fragments(tile, s + 1);   // an LDS round trip ahead of the instructions they feed
                        }
                        multiply(s);
                        request_cotangent(step + 1, s);
                    }
                    if (s == 0 || s == 2) {
                        decode_pass(step + 1, s >> 1, next_raw, next_tile);
                    }
                    if (s == 1) {
                        park(step + 2, parity != 0 ? raw_odd : raw);
                    }
                    if (s == 3) {
                        request(step + 3);
                    }
                    if constexpr (ACTIVE && !SHORT) {
                        // one matrix instruction, then a run of the vector instructions that share its chunk
#pragma unroll
                        for (int i = 0; i < 2 * KT; ++i) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, INTERLEAVED_VALU, 0);
                        }
                    }
                }
                __syncthreads();
            }
            if constexpr (ACTIVE) {
                const uint16_t * tile = wb[(last - step_begin) & 1];
                read_fragments(tile, 0);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    if (s + 1 < 4) {
                        read_fragments(tile, s + 1);
                    }
                    multiply(s);
                }
            }
        };
        if (wave_active) {
            run(std::true_type{});
        } else {
            run(std::false_type{});
        }
    } else {
        // prologue: the first step staged and decoded, its cotangent fragments requested
        load_raw(step_begin);
        if (wave_active) {
            load_cotangent(step_begin);
        }
        store_raw(step_begin);
        decode(step_begin, wb[0]);

        for (int step = step_begin; step < step_end; ++step) {
            const bool more = step + 1 < step_end;
            if (more) {
                if constexpr (AHEAD) {
                    load_raw(step + 1);      // in flight during the MFMAs below
                }
            }
            if (wave_active) {
                const uint16_t * tile = wb[(step - step_begin) & 1];
#pragma unroll
                for (int s = 0; s < 4; ++s) {
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) {
                        const int k = (SHORT ? wave : kt) * 32 + l32;
                        const uint4 bits = *reinterpret_cast<const uint4 *>(&tile[k * BWD_PITCH + 16 * s + 8 * half]);
                        const v8bf bfrag = __builtin_bit_cast(v8bf, bits);
#pragma unroll
                        for (int rt = 0; rt < 2; ++rt) {
                            if (SHORT && rt >= row_tiles) {
                                break;
                            }
                            acc[rt][kt] = SHORT ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                                      __builtin_bit_cast(v8bf, afrag[rt][s]), bfrag, acc[rt][kt], 0, 0, 0)
                                                : __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                                      bfrag, __builtin_bit_cast(v8bf, afrag[rt][s]), acc[rt][kt], 0, 0, 0);
                        }
                    }
                }
            }
            if (more) {
                if (wave_active) {
                    load_cotangent(step + 1);   // in flight while the next tile is decoded
                }
                if constexpr (AHEAD) {
                    store_raw(step + 1);
                } else {
                    load_raw(step + 1);
                }
                decode(step + 1, wb[(step + 1 - step_begin) & 1]);
            }
        }

    }

    __syncthreads();   // the tiles are free: each wave reuses 8.5 KiB of them to transpose its results
    if constexpr (SHORT) {
        // the four 32-column slices of a 32-row tile meet in LDS and leave as whole 256-byte rows
        constexpr int STAGE_PITCH = BWD_TK + 8;
        static_assert(2 * 32 * STAGE_PITCH <= 2 * BWD_TK * BWD_PITCH, "both row tiles fit the weight tiles");
        uint16_t * stage = &wb[0][0];
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            if (rt < row_tiles) {
                stage_tile_32x32<STAGE_PITCH>(stage + rt * 32 * STAGE_PITCH, acc[rt][0], wave * 32, lane);
            }
        }
        __syncthreads();
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const int r0 = row_start + rt * 32;
            if (rt < row_tiles) {
                store_staged_rows<STAGE_PITCH>(stage + rt * 32 * STAGE_PITCH,
                                               a.dx + static_cast<int64_t>(r0) * a.in_features + k_tile * BWD_TK,
                                               a.in_features, row_end - r0, BWD_TK, tid, BWD_THREADS);
            }
        }
        return;
    } else {
    if (!wave_active) {
        return;
    }
    if (a.n_splits > 1) {
        // fp32 partial sums straight from the accumulators (operands swapped): a lane holds row l32 of its tile
        // and, as elements 4 j .. 4 j + 3, the four columns from 8 j + 4 half on: 16-byte stores
        float * out = a.partial + (static_cast<int64_t>(split) * a.rows + wave_row + l32) * a.in_features + k_tile * BWD_TK + 4 * half;
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            if (wave_row + rt * 32 + l32 < row_end) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        *reinterpret_cast<float4 *>(out + static_cast<int64_t>(rt * 32) * a.in_features + kt * 32 + 8 * j) =
                            make_float4(acc[rt][kt][4 * j], acc[rt][kt][4 * j + 1], acc[rt][kt][4 * j + 2], acc[rt][kt][4 * j + 3]);
                    }
                }
            }
        }
        return;
    }
    uint16_t * stage = &wb[0][0] + wave * (32 * (BWD_TK + 8));
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        const int r0 = wave_row + rt * 32;
        if (r0 < row_end) {
            store_rows_32x128<BWD_TK + 8, true, true>(stage, acc[rt], a.dx + static_cast<int64_t>(r0) * a.in_features + k_tile * BWD_TK,
                                                a.in_features, row_end - r0, BWD_TK, lane);
        }
    }
    }
}

// ---- role-split variant (Q4_K / Q5_K) ------------------------------------------------------------------------
// Same tile as above (256 rows x 128 values of K, reduction steps of 64 weight rows, double-buffered bf16
// tile), but the eight waves of a workgroup are specialised: waves 0-3 only multiply (64 rows each), waves
// 4-7 only dequantize.  Each SIMD then holds one wave that keeps the matrix pipe busy and one that keeps the
// vector ALU busy, and the two kinds of work overlap instead of alternating; one barrier per step hands the
// finished tile over.
//
// A workgroup is persistent: it owns every gridDim.x-th (task, column tile) item and runs their reduction
// steps as one stream, so the memory latency of an item's first loads and the drain of its last step are
// paid once per workgroup instead of once per item.  Nothing is loaded where it is used.  A decoder wave owns
// 16 of a step's 64 weight rows from global load to tile write (no barrier of its own; LDS traffic inside a
// wave is ordered) and works on four consecutive steps at once: while the multipliers consume step g it
// dequantizes step g+1, derives the block scales of step g+2, parks the packed blocks of step g+3 in LDS and
// has the blocks of steps g+4..g+7 in flight in registers, so no stage waits for the one before it.  A
// multiplier wave keeps the cotangent fragments of the next step in flight (two steps were measured: no faster, and
// the registers serve the weight-fragment look-ahead better).
constexpr int BSP_THREADS = 512;
constexpr int BSP_ROWS_PER_DECODER = BWD_NS / 4;   // weight rows a decoder wave owns per step
constexpr int BSP_RAW_DEPTH = 4;                   // steps of packed blocks in flight per decoder wave
constexpr int BSP_COT_DEPTH = 2;                   // cotangent fragment sets per multiplier wave (1 in use)
constexpr int BSP_SM_PITCH = BSP_ROWS_PER_DECODER + 1;
constexpr int BSP_MAX_ITEMS = 64;                  // items per workgroup (one wave builds the table)
constexpr int BSP_GRID = 256;                      // one workgroup per CU

// The compiler's wait-count bookkeeping gives up on loads that stay in flight across the back edge of the
// persistent loop (it drains the queue once per round, which exposes a full memory latency every few steps),
// so the prefetches of the role-split kernel are issued and awaited by hand.  Global loads return in order:
// waiting until at most N of them are outstanding completes everything but the N youngest.  The wait names
// the awaited registers as read-write operands so that no use of them can be scheduled ahead of it.

// `base` must be wave-uniform (it travels in scalar registers); `offset` is this lane's byte offset.
template <int IMMEDIATE = 0>
TGO_DEVICE void async_load16(u32x4 & destination, const void * base, uint32_t offset) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(destination) : "v"(offset), "s"(base), "n"(IMMEDIATE));
}
template <int YOUNGER>
TGO_DEVICE void await_loads(u32x4 (&r)[3]) {
    asm volatile("s_waitcnt vmcnt(%3)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]) : "n"(YOUNGER));
}
template <int YOUNGER>
TGO_DEVICE void await_loads(u32x4 (&r)[2][4]) {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(r[0][0]), "+v"(r[0][1]), "+v"(r[0][2]), "+v"(r[0][3]), "+v"(r[1][0]), "+v"(r[1][1]),
                   "+v"(r[1][2]), "+v"(r[1][3])
                 : "n"(YOUNGER));
}

struct SplitItem {
    int expert;
    int row_start;
    int row_end;
    int k_tile;
};

// Position in a workgroup's stream of reduction steps, with the item's description cached in scalars.
struct SplitCursor {
    int item;
    int source;
    int n_step;
    int expert;
    int row_start;
    int row_end;
    int k_tile;
    const uint8_t * base;   // where this step's loads start (meaning depends on the stage that owns the cursor)
};

template <int TYPE>
__global__ __launch_bounds__(BSP_THREADS, 2) void mmq_grad_input_split_kernel(const BackwardArgs a,
                                                                              const int total_items) {
    using F = Format<TYPE>;
    static_assert(TYPE == Q4_K || TYPE == Q5_K, "16-byte aligned blocks only");
    constexpr int RAW_UNITS = F::BLOCK_BYTES / 16;
    // LDS pitch of a parked block: the block itself (a multiple of 16 bytes for these formats), so a wave's units
    // land back to back with 16-byte writes; its readers address 16 rows at a time, which 36 or 44 words per row
    // still spread over distinct banks
    constexpr int BSP_RAW_PITCH = F::BLOCK_BYTES;
    constexpr int RAW_REGS = (BSP_ROWS_PER_DECODER * RAW_UNITS + 63) / 64;
    static_assert(RAW_REGS == 3, "await_loads takes three registers per step");
    constexpr int QS = TYPE == Q4_K ? 16 : 48;
    __shared__ __attribute__((aligned(16))) uint16_t wb[2][BWD_TK * BWD_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t raw_all[4][3][BSP_ROWS_PER_DECODER * BSP_RAW_PITCH];
    __shared__ float2 scale_min_all[4][2][4 * BSP_SM_PITCH];
    __shared__ __attribute__((aligned(16))) uint16_t stage_all[4][32 * (BWD_TK + 8)];
    __shared__ SplitItem items[BSP_MAX_ITEMS];
    __shared__ int item_count;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;

    // item table: slot i of this workgroup is linear item blockIdx.x + i * gridDim.x; empty slots (padding of
    // the task list) are squeezed out
    if (wave == 0) {
        SplitItem item = {0, 0, 0, -1};
        const int64_t linear = blockIdx.x + static_cast<int64_t>(lane) * gridDim.x;
        if (linear < total_items) {
            int k_tile, task, first_task = 0, ordinary = 0;
            int tasks = (a.rows + BWD_TR - 1) / BWD_TR;
            if (a.task_count != nullptr) {
                task_segment(a, first_task, tasks, ordinary);   // (never the short segment: first_task is 0)
                xcd_chunk(static_cast<int>(linear), a.k_tiles, tasks, ordinary, k_tile, task);
            } else {
                xcd_tile<BWD_XCD_RUN>(static_cast<int>(linear), a.k_tiles, tasks, k_tile, task);
            }
            if (a.task_count != nullptr) {
                if (task < tasks) {
                    item.expert = a.task_expert[task];
                    item.row_start = a.task_row_start[task];
                    item.row_end = a.task_row_end[task];
                    item.k_tile = k_tile;
                }
            } else if (task * BWD_TR < a.rows) {
                item.row_start = task * BWD_TR;
                item.row_end = min(a.rows, item.row_start + BWD_TR);
                item.k_tile = k_tile;
            }
        }
        const bool valid = item.k_tile >= 0;
        const unsigned long long mask = __ballot(valid);
        if (valid) {
            items[__popcll(mask & ((1ull << lane) - 1ull))] = item;
        }
        if (lane == 0) {
            item_count = __popcll(mask);
        }
    }
    __syncthreads();
    const int n_items = item_count;
    if (n_items == 0) {
        return;
    }
    const int n_total = a.out_features;
    const int steps_per_source = (n_total + BWD_NS - 1) / BWD_NS;
    const int total_steps = n_items * steps_per_source * a.sources;

    auto item_field = [&](int item, int field) {
        return __builtin_amdgcn_readfirstlane(reinterpret_cast<const int *>(&items[item])[field]);
    };
    auto open_item = [&](SplitCursor & c, int item) {
        c.item = item;
        c.expert = item_field(item, 0);
        c.row_start = item_field(item, 1);
        c.row_end = item_field(item, 2);
        c.k_tile = item_field(item, 3);
    };
    // `rebase(cursor)` sets cursor.base for step 0 of the cursor's (item, source); within a source the base
    // moves by `step_bytes` per step.
    auto first_step = [&](auto && rebase) {
        SplitCursor c;
        c.source = 0;
        c.n_step = 0;
        open_item(c, 0);
        rebase(c);
        return c;
    };
    // A cursor at the last step stays there: stages that look past the end repeat it (harmless re-reads
    // instead of branches).  Returns true when the cursor moved to another item.
    auto advance = [&](SplitCursor & c, auto && rebase, int64_t step_bytes) {
        if (c.n_step + 1 < steps_per_source) {
            ++c.n_step;
            c.base += step_bytes;
            return false;
        }
        if (c.source + 1 < a.sources) {
            c.n_step = 0;
            ++c.source;
            rebase(c);
            return false;
        }
        if (c.item + 1 < n_items) {
            c.n_step = 0;
            c.source = 0;
            open_item(c, c.item + 1);
            rebase(c);
            return true;
        }
        return false;
    };
    const uint8_t * const packed_of[2] = {a.packed[0], a.packed[1]};
    const uint8_t * const cotangent_of[2] = {a.cotangent[0], a.cotangent[1]};

    // Both roles run the same number of barriers: one after the first tile, then one per step.
    if (wave >= 4) {
        // ---------------- decoder wave ----------------
        const int dw = wave - 4;
        u32x4 ring[BSP_RAW_DEPTH][RAW_REGS];
        // loads of the other BSP_RAW_DEPTH - 1 register sets are younger than the set about to be parked
        constexpr int RAW_YOUNGER = (BSP_RAW_DEPTH - 1) * RAW_REGS;

        // Lane offsets of the 16-byte units this lane fetches per step, relative to the step's first weight
        // row; the last step of a source clamps rows past the end of the matrix to its last row.
        const int tail_rows = n_total - (steps_per_source - 1) * BWD_NS;
        uint32_t unit_offset[RAW_REGS], unit_offset_tail[RAW_REGS];
#pragma unroll
        for (int i = 0; i < RAW_REGS; ++i) {
            const int id = min(lane + 64 * i, BSP_ROWS_PER_DECODER * RAW_UNITS - 1);
            const int row = dw * BSP_ROWS_PER_DECODER + id / RAW_UNITS;
            const int unit = id % RAW_UNITS;
            unit_offset[i] = static_cast<uint32_t>(row * a.row_bytes + unit * 16);
            unit_offset_tail[i] = static_cast<uint32_t>(min(row, tail_rows - 1) * a.row_bytes + unit * 16);
        }
        auto rebase = [&](SplitCursor & c) {
            c.base = (c.source == 0 ? packed_of[0] : packed_of[1]) + static_cast<int64_t>(c.expert) * a.bytes_per_expert +
                     static_cast<int64_t>(c.k_tile >> 1) * F::BLOCK_BYTES;
        };
        const int64_t step_bytes = BWD_NS * a.row_bytes;
        auto load_raw = [&](const SplitCursor & c, u32x4 (&regs)[RAW_REGS]) {
            const bool tail = c.n_step == steps_per_source - 1;
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                async_load16(regs[i], c.base, tail ? unit_offset_tail[i] : unit_offset[i]);
            }
        };
        // stage 1: packed blocks from registers to an LDS slot
        auto park = [&](u32x4 (&regs)[RAW_REGS], uint8_t * raw) {
            await_loads<RAW_YOUNGER>(regs);
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = min(lane + 64 * i, BSP_ROWS_PER_DECODER * RAW_UNITS - 1);
                const int row = id / RAW_UNITS;
                const int unit = id - row * RAW_UNITS;
                static_assert(BSP_RAW_PITCH == RAW_UNITS * 16, "consecutive lanes write consecutive 16-byte units");
                *reinterpret_cast<u32x4 *>(raw + row * BSP_RAW_PITCH + unit * 16) = regs[i];
            }
        };
        // Stages 2 and 3 are each split into the LDS reads and the arithmetic on what was read, so that the
        // reads can be issued well before their results are needed (a lone wave has nothing else to cover an
        // LDS round trip with).
        //
        // stage 2: (d * sc, dmin * m) of this lane's (row, 32-value group); rows past the end of the weight
        // matrix get (0, 0) and therefore decode to exact zeros
        struct ScaleInputs {
            uint32_t d_dmin, low, mid, high;   // the 16-byte block header: two halves, then 12 bytes of 6-bit fields
        };
        auto scales_fetch = [&](const uint8_t * raw) {
            const uint8_t * blk = raw + (lane & 15) * BSP_RAW_PITCH;
            ScaleInputs in;
            in.d_dmin = lds_u32(blk);
            in.low = lds_u32(blk + 4);
            in.mid = lds_u32(blk + 8);
            in.high = lds_u32(blk + 12);
            return in;
        };
        auto scales_finish = [&](int info, const ScaleInputs & in, float2 * scale_min) {
            const int n = lane & 15;
            const int group_local = lane >> 4;
            const int shift = 8 * group_local;
            const uint32_t b0 = (in.low >> shift) & 0xffu, b1 = (in.mid >> shift) & 0xffu, b2 = (in.high >> shift) & 0xffu;
            uint32_t sc, mn;
            if ((info & 1) == 0) {   // groups 0..3 of the super-block: plain 6-bit fields
                sc = b0 & 63u;
                mn = b1 & 63u;
            } else {                 // groups 4..7: low nibbles in the third word, top two bits above the first eight
                sc = (b2 & 15u) | ((b0 >> 6) << 4);
                mn = (b2 >> 4) | ((b1 >> 6) << 4);
            }
            const bool valid = (info >> 1) * BWD_NS + dw * BSP_ROWS_PER_DECODER + n < n_total;
            scale_min[group_local * BSP_SM_PITCH + n] =
                valid ? make_float2(half_bits_to_float(in.d_dmin & 0xffffu) * static_cast<float>(sc),
                                    half_bits_to_float(in.d_dmin >> 16) * static_cast<float>(mn))
                      : make_float2(0.0f, 0.0f);
        };
        // stage 3: a lane decodes 8 weight rows x 4 consecutive K positions and stores each K position's
        // eight bf16 values with one 16-byte write
        struct DecodeInputs {
            uint32_t qs[8], qh[8];
            float2 sm[8];
        };
        const int octet = lane & 1;
        const int word = (lane >> 1) & 15;
        const int nibble = lane >> 5;
        const int position = (word & 7) * 4;
        const int group_local = 2 * (word >> 3) + nibble;
        auto decode_fetch = [&](int info, const uint8_t * raw, const float2 * scale_min) {
            const int half_block = info & 1;
            DecodeInputs in;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int n = 8 * octet + i;
                const uint8_t * blk = raw + n * BSP_RAW_PITCH;
                in.qs[i] = lds_u32(blk + QS + 64 * half_block + 4 * word);
                in.qh[i] = TYPE == Q5_K ? lds_u32(blk + 16 + position) : 0u;
                in.sm[i] = scale_min[group_local * BSP_SM_PITCH + n];
            }
            return in;
        };
        auto decode_finish = [&](int info, const DecodeInputs & in, uint16_t * tile) {
            const int group = 4 * (info & 1) + group_local;
            float w[4][8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                uint32_t q = (in.qs[i] >> (4 * nibble)) & 0x0f0f0f0fu;
                if constexpr (TYPE == Q5_K) {
                    q |= ((in.qh[i] >> group) & 0x01010101u) << 4;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    w[e][i] = in.sm[i].x * static_cast<float>((q >> (8 * e)) & 0xffu) - in.sm[i].y;
                }
            }
            const int k_local = 32 * group_local + position;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint4 packed = make_uint4(pack_bf16x2(w[e][0], w[e][1]), pack_bf16x2(w[e][2], w[e][3]),
                                                pack_bf16x2(w[e][4], w[e][5]), pack_bf16x2(w[e][6], w[e][7]));
                *reinterpret_cast<uint4 *>(
                    &tile[(k_local + e) * BWD_PITCH + dw * BSP_ROWS_PER_DECODER + 8 * octet]) = packed;
            }
        };
        auto wave_sync = [&]() {
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        };
        auto raw_slot = [&](int slot) { return raw_all[dw][slot]; };
        auto sm_slot = [&](int slot) { return scale_min_all[dw][slot]; };

        // Step t uses raw slot t % 3, scale slot t & 1, tile t & 1 and register set t % 4.  Only the load
        // stage walks the item list; what the later stages need to know about a step (which half of the
        // super-block, which 64 weight rows) follows it through a seven-deep queue of scalars.
        SplitCursor c_load = first_step(rebase);
        int info[7];   // info[i]: step g + 6 - i while the multipliers consume step g
        auto request = [&](u32x4 (&regs)[RAW_REGS]) {
            load_raw(c_load, regs);
#pragma unroll
            for (int i = 6; i > 0; --i) {
                info[i] = info[i - 1];
            }
            info[0] = (c_load.n_step << 1) | (c_load.k_tile & 1);
            advance(c_load, rebase, step_bytes);
        };
#pragma unroll
        for (int p = 0; p < BSP_RAW_DEPTH; ++p) {
            request(ring[p]);
        }
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            park(ring[t], raw_slot(t));
            request(ring[t]);
        }
        wave_sync();
        scales_finish(info[6], scales_fetch(raw_slot(0)), sm_slot(0));
        scales_finish(info[5], scales_fetch(raw_slot(1)), sm_slot(1));
        wave_sync();
        decode_finish(info[6], decode_fetch(info[6], raw_slot(0), sm_slot(0)), wb[0]);
        DecodeInputs pending = decode_fetch(info[5], raw_slot(1), sm_slot(1));   // step 1
        __syncthreads();
        // While the multipliers consume step g: finish decoding g + 1 (its inputs were read from LDS during
        // the previous round), scales of g + 2 (inputs read first thing, used after the decode), park g + 3,
        // request g + 7, and read the decode inputs of g + 2 so that they arrive during the barrier.  LDS
        // executes a wave's accesses in order, so a stage may read what an earlier stage of the same round
        // wrote without waiting; the fences only keep the compiler from reordering them.
        int g3 = 0;   // g % 3
#pragma unroll 1
        for (int base = 0; base < total_steps; base += BSP_RAW_DEPTH) {
#pragma unroll
            for (int u = 0; u < BSP_RAW_DEPTH; ++u) {
                const int g = base + u;
                if (g < total_steps) {
                    const int g3_plus1 = g3 == 2 ? 0 : g3 + 1;
                    const int g3_plus2 = g3_plus1 == 2 ? 0 : g3_plus1 + 1;
                    const ScaleInputs scale_inputs = scales_fetch(raw_slot(g3_plus2));
                    __builtin_amdgcn_sched_barrier(0);
                    decode_finish(info[5], pending, wb[(g + 1) & 1]);
                    scales_finish(info[4], scale_inputs, sm_slot(g & 1));
                    park(ring[(u + 3) % BSP_RAW_DEPTH], raw_slot(g3));
                    wave_sync();
                    pending = decode_fetch(info[4], raw_slot(g3_plus2), sm_slot(g & 1));
                    request(ring[(u + 3) % BSP_RAW_DEPTH]);
                    __builtin_amdgcn_sched_barrier(0);
                    g3 = g3_plus1;
                    __syncthreads();
                }
            }
        }
        return;
    }

    // ---------------- multiplier wave ----------------
    // byte offsets of this lane's fragment pieces inside the packed cotangent for an item, per 32-row tile of
    // the wave; a wave without rows in the item points every lane at one line (the loads stay, the cost goes)
    auto lane_offsets = [&](const SplitCursor & c, uint32_t (&offset)[2]) {
        const int wave_row = c.row_start + wave * 64;
        const bool active = wave_row < c.row_end;
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            int r = wave_row + rt * 32 + l32;
            r = r < a.rows_padded ? r : a.rows_padded - 1;
            offset[rt] = active ? static_cast<uint32_t>(r >> 5) * a.n_chunks * 1024 + ((r & 31) + 32 * half) * 16 : 0;
        }
    };
    // A step covers four 16-column chunks (the packed cotangent is zero padded to whole steps); a fragment
    // set is 2 row tiles x 4 chunks.
    u32x4 cot[BSP_COT_DEPTH][2][4];
    constexpr int COT_YOUNGER = (BSP_COT_DEPTH - 1) * 8;
    uint32_t fetch_offset[2];
    auto load_cotangent = [&](const SplitCursor & c, u32x4 (&regs)[2][4]) {
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            async_load16<0>(regs[rt][0], c.base, fetch_offset[rt]);
            async_load16<1024>(regs[rt][1], c.base, fetch_offset[rt]);
            async_load16<2048>(regs[rt][2], c.base, fetch_offset[rt]);
            async_load16<3072>(regs[rt][3], c.base, fetch_offset[rt]);
        }
    };
    auto rebase_fetch = [&](SplitCursor & c) { c.base = c.source == 0 ? cotangent_of[0] : cotangent_of[1]; };
    auto rebase_none = [&](SplitCursor &) {};

    v16f acc[2][4];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rt][kt][v] = 0.0f;

    SplitCursor c_fetch = first_step(rebase_fetch), c_now = c_fetch;
    lane_offsets(c_fetch, fetch_offset);
    auto fetch_next = [&]() {
        if (advance(c_fetch, rebase_fetch, (BWD_NS / 16) * 1024)) {
            lane_offsets(c_fetch, fetch_offset);
        }
    };
#pragma unroll
    for (int d = 0; d + 1 < BSP_COT_DEPTH; ++d) {
        load_cotangent(c_fetch, cot[d]);
        fetch_next();
    }
    __syncthreads();
#pragma unroll 1
    for (int base = 0; base < total_steps; base += BSP_COT_DEPTH) {
#pragma unroll
        for (int u = 0; u < BSP_COT_DEPTH; ++u) {
            const int g = base + u;
            if (g < total_steps) {
                load_cotangent(c_fetch, cot[(u + BSP_COT_DEPTH - 1) % BSP_COT_DEPTH]);
                fetch_next();
                await_loads<COT_YOUNGER>(cot[u]);
                const int wave_row = c_now.row_start + wave * 64;
                const int row_end = c_now.row_end;
                if (wave_row < row_end) {
                    // 16 weight fragments (4 chunks x 4 column tiles), two MFMAs each.  An LDS read takes
                    // longer than the two MFMAs it feeds, so fragment j + AHEAD is requested before fragment j
                    // is used; the scheduling groups below pin that interleaving.
                    const uint16_t * tile = wb[g & 1] + l32 * BWD_PITCH + 8 * half;
                    auto read_fragment = [&](int j) {
                        return *reinterpret_cast<const uint4 *>(&tile[(j & 3) * 32 * BWD_PITCH + 16 * (j >> 2)]);
                    };
                    constexpr int AHEAD = 6;
                    uint4 fragment[16];
#pragma unroll
                    for (int j = 0; j < AHEAD; ++j) {
                        fragment[j] = read_fragment(j);
                    }
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        if (j + AHEAD < 16) {
                            fragment[j + AHEAD] = read_fragment(j + AHEAD);
                        }
#pragma unroll
                        for (int rt = 0; rt < 2; ++rt) {
                            // (operands swapped: the lane ends up with one task row and runs of four neighbouring
                            // columns, which the epilogue stages with 8-byte LDS writes instead of 2-byte ones)
                            acc[rt][j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                __builtin_bit_cast(v8bf, fragment[j]), __builtin_bit_cast(v8bf, cot[u][rt][j >> 2]),
                                acc[rt][j & 3], 0, 0, 0);
                        }
                    }
                    __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);   // LDS reads
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        if (j + AHEAD < 16) {
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);   // MFMAs
                    }
                    if (c_now.source == a.sources - 1 && c_now.n_step == steps_per_source - 1) {
                        // last step of the item: transpose the results through this wave's staging area
                        // and write whole rows, then start the next item from zero
                        const int k_tile = c_now.k_tile;
                        // recomputing the per-lane store offsets here is cheaper than keeping them alive
                        // (spilled) through the loop, which is what happens if they can be hoisted
                        int lane_here = lane;
                        asm volatile("" : "+v"(lane_here));
#pragma unroll
                        for (int rt = 0; rt < 2; ++rt) {
                            const int r0 = wave_row + rt * 32;
                            if (r0 < row_end) {
                                store_rows_32x128<BWD_TK + 8, true, true>(
                                    stage_all[wave], acc[rt],
                                    a.dx + static_cast<int64_t>(r0) * a.in_features + k_tile * BWD_TK, a.in_features,
                                    row_end - r0, BWD_TK, lane_here);
                            }
#pragma unroll
                            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                                for (int v = 0; v < 16; ++v) acc[rt][kt][v] = 0.0f;
                        }
                    }
                }
                advance(c_now, rebase_none, 0);
                __syncthreads();
            }
        }
    }
}

// ---- short tasks ----------------------------------------------------------------------------------------------
// Tasks of at most BACKWARD_SHORT_ROWS rows.  Dequantizing a step's 64 x 128 weights costs the same however few
// rows multiply them, so here it is nearly all of the work and every wave does it: a wave owns 16 of the step's 64
// weight rows from the global load to the bf16 tile (packed blocks DEPTH steps ahead in registers, parked in the
// wave's own LDS slot, block scales, decode; LDS executes a wave's accesses in order, so these stages need no
// workgroup barrier), one barrier per step publishes the tile, and then every wave multiplies the task's rows with
// one 32-column slice of it (4 or 8 matrix instructions).  Small footprint: three workgroups share a CU, so one's
// barrier and memory waits are covered by the others' decoding.  One workgroup per (task, column tile).
// Q4_K / Q5_K fetch their blocks as the 16-byte units they consist of and have the block-scale stage; the other
// formats fetch the aligned units that cover their blocks (wide_fetch, callers check wide_stage_ok) and decode
// 16-value units straight from the parked blocks.
constexpr int BSH_THREADS = 256;
constexpr int BSH_ROWS_PER_WAVE = BWD_NS / 4;
constexpr int BSH_SM_PITCH = BSH_ROWS_PER_WAVE + 1;
constexpr int BSH_DEPTH = 2;

template <int TYPE>
__global__ __launch_bounds__(BSH_THREADS, 3) void mmq_grad_input_short_kernel(const BackwardArgs a) {
    using F = Format<TYPE>;
    constexpr bool K45 = TYPE == Q4_K || TYPE == Q5_K;
    using W = WideStage<TYPE>;
    constexpr int RAW_UNITS = K45 ? F::BLOCK_BYTES / 16 : W::UNITS;
    constexpr int BSH_RAW_PITCH = F::BLOCK_BYTES;   // Q4_K / Q5_K: as in the role-split kernel (16-byte park writes)
    constexpr int RAW_REGS = (BSH_ROWS_PER_WAVE * RAW_UNITS + 63) / 64;
    constexpr int SLOT_PITCH = K45 ? BSH_RAW_PITCH : W::PITCH;
    constexpr int SLOT_FRONT = K45 ? 0 : W::FRONT;
    constexpr int QS = TYPE == Q4_K ? 16 : 48;
    __shared__ __attribute__((aligned(16))) uint16_t wb[2][BWD_TK * BWD_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t raw_all[4][BSH_ROWS_PER_WAVE * SLOT_PITCH];
    __shared__ float2 scale_min_all[K45 ? 4 : 1][4 * BSH_SM_PITCH];
    // (the magnitude grid, not the 16 KiB selector table of decode16_bf16: with that table only two of these
    // workgroups fit a CU instead of three, which costs more than the cheaper decode brings -- measured)
    __shared__ uint2 grid[TYPE == IQ2_S ? TGO_IQ2S_GRID_ENTRIES : 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;

    int k_tile, task, first_task, tasks;
    task_segment(a, first_task, tasks);
    xcd_tile<1>(blockIdx.x, a.k_tiles, tasks, k_tile, task);
    if (task >= tasks) {
        return;
    }
    task += first_task;
    const int expert = a.task_expert[task];
    const int row_start = a.task_row_start[task];
    const int row_end = a.task_row_end[task];
    const int kb = k_tile >> 1;
    const int half_block = k_tile & 1;
    const int row_tiles = (row_end - row_start + 31) / 32;   // 1 or 2
    const int n_total = a.out_features;
    const int steps_per_source = (n_total + BWD_NS - 1) / BWD_NS;
    const int steps = steps_per_source * a.sources;
    const int last = steps - 1;

    uint8_t * const raw = raw_all[wave];
    float2 * const scale_min = scale_min_all[K45 ? wave : 0];
    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_grid(grid, tid, BSH_THREADS);   // (visible after the barrier that follows the first decode's inputs)
        __syncthreads();
    }

    // lane offsets of the 16-byte units this lane fetches per step, relative to the step's first weight row
    // (the last step of a source clamps rows past the end of the matrix to its last row)
    const int tail_rows = n_total - (steps_per_source - 1) * BWD_NS;
    uint32_t unit_offset[RAW_REGS], unit_offset_tail[RAW_REGS];
    if constexpr (K45) {
#pragma unroll
        for (int i = 0; i < RAW_REGS; ++i) {
            const int id = min(lane + 64 * i, BSH_ROWS_PER_WAVE * RAW_UNITS - 1);
            const int row = wave * BSH_ROWS_PER_WAVE + id / RAW_UNITS;
            const int unit = id % RAW_UNITS;
            unit_offset[i] = static_cast<uint32_t>(row * a.row_bytes + unit * 16);
            unit_offset_tail[i] = static_cast<uint32_t>(min(row, tail_rows - 1) * a.row_bytes + unit * 16);
        }
    }
    const int64_t expert_offset = static_cast<int64_t>(expert) * a.bytes_per_expert + static_cast<int64_t>(kb) * F::BLOCK_BYTES;
    // A step's packed blocks in flight: the units themselves (Q4_K / Q5_K) or the covering aligned units.
    struct InFlight {
        u32x4 unit[RAW_REGS];
        WideRegs<K45 ? 1 : RAW_REGS> wide;
    };
    // first of this wave's weight rows in a step and how many of them exist (at least one is read: a wave whose rows
    // all lie past the end of the matrix repeats the last row and decodes zeros)
    auto wave_rows = [&](int step, const uint8_t *& rows, int & rows_valid, int & n0) __attribute__((always_inline)) {
        step = min(step, last);
        const int source = step >= steps_per_source ? 1 : 0;
        n0 = (step - source * steps_per_source) * BWD_NS;
        const int first = min(n0 + wave * BSH_ROWS_PER_WAVE, n_total - 1);
        rows_valid = min(BSH_ROWS_PER_WAVE, n_total - first);
        rows = (source == 0 ? a.packed[0] : a.packed[1]) + static_cast<int64_t>(expert) * a.bytes_per_expert +
               static_cast<int64_t>(first) * a.row_bytes;
    };
    auto request = [&](int step, InFlight & regs) __attribute__((always_inline)) {
        if constexpr (K45) {
            step = min(step, last);
            const int source = step >= steps_per_source ? 1 : 0;
            const int n_step = step - source * steps_per_source;
            const uint8_t * base = (source == 0 ? a.packed[0] : a.packed[1]) + expert_offset +
                                   static_cast<int64_t>(n_step) * BWD_NS * a.row_bytes;
            const bool tail = n_step == steps_per_source - 1;
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                regs.unit[i] = *reinterpret_cast<const u32x4 *>(base + (tail ? unit_offset_tail[i] : unit_offset[i]));
            }
        } else {
            const uint8_t * rows;
            int rows_valid, n0;
            wave_rows(step, rows, rows_valid, n0);
            wide_fetch<TYPE, BSH_ROWS_PER_WAVE, 64, RAW_REGS>(regs.wide, rows, static_cast<int>(a.row_bytes), rows_valid, kb, lane);
        }
    };
    // (`step`: the one the registers were requested for)
    auto park = [&](int step, const InFlight & regs) __attribute__((always_inline)) {
        if constexpr (K45) {
#pragma unroll
            for (int i = 0; i < RAW_REGS; ++i) {
                const int id = min(lane + 64 * i, BSH_ROWS_PER_WAVE * RAW_UNITS - 1);
                const int row = id / RAW_UNITS;
                const int unit = id - row * RAW_UNITS;
                *reinterpret_cast<u32x4 *>(raw + row * BSH_RAW_PITCH + unit * 16) = regs.unit[i];
            }
        } else {
            const uint8_t * rows;
            int rows_valid, n0;
            wave_rows(step, rows, rows_valid, n0);
            wide_park<TYPE, BSH_ROWS_PER_WAVE, 64, RAW_REGS>(raw, regs.wide, rows, static_cast<int>(a.row_bytes), rows_valid, kb, lane);
        }
    };
    auto wave_sync = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
    // (d * sc, dmin * m) of this lane's (row, 32-value group); rows past the end of the weight matrix get (0, 0)
    // and therefore decode to exact zeros
    auto scales = [&](int step) __attribute__((always_inline)) {
        const int n = lane & 15;
        const int group_local = lane >> 4;
        const uint8_t * blk = raw + n * BSH_RAW_PITCH;
        const uint32_t d_dmin = lds_u32(blk), low = lds_u32(blk + 4), mid = lds_u32(blk + 8), high = lds_u32(blk + 12);
        const int shift = 8 * group_local;
        const uint32_t b0 = (low >> shift) & 0xffu, b1 = (mid >> shift) & 0xffu, b2 = (high >> shift) & 0xffu;
        uint32_t sc, mn;
        if (half_block == 0) {   // groups 0..3 of the super-block: plain 6-bit fields
            sc = b0 & 63u;
            mn = b1 & 63u;
        } else {                 // groups 4..7: low nibbles in the third word, top two bits above the first eight
            sc = (b2 & 15u) | ((b0 >> 6) << 4);
            mn = (b2 >> 4) | ((b1 >> 6) << 4);
        }
        const int source = step >= steps_per_source ? 1 : 0;
        const int n0 = (step - source * steps_per_source) * BWD_NS;
        const bool valid = n0 + wave * BSH_ROWS_PER_WAVE + n < n_total;
        scale_min[group_local * BSH_SM_PITCH + n] =
            valid ? make_float2(half_bits_to_float(d_dmin & 0xffffu) * static_cast<float>(sc),
                                half_bits_to_float(d_dmin >> 16) * static_cast<float>(mn))
                  : make_float2(0.0f, 0.0f);
    };
    // a lane decodes 8 weight rows x 4 consecutive K positions and stores each K position's eight bf16 values with
    // one 16-byte write
    const int octet = lane & 1;
    const int word = (lane >> 1) & 15;
    const int nibble = lane >> 5;
    const int position = (word & 7) * 4;
    const int group_local = 2 * (word >> 3) + nibble;
    const int group = 4 * half_block + group_local;
    auto decode = [&](int step, uint16_t * tile) __attribute__((always_inline)) {
        if constexpr (!K45) {
            // 16 rows x 8 units of 16 values: a lane takes one row and two units; neighbouring lanes hold neighbouring
            // rows of the same values and swap halves so that each writes both rows of one k, four bytes at a time
            const uint8_t * rows;
            int rows_valid, n0;
            wave_rows(step, rows, rows_valid, n0);
            const int n = lane & 15;
            uint32_t keep = n0 + wave * BSH_ROWS_PER_WAVE + n < n_total ? 0xffffffffu : 0u;
            asm volatile("" : "+v"(keep));   // (a mask, not a branch around part of the arithmetic)
            const uint32_t selector = (lane & 1) != 0 ? 0x03020706u : 0x05040100u;
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                const int unit = (lane >> 4) + 4 * pass;
                uint32_t pairs[8];
                decode16_bf16<TYPE>(raw + n * SLOT_PITCH + SLOT_FRONT, 8 * half_block + unit, grid, pairs);
                uint32_t * const pair_row = reinterpret_cast<uint32_t *>(
                    &tile[(unit * 16 + (lane & 1)) * BWD_PITCH + wave * BSH_ROWS_PER_WAVE + (n & ~1)]);
#pragma unroll
                for (int j = 0; j < 16; j += 2) {
                    const uint32_t own = pairs[j / 2] & keep;
                    const uint32_t other = static_cast<uint32_t>(
                        __builtin_amdgcn_mov_dpp(static_cast<int>(own), 0xB1, 0xf, 0xf, true));   // lane ^ 1
                    pair_row[j * (BWD_PITCH / 2)] = __builtin_amdgcn_perm(other, own, selector);
                }
            }
            return;
        }
        uint32_t qs[8], qh[8];
        float2 sm[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int n = 8 * octet + i;
            const uint8_t * blk = raw + n * BSH_RAW_PITCH;
            qs[i] = lds_u32(blk + QS + 64 * half_block + 4 * word);
            qh[i] = TYPE == Q5_K ? lds_u32(blk + 16 + position) : 0u;
            sm[i] = scale_min[group_local * BSH_SM_PITCH + n];
        }
        float w[4][8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint32_t q = (qs[i] >> (4 * nibble)) & 0x0f0f0f0fu;
            if constexpr (TYPE == Q5_K) {
                q |= ((qh[i] >> group) & 0x01010101u) << 4;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                w[e][i] = sm[i].x * static_cast<float>((q >> (8 * e)) & 0xffu) - sm[i].y;
            }
        }
        const int k_local = 32 * group_local + position;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint4 packed = make_uint4(pack_bf16x2(w[e][0], w[e][1]), pack_bf16x2(w[e][2], w[e][3]),
                                            pack_bf16x2(w[e][4], w[e][5]), pack_bf16x2(w[e][6], w[e][7]));
            *reinterpret_cast<uint4 *>(&tile[(k_local + e) * BWD_PITCH + wave * BSH_ROWS_PER_WAVE + 8 * octet]) = packed;
        }
    };

    // cotangent fragments of the task's (up to) two 32-row tiles; one set, requested right after the
    // multiplications that used the previous one and awaited a whole decode later
    uint32_t lane_offset[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        int r = row_start + rt * 32 + l32;
        r = r < a.rows_padded ? r : a.rows_padded - 1;
        lane_offset[rt] = static_cast<uint32_t>(r >> 5) * a.n_chunks * 1024 + ((r & 31) + 32 * half) * 16;
    }
    u32x4 cot[2][4] = {};
    auto request_cotangent = [&](int step) __attribute__((always_inline)) {
        step = min(step, last);
        const int source = step >= steps_per_source ? 1 : 0;
        const int n0 = (step - source * steps_per_source) * BWD_NS;
        // (the packed cotangent is zero padded to whole steps of 64 columns)
        const uint8_t * base = (source == 0 ? a.cotangent[0] : a.cotangent[1]) + static_cast<int64_t>(n0 >> 4) * 1024;
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            if (rt < row_tiles) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    cot[rt][c] = *reinterpret_cast<const u32x4 *>(base + lane_offset[rt] + c * 1024);
                }
            }
        }
    };
    v16f acc[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rt][v] = 0.0f;
    auto multiply = [&](const uint16_t * tile) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint4 bits = *reinterpret_cast<const uint4 *>(&tile[(wave * 32 + l32) * BWD_PITCH + 16 * c + 8 * half]);
            const v8bf bfrag = __builtin_bit_cast(v8bf, bits);
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                if (rt < row_tiles) {
                    acc[rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, cot[rt][c]), bfrag, acc[rt], 0, 0, 0);
                }
            }
        }
    };

    InFlight ring[BSH_DEPTH];
#pragma unroll
    for (int d = 0; d < BSH_DEPTH; ++d) {
        request(d, ring[d]);
    }
    request_cotangent(0);
    park(0, ring[0]);
    request(BSH_DEPTH, ring[0]);
    wave_sync();
    if constexpr (K45) {
        scales(0);
        wave_sync();
    }
    decode(0, wb[0]);
    __syncthreads();
    // A step that has a successor: multiply its tile and prepare the next one.  The loop below holds no branch, so
    // the compiler's wait-count bookkeeping sees every request on every path; with the last step's exceptions inside
    // it, the paths that skip a wait made it wait for the newest requests before the matrix instructions (a whole
    // memory round trip per step).
    static_assert(BSH_DEPTH == 2, "tile and ring parity follow the position in the unrolled round");
    auto advance = [&](int step, auto parity_tag) __attribute__((always_inline)) {
        constexpr int u = decltype(parity_tag)::value;
        // (this wave's decode of the current step, the last reader of its slot, is behind it in program order)
        // the chain of dependent waits goes first, the arithmetic of the decode fills in (measured: 1 %)
        __builtin_amdgcn_s_setprio(3);
        park(step + 1, ring[u ^ 1]);
        multiply(wb[u]);
        // both requests go out behind the matrix instructions, which wait for the previous step's cotangent only
        request_cotangent(step + 1);
        request(step + 1 + BSH_DEPTH, ring[u ^ 1]);
        wave_sync();
        if constexpr (K45) {
            scales(step + 1);
            wave_sync();
        }
        __builtin_amdgcn_s_setprio(0);
        decode(step + 1, wb[u ^ 1]);
        __syncthreads();
    };
    int step = 0;
#pragma unroll 1
    for (; step + 2 <= last; step += 2) {
        advance(step, std::integral_constant<int, 0>{});
        advance(step + 1, std::integral_constant<int, 1>{});
    }
    if (step < last) {   // uniform
        advance(step, std::integral_constant<int, 0>{});
        multiply(wb[1]);
    } else {
        multiply(wb[0]);
    }
    __syncthreads();
    // the tiles are free (every wave is past its last multiplication): the four 32-column slices of a 32-row tile
    // meet in LDS and leave as whole 256-byte rows
    constexpr int STAGE_PITCH = BWD_TK + 8;
    static_assert(2 * 32 * STAGE_PITCH <= 2 * BWD_TK * BWD_PITCH, "both row tiles fit the weight tiles");
    static_assert(BSH_DEPTH % 2 == 0, "tile parity follows the position in the unrolled round");
    uint16_t * stage = &wb[0][0];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        if (rt < row_tiles) {
            stage_tile_32x32<STAGE_PITCH>(stage + rt * 32 * STAGE_PITCH, acc[rt], wave * 32, lane);
        }
    }
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        const int r0 = row_start + rt * 32;
        if (rt < row_tiles) {
            store_staged_rows<STAGE_PITCH>(stage + rt * 32 * STAGE_PITCH,
                                           a.dx + static_cast<int64_t>(r0) * a.in_features + k_tile * BWD_TK,
                                           a.in_features, row_end - r0, BWD_TK, tid, BSH_THREADS);
        }
    }
}

// dx[i] = bf16(partial[0][i] + partial[1][i] + ...), eight values per thread; `count` is a multiple of 8.
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float * __restrict__ partial,
                                                              uint16_t * __restrict__ dx, int64_t count, int n_splits) {
    const int64_t first = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
    if (first >= count) {
        return;
    }
    float sum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sum[e] = 0.0f;
    for (int s = 0; s < n_splits; ++s) {
        const float4 lo = *reinterpret_cast<const float4 *>(partial + s * count + first);
        const float4 hi = *reinterpret_cast<const float4 *>(partial + s * count + first + 4);
        sum[0] += lo.x; sum[1] += lo.y; sum[2] += lo.z; sum[3] += lo.w;
        sum[4] += hi.x; sum[5] += hi.y; sum[6] += hi.z; sum[7] += hi.w;
    }
    *reinterpret_cast<uint4 *>(dx + first) = make_uint4(pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3]),
                                                        pack_bf16x2(sum[4], sum[5]), pack_bf16x2(sum[6], sum[7]));
}

template <int TYPE>
static hipError_t launch_backward_typed(const BackwardArgs & args, hipStream_t stream) {
    const int64_t total = static_cast<int64_t>(args.k_tiles) *
                          (args.task_count != nullptr ? xcd_chunk_slots(args.task_slots) : pad_task_slots(args.task_slots, BWD_XCD_RUN));
    const int64_t total_short = static_cast<int64_t>(args.k_tiles) * pad_task_slots(args.short_slots);
    if (total <= 0 || total > 0x7fffffffLL || total_short > 0x7fffffffLL) {
        return hipErrorInvalidValue;
    }
    const ProfileScope scope(3, stream);
    // the general kernel, in its variant for short tasks or not, with the packed blocks fetched as wide units
    // where the format needs that and the weights allow it
    const auto general = [&](auto short_tag, dim3 grid, const BackwardArgs & launch_args) {
        constexpr bool SHORT = decltype(short_tag)::value;
        if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
            const int64_t weight_bytes = static_cast<int64_t>(args.out_features) * args.row_bytes;
            // (and the rows short enough for the 24-bit multiplies of the unit offsets)
            if (args.row_bytes < (1 << 24) && wide_stage_ok(args.packed[0], weight_bytes) &&
                (args.packed[1] == nullptr || wide_stage_ok(args.packed[1], weight_bytes))) {
                mmq_grad_input_kernel<TYPE, SHORT, true><<<grid, BWD_THREADS, 0, stream>>>(launch_args);
                return;
            }
        }
        mmq_grad_input_kernel<TYPE, SHORT, false><<<grid, BWD_THREADS, 0, stream>>>(launch_args);
    };
    if (args.segment == 1) {
        // grouped call: the short tasks (a separate segment of the task list) run in a launch of their own
        BackwardArgs short_args = args;
        short_args.segment = 2;
        bool launched = false;
        // (32-bit lane offsets into the packed cotangent and a step's weight rows, as in the role-split kernel)
        if (cotangent_workspace_bytes(args.rows, args.out_features) < (int64_t{1} << 32) &&
            args.row_bytes * 2 * BWD_NS < (int64_t{1} << 32)) {
            bool fits = true;
            if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
                const int64_t weight_bytes = static_cast<int64_t>(args.out_features) * args.row_bytes;
                fits = args.row_bytes < (1 << 24) && wide_stage_ok(args.packed[0], weight_bytes) &&
                       (args.packed[1] == nullptr || wide_stage_ok(args.packed[1], weight_bytes));
            }
            if (fits) {
                mmq_grad_input_short_kernel<TYPE><<<static_cast<unsigned>(total_short), BSH_THREADS, 0, stream>>>(short_args);
                launched = true;
            }
        }
        if (!launched) {
            general(std::true_type{}, dim3(static_cast<unsigned>(total_short)), short_args);
        }
        const hipError_t status = hipGetLastError();
        if (status != hipSuccess) {
            return status;
        }
    }
    if (args.n_splits > 1) {
        // (every format takes the general kernel here: what this path needs is many short workgroups)
        const dim3 grid(static_cast<unsigned>(total), static_cast<unsigned>(args.n_splits));
        general(std::false_type{}, grid, args);
        const int64_t count = static_cast<int64_t>(args.rows) * args.in_features;
        reduce_partials_kernel<<<static_cast<unsigned>((count / 8 + 255) / 256), 256, 0, stream>>>(
            args.partial, args.dx, count, args.n_splits);
        return hipGetLastError();
    }
    // the role-split kernel addresses the packed cotangent and a step's weight rows with 32-bit lane offsets
    const bool small_offsets = cotangent_workspace_bytes(args.rows, args.out_features) < (int64_t{1} << 32) &&
                               args.row_bytes * 2 * BWD_NS < (int64_t{1} << 32);
    if constexpr (TYPE == Q4_K || TYPE == Q5_K) {
        if (small_offsets) {
            // one persistent workgroup per CU, more only when a workgroup's item table would overflow
            const int64_t needed = (total + BSP_MAX_ITEMS - 1) / BSP_MAX_ITEMS;
            const int64_t grid =
                (std::max<int64_t>(std::min<int64_t>(total, BSP_GRID), needed) + XCDS - 1) / XCDS * XCDS;
            mmq_grad_input_split_kernel<TYPE><<<static_cast<unsigned>(grid), BSP_THREADS, 0, stream>>>(
                args, static_cast<int>(total));
            return hipGetLastError();
        }
    }
    general(std::false_type{}, dim3(static_cast<unsigned>(total)), args);
    return hipGetLastError();
}

hipError_t launch_mmq_grad_input(const uint8_t * cotangent_first, const uint8_t * cotangent_second,
                                 const uint8_t * packed_first, const uint8_t * packed_second,
                                 int64_t bytes_per_expert, uint16_t * grad_input, const TaskList * tasks,
                                 int rows, int out_features, int in_features, int quant_type,
                                 hipStream_t stream, float * partial) {
    BackwardArgs args;
    // `partial` (dense calls only): room for dense_grad_splits() fp32 copies of the result, or nullptr
    args.partial = partial;
    args.n_splits = tasks == nullptr && partial != nullptr
        ? dense_grad_splits(rows, out_features, in_features, has_role_split(quant_type)) : 1;
    args.cotangent[0] = cotangent_first;
    args.cotangent[1] = cotangent_second;
    args.packed[0] = packed_first;
    args.packed[1] = packed_second;
    args.sources = packed_second != nullptr ? 2 : 1;
    args.bytes_per_expert = bytes_per_expert;
    args.row_bytes = static_cast<int64_t>(in_features / QK_K) * block_bytes(quant_type);
    args.dx = grad_input;
    args.rows = rows;
    args.rows_padded = static_cast<int>(pad_rows(rows));
    args.out_features = out_features;
    args.n_chunks = cotangent_chunks(out_features);
    args.in_features = in_features;
    args.k_tiles = in_features / BWD_TK;
    if (tasks != nullptr) {
        args.task_count = tasks->count;
        args.task_early = tasks->early;
        args.task_expert = tasks->expert;
        args.task_row_start = tasks->row_start;
        args.task_row_end = tasks->row_end;
        args.task_slots = tasks->max_tasks;
        // max_tasks = full row tiles + one remainder per group: the remainders are all that can be short
        args.short_slots = tasks->max_tasks - (rows + BWD_TR - 1) / BWD_TR;
        args.segment = 1;
    } else {
        args.task_count = nullptr;
        args.task_early = nullptr;
        args.short_slots = 0;
        args.segment = 0;
        args.task_expert = nullptr;
        args.task_row_start = nullptr;
        args.task_row_end = nullptr;
        args.task_slots = (rows + BWD_TR - 1) / BWD_TR;
    }
    switch (quant_type) {
        case Q3_K: return launch_backward_typed<Q3_K>(args, stream);
        case Q4_K: return launch_backward_typed<Q4_K>(args, stream);
        case Q5_K: return launch_backward_typed<Q5_K>(args, stream);
        case Q6_K: return launch_backward_typed<Q6_K>(args, stream);
        case IQ2_S: return launch_backward_typed<IQ2_S>(args, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace tgo
