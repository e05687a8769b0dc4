// Auxiliary gfx950 kernels: weight dequantizer, q8_1 activation quantizer (which also builds the tile-task list
// of a grouped call on the side), workspace inspection and the routing-weighted row -> token combine.
#include <atomic>
#include "tgo_device.h"
#include "tgo_launch.h"

namespace tgo {

// ---- packed rows -> bf16 ---------------------------------------------------------------------
// One workgroup decodes 16 rows x one super-block: blocks are staged in LDS with coalesced loads,
// then each thread turns 16 consecutive weights into 32 bytes of bf16.
constexpr int DEQUANT_ROWS = 16;

template <int TYPE>
__global__ __launch_bounds__(256) void dequant_bf16_kernel(const uint8_t * __restrict__ packed,
                                                          uint16_t * __restrict__ out, int rows,
                                                          int in_features, int64_t row_bytes) {
    using F = Format<TYPE>;
    __shared__ __attribute__((aligned(16))) uint8_t raw[DEQUANT_ROWS * F::RAW_PITCH];
    __shared__ uint2 grid[TYPE == IQ2_S ? TGO_IQ2S_GRID_ENTRIES : 1];
    const int tid = threadIdx.x;
    const int row0 = blockIdx.x * DEQUANT_ROWS;
    const int kb = blockIdx.y;
    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_grid(grid, tid, 256);
    }
    stage_blocks<TYPE>(raw, packed, row_bytes, row0, rows, kb, DEQUANT_ROWS, tid, 256);
    __syncthreads();

    const int row = tid >> 4;
    const int unit = tid & 15;
    if (row0 + row >= rows) {
        return;
    }
    float w[16];
    decode16_f32<TYPE>(raw + row * F::RAW_PITCH + F::RAW_SHIFT, unit, grid, w);
    uint4 lo, hi;
    lo.x = pack_bf16x2(w[0], w[1]);   lo.y = pack_bf16x2(w[2], w[3]);
    lo.z = pack_bf16x2(w[4], w[5]);   lo.w = pack_bf16x2(w[6], w[7]);
    hi.x = pack_bf16x2(w[8], w[9]);   hi.y = pack_bf16x2(w[10], w[11]);
    hi.z = pack_bf16x2(w[12], w[13]); hi.w = pack_bf16x2(w[14], w[15]);
    uint4 * dst = reinterpret_cast<uint4 *>(out + static_cast<int64_t>(row0 + row) * in_features + kb * QK_K + unit * 16);
    dst[0] = lo;
    dst[1] = hi;
}

hipError_t launch_dequant_bf16(const uint8_t * packed, uint16_t * out, int64_t rows, int64_t in_features,
                               int quant_type, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>((rows + DEQUANT_ROWS - 1) / DEQUANT_ROWS),
                    static_cast<unsigned>(in_features / QK_K));
    const int64_t row_bytes = (in_features / QK_K) * block_bytes(quant_type);
    const int r = static_cast<int>(rows), k = static_cast<int>(in_features);
    const ProfileScope scope(4, stream);
    switch (quant_type) {
        case Q3_K: dequant_bf16_kernel<Q3_K><<<grid, 256, 0, stream>>>(packed, out, r, k, row_bytes); break;
        case Q4_K: dequant_bf16_kernel<Q4_K><<<grid, 256, 0, stream>>>(packed, out, r, k, row_bytes); break;
        case Q5_K: dequant_bf16_kernel<Q5_K><<<grid, 256, 0, stream>>>(packed, out, r, k, row_bytes); break;
        case Q6_K: dequant_bf16_kernel<Q6_K><<<grid, 256, 0, stream>>>(packed, out, r, k, row_bytes); break;
        case IQ2_S: dequant_bf16_kernel<IQ2_S><<<grid, 256, 0, stream>>>(packed, out, r, k, row_bytes); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---- matrix operands of the forward kernels (process-wide) -------------------------------------------
static std::atomic<int> g_forward_operand{OPERAND_AUTO};
int forward_operand_setting() { return g_forward_operand.load(std::memory_order_relaxed); }
void set_forward_operand_setting(int operand) { g_forward_operand.store(operand, std::memory_order_relaxed); }

// ---- bf16 activations -> q8_1 -------------------------------------------------------------------
// The arithmetic is quantize_eight's (tgo_device.h).  The tile layouts: one workgroup handles 32 rows x 256 values and
// writes one contiguous 8 KiB run of fragment-ordered int8.
// Row-major variant for calls that take the GEMV kernels (a handful of rows): workgroup = one row x 2048 values.
__global__ __launch_bounds__(256) void quantize_q8_1_rows_kernel(const uint16_t * __restrict__ input,
                                                                int8_t * __restrict__ q_out,
                                                                float * __restrict__ d_out,
                                                                float * __restrict__ sum_out, int in_features,
                                                                const int64_t * __restrict__ gather,
                                                                int64_t input_rows, uint32_t * __restrict__ tag,
                                                                const TaskBuild build) {
    if (build.tasks.count != nullptr && blockIdx.x == 0 && blockIdx.y == 0) {
        build_tasks(build, threadIdx.x);
    }
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
        *tag = WORKSPACE_TAG_MAGIC | LAYOUT_ROWS;
    }
    const int row = blockIdx.x;
    const int k = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (k >= in_features) {   // whole groups of four lanes leave together (in_features is a multiple of 256)
        return;
    }
    int64_t source = row;
    bool present = true;
    if (gather != nullptr) {
        source = gather[row];
        present = source >= 0 && source < input_rows;
    }
    uint4 bits = make_uint4(0, 0, 0, 0);
    if (present) {
        bits = *reinterpret_cast<const uint4 *>(input + source * in_features + k);
    }
    float x[8];
    unpack_bf16x8(bits, x);
    uint32_t packed[2], halves[4];
    int magnitude[8];
    float d, total;
    quantize_eight(bits, x, packed, d, total, halves, magnitude);
    *reinterpret_cast<uint2 *>(q_out + static_cast<int64_t>(row) * in_features + k) = make_uint2(packed[0], packed[1]);
    if ((threadIdx.x & 3) == 0) {
        const int64_t block = static_cast<int64_t>(row) * (in_features / 32) + k / 32;
        d_out[block] = d;
        sum_out[block] = total;
    }
}

// Where 16-byte piece `piece` of a quantizer's LDS tile lives.  The lanes of a store differ in the 8 values of K they
// hold, and those land a whole run of 32 pieces (512 bytes) apart: all on the same four banks.  So a piece's place inside
// its run is exchanged by the run's number, which spreads the pieces of one store over all banks; the copy out of the
// tile reads the pieces back through the same exchange.
TGO_DEVICE int swizzled_piece(int piece) { return piece ^ ((piece >> 5) & 15); }

// LAYOUT_HALF_TILES: the quants leave as fp16 numbers for the fp16-operand forward kernels, 16 KiB per workgroup:
// per 32-value block two 1 KiB slabs (k-halves of 16 values), each 64 pieces of eight values = (eighth of the
// k-half, row).
template <int LAYOUT>
__global__ __launch_bounds__(256) void quantize_q8_1_kernel(const uint16_t * __restrict__ input,
                                                           int8_t * __restrict__ q_out,
                                                           float * __restrict__ d_out,
                                                           float * __restrict__ sum_out,
                                                           uint32_t * __restrict__ tag, int rows,
                                                           int in_features,
                                                           const int64_t * __restrict__ gather,
                                                           int64_t input_rows, const TaskBuild build) {
    constexpr bool WIDE_VALUES = LAYOUT != LAYOUT_INT8_TILES;   // two bytes per value
    static_assert(LAYOUT == LAYOUT_INT8_TILES || LAYOUT == LAYOUT_HALF_TILES, "the scaled layout has a kernel of its own");
    if (build.tasks.count != nullptr && blockIdx.x == 0 && blockIdx.y == 0) {
        build_tasks(build, threadIdx.x);
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        *tag = WORKSPACE_TAG_MAGIC | LAYOUT;
    }
    // Workgroups that are launched together take neighbouring column chunks of the same 32 rows, so that what the
    // chip reads and writes at any time are whole rows and 8 KiB fragment runs next to each other (with the row
    // tiles of one chunk launched together instead, the same kernel ran at 4.8 instead of 5.9 TB/s).
    const int chunks = in_features / 256;
    const int64_t rows_padded = (static_cast<int64_t>(rows) + 31) / 32 * 32;
    __shared__ __attribute__((aligned(16))) uint8_t tile[(WIDE_VALUES ? 16 : 8) * 1024];
    __shared__ __attribute__((aligned(16))) float scales[2][8][32];   // d and sum of the tile: [which][block][row]
    const int tid = threadIdx.x;
    const int row_tile = blockIdx.x / chunks;                 // 32-row tile
    const int chunk = blockIdx.x - row_tile * chunks;         // 256-value column chunk
    const int blocks_per_row = in_features / 32;
    const int lane_k = tid & 31;       // 8 values each
    const int block = lane_k >> 2;     // 32-value block inside the chunk
    const int quarter = lane_k & 3;

    // All four row loads of a thread are in flight together (rows past the end and gather indices outside the
    // input read a valid row and are zeroed afterwards): with a branch around each load the passes would run one
    // memory round trip after the other.
    int64_t source[4];
    bool present[4];
    const int last_row = rows - 1;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int row = row_tile * 32 + (tid >> 5) + 8 * pass;
        present[pass] = row < rows;
        source[pass] = min(row, last_row);
        if (gather != nullptr) {   // uniform
            source[pass] = gather[source[pass]];
        }
    }
    uint4 bits[4];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        if (gather != nullptr) {
            present[pass] = present[pass] && source[pass] >= 0 && source[pass] < input_rows;
            source[pass] = present[pass] ? source[pass] : 0;
        }
        bits[pass] = *reinterpret_cast<const uint4 *>(input + source[pass] * in_features + chunk * 256 + lane_k * 8);
    }
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int rr = (tid >> 5) + 8 * pass;
        float x[8];
        const uint4 row_bits = present[pass] ? bits[pass] : uint4{0, 0, 0, 0};
        unpack_bf16x8(row_bits, x);
        uint32_t packed[2], halves[4];
        int magnitude[8];
        float d, total;
        quantize_eight(row_bits, x, packed, d, total, halves, magnitude);
        const int half = quarter >> 1;
        if constexpr (WIDE_VALUES) {
            // values 8 * quarter .. + 7 of the block: k-half quarter / 2, eighth quarter % 2, i.e. piece lane_k * 32 + rr
            *reinterpret_cast<uint4 *>(tile + swizzled_piece(lane_k * 32 + rr) * 16) =
                make_uint4(halves[0], halves[1], halves[2], halves[3]);
        } else {
            // (piece (2 * block + half) * 32 + rr, one half of it per lane)
            uint2 * dst = reinterpret_cast<uint2 *>(tile + swizzled_piece((lane_k >> 1) * 32 + rr) * 16 + 8 * (quarter & 1));
            *dst = make_uint2(packed[0], packed[1]);
        }
        if (quarter == 0) {
            scales[0][block][rr] = d;
            scales[1][block][rr] = total;
        }
    }
    __syncthreads();
    // the 32 rows of a block are one 128-byte line of each scale plane: 2 planes x 8 blocks x 8 pieces
    if (tid < 128) {
        const int which = tid >> 6, b = (tid >> 3) & 7, piece = tid & 7;
        float * plane = which == 0 ? d_out : sum_out;
        *reinterpret_cast<float4 *>(plane + static_cast<int64_t>(chunk * 8 + b) * rows_padded + row_tile * 32 + piece * 4) =
            *reinterpret_cast<const float4 *>(&scales[which][b][piece * 4]);
    }
    constexpr int BLOCK_BYTES = WIDE_VALUES ? 2048 : 1024;
    uint4 * dst = reinterpret_cast<uint4 *>(
        q_out + (static_cast<int64_t>(row_tile) * blocks_per_row + chunk * 8) * BLOCK_BYTES);
    const uint4 * src = reinterpret_cast<const uint4 *>(tile);
#pragma unroll
    for (int piece = 0; piece < 8 * BLOCK_BYTES / 16 / 256; ++piece) {
        dst[tid + 256 * piece] = src[swizzled_piece(tid + 256 * piece)];
    }
}

// LAYOUT_SCALED_TILES: the fp16 slabs of the half layout hold the dequantized values d * q instead of q, normalised
// per row and super-block (the 256 values of a row that a workgroup handles) by the power of two 2^e that brings the
// super-block's largest block scale into [2^1, 2^2): every |d * q * 2^-e| stays below 2^9 and is rounded once to fp16
// (relative 2^-12).  The block sums, scaled alike, go to `block_sums` as fp16, eight per row and super-block: the
// operand that meets the block minima of Q4_K/Q5_K.  2^e goes to the `power` plane; a second, small pass
// (scaled_row_power_kernel) turns it into 2^(e - E) with E the row's largest exponent, which the forward kernel
// multiplies into the fragments of the super-block (exact: a power of two), and writes 2^E per row.  The scale and
// sum planes are written as in every layout.
__global__ __launch_bounds__(256) void quantize_q8_1_scaled_kernel(const uint16_t * __restrict__ input,
                                                                  int8_t * __restrict__ q_out,
                                                                  float * __restrict__ d_out,
                                                                  float * __restrict__ sum_out,
                                                                  float * __restrict__ power_out,
                                                                  uint16_t * __restrict__ block_sums_out,
                                                                  uint32_t * __restrict__ tag, int rows,
                                                                  int in_features,
                                                                  const int64_t * __restrict__ gather,
                                                                  int64_t input_rows, const TaskBuild build) {
    if (build.tasks.count != nullptr && blockIdx.x == 0) {
        build_tasks(build, threadIdx.x);
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        *tag = WORKSPACE_TAG_MAGIC | LAYOUT_SCALED_TILES;
    }
    // (workgroup order as in quantize_q8_1_kernel: neighbouring workgroups take neighbouring chunks of the same rows)
    const int chunks = in_features / 256;
    const int64_t rows_padded = (static_cast<int64_t>(rows) + 31) / 32 * 32;
    __shared__ __attribute__((aligned(16))) uint8_t tile[16 * 1024];
    __shared__ __attribute__((aligned(16))) float scales[2][8][32];   // d and sum of the tile: [which][block][row]
    __shared__ __attribute__((aligned(16))) float powers[32];
    __shared__ __attribute__((aligned(16))) uint16_t sums_half[32][8];
    const int tid = threadIdx.x;
    const int row_tile = blockIdx.x / chunks;                 // 32-row tile
    const int chunk = blockIdx.x - row_tile * chunks;         // 256-value column chunk
    const int blocks_per_row = in_features / 32;
    const int lane_k = tid & 31;       // 8 values each
    const int block = lane_k >> 2;     // 32-value block inside the chunk
    const int quarter = lane_k & 3;

    int64_t source[4];
    bool present[4];
    const int last_row = rows - 1;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int row = row_tile * 32 + (tid >> 5) + 8 * pass;
        present[pass] = row < rows;
        source[pass] = min(row, last_row);
        if (gather != nullptr) {   // uniform
            source[pass] = gather[source[pass]];
        }
    }
    uint4 bits[4];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        if (gather != nullptr) {
            present[pass] = present[pass] && source[pass] >= 0 && source[pass] < input_rows;
            source[pass] = present[pass] ? source[pass] : 0;
        }
        bits[pass] = *reinterpret_cast<const uint4 *>(input + source[pass] * in_features + chunk * 256 + lane_k * 8);
    }
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int rr = (tid >> 5) + 8 * pass;
        float x[8];
        const uint4 row_bits = present[pass] ? bits[pass] : uint4{0, 0, 0, 0};
        unpack_bf16x8(row_bits, x);
        uint32_t packed[2], halves[4];
        int magnitude[8];
        float d, total;
        quantize_eight(row_bits, x, packed, d, total, halves, magnitude);
        // the row's 32 lanes hold its eight block scales; the largest one fixes the super-block's exponent
        float largest = fmaxf(d, __shfl_xor(d, 4));
        largest = fmaxf(largest, __shfl_xor(largest, 8));
        largest = fmaxf(largest, __shfl_xor(largest, 16));
        int exponent = static_cast<int>(__float_as_uint(largest) >> 23);   // biased; d is never negative
        exponent = min(max(exponent, 2), 254);
        const float power = __uint_as_float(static_cast<uint32_t>(exponent - 1) << 23);     // 2^e
        const float inverse = __uint_as_float(static_cast<uint32_t>(255 - exponent) << 23);   // 2^-e
        const float lane_scale = d * inverse;
        const uint32_t words[4] = {row_bits.x, row_bits.y, row_bits.z, row_bits.w};
#pragma unroll
        for (int pair = 0; pair < 4; ++pair) {
            const half2_t values = {static_cast<_Float16>(static_cast<float>(magnitude[2 * pair]) * lane_scale),
                                    static_cast<_Float16>(static_cast<float>(magnitude[2 * pair + 1]) * lane_scale)};
            halves[pair] = __builtin_bit_cast(uint32_t, values) | (words[pair] & 0x80008000u);
        }
        // values 8 * quarter .. + 7 of the block: k-half quarter / 2, eighth quarter % 2, i.e. piece lane_k * 32 + rr
        *reinterpret_cast<uint4 *>(tile + swizzled_piece(lane_k * 32 + rr) * 16) =
            make_uint4(halves[0], halves[1], halves[2], halves[3]);
        if (quarter == 0) {
            scales[0][block][rr] = d;
            scales[1][block][rr] = total;
            sums_half[rr][block] = __builtin_bit_cast(uint16_t, static_cast<_Float16>(total * inverse));
        }
        if (lane_k == 0) {
            powers[rr] = power;
        }
    }
    __syncthreads();
    // the 32 rows of a block are one 128-byte line of each scale plane: 2 planes x 8 blocks x 8 pieces
    if (tid < 128) {
        const int which = tid >> 6, b = (tid >> 3) & 7, piece = tid & 7;
        float * plane = which == 0 ? d_out : sum_out;
        *reinterpret_cast<float4 *>(plane + static_cast<int64_t>(chunk * 8 + b) * rows_padded + row_tile * 32 + piece * 4) =
            *reinterpret_cast<const float4 *>(&scales[which][b][piece * 4]);
    } else if (tid < 136) {
        const int piece = tid - 128;
        *reinterpret_cast<float4 *>(power_out + static_cast<int64_t>(chunk) * rows_padded + row_tile * 32 + piece * 4) =
            *reinterpret_cast<const float4 *>(&powers[piece * 4]);
    } else if (tid >= 192 && tid < 224) {
        const int row = tid - 192;
        *reinterpret_cast<uint4 *>(block_sums_out + ((static_cast<int64_t>(row_tile) * chunks + chunk) * 32 + row) * 8) =
            *reinterpret_cast<const uint4 *>(&sums_half[row][0]);
    }
    uint4 * dst = reinterpret_cast<uint4 *>(q_out + (static_cast<int64_t>(row_tile) * blocks_per_row + chunk * 8) * 2048);
    const uint4 * src = reinterpret_cast<const uint4 *>(tile);
#pragma unroll
    for (int piece = 0; piece < 4; ++piece) {
        dst[tid + 256 * piece] = src[swizzled_piece(tid + 256 * piece)];
    }
}

// Second pass of the scaled layout: power[sb][row] = 2^e  ->  2^(e - E), row_power[row] = 2^E with E = max over sb.
__global__ __launch_bounds__(256) void scaled_row_power_kernel(float * __restrict__ power, float * __restrict__ row_power,
                                                              int64_t rows_padded, int chunks) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (row >= rows_padded) {
        return;
    }
    float largest = 0.0f;
    for (int c = 0; c < chunks; ++c) {
        largest = fmaxf(largest, power[c * rows_padded + row]);
    }
    // (all entries are powers of two between 2^-126 and 2^126: the quotient is exact)
    const float inverse = __uint_as_float((254u - (__float_as_uint(largest) >> 23)) << 23);
    for (int c = 0; c < chunks; ++c) {
        power[c * rows_padded + row] *= inverse;
    }
    row_power[row] = largest;
}

hipError_t launch_quantize_q8_1(const uint16_t * input, const Q8Workspace & ws, int64_t rows,
                                int64_t in_features, hipStream_t stream, const int64_t * gather,
                                int64_t input_rows, const TaskBuild * build) {
    const ProfileScope scope(0, stream);
    const TaskBuild on_the_side = build != nullptr ? *build : no_task_build();
    if (ws.by_rows()) {
        const dim3 grid(static_cast<unsigned>(rows), static_cast<unsigned>((in_features + 2047) / 2048));
        quantize_q8_1_rows_kernel<<<grid, 256, 0, stream>>>(input, ws.q, ws.d, ws.sum, static_cast<int>(in_features),
                                                            gather, input_rows, ws.tag, on_the_side);
        return hipGetLastError();
    }
    const int r = static_cast<int>(rows), k = static_cast<int>(in_features);
    const int64_t workgroups = ws.rows_padded / 32 * (in_features / 256);
    if (workgroups > 0x7fffffffLL) {
        return hipErrorInvalidValue;
    }
    const dim3 grid(static_cast<unsigned>(workgroups));
    if (ws.scaled_tiles()) {
        quantize_q8_1_scaled_kernel<<<grid, 256, 0, stream>>>(input, ws.q, ws.d, ws.sum, ws.power, ws.block_sums, ws.tag, r, k,
                                                              gather, input_rows, on_the_side);
        scaled_row_power_kernel<<<static_cast<unsigned>((ws.rows_padded + 255) / 256), 256, 0, stream>>>(
            ws.power, ws.row_power, ws.rows_padded, k / 256);
        return hipGetLastError();
    }
    if (ws.half_tiles()) {
        quantize_q8_1_kernel<LAYOUT_HALF_TILES><<<grid, 256, 0, stream>>>(input, ws.q, ws.d, ws.sum, ws.tag, r, k, gather,
                                                                           input_rows, on_the_side);
    } else {
        quantize_q8_1_kernel<LAYOUT_INT8_TILES><<<grid, 256, 0, stream>>>(input, ws.q, ws.d, ws.sum, ws.tag, r, k, gather,
                                                                           input_rows, on_the_side);
    }
    return hipGetLastError();
}

// Workspace inspection for tests: the quants, scales and sums as plain rows, whichever layout the quantizer wrote
// (read from the workspace's tag; a workspace without a valid tag yields zeros).  The scaled layout stores d * q:
// its quants are recovered as round(value * 2^e / d), exact because the fp16 rounding moves a value by less than
// 127 * 2^-12 of a quant step (values that the normalisation pushed below the fp16 range come back as zero).
__global__ __launch_bounds__(256) void q8_unpack_kernel(const int8_t * __restrict__ q_frag,
                                                       const float * __restrict__ d_in,
                                                       const float * __restrict__ sum_in,
                                                       const float * __restrict__ power_in,
                                                       const float * __restrict__ row_power_in,
                                                       const uint32_t * __restrict__ tag,
                                                       int8_t * __restrict__ q, float * __restrict__ d,
                                                       float * __restrict__ sum, int rows,
                                                       int in_features) {
    const int64_t index = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t total = static_cast<int64_t>(rows) * in_features;
    if (index >= total) {
        return;
    }
    const uint32_t word = *tag;
    const int layout = (word & 0xffff0000u) == WORKSPACE_TAG_MAGIC ? static_cast<int>(word & 0xffffu) : -1;
    const int row = static_cast<int>(index / in_features);
    const int k = static_cast<int>(index % in_features);
    const int blocks_per_row = in_features / 32;
    const int block = k >> 5, half = (k >> 4) & 1, byte = k & 15;
    const int64_t block_index = static_cast<int64_t>(row) * blocks_per_row + block;
    if (layout < 0 || layout > LAYOUT_SCALED_TILES) {
        q[index] = 0;
        if ((k & 31) == 0) {
            d[block_index] = 0.0f;
            sum[block_index] = 0.0f;
        }
        return;
    }
    if (layout == LAYOUT_ROWS) {
        q[index] = q_frag[index];
        if ((k & 31) == 0) {
            d[block_index] = d_in[block_index];
            sum[block_index] = sum_in[block_index];
        }
        return;
    }
    const int64_t rows_padded = (static_cast<int64_t>(rows) + 31) / 32 * 32;
    const float scale = d_in[block * rows_padded + row];
    if (layout == LAYOUT_INT8_TILES) {
        q[index] = q_frag[(static_cast<int64_t>(row >> 5) * blocks_per_row + block) * 1024 +
                          ((row & 31) + 32 * half) * 16 + byte];
    } else {
        const _Float16 * values = reinterpret_cast<const _Float16 *>(q_frag);
        float value = static_cast<float>(
            values[(static_cast<int64_t>(row >> 5) * blocks_per_row + block) * 1024 + half * 512 +
                   ((row & 31) + 32 * (byte >> 3)) * 8 + (byte & 7)]);
        if (layout == LAYOUT_SCALED_TILES) {
            value = scale == 0.0f ? 0.0f : rintf(value * (power_in[(k >> 8) * rows_padded + row] * row_power_in[row]) / scale);
        }
        q[index] = static_cast<int8_t>(value);
    }
    if ((k & 31) == 0) {
        d[block_index] = scale;
        sum[block_index] = sum_in[block * rows_padded + row];
    }
}

hipError_t launch_q8_unpack(const Q8Workspace & ws, int8_t * q, float * d, float * sum, int64_t rows,
                            int64_t in_features, hipStream_t stream) {
    const int64_t total = rows * in_features;
    q8_unpack_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, stream>>>(
        ws.q, ws.d, ws.sum, ws.power, ws.row_power, ws.tag, q, d, sum, static_cast<int>(rows), static_cast<int>(in_features));
    return hipGetLastError();
}

// ---- a prepared workspace consumed as the wrong kind ---------------------------------------------------------
// The quantizer and a later tgo_mmq_forward_prepared each derive the workspace layout from the process-wide operand
// setting; a change of the setting between the two would make the multiply kernel read the bytes as another layout.
// The host cannot see the tag without a synchronisation, so this runs behind the multiply kernel: when the tag is not
// the one the launch assumed, every output becomes NaN (bf16 0x7fc0) instead of plausible garbage.  With the right
// tag each thread reads one word and leaves.
__global__ __launch_bounds__(256) void workspace_guard_kernel(const uint32_t * __restrict__ tag, uint32_t expected,
                                                              uint16_t * __restrict__ out, int64_t count) {
    if (*tag == expected) {
        return;
    }
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += static_cast<int64_t>(gridDim.x) * 256) {
        out[i] = 0x7fc0u;
    }
}

hipError_t launch_workspace_guard(const Q8Workspace & ws, uint16_t * out, int64_t count, hipStream_t stream) {
    const unsigned grid = static_cast<unsigned>(count < 256 * 1024 ? (count + 255) / 256 : 1024);
    workspace_guard_kernel<<<grid == 0 ? 1 : grid, 256, 0, stream>>>(ws.tag, WORKSPACE_TAG_MAGIC | static_cast<uint32_t>(ws.layout),
                                                                     out, count);
    return hipGetLastError();
}

// ---- expert-sorted rows -> tokens --------------------------------------------------------------
// out[t, :] = sum over the token's choices j of weight[t, j] * rows[slot_row[t, j], :].
// One workgroup per token and 2048-feature span; a thread owns 8 consecutive features, i.e. one 16-byte
// load per choice, four choices in flight.  Choices are added in index order into fp32 with fused
// multiply-adds and rounded to bf16 once, so the result does not depend on scheduling.
constexpr int COMBINE_SPAN = 256 * 8;

__global__ __launch_bounds__(256) void moe_combine_kernel(const uint16_t * __restrict__ rows,
                                                          const int64_t * __restrict__ slot_rows,
                                                          const float * __restrict__ slot_weights,
                                                          uint16_t * __restrict__ out, int top_k, int64_t num_rows,
                                                          int features) {
    const int64_t token = blockIdx.x;
    const int feature = blockIdx.y * COMBINE_SPAN + threadIdx.x * 8;
    if (feature >= features) {
        return;
    }
    const int64_t * choice_rows = slot_rows + token * top_k;
    const float * choice_weights = slot_weights + token * top_k;
    float acc[8] = {};
    for (int first = 0; first < top_k; first += 4) {
        uint4 bits[4];
        float weight[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int choice = min(first + u, top_k - 1);
            const int64_t row = choice_rows[choice];
            const bool present = first + u < top_k && row >= 0 && row < num_rows;
            weight[u] = present ? choice_weights[choice] : 0.0f;
            bits[u] = present ? *reinterpret_cast<const uint4 *>(rows + row * features + feature) : uint4{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t words[4] = {bits[u].x, bits[u].y, bits[u].z, bits[u].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] = __builtin_fmaf(weight[u], bf16_bits_to_float(words[i] & 0xffffu), acc[2 * i]);
                acc[2 * i + 1] = __builtin_fmaf(weight[u], bf16_bits_to_float(words[i] >> 16), acc[2 * i + 1]);
            }
        }
    }
    uint4 packed;
    packed.x = pack_bf16x2(acc[0], acc[1]);
    packed.y = pack_bf16x2(acc[2], acc[3]);
    packed.z = pack_bf16x2(acc[4], acc[5]);
    packed.w = pack_bf16x2(acc[6], acc[7]);
    *reinterpret_cast<uint4 *>(out + token * features + feature) = packed;
}

// activated[i] = bf16(silu(gate[i]) * up[i]): the second pass of a SwiGLU pair whose multiply kernel has no fused
// epilogue.  `activated` may be the tensor that holds the up projection (the value is read before it is replaced).
// Eight values per thread and step when all three tensors start on a 16-byte boundary.
__global__ __launch_bounds__(256) void swiglu_rows_kernel(const uint16_t * __restrict__ gate, const uint16_t * up,
                                                           uint16_t * activated, int64_t count, int vector) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    const int64_t first = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t pieces = vector != 0 ? count / 8 : 0;
    for (int64_t piece = first; piece < pieces; piece += stride) {
        reinterpret_cast<uint4 *>(activated)[piece] =
            swiglu_bf16x8(reinterpret_cast<const uint4 *>(gate)[piece], reinterpret_cast<const uint4 *>(up)[piece]);
    }
    for (int64_t index = pieces * 8 + first; index < count; index += stride) {
        activated[index] = swiglu_bf16(gate[index], up[index]);
    }
}

hipError_t launch_swiglu_rows(const uint16_t * gate, const uint16_t * up, uint16_t * activated, int64_t count,
                              hipStream_t stream) {
    const int vector =
        (reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) | reinterpret_cast<uintptr_t>(activated)) % 16 == 0;
    const int64_t blocks = (count / (vector != 0 ? 8 : 1) + 255) / 256;
    const ProfileScope scope(2, stream);
    swiglu_rows_kernel<<<static_cast<unsigned>(blocks < 1 ? 1 : blocks > 8 * 256 * 8 ? 8 * 256 * 8 : blocks), 256, 0, stream>>>(
        gate, up, activated, count, vector);
    return hipGetLastError();
}

// Routing of a small batch in one launch: the (token, choice) slots sorted by expert, stably, by one workgroup.
//   slot_rows[i]      sorted row of slot i (-1 for a slot whose expert is out of range)
//   row_index[r]      token of sorted row r (slot / top_k); -1 behind the last row
//   expert_offsets[e] rows of experts 0..e (the grouped operators' offsets with one group per expert),
//   expert_indices[e] = e
// A counting sort: the experts' counts (LDS atomics), their prefix sum, then the slots 256 at a time in slot order,
// each taking the next place of its expert plus the number of earlier slots of the same expert in its batch of 256.
// What a decode step otherwise does with a sort and a dozen tensor operations, each a launch of its own.
constexpr int ROUTE_SMALL_LIMIT = 4096;   // slots and experts one workgroup handles
__global__ __launch_bounds__(256) void route_small_kernel(const int64_t * __restrict__ slot_experts, int slots, int top_k,
                                                          int num_experts, int64_t * __restrict__ row_index,
                                                          int64_t * __restrict__ slot_rows,
                                                          int64_t * __restrict__ expert_indices,
                                                          int32_t * __restrict__ expert_offsets) {
    __shared__ int next_row[ROUTE_SMALL_LIMIT];   // counts, then each expert's next free row
    __shared__ int batch_expert[256];
    __shared__ int thread_total[256];
    const int tid = threadIdx.x;
    for (int e = tid; e < num_experts; e += 256) {
        next_row[e] = 0;
    }
    for (int i = tid; i < slots; i += 256) {
        row_index[i] = -1;
    }
    __syncthreads();
    for (int i = tid; i < slots; i += 256) {
        const int64_t expert = slot_experts[i];
        if (expert >= 0 && expert < num_experts) {
            atomicAdd(&next_row[static_cast<int>(expert)], 1);
        }
    }
    __syncthreads();
    // prefix sum over the experts: a thread owns a run of consecutive experts
    const int run = (num_experts + 255) / 256;
    const int first = tid * run;
    int mine = 0;
    for (int e = first; e < min(first + run, num_experts); ++e) {
        mine += next_row[e];
    }
    thread_total[tid] = mine;
    __syncthreads();
    for (int offset = 1; offset < 256; offset <<= 1) {
        const int add = tid >= offset ? thread_total[tid - offset] : 0;
        __syncthreads();
        thread_total[tid] += add;
        __syncthreads();
    }
    int before = thread_total[tid] - mine;
    for (int e = first; e < min(first + run, num_experts); ++e) {
        const int count = next_row[e];
        next_row[e] = before;
        before += count;
        expert_offsets[e] = before;
        expert_indices[e] = e;
    }
    __syncthreads();
    for (int base = 0; base < slots; base += 256) {
        const int i = base + tid;
        int expert = -1;
        if (i < slots) {
            const int64_t named = slot_experts[i];
            expert = named >= 0 && named < num_experts ? static_cast<int>(named) : -1;
        }
        batch_expert[tid] = expert;
        __syncthreads();
        int row = -1;
        if (expert >= 0) {
            int earlier = 0;
            for (int j = 0; j < tid; ++j) {
                earlier += batch_expert[j] == expert ? 1 : 0;
            }
            row = next_row[expert] + earlier;
        }
        __syncthreads();   // (every slot of the batch has read its expert's next row)
        if (expert >= 0) {
            atomicAdd(&next_row[expert], 1);
            row_index[row] = i / top_k;
        }
        if (i < slots) {
            slot_rows[i] = row;
        }
        __syncthreads();
    }
}

hipError_t launch_route_small(const int64_t * slot_experts, int slots, int top_k, int num_experts, int64_t * row_index,
                              int64_t * slot_rows, int64_t * expert_indices, int32_t * expert_offsets, hipStream_t stream) {
    if (slots > ROUTE_SMALL_LIMIT || num_experts > ROUTE_SMALL_LIMIT) {
        return hipErrorInvalidValue;
    }
    route_small_kernel<<<1, 256, 0, stream>>>(slot_experts, slots, top_k, num_experts, row_index, slot_rows, expert_indices,
                                              expert_offsets);
    return hipGetLastError();
}

// The gather of the grouped operators run backwards: out[t, :] = bf16(sum of rows[order[i], :] for i in
// [starts[t], starts[t + 1])), added in list order in fp32 and rounded once (no atomics: the same bits every time).
// `order` lists the sorted rows token by token, `starts` where each token's run begins.  Entries that name no row,
// and runs that reach outside the list, contribute nothing.  Same shape of work as moe_combine_kernel.
__global__ __launch_bounds__(256) void rows_to_tokens_kernel(const uint16_t * __restrict__ rows,
                                                             const int64_t * __restrict__ order,
                                                             const int64_t * __restrict__ starts,
                                                             uint16_t * __restrict__ out, int64_t num_rows, int features) {
    const int64_t token = blockIdx.x;
    const int feature = blockIdx.y * COMBINE_SPAN + threadIdx.x * 8;
    if (feature >= features) {
        return;
    }
    const int64_t begin = max(starts[token], int64_t{0});
    const int64_t end = min(starts[token + 1], num_rows);
    float acc[8] = {};
    for (int64_t first = begin; first < end; first += 4) {
        uint4 bits[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t row = order[min(first + u, end - 1)];
            const bool present = first + u < end && row >= 0 && row < num_rows;
            bits[u] = present ? *reinterpret_cast<const uint4 *>(rows + row * features + feature) : uint4{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t words[4] = {bits[u].x, bits[u].y, bits[u].z, bits[u].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] += bf16_bits_to_float(words[i] & 0xffffu);
                acc[2 * i + 1] += bf16_bits_to_float(words[i] >> 16);
            }
        }
    }
    *reinterpret_cast<uint4 *>(out + token * features + feature) =
        uint4{pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]), pack_bf16x2(acc[4], acc[5]), pack_bf16x2(acc[6], acc[7])};
}

hipError_t launch_rows_to_tokens(const uint16_t * rows, const int64_t * order, const int64_t * starts, uint16_t * out,
                                 int tokens, int64_t num_rows, int features, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>((features + COMBINE_SPAN - 1) / COMBINE_SPAN));
    const ProfileScope scope(7, stream);
    rows_to_tokens_kernel<<<grid, 256, 0, stream>>>(rows, order, starts, out, num_rows, features);
    return hipGetLastError();
}

// The activation's cotangent taken back to the two projections, elementwise: with s = sigmoid(gate),
//   d_up = bf16(dy * gate * s),   d_gate = bf16(dy * up * s * (1 + gate * (1 - s)) [+ grad_gate]),
// all factors read as bf16 and multiplied in fp32.  `grad_gate` (a cotangent that reached the gate output itself) may
// be null.  One pass over five (six) tensors instead of the dozen fp32 passes of the same formulas written with
// tensor operations.
TGO_DEVICE void swiglu_backward(float gate, float up, float dy, float direct, float & d_gate, float & d_up) {
    const float s = __builtin_amdgcn_rcpf(1.0f + __expf(-gate));
    d_up = dy * (gate * s);
    d_gate = dy * up * (s * (1.0f + gate * (1.0f - s))) + direct;
}

__global__ __launch_bounds__(256) void swiglu_backward_rows_kernel(const uint16_t * __restrict__ gate,
                                                                    const uint16_t * __restrict__ up,
                                                                    const uint16_t * __restrict__ grad_activated,
                                                                    const uint16_t * __restrict__ grad_gate,
                                                                    uint16_t * __restrict__ d_gate,
                                                                    uint16_t * __restrict__ d_up, int64_t count, int vector) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    const int64_t first = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t pieces = vector != 0 ? count / 8 : 0;
    for (int64_t piece = first; piece < pieces; piece += stride) {
        const uint4 g4 = reinterpret_cast<const uint4 *>(gate)[piece];
        const uint4 u4 = reinterpret_cast<const uint4 *>(up)[piece];
        const uint4 y4 = reinterpret_cast<const uint4 *>(grad_activated)[piece];
        const uint4 r4 = grad_gate != nullptr ? reinterpret_cast<const uint4 *>(grad_gate)[piece] : uint4{0, 0, 0, 0};
        const uint32_t g[4] = {g4.x, g4.y, g4.z, g4.w}, u[4] = {u4.x, u4.y, u4.z, u4.w};
        const uint32_t y[4] = {y4.x, y4.y, y4.z, y4.w}, r[4] = {r4.x, r4.y, r4.z, r4.w};
        uint32_t out_gate[4], out_up[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float dg[2], du[2];
            swiglu_backward(bf16_bits_to_float(g[i] & 0xffffu), bf16_bits_to_float(u[i] & 0xffffu),
                            bf16_bits_to_float(y[i] & 0xffffu), bf16_bits_to_float(r[i] & 0xffffu), dg[0], du[0]);
            swiglu_backward(bf16_bits_to_float(g[i] >> 16), bf16_bits_to_float(u[i] >> 16), bf16_bits_to_float(y[i] >> 16),
                            bf16_bits_to_float(r[i] >> 16), dg[1], du[1]);
            out_gate[i] = pack_bf16x2(dg[0], dg[1]);
            out_up[i] = pack_bf16x2(du[0], du[1]);
        }
        reinterpret_cast<uint4 *>(d_gate)[piece] = uint4{out_gate[0], out_gate[1], out_gate[2], out_gate[3]};
        reinterpret_cast<uint4 *>(d_up)[piece] = uint4{out_up[0], out_up[1], out_up[2], out_up[3]};
    }
    for (int64_t index = pieces * 8 + first; index < count; index += stride) {
        float dg, du;
        swiglu_backward(bf16_bits_to_float(gate[index]), bf16_bits_to_float(up[index]), bf16_bits_to_float(grad_activated[index]),
                        grad_gate != nullptr ? bf16_bits_to_float(grad_gate[index]) : 0.0f, dg, du);
        d_gate[index] = to_bf16_bits(dg);
        d_up[index] = to_bf16_bits(du);
    }
}

hipError_t launch_swiglu_backward_rows(const uint16_t * gate, const uint16_t * up, const uint16_t * grad_activated,
                                       const uint16_t * grad_gate, uint16_t * d_gate, uint16_t * d_up, int64_t count,
                                       hipStream_t stream) {
    const uintptr_t addresses = reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) |
                                reinterpret_cast<uintptr_t>(grad_activated) | reinterpret_cast<uintptr_t>(grad_gate) |
                                reinterpret_cast<uintptr_t>(d_gate) | reinterpret_cast<uintptr_t>(d_up);
    const int vector = addresses % 16 == 0;
    const int64_t blocks = (count / (vector != 0 ? 8 : 1) + 255) / 256;
    swiglu_backward_rows_kernel<<<static_cast<unsigned>(blocks < 1 ? 1 : blocks > 8 * 256 * 8 ? 8 * 256 * 8 : blocks), 256, 0,
                                  stream>>>(gate, up, grad_activated, grad_gate, d_gate, d_up, count, vector);
    return hipGetLastError();
}

hipError_t launch_moe_combine(const uint16_t * rows, const int64_t * slot_rows, const float * slot_weights,
                              uint16_t * out, int tokens, int top_k, int64_t num_rows, int features,
                              hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>((features + COMBINE_SPAN - 1) / COMBINE_SPAN));
    const ProfileScope scope(7, stream);
    moe_combine_kernel<<<grid, 256, 0, stream>>>(rows, slot_rows, slot_weights, out, top_k, num_rows, features);
    return hipGetLastError();
}

}  // namespace tgo
