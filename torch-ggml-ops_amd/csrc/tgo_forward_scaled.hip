// Forward kernel with scaled fp16 operands: q8_1 activations x packed GGUF weights as one fp16 matrix product per
// task, bounded by the matrix pipe instead of the vector pipe.
//
//   y[r, n] = 2^(E[r] + S[n]) * sum over k of  w[n, k] * h[r, k]      (v_mfma_f32_32x32x16_f16, fp32 accumulation)
//   h[r, k] = fp16(dx * qx * 2^-E[r])     the dequantized q8_1 activation, normalised per row, rounded once
//   w[n, k] = fp16(v[n, k] * fp16(scale * 2^-S[n]))   the integer operand v = sub-scale x quant (exact in fp16) times
//             the weight scale of its group, normalised per weight row
// Q4_K/Q5_K: v = q, scale = d * sc, and the minimum term -dmin * m * (block sum) is one more reduction step per
// super-block whose operands are fp16(-dmin * m * 2^-S[n]) and fp16(block sum * 2^-E[r]).  The quantizer writes h, the
// block sums and 2^E (quantize_q8_1_scaled_kernel); S[n] comes from a scan of the weight row's super-block scales.
// The algebra is the q8_1 one (same quants, block scales and sums as the int8 kernels of tgo_forward.hip); what
// differs is that both operands carry their scales into the matrix instruction, each rounded to fp16 once (relative
// 2^-11: the reference keeps its own scale products d * sc and dmin * m as halves too,
// csrc/vendor/llama_cpp/mmq-load-targets.cuh:190-195), so that no vector instruction touches a result between the
// first and the last reduction step.  The int8 kernels spend two or three vector operations per result on every 32
// values, which bounds them at a quarter of the matrix pipe's rate.
//
// Work split: role-split workgroup of eight waves, one per CU.  Waves 0-3 multiply: wave w owns activation rows
// [64w, 64w + 64) of the task and all 128 weight rows of the column tile (2 x 4 tiles of 32 x 32, 128 accumulator
// registers; the activations are the A operand, so a lane holds one weight row per tile and 16 activation rows).
// Waves 4-7 unpack: wave 4 + t owns weight rows [32t, 32t + 32) from the global load of their packed blocks to
// their fp16 operand tile (packed blocks FSC_RAW_DEPTH super-blocks ahead in registers, parked in the wave's own LDS
// slot; LDS executes a wave's accesses in order, so these steps need no workgroup barrier).  Each SIMD then holds one
// wave that feeds the matrix pipe and one that keeps the vector pipe busy.  A super-block is two stages of 128
// values; the operand tile of a stage (32 KiB, fragment order) is double buffered and one barrier per stage hands
// it over: while the multipliers work on stage g, the unpackers write stage g + 1.
#include <type_traits>

#include "tgo_device.h"
#include "tgo_forward_args.h"
#include "tgo_launch.h"

namespace tgo {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int FSC_THREADS = 512;
constexpr int FSC_STEPS = 8;                                // 16-value reduction steps per stage
constexpr int FSC_TILE_BYTES = FWD_NT * FSC_STEPS * 1024;   // fp16 operand of a stage: [tile][step][64 lanes][16 bytes]
constexpr int FSC_ROWS = 256;                               // activation rows per task
static_assert(FSC_ROWS == forward_row_tile(12, OPERAND_SCALED), "task rows match the workgroup");
#ifndef FSC_RAW_DEPTH
#define FSC_RAW_DEPTH 3
#endif
#ifndef FSC_TOUCH_AHEAD
#define FSC_TOUCH_AHEAD 4
#endif
#ifndef FSC_W_AHEAD
#define FSC_W_AHEAD 2
#endif
#ifndef FSC_X_AHEAD
#define FSC_X_AHEAD 8
#endif

template <int TYPE>
struct ScaledLds {
    static constexpr bool K45 = TYPE == Q4_K || TYPE == Q5_K;
    // slot of one packed block: Q4_K/Q5_K blocks are whole 16-byte units and lie back to back (16-byte reads of 32
    // consecutive rows then cover all banks); the other formats take the larger of their two staging pitches
    static constexpr int RAW_SLOT = K45 ? Format<TYPE>::BLOCK_BYTES
                                        : (Format<TYPE>::RAW_PITCH > WideStage<TYPE>::PITCH ? Format<TYPE>::RAW_PITCH
                                                                                             : WideStage<TYPE>::PITCH);
    alignas(16) uint8_t wq[2][FSC_TILE_BYTES];                 // operand tiles of two stages
    alignas(16) uint8_t raw[4][2][32 * RAW_SLOT];              // per unpacking wave: packed blocks of two super-blocks
    alignas(16) uint8_t mins[2][K45 ? FWD_NT * 512 : 16];      // fp16(-dmin * m * 2^-S): [tile][32 rows][8 blocks], by parity
    alignas(16) float row_power[FWD_TN];                       // 2^S of the tile's weight rows
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

#ifdef FSC_TIMING
__device__ unsigned long long fsc_times[8][2][96];
// phase accumulators in scalar registers; nothing is stored before the end of the kernel
#define FSC_LAP(slot) do { const unsigned long long now_ = __builtin_readcyclecounter(); lap[slot] += now_ - lap_last; lap_last = now_; } while (0)
#else
#define FSC_LAP(slot) do {} while (0)
#endif

template <int TYPE, bool WIDE>
__global__ __launch_bounds__(FSC_THREADS, 2) void mmq_forward_scaled_kernel(const ForwardArgs a) {
#ifdef FSC_TIMING
    const int profiled_early = blockIdx.x % 1000 == 7 && blockIdx.x / 1000 < 8 ? blockIdx.x / 1000 : -1;
    if (profiled_early >= 0 && threadIdx.x == 0) fsc_times[profiled_early][0][0] = __builtin_readcyclecounter();
    if (profiled_early >= 0 && threadIdx.x == 0) fsc_times[profiled_early][0][93] = wall_clock64();
    if (profiled_early >= 0 && threadIdx.x == 256) fsc_times[profiled_early][1][0] = __builtin_readcyclecounter();
#endif
    using F = Format<TYPE>;
    using L = ScaledLds<TYPE>;
    constexpr bool K45 = L::K45;
    __shared__ L lds;

    int n_tile, expert, row_start, row_end;
    bool second;
    if (!forward_pick(a, n_tile, second, expert, row_start, row_end)) {
        return;
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;
#ifdef FSC_TIMING
    const int profiled = (wave == 0 || wave == 4) ? profiled_early : -1;
    if (profiled >= 0 && tid == 0) { fsc_times[profiled][0][95] = (static_cast<unsigned long long>(row_end - row_start) << 32) | static_cast<unsigned>(n_tile); }
    unsigned long long lap[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    unsigned long long lap_last = __builtin_readcyclecounter();
    if (profiled >= 0 && lane == 0) { fsc_times[profiled][wave >> 2][90] = lap_last; }
#endif

    const uint8_t * weights = (second ? a.packed_second : a.packed) + static_cast<int64_t>(expert) * a.bytes_per_expert;
    uint16_t * const y = second ? a.y_second : a.y;
    const int n0 = n_tile * FWD_TN;
    const int super_blocks = a.in_features / QK_K;
    const int tile_rows = min(FWD_TN, a.out_features - n0);   // weight rows of this tile that exist

    if constexpr (TYPE == IQ2_S) {
        expand_iq2s_selectors(lds.codebook, tid, FSC_THREADS);
        __syncthreads();
    }

    if (wave >= 4) {
        // ---------------- unpacking wave ----------------
        const int dw = wave - 4;
        // rows past the end of the weight matrix repeat its last row (their results are never stored)
        const int first_row = min(32 * dw, tile_rows - 1);
        const int rows_valid = max(1, min(32, tile_rows - 32 * dw));
        const uint8_t * const wave_weights = weights + static_cast<int64_t>(n0 + first_row) * a.row_bytes;
        constexpr int RAW_UNITS = K45 ? F::BLOCK_BYTES / 16 : 1;
        constexpr int RAW_REGS = K45 ? (32 * RAW_UNITS + 63) / 64 : 1;
        using W = WideStage<TYPE>;
        constexpr int WIDE_REGS = WIDE ? W::template regs<32, 64>() : 1;
        constexpr int SLOT_PITCH = K45 ? F::BLOCK_BYTES : (WIDE ? W::PITCH : F::RAW_PITCH);
        constexpr int SLOT_FRONT = K45 ? 0 : (WIDE ? W::FRONT : F::RAW_SHIFT);

        // ---- S of this lane's weight row: the largest weight magnitude over the row's super-blocks goes to [2^8, 2^9)
        const uint8_t * const lane_row_blocks = wave_weights + static_cast<int64_t>(min(l32, rows_valid - 1)) * a.row_bytes;
        float reach = 0.0f;
        for (int kb = half; kb < super_blocks; kb += 2) {
            const uint8_t * blk = lane_row_blocks + static_cast<int64_t>(kb) * F::BLOCK_BYTES;
            if constexpr (K45) {
                const uint32_t pair = *reinterpret_cast<const uint32_t *>(blk);
                reach = fmaxf(reach, fabsf(half_bits_to_float(pair & 0xffffu)) * weight_reach<TYPE>());
                reach = fmaxf(reach, fabsf(half_bits_to_float(pair >> 16)) * 63.0f);
            } else {
                const uint32_t bits = *reinterpret_cast<const uint16_t *>(blk + scale_offset<TYPE>());
                reach = fmaxf(reach, fabsf(half_bits_to_float(bits)) * weight_reach<TYPE>());
            }
        }
        reach = fmaxf(reach, __shfl_xor(reach, 32));
        int reach_exponent = static_cast<int>(__float_as_uint(reach) >> 23);   // biased
        reach_exponent = min(max(reach_exponent, 9), 254);
        const float shrink = __uint_as_float(static_cast<uint32_t>(262 - reach_exponent) << 23);   // 2^-S
        if (half == 0) {
            lds.row_power[32 * dw + l32] = __uint_as_float(static_cast<uint32_t>(reach_exponent - 8) << 23);   // 2^S
        }

        // Packed blocks of FSC_RAW_DEPTH super-blocks are in flight in registers: a lone request per super-block would
        // leave the wave waiting for memory once per super-block.
        struct RawSet {
            u32x4_t units[RAW_REGS];
            WideRegs<WIDE_REGS> wide;
        };
        RawSet ring[FSC_RAW_DEPTH];
        auto request = [&](int kb, RawSet & set) {
            if constexpr (K45) {
                const uint8_t * base = wave_weights + static_cast<int64_t>(kb) * F::BLOCK_BYTES;
#pragma unroll
                for (int i = 0; i < RAW_REGS; ++i) {
                    // ids past the wave's blocks repeat the last unit, so no lane branches around a load
                    const int id = min(lane + 64 * i, 32 * RAW_UNITS - 1);
                    const int row = id / RAW_UNITS;
                    const int unit = id - row * RAW_UNITS;
                    const uint32_t offset = __umul24(min(row, rows_valid - 1), static_cast<uint32_t>(a.row_bytes)) + unit * 16;
                    set.units[i] = *reinterpret_cast<const u32x4_t *>(base + offset);
                }
            } else if constexpr (WIDE) {
                wide_fetch<TYPE, 32, 64, WIDE_REGS>(set.wide, wave_weights, static_cast<int>(a.row_bytes), rows_valid, kb, lane);
            }
        };
        // `kb`: the super-block the registers were requested for; `slot_parity`: where it goes
        auto park = [&](int kb, int slot_parity, const RawSet & set) {
            uint8_t * const slot = lds.raw[dw][slot_parity];
            if constexpr (K45) {
#pragma unroll
                for (int i = 0; i < RAW_REGS; ++i) {
                    const int id = min(lane + 64 * i, 32 * RAW_UNITS - 1);
                    *reinterpret_cast<u32x4_t *>(slot + id * 16) = set.units[i];   // (slots lie back to back: row * BLOCK_BYTES + unit * 16)
                }
            } else if constexpr (WIDE) {
                wide_park<TYPE, 32, 64, WIDE_REGS>(slot, set.wide, wave_weights, static_cast<int>(a.row_bytes), rows_valid, kb, lane);
            } else {
                stage_blocks<TYPE>(slot, weights, a.row_bytes, n0 + 32 * dw, a.out_features, kb, 32, lane, 64);
            }
        };
        // A lane keeps weight row `l32` of the wave's 32 and takes k-half `half` of every 32-value block.
        const uint32_t out_lane = static_cast<uint32_t>(dw * (FSC_STEPS * 1024) + half * 1024 + l32 * 16);
        auto block_of = [&](int kb) { return lds.raw[dw][kb & 1] + l32 * SLOT_PITCH + SLOT_FRONT; };
        // Q4_K/Q5_K: what a stage's unpack reads from the parked block, fetched a phase before it is used (a lone
        // wave has nothing else to cover an LDS round trip with): the 16-byte header (d, dmin, 12 bytes of 6-bit
        // scales and minima), this k-half's fifth-bit bytes, and its 16 bytes of each of the stage's two nibble chunks.
        struct StageInputs {
            u32x4_t header, planes, nibbles[2];
        };
        auto fetch_inputs = [&](int stage_of_block, int kb) {
            constexpr int QS = TYPE == Q4_K ? 16 : 48;
            const uint8_t * blk = block_of(kb);
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
        // the eight block minima of a Q4_K/Q5_K super-block as the operand of its extra reduction step
        auto minima_from_header = [&](int parity, const u32x4_t header) {
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
                *reinterpret_cast<uint4 *>(&lds.mins[parity][dw * 512 + l32 * 16]) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
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
        // the other formats: stage S of super-block kb straight from the parked block
        auto unpack = [&](auto stage_tag, int kb, int target) {
            constexpr int S = decltype(stage_tag)::value;
            if constexpr (!K45) {
                const uint8_t * blk = block_of(kb);
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

        // The multiplying waves request their activation fragments a few reduction steps ahead, which covers a trip to
        // L2 but not one to HBM; this wave therefore touches, FSC_TOUCH_AHEAD stages ahead, one word of every 128-byte
        // line that two of the task's 32-row tiles will need (tiles first + 2 dw and + 2 dw + 1; wave 0 also a ninth
        // one that an unaligned task reaches into), so that the lines wait in L2.  The words are summed into a value
        // that is never used for anything else.
        const int stages = 2 * super_blocks;
        const int first_tile = row_start >> 5;
        const int last_tile = (min(row_end, a.rows_padded) - 1) >> 5;
        const int64_t tile_stride = static_cast<int64_t>(a.in_features / 32) * 2048;
        const uint8_t * const touch_base[3] = {
            reinterpret_cast<const uint8_t *>(a.qx) + min(first_tile + 2 * dw, last_tile) * tile_stride,
            reinterpret_cast<const uint8_t *>(a.qx) + min(first_tile + 2 * dw + 1, last_tile) * tile_stride,
            reinterpret_cast<const uint8_t *>(a.qx) + min(first_tile + 8, last_tile) * tile_stride};
        uint32_t touched[FSC_TOUCH_AHEAD][3];
        uint32_t touch_sink = 0;
        auto touch = [&](int stage_index, uint32_t (&words)[3]) {
            const int64_t offset = static_cast<int64_t>(min(stage_index, stages - 1)) * (FSC_STEPS * 1024) + lane * 128;
            words[0] = *reinterpret_cast<const uint32_t *>(touch_base[0] + offset);
            words[1] = *reinterpret_cast<const uint32_t *>(touch_base[1] + offset);
            words[2] = dw == 0 ? *reinterpret_cast<const uint32_t *>(touch_base[2] + offset) : 0u;
        };
        auto touch_advance = [&](int stage_index) {
            touch_sink += touched[0][0] + touched[0][1] + touched[0][2];
#pragma unroll
            for (int ahead = 0; ahead + 1 < FSC_TOUCH_AHEAD; ++ahead) {
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    touched[ahead][i] = touched[ahead + 1][i];
                }
            }
            touch(stage_index + FSC_TOUCH_AHEAD, touched[FSC_TOUCH_AHEAD - 1]);
        };
#pragma unroll
        for (int ahead = 0; ahead < FSC_TOUCH_AHEAD; ++ahead) {
            touch(1 + ahead, touched[ahead]);
        }
        const int last = super_blocks - 1;
#pragma unroll
        for (int ahead = 0; ahead < FSC_RAW_DEPTH; ++ahead) {
            request(min(ahead, last), ring[ahead]);
        }
        // the oldest set goes to LDS, the others move up, the newest is requested
        auto advance = [&](int parked_kb, int slot_parity, int requested_kb) {
            park(parked_kb, slot_parity, ring[0]);
#pragma unroll
            for (int ahead = 0; ahead + 1 < FSC_RAW_DEPTH; ++ahead) {
                ring[ahead] = ring[ahead + 1];
            }
            request(requested_kb, ring[FSC_RAW_DEPTH - 1]);
        };
        advance(0, 0, min(FSC_RAW_DEPTH, last));
        StageInputs inputs = {};
        if constexpr (K45) {
            inputs = fetch_inputs(0, 0);
            minima_from_header(0, inputs.header);
            finish_stage(std::integral_constant<int, 0>{}, inputs, 0);
            inputs = fetch_inputs(1, 0);
        } else {
            unpack(std::integral_constant<int, 0>{}, 0, 0);
        }
        FSC_LAP(0);
        __syncthreads();
        FSC_LAP(1);
#pragma unroll 1
        for (int kb = 0; kb < super_blocks; ++kb) {
            // (past the last super-block the wave works on a repeat of it: nobody reads what that writes)
            // while the multipliers work on stage 0 of kb: stage 1 of kb, then the next super-block's blocks
#ifndef FSC_NO_UNPACK
            if constexpr (K45) {
                finish_stage(std::integral_constant<int, 1>{}, inputs, 1);
            } else {
                unpack(std::integral_constant<int, 1>{}, kb, 1);
            }
#endif
            FSC_LAP(4);
            advance(min(kb + 1, last), (kb + 1) & 1, min(kb + 1 + FSC_RAW_DEPTH, last));
            FSC_LAP(2);
            touch_advance(2 * kb + 1);
            FSC_LAP(3);
            if constexpr (K45) {
                inputs = fetch_inputs(0, kb + 1);
            }
            __syncthreads();
            FSC_LAP(5);
            // while they work on stage 1: stage 0 of kb + 1
#ifndef FSC_NO_UNPACK
            if constexpr (K45) {
                minima_from_header((kb + 1) & 1, inputs.header);
                finish_stage(std::integral_constant<int, 0>{}, inputs, 0);
                inputs = fetch_inputs(1, kb + 1);
            } else {
                unpack(std::integral_constant<int, 0>{}, kb + 1, 0);
            }
#endif
            FSC_LAP(6);
            touch_advance(2 * kb + 2);
            FSC_LAP(3);
            __syncthreads();
            FSC_LAP(5);
        }
#pragma unroll
        for (int ahead = 0; ahead < FSC_TOUCH_AHEAD; ++ahead) {
            touch_sink += touched[ahead][0] + touched[ahead][1] + touched[ahead][2];
        }
        if (touch_sink == 0x5ca1ab1eu && a.rows < 0) {   // (never true: keeps the touches alive)
            lds.row_power[lane] = 1.0f;
        }
        __syncthreads();
#ifdef FSC_TIMING
        if (profiled >= 0 && lane == 0) { for (int i = 0; i < 8; ++i) fsc_times[profiled][1][i + 1] = lap[i]; }
#endif
        return;
    }

    // ---------------- multiplying wave ----------------
#ifdef FSC_MULT_PRIO
    __builtin_amdgcn_s_setprio(FSC_MULT_PRIO);
#endif
    const int wave_row = row_start + wave * 64;
    const bool wave_active = wave_row < row_end;
    if (!wave_active) {
        __syncthreads();
#pragma unroll 1
        for (int kb = 0; kb < super_blocks; ++kb) {
            __syncthreads();
            __syncthreads();
        }
        __syncthreads();
        return;
    }
    // Every global address is a uniform 64-bit base, advanced with scalar arithmetic, plus a 32-bit lane offset.
    const int blocks_per_row = a.in_features / 32;
    const int total_steps = a.in_features / 16;
    const int first_tile = row_start >> 5;
    const uint8_t * const qx_task = reinterpret_cast<const uint8_t *>(a.qx) + static_cast<int64_t>(first_tile) * blocks_per_row * 2048;
    const uint8_t * const sums_task = reinterpret_cast<const uint8_t *>(a.block_sums) + static_cast<int64_t>(first_tile) * super_blocks * 512;
    uint32_t x_lane_offset[2], sums_lane_offset[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        int lane_row = wave_row + 32 * rt + l32;
        lane_row = lane_row < a.rows_padded ? lane_row : a.rows_padded - 1;
        x_lane_offset[rt] = static_cast<uint32_t>((lane_row >> 5) - first_tile) * blocks_per_row * 2048u +
                            static_cast<uint32_t>(((lane_row & 31) + 32 * half) * 16);
        sums_lane_offset[rt] = static_cast<uint32_t>((lane_row >> 5) - first_tile) * super_blocks * 512u +
                               static_cast<uint32_t>((lane_row & 31) * 16);
    }

    // reduction step G (16 values) of the task's rows: one 1 KiB slab per 32-row tile
    auto load_x = [&](int step, half8_t (&out)[2]) {
#ifdef FSC_X_HOT
        const int clamped = step & 7;
#else
        const int clamped = step < total_steps ? step : total_steps - 1;
#endif
        const uint8_t * base = qx_task + static_cast<int64_t>(clamped) * 1024;
        out[0] = *reinterpret_cast<const half8_t *>(base + x_lane_offset[0]);
        out[1] = *reinterpret_cast<const half8_t *>(base + x_lane_offset[1]);
    };
    auto load_sums = [&](int kb, uint4 (&out)[2]) {
        const int clamped = kb < super_blocks ? kb : super_blocks - 1;
        const uint8_t * base = sums_task + static_cast<int64_t>(clamped) * 512;
        out[0] = *reinterpret_cast<const uint4 *>(base + sums_lane_offset[0]);
        out[1] = *reinterpret_cast<const uint4 *>(base + sums_lane_offset[1]);
    };

    // activation fragments are requested FSC_X_AHEAD reduction steps before their matrix instructions
    half8_t x[FSC_X_AHEAD][2];
#pragma unroll
    for (int i = 0; i < FSC_X_AHEAD; ++i) {
        load_x(i, x[i]);
    }
    uint4 sums[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
    if constexpr (K45) {
        load_sums(0, sums);
    }

    v16f acc[2][FWD_NT];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int nt = 0; nt < FWD_NT; ++nt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rt][nt][v] = 0.0f;

    // weight fragments are read FSC_W_AHEAD reduction steps before their matrix instructions
    constexpr int RING = FSC_W_AHEAD + 1;
    half8_t w[RING][FWD_NT];
    auto read_step = [&](int buffer, int step, half8_t (&out)[FWD_NT]) {
#pragma unroll
        for (int nt = 0; nt < FWD_NT; ++nt) {
            out[nt] = *reinterpret_cast<const half8_t *>(&lds.wq[buffer][((nt * FSC_STEPS + step) * 64 + lane) * 16]);
        }
    };
    static_assert(FSC_STEPS % FSC_X_AHEAD == 0, "a stage starts at slot 0 of the activation ring");
    // one stage: eight reduction steps from operand tile `buffer` (its first FSC_W_AHEAD steps have been read)
    auto stage = [&](int buffer, int first_step) {
#pragma unroll
        for (int s = 0; s < FSC_STEPS; ++s) {
#ifndef FSC_NO_AREAD
            if (s + FSC_W_AHEAD < FSC_STEPS) {
                read_step(buffer, s + FSC_W_AHEAD, w[(s + FSC_W_AHEAD) % RING]);
            }
#endif
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
                for (int nt = 0; nt < FWD_NT; ++nt) {
                    acc[rt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(x[s % FSC_X_AHEAD][rt], w[s % RING][nt], acc[rt][nt], 0, 0, 0);
                }
            }
#ifndef FSC_NO_XLOAD
            load_x(first_step + s + FSC_X_AHEAD, x[s % FSC_X_AHEAD]);
#endif
        }
    };
    auto read_first_steps = [&](int buffer) {
#pragma unroll
        for (int s = 0; s < FSC_W_AHEAD; ++s) {
            read_step(buffer, s, w[s]);
        }
    };
    FSC_LAP(0);
    __syncthreads();
    FSC_LAP(1);
    read_first_steps(0);
#pragma unroll 1
    for (int kb = 0; kb < super_blocks; ++kb) {
        uint4 sums_next[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
        if constexpr (K45) {
            load_sums(kb + 1, sums_next);
        }
        stage(0, kb * 16);
        FSC_LAP(2);
        __syncthreads();
        FSC_LAP(3);
        read_first_steps(1);
        stage(1, kb * 16 + 8);
        if constexpr (K45) {
            // the super-block's extra reduction step: block sums x block minima (slots 8..15 of the instruction are empty)
#pragma unroll
            for (int nt = 0; nt < FWD_NT; ++nt) {
                uint4 minima = *reinterpret_cast<const uint4 *>(&lds.mins[kb & 1][nt * 512 + l32 * 16]);
                if (half != 0) {
                    minima = make_uint4(0, 0, 0, 0);
                }
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) {
                    const uint4 block_sums = half != 0 ? make_uint4(0, 0, 0, 0) : sums[rt];
                    acc[rt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, block_sums),
                                                                         __builtin_bit_cast(half8_t, minima), acc[rt][nt], 0, 0, 0);
                }
            }
            sums[0] = sums_next[0];
            sums[1] = sums_next[1];
        }
        FSC_LAP(4);
        __syncthreads();
        FSC_LAP(3);
        read_first_steps(0);   // of the next super-block (a stale tile after the last one: never used)
    }
    __syncthreads();
    FSC_LAP(6);

    // The operand tiles are free now: each wave scales its results by 2^(E[r] + S[n]), transposes them 32 rows at a
    // time through its share of that memory (rows padded to 136) and writes whole 256-byte rows.
    constexpr int STAGE_PITCH = 136;
    static_assert(sizeof(lds.wq) >= 4 * 32 * STAGE_PITCH * sizeof(uint16_t), "the staging area fits");
    uint16_t * const stage_base = reinterpret_cast<uint16_t *>(&lds.wq[0][0]);
    typedef float float4_unaligned __attribute__((ext_vector_type(4), aligned(4)));
    float column_power[FWD_NT];
#pragma unroll
    for (int nt = 0; nt < FWD_NT; ++nt) {
        column_power[nt] = lds.row_power[nt * 32 + l32];
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        const int r0 = wave_row + 32 * rt;
        if (r0 < row_end) {
            // the lane's rows r0 + 8 j + 4 half + 0..3 (rows past the workspace read on into the plane's successor:
            // their results are never stored)
            const float * powers = a.power + r0 + 4 * half;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float4_unaligned run = *reinterpret_cast<const float4_unaligned *>(powers + 8 * j);
                const float row_power[4] = {run.x, run.y, run.z, run.w};
#pragma unroll
                for (int nt = 0; nt < FWD_NT; ++nt) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[rt][nt][4 * j + i] *= row_power[i] * column_power[nt];
                    }
                }
            }
            const int64_t origin = static_cast<int64_t>(r0) * a.out_features + n0;
            store_rows_32x128<STAGE_PITCH, false, false>(stage_base + wave * (32 * STAGE_PITCH), acc[rt], y + origin, a.out_features,
                                                         row_end - r0, a.out_features - n0, lane, nullptr);
        }
    }
#ifdef FSC_TIMING
    FSC_LAP(7);
    if (profiled >= 0 && lane == 0) { fsc_times[profiled][0][94] = wall_clock64(); for (int i = 0; i < 8; ++i) fsc_times[profiled][0][i + 1] = lap[i]; }
#endif
}

#ifdef FSC_TIMING
extern "C" int tgo_debug_read(void * destination, int bytes) {
    return static_cast<int>(hipMemcpyFromSymbol(destination, HIP_SYMBOL(fsc_times), bytes));
}
#endif

template <int TYPE>
static hipError_t launch_forward_scaled_typed(const ForwardArgs & args, hipStream_t stream) {
    const int64_t total = static_cast<int64_t>(args.n_tiles) * args.projections *
                          (args.task_count != nullptr ? xcd_chunk_slots(args.task_slots) : pad_task_slots(args.task_slots, FWD_XCD_RUN));
    if (total <= 0 || total > 0x7fffffffLL || args.swiglu != 0 || args.in_features > (1 << 22)) {
        return hipErrorInvalidValue;
    }
    const ProfileScope scope(2, stream);
    if constexpr (Format<TYPE>::BLOCK_BYTES % 16 != 0) {
        if (args.wide != 0) {
            mmq_forward_scaled_kernel<TYPE, true><<<static_cast<unsigned>(total), FSC_THREADS, 0, stream>>>(args);
            return hipGetLastError();
        }
    }
    mmq_forward_scaled_kernel<TYPE, false><<<static_cast<unsigned>(total), FSC_THREADS, 0, stream>>>(args);
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
