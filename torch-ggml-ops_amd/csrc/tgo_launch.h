// Host-side launchers behind the C ABI.  Each returns the hipError_t of its launch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tgo {

// Matrix operands of the MFMA forward kernels, a process-wide setting (tgo_set_forward_operand):
//   OPERAND_INT8    int8 quants on the int8 matrix instruction; every 32-value block result is scaled with two or
//                   three fp32 vector operations (tgo_forward.hip), which bound those kernels.
//   OPERAND_HALF    fp16 numbers holding the same integers exactly; one vector operation per result and block is
//                   left (tgo_forward_half.hip).
//   OPERAND_SCALED  both operands carry their scales: the dequantized q8_1 activation d * q and the dequantized
//                   weight, each normalised by a power of two per row and rounded to fp16 once.  The matrix
//                   instruction then accumulates the whole reduction and no vector instruction touches a result
//                   before the epilogue (tgo_forward_scaled.hip): the only kind whose bound is the matrix pipe.
//   OPERAND_AUTO    (default) scaled operands for calls with enough tasks to fill the chip with its 256-row x
//                   128-column tiles, otherwise exact fp16 for IQ2_S and int8 for the other formats (their smaller
//                   tiles spread a small call over more CUs).
// `quant_type` 0 stands for a workspace that is quantized without knowing the format it will be used with
// (tgo_quantize_q8_1, tgo_mmq_forward_prepared): int8 unless exact fp16 is forced.  The activation workspace is
// written for one kind of operand and records which (Q8Workspace::tag); it must be consumed as that kind.  A call
// reads the setting once, so a change by another thread never splits a call between two kinds.
enum ForwardOperand : int { OPERAND_INT8 = 0, OPERAND_HALF = 1, OPERAND_AUTO = 2, OPERAND_SCALED = 3 };
int forward_operand_setting();
void set_forward_operand_setting(int operand);
// Formats of the scaled-operand kernel (all five).
static constexpr bool scaled_forward_format(int quant_type) {
    return quant_type == 11 || quant_type == 12 || quant_type == 13 || quant_type == 14 || quant_type == 22;
}
// Fewest (256-row x 128-column) tiles for which OPERAND_AUTO picks the scaled kernel: one workgroup per CU runs them,
// so half a chip's worth is where it starts to beat the kernels with smaller tiles (dense 512 x 4096: 64 tiles, a
// tie; 4096 x 2048: 256 tiles, 12 % faster).
constexpr int64_t SCALED_AUTO_MIN_TILES = 128;
// The operand kind a call of this format and size uses under the current setting (never OPERAND_AUTO).  Grouped
// calls pass their total rows: the tiles of a ragged list are at least that many.
static inline int forward_operand_kind(int quant_type, int64_t rows = 0, int64_t out_features = 0, int projections = 1) {
    const int setting = forward_operand_setting();
    const int exact = quant_type == 22 ? OPERAND_HALF : OPERAND_INT8;
    if (setting == OPERAND_SCALED) {
        return scaled_forward_format(quant_type) ? OPERAND_SCALED : exact;
    }
    if (setting == OPERAND_AUTO) {
        const int64_t tiles = ((rows + 255) / 256) * ((out_features + 127) / 128) * projections;
        return scaled_forward_format(quant_type) && tiles >= SCALED_AUTO_MIN_TILES ? OPERAND_SCALED : exact;
    }
    return setting;
}
// Waves per workgroup of the fp16-operand kernels, 32 activation rows each (8: the pipelined variant, measured 5 to
// 11 % faster than the 4-wave one for the formats with 16-value scale groups, and no faster for the others).
static constexpr int half_forward_waves(int quant_type) { return quant_type == 14 || quant_type == 22 ? 8 : 4; }
// Row tile of one forward task; the task list is built for these.  int8 operands: 256 rows for the formats whose
// weights unpack into two int8 planes (Q6_K = 14, IQ2_S = 22), 128 rows for the single-plane ones; exact fp16
// operands: 32 rows per wave of the format's workgroup; scaled operands: 256 (eight multiplying waves of 32 rows).
static constexpr int forward_row_tile(int quant_type, int operand_kind) {
    return operand_kind == OPERAND_SCALED ? 256
           : operand_kind == OPERAND_HALF ? 32 * half_forward_waves(quant_type)
                                          : (quant_type == 14 || quant_type == 22 ? 256 : 128);
}
constexpr int BACKWARD_ROW_TILE = 256;
// Grad-input tasks of at most this many rows (a group's remainder) are listed behind the others and run by a
// kernel variant whose waves split the K columns of the tile instead of its rows.
constexpr int BACKWARD_SHORT_ROWS = 64;
// Decode regime: tasks of at most this many rows go to the bandwidth-oriented GEMV kernel.
constexpr int GEMV_ROW_TILE = 8;
// Dense calls of up to this many rows take it too, GEMV_ROW_TILE rows at a time: the MFMA kernel's 128-row
// column tiles leave most of the chip idle on a matrix of a few thousand rows, and its latency per tile is long.
constexpr int GEMV_DENSE_ROWS = 32;

// Dense grad-input: a workgroup owns 256 rows x 128 columns of the result and walks the whole reduction (N weight
// rows, 64 per step) alone, so a call of a few hundred rows keeps K / 128 workgroups busy and takes as long as one
// of them needs for N / 64 dependent steps.  Such calls cut the reduction into this many ranges, one workgroup each,
// which leave fp32 partial results that a second kernel adds up in a fixed order.  1: no split.
// `role_split`: the format has the role-split kernel (Q4_K, Q5_K), which loses to this scheme only up to 32
// items; the general kernel of the other formats gains from a second workgroup per CU up to 256 items.
static inline int dense_grad_splits(int64_t rows, int64_t out_features, int64_t in_features, bool role_split) {
    const int64_t items = (rows + BACKWARD_ROW_TILE - 1) / BACKWARD_ROW_TILE * (in_features / 128);
    const int64_t steps = (out_features + 63) / 64;
    if (items > (role_split ? 32 : 256)) {
        return 1;
    }
    // about one workgroup per CU for a single row tile, two beyond (measured: with one row tile a second
    // workgroup per CU only lengthens everyone's first loads)
    int64_t splits = (rows <= BACKWARD_ROW_TILE ? 256 : 512) / items;
    splits = splits < steps / 2 ? splits : steps / 2;   // at least two steps each
    splits = splits < 16 ? splits : 16;
    return splits < 2 ? 1 : static_cast<int>(splits);
}
// Q4_K (12) and Q5_K (13) have the role-split kernel.
static inline bool has_role_split(int quant_type) { return quant_type == 12 || quant_type == 13; }
// fp32 scratch of the split reduction for a dense call of this format: the same decision as the launcher's
static inline int64_t dense_grad_partial_bytes(int64_t rows, int64_t out_features, int64_t in_features, int quant_type) {
    const int splits = dense_grad_splits(rows, out_features, in_features, has_role_split(quant_type));
    return splits > 1 ? splits * rows * in_features * 4 : 0;
}

// Forward kernel family for a shape: dense calls with up to GEMV_DENSE_ROWS rows and grouped calls that
// average at most four rows per group are HBM-bound and take the GEMV kernel, everything else the MFMA one.
static inline bool use_gemv(int64_t rows, int64_t groups) {
    return groups <= 0 ? rows <= GEMV_DENSE_ROWS : rows <= 4 * groups;
}

// q8_1 workspace: quantized values, then fp32 scales, then fp32 sums, in one of four layouts over the same bytes.
// The MFMA kernels want 32-row tiles in fragment order: int8, fp16 numbers holding the same integers, or (scaled)
// the dequantized values d * q * 2^-e as fp16 with e chosen per row and super-block; the GEMV family reads a few
// rows along K, for which that order would scatter every 16 bytes into a cache line of their own, so calls that
// take the GEMV family (use_gemv) quantize into plain int8 rows instead.
enum WorkspaceLayout : int { LAYOUT_INT8_TILES = 0, LAYOUT_HALF_TILES = 1, LAYOUT_ROWS = 2, LAYOUT_SCALED_TILES = 3 };
constexpr uint32_t WORKSPACE_TAG_MAGIC = 0x71380000u;   // | layout: first word of the workspace's 1 KiB tail

struct Q8Workspace {
    int8_t * q;     // int8 tiles: [rows_padded/32][K/32][2 halves][32 rows][16 bytes]   rows: [rows][K]
                    // half and scaled tiles: [rows_padded/32][K/32][2 k-halves][2 eighths x 32 rows][8 fp16]
    float * d;      // tiles: [K/32][rows_padded]                                         rows: [rows][K/32]
    float * sum;    // same as d
    float * power;  // scaled tiles: 2^(e - E) per row and super-block, [K/256][rows_padded] (2^e until the second pass)
    uint16_t * block_sums;   // scaled tiles: fp16(sum * 2^-e) per block, [rows_padded/32][K/256][32 rows][8 blocks]
    float * row_power;       // scaled tiles: 2^E per row, [rows_padded]
    uint32_t * tag;          // WORKSPACE_TAG_MAGIC | layout, written by the quantizer
    int64_t rows_padded;
    int layout;
    bool by_rows() const { return layout == LAYOUT_ROWS; }
    bool half_tiles() const { return layout == LAYOUT_HALF_TILES; }
    bool scaled_tiles() const { return layout == LAYOUT_SCALED_TILES; }
    int operand_kind() const {
        return layout == LAYOUT_SCALED_TILES ? OPERAND_SCALED : layout == LAYOUT_HALF_TILES ? OPERAND_HALF : OPERAND_INT8;
    }
};

static inline int64_t pad_rows(int64_t rows) { return (rows + 31) / 32 * 32; }

// (sized for the scaled fp16 tiles whichever layout a call ends up using)
static inline int64_t q8_workspace_bytes(int64_t rows, int64_t in_features) {
    const int64_t padded = pad_rows(rows);
    // the 1 KiB tail lets kernels fetch the scales of a whole 32-row tile with 16-byte loads even when the
    // tile starts at the last row; its first word is the layout tag
    return 2 * padded * in_features + 2 * padded * (in_features / 32) * static_cast<int64_t>(sizeof(float)) +
           padded * (in_features / 256) * (static_cast<int64_t>(sizeof(float)) + 16) +
           padded * static_cast<int64_t>(sizeof(float)) + 1024;
}

// `operand_kind`: OPERAND_INT8, OPERAND_HALF or OPERAND_SCALED (forward_operand_kind); ignored for by_rows.
static inline Q8Workspace q8_workspace_view(void * base, int64_t rows, int64_t in_features, bool by_rows, int operand_kind) {
    Q8Workspace view;
    view.layout = by_rows ? LAYOUT_ROWS
                  : operand_kind == OPERAND_SCALED ? LAYOUT_SCALED_TILES
                  : operand_kind == OPERAND_HALF ? LAYOUT_HALF_TILES : LAYOUT_INT8_TILES;
    view.rows_padded = pad_rows(rows);
    view.q = static_cast<int8_t *>(base);
    view.d = reinterpret_cast<float *>(view.q + 2 * view.rows_padded * in_features);
    view.sum = view.d + view.rows_padded * (in_features / 32);
    view.power = view.sum + view.rows_padded * (in_features / 32);
    view.block_sums = reinterpret_cast<uint16_t *>(view.power + view.rows_padded * (in_features / 256));
    view.row_power = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(view.block_sums) + view.rows_padded * (in_features / 256) * 16);
    view.tag = reinterpret_cast<uint32_t *>(view.row_power + view.rows_padded);
    return view;
}

// Tile tasks of the grouped operators: [count][early][expert x max][row_start x max][row_end x max][cursors].
// `early` is the number of tasks listed before the short ones (TaskBuild::late_rows); count when nothing is short.
// `cursor`: TASK_CURSORS counters, TASK_CURSOR_STRIDE words apart (a cache line each), zero when the list is built: a
// kernel whose workgroups take items of the list in turn counts them there.
constexpr int TASK_CURSORS = 8;
constexpr int TASK_CURSOR_STRIDE = 32;
struct TaskList {
    int32_t * count;
    int32_t * early;
    int32_t * expert;
    int32_t * row_start;
    int32_t * row_end;
    int32_t * cursor;
    int max_tasks;
};

static inline int max_tasks_for(int64_t rows, int64_t groups, int row_tile) {
    return static_cast<int>((rows + row_tile - 1) / row_tile + groups);
}

static inline int64_t task_workspace_bytes(int64_t rows, int64_t groups) {
    // sized for the smallest tile any kernel uses so one buffer fits every path
    return (2 + 3 * static_cast<int64_t>(max_tasks_for(rows, groups, GEMV_ROW_TILE)) + TASK_CURSOR_STRIDE * (TASK_CURSORS + 1)) *
           static_cast<int64_t>(sizeof(int32_t));
}

static inline TaskList task_list_view(void * base, int64_t rows, int64_t groups, int row_tile) {
    TaskList list;
    list.max_tasks = max_tasks_for(rows, groups, row_tile);
    list.count = static_cast<int32_t *>(base);
    list.early = list.count + 1;
    list.expert = list.count + 2;
    list.row_start = list.expert + list.max_tasks;
    list.row_end = list.row_start + list.max_tasks;
    // (the cursors start on a cache line of their own)
    int32_t * const end = list.row_end + list.max_tasks;
    list.cursor = end + (TASK_CURSOR_STRIDE - (end - list.count) % TASK_CURSOR_STRIDE) % TASK_CURSOR_STRIDE;
    return list;
}

// What a kernel needs to build the tile-task list of a grouped call on the side (one of its workgroups does it
// before its own share of the work), so that the list costs neither a launch nor a place in the stream's
// critical path.  tasks.count == nullptr: nothing to build.
struct TaskBuild {
    const int64_t * expert_indices;
    const int32_t * expert_offsets;
    TaskList tasks;
    int num_experts, num_groups, rows, row_tile;
    int late_rows;  // tasks of at most this many rows are listed after all the others; 0: group order throughout
    int late_whole_groups;   // 1: only groups of at most late_rows rows are listed late, not the remainders of larger ones
};

static inline TaskBuild no_task_build() {
    TaskBuild build = {};
    build.tasks.count = nullptr;
    return build;
}

// Optional event bracket around a kernel launch (see tgo_profile_enable in the C ABI).
struct ProfileScope {
    ProfileScope(int kernel, hipStream_t stream);
    ~ProfileScope();
    int kernel;
    hipStream_t stream;
    hipEvent_t start;
    bool active;
};

hipError_t launch_dequant_bf16(const uint8_t * packed, uint16_t * out, int64_t rows, int64_t in_features,
                               int quant_type, hipStream_t stream);
// With `gather` set, workspace row r is quantized from input row gather[r] (rows outside [0, input_rows)
// quantize as zeros), i.e. the token -> expert-sorted-row gather of a MoE layer is folded into the read.
// With `build` set, one workgroup of the launch also writes the tile-task list.
hipError_t launch_quantize_q8_1(const uint16_t * input, const Q8Workspace & ws, int64_t rows,
                                int64_t in_features, hipStream_t stream, const int64_t * gather = nullptr,
                                int64_t input_rows = 0, const TaskBuild * build = nullptr);
// up_then_activated[i] = swiglu(gate[i], up_then_activated[i]) over `count` bf16 values (timed with the forward kernels).
hipError_t launch_swiglu_rows(const uint16_t * gate, const uint16_t * up, uint16_t * activated, int64_t count,
                              hipStream_t stream);   // (`activated` may be `up`)
// The (token, choice) slots of a small batch sorted by expert in one launch (at most 4096 slots and experts).
hipError_t launch_route_small(const int64_t * slot_experts, int slots, int top_k, int num_experts, int64_t * row_index,
                              int64_t * slot_rows, int64_t * expert_indices, int32_t * expert_offsets, hipStream_t stream);
// out[t, :] = sum of rows[order[i], :] over i in [starts[t], starts[t + 1]), in list order (fp32, one rounding).
hipError_t launch_rows_to_tokens(const uint16_t * rows, const int64_t * order, const int64_t * starts, uint16_t * out,
                                 int tokens, int64_t num_rows, int features, hipStream_t stream);
// d_gate, d_up of silu(gate) * up for the cotangent `grad_activated` (and `grad_gate`, a cotangent of the gate output
// itself, or nullptr), elementwise over `count` bf16 values.
hipError_t launch_swiglu_backward_rows(const uint16_t * gate, const uint16_t * up, const uint16_t * grad_activated,
                                       const uint16_t * grad_gate, uint16_t * d_gate, uint16_t * d_up, int64_t count,
                                       hipStream_t stream);
// Turns `count` bf16 outputs into NaN when the workspace's tag is not the layout of `ws` (runs behind the multiply kernel).
hipError_t launch_workspace_guard(const Q8Workspace & ws, uint16_t * out, int64_t count, hipStream_t stream);
hipError_t launch_q8_unpack(const Q8Workspace & ws, int8_t * q, float * d, float * sum, int64_t rows,
                            int64_t in_features, hipStream_t stream);

// out[t, :] = sum_j slot_weights[t, j] * rows[slot_rows[t, j], :] (bf16 rows, fp32 accumulation in choice order,
// one rounding); a slot whose row is outside [0, num_rows) contributes nothing.  `features` is a multiple of 8.
hipError_t launch_moe_combine(const uint16_t * rows, const int64_t * slot_rows, const float * slot_weights,
                              uint16_t * out, int tokens, int top_k, int64_t num_rows, int features,
                              hipStream_t stream);
// Dense when tasks == nullptr (row tiles follow from `rows`), grouped otherwise.  With `packed_second` and
// `output_second` set, one launch computes both projections of a pair from the same activation workspace.
hipError_t launch_mmq_forward(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                              const Q8Workspace & ws, uint16_t * output, uint16_t * output_second,
                              const TaskList * tasks, int rows, int in_features, int out_features,
                              int quant_type, hipStream_t stream);
// Pair only: `output` receives the first projection (gate) and `output_second` silu(gate) * second projection,
// both factors rounded to bf16 first, the product rounded once.
hipError_t launch_mmq_forward_swiglu(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                                     const Q8Workspace & ws, uint16_t * output, uint16_t * output_second,
                                     const TaskList * tasks, int rows, int in_features, int out_features,
                                     int quant_type, hipStream_t stream);
hipError_t launch_mmq_gemv(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                           const Q8Workspace & ws, uint16_t * output, uint16_t * output_second,
                           const TaskList * tasks, int rows, int in_features, int out_features,
                           int quant_type, hipStream_t stream);
// The same from bf16 activations in one launch: every workgroup quantizes its task's rows itself and, for a grouped
// call (`expert_offsets` set), finds its task in the group list, so neither a quantizer launch nor a task list
// exists.  Formats whose decode-regime routines read their activations one 16-value unit per lane.
// `gather` (or nullptr): row r of the call is row gather[r] of `input`, which has `input_rows` rows.
// The quantization is repeated by every workgroup that shares a task's rows (one per 16 weight rows), which costs a
// workgroup about as much as its dot products once a task has eight rows; it pays while the call is bound by its
// launches and their latencies: dense calls of one task, grouped calls of at most 64 rows (measured on a 256-expert
// layer: 1 token x top-8 32 -> 20 us of kernel time, 8 tokens 52 -> 48 us, 256 rows with 200 in one group 68 -> 101 us).
// Every workgroup of a fused grouped call reads the whole group list to find its task, so a list far longer than any
// expert count in use (GEMV_FUSED_GROUPS) keeps the task list that one workgroup builds for all.
constexpr int GEMV_FUSED_GROUPED_ROWS = 64;
constexpr int GEMV_FUSED_GROUPS = 1024;
static inline bool gemv_fuses(int quant_type, int64_t rows, int64_t groups) {
    const bool format = quant_type == 11 || quant_type == 14 || quant_type == 22;   // Q3_K, Q6_K, IQ2_S
    return format && use_gemv(rows, groups) && groups <= GEMV_FUSED_GROUPS &&
           rows <= (groups <= 0 ? GEMV_ROW_TILE : GEMV_FUSED_GROUPED_ROWS);
}
hipError_t launch_mmq_gemv_fused(const uint8_t * packed, const uint8_t * packed_second, int64_t bytes_per_expert,
                                 const uint16_t * input, const int64_t * gather, int64_t input_rows,
                                 const int64_t * expert_indices, const int32_t * expert_offsets, int num_experts,
                                 int num_groups, uint16_t * output, uint16_t * output_second, int rows, int in_features,
                                 int out_features, int quant_type, hipStream_t stream);
// Cotangent in MFMA fragment order: [rows_padded/32][chunks] slabs of 1 KiB (32 rows x 16 columns), zero
// padded; the column count is rounded up to 64 so that kernels can walk it four chunks at a time.
static inline int cotangent_chunks(int64_t out_features) { return static_cast<int>((out_features + 63) / 64 * 4); }
static inline int64_t cotangent_workspace_bytes(int64_t rows, int64_t out_features) {
    return pad_rows(rows) / 32 * cotangent_chunks(out_features) * 1024;
}
// One launch packs one cotangent or both of a pair (`grad_second`/`packed_second` null or set together) and, with
// `build` set, writes the tile-task list on the side.  With `gather` set (single cotangent), packed row r is
// bf16(scale[r] * grad[gather[r], :]) with `grad` holding `gather_rows` rows; an index outside them gives zeros.
hipError_t launch_pack_cotangent(const uint16_t * grad, const uint16_t * grad_second, uint8_t * packed,
                                 uint8_t * packed_second, int rows, int out_features, hipStream_t stream,
                                 const TaskBuild * build = nullptr, const int64_t * gather = nullptr,
                                 const float * scale = nullptr, int64_t gather_rows = 0);
// `cotangent_*` are buffers written by launch_pack_cotangent.
// `partial` (dense calls): dense_grad_partial_bytes() of scratch for the split reduction, or nullptr.
hipError_t launch_mmq_grad_input(const uint8_t * cotangent_first, const uint8_t * cotangent_second,
                                 const uint8_t * packed_first, const uint8_t * packed_second,
                                 int64_t bytes_per_expert, uint16_t * grad_input, const TaskList * tasks,
                                 int rows, int out_features, int in_features, int quant_type,
                                 hipStream_t stream, float * partial = nullptr);

}  // namespace tgo
