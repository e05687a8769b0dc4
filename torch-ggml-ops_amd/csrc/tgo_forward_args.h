// What the forward kernel families (int8, exact fp16 and scaled fp16 matrix operands) share: the launch arguments and the
// mapping from a workgroup to its (column tile, projection, row task).
#pragma once

#include "tgo_device.h"
#include "tgo_launch.h"

namespace tgo {

constexpr int FWD_TN = 128;          // weight rows per workgroup
constexpr int FWD_XCD_RUN = 4;       // dense calls: consecutive row tasks that share an XCD (grouped calls: xcd_chunk)
constexpr int FWD_NT = FWD_TN / 32;  // 32-row weight tiles per workgroup

struct ForwardArgs {
    const uint8_t * packed;
    const uint8_t * packed_second;   // second projection of a pair, or nullptr
    int64_t bytes_per_expert;
    int64_t row_bytes;
    const int8_t * qx;               // int8 tiles, or fp16 tiles (Q8Workspace::layout)
    const float * dx;
    const float * sx;
    const float * power;             // scaled tiles only: 2^(e - E) per row and super-block
    const float * row_power;         // scaled tiles only: 2^E per row
    const uint16_t * block_sums;     // scaled tiles only: fp16 block sums, eight per row and super-block
    uint16_t * y;
    uint16_t * y_second;
    const int32_t * task_count;   // nullptr: dense
    const int32_t * task_early;   // tasks listed before those of at most 32 rows
    int32_t * task_cursor;        // zero at launch; counts the short items that workgroups have taken
    const int32_t * task_expert;
    const int32_t * task_row_start;
    const int32_t * task_row_end;
    int rows;
    int rows_padded;
    int in_features;
    int out_features;
    int n_tiles;
    int projections;   // 1, or 2 for a pair: both share the task's activations, so their tiles run side by side
    int swiglu;        // 1: a workgroup runs gate (-> y) then up and stores swiglu(gate, up) -> y_second
    int task_slots;
    int dense_row_tile;   // dense calls: rows per workgroup (the format's row tile, or 32 when that fills the chip better)
    int wide;             // 2-byte aligned formats: the weights may be fetched as aligned 16-byte units (wide_stage_ok)
    int early_only;       // grouped calls: 1 = this launch runs the tasks listed before the short ones, another kernel the rest
};

// The (column tile, projection, task) of this workgroup; false when the slot holds no task.
// `linear`: position in the launch order of workgroups (blockIdx.x for kernels that run one task per workgroup).
TGO_DEVICE bool forward_pick_linear(const ForwardArgs & a, int linear, int & n_tile, bool & second, int & expert,
                                    int & row_start, int & row_end) {
    int task;
    int tasks = a.task_count != nullptr ? a.task_count[0] : (a.rows + a.dense_row_tile - 1) / a.dense_row_tile;
    if (a.task_count != nullptr) {
        const int early = min(a.task_early[0], tasks);
        tasks = a.early_only != 0 ? early : tasks;
        xcd_chunk(linear, a.n_tiles * a.projections, tasks, early, n_tile, task);
    } else {
        xcd_tile<FWD_XCD_RUN>(linear, a.n_tiles * a.projections, tasks, n_tile, task);
    }
    second = n_tile >= a.n_tiles;
    n_tile -= second ? a.n_tiles : 0;
    expert = 0;
    if (a.task_count != nullptr) {
        if (task >= tasks) {
            return false;
        }
        expert = a.task_expert[task];
        row_start = a.task_row_start[task];
        row_end = a.task_row_end[task];
    } else {
        row_start = task * a.dense_row_tile;
        if (row_start >= a.rows) {
            return false;
        }
        row_end = min(a.rows, row_start + a.dense_row_tile);
    }
    return true;
}

TGO_DEVICE bool forward_pick(const ForwardArgs & a, int & n_tile, bool & second, int & expert, int & row_start,
                             int & row_end) {
    return forward_pick_linear(a, blockIdx.x, n_tile, second, expert, row_start, row_end);
}

// Launch of the fp16-operand kernels for arguments prepared by the common launcher (tgo_forward.hip).
hipError_t launch_forward_half(const ForwardArgs & args, int quant_type, hipStream_t stream);
hipError_t launch_forward_scaled(const ForwardArgs & args, int quant_type, hipStream_t stream);

}  // namespace tgo
