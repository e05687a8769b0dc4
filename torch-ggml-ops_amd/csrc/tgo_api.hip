// C ABI of libtgo_hip.so (declared in include/tgo.h): argument checks, workspace carving and
// kernel dispatch.  Nothing here allocates or synchronises.
#include "../../include/tgo.h"

#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <utility>
#include <vector>

#include "tgo_device.h"
#include "tgo_launch.h"

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char * format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(g_error, sizeof(g_error), format, args);
    va_end(args);
    return code;
}

int check_hip(hipError_t status, const char * what) {
    if (status == hipSuccess) {
        return TGO_OK;
    }
    return fail(TGO_ERR_HIP, "%s failed: %s", what, hipGetErrorString(status));
}

bool aligned16(const void * pointer) {
    return (reinterpret_cast<uintptr_t>(pointer) & 15u) == 0;
}

constexpr int64_t INT_LIMIT = 0x7fffffffLL;

// Shape rules shared by every matmul entry point (reference: csrc/mmq_hip.cu:599-631, :360-396).
int check_matmul_shape(int64_t rows, int64_t in_features, int64_t out_features, int quant_type) {
    if (tgo::block_bytes(quant_type) == 0) {
        return fail(TGO_ERR_INVALID, "unsupported quant_type: %d", quant_type);
    }
    if (rows <= 0) {
        return fail(TGO_ERR_INVALID, "zero-row inputs are not supported");
    }
    if (in_features <= 0 || in_features % tgo::QK_K != 0) {
        return fail(TGO_ERR_INVALID, "in_features must be a positive multiple of 256; got %lld",
                    static_cast<long long>(in_features));
    }
    if (out_features <= 0) {
        return fail(TGO_ERR_INVALID, "out_features must be positive; got %lld", static_cast<long long>(out_features));
    }
    if (rows > INT_LIMIT || in_features > INT_LIMIT || out_features > INT_LIMIT) {
        return fail(TGO_ERR_INVALID, "a dimension exceeds the kernel limit of 2^31-1");
    }
    if (in_features >= (1 << 24)) {
        return fail(TGO_ERR_INVALID, "in_features exceeds the kernel limit of 2^24-1");
    }
    return TGO_OK;
}

int check_pointer(const void * pointer, const char * name) {
    if (pointer == nullptr) {
        return fail(TGO_ERR_INVALID, "%s must not be null", name);
    }
    if (!aligned16(pointer)) {
        return fail(TGO_ERR_INVALID, "%s data pointer must be 16-byte aligned", name);
    }
    return TGO_OK;
}

int check_grouped(int64_t num_experts, int64_t num_groups, const void * indices, const void * offsets) {
    if (num_experts <= 0) {
        return fail(TGO_ERR_INVALID, "packed_weight must contain at least one expert");
    }
    if (num_groups <= 0) {
        return fail(TGO_ERR_INVALID, "grouped MMQ requires at least one active expert");
    }
    if (num_groups > num_experts) {
        return fail(TGO_ERR_INVALID, "active expert count exceeds packed expert count");
    }
    if (num_experts > INT_LIMIT) {
        return fail(TGO_ERR_INVALID, "expert count exceeds the kernel limit");
    }
    if (indices == nullptr || offsets == nullptr) {
        return fail(TGO_ERR_INVALID, "expert_indices and expert_offsets must not be null");
    }
    return TGO_OK;
}

// Activation workspace of tgo_mmq_forward_static: one array per GPU, part of the loaded code object, so the
// entry point needs no allocation.  In host code the name is only a handle for hipGetSymbolAddress; kernels
// and copies get the per-device address looked up below.
constexpr int64_t STATIC_SCRATCH_BYTES = TGO_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) uint8_t scratch[STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void * g_scratch_address[MAX_DEVICES] = {};

// Address of `scratch` on the current device, looked up once per device (with that device current).
int static_scratch(void ** address) {
    int device = -1;
    const hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess) {
        return fail(TGO_ERR_HIP, "hipGetDevice failed: %s", hipGetErrorString(status));
    }
    if (device < 0 || device >= MAX_DEVICES) {
        return fail(TGO_ERR_INVALID, "device ordinal %d is outside the table of static workspaces", device);
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_address[device] == nullptr) {
        void * found = nullptr;
        const hipError_t lookup = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
        if (lookup != hipSuccess || found == nullptr) {
            return fail(TGO_ERR_HIP, "hipGetSymbolAddress(static workspace) failed: %s", hipGetErrorString(lookup));
        }
        g_scratch_address[device] = found;
    }
    *address = g_scratch_address[device];
    return TGO_OK;
}

// Opt-in launch timing.  The lists are shared by every thread that launches; the mutex guards them, and a list
// stops growing at PROFILE_EVENT_LIMIT brackets (later launches go untimed until the next tgo_profile_enable).
bool g_profile = false;
std::mutex g_profile_mutex;
constexpr size_t PROFILE_EVENT_LIMIT = 1 << 16;
std::vector<std::pair<hipEvent_t, hipEvent_t>> g_profile_events[TGO_KERNEL_COUNT];

void drop_profile_events() {
    for (auto & list : g_profile_events) {
        for (auto & pair : list) {
            (void)hipEventDestroy(pair.first);
            (void)hipEventDestroy(pair.second);
        }
        list.clear();
    }
}

#define TGO_TRY(expression)            \
    do {                               \
        const int status_ = (expression); \
        if (status_ != TGO_OK) {       \
            return status_;            \
        }                              \
    } while (0)

}  // namespace

namespace tgo {

ProfileScope::ProfileScope(int kernel_id, hipStream_t launch_stream)
    : kernel(kernel_id), stream(launch_stream), start(nullptr), active(false) {
    if (!g_profile) {
        return;
    }
    {
        std::lock_guard<std::mutex> lock(g_profile_mutex);
        if (g_profile_events[kernel].size() >= PROFILE_EVENT_LIMIT) {
            return;
        }
    }
    if (hipEventCreate(&start) == hipSuccess) {
        active = hipEventRecord(start, stream) == hipSuccess;
        if (!active) {
            (void)hipEventDestroy(start);
        }
    }
}

ProfileScope::~ProfileScope() {
    if (!active) {
        return;
    }
    hipEvent_t stop = nullptr;
    if (hipEventCreate(&stop) == hipSuccess && hipEventRecord(stop, stream) == hipSuccess) {
        std::lock_guard<std::mutex> lock(g_profile_mutex);
        g_profile_events[kernel].emplace_back(start, stop);
    } else {
        (void)hipEventDestroy(start);
        if (stop != nullptr) {
            (void)hipEventDestroy(stop);
        }
    }
}

}  // namespace tgo

extern "C" {

int tgo_version(void) { return 112; }

int tgo_profile_enable(int enabled) {
    std::lock_guard<std::mutex> lock(g_profile_mutex);
    drop_profile_events();
    g_profile = enabled != 0;
    return TGO_OK;
}

int tgo_set_forward_operand(int operand) {
    if (operand != TGO_OPERAND_INT8 && operand != TGO_OPERAND_HALF && operand != TGO_OPERAND_AUTO &&
        operand != TGO_OPERAND_SCALED) {
        return fail(TGO_ERR_INVALID,
                    "operand must be TGO_OPERAND_INT8, TGO_OPERAND_HALF, TGO_OPERAND_SCALED or TGO_OPERAND_AUTO; got %d", operand);
    }
    tgo::set_forward_operand_setting(operand);
    return TGO_OK;
}

int tgo_forward_operand(void) { return tgo::forward_operand_setting(); }

int tgo_forward_operand_for(int quant_type, int64_t rows, int64_t out_features, int projections) {
    return tgo::forward_operand_kind(quant_type, rows, out_features, projections);
}

int tgo_profile_read(int kernel, double * total_ms, int64_t * launches) {
    if (kernel < 0 || kernel >= TGO_KERNEL_COUNT || total_ms == nullptr || launches == nullptr) {
        return fail(TGO_ERR_INVALID, "bad profile query");
    }
    double total = 0.0;
    std::lock_guard<std::mutex> lock(g_profile_mutex);
    for (auto & pair : g_profile_events[kernel]) {
        TGO_TRY(check_hip(hipEventSynchronize(pair.second), "hipEventSynchronize"));
        float ms = 0.0f;
        TGO_TRY(check_hip(hipEventElapsedTime(&ms, pair.first, pair.second), "hipEventElapsedTime"));
        total += ms;
    }
    *total_ms = total;
    *launches = static_cast<int64_t>(g_profile_events[kernel].size());
    return TGO_OK;
}

const char * tgo_last_error(void) { return g_error; }

int tgo_block_bytes(int quant_type) { return tgo::block_bytes(quant_type); }

int64_t tgo_q8_workspace_bytes(int64_t rows, int64_t in_features) {
    if (rows <= 0 || in_features <= 0) {
        return 0;
    }
    return tgo::q8_workspace_bytes(rows, in_features);
}

int64_t tgo_task_workspace_bytes(int64_t rows, int64_t num_groups) {
    if (rows <= 0 || num_groups <= 0) {
        return 0;
    }
    // keep the next region 16-byte aligned when a caller packs buffers back to back
    return (tgo::task_workspace_bytes(rows, num_groups) + 15) / 16 * 16;
}

int64_t tgo_dense_grad_workspace_bytes(int64_t rows, int64_t out_features, int64_t in_features, int quant_type) {
    if (rows <= 0 || out_features <= 0 || in_features <= 0 || in_features % tgo::QK_K != 0 ||
        tgo::block_bytes(quant_type) == 0) {
        return -1;
    }
    return (tgo::cotangent_workspace_bytes(rows, out_features) + 15) / 16 * 16 +
           tgo::dense_grad_partial_bytes(rows, out_features, in_features, quant_type);
}

int64_t tgo_grad_workspace_bytes(int64_t rows, int64_t out_features, int64_t num_groups, int sources) {
    if (rows <= 0 || out_features <= 0 || sources < 1 || sources > 2) {
        return 0;
    }
    const int64_t tasks = num_groups > 0 ? tgo_task_workspace_bytes(rows, num_groups) : 0;
    return tasks + sources * tgo::cotangent_workspace_bytes(rows, out_features);
}

const char * tgo_forward_kernel_family(int64_t rows, int64_t num_groups) {
    return tgo::use_gemv(rows, num_groups) ? "gemv" : "mfma";
}

int tgo_dequant_bf16(const void * packed, void * out_bf16, int64_t rows, int64_t in_features,
                     int quant_type, void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, 1, quant_type));
    TGO_TRY(check_pointer(packed, "packed_weight"));
    TGO_TRY(check_pointer(out_bf16, "output"));
    return check_hip(tgo::launch_dequant_bf16(static_cast<const uint8_t *>(packed), static_cast<uint16_t *>(out_bf16),
                                              rows, in_features, quant_type, static_cast<hipStream_t>(stream)),
                     "dequant_bf16 launch");
}

static int check_workspace_operand(int operand) {
    if (operand != TGO_OPERAND_INT8 && operand != TGO_OPERAND_HALF && operand != TGO_OPERAND_SCALED) {
        return fail(TGO_ERR_INVALID,
                    "a workspace holds TGO_OPERAND_INT8, TGO_OPERAND_HALF or TGO_OPERAND_SCALED operands; got %d", operand);
    }
    return TGO_OK;
}

int tgo_quantize_q8_1_as(const void * input_bf16, void * workspace, int64_t rows, int64_t in_features, int operand,
                         void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, 1, TGO_TYPE_Q4_K));
    TGO_TRY(check_pointer(input_bf16, "input"));
    TGO_TRY(check_pointer(workspace, "workspace"));
    TGO_TRY(check_workspace_operand(operand));
    const tgo::Q8Workspace view = tgo::q8_workspace_view(workspace, rows, in_features, tgo::use_gemv(rows, 0), operand);
    return check_hip(tgo::launch_quantize_q8_1(static_cast<const uint16_t *>(input_bf16), view, rows, in_features,
                                               static_cast<hipStream_t>(stream)),
                     "quantize_q8_1 launch");
}

int tgo_quantize_q8_1(const void * input_bf16, void * workspace, int64_t rows, int64_t in_features,
                      void * stream) {
    return tgo_quantize_q8_1_as(input_bf16, workspace, rows, in_features, tgo::forward_operand_kind(0), stream);
}

int tgo_q8_workspace_unpack(const void * workspace, void * q_int8, void * d_f32, void * sum_f32,
                            int64_t rows, int64_t in_features, void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, 1, TGO_TYPE_Q4_K));
    TGO_TRY(check_pointer(workspace, "workspace"));
    if (q_int8 == nullptr || d_f32 == nullptr || sum_f32 == nullptr) {
        return fail(TGO_ERR_INVALID, "output pointers must not be null");
    }
    const tgo::Q8Workspace view =
        tgo::q8_workspace_view(const_cast<void *>(workspace), rows, in_features, tgo::use_gemv(rows, 0), tgo::forward_operand_kind(0));
    return check_hip(tgo::launch_q8_unpack(view, static_cast<int8_t *>(q_int8), static_cast<float *>(d_f32),
                                           static_cast<float *>(sum_f32), rows, in_features,
                                           static_cast<hipStream_t>(stream)),
                     "q8_unpack launch");
}

int tgo_mmq_forward(const void * input_bf16, const void * packed, void * output_bf16, void * workspace,
                    int64_t rows, int64_t in_features, int64_t out_features, int quant_type, void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, out_features, quant_type));
    TGO_TRY(check_pointer(input_bf16, "input"));
    TGO_TRY(check_pointer(packed, "packed_weight"));
    TGO_TRY(check_pointer(output_bf16, "output"));
    TGO_TRY(check_pointer(workspace, "workspace"));
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    if (tgo::gemv_fuses(quant_type, rows, 0)) {
        // one launch: the decode-regime kernels of these formats quantize their activations themselves
        return check_hip(tgo::launch_mmq_gemv_fused(static_cast<const uint8_t *>(packed), nullptr, 0,
                                                    static_cast<const uint16_t *>(input_bf16), nullptr, rows, nullptr,
                                                    nullptr, 0, 0, static_cast<uint16_t *>(output_bf16), nullptr,
                                                    static_cast<int>(rows), static_cast<int>(in_features),
                                                    static_cast<int>(out_features), quant_type, hip_stream),
                         "mmq_forward launch");
    }
    const tgo::Q8Workspace view = tgo::q8_workspace_view(workspace, rows, in_features, tgo::use_gemv(rows, 0),
                                                         tgo::forward_operand_kind(quant_type, rows, out_features, 1));
    TGO_TRY(check_hip(tgo::launch_quantize_q8_1(static_cast<const uint16_t *>(input_bf16), view, rows, in_features,
                                                hip_stream),
                      "quantize_q8_1 launch"));
    const auto launch = tgo::use_gemv(rows, 0) ? tgo::launch_mmq_gemv : tgo::launch_mmq_forward;
    return check_hip(launch(static_cast<const uint8_t *>(packed), nullptr, 0, view,
                            static_cast<uint16_t *>(output_bf16), nullptr, nullptr, static_cast<int>(rows),
                            static_cast<int>(in_features),
                            static_cast<int>(out_features), quant_type, hip_stream),
                     "mmq_forward launch");
}

int tgo_mmq_forward_static(const void * input_bf16, const void * packed, void * output_bf16, int64_t rows,
                           int64_t in_features, int64_t out_features, int quant_type, void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, out_features, quant_type));
    const int64_t needed = tgo::q8_workspace_bytes(rows, in_features);
    if (needed > STATIC_SCRATCH_BYTES) {
        return fail(TGO_ERR_INVALID,
                    "rows x in_features = %lld x %lld needs %lld bytes of activation workspace; the static workspace "
                    "holds %lld (use tgo_mmq_forward with a caller-provided workspace)",
                    static_cast<long long>(rows), static_cast<long long>(in_features), static_cast<long long>(needed),
                    static_cast<long long>(STATIC_SCRATCH_BYTES));
    }
    void * workspace = nullptr;
    TGO_TRY(static_scratch(&workspace));
    // every byte of the workspace that the multiply kernels read is rewritten by the quantizer of the same
    // call (padding rows included), so nothing carries over from the previous call
    return tgo_mmq_forward(input_bf16, packed, output_bf16, workspace, rows, in_features, out_features, quant_type,
                           stream);
}

int tgo_mmq_forward_prepared_as(const void * workspace, const void * packed, void * output_bf16, int64_t rows,
                                int64_t in_features, int64_t out_features, int quant_type, int operand, void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, out_features, quant_type));
    TGO_TRY(check_pointer(workspace, "workspace"));
    TGO_TRY(check_pointer(packed, "packed_weight"));
    TGO_TRY(check_pointer(output_bf16, "output"));
    TGO_TRY(check_workspace_operand(operand));
    const tgo::Q8Workspace view =
        tgo::q8_workspace_view(const_cast<void *>(workspace), rows, in_features, tgo::use_gemv(rows, 0), operand);
    const auto launch = tgo::use_gemv(rows, 0) ? tgo::launch_mmq_gemv : tgo::launch_mmq_forward;
    TGO_TRY(check_hip(launch(static_cast<const uint8_t *>(packed), nullptr, 0, view,
                             static_cast<uint16_t *>(output_bf16), nullptr, nullptr, static_cast<int>(rows),
                             static_cast<int>(in_features), static_cast<int>(out_features), quant_type,
                             static_cast<hipStream_t>(stream)),
                      "mmq_forward_prepared launch"));
    // (the workspace was quantized by an earlier call: were it of another kind than this call was told, its layout
    // would not be the one this launch assumed)
    return check_hip(tgo::launch_workspace_guard(view, static_cast<uint16_t *>(output_bf16), rows * out_features,
                                                 static_cast<hipStream_t>(stream)),
                     "workspace guard launch");
}

int tgo_mmq_forward_prepared(const void * workspace, const void * packed, void * output_bf16, int64_t rows,
                             int64_t in_features, int64_t out_features, int quant_type, void * stream) {
    return tgo_mmq_forward_prepared_as(workspace, packed, output_bf16, rows, in_features, out_features, quant_type,
                                       tgo::forward_operand_kind(0), stream);
}

int tgo_mmq_grad_input(const void * grad_output_bf16, const void * packed, void * grad_input_bf16,
                       void * workspace, int64_t rows, int64_t out_features, int64_t in_features,
                       int quant_type, void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, out_features, quant_type));
    TGO_TRY(check_pointer(grad_output_bf16, "grad_output"));
    TGO_TRY(check_pointer(packed, "packed_weight"));
    TGO_TRY(check_pointer(grad_input_bf16, "grad_input"));
    TGO_TRY(check_pointer(workspace, "workspace"));
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    uint8_t * cotangent = static_cast<uint8_t *>(workspace);
    TGO_TRY(check_hip(tgo::launch_pack_cotangent(static_cast<const uint16_t *>(grad_output_bf16), nullptr, cotangent,
                                                 nullptr, static_cast<int>(rows), static_cast<int>(out_features),
                                                 hip_stream),
                      "pack_cotangent launch"));
    // scratch for the split reduction of small calls follows the packed cotangent
    float * partial = tgo::dense_grad_partial_bytes(rows, out_features, in_features, quant_type) > 0
        ? reinterpret_cast<float *>(cotangent + (tgo::cotangent_workspace_bytes(rows, out_features) + 15) / 16 * 16)
        : nullptr;
    return check_hip(tgo::launch_mmq_grad_input(cotangent, nullptr, static_cast<const uint8_t *>(packed), nullptr, 0,
                                                static_cast<uint16_t *>(grad_input_bf16), nullptr,
                                                static_cast<int>(rows), static_cast<int>(out_features),
                                                static_cast<int>(in_features), quant_type, hip_stream, partial),
                     "mmq_grad_input launch");
}

// Shared body of the grouped forward entry points; `row_index` is null for pre-sorted rows.
static int grouped_forward(const void * input_bf16, const int64_t * row_index, int64_t input_rows,
                           const void * packed_first, const void * packed_second, void * output_first,
                           void * output_second, const int64_t * expert_indices, const int32_t * expert_offsets,
                           void * workspace, int64_t rows, int64_t in_features, int64_t out_features,
                           int64_t num_experts, int64_t num_groups, int quant_type, void * stream,
                           bool swiglu = false) {
    TGO_TRY(check_matmul_shape(rows, in_features, out_features, quant_type));
    TGO_TRY(check_grouped(num_experts, num_groups, expert_indices, expert_offsets));
    TGO_TRY(check_pointer(input_bf16, "input"));
    TGO_TRY(check_pointer(packed_first, "packed_weight"));
    TGO_TRY(check_pointer(output_first, "output"));
    TGO_TRY(check_pointer(workspace, "workspace"));
    if ((packed_second == nullptr) != (output_second == nullptr)) {
        return fail(TGO_ERR_INVALID, "second packed_weight and second output must be given together");
    }
    if (packed_second != nullptr) {
        TGO_TRY(check_pointer(packed_second, "second packed_weight"));
        TGO_TRY(check_pointer(output_second, "second output"));
    }
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    const int64_t bytes_per_expert = out_features * (in_features / tgo::QK_K) * tgo::block_bytes(quant_type);
    // SwiGLU: the int8 and exact-fp16 matrix-core kernels have the fused epilogue; after the decode-regime kernels and
    // the scaled-operand kernel, which store both projections (the up projection where the result goes), an
    // elementwise pass finishes -- for calls of decode size that costs far less than leaving their kernel family
    const auto finish_swiglu = [&]() {
        return check_hip(tgo::launch_swiglu_rows(static_cast<const uint16_t *>(output_first),
                                                 static_cast<const uint16_t *>(output_second),
                                                 static_cast<uint16_t *>(output_second), rows * out_features, hip_stream),
                         "swiglu launch");
    };
    const bool gemv = tgo::use_gemv(rows, num_groups);
    if (gemv && tgo::gemv_fuses(quant_type, rows, num_groups)) {
        // one launch: the decode-regime kernels of these formats quantize their activations and find their tasks
        // themselves
        TGO_TRY(check_hip(tgo::launch_mmq_gemv_fused(
                             static_cast<const uint8_t *>(packed_first), static_cast<const uint8_t *>(packed_second),
                             bytes_per_expert, static_cast<const uint16_t *>(input_bf16), row_index,
                             row_index != nullptr ? input_rows : rows, expert_indices, expert_offsets,
                             static_cast<int>(num_experts), static_cast<int>(num_groups),
                             static_cast<uint16_t *>(output_first), static_cast<uint16_t *>(output_second),
                             static_cast<int>(rows), static_cast<int>(in_features), static_cast<int>(out_features),
                             quant_type, hip_stream),
                         "grouped mmq_forward launch"));
        return swiglu ? finish_swiglu() : TGO_OK;
    }
    const int operand_kind = tgo::forward_operand_kind(quant_type, rows, out_features, packed_second != nullptr ? 2 : 1);
    // (the scaled-operand kernel without the epilogue plus the elementwise pass costs less than the other kinds'
    // kernels lose to it)
    const bool fused = swiglu && !gemv && operand_kind != tgo::OPERAND_SCALED;
    const tgo::Q8Workspace view = tgo::q8_workspace_view(workspace, rows, in_features, gemv, operand_kind);
    void * task_base = static_cast<char *>(workspace) + (tgo::q8_workspace_bytes(rows, in_features) + 15) / 16 * 16;
    const int row_tile = gemv ? tgo::GEMV_ROW_TILE : tgo::forward_row_tile(quant_type, view.operand_kind());
    const auto launch = fused ? tgo::launch_mmq_forward_swiglu : gemv ? tgo::launch_mmq_gemv : tgo::launch_mmq_forward;
    const tgo::TaskList tasks = tgo::task_list_view(task_base, rows, num_groups, row_tile);

    // the quantizer writes the tile-task list on the side; the MFMA kernel runs a task of at most 32 rows in
    // about a third of a full task's time, so the groups of that size are listed last and fill the grid's tail
    // (a larger group's remainder stays with the group: its weights are in that XCD's L2 already)
    const tgo::TaskBuild build = {expert_indices, expert_offsets, tasks, static_cast<int>(num_experts),
                                  static_cast<int>(num_groups), static_cast<int>(rows), row_tile, gemv ? 0 : 32, 1};
    TGO_TRY(check_hip(tgo::launch_quantize_q8_1(static_cast<const uint16_t *>(input_bf16), view, rows, in_features,
                                                hip_stream, row_index, input_rows, &build),
                      "quantize_q8_1 launch"));
    // a pair is one launch: both projections of a task run side by side and share its activations in L2
    TGO_TRY(check_hip(launch(static_cast<const uint8_t *>(packed_first), static_cast<const uint8_t *>(packed_second),
                             bytes_per_expert, view, static_cast<uint16_t *>(output_first),
                             static_cast<uint16_t *>(output_second), &tasks, static_cast<int>(rows),
                             static_cast<int>(in_features), static_cast<int>(out_features), quant_type, hip_stream),
                      "grouped mmq_forward launch"));
    return swiglu && !fused ? finish_swiglu() : TGO_OK;
}

int tgo_grouped_mmq_forward(const void * input_bf16, const void * packed_first, const void * packed_second,
                            void * output_first, void * output_second, const int64_t * expert_indices,
                            const int32_t * expert_offsets, void * workspace, int64_t rows,
                            int64_t in_features, int64_t out_features, int64_t num_experts,
                            int64_t num_groups, int quant_type, void * stream) {
    return grouped_forward(input_bf16, nullptr, 0, packed_first, packed_second, output_first, output_second,
                           expert_indices, expert_offsets, workspace, rows, in_features, out_features, num_experts,
                           num_groups, quant_type, stream);
}

int tgo_grouped_mmq_forward_gathered(const void * input_bf16, const int64_t * row_index, int64_t input_rows,
                                     const void * packed_first, const void * packed_second, void * output_first,
                                     void * output_second, const int64_t * expert_indices,
                                     const int32_t * expert_offsets, void * workspace, int64_t rows,
                                     int64_t in_features, int64_t out_features, int64_t num_experts,
                                     int64_t num_groups, int quant_type, void * stream) {
    if (row_index == nullptr) {
        return fail(TGO_ERR_INVALID, "row_index must not be null");
    }
    if (input_rows <= 0) {
        return fail(TGO_ERR_INVALID, "input_rows must be positive; got %lld", static_cast<long long>(input_rows));
    }
    return grouped_forward(input_bf16, row_index, input_rows, packed_first, packed_second, output_first,
                           output_second, expert_indices, expert_offsets, workspace, rows, in_features, out_features,
                           num_experts, num_groups, quant_type, stream);
}

int tgo_grouped_mmq_swiglu(const void * input_bf16, const int64_t * row_index, int64_t input_rows,
                           const void * packed_gate, const void * packed_up, void * output_gate,
                           void * output_activated, const int64_t * expert_indices, const int32_t * expert_offsets,
                           void * workspace, int64_t rows, int64_t in_features, int64_t out_features,
                           int64_t num_experts, int64_t num_groups, int quant_type, void * stream) {
    if (packed_up == nullptr || output_activated == nullptr) {
        return fail(TGO_ERR_INVALID, "the up weight and the activated output must not be null");
    }
    if (row_index != nullptr && input_rows <= 0) {
        return fail(TGO_ERR_INVALID, "input_rows must be positive; got %lld", static_cast<long long>(input_rows));
    }
    return grouped_forward(input_bf16, row_index, input_rows, packed_gate, packed_up, output_gate, output_activated,
                           expert_indices, expert_offsets, workspace, rows, in_features, out_features, num_experts,
                           num_groups, quant_type, stream, true);
}

int tgo_swiglu_rows(const void * gate_bf16, const void * up_bf16, void * activated_bf16, int64_t count, void * stream) {
    if (count <= 0) {
        return fail(TGO_ERR_INVALID, "count must be positive; got %lld", static_cast<long long>(count));
    }
    if (gate_bf16 == nullptr || up_bf16 == nullptr || activated_bf16 == nullptr) {
        return fail(TGO_ERR_INVALID, "gate, up and activated must not be null");
    }
    return check_hip(tgo::launch_swiglu_rows(static_cast<const uint16_t *>(gate_bf16), static_cast<const uint16_t *>(up_bf16),
                                             static_cast<uint16_t *>(activated_bf16), count, static_cast<hipStream_t>(stream)),
                     "swiglu launch");
}

int tgo_swiglu_backward(const void * gate_bf16, const void * up_bf16, const void * grad_activated_bf16,
                        const void * grad_gate_bf16, void * d_gate_bf16, void * d_up_bf16, int64_t count, void * stream) {
    if (count <= 0) {
        return fail(TGO_ERR_INVALID, "count must be positive; got %lld", static_cast<long long>(count));
    }
    if (gate_bf16 == nullptr || up_bf16 == nullptr || grad_activated_bf16 == nullptr || d_gate_bf16 == nullptr ||
        d_up_bf16 == nullptr) {
        return fail(TGO_ERR_INVALID, "gate, up, grad_activated, d_gate and d_up must not be null");
    }
    return check_hip(tgo::launch_swiglu_backward_rows(
                         static_cast<const uint16_t *>(gate_bf16), static_cast<const uint16_t *>(up_bf16),
                         static_cast<const uint16_t *>(grad_activated_bf16), static_cast<const uint16_t *>(grad_gate_bf16),
                         static_cast<uint16_t *>(d_gate_bf16), static_cast<uint16_t *>(d_up_bf16), count,
                         static_cast<hipStream_t>(stream)),
                     "swiglu_backward launch");
}

int tgo_moe_combine(const void * rows_bf16, const int64_t * slot_rows, const float * slot_weights,
                    void * output_bf16, int64_t tokens, int64_t top_k, int64_t num_rows, int64_t features,
                    void * stream) {
    if (tokens <= 0 || top_k <= 0 || num_rows <= 0) {
        return fail(TGO_ERR_INVALID, "tokens, top_k and num_rows must be positive");
    }
    if (features <= 0 || features % 8 != 0) {
        return fail(TGO_ERR_INVALID, "features must be a positive multiple of 8; got %lld",
                    static_cast<long long>(features));
    }
    if (tokens > INT_LIMIT || top_k > INT_LIMIT || features > INT_LIMIT || num_rows > INT_LIMIT ||
        (features + 2047) / 2048 > 65535) {
        return fail(TGO_ERR_INVALID, "a dimension exceeds the kernel limit");
    }
    TGO_TRY(check_pointer(rows_bf16, "rows"));
    TGO_TRY(check_pointer(output_bf16, "output"));
    if (slot_rows == nullptr || slot_weights == nullptr) {
        return fail(TGO_ERR_INVALID, "slot_rows and slot_weights must not be null");
    }
    return check_hip(tgo::launch_moe_combine(static_cast<const uint16_t *>(rows_bf16), slot_rows, slot_weights,
                                             static_cast<uint16_t *>(output_bf16), static_cast<int>(tokens),
                                             static_cast<int>(top_k), num_rows, static_cast<int>(features),
                                             static_cast<hipStream_t>(stream)),
                     "moe_combine launch");
}

int tgo_route_small(const int64_t * slot_experts, int64_t tokens, int64_t top_k, int64_t num_experts, int64_t * row_index,
                    int64_t * slot_rows, int64_t * expert_indices, int32_t * expert_offsets, void * stream) {
    if (tokens <= 0 || top_k <= 0 || num_experts <= 0) {
        return fail(TGO_ERR_INVALID, "tokens, top_k and num_experts must be positive");
    }
    if (tokens > TGO_ROUTE_SMALL_LIMIT || top_k > TGO_ROUTE_SMALL_LIMIT || tokens * top_k > TGO_ROUTE_SMALL_LIMIT ||
        num_experts > TGO_ROUTE_SMALL_LIMIT) {
        return fail(TGO_ERR_INVALID, "tgo_route_small sorts at most %d slots over at most %d experts; got %lld x %lld over %lld",
                    TGO_ROUTE_SMALL_LIMIT, TGO_ROUTE_SMALL_LIMIT, static_cast<long long>(tokens),
                    static_cast<long long>(top_k), static_cast<long long>(num_experts));
    }
    if (slot_experts == nullptr || row_index == nullptr || slot_rows == nullptr || expert_indices == nullptr ||
        expert_offsets == nullptr) {
        return fail(TGO_ERR_INVALID, "slot_experts, row_index, slot_rows, expert_indices and expert_offsets must not be null");
    }
    return check_hip(tgo::launch_route_small(slot_experts, static_cast<int>(tokens * top_k), static_cast<int>(top_k),
                                             static_cast<int>(num_experts), row_index, slot_rows, expert_indices,
                                             expert_offsets, static_cast<hipStream_t>(stream)),
                     "route_small launch");
}

int tgo_rows_to_tokens(const void * rows_bf16, const int64_t * order, const int64_t * starts, void * output_bf16,
                       int64_t tokens, int64_t num_rows, int64_t features, void * stream) {
    if (tokens <= 0 || num_rows <= 0) {
        return fail(TGO_ERR_INVALID, "tokens and num_rows must be positive");
    }
    if (features <= 0 || features % 8 != 0) {
        return fail(TGO_ERR_INVALID, "features must be a positive multiple of 8; got %lld",
                    static_cast<long long>(features));
    }
    if (tokens > INT_LIMIT || features > INT_LIMIT || num_rows > INT_LIMIT || (features + 2047) / 2048 > 65535) {
        return fail(TGO_ERR_INVALID, "a dimension exceeds the kernel limit");
    }
    TGO_TRY(check_pointer(rows_bf16, "rows"));
    TGO_TRY(check_pointer(output_bf16, "output"));
    if (order == nullptr || starts == nullptr) {
        return fail(TGO_ERR_INVALID, "order and starts must not be null");
    }
    return check_hip(tgo::launch_rows_to_tokens(static_cast<const uint16_t *>(rows_bf16), order, starts,
                                                static_cast<uint16_t *>(output_bf16), static_cast<int>(tokens), num_rows,
                                                static_cast<int>(features), static_cast<hipStream_t>(stream)),
                     "rows_to_tokens launch");
}

// Shared body of the grouped grad-input entry points; `row_token` is null for a cotangent given row by row.
static int grouped_grad_input(const void * grad_output_first, const void * grad_output_second,
                              const int64_t * row_token, const float * row_weight, int64_t tokens,
                              const void * packed_first, const void * packed_second, void * grad_input_bf16,
                              const int64_t * expert_indices, const int32_t * expert_offsets, void * workspace,
                              int64_t rows, int64_t out_features, int64_t in_features, int64_t num_experts,
                              int64_t num_groups, int quant_type, void * stream) {
    TGO_TRY(check_matmul_shape(rows, in_features, out_features, quant_type));
    TGO_TRY(check_grouped(num_experts, num_groups, expert_indices, expert_offsets));
    TGO_TRY(check_pointer(grad_output_first, "grad_output"));
    TGO_TRY(check_pointer(packed_first, "packed_weight"));
    TGO_TRY(check_pointer(grad_input_bf16, "grad_input"));
    TGO_TRY(check_pointer(workspace, "workspace"));
    if ((packed_second == nullptr) != (grad_output_second == nullptr)) {
        return fail(TGO_ERR_INVALID, "second packed_weight and second grad_output must be given together");
    }
    if (packed_second != nullptr) {
        TGO_TRY(check_pointer(packed_second, "second packed_weight"));
        TGO_TRY(check_pointer(grad_output_second, "second grad_output"));
    }
    hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    const int64_t bytes_per_expert = out_features * (in_features / tgo::QK_K) * tgo::block_bytes(quant_type);
    const int row_tile = tgo::BACKWARD_ROW_TILE;
    const tgo::TaskList tasks = tgo::task_list_view(workspace, rows, num_groups, row_tile);
    // workspace: task list, then one fragment-ordered cotangent per source; one launch packs the cotangent(s) and
    // writes the task list on the side
    uint8_t * cotangent_first = static_cast<uint8_t *>(workspace) + tgo_task_workspace_bytes(rows, num_groups);
    uint8_t * cotangent_second =
        packed_second != nullptr ? cotangent_first + tgo::cotangent_workspace_bytes(rows, out_features) : nullptr;
    // tasks of at most BACKWARD_SHORT_ROWS rows go behind the others: a kernel variant of their own runs them
    const tgo::TaskBuild build = {expert_indices, expert_offsets, tasks, static_cast<int>(num_experts),
                                  static_cast<int>(num_groups), static_cast<int>(rows), row_tile,
                                  tgo::BACKWARD_SHORT_ROWS, 0};
    TGO_TRY(check_hip(tgo::launch_pack_cotangent(static_cast<const uint16_t *>(grad_output_first),
                                                 static_cast<const uint16_t *>(grad_output_second), cotangent_first,
                                                 cotangent_second, static_cast<int>(rows),
                                                 static_cast<int>(out_features), hip_stream, &build, row_token,
                                                 row_weight, tokens),
                      "pack_cotangent launch"));
    return check_hip(tgo::launch_mmq_grad_input(cotangent_first, cotangent_second,
                                                static_cast<const uint8_t *>(packed_first),
                                                static_cast<const uint8_t *>(packed_second), bytes_per_expert,
                                                static_cast<uint16_t *>(grad_input_bf16), &tasks,
                                                static_cast<int>(rows), static_cast<int>(out_features),
                                                static_cast<int>(in_features), quant_type, hip_stream),
                     "grouped mmq_grad_input launch");
}

int tgo_grouped_mmq_grad_input(const void * grad_output_first, const void * grad_output_second,
                               const void * packed_first, const void * packed_second, void * grad_input_bf16,
                               const int64_t * expert_indices, const int32_t * expert_offsets,
                               void * workspace, int64_t rows, int64_t out_features, int64_t in_features,
                               int64_t num_experts, int64_t num_groups, int quant_type, void * stream) {
    return grouped_grad_input(grad_output_first, grad_output_second, nullptr, nullptr, 0, packed_first, packed_second,
                              grad_input_bf16, expert_indices, expert_offsets, workspace, rows, out_features,
                              in_features, num_experts, num_groups, quant_type, stream);
}

int tgo_grouped_mmq_grad_input_weighted(const void * grad_tokens_bf16, const int64_t * row_token,
                                        const float * row_weight, int64_t tokens, const void * packed,
                                        void * grad_input_bf16, const int64_t * expert_indices,
                                        const int32_t * expert_offsets, void * workspace, int64_t rows,
                                        int64_t out_features, int64_t in_features, int64_t num_experts,
                                        int64_t num_groups, int quant_type, void * stream) {
    if (row_token == nullptr || row_weight == nullptr) {
        return fail(TGO_ERR_INVALID, "row_token and row_weight must not be null");
    }
    if (tokens <= 0) {
        return fail(TGO_ERR_INVALID, "tokens must be positive; got %lld", static_cast<long long>(tokens));
    }
    return grouped_grad_input(grad_tokens_bf16, nullptr, row_token, row_weight, tokens, packed, nullptr,
                              grad_input_bf16, expert_indices, expert_offsets, workspace, rows, out_features,
                              in_features, num_experts, num_groups, quant_type, stream);
}

}  // extern "C"
