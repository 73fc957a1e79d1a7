// Shared enums, error codes and logging of the host-side `dl::` layer.
//
// The names and numeric values follow the reference so that code written against ESP-DL's public
// headers keeps compiling (esp-dl/dl/dl_define.hpp:75-140): quant_type_t, activation_type_t,
// runtime_mode_t, DL_SCALE / DL_RESCALE, DL_CLIP.  What is different by design: memory
// "capabilities" describe host RAM vs device HBM instead of internal RAM vs PSRAM.
#pragma once

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <string>

// esp_err_t subset used by the Model API (load / test return it).
typedef int esp_err_t;
#ifndef ESP_OK
#define ESP_OK 0
#define ESP_FAIL (-1)
#endif

namespace dl {
/// Number of errors logged by this process so far.  Module::forward returns void, as in the reference,
/// so a launch that a kernel rejects can only log; dl::Model compares this count before and after a
/// pass to report the failure to its caller (Model::last_run_failed).  The count is process-wide: an
/// error logged by another thread during the pass is attributed to the pass as well.
inline std::atomic<long> &error_log_count()
{
    static std::atomic<long> count{0};
    return count;
}
} // namespace dl

#define DL_LOGE(tag, fmt, ...) \
    (dl::error_log_count().fetch_add(1), std::fprintf(stderr, "E (%s) " fmt "\n", tag, ##__VA_ARGS__))
#define DL_LOGW(tag, fmt, ...) std::fprintf(stderr, "W (%s) " fmt "\n", tag, ##__VA_ARGS__)
#define DL_LOGI(tag, fmt, ...) std::fprintf(stdout, "I (%s) " fmt "\n", tag, ##__VA_ARGS__)

#define DL_MAX(x, y) (((x) < (y)) ? (y) : (x))
#define DL_MIN(x, y) (((x) < (y)) ? (x) : (y))
#define DL_CLIP(x, low, high) (((x) < (low)) ? (low) : (((x) > (high)) ? (high) : (x)))
#define DL_SCALE(exponent) (((exponent) > 0) ? (float)(1 << (exponent)) : ((float)1.0 / (float)(1 << -(exponent))))
#define DL_RESCALE(exponent) (((exponent) > 0) ? ((float)1.0 / (float)(1 << (exponent))) : (float)(1 << -(exponent)))

#define DL_QUANT8_MAX 127
#define DL_QUANT8_MIN -128
#define DL_QUANT16_MAX 32767
#define DL_QUANT16_MIN -32768

// Where a tensor's bytes live.  Activations and parameters of a built Model live in HBM; tensors a
// caller creates are host tensors unless asked otherwise.
#define MALLOC_CAP_DEFAULT 0u /* host memory */
#define MALLOC_CAP_HOST 0u
#define MALLOC_CAP_DEVICE 1u /* device memory (hipMalloc) */

namespace dl {

typedef enum {
    QUANT_TYPE_NONE,
    QUANT_TYPE_FLOAT32,
    QUANT_TYPE_SYMM_8BIT,
    QUANT_TYPE_SYMM_16BIT,
    QUANT_TYPE_SYMM_32BIT,
} quant_type_t;

typedef enum {
    Linear,
    ReLU,
    LeakyReLU,
    PReLU,
} activation_type_t;

// Kept for API compatibility.  On one GPU every mode runs the same batched kernels.
typedef enum {
    RUNTIME_MODE_AUTO = 0,
    RUNTIME_MODE_SINGLE_CORE = 1,
    RUNTIME_MODE_MULTI_CORE = 2,
} runtime_mode_t;

// tool::shift_and_round flavour; the portable C path of the reference is half-up, ESP32-P4 builds
// are half-even (esp-dl/dl/dl_define_private.hpp:44-48).  Selectable per Model here.
typedef enum {
    ROUND_MODE_HALF_UP = 0,
    ROUND_MODE_HALF_EVEN = 1,
} round_mode_t;

typedef struct {
    size_t device; /*!< HBM bytes  */
    size_t host;   /*!< host bytes */
} mem_info_t;

const char *quant_type_to_string(quant_type_t type);
const char *activation_type_to_string(activation_type_t type);

} // namespace dl
