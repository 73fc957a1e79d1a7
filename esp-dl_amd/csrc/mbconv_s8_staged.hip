// espdl_hip_mbconv_s8_staged: the inverted-residual block of espdl_hip_mbconv_s8 as its separate stages
// ([1x1 Conv] -> depthwise Conv -> 1x1 Conv [+ Add]) with the intermediate activations in device memory
// that belongs to the library, for callers that cannot allocate (code under HIP-graph capture, serving
// loops, harnesses that forbid hipMalloc) and whose block shape the single-launch kernels do not cover.
//
// The intermediates live in one file-scope device array.  Host code never uses the array's name as an
// address: the address is asked from the runtime once per device (hipGetSymbolAddress) and kept.
// Every call on a device shares that device's array, so calls that overlap on one device race; calls
// on one stream, or otherwise ordered, are safe.  Nothing in the array has to start at zero: every
// byte a stage reads was written by the stage before it in the same call.
#include <hip/hip_runtime.h>

#include <mutex>

#include "../../include/espdl_hip.h"
#include "espdl_kernels.h"

namespace {

constexpr size_t kScratchBytes = ESPDL_HIP_MBCONV_STAGED_MAX_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_lock;
unsigned char *g_scratch_ptr[kMaxDevices] = {};

// Device address of this device's copy of `scratch`; nullptr (and *err set) when the runtime refuses.
unsigned char *scratch_of_current_device(hipError_t *err)
{
    int dev = -1;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess)
        return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        *err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (*err != hipSuccess)
            return nullptr;
        g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
    }
    return g_scratch_ptr[dev];
}

size_t align256(size_t n)
{
    return (n + 255) & ~static_cast<size_t>(255);
}

} // namespace

extern "C" int espdl_hip_mbconv_s8_staged(const espdl_hip_mbconv_desc *d, const int8_t *in,
                                           const espdl_hip_mbconv_weights *w, const int8_t *residual, int8_t *out,
                                           void *stream)
{
    int32_t out_h = 0, out_w = 0;
    int rc = espdl_hip_mbconv_out_shape(d, &out_h, &out_w); // validates the descriptor
    if (rc != ESPDL_HIP_OK)
        return rc;
    if (d->batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr || w == nullptr)
        return espdl::set_error(ESPDL_HIP_EINVAL, "in, out and weights must not be NULL");
    if (d->residual_shift != 0 && residual != nullptr)
        return espdl::set_error(ESPDL_HIP_ENOTSUP, "the staged form adds the residual operand as it is (residual_shift %d): "
                                                   "requantize it first with espdl_hip_requantize_s8", d->residual_shift);
    // extents of the depthwise stage's input: the block input's, or those of an expand stage with a window
    const bool windowed = d->exp_k_h > 0;
    const int mid_h = windowed ? (d->in_h + d->exp_pad_top + d->exp_pad_bottom - d->exp_k_h) / d->exp_stride_h + 1 : d->in_h;
    const int mid_w = windowed ? (d->in_w + d->exp_pad_left + d->exp_pad_right - d->exp_k_w) / d->exp_stride_w + 1 : d->in_w;
    const size_t expanded = d->has_expand ? align256((size_t)d->batch * mid_h * mid_w * d->exp_c) : 0;
    const size_t dw_out = align256((size_t)d->batch * out_h * out_w * d->exp_c);
    if (expanded + dw_out > kScratchBytes)
        return espdl::set_error(ESPDL_HIP_ENOTSUP,
                                "the intermediates of this block need %zu bytes, the library's array holds %zu "
                                "(ESPDL_HIP_MBCONV_STAGED_MAX_BYTES): use a smaller batch per call",
                                expanded + dw_out, kScratchBytes);
    hipError_t err = hipSuccess;
    {
        // The array's address is looked up on the first call on a device, which may load the code object: not
        // something to do while `stream` records a graph.  One call (or espdl_hip_mbconv_s8_staged_init) outside
        // capture comes first.
        int dev = -1;
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices && g_scratch_ptr[dev] == nullptr &&
            hipStreamIsCapturing(reinterpret_cast<hipStream_t>(stream), &capturing) == hipSuccess &&
            capturing != hipStreamCaptureStatusNone)
            return espdl::set_error(ESPDL_HIP_ENOTSUP, "the first espdl_hip_mbconv_s8_staged call on a device must not be "
                                                       "under stream capture: call espdl_hip_mbconv_s8_staged_init first");
    }
    unsigned char *base = scratch_of_current_device(&err);
    if (base == nullptr)
        return espdl::set_error(ESPDL_HIP_EDEVICE, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(err));
    int8_t *t_expand = reinterpret_cast<int8_t *>(base);
    int8_t *t_dw = reinterpret_cast<int8_t *>(base + expanded);

    const int8_t *dw_in = in;
    if (d->has_expand) {
        espdl_hip_conv_desc c = {};
        c.dtype = ESPDL_HIP_S8;
        c.batch = d->batch;
        c.in_h = d->in_h;
        c.in_w = d->in_w;
        c.in_c = d->in_c;
        c.out_c = d->exp_c;
        c.k_h = c.k_w = c.stride_h = c.stride_w = c.dil_h = c.dil_w = 1;
        if (windowed) {
            c.k_h = d->exp_k_h;
            c.k_w = d->exp_k_w;
            c.stride_h = d->exp_stride_h;
            c.stride_w = d->exp_stride_w;
            c.pad_top = d->exp_pad_top;
            c.pad_bottom = d->exp_pad_bottom;
            c.pad_left = d->exp_pad_left;
            c.pad_right = d->exp_pad_right;
        }
        c.group = 1;
        c.activation = d->act_expand;
        c.round_mode = d->round_mode;
        c.n_shift = d->n_shift_expand;
        rc = espdl_hip_conv2d(&c, in, w->w_expand, w->b_expand, w->s_expand, nullptr, t_expand, stream);
        if (rc == ESPDL_HIP_OK && d->clip_expand != 0) // a Clip with equal exponents: in place on the intermediate
            rc = espdl_hip_clip_s8(t_expand, (int64_t)d->batch * mid_h * mid_w * d->exp_c, d->clip_expand_min,
                                   d->clip_expand_max, 0, 0, t_expand, stream);
        if (rc != ESPDL_HIP_OK)
            return rc;
        dw_in = t_expand;
    }
    {
        espdl_hip_conv_desc c = {};
        c.dtype = ESPDL_HIP_S8;
        c.batch = d->batch;
        c.in_h = mid_h;
        c.in_w = mid_w;
        c.in_c = d->exp_c;
        c.out_c = d->exp_c;
        c.k_h = d->k_h;
        c.k_w = d->k_w;
        c.stride_h = d->stride_h;
        c.stride_w = d->stride_w;
        c.dil_h = d->dil_h;
        c.dil_w = d->dil_w;
        c.pad_top = d->pad_top;
        c.pad_bottom = d->pad_bottom;
        c.pad_left = d->pad_left;
        c.pad_right = d->pad_right;
        c.group = d->exp_c;
        c.activation = d->act_dw;
        c.round_mode = d->round_mode;
        c.n_shift = d->n_shift_dw;
        rc = espdl_hip_conv2d(&c, dw_in, w->w_dw, w->b_dw, w->s_dw, nullptr, t_dw, stream);
        if (rc == ESPDL_HIP_OK && d->clip_dw != 0)
            rc = espdl_hip_clip_s8(t_dw, (int64_t)d->batch * out_h * out_w * d->exp_c, d->clip_dw_min, d->clip_dw_max, 0, 0,
                                   t_dw, stream);
        if (rc != ESPDL_HIP_OK)
            return rc;
    }
    espdl_hip_conv_desc c = {};
    c.dtype = ESPDL_HIP_S8;
    c.batch = d->batch;
    c.in_h = out_h;
    c.in_w = out_w;
    c.in_c = d->exp_c;
    c.out_c = d->out_c;
    c.k_h = c.k_w = c.stride_h = c.stride_w = c.dil_h = c.dil_w = 1;
    c.group = 1;
    c.activation = d->act_project;
    c.round_mode = d->round_mode;
    c.n_shift = d->n_shift_project;
    return espdl_hip_conv2d_add(&c, t_dw, w->w_project, w->b_project, w->s_project, nullptr, residual, out, stream);
}

extern "C" int espdl_hip_mbconv_s8_staged_init(void)
{
    hipError_t err = hipSuccess;
    if (scratch_of_current_device(&err) == nullptr)
        return espdl::set_error(ESPDL_HIP_EDEVICE, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(err));
    return ESPDL_HIP_OK;
}
