// C entry points of libxnor_nn.so (include/xnor_nn.h, include/xnor_nn_hip.h): descriptor
// setup, device resources, the four stage executors and the export helpers.
//
// Host side only; every kernel lives in the kernels_*.hip files behind the launch_*
// functions of plan.hpp.  There is no CPU implementation of any stage: when no GPU is
// usable the executors report xnor_nn_error_memory.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <mutex>
#include <new>
#include <unordered_map>
#include <utility>
#include <vector>

#include "plan.hpp"
#include "xnor_nn_hip.h"

using namespace xnor_hip;

namespace {

bool is_data_format(int f) {
    return f == xnor_nn_data_format_nchw || f == xnor_nn_data_format_nhwc;
}
bool is_weights_format(int f) {
    return f == xnor_nn_weights_format_oihw || f == xnor_nn_weights_format_hwio;
}

size_t src_elems(const Geometry &g) { return (size_t)g.mb * g.ic * g.ih * g.iw; }
size_t weights_elems(const Geometry &g) { return (size_t)g.oc * g.ic * g.kh * g.kw; }
size_t dst_elems(const Geometry &g) { return (size_t)g.mb * g.oc * g.oh * g.ow; }

// True when a kernel can dereference p (device or managed allocation).
bool on_device(const void *p) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError(); // plain host memory: clear the sticky error
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

// Device view of a user tensor the kernels read: the pointer itself, or a staged copy.
xnor_nn_status_t stage_in(State *st, void **slot, const void *user, size_t bytes,
        const void **dev) {
    if (on_device(user)) { *dev = user; return xnor_nn_success; }
    if (!*slot && hipMalloc(slot, bytes) != hipSuccess) return xnor_nn_error_memory;
    if (hipMemcpyAsync(*slot, user, bytes, hipMemcpyHostToDevice, st->stream) != hipSuccess)
        return xnor_nn_error_memory;
    // the host buffer may be pageable: the copy must have left it before we return
    if (hipStreamSynchronize(st->stream) != hipSuccess) return xnor_nn_error_memory;
    *dev = *slot;
    return xnor_nn_success;
}

xnor_nn_status_t unimplemented_stage(const xnor_nn_convolution_t *, xnor_nn_resources_t) {
    return xnor_nn_unimplemented;
}

// ---- what one stage hands to the next ---------------------------------------------------
// The executors are stateless apart from the launch plan behind c->state, like the
// reference's (reference src/bcast_convolution.hpp:77-93): what a stage hands to a later one
// is recorded against the device buffers of the caller's resource table, so two threads
// that share a descriptor and bring a table each do not see each other's hand-overs.
//   ready: binarize_data has also left mean|x| of this input in this `a` plane; the
//          calculate_k that follows it immediately on the same buffers skips its own pass
//          over the input.  Any other executor on the table withdraws the offer.
//   owed:  calculate_k has mean|x| in `a` and has not run the box filter, because the
//          matrix-core convolution sums K from mean|x| on the fly and stores it to this K
//          plane.  Whatever else needs the K plane, or is about to overwrite that mean|x|,
//          runs the box filter first.
// Entries die with the buffers (xnor_nn_free_resources) and with the descriptor.
// An Owed entry also names the stream on which its mean|x| was written: the box filter that
// settles it runs there, whichever descriptor's call triggers it.
struct Ready { const State *st; const void *src; };
struct Owed { const State *st; const float *a; hipStream_t stream; };
std::mutex handover_mu;
std::unordered_map<const void *, Ready> ready_by_a;
std::unordered_map<const void *, Owed> owed_by_k;

// (XNOR_NN_HIP_SEPARATE_K is read once, when the descriptor is initialised)
bool fusion_on(const State *st) { return st->fuse_stages; }

void withdraw_ready(const void *a) {
    if (a == nullptr) return;
    std::lock_guard<std::mutex> lock(handover_mu);
    ready_by_a.erase(a);
}

// Takes the entry for k out of the table; false when there is none.
bool take_owed(const void *k, Owed *out) {
    std::lock_guard<std::mutex> lock(handover_mu);
    auto it = owed_by_k.find(k);
    if (it == owed_by_k.end()) return false;
    *out = it->second;
    owed_by_k.erase(it);
    return true;
}

// The box filter owed to k, with the geometry of the descriptor that owes it (fixed at its
// initialisation) and on the stream its mean|x| was written on.  When that is not the
// calling descriptor's stream, the two are ordered with events in both directions: the
// filter runs after what the caller has enqueued so far (which may still read the old K
// plane), and what the caller enqueues next (a kernel that reads K, or one that overwrites
// mean|x|) runs after the filter.  Called with st->mu held.
xnor_nn_status_t run_box_filter(State *st, const Owed &o, float *k) {
    if (st->verbose) printf("xnor_nn exec (deferred calculate_k): box_filter_kernel\n");
    const bool other_stream = o.stream != st->stream;
    if (other_stream) {
        if (!st->order_before
                && (hipEventCreateWithFlags(&st->order_before, hipEventDisableTiming) != hipSuccess
                    || hipEventCreateWithFlags(&st->order_after, hipEventDisableTiming)
                        != hipSuccess)) {
            (void)hipGetLastError();
            return xnor_nn_error_memory;
        }
        if (hipEventRecord(st->order_before, st->stream) != hipSuccess
                || hipStreamWaitEvent(o.stream, st->order_before, 0) != hipSuccess)
            return xnor_nn_error_memory;
    }
    if (launch_box_filter(o.st->g, o.a, k, o.stream) != hipSuccess) return xnor_nn_error_memory;
    if (other_stream
            && (hipEventRecord(st->order_after, o.stream) != hipSuccess
                || hipStreamWaitEvent(st->stream, st->order_after, 0) != hipSuccess))
        return xnor_nn_error_memory;
    return xnor_nn_success;
}

// Runs the box filter owed to the K plane k, if any.
xnor_nn_status_t settle_k(State *st, float *k) {
    Owed o;
    if (!take_owed(k, &o)) return xnor_nn_success;
    return run_box_filter(st, o, k);
}

// Runs every box filter that still has to read the mean|x| plane a (about to be overwritten),
// except the one owed to skip_k, which is dropped: its K plane is about to be recomputed.
xnor_nn_status_t settle_readers_of(State *st, const float *a, const void *skip_k) {
    std::vector<std::pair<float *, Owed>> todo;
    {
        std::lock_guard<std::mutex> lock(handover_mu);
        if (skip_k) owed_by_k.erase(skip_k);
        for (auto it = owed_by_k.begin(); it != owed_by_k.end();) {
            if (it->second.a == a) {
                todo.emplace_back(static_cast<float *>(const_cast<void *>(it->first)),
                        it->second);
                it = owed_by_k.erase(it);
            } else {
                ++it;
            }
        }
    }
    for (auto &t : todo) {
        const xnor_nn_status_t rc = run_box_filter(st, t.second, t.first);
        if (rc != xnor_nn_success) return rc;
    }
    return xnor_nn_success;
}

void forget_buffers(const void *a, const void *k) {
    std::lock_guard<std::mutex> lock(handover_mu);
    if (a) ready_by_a.erase(a);
    if (k) owed_by_k.erase(k);
    if (a)
        for (auto it = owed_by_k.begin(); it != owed_by_k.end();)
            it = it->second.a == a ? owed_by_k.erase(it) : std::next(it);
}

void forget_descriptor(const State *st) {
    std::lock_guard<std::mutex> lock(handover_mu);
    for (auto it = ready_by_a.begin(); it != ready_by_a.end();)
        it = it->second.st == st ? ready_by_a.erase(it) : std::next(it);
    for (auto it = owed_by_k.begin(); it != owed_by_k.end();)
        it = it->second.st == st ? owed_by_k.erase(it) : std::next(it);
}

// ---- stage 1 --------------------------------------------------------------------------
// Replaces reference src/bcast_binarize_data.cpp:13-76 (same null checks, same
// "unimplemented" for an unknown format).
xnor_nn_status_t exec_binarize_data(const xnor_nn_convolution_t *c, xnor_nn_resources_t res) {
    if (c == nullptr || res[xnor_nn_resource_user_src] == nullptr
            || res[xnor_nn_resource_bin_src] == nullptr)
        return xnor_nn_error_invalid_input;
    if (!is_data_format(c->src_format)) return xnor_nn_unimplemented;
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    const void *x = nullptr;
    xnor_nn_status_t rc = stage_in(st, &st->stage_src, res[xnor_nn_resource_user_src],
            src_elems(st->g) * sizeof(float), &x);
    if (rc != xnor_nn_success) return rc;
    float *a = static_cast<float *>(res[xnor_nn_resource_a]); // optional by-product
    if (a != nullptr) { // about to overwrite the mean|x| a K may be owed from
        withdraw_ready(a);
        rc = settle_readers_of(st, a, nullptr);
        if (rc != xnor_nn_success) return rc;
    }
    if (st->verbose) printf("xnor_nn exec binarize_data: %s\n", binarize_kernel_name(st->g));
    if (launch_binarize_data(st->g, static_cast<const float *>(x),
                static_cast<uint32_t *>(res[xnor_nn_resource_bin_src]), a, st->stream,
                st->time_binarize.next())
            != hipSuccess)
        return xnor_nn_error_memory;
    if (a != nullptr && fusion_on(st)) {
        std::lock_guard<std::mutex> lock(handover_mu);
        ready_by_a[a] = Ready{st, res[xnor_nn_resource_user_src]};
    }
    return xnor_nn_success;
}

// ---- stage 2 --------------------------------------------------------------------------
// Replaces reference src/bcast_calculate_k.cpp:13-88.  When the preceding
// binarize_data call on the same src/a buffers already produced mean|x|, only the box
// filter runs; otherwise the input is read here.
xnor_nn_status_t exec_calculate_k(const xnor_nn_convolution_t *c, xnor_nn_resources_t res) {
    if (c == nullptr || res[xnor_nn_resource_user_src] == nullptr
            || res[xnor_nn_resource_a] == nullptr || res[xnor_nn_resource_k] == nullptr)
        return xnor_nn_error_invalid_input;
    if (!is_data_format(c->src_format)) return xnor_nn_unimplemented;
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    float *a = static_cast<float *>(res[xnor_nn_resource_a]);
    float *k = static_cast<float *>(res[xnor_nn_resource_k]);
    const bool fuse = fusion_on(st);
    bool a_ready = false;
    {
        std::lock_guard<std::mutex> lock(handover_mu);
        auto it = ready_by_a.find(a);
        if (it != ready_by_a.end()) { // one-shot
            a_ready = fuse && it->second.st == st
                && it->second.src == res[xnor_nn_resource_user_src];
            ready_by_a.erase(it);
        }
    }
    xnor_nn_status_t rc;
    if (!a_ready) {
        // mean|x| is about to be overwritten: box filters that still read it run first (the
        // one owed to this K plane is dropped, the plane is recomputed below)
        rc = settle_readers_of(st, a, k);
        if (rc != xnor_nn_success) return rc;
        const void *x = nullptr;
        rc = stage_in(st, &st->stage_src, res[xnor_nn_resource_user_src],
                src_elems(st->g) * sizeof(float), &x);
        if (rc != xnor_nn_success) return rc;
        if (launch_mean_abs(st->g, static_cast<const float *>(x), a, st->stream) != hipSuccess)
            return xnor_nn_error_memory;
    }
    // The matrix-core convolution sums K from mean|x| itself, which saves this launch; the
    // K plane is then written by the forward executor (or by whatever needs it earlier).
    if (st->g.use_mfma && fuse) {
        if (st->verbose)
            printf("xnor_nn exec calculate_k: %sbox filter deferred to the convolution\n",
                    a_ready ? "" : "mean_abs, ");
        std::lock_guard<std::mutex> lock(handover_mu);
        owed_by_k[k] = Owed{st, a, st->stream};
        return xnor_nn_success;
    }
    {
        std::lock_guard<std::mutex> lock(handover_mu);
        owed_by_k.erase(k); // superseded by the filter below
    }
    if (st->verbose)
        printf("xnor_nn exec calculate_k: %sbox_filter_kernel\n", a_ready ? "" : "mean_abs + ");
    if (launch_box_filter(st->g, a, k, st->stream) != hipSuccess) return xnor_nn_error_memory;
    return xnor_nn_success;
}

// ---- weights --------------------------------------------------------------------------
// Replaces reference src/bcast_binarize_weights.cpp:13-145.
xnor_nn_status_t exec_binarize_weights(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res) {
    if (c == nullptr || res[xnor_nn_resource_user_weights] == nullptr
            || res[xnor_nn_resource_bin_weights] == nullptr
            || res[xnor_nn_resource_operations_count] == nullptr
            || res[xnor_nn_resource_alpha] == nullptr)
        return xnor_nn_error_invalid_input;
    if (!is_weights_format(c->weights_format)) return xnor_nn_unimplemented;
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    withdraw_ready(res[xnor_nn_resource_a]);
    const void *w = nullptr;
    xnor_nn_status_t rc = stage_in(st, &st->stage_weights, res[xnor_nn_resource_user_weights],
            weights_elems(st->g) * sizeof(float), &w);
    if (rc != xnor_nn_success) return rc;
    if (st->verbose) printf("xnor_nn exec binarize_weights: pack/alpha/op_count kernels\n");
    if (launch_binarize_weights(st->g, static_cast<const float *>(w),
                static_cast<uint32_t *>(res[xnor_nn_resource_bin_weights]),
                static_cast<float *>(res[xnor_nn_resource_alpha]),
                static_cast<int32_t *>(res[xnor_nn_resource_operations_count]), st->stream)
            != hipSuccess)
        return xnor_nn_error_memory;
    if (st->g.use_mfma && launch_pack_weights_fp4(st->g, static_cast<const float *>(w),
                reinterpret_cast<uint32_t *>(static_cast<char *>(
                        res[xnor_nn_resource_bin_weights]) + st->g.wfrag_offset), st->stream)
            != hipSuccess)
        return xnor_nn_error_memory;
    return xnor_nn_success;
}

// ---- stage 3 --------------------------------------------------------------------------
xnor_nn_status_t run_convolution(const xnor_nn_convolution_t *c, xnor_nn_resources_t res,
        void *user_out, bool raw) {
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    withdraw_ready(res[xnor_nn_resource_a]);
    const size_t bytes = dst_elems(st->g) * 4;
    void *out = user_out;
    const bool direct = on_device(user_out);
    if (!direct) {
        if (!st->stage_dst && hipMalloc(&st->stage_dst, bytes) != hipSuccess)
            return xnor_nn_error_memory;
        out = st->stage_dst;
    }
    const uint32_t *xbits = static_cast<const uint32_t *>(res[xnor_nn_resource_bin_src]);
    const float *alpha = static_cast<const float *>(res[xnor_nn_resource_alpha]);
    float *k = static_cast<float *>(res[xnor_nn_resource_k]);
    const int32_t *opc = static_cast<const int32_t *>(res[xnor_nn_resource_operations_count]);
    float *dst = raw ? nullptr : static_cast<float *>(out);
    int32_t *popc = raw ? static_cast<int32_t *>(out) : nullptr;
    hipError_t err;
    // a K owed to exactly this K plane is computed inside the matrix-core kernel; the raw
    // accumulators need no K at all
    const float *a = nullptr;
    Owed o;
    if (!raw && take_owed(k, &o)) {
        if (st->g.use_mfma && o.st == st && o.stream == st->stream) {
            a = o.a;
        } else {
            const xnor_nn_status_t rc = run_box_filter(st, o, k);
            if (rc != xnor_nn_success) return rc;
        }
    }
    if (st->g.use_mfma) {
        const uint32_t *wfrag = reinterpret_cast<const uint32_t *>(
                static_cast<const char *>(res[xnor_nn_resource_bin_weights]) + st->g.wfrag_offset);
        if (st->verbose)
            printf("xnor_nn exec forward: %s%s\n", convolution_kernel_name(st->g),
                    a ? " (with the box filter of calculate_k)" : "");
        err = launch_convolution_mfma(st->g, xbits, wfrag, alpha, k, dst, popc, a, k,
                st->stream, st->time_convolution.next());
    } else {
        if (st->verbose) printf("xnor_nn exec forward: %s\n", convolution_kernel_name(st->g));
        err = launch_convolution(st->g, xbits,
                static_cast<const uint32_t *>(res[xnor_nn_resource_bin_weights]), alpha, k, opc,
                dst, popc, st->stream, st->time_convolution.next());
    }
    if (err != hipSuccess) return xnor_nn_error_memory;
    if (!direct) {
        if (hipMemcpyAsync(user_out, out, bytes, hipMemcpyDeviceToHost, st->stream) != hipSuccess
                || hipStreamSynchronize(st->stream) != hipSuccess)
            return xnor_nn_error_memory;
    }
    return xnor_nn_success;
}

// Replaces reference src/default/bcast_convolution_default.cpp:14-108 / :110-216 and the
// ISA-specific kernels selected in reference src/bcast_convolution.cpp:93-116.
xnor_nn_status_t exec_forward(const xnor_nn_convolution_t *c, xnor_nn_resources_t res) {
    if (c == nullptr || res[xnor_nn_resource_bin_src] == nullptr
            || res[xnor_nn_resource_bin_weights] == nullptr
            || res[xnor_nn_resource_user_dst] == nullptr
            || res[xnor_nn_resource_k] == nullptr
            || res[xnor_nn_resource_alpha] == nullptr
            || res[xnor_nn_resource_operations_count] == nullptr)
        return xnor_nn_error_invalid_input;
    if (!is_data_format(c->dst_format)) return xnor_nn_unimplemented;
    return run_convolution(c, res, res[xnor_nn_resource_user_dst], false);
}

xnor_nn_status_t to_host(const xnor_nn_convolution_t *c, const void *dev, void *dst,
        size_t bytes) {
    State *st = state_of(c);
    if (hipMemcpyAsync(dst, dev, bytes, hipMemcpyDeviceToHost, st->stream) != hipSuccess
            || hipStreamSynchronize(st->stream) != hipSuccess)
        return xnor_nn_error_memory;
    return xnor_nn_success;
}

void drop_timer(KernelTimer &t) {
    for (KernelEvents &e : t.ring) {
        if (e.start) (void)hipEventDestroy(e.start);
        if (e.stop) (void)hipEventDestroy(e.stop);
    }
    t.ring.clear();
    t.launches = 0;
}

bool make_timer(KernelTimer &t, int capacity) {
    drop_timer(t);
    for (int i = 0; i < capacity; i++) {
        KernelEvents e;
        if (hipEventCreate(&e.start) != hipSuccess || hipEventCreate(&e.stop) != hipSuccess) {
            if (e.start) (void)hipEventDestroy(e.start);
            (void)hipGetLastError();
            drop_timer(t);
            return false;
        }
        t.ring.push_back(e);
    }
    return true;
}

int canonical_bici(const Geometry &g) { return (g.ic * g.kh * g.kw < 32767) ? 2 : 4; }
int div_up(int a, int b) { return (a + b - 1) / b; }

bool bcast_descriptor(const xnor_nn_convolution_t *c) {
    return c != nullptr && c->state != nullptr && c->algorithm == xnor_nn_algorithm_bcast;
}

} // namespace

extern "C" {

void xnor_nn_get_status_message(char *msg, xnor_nn_status_t status) {
    const char *text = "unimplemented";
    switch (status) {
    case xnor_nn_success: text = "success"; break;
    case xnor_nn_error_memory: text = "memory_error"; break;
    case xnor_nn_error_invalid_input: text = "bad_input"; break;
    case xnor_nn_unimplemented: text = "unimplemented"; break;
    }
    strcpy(msg, text);
}

xnor_nn_status_t xnor_nn_init_convolution(xnor_nn_convolution_t *c,
        const xnor_nn_algorithm_t algorithm,
        const xnor_nn_tensor_format_t src_fmt,
        const xnor_nn_tensor_format_t weights_fmt,
        const xnor_nn_tensor_format_t dst_fmt,
        int mb, int oc, int ic, int ih, int iw,
        int kh, int kw, int sh, int sw, int ph, int pw) {
    c->algorithm = algorithm;
    c->mb = mb;
    c->ic = ic; c->ih = ih; c->iw = iw;
    c->oc = oc;
    // The reference derives BOTH extents from pw (src/common_convolution.cpp:16-17).
    c->oh = (ih + 2 * pw - kh) / sh + 1;
    c->ow = (iw + 2 * pw - kw) / sw + 1;
    c->sh = sh; c->sw = sw;
    c->kh = kh; c->kw = kw;
    c->ph = ph; c->pw = pw;
    c->src_format = src_fmt;
    c->weights_format = weights_fmt;
    c->dst_format = dst_fmt;
    for (int i = xnor_nn_resource_internal; i < xnor_nn_resource_number; i++)
        c->resource_size[i] = 0;
    c->binarize_weights = unimplemented_stage;
    c->binarize_data = unimplemented_stage;
    c->calculate_k = unimplemented_stage;
    c->forward = unimplemented_stage;
    c->state = nullptr;

    if (algorithm != xnor_nn_algorithm_bcast) return xnor_nn_success;

    State *st = new (std::nothrow) State();
    if (!st) return xnor_nn_success; // executors stay "unimplemented", like a failed match
    Geometry &g = st->g;
    g.mb = mb; g.ic = ic; g.ih = ih; g.iw = iw; g.oc = oc; g.oh = c->oh; g.ow = c->ow;
    g.kh = kh; g.kw = kw; g.sh = sh; g.sw = sw; g.ph = ph; g.pw = pw;
    g.src_fmt = src_fmt; g.w_fmt = weights_fmt; g.dst_fmt = dst_fmt;
    g.xw = div_up(ic, 32);
    g.q = pick_q(oc, g.xw);
    g.ocb = div_up(oc, g.q);
    g.ihw = ih * iw;
    g.ohw = g.oh * g.ow;
    g.npix_in = (uint32_t)mb * g.ihw;
    g.npix_out = (uint32_t)mb * g.ohw;
    g.div_ihw = FastDiv::make(g.ihw);
    g.div_iw = FastDiv::make(iw);
    g.div_ohw = FastDiv::make(g.ohw);
    g.div_ow = FastDiv::make(g.ow);
    const char *v = getenv("XNOR_NN_VERBOSE");
    st->verbose = v && v[0] == '1';
    st->fuse_stages = getenv("XNOR_NN_HIP_SEPARATE_K") == nullptr; // read here, once

    // Byte sizes of the device buffers (the reference's are host sizes of its CPU layout,
    // src/bcast_convolution.cpp:72-82).
    c->resource_size[xnor_nn_resource_bin_src] = (size_t)g.npix_in * g.xw * 4;
    const size_t bit_bytes = (size_t)g.ocb * kh * kw * g.xw * g.q * 4;
    g.cus = 256;
    {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n,
                    hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) {
            g.cus = n;
            // the device address of the library's static partial-sum array is looked up here,
            // once per device, so that xnor_nn_hip_binarize_weights_float_noalloc itself
            // only reads it back (it may be called where nothing may be set up any more)
            float *unused = nullptr;
            if (weights_float_scratch(&unused) != hipSuccess) (void)hipGetLastError();
        } else {
            (void)hipGetLastError();
        }
    }
    mfma_plan(g);
    g.wfrag_offset = (bit_bytes + 255) / 256 * 256;
    c->resource_size[xnor_nn_resource_bin_weights] =
        g.use_mfma ? g.wfrag_offset + g.mfma_wbytes : bit_bytes;
    c->resource_size[xnor_nn_resource_a] = (size_t)g.npix_in * 4;
    c->resource_size[xnor_nn_resource_k] = (size_t)g.npix_out * 4;
    c->resource_size[xnor_nn_resource_alpha] = (size_t)oc * 4;
    c->resource_size[xnor_nn_resource_operations_count] = (size_t)g.ohw * 4;

    c->binarize_weights = exec_binarize_weights;
    c->binarize_data = exec_binarize_data;
    c->calculate_k = exec_calculate_k;
    c->forward = exec_forward;
    c->state = st;
    if (st->verbose)
        printf("xnor_nn init: bcast gfx950 mb=%d ic=%d %dx%d oc=%d %dx%d k=%dx%d s=%dx%d "
               "p=%dx%d words/pixel=%d conv=%s\n", mb, ic, ih, iw, oc, c->oh, c->ow, kh, kw,
               sh, sw, ph, pw, g.xw, convolution_kernel_name(g));
    return xnor_nn_success;
}

void xnor_nn_destroy_convolution(xnor_nn_convolution_t *c) {
    if (c == nullptr || c->state == nullptr) return;
    State *st = state_of(c);
    forget_descriptor(st);
    if (st->stage_src) (void)hipFree(st->stage_src);
    if (st->stage_weights) (void)hipFree(st->stage_weights);
    if (st->stage_dst) (void)hipFree(st->stage_dst);
    if (st->float_parts) (void)hipFree(st->float_parts);
    if (st->order_before) (void)hipEventDestroy(st->order_before);
    if (st->order_after) (void)hipEventDestroy(st->order_after);
    drop_timer(st->time_binarize);
    drop_timer(st->time_convolution);
    delete st;
    c->state = nullptr;
}

xnor_nn_status_t xnor_nn_allocate_resources(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res) {
    for (int i = xnor_nn_resource_internal; i < xnor_nn_resource_number; i++) {
        void *p = nullptr;
        // a zero-sized slot still gets a distinct non-null buffer, as aligned_alloc gives
        const size_t bytes = c->resource_size[i] ? c->resource_size[i] : 4;
        if (hipMalloc(&p, bytes) != hipSuccess) {
            (void)hipGetLastError();
            xnor_nn_free_resources(res);
            return xnor_nn_error_memory;
        }
        res[i] = p;
    }
    return xnor_nn_success;
}

void xnor_nn_free_resources(xnor_nn_resources_t res) {
    // nothing may be handed over through buffers that are about to go
    forget_buffers(res[xnor_nn_resource_a], res[xnor_nn_resource_k]);
    for (int i = xnor_nn_resource_internal; i < xnor_nn_resource_number; i++) {
        if (res[i]) (void)hipFree(res[i]);
        res[i] = nullptr;
    }
}

// Replaces reference src/binarize_weights_float.cpp:3-25.  Host buffers are staged through
// device copies and the call returns when `to` is written; with both buffers on the device
// it only enqueues two kernels on the descriptor's stream, like the executors.
void xnor_nn_binarize_weights_float(const xnor_nn_convolution_t *c,
        const float *from, float *to) {
    const size_t n = (size_t)c->oc * c->ic * c->kh * c->kw;
    const size_t bytes = n * sizeof(float);
    State *st = c->state ? state_of(c) : nullptr;
    hipStream_t s = st ? st->stream : nullptr;
    const bool from_dev = on_device(from), to_dev = on_device(to);
    float *dfrom = nullptr, *dto = nullptr, *own_parts = nullptr, *parts = nullptr;
    bool ok = true;
    std::unique_lock<std::mutex> call;
    if (st) { // the partial sums live with the descriptor
        call = std::unique_lock<std::mutex>(st->mu);
        if (!st->float_parts)
            ok = hipMalloc((void **)&st->float_parts, weights_float_parts() * sizeof(float))
                == hipSuccess;
        parts = st->float_parts;
    } else {
        ok = hipMalloc((void **)&own_parts, weights_float_parts() * sizeof(float)) == hipSuccess;
        parts = own_parts;
    }
    if (ok && !from_dev) ok = hipMalloc((void **)&dfrom, bytes) == hipSuccess
        && hipMemcpyAsync(dfrom, from, bytes, hipMemcpyHostToDevice, s) == hipSuccess
        && hipStreamSynchronize(s) == hipSuccess;
    if (ok && !to_dev) ok = hipMalloc((void **)&dto, bytes) == hipSuccess;
    if (ok) ok = launch_weights_float(from_dev ? from : dfrom, to_dev ? to : dto, n, parts, s)
        == hipSuccess;
    if (ok && !to_dev) ok = hipMemcpyAsync(to, dto, bytes, hipMemcpyDeviceToHost, s) == hipSuccess;
    if (dfrom || dto || own_parts || !ok) { // something of this call's has to outlive the kernels
        if (hipStreamSynchronize(s) != hipSuccess) ok = false;
    }
    if (!ok) {
        (void)hipGetLastError();
        fprintf(stderr, "xnor_nn_binarize_weights_float: HIP failure, output not written\n");
    }
    if (dfrom) (void)hipFree(dfrom);
    if (dto) (void)hipFree(dto);
    if (own_parts) (void)hipFree(own_parts);
}

// ---- include/xnor_nn_hip.h --------------------------------------------------------------

// xnor_nn_binarize_weights_float for callers that may not allocate: both buffers on the
// device, partial sums in the library's static device array, two kernels enqueued on the
// descriptor's stream, nothing else.
xnor_nn_status_t xnor_nn_hip_binarize_weights_float_noalloc(const xnor_nn_convolution_t *c,
        const float *from, float *to) {
    if (c == nullptr || from == nullptr || to == nullptr) return xnor_nn_error_invalid_input;
    const long long n = (long long)c->oc * c->ic * c->kh * c->kw;
    if (c->oc <= 0 || c->ic <= 0 || c->kh <= 0 || c->kw <= 0
            || n > XNOR_NN_HIP_NOALLOC_MAX_WEIGHTS) {
        fprintf(stderr, "xnor_nn_hip_binarize_weights_float_noalloc: %lld weights, the limit "
                "is %lld\n", n, (long long)XNOR_NN_HIP_NOALLOC_MAX_WEIGHTS);
        return xnor_nn_error_invalid_input;
    }
    // hipPointerGetAttributes allocates nothing; a host pointer handed to the kernels would be
    // a GPU memory fault
    if (!on_device(from) || !on_device(to)) {
        fprintf(stderr, "xnor_nn_hip_binarize_weights_float_noalloc: `from` and `to` must be "
                "device pointers\n");
        return xnor_nn_error_invalid_input;
    }
    float *parts = nullptr;
    if (weights_float_scratch(&parts) != hipSuccess) {
        (void)hipGetLastError();
        return xnor_nn_error_memory;
    }
    hipStream_t s = c->state ? state_of(c)->stream : nullptr;
    return launch_weights_float(from, to, (size_t)n, parts, s) == hipSuccess
        ? xnor_nn_success : xnor_nn_error_memory;
}

xnor_nn_status_t xnor_nn_hip_set_stream(const xnor_nn_convolution_t *c, void *stream) {
    if (!bcast_descriptor(c)) return xnor_nn_error_invalid_input;
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    hipStream_t to = static_cast<hipStream_t>(stream);
    // xnor_nn_binarize_weights_float keeps its partial sums with the descriptor: kernels of an
    // earlier call that are still under way on the old stream must be through with them
    // before a call on the new stream may overwrite them
    if (to != st->stream && st->float_parts != nullptr
            && hipStreamSynchronize(st->stream) != hipSuccess)
        return xnor_nn_error_memory;
    st->stream = to;
    return xnor_nn_success;
}

xnor_nn_status_t xnor_nn_hip_set_stage_fusion(const xnor_nn_convolution_t *c, int on) {
    if (!bcast_descriptor(c)) return xnor_nn_error_invalid_input;
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    st->fuse_stages = on != 0;
    return xnor_nn_success;
}

xnor_nn_status_t xnor_nn_hip_time_kernels(const xnor_nn_convolution_t *c, int capacity) {
    if (!bcast_descriptor(c) || capacity < 0 || capacity > 65536)
        return xnor_nn_error_invalid_input;
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    if (hipStreamSynchronize(st->stream) != hipSuccess) return xnor_nn_error_memory;
    if (!make_timer(st->time_binarize, capacity) || !make_timer(st->time_convolution, capacity)) {
        drop_timer(st->time_binarize); // never one stage timed and the other not
        drop_timer(st->time_convolution);
        return xnor_nn_error_memory;
    }
    return xnor_nn_success;
}

int xnor_nn_hip_kernel_times(const xnor_nn_convolution_t *c, int stage, float *ms, int max) {
    if (!bcast_descriptor(c) || ms == nullptr || max < 0) return -1;
    State *st = state_of(c);
    std::lock_guard<std::mutex> call(st->mu);
    KernelTimer *t = stage == xnor_nn_operation_binarize_data ? &st->time_binarize
        : stage == xnor_nn_operation_convolution_forward ? &st->time_convolution : nullptr;
    if (t == nullptr) return -1;
    if (hipStreamSynchronize(st->stream) != hipSuccess) return -1;
    const size_t have = t->launches < t->ring.size() ? t->launches : t->ring.size();
    const size_t first = t->launches - have; // oldest launch still in the ring
    int n = 0;
    for (size_t i = first; i < t->launches && n < max; i++) {
        const KernelEvents &e = t->ring[i % t->ring.size()];
        if (hipEventElapsedTime(&ms[n], e.start, e.stop) != hipSuccess) {
            (void)hipGetLastError();
            return -1;
        }
        n++;
    }
    t->launches = 0;
    return n;
}

xnor_nn_status_t xnor_nn_hip_synchronize(const xnor_nn_convolution_t *c) {
    if (!bcast_descriptor(c)) return xnor_nn_error_invalid_input;
    return hipStreamSynchronize(state_of(c)->stream) == hipSuccess ? xnor_nn_success
                                                                   : xnor_nn_error_memory;
}

int xnor_nn_hip_canonical_bici(const xnor_nn_convolution_t *c) {
    return (c->ic * c->kh * c->kw < 32767) ? 2 : 4;
}

xnor_nn_status_t xnor_nn_hip_export_bin_src(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, void *dst, size_t dst_bytes) {
    if (!bcast_descriptor(c) || !res[xnor_nn_resource_bin_src] || !dst)
        return xnor_nn_error_invalid_input;
    const Geometry &g = state_of(c)->g;
    const int bici = canonical_bici(g);
    const int abic = div_up(div_up(g.ic, 8), bici) * bici;
    if (dst_bytes != (size_t)g.npix_in * abic) return xnor_nn_error_invalid_input;
    std::vector<uint32_t> words((size_t)g.npix_in * g.xw);
    xnor_nn_status_t rc = to_host(c, res[xnor_nn_resource_bin_src], words.data(),
            words.size() * 4);
    if (rc != xnor_nn_success) return rc;
    unsigned char *out = static_cast<unsigned char *>(dst);
    for (size_t p = 0; p < g.npix_in; p++)
        for (int b = 0; b < abic; b++) {
            const int j = b / 4;
            out[p * abic + b] = j < g.xw
                ? (unsigned char)(words[p * g.xw + j] >> (24 - 8 * (b % 4))) : 0;
        }
    return xnor_nn_success;
}

xnor_nn_status_t xnor_nn_hip_export_bin_weights(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int oci, void *dst, size_t dst_bytes) {
    if (!bcast_descriptor(c) || !res[xnor_nn_resource_bin_weights] || !dst || oci <= 0)
        return xnor_nn_error_invalid_input;
    const Geometry &g = state_of(c)->g;
    if (g.oc % oci != 0) return xnor_nn_error_invalid_input;
    const int bici = canonical_bici(g);
    const int ico = div_up(div_up(g.ic, bici), 8);
    const int taps = g.kh * g.kw;
    const size_t need = (size_t)(g.oc / oci) * taps * ico * oci * bici;
    if (dst_bytes != need) return xnor_nn_error_invalid_input;
    std::vector<uint32_t> words((size_t)g.ocb * taps * g.xw * g.q);
    xnor_nn_status_t rc = to_host(c, res[xnor_nn_resource_bin_weights], words.data(),
            words.size() * 4);
    if (rc != xnor_nn_success) return rc;
    unsigned char *out = static_cast<unsigned char *>(dst);
    for (int oc = 0; oc < g.oc; oc++)
        for (int t = 0; t < taps; t++)
            for (int b = 0; b < ico * bici; b++) {
                const int j = b / 4;
                unsigned char byte = 0xFF; // bytes past the device words: channels >= IC
                if (j < g.xw) {
                    const uint32_t w = words[(((size_t)(oc / g.q) * taps + t) * g.xw + j) * g.q
                        + oc % g.q];
                    byte = (unsigned char)(w >> (24 - 8 * (b % 4)));
                }
                const size_t at = ((((size_t)(oc / oci) * taps + t) * ico + b / bici) * oci
                        + oc % oci) * bici + b % bici;
                out[at] = byte;
            }
    return xnor_nn_success;
}

xnor_nn_status_t xnor_nn_hip_export_floats(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int slot, float *dst, size_t dst_bytes) {
    if (!bcast_descriptor(c) || !dst) return xnor_nn_error_invalid_input;
    if (slot != xnor_nn_resource_alpha && slot != xnor_nn_resource_a
            && slot != xnor_nn_resource_k)
        return xnor_nn_error_invalid_input;
    if (!res[slot] || dst_bytes != c->resource_size[slot]) return xnor_nn_error_invalid_input;
    if (slot == xnor_nn_resource_k) { // a deferred box filter has to run before K is read
        State *st = state_of(c);
        std::lock_guard<std::mutex> call(st->mu);
        xnor_nn_status_t rc = settle_k(st, static_cast<float *>(res[slot]));
        if (rc != xnor_nn_success) return rc;
    }
    return to_host(c, res[slot], dst, dst_bytes);
}

xnor_nn_status_t xnor_nn_hip_export_operations_count(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int32_t *dst, size_t dst_bytes) {
    if (!bcast_descriptor(c) || !dst || !res[xnor_nn_resource_operations_count]
            || dst_bytes != c->resource_size[xnor_nn_resource_operations_count])
        return xnor_nn_error_invalid_input;
    return to_host(c, res[xnor_nn_resource_operations_count], dst, dst_bytes);
}

xnor_nn_status_t xnor_nn_hip_forward_popcount(const xnor_nn_convolution_t *c,
        xnor_nn_resources_t res, int32_t *popc) {
    if (!bcast_descriptor(c) || res[xnor_nn_resource_bin_src] == nullptr
            || res[xnor_nn_resource_bin_weights] == nullptr || popc == nullptr)
        return xnor_nn_error_invalid_input;
    return run_convolution(c, res, popc, true);
}

xnor_nn_status_t xnor_nn_hip_plain_read(const void *device_buffer, size_t bytes,
        void *stream) {
    if (device_buffer == nullptr || bytes < 16 || ((size_t)device_buffer & 15) != 0
            || !on_device(device_buffer))
        return xnor_nn_error_invalid_input;
    return launch_plain_read(device_buffer, bytes, static_cast<hipStream_t>(stream))
            == hipSuccess ? xnor_nn_success : xnor_nn_error_memory;
}

xnor_nn_status_t xnor_nn_hip_mfma_only(int workgroups, int iterations, void *stream) {
    if (workgroups < 1 || workgroups > (1 << 20) || iterations < 1 || iterations > (1 << 20))
        return xnor_nn_error_invalid_input;
    return launch_mfma_only(workgroups, iterations, static_cast<hipStream_t>(stream))
            == hipSuccess ? xnor_nn_success : xnor_nn_error_memory;
}

xnor_nn_status_t xnor_nn_hip_device_info(int *compute_units, int *clock_khz) {
    int dev = 0, cus = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess
            || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess
            || hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, dev) != hipSuccess) {
        (void)hipGetLastError();
        return xnor_nn_error_memory;
    }
    if (compute_units) *compute_units = cus;
    if (clock_khz) *clock_khz = khz;
    return xnor_nn_success;
}

int xnor_nn_hip_kernel_name(const xnor_nn_convolution_t *c, int stage, char *buf,
        size_t buf_bytes) {
    if (!bcast_descriptor(c) || !buf || buf_bytes == 0) return 0;
    const Geometry &g = state_of(c)->g;
    const char *name = "";
    switch (stage) {
    case xnor_nn_operation_convolution_forward: name = convolution_kernel_name(g); break;
    case xnor_nn_operation_binarize_data: name = binarize_kernel_name(g); break;
    case xnor_nn_operation_calculate_k: name = "box_filter_kernel"; break;
    case xnor_nn_operation_binarize_weights: name = "pack_weights_kernel"; break;
    }
    snprintf(buf, buf_bytes, "%s", name);
    return (int)strlen(buf);
}

} // extern "C"
