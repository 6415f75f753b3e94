/*
 * C++ convenience wrapper over the C API (MI355X / gfx950 build).
 *
 * Same class, constructor arguments and methods as the reference wrapper
 * (reference include/xnor_nn.hpp:11-68), so callers such as the Caffe layer
 * (reference external/caffe/src/caffe/layers/xnor_nn_conv_layer.cpp:46-66) compile
 * unchanged.  `weights`, `src` and `dst` may be host or device pointers.
 */
#ifndef XNOR_NN_HPP
#define XNOR_NN_HPP

#include <stdexcept>
#include <string>

#include "xnor_nn.h"

namespace xnor_nn {

class Convolution {
public:
    /* init -> allocate device resources -> binarize the weights once
     * (reference include/xnor_nn.hpp:13-29). */
    Convolution(const xnor_nn_algorithm_t algorithm,
            const xnor_nn_tensor_format_t src_fmt,
            const xnor_nn_tensor_format_t weights_fmt,
            const xnor_nn_tensor_format_t dst_fmt,
            int MB, int OC, int IC, int IH, int IW,
            int KH, int KW, int SH, int SW, int PH, int PW,
            const void *weights) : res_{nullptr} {
        raise_unless_ok(xnor_nn_init_convolution(&conv_, algorithm,
                src_fmt, weights_fmt, dst_fmt,
                MB, OC, IC, IH, IW, KH, KW, SH, SW, PH, PW));
        raise_unless_ok(xnor_nn_allocate_resources(&conv_, res_));
        change_weights(weights);
    }

    Convolution(const Convolution &) = delete;
    Convolution &operator=(const Convolution &) = delete;

    ~Convolution() {
        xnor_nn_free_resources(res_);
        xnor_nn_destroy_convolution(&conv_);
    }

    /* Re-pack sign bits, alpha and the per-pixel operation counts for a new weight set
     * (reference include/xnor_nn.hpp:36-39). */
    void change_weights(const void *weights) {
        res_[xnor_nn_resource_user_weights] = const_cast<void *>(weights);
        raise_unless_ok(conv_.binarize_weights(&conv_, res_));
    }

    /* Float sign(w)*mean(w) weights for a framework's backward pass
     * (reference include/xnor_nn.hpp:41-43). */
    void binarizeWeightsFloat(const void *from, void *to) {
        xnor_nn_binarize_weights_float(&conv_,
                static_cast<const float *>(from), static_cast<float *>(to));
    }

    /* One forward pass = binarize_data, calculate_k, forward, in that order
     * (reference include/xnor_nn.hpp:45-53). */
    void forward(const void *src, void *dst) {
        res_[xnor_nn_resource_user_src] = const_cast<void *>(src);
        res_[xnor_nn_resource_user_dst] = dst;
        raise_unless_ok(conv_.binarize_data(&conv_, res_));
        raise_unless_ok(conv_.calculate_k(&conv_, res_));
        raise_unless_ok(conv_.forward(&conv_, res_));
        res_[xnor_nn_resource_user_src] = nullptr;
        res_[xnor_nn_resource_user_dst] = nullptr;
    }

    /* Access for callers that want the stream / export helpers of xnor_nn_hip.h. */
    const xnor_nn_convolution_t *descriptor() const { return &conv_; }
    void **resources() { return res_; }

private:
    xnor_nn_convolution_t conv_;
    xnor_nn_resources_t res_;

    /* The reference throws a heap-allocated std::runtime_error *pointer*
     * (reference include/xnor_nn.hpp:62-67); kept so existing catch sites still match. */
    static void raise_unless_ok(xnor_nn_status_t st) {
        if (st == xnor_nn_success) return;
        char text[16] = {0};
        xnor_nn_get_status_message(text, st);
        throw new std::runtime_error{std::string(text)};
    }
};

} // namespace xnor_nn
#endif // XNOR_NN_HPP
