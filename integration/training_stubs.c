/*
 * training_stubs.c - the device symbols a pjreddie/darknet tree built with -DGPU still references
 * from its host files once src/cuda.c, the CUDA translation units and cuBLAS are gone, and which
 * libdarknet_hip.so does not serve: everything only training, a recurrent / deconvolutional layer or
 * a class tree reaches.  Each one ends the process with a message that names it, the tree's own
 * convention for an unrecoverable condition (src/utils.c:253-258).
 *
 * This file includes none of the tree's headers on purpose: the stubs take no arguments (they never
 * return, so nothing reads them), which keeps the list a list.  The inference forward pass of the
 * conv-dominated cfgs calls none of them; tests/test_integration_link.py checks that this list is
 * exactly what the link of the tree needs beyond adapters.c and the library.
 *
 * Where each one lived in the tree:
 *   src/blas_kernels.cu        axpy, scal, add, mul, pow, const, constrain, supp, mask, scale_mask,
 *                              mult_add_into, weighted_sum, weighted_delta, fast_mean, fast_variance,
 *                              fast_mean_delta, fast_variance_delta, normalize_delta, backward_scale,
 *                              backward_bias, l1, l2, smooth_l1, softmax_x_ent, logistic_x_ent, wgan,
 *                              l2normalize, adam_update, softmax_tree
 *   src/activation_kernels.cu  gradient_array_gpu
 *   src/col2im_kernels.cu      col2im_gpu
 *   src/gemm.c:172-182         gemm_gpu: the cuBLAS wrapper.  The library has no BLAS-shaped entry on
 *                              purpose; connected and local layers are served by their own entry
 *                              points (forward_connected_stream_gpu / forward_convolutional_gpu,
 *                              forward_local_gpu), bound by replacing the bodies of
 *                              forward_connected_layer_gpu (src/connected_layer.c:286-303) and
 *                              forward_local_layer_gpu (src/local_layer.c:186-215)
 *   the CUDA translation units backward_* / update_* of convolutional, deconvolutional, maxpool,
 *                              avgpool, dropout; forward_deconvolutional_layer_gpu
 */
#include <stdio.h>
#include <stdlib.h>

static void training_stub(const char *name)
{
    fprintf(stderr, "darknet-hip adapters: %s is not served (inference forward path only)\n", name);
    fflush(stderr);
    exit(-1);
}

#define DN_NOT_SERVED(name) void name(void) { training_stub(#name); }

/* BLAS-1 and element-wise kernels of the update, recurrent and loss code */
DN_NOT_SERVED(axpy_gpu)
DN_NOT_SERVED(scal_gpu)
DN_NOT_SERVED(add_gpu)
DN_NOT_SERVED(mul_gpu)
DN_NOT_SERVED(pow_gpu)
DN_NOT_SERVED(const_gpu)
DN_NOT_SERVED(constrain_gpu)
DN_NOT_SERVED(supp_gpu)
DN_NOT_SERVED(mask_gpu)
DN_NOT_SERVED(scale_mask_gpu)
DN_NOT_SERVED(mult_add_into_gpu)
DN_NOT_SERVED(weighted_sum_gpu)
DN_NOT_SERVED(weighted_delta_gpu)
/* batch-norm statistics and gradients */
DN_NOT_SERVED(fast_mean_gpu)
DN_NOT_SERVED(fast_variance_gpu)
DN_NOT_SERVED(fast_mean_delta_gpu)
DN_NOT_SERVED(fast_variance_delta_gpu)
DN_NOT_SERVED(normalize_delta_gpu)
DN_NOT_SERVED(backward_scale_gpu)
DN_NOT_SERVED(backward_bias_gpu)
/* losses and the l2norm layer */
DN_NOT_SERVED(l1_gpu)
DN_NOT_SERVED(l2_gpu)
DN_NOT_SERVED(smooth_l1_gpu)
DN_NOT_SERVED(softmax_x_ent_gpu)
DN_NOT_SERVED(logistic_x_ent_gpu)
DN_NOT_SERVED(wgan_gpu)
DN_NOT_SERVED(l2normalize_gpu)
/* gradients, optimiser, class tree */
DN_NOT_SERVED(gradient_array_gpu)
DN_NOT_SERVED(adam_update_gpu)
DN_NOT_SERVED(softmax_tree)
/* backward / update of the layers whose forward adapters.c provides; the deconvolutional layer */
DN_NOT_SERVED(backward_convolutional_layer_gpu)
DN_NOT_SERVED(update_convolutional_layer_gpu)
DN_NOT_SERVED(backward_maxpool_layer_gpu)
DN_NOT_SERVED(backward_avgpool_layer_gpu)
DN_NOT_SERVED(backward_dropout_layer_gpu)
DN_NOT_SERVED(forward_deconvolutional_layer_gpu)
DN_NOT_SERVED(backward_deconvolutional_layer_gpu)
DN_NOT_SERVED(update_deconvolutional_layer_gpu)
DN_NOT_SERVED(col2im_gpu)
/* the cuBLAS wrapper */
DN_NOT_SERVED(gemm_gpu)
