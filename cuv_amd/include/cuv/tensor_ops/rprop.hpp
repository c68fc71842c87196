// learn_step_weight_decay(): the gradient-descent step with L2 weight decay.
//
// Mirrors src/cuv/tensor_ops/rprop.hpp:127-128,150-154 of the reference
// (bodies in src/cuv/tensor_ops/rprop.cu:148-156,324-346) for
// dev_memory_space: same signature and preconditions, result visible on
// return.  For a DIA weight matrix call it on W.vec() and dW.vec().  This
// tree has no host_memory_space twin of it (the reference's is rprop.cu:148-156 on host tensors).
#ifndef __CUV_RPROP_HPP__
#define __CUV_RPROP_HPP__

#include <cuv/basics/tensor.hpp>

namespace cuv {

/// W = (1 - decay*learnrate) * W - learnrate * dW  (sparsedecay is accepted and ignored, as in the reference)
template <class L>
inline void learn_step_weight_decay(tensor<float, dev_memory_space, L> &W, const tensor<float, dev_memory_space, L> &dW,
                                    const float &learnrate, const float &decay = 0.0f, const float &sparsedecay = 0.0f)
{
    (void)sparsedecay;
    cuvAssert(dW.ptr());
    cuvAssert(W.ptr());
    cuvAssert(W.size() == dW.size());
    checkDiaCall(cuvdia_learn_step_weight_decay_f32(W.ptr(), dW.ptr(), (long long)W.size(), learnrate, decay, NULL),
                 "cuvdia_learn_step_weight_decay_f32");
    cuvSafeCall(hipStreamSynchronize(NULL));
}

/// m = momentum_weight*momentum - learnrate*(dW + decay*W); W += m; momentum = m  (sparsedecay ignored, as in the
/// reference's kernel)
template <class L>
inline void learn_step_weight_decay_momentum(tensor<float, dev_memory_space, L> &W,
                                             tensor<float, dev_memory_space, L> &momentum,
                                             const tensor<float, dev_memory_space, L> &dW, const float &learnrate,
                                             const float &momentum_weight = 0.9f, const float &decay = 0.0f,
                                             const float &sparsedecay = 0.0f)
{
    (void)sparsedecay;
    cuvAssert(dW.ptr());
    cuvAssert(W.ptr());
    cuvAssert(W.size() == dW.size());
    cuvAssert(W.size() == momentum.size());
    checkDiaCall(cuvdia_learn_step_weight_decay_momentum_f32(W.ptr(), momentum.ptr(), dW.ptr(), (long long)W.size(),
                                                             learnrate, momentum_weight, decay, NULL),
                 "cuvdia_learn_step_weight_decay_momentum_f32");
    cuvSafeCall(hipStreamSynchronize(NULL));
}

}  // namespace cuv
#endif
