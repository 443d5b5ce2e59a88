// The update rules of the eight algorithms as device functions, one rounding per reference op (compile the including file
// with -ffp-contract=off): shared by the streaming optimizer kernels and by kernels that finish a gradient and apply it to
// the parameter on the spot.
#pragma once
#include "common.hpp"

namespace sn {

// decayingAvg(avg, next, decay) = decay*avg + (1-decay)*next (math/alg/AllKernels.scala:541-544)
__device__ __forceinline__ float decaying_avg(float avg, float next, float d, float one_minus_d) {
  return d * avg + one_minus_d * next;
}

template <int KIND>
__device__ __forceinline__ void update_one(float& w, float g, float& s0, float& s1, float& s2, const OptScalars& p) {
  float delta;
  if constexpr (KIND == SN_OPT_SGD) {  // SGD.scala:15-25
    float v = (p.rate * g) - (p.b1 * s0);
    delta = p.nesterov ? (p.rate * g) - (p.b1 * v) : v;
    s0 = v;
  } else if constexpr (KIND == SN_OPT_ADAGRAD) {  // AdaGrad.scala:21-32
    float acc = s0 + g * g;
    float rates = p.rate / sqrtf(acc + p.eps);
    delta = rates * g;
    s0 = acc;
  } else if constexpr (KIND == SN_OPT_ADADELTA) {  // AdaDelta.scala:33-44
    float avg_grad = decaying_avg(s0, g * g, p.b1, p.one_minus_b1);
    delta = p.rate * ((sqrtf(s1 + p.eps) / sqrtf(avg_grad + p.eps)) * g);
    s1 = decaying_avg(s1, delta * delta, p.b1, p.one_minus_b1);
    s0 = avg_grad;
  } else if constexpr (KIND == SN_OPT_RMSPROP) {  // RMSProp.scala:24-32
    float avg_grad = decaying_avg(s0, g * g, p.b1, p.one_minus_b1);
    delta = (p.rate / sqrtf(avg_grad + p.eps)) * g;
    s0 = avg_grad;
  } else if constexpr (KIND == SN_OPT_ADAM) {  // Adam.scala:29-41
    float m = decaying_avg(s0, g, p.b1, p.one_minus_b1);
    float v = decaying_avg(s1, g * g, p.b2, p.one_minus_b2);
    delta = (p.rate / sqrtf(v / p.bc2 + p.eps)) * (m / p.bc1);
    s0 = m;
    s1 = v;
  } else if constexpr (KIND == SN_OPT_NADAM) {  // Nadam.scala:37-49
    float m = decaying_avg(s0, g, p.b1, p.one_minus_b1);
    float v = decaying_avg(s1, g * g, p.b2, p.one_minus_b2);
    float m_nesterov = (p.b1 * (m / p.bc1)) + (p.one_minus_b1 * (g / p.bc1));
    delta = m_nesterov / (sqrtf(v / p.bc2) + p.eps);
    s0 = m;
    s1 = v;
  } else if constexpr (KIND == SN_OPT_ADAMAX) {  // Adamax.scala:41-52
    float m1 = decaying_avg(s0, g, p.b1, p.one_minus_b1);
    float m2 = fmaxf(p.b2 * s1, p.one_minus_b2 * fabsf(g));
    delta = (p.rate * (m1 / p.bc1)) / (m2 + p.eps);
    s0 = m1;
    s1 = m2;
  } else {  // AMSGrad.scala:34-46
    float m = decaying_avg(s0, g, p.b1, p.one_minus_b1);
    float v_cur = decaying_avg(s1, g * g, p.b2, p.one_minus_b2);
    float v = fmaxf(s2, v_cur);
    delta = (p.rate * m) / (sqrtf(v) + p.eps);
    s0 = m;
    s1 = v_cur;
    s2 = v;
  }
  w = p.maximize ? w + delta : w - delta;  // Optimizer.scala:186: `if (minimizing) w - del else w + del`
}

template <int KIND>
constexpr int n_states() {
  return (KIND == SN_OPT_SGD || KIND == SN_OPT_ADAGRAD || KIND == SN_OPT_RMSPROP) ? 1 : (KIND == SN_OPT_AMSGRAD ? 3 : 2);
}

// the same by a run-time kind (kernels that are not compiled per algorithm)
__device__ __forceinline__ void update_any(int kind, float& w, float g, float& s0, float& s1, float& s2, const OptScalars& p) {
  switch (kind) {
    case SN_OPT_SGD: update_one<SN_OPT_SGD>(w, g, s0, s1, s2, p); break;
    case SN_OPT_ADAGRAD: update_one<SN_OPT_ADAGRAD>(w, g, s0, s1, s2, p); break;
    case SN_OPT_ADADELTA: update_one<SN_OPT_ADADELTA>(w, g, s0, s1, s2, p); break;
    case SN_OPT_RMSPROP: update_one<SN_OPT_RMSPROP>(w, g, s0, s1, s2, p); break;
    case SN_OPT_ADAM: update_one<SN_OPT_ADAM>(w, g, s0, s1, s2, p); break;
    case SN_OPT_NADAM: update_one<SN_OPT_NADAM>(w, g, s0, s1, s2, p); break;
    case SN_OPT_ADAMAX: update_one<SN_OPT_ADAMAX>(w, g, s0, s1, s2, p); break;
    default: update_one<SN_OPT_AMSGRAD>(w, g, s0, s1, s2, p); break;
  }
}

}  // namespace sn
