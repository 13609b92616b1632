// Builds the reference's own host rotation (src/q_rope.h:3-35, rope_cpu) from where it lies under
// /root/reference into oracle/_ref/.  Only this shim is ours; no reference source is copied.
// TEST INFRASTRUCTURE ONLY.
#include REF_Q_ROPE_H

extern "C" void ref_rope_cpu_f32(float* rq, const float* q, const float* cosv, const float* sinv,
                                 int F, int W, int Hq, int S, int E, int R) {
    rope_cpu<float>(rq, q, cosv, sinv, F, W, Hq, S, E, R);
}
