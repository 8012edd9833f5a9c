/*
 * C ABI of the hand-written LSTM cell kernels for AMD GPUs (libovl_lstm.so).
 *
 * The fused LSTM cell of the reference is an OVL operator written in the DSL (lstm/lstm.py:32-59 `lstm`,
 * lstm/lstm.py:62-105 `lstm_grad`, helpers `sig`, `sig_grad`, `tanh_grad` at lstm/lstm.py:14-29), generated and
 * compiled for one fixed shape per trace, and used by the reference's recurrent cell in place of TensorFlow's
 * sigmoid/tanh graph (lstm/rnn_cell.py:313-327).  These two entry points compute the same two functions with the
 * same float32 operations in the same order - so results equal the generated operator's, bit for bit - but take the
 * shape at run time and need no code generation or compiler on the machine that calls them:
 *
 *   reference interface                                              replaced by
 *   ---------------------------------------------------------------  -----------------------
 *   lstm(concat, c, forget_bias=fb) -> new_c, new_h                   ovl_lstm_forward
 *       lstm/lstm.py:32-59
 *   lstm_grad(concat, c, d_new_c, d_new_h, forget_bias=fb)            ovl_lstm_backward
 *       -> d_concat, d_c      lstm/lstm.py:62-105
 *
 * Layout: `concat` is [batch, 4 * units], the gate pre-activations side by side in the order input (i), candidate
 * (j), forget (f), output (o) (lstm/lstm.py:45-48); every other tensor is [batch, units]; all are dense, C-ordered
 * float32 in device memory.
 *
 *   new_c = c * sigmoid(f + forget_bias) + sigmoid(i) * tanh(j)          new_h = tanh(new_c) * sigmoid(o)
 *
 * Conventions: tensor memory belongs to the caller; the functions only enqueue one kernel on `hip_stream`
 * (a hipStream_t; NULL is the default stream) and return without synchronising; they allocate nothing.  They return
 * an ovl_status (ovl_launch.h): OVL_EINVAL for null pointers, zero sizes or more than 2^32 - 1 elements, OVL_EHIP
 * for a HIP error (text from ovl_lstm_last_error).  `fast_math` = 0 selects the float32 exp/tanh/division that
 * reproduce the host C library (the reference's results); 1 selects the device's hardware based routines (each call
 * within 2 units in the last place).  128-bit accesses are used when `units` is a multiple of 4 and every pointer is
 * 16-byte aligned, scalar accesses otherwise.
 */
#ifndef OVL_LSTM_H_
#define OVL_LSTM_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int ovl_lstm_forward(const float* concat, const float* c, float forget_bias, uint32_t batch, uint32_t units,
                     int32_t fast_math, float* new_c, float* new_h, void* hip_stream);

int ovl_lstm_backward(const float* concat, const float* c, const float* d_new_c, const float* d_new_h,
                      float forget_bias, uint32_t batch, uint32_t units, int32_t fast_math,
                      float* d_concat, float* d_c, void* hip_stream);

/* Text of the last error on the calling thread ("" if none). */
const char* ovl_lstm_last_error(void);

#ifdef __cplusplus
}
#endif

#endif  /* OVL_LSTM_H_ */
