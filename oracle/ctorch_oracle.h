/* TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's CPU-BASIC arithmetic.
 * See ctorch_oracle.c for what each function follows.  Not part of the shipped library. */
#ifndef CTORCH_ORACLE_H
#define CTORCH_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* forward, dispatched kernels */
void co_add(const float* a, const float* b, float* r, long n);
void co_sub(const float* a, const float* b, float* r, long n);
void co_mul(const float* a, const float* b, float* r, long n);
void co_div(const float* a, const float* b, float* r, long n);
void co_add_scalar_tensor(const float* a, const float* b1, float* r, long n);
void co_add_rowbcast(const float* a, const float* b, float* r, long rows, long cols);
void co_binary_rowbcast(int op, const float* a, const float* b, float* r, long rows, long cols);
void co_neg(const float* a, float* r, long n);
void co_relu(const float* a, float* r, long n);
void co_sin(const float* a, float* r, long n);
void co_cos(const float* a, float* r, long n);
void co_tanh(const float* a, float* r, long n);
void co_sigmoid(const float* a, float* r, long n);
void co_softmax(const float* x, float* y, long rows, long cols, int dim, int guard_zero_sum);
void co_matmul(const float* a, long as0, long as1, const float* b, long bs0, long bs1, float* c,
               long m, long n, long k);
float co_dot(const float* a, const float* b, long n);
float co_mse(const float* a, const float* b, long n);
float co_mae(const float* a, const float* b, long n);
float co_ce_onehot(const float* x, const float* t, long rows, long cols);
int co_ce_index(const float* x, const float* idx, long rows, long cols, float* out);

/* forward, host-inline arithmetic of the Tensor front-end */
float co_sum(const float* a, long n);
void co_scalar_add(const float* a, float s, float* r, long n);
void co_scalar_mul(const float* a, float s, float* r, long n);
void co_scalar_div(const float* a, float s, float* r, long n);

/* backward arithmetic of the tape */
void co_fill(float* r, float v, long n);
void co_accumulate(float* grad, const float* val, long n);
void co_adjust_row0(const float* g, float* r, long rows, long cols);
void co_colsum_f64(const float* g, double* r, long rows, long cols);
void co_relu_bwd(const float* x, const float* g, float* dx, long n);
void co_sigmoid_bwd(const float* x, const float* g, float* dx, long n);
void co_tanh_bwd(const float* x, const float* g, float* dx, long n);
void co_sin_bwd(const float* x, const float* g, float* dx, long n);
void co_cos_bwd(const float* x, const float* g, float* dx, long n);
void co_softmax_bwd(const float* y, const float* g, float* dx, long rows, long cols, int dim);
void co_mse_bwd(const float* p, const float* t, float g, float* dp, long n);
void co_mae_bwd(const float* p, const float* t, float g, float* dp, long n);
void co_ce_bwd_onehot(const float* x, const float* t, float g, float* dx, long rows, long cols);
void co_ce_bwd_index(const float* x, const float* idx, float g, float* dx, long rows, long cols);
void co_div_bwd_a(const float* g, const float* b, float* da, long n);
void co_div_bwd_b(const float* a, const float* b, const float* g, float* db, long n);
int co_any_abs_lt_eps(const float* b, long n);

int co_adjust_grad_shape(const float* g, const long* gs, int gr, float* out, const long* ts, int tr);
int co_broadcast_reduce(const float* g, const long* gs, int gr, float* out, const long* ts, int tr);

/* methods the reference declares and never defines (pinned by mathematics) */
void co_unary_ext(int op, const float* a, float p, float* r, long n);
void co_unary_ext_bwd(int op, const float* v, const float* g, float p, float* dx, long n);
void co_reduce_dim(int kind, const float* x, float* out, int* index, float* mean_out, long outer, long len, long inner, int ddof);
void co_reduce_dim_bwd(int kind, const float* x, const float* y, const int* index, const float* mean, const float* g, float* dx,
                       long outer, long len, long inner, int ddof);
void co_log_softmax(const float* x, float* y, long rows, long cols, int dim);
void co_log_softmax_bwd(const float* y, const float* g, float* dx, long rows, long cols, int dim);

/* whole configurations, composed from the pieces above in the reference's op order */
void co_chain(const float* a, const float* b, long n, float* s, float* ga, float* gb);
void co_mlp_step(const float* x, long B, long I, const float* W1, const float* b1, long H,
                 const float* W2, const float* b2, long C, const float* onehot, int strict_row0,
                 float* loss, float* logits, float* gW1, float* gb1, float* gW2, float* gb2);
void co_expr(const float* X, const float* R, const float* T, long rows, long cols, float* Y,
             float* mse, float* mae, float* gX, float* gR);

/* the MNIST demo's path (mnist/mnist.cpp, mnist/mnist_loader.cpp) */
void co_u8_to_unit(const unsigned char* src, float* dst, long n);
void co_onehot(const float* labels, float* out, long rows, long classes);
void co_sgd_step(float* p, const float* g, float lr, long n);
long co_count_correct(const float* pred, const float* labels, long rows, long classes);
void co_mnist_train(const float* images, const float* labels, long n_images, long I, long H1, long H2,
                    long C, float* W1, float* b1, float* W2, float* b2, float* W3, float* b3, long batch,
                    long steps, float lr, int strict_row0, int stale_snapshot, float* losses);
void co_mnist_predict(const float* x, long B, long I, long H1, long H2, long C, const float* W1,
                      const float* b1, const float* W2, const float* b2, const float* W3, const float* b3,
                      float* probs);

/* seeded input generator shared by tests and fixtures (not from the reference) */
void co_fill_uniform(float* r, long n, uint64_t seed, double lo, double hi);
void co_fill_normal(float* r, long n, uint64_t seed, double mean, double sigma);
void co_fill_int(float* r, long n, uint64_t seed, long range);

void co_compare(int cmp, const float* a, const float* b, float s, unsigned char* out, long n);
int co_cast_from_f32(const float* in, void* out, int dtype, long n);
int co_scalar_op_typed(const void* in, void* out, int dtype, int op, float s, long n);
int co_accumulate_typed(void* acc, const void* val, int dtype, long n);
void co_softmax_f64(const double* x, double* y, long rows, long cols, int dim);

/* extension: a straight-line per-element program of the operators above (see the .c file) */
int co_expr_run(const int* prog, const float* imm, int n, const float* const* in, int n_in, float* const* out, int n_out,
                long rows, long cols, int* status);

#ifdef __cplusplus
}
#endif
#endif
