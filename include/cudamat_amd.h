/*
 * C ABI of the MI355X matrix backend (libcudamat.so).
 *
 * Every entry point keeps the name, argument order, argument meaning and error
 * code of the function it replaces in the reference's cudamat/cudamat.cu (cited
 * per group as file:line), so the reference's cudamat.py binds it unchanged
 * through ctypes.  All matrices are fp32, column-major, leading dimension
 * size[0], no padding.  Work is queued on the NULL HIP stream; only the calls
 * that hand a value back to the host (copy_to_host, vdot, euclid_norm,
 * cuda_sync_threads) wait for the device.
 */
#ifndef CUDAMAT_AMD_H_
#define CUDAMAT_AMD_H_

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes: cudamat/cudamat.cuh:1-9. */
#define ERROR_INCOMPATIBLE_DIMENSIONS -1
#define CUBLAS_ERROR -2
#define CUDA_ERROR -3
#define VIEW_ERROR -4
#define ERROR_TRANSPOSED -5
#define ERROR_GENERIC -6
#define ERROR_TRANSPOSEDNESS -7
#define ERROR_NOT_ON_DEVICE -8
#define ERROR_UNSUPPORTED -9

/* Matrix handle: cudamat/cudamat.cuh:21-29 (ctypes mirror cudamat.py:126-133). */
typedef struct cudamat {
  float* data_host;
  float* data_device;
  int on_device;
  int on_host;
  int size[2];
  int is_trans; /* 0 or 1 */
  int owns_data;
} cudamat;

/* RNG state: cudamat/cudamat.cuh:31-34.  12288 multipliers and 12288 64-bit words. */
typedef struct rnd_struct {
  unsigned int* dev_mults;
  unsigned long long* dev_words;
} rnd_struct;

/* Compressed-sparse-row matrix handle: cudamat/cudamat.cuh:36-50.  indptr has
 * size[0] + 1 entries, indices and data nnz entries each. */
typedef struct sparse_data {
  int* indices;
  int* indptr;
  float* data;
} sparse_data;

typedef struct cudamat_sparse {
  sparse_data data_host;
  sparse_data data_device;
  int on_device;
  int on_host;
  int size[2];
  int is_trans; /* 0 or 1 */
  int owns_data;
  int nnz;
} cudamat_sparse;

#define NUM_RND_STREAMS 12288 /* cudamat_kernels.cuh:4-6 */
#define NUM_RND_BURNIN 100    /* cudamat_kernels.cuh:18 */

/* ---- device / library lifetime: cudamat.cu:25-53, 103-105 ---- */
const char* get_last_cuda_error(void);
int cublas_init(void);
int cublas_shutdown(void);
int cuda_set_device(int deviceId);
void cuda_sync_threads(void);

/* ---- handle fields and views: cudamat.cu:87-101, 312-434 ---- */
int get_leading_dimension(cudamat* mat);
int get_nonleading_dimension(cudamat* mat);
void set_transpose(cudamat* mat, int is_trans);
int set_shape(cudamat* mat, unsigned int m, unsigned int n);
int reshape(cudamat* mat, unsigned int m, unsigned int n);
int get_slice(cudamat* source, cudamat* target, unsigned int first_col, unsigned int last_col);
int get_vector_slice(cudamat* source, cudamat* target, unsigned int first_ind, unsigned int last_ind);
void init_from_array(cudamat* mat, float* data, int m, int n);
void set_on_device(cudamat* mat);
int init_empty(cudamat* mat, int m, int n);

/* ---- allocation and transfers: cudamat.cu:109-123, 153-186, 217-229, 298-310 ---- */
int allocate_device_memory(cudamat* mat);
int copy_to_host(cudamat* mat);
int copy_to_device(cudamat* mat);
int copy_on_device(cudamat* mat1, cudamat* mat2);
int free_device_memory(cudamat* mat);

/* ---- row slices and transpose: cudamat.cu:231-296 ---- */
int get_row_slice(cudamat* source, cudamat* target, unsigned int start, unsigned int end);
int set_row_slice(cudamat* source, cudamat* target, unsigned int start, unsigned int end);
int copy_transpose(cudamat* source, cudamat* target);

/* ---- multiply-with-carry RNG: cudamat.cu:55-83, 437-588; kernels cudamat_kernels.cu:96-239 ---- */
int init_random(rnd_struct* rnd_state, int seed, char* cudamatpath);
int fill_with_rand(rnd_struct* rnd_state, cudamat* mat);
int fill_with_randn(rnd_struct* rnd_state, cudamat* mat);
int sample_bernoulli(rnd_struct* rnd_state, cudamat* mat, cudamat* target);
int sample_bernoulli_tanh(rnd_struct* rnd_state, cudamat* mat, cudamat* target);
int sample_poisson(rnd_struct* rnd_state, cudamat* mat, cudamat* target);
int sample_gaussian(rnd_struct* rnd_state, cudamat* mat, cudamat* target, float mult);
int perturb_energy(rnd_struct* rnd_state, cudamat* mat, cudamat* target);
int perturb_prob(rnd_struct* rnd_state, cudamat* mat, cudamat* target);
int dropout(rnd_struct* rnd_state, cudamat* mat, float dropprob, float val);

/* ---- broadcasts of a row / column / diagonal vector: cudamat.cu:592-877 ---- */
int add_col_vec(cudamat* mat, cudamat* vec, cudamat* target);
int add_col_mult(cudamat* mat, cudamat* vec, cudamat* target, float mult);
int add_row_vec(cudamat* mat, cudamat* vec, cudamat* target);
int add_row_mult(cudamat* mat, cudamat* vec, cudamat* target, float mult);
int mult_by_col_vec(cudamat* mat, cudamat* vec, cudamat* target);
int mult_by_row_vec(cudamat* mat, cudamat* vec, cudamat* target);
int div_by_col_vec(cudamat* mat, cudamat* vec, cudamat* target);
int div_by_row_vec(cudamat* mat, cudamat* vec, cudamat* target);
int mult_diagonal_scalar(cudamat* mat, float val, cudamat* target);
int add_diagonal_scalar(cudamat* mat, float val, cudamat* target);
int mult_diagonal(cudamat* mat, cudamat* vec, cudamat* target);
int add_diagonal(cudamat* mat, cudamat* vec, cudamat* target);

/* ---- comparisons and clamps: cudamat.cu:878-1146 ---- */
int less_than_eq(cudamat* mat1, cudamat* mat2, cudamat* target);
int less_than(cudamat* mat1, cudamat* mat2, cudamat* target);
int less_than_eq_scalar(cudamat* mat, float val, cudamat* target);
int less_than_scalar(cudamat* mat, float val, cudamat* target);
int greater_than_eq(cudamat* mat1, cudamat* mat2, cudamat* target);
int greater_than(cudamat* mat1, cudamat* mat2, cudamat* target);
int greater_than_eq_scalar(cudamat* mat, float val, cudamat* target);
int greater_than_scalar(cudamat* mat, float val, cudamat* target);
int upper_bound(cudamat* mat1, cudamat* mat2, cudamat* target);
int lower_bound(cudamat* mat1, cudamat* mat2, cudamat* target);
int upper_bound_scalar(cudamat* mat, float val, cudamat* target);
int lower_bound_scalar(cudamat* mat, float val, cudamat* target);

/* ---- reductions along an axis: cudamat.cu:1148-1315.
 * axis 0 reduces each column (the reference's only supported case).  axis 1,
 * which the reference answers with ERROR_UNSUPPORTED, reduces each row here with
 * the semantics of eigenmat/eigenmat.cc:617-731. ---- */
int max_by_axis(cudamat* mat, cudamat* target, int axis);
/* No counterpart in the reference.  max_by_axis for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): same kernels, same results, but the slice partials and arrival counters of
 * the axis-1 kernel sit in a fixed 260 KiB workspace inside the library's code object
 * (one copy per GPU, held until the process ends) and nothing is allocated or freed.
 * ERROR_UNSUPPORTED (-9) when the shape would need more than 65536 partial floats or 1024
 * row blocks with column slices.  Calls that overlap on one GPU race on the workspace. */
int max_by_axis_noalloc(cudamat* mat, cudamat* target, int axis);
int argmax_by_axis(cudamat* mat, cudamat* target, int axis);
int choose_max_by_axis(cudamat* mat, cudamat* target, int axis);
int choose_max_and_accumulate(cudamat* mat, cudamat* acc);
/* eigenmat.cc:733-760 (exported by the reference's CPU backend; its cudamat.py spells them as
 * dot() with a vector of ones, cudamat.py:724-748 and 1546-1577): target = sums of mat along
 * axis (0: one per column, 1: one per row; the other axis for a transposed mat), or
 * target += mult * sums.  The kernels of those dot() calls without the vector: same bits. */
int sum_by_axis(cudamat* mat, cudamat* target, int axis);
int add_sum_by_axis(cudamat* mat, cudamat* target, int axis, float mult);
/* eigenmat.cc:864 (sum of every element; cudamat.py:719-720 spells it vdot() with a vector of ones
 * as long as the matrix).  vdot's kernel without the vector, same bits; the error code comes back
 * the way vdot and euclid_norm hand it back. */
float sum_all(cudamat* mat, int* err_code);
int sqsum_by_axis(cudamat* mat, cudamat* target, int axis, float mult, float p);
int normlimit_by_axis(cudamat* mat, cudamat* target, int axis, float norm);

/* ---- unary math: cudamat.cu:1318-1669 ---- */
int sign(cudamat* mat, cudamat* target);
int apply_cos(cudamat* mat, cudamat* target);
int apply_sin(cudamat* mat, cudamat* target);
int apply_sigmoid(cudamat* mat, cudamat* target);
int apply_tanh(cudamat* mat, cudamat* target);
int apply_abs(cudamat* mat, cudamat* target);
int apply_log_1_plus_exp(cudamat* mat, cudamat* target);
int apply_log(cudamat* mat, cudamat* target, float tiny);
int apply_exp(cudamat* mat, cudamat* target);
int apply_ceil(cudamat* mat, cudamat* target);
int apply_floor(cudamat* mat, cudamat* target);
int apply_sqrt(cudamat* mat, cudamat* target);
int apply_pow(cudamat* mat, float pow, cudamat* target);
int apply_pow_matrix(cudamat* mat, cudamat* pow, cudamat* target);
int compute_cross_entropy(cudamat* mat, cudamat* p, cudamat* target, float tiny);
int compute_cross_entropy_bernoulli(cudamat* mat, cudamat* p, cudamat* target, float tiny);
int correct_preds(cudamat* mat, cudamat* p, cudamat* target, float cutoff);
int reciprocal(cudamat* mat, cudamat* target);

/* ---- dense contraction and BLAS-1: cudamat.cu:1671-1781, 2104-2118.
 * dot: target = beta*target + alpha*op(mat1)*op(mat2), op chosen by is_trans;
 * the target's is_trans flag is ignored (beta comes before alpha). ---- */
int dot(cudamat* mat1, cudamat* mat2, cudamat* target, float beta, float alpha);
float vdot(cudamat* mat1, cudamat* mat2, int* err_code);
int add_mult(cudamat* mat1, cudamat* mat2, float alpha);
float euclid_norm(cudamat* mat, int* err_code);
/* Extension, no counterpart in cudamat.cu: target = act(op(mat1)*op(mat2) + bias) in one
 * launch, bit-identical to dot -> add_col_vec -> apply_sigmoid / lower_bound_scalar(0) /
 * apply_tanh (the sequence of deepnet/dbm.py:95-105, deepnet/neuralnet.py:138-160).
 * bias: rows(target) x 1 or NULL; act: 0 none, 1 sigmoid, 2 max(x,0), 3 tanh. */
int dot_bias_act(cudamat* mat1, cudamat* mat2, cudamat* bias, cudamat* target, int act);
/* Extension, no counterpart in cudamat.cu: dot_bias_act followed by
 * sample_bernoulli(rnd_state, target, sample) (the up-pass of an RBM with its hidden sample,
 * deepnet/dbm.py:95-105), bit-identical to the two calls including the generator's state
 * afterwards; one launch for single-kernel products of at most 16 * 12288 outputs, the
 * separate kernels otherwise.  sample: target's shape, another buffer. */
int dot_bias_act_sample(rnd_struct* rnd_state, cudamat* mat1, cudamat* mat2, cudamat* bias, cudamat* target,
                        cudamat* sample, int act);

/* Extension, no counterpart in cudamat.cu: the parameter update of deepnet/parameter.py:80-106
 * in one pass, the same bits as the calls it replaces:
 *   w_delta.mult(momentum); [w_delta.add_mult(w, l2_decay);] [w_delta.add_mult_sign(w, l1_decay);]
 *   w_delta.add_mult(gradient); w.add_mult(w_delta, -epsilon); [gradient.assign(0)]
 * flags: bit 0 apply l2_decay, bit 1 apply l1_decay, bit 2 clear the gradient. */
int momentum_update(cudamat* w, cudamat* w_delta, cudamat* gradient, float momentum, float l2_decay, float l1_decay,
                    float epsilon, int flags);

/* Extension, no counterpart in cudamat.cu: momentum_update for count parameters in one
 * launch per 8 of them (the weights and biases of a net after a step, deepnet/neuralnet.py:
 * UpdateEdgeParams / UpdateLayerParams call parameter.py:80-106 once per parameter); every
 * argument is an array of count entries, results are the bits of count separate calls. */
int momentum_update_many(int count, cudamat** w, cudamat** w_delta, cudamat** gradient, const float* momentum,
                         const float* l2_decay, const float* l1_decay, const float* epsilon, const int* flags);


/* Extension, no counterpart in cudamat.cu: softmax(mat) -> probs, and from the stored probs
 * loss = -log(probs[label] + tiny) (1 x cols, may be NULL) and grad = probs - onehot(label)
 * (may be NULL) in the same launch: the bits of softmax -> get_softmax_cross_entropy ->
 * apply_softmax_grad (deepnet/softmax_layer.py:11-86).  probs may be mat itself. */
int softmax_ce_grad(cudamat* mat, cudamat* labels, cudamat* probs, cudamat* loss, cudamat* grad, float tiny);

/* ---- sparse (CSR) x dense: cudamat.cu:125-153, 188-213, 407-418, 1698-1727.
 * sparse_dot: target = beta*target + alpha * mat1 * mat2 with mat2 (k x n) and target
 * (m x n) read as plain column-major arrays (their is_trans flags are ignored, as in the
 * reference).  Unlike the reference, a target that is not m x n is refused (-1). ---- */
void init_from_sparse_array(cudamat_sparse* mat, float* data, int* indices, int* indptr, int m, int n, int nnz);
int allocate_device_memory_sparse(cudamat_sparse* mat);
int copy_sparse_to_device(cudamat_sparse* mat);
int sparse_dot(cudamat_sparse* mat1, cudamat* mat2, cudamat* target, float beta, float alpha);
/* Extension, no counterpart in cudamat.cu (which never frees a sparse matrix). */
int free_device_memory_sparse(cudamat_sparse* mat);

/* ---- binary elementwise and activation derivatives: cudamat.cu:1782-2030 ---- */
int add_mult_sign(cudamat* mat1, cudamat* mat2, float mult);
int add_elementwise(cudamat* mat1, cudamat* mat2, cudamat* target);
int subtract_elementwise(cudamat* mat1, cudamat* mat2, cudamat* target);
int divide_elementwise(cudamat* mat1, cudamat* mat2, cudamat* target);
int mult_elementwise(cudamat* mat1, cudamat* mat2, cudamat* target);
int apply_sin_deriv(cudamat* mat1, cudamat* mat2, cudamat* target);
int apply_cos_deriv(cudamat* mat1, cudamat* mat2, cudamat* target);
int apply_logistic_deriv(cudamat* mat1, cudamat* mat2, cudamat* target);
int apply_tanh_deriv(cudamat* mat1, cudamat* mat2, cudamat* target);
int apply_rectified_linear_deriv(cudamat* mat1, cudamat* mat2, cudamat* target);
int apply_rectified_linear_smooth_deriv(cudamat* mat1, cudamat* mat2, cudamat* target);

/* ---- scalar ops: cudamat.cu:2031-2102 ---- */
int assign_scalar(cudamat* mat, float alpha);
int mult_by_scalar(cudamat* mat, float alpha, cudamat* target);
int divide_by_scalar(cudamat* mat, float alpha, cudamat* target);
int add_scalar(cudamat* mat, float alpha, cudamat* target);

/* ---- column gather / scatter with float-encoded indices: cudamat.cu:2120-2189, 2295-2399 ---- */
int selectRows(cudamat* source, cudamat* target, cudamat* indices);
int swapColumns(cudamat* source, cudamat* target, cudamat* indices1, cudamat* indices2);
int setSelectedRows(cudamat* target, cudamat* source, cudamat* indices);
int generate_translations_big_var_off(cudamat* source, cudamat* target, cudamat* off_x, cudamat* off_y,
                                      int source_w, int target_w, int num_channels);
int blockify(cudamat* source, cudamat* target, int blocksize);
int accumulate_columns(cudamat* mat, cudamat* indices, cudamat* target, float mult, int avg);
int expand(cudamat* source, cudamat* indices, cudamat* target);
int expand_and_add(cudamat* source, cudamat* mat, cudamat* indices, cudamat* target, float mult);

/* ---- column softmax and its loss helpers: cudamat.cu:2192-2346 ---- */
int softmax(cudamat* mat, cudamat* target);
int softmax_overwrite(cudamat* mat);
int apply_softmax_grad(cudamat* mat, cudamat* labels, cudamat* target);
int get_softmax_correct(cudamat* mat, cudamat* labels, cudamat* target);
int get_softmax_cross_entropy(cudamat* mat, cudamat* labels, cudamat* target, float tiny);

/* ---- Extension: deferred epilogues.  dot() with alpha = 1, beta = 0 into an untransposed target holds
 * its launch back; add_col_vec(target, bias, target), then apply_sigmoid / apply_tanh /
 * lower_bound_scalar(.., 0, ..) in place, then sample_bernoulli(rnd, target, sample) are folded into that
 * launch while they follow it directly (the sequence of cudamat/examples/rbm_cudamat.py:46-70 and
 * deepnet/neuralnet.py:138-160); so are mult_elementwise(target, mask, target) and
 * apply_rectified_linear_deriv(target, state, target) directly behind the product (the backward pass of a layer
 * of rectified linear units with dropout, deepnet/neuralnet.py:203-222).  Any other
 * call launches what is held back first, so work is queued in
 * call order and results are those of the separate launches, bit for bit.  Likewise an in-place
 * mult_by_scalar is held back and the add_mult / add_mult_sign calls of a parameter update
 * (deepnet/parameter.py:80-106: w_delta *= momentum [; w_delta += l2 w] [; w_delta += l1 sign(w)] ;
 * w_delta += gradient ; w += -epsilon w_delta [; gradient = 0]) run as one pass when they spell it, and
 * updates that follow each other directly (up to eight, on arrays that do not overlap) as one launch.
 * A product with beta = 1 (add_dot, subtract_dot) of at most 128 terms waits for a second one of the
 * same shape into the same target, and up to four add_sum_by_axis calls along the rows onto at most two
 * vectors wait for each other (the statistics of cudamat/examples/rbm_cudamat.py:73-86: six calls, two
 * launches; a product that stays alone takes the sums along in its own launch where its kernel can: a weight
 * gradient and the bias gradient of its layer, deepnet/edge.py:236-242, layer.py:206-211); same bits, call order
 * kept wherever two calls touch the same memory.  fill_with_rand is held
 * back likewise: greater_than_scalar of that matrix in place and mult_elementwise of another matrix by it in
 * place (the dropout mask of deepnet/neuralnet.py:194-198) run with it as one pass, same draws and values.
 * Behind a held-back product with lower_bound_scalar(.., 0, ..) such a mask for the product's own target (at most
 * 16 * 12288 elements) is drawn in the product's epilogue: one launch for the six calls of a layer with dropout.
 * less_than(r, h, h) behind a held-back fill_with_rand(r) is one pass as well (cudamat/examples/rbm_cudamat.py:63-65).
 * softmax / softmax_overwrite are held back too: get_softmax_cross_entropy and apply_softmax_grad (into another
 * matrix) of the result join it and the three run as softmax_ce_grad's launch (deepnet/softmax_layer.py:25-62).
 * set_deferred_epilogues(0) makes every call launch at once; returns the previous setting (default 1).
 * launch_deferred() queues what is held back now and waits for nothing: for a caller that records its own
 * events on the library's stream (the NULL stream) or queues other work behind the library's. ---- */
int set_deferred_epilogues(int on);
int launch_deferred(void);

/* ---- Extension: the contrastive-divergence update of an RBM in one launch,
 *   W += eps (v h^T - v2 h2^T),  bv += eps (rowsums v - rowsums v2),  bh += eps (rowsums h - rowsums h2),
 * the six calls (two add_dot, four add_sums) of cudamat/examples/rbm_cudamat.py:57-85 and the statistics
 * of deepnet/edge.py:236-242, layer.py:206-211, as one product over the concatenated reduction with a
 * row of ones appended to each operand.  W nv x nh, v / v2 nv x batch, h / h2 nh x batch, bv nv x 1,
 * bh nh x 1 (bv, bh may be NULL); nothing transposed.  Equal to the six calls to rounding (for batches
 * of up to 128 the products and sums of the six calls themselves, in one launch: the same bits). ---- */
int cd_update(cudamat* W, cudamat* bv, cudamat* bh, cudamat* v, cudamat* h, cudamat* v2, cudamat* h2, float eps);

/* ---- HIP graphs: no counterpart in the reference.  graph_capture_begin() makes the library
 * record every following call (with the pointers and scalars it is given) into a HIP graph
 * instead of running it, until graph_capture_end() returns the executable graph;
 * graph_launch() replays it with one launch on the NULL stream.  For step sequences that are
 * bound by the cost of launching (the RBM and MLP steps).  Calls that wait for the device
 * and workspaces that would have to grow fail with their error codes while recording; run
 * the sequence once before recording it.
 * graph_capture_begin returns the capturing stream (NULL on failure).  graph_set_stream makes
 * the library queue on a stream of the caller's (capturing = 1: that stream is being captured by
 * the caller; NULL, 0 returns to the NULL stream). ---- */
void* graph_capture_begin(void);
void* graph_capture_end(void);
int graph_launch(void* graph_exec);
int graph_free(void* graph_exec);
int graph_set_stream(void* stream, int capturing);

#ifdef __cplusplus
}
#endif
#endif /* CUDAMAT_AMD_H_ */
