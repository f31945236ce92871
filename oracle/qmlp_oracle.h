/*
 * CPU oracle for the fused input-encoding + MLP path of QuickMLP.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C, fp32 restatement of the
 * evaluation the reference's own tests use as ground truth. Nothing in the
 * shipped library may include, link or call it; only the test-suite, the
 * smoke check and the benchmark's CPU-baseline leg do, and there only as the
 * checker / the reported baseline.
 *
 * What each function follows in the reference (paths under the reference root):
 *   qo_hashgrid_init      src_cpp/src/encoding_hashgrid.cpp:41-97   (level table)
 *   qo_index_dense/hash   src_cpp/include/qmlp/kernels/encoding_hashgrid.cuh:17-60
 *   qo_hashgrid_corners   encoding_hashgrid.cuh:72-85,174-215,267-285 (corner set + weights)
 *   qo_hashgrid_forward   encoding_hashgrid.cuh:92-115,267-336
 *   qo_hashgrid_adjoint   encoding_hashgrid.cuh:117-166,187-241,345-422
 *   qo_line_forward/adjoint  src_cpp/include/qmlp/kernels/encoding_line_integration.cuh:26-166
 *                         (slab test :26-49, march + blending :62-100, adjoint :103-163)
 *   identity encoding     src_cpp/include/qmlp/kernels/encoding_identity.cuh:12-39
 *   activations           src_cpp/include/qmlp/builtin-activations.json:1-21,
 *                         tests_cpp/test_against_eigen.h:31-87
 *   qo_network_forward    tests_cpp/test_against_eigen1.cpp:162-172,
 *                         tests_cpp/test_against_eigen2.cpp:134-150  (act(W X^T + b))
 *   qo_network_backward   tests_cpp/test_against_eigen1.cpp:187-213,
 *                         tests_cpp/test_against_eigen2.cpp:166-207
 *                         (dpre = act'(pre,dY), db = rowsum, dW = dpre in^T, dX = W^T dpre)
 *   padding rules         tests_cpp/test_against_eigen.h:167-191,
 *                         src_cpp/src/fused_network.cpp:147-206
 *
 * Precision rule: parameters are handed over as floats that the caller has
 * already rounded to fp16 where the GPU stores fp16; everything else is fp32
 * (round_mode 0). round_mode 1 additionally rounds at the fp16 rounding points
 * of the device pipeline (encoded features, pre-activations, activations,
 * adjoints between layers); it is used for tighter secondary checks only.
 *
 * Pin status: every function here is pinned by tests/test_oracle_*.py against
 * closed forms, hand-computed known answers, torch.nn.functional.linear +
 * autograd, torch grid_sample, brute force and finite differences.
 * Deliberate divergence from the reference: the grid input gradient includes
 * the (resolution-1) chain-rule factor the reference omits
 * (encoding_hashgrid.cuh:232,238,414-420); pass res_factor=0 to get the
 * reference's formula. The line integration takes no sample for rays whose
 * parameter interval is unbounded or holds 2^20 steps or more, where the
 * reference's loop would not end.
 */
#ifndef QMLP_ORACLE_H
#define QMLP_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QO_MAX_LEVELS 32
#define QO_MAX_DIM 6
#define QO_MAX_ENCODINGS 8
#define QO_MAX_LAYERS 16

enum { QO_ACT_RELU = 0, QO_ACT_CELU = 1, QO_ACT_SINE = 2, QO_ACT_IDENTITY = 3,
       QO_ACT_SINE_FREQ = 4 /* z = sin(param*x) */ };
enum { QO_CONCAT = 0, QO_ADD = 1 };
enum { QO_ENC_IDENTITY = 0, QO_ENC_HASHGRID = 1, QO_ENC_LINE = 2 };
enum { QO_BLEND_ADDITIVE = 0, QO_BLEND_AVERAGE = 1 };
enum { QO_GRAD_INPUT = 1, QO_GRAD_WEIGHTS = 2, QO_GRAD_ENCODINGS = 4 };

typedef struct {
    int start_in, dim, n_levels, n_feat, combination;
    int n_params;
    int mem_offset[QO_MAX_LEVELS];
    int resolution[QO_MAX_LEVELS];
    int hash_size[QO_MAX_LEVELS];
    int hashed[QO_MAX_LEVELS];
    float bb_min[QO_MAX_DIM];
    float bb_inv[QO_MAX_DIM];
} qo_hashgrid;

/* Fixed-step line integration through a 3-D child grid (whose start_in must be 0): ray
 * start in columns [start_in, start_in+3), direction in the 3 columns after. */
typedef struct {
    int start_in;
    int blending;
    float stepsize;
    float bb_min[3];
    float bb_size[3];
} qo_line;

typedef struct {
    int n_in;                              /* columns of the raw input */
    int n_enc;
    int enc_kind[QO_MAX_ENCODINGS];
    int enc_start[QO_MAX_ENCODINGS];       /* identity: first input column */
    int enc_nin[QO_MAX_ENCODINGS];         /* identity: number of columns */
    const qo_hashgrid* enc_grid[QO_MAX_ENCODINGS];
    const float* enc_table[QO_MAX_ENCODINGS];
    float* enc_grad[QO_MAX_ENCODINGS];     /* += ; may be NULL */
    const qo_line* enc_line[QO_MAX_ENCODINGS]; /* QO_ENC_LINE: the march; enc_grid is its child */
    int n_layers;
    int cin[QO_MAX_LAYERS];                /* padded widths (multiples of 16) */
    int cout[QO_MAX_LAYERS];
    int act[QO_MAX_LAYERS];
    float act_param[QO_MAX_LAYERS];
    /* optional: one activation per (padded) output channel, cout[l] entries; NULL = act[l] for
     * all channels (the per-channel lists of src_cpp/src/fused_network.cpp:112-125) */
    const int* act_channel[QO_MAX_LAYERS];
    const float* act_param_channel[QO_MAX_LAYERS];
    const float* W[QO_MAX_LAYERS];         /* row-major (cout, cin) */
    const float* b[QO_MAX_LAYERS];         /* NULL if no bias */
    float* dW[QO_MAX_LAYERS];              /* += ; may be NULL */
    float* db[QO_MAX_LAYERS];              /* += ; may be NULL */
    int round_mode;
    int res_factor;                        /* 1: include (R-1) in grid input grads */
} qo_network;

float qo_round_half(float x);
void qo_round_half_array(float* x, long n);

int qo_hashgrid_init(qo_hashgrid* g, int start_in, int dim, int n_levels, int n_feat,
                     int log2_hashmap_size, int min_res, int max_res, int combination,
                     const float* bb_min, const float* bb_size);
int qo_hashgrid_num_outputs(const qo_hashgrid* g);
uint32_t qo_index_dense(int dim, const uint32_t* pos, uint32_t resolution);
uint32_t qo_index_hash(int dim, const uint32_t* pos);
/* element offset (memoryOffset + idx*F) of feature 0 and the interpolation weight of
 * every corner: idx/w have shape [N][n_levels][2^dim]. */
void qo_hashgrid_corners(const qo_hashgrid* g, const float* x, long N, long x_stride,
                         uint32_t* idx, float* w);
void qo_hashgrid_forward(const qo_hashgrid* g, const float* table, const float* x, long N,
                         long x_stride, float* out, long out_stride);
void qo_hashgrid_adjoint(const qo_hashgrid* g, const float* table, const float* x, long N,
                         long x_stride, const float* adj_out, long adj_out_stride,
                         float* adj_x, long adj_x_stride, float* grad_table, int res_factor);

void qo_line_forward(const qo_line* line, const qo_hashgrid* child, const float* table, const float* x,
                     long N, long x_stride, float* out, long out_stride);
void qo_line_adjoint(const qo_line* line, const qo_hashgrid* child, const float* table, const float* x,
                     long N, long x_stride, const float* adj_out, long adj_out_stride,
                     float* adj_x, long adj_x_stride, float* grad_table, int res_factor);

float qo_act_forward(int act, float param, float x);
float qo_act_adjoint(int act, float param, float x, float adjz);

int qo_network_encoded_channels(const qo_network* net);
/* out: (N, n_out) row-major. enc_out: NULL or (N, cin[0]). pre: NULL or array of n_layers
 * pointers to (N, cout[l]). */
void qo_network_forward(const qo_network* net, const float* X, long N, long x_stride,
                        float* out, int n_out, float* enc_out, float* const* pre);
/* adj_out: (N, n_out). adj_x: NULL or (N, n_in), accumulated. dpre: NULL or n_layers
 * pointers (N, cout[l]). flags: QO_GRAD_*. enc_out/pre come from qo_network_forward. */
void qo_network_backward(const qo_network* net, const float* X, long N, long x_stride,
                         const float* adj_out, int n_out, int flags,
                         const float* enc_out, float* const* pre,
                         float* adj_x, float* const* dpre);
int qo_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
