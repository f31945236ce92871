/*
 * CPU oracle (test infrastructure, see qmlp_oracle.h for what pins it and which
 * reference lines each function restates). Plain C99 + OpenMP, fp32.
 */
#include "qmlp_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ fp16 rounding */

/* float -> IEEE binary16 (round to nearest even) -> float, by bit manipulation. */
float qo_round_half(float x)
{
    union { float f; uint32_t u; } v;
    v.f = x;
    uint32_t sign = v.u & 0x80000000u;
    uint32_t a = v.u & 0x7fffffffu;
    if (a >= 0x7f800000u) return x;                 /* inf / nan */
    if (a >= 0x477ff000u) {                         /* >= 65520 rounds to inf */
        v.u = sign | 0x7f800000u;
        return v.f;
    }
    if (a < 0x38800000u) {                          /* below 2^-14: fp16 subnormal grid 2^-24 */
        union { float f; uint32_t u; } m;
        m.u = a;
        float q = m.f * 16777216.0f;                /* exact scaling by 2^24 */
        q = nearbyintf(q);                          /* default rounding = nearest even */
        m.f = q / 16777216.0f;
        v.u = sign | m.u;
        return v.f;
    }
    uint32_t lsb = (a >> 13) & 1u;                  /* keep 10 mantissa bits */
    a += 0x0fffu + lsb;
    a &= ~0x1fffu;
    v.u = sign | a;
    return v.f;
}

void qo_round_half_array(float* x, long n)
{
    for (long i = 0; i < n; ++i) x[i] = qo_round_half(x[i]);
}

int qo_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ hash grid: level table */

static size_t ipow_size(size_t x, unsigned p)
{
    size_t r = 1;
    for (unsigned i = 0; i < p; ++i) r *= x;
    return r;
}

/* encoding_hashgrid.cpp:41-97. All of it in double libm exactly as written there:
 * scale = exp((log(max)-log(min))/(L-1)); R_l = floor(min * pow(scale, l)). */
int qo_hashgrid_init(qo_hashgrid* g, int start_in, int dim, int n_levels, int n_feat,
                     int log2_hashmap_size, int min_res, int max_res, int combination,
                     const float* bb_min, const float* bb_size)
{
    if (dim < 1 || dim > QO_MAX_DIM) return -1;
    if (n_levels <= 0 || n_levels > QO_MAX_LEVELS) return -2;
    if (n_feat <= 0) return -3;
    if (min_res <= 0) return -4;
    if (max_res < min_res) return -5;
    memset(g, 0, sizeof(*g));
    g->start_in = start_in;
    g->dim = dim;
    g->n_levels = n_levels;
    g->n_feat = n_feat;
    g->combination = combination;
    for (int d = 0; d < dim; ++d) {
        float mn = bb_min ? bb_min[d] : -0.5f;
        float sz = bb_size ? bb_size[d] : 1.0f;
        g->bb_min[d] = mn;
        g->bb_inv[d] = 1.f / sz;
    }
    int hashmap_size = log2_hashmap_size > 0 ? (1 << log2_hashmap_size) : -1;
    double level_scale = 1;
    if (n_levels > 1)
        level_scale = exp((log((double)max_res) - log((double)min_res)) / (n_levels - 1));
    int num = 0;
    for (int l = 0; l < n_levels; ++l) {
        int resolution = (int)floor(min_res * pow(level_scale, l));
        size_t cells = ipow_size((size_t)resolution, (unsigned)dim);
        g->mem_offset[l] = num;
        g->resolution[l] = resolution;
        if (hashmap_size < 0 || cells <= (size_t)hashmap_size) {
            g->hash_size[l] = 0;
            g->hashed[l] = 0;
            num += (int)cells * n_feat;
        } else {
            g->hash_size[l] = hashmap_size;
            g->hashed[l] = 1;
            num += hashmap_size * n_feat;
        }
    }
    g->n_params = num;
    return 0;
}

int qo_hashgrid_num_outputs(const qo_hashgrid* g)
{
    return g->combination == QO_CONCAT ? g->n_levels * g->n_feat : g->n_feat;
}

/* ------------------------------------------------------------------ hash grid: indices */

static const uint32_t QO_HASH[QO_MAX_DIM] = { 1u, 43857811u, 83857661u, 73856093u, 19349663u, 834927u };

/* encoding_hashgrid.cuh:35-39,49-52: last coordinate fastest. */
uint32_t qo_index_dense(int dim, const uint32_t* pos, uint32_t resolution)
{
    uint32_t idx = pos[0];
    for (int d = 1; d < dim; ++d) idx = idx * resolution + pos[d];
    return idx;
}

/* encoding_hashgrid.cuh:41-45,54-58: xor of coordinate * per-dimension multiplier (uint32 wrap). */
uint32_t qo_index_hash(int dim, const uint32_t* pos)
{
    uint32_t h = 0;
    for (int d = 0; d < dim; ++d) h ^= pos[d] * QO_HASH[d];
    return h;
}

/* encoding_hashgrid.cuh:72-85: idx (* F) of one corner, without the level offset. */
static uint32_t corner_index(const qo_hashgrid* g, int l, const uint32_t* pos)
{
    uint32_t idx;
    if (g->hashed[l]) idx = qo_index_hash(g->dim, pos) % (uint32_t)g->hash_size[l];
    else idx = qo_index_dense(g->dim, pos, (uint32_t)g->resolution[l]);
    return idx * (uint32_t)g->n_feat;
}

/* encoding_hashgrid.cuh:279-287: cell corners and fractional position of one level. */
static void level_setup(const qo_hashgrid* g, int l, const float* pos,
                        uint32_t* iL, uint32_t* iH, float* f)
{
    const int rm1 = g->resolution[l] - 1;
    for (int d = 0; d < g->dim; ++d) {
        float p = pos[d] * (float)rm1;
        int ip = (int)p;
        int lo = ip < rm1 ? ip : rm1; if (lo < 0) lo = 0;
        int hi = (ip + 1) < rm1 ? (ip + 1) : rm1; if (hi < 0) hi = 0;
        iL[d] = (uint32_t)lo;
        iH[d] = (uint32_t)hi;
        f[d] = p - (float)iL[d];
    }
}

static void unit_position(const qo_hashgrid* g, const float* x, float* pos)
{
    for (int d = 0; d < g->dim; ++d)
        pos[d] = (x[d + g->start_in] - g->bb_min[d]) * g->bb_inv[d];
}

/* Corner c has bit d set iff dimension d uses the upper cell corner; dimension 0
 * toggles fastest and the weight is multiplied from dimension D-1 down to 0
 * (encoding_hashgrid.cuh:177-186,198-206). */
static void corner(const qo_hashgrid* g, int c, const uint32_t* iL, const uint32_t* iH,
                   const float* f, uint32_t* pos, float* w)
{
    float a = 1.f;
    for (int d = g->dim - 1; d >= 0; --d) {
        int hi = (c >> d) & 1;
        pos[d] = hi ? iH[d] : iL[d];
        a = a * (hi ? f[d] : (1 - f[d]));
    }
    *w = a;
}

void qo_hashgrid_corners(const qo_hashgrid* g, const float* x, long N, long x_stride,
                         uint32_t* idx, float* w)
{
    const int nc = 1 << g->dim;
#pragma omp parallel for schedule(static)
    for (long n = 0; n < N; ++n) {
        float pos[QO_MAX_DIM], f[QO_MAX_DIM];
        uint32_t iL[QO_MAX_DIM], iH[QO_MAX_DIM], cp[QO_MAX_DIM];
        unit_position(g, x + n * x_stride, pos);
        for (int l = 0; l < g->n_levels; ++l) {
            level_setup(g, l, pos, iL, iH, f);
            for (int c = 0; c < nc; ++c) {
                float a;
                corner(g, c, iL, iH, f, cp, &a);
                long o = (n * g->n_levels + l) * nc + c;
                idx[o] = (uint32_t)g->mem_offset[l] + corner_index(g, l, cp);
                w[o] = a;
            }
        }
    }
}

static void hashgrid_forward_point(const qo_hashgrid* g, const float* table, const float* x,
                                   float* out)
{
    const int nc = 1 << g->dim, F = g->n_feat;
    float pos[QO_MAX_DIM], f[QO_MAX_DIM];
    uint32_t iL[QO_MAX_DIM], iH[QO_MAX_DIM], cp[QO_MAX_DIM];
    float feat[64];
    unit_position(g, x, pos);
    for (int l = 0; l < g->n_levels; ++l) {
        level_setup(g, l, pos, iL, iH, f);
        for (int i = 0; i < F; ++i) feat[i] = 0.f;
        for (int c = 0; c < nc; ++c) {
            float a;
            corner(g, c, iL, iH, f, cp, &a);
            const float* t = table + (size_t)g->mem_offset[l] + corner_index(g, l, cp);
            for (int i = 0; i < F; ++i) feat[i] += a * t[i];
        }
        if (g->combination == QO_CONCAT) {
            for (int i = 0; i < F; ++i) out[l * F + i] = feat[i];
        } else {
            for (int i = 0; i < F; ++i) out[i] = (l == 0 ? 0.f : out[i]) + feat[i];
        }
    }
}

void qo_hashgrid_forward(const qo_hashgrid* g, const float* table, const float* x, long N,
                         long x_stride, float* out, long out_stride)
{
#pragma omp parallel for schedule(static)
    for (long n = 0; n < N; ++n)
        hashgrid_forward_point(g, table, x + n * x_stride, out + n * out_stride);
}

/* One point of the adjoint. grad_table gets w*adjFeat per corner (atomic when shared),
 * adj_x gets the analytic multilinear derivative times bb_inv (times (R-1) if res_factor). */
static void hashgrid_adjoint_point(const qo_hashgrid* g, const float* table, const float* x,
                                   const float* adj_out, float* adj_x, float* grad_table,
                                   int res_factor, int atomic)
{
    const int nc = 1 << g->dim, F = g->n_feat, D = g->dim;
    float pos[QO_MAX_DIM], f[QO_MAX_DIM], adj_pos[QO_MAX_DIM];
    uint32_t iL[QO_MAX_DIM], iH[QO_MAX_DIM], cp[QO_MAX_DIM];
    unit_position(g, x, pos);
    for (int d = 0; d < D; ++d) adj_pos[d] = 0.f;
    for (int l = 0; l < g->n_levels; ++l) {
        level_setup(g, l, pos, iL, iH, f);
        const float* adj_feat = adj_out + (g->combination == QO_CONCAT ? l * F : 0);
        float lvl[QO_MAX_DIM];
        for (int d = 0; d < D; ++d) lvl[d] = 0.f;
        for (int c = 0; c < nc; ++c) {
            float a;
            corner(g, c, iL, iH, f, cp, &a);
            size_t e = (size_t)g->mem_offset[l] + corner_index(g, l, cp);
            if (grad_table) {
                for (int i = 0; i < F; ++i) {
                    float v = a * adj_feat[i];
                    if (atomic) {
#pragma omp atomic
                        grad_table[e + i] += v;
                    } else {
                        grad_table[e + i] += v;
                    }
                }
            }
            if (adj_x) {
                float dot = 0.f;
                for (int i = 0; i < F; ++i) dot += adj_feat[i] * table[e + i];
                for (int d = 0; d < D; ++d) {
                    float prod = 1.f;
                    for (int e2 = D - 1; e2 >= 0; --e2) {
                        if (e2 == d) continue;
                        prod *= ((c >> e2) & 1) ? f[e2] : (1 - f[e2]);
                    }
                    float sign = ((c >> d) & 1) ? 1.f : -1.f;
                    lvl[d] += sign * prod * dot;
                }
            }
        }
        if (adj_x) {
            float s = res_factor ? (float)(g->resolution[l] - 1) : 1.f;
            for (int d = 0; d < D; ++d) adj_pos[d] += s * lvl[d];
        }
    }
    if (adj_x)
        for (int d = 0; d < D; ++d) adj_x[d + g->start_in] += adj_pos[d] * g->bb_inv[d];
}

void qo_hashgrid_adjoint(const qo_hashgrid* g, const float* table, const float* x, long N,
                         long x_stride, const float* adj_out, long adj_out_stride,
                         float* adj_x, long adj_x_stride, float* grad_table, int res_factor)
{
#pragma omp parallel for schedule(static)
    for (long n = 0; n < N; ++n)
        hashgrid_adjoint_point(g, table, x + n * x_stride, adj_out + n * adj_out_stride,
                               adj_x ? adj_x + n * adj_x_stride : NULL, grad_table,
                               res_factor, 1);
}

/* ------------------------------------------------------------------ line integration */

/* Slab test of encoding_line_integration.cuh:33-49: fp32, IEEE division (a zero direction
 * component gives +-inf or NaN, which fminf/fmaxf drop). */
static void line_intersect(const qo_line* line, const float* start, const float* dir,
                           float* tmin, float* tmax)
{
    float lo[3], hi[3];
    for (int d = 0; d < 3; ++d) {
        const float inv = 1.0f / dir[d];
        const float ta = (line->bb_min[d] - start[d]) * inv;
        const float tb = (line->bb_min[d] + line->bb_size[d] - start[d]) * inv;
        lo[d] = fminf(ta, tb);
        hi[d] = fmaxf(ta, tb);
    }
    *tmin = fmaxf(fmaxf(lo[0], lo[1]), lo[2]);
    *tmax = fminf(fminf(hi[0], hi[1]), hi[2]);
}

/* Steps in [tmin, tmax), or -2 (steps + 2 iterations are none) for rays that take no sample. Deliberate difference to the
 * reference, whose loop (encoding_line_integration.cuh:81) does not end for them: the
 * interval must be finite and hold fewer than 2^20 steps; the loops below also stop after
 * steps + 2 iterations. */
static int line_num_steps(float tmin, float tmax, float stepsize)
{
    const float steps = floorf((tmax - tmin) / stepsize);
    if (!(fabsf(tmin) < INFINITY && fabsf(tmax) < INFINITY) || !(steps < 1048576.f)) return -2;
    return (int)steps;
}

static void line_forward_point(const qo_line* line, const qo_hashgrid* child, const float* table,
                               const float* x, float* out)
{
    const int C = qo_hashgrid_num_outputs(child);
    const float* start = x + line->start_in;
    const float* dir = start + 3;
    float tmin, tmax, contribution[QO_MAX_LEVELS * 16], pos[3];
    line_intersect(line, start, dir, &tmin, &tmax);
    const int steps = line_num_steps(tmin, tmax, line->stepsize);
    int it = 0;
    for (int i = 0; i < C; ++i) out[i] = 0.f;
    for (float t = tmin; t < tmax && it < steps + 2; t += line->stepsize, ++it) {
        for (int d = 0; d < 3; ++d) pos[d] = fmaf(t, dir[d], start[d]);
        hashgrid_forward_point(child, table, pos, contribution);
        for (int i = 0; i < C; ++i) out[i] += contribution[i];
    }
    if (line->blending == QO_BLEND_AVERAGE && steps > 0) {
        const float scale = 1.0f / (float)steps;
        for (int i = 0; i < C; ++i) out[i] *= scale;
    }
}

/* tmin / tmax are constants of the adjoint (encoding_line_integration.cuh:138-152). */
static void line_adjoint_point(const qo_line* line, const qo_hashgrid* child, const float* table,
                               const float* x, const float* adj_out, float* adj_x, float* grad_table,
                               int res_factor, int atomic)
{
    const int C = qo_hashgrid_num_outputs(child);
    const float* start = x + line->start_in;
    const float* dir = start + 3;
    float tmin, tmax, adj_accu[QO_MAX_LEVELS * 16], pos[3], adj_pos[3];
    float adj_start[3] = {0.f, 0.f, 0.f}, adj_dir[3] = {0.f, 0.f, 0.f};
    line_intersect(line, start, dir, &tmin, &tmax);
    const int steps = line_num_steps(tmin, tmax, line->stepsize);
    int it = 0;
    float scale = 1.0f;
    if (line->blending == QO_BLEND_AVERAGE) scale = steps > 0 ? 1.0f / (float)steps : 1.0f;
    for (int i = 0; i < C; ++i) adj_accu[i] = scale * adj_out[i];
    for (float t = tmin; t < tmax && it < steps + 2; t += line->stepsize, ++it) {
        for (int d = 0; d < 3; ++d) { pos[d] = fmaf(t, dir[d], start[d]); adj_pos[d] = 0.f; }
        hashgrid_adjoint_point(child, table, pos, adj_accu, adj_x ? adj_pos : NULL, grad_table,
                               res_factor, atomic);
        if (adj_x)
            for (int d = 0; d < 3; ++d) { adj_start[d] += adj_pos[d]; adj_dir[d] += adj_pos[d] * t; }
    }
    if (adj_x)
        for (int d = 0; d < 3; ++d) {
            adj_x[line->start_in + d] += adj_start[d];
            adj_x[line->start_in + 3 + d] += adj_dir[d];
        }
}

void qo_line_forward(const qo_line* line, const qo_hashgrid* child, const float* table, const float* x,
                     long N, long x_stride, float* out, long out_stride)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (long n = 0; n < N; ++n)
        line_forward_point(line, child, table, x + n * x_stride, out + n * out_stride);
}

void qo_line_adjoint(const qo_line* line, const qo_hashgrid* child, const float* table, const float* x,
                     long N, long x_stride, const float* adj_out, long adj_out_stride,
                     float* adj_x, long adj_x_stride, float* grad_table, int res_factor)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (long n = 0; n < N; ++n)
        line_adjoint_point(line, child, table, x + n * x_stride, adj_out + n * adj_out_stride,
                           adj_x ? adj_x + n * adj_x_stride : NULL, grad_table, res_factor, 1);
}

/* ------------------------------------------------------------------ activations */

float qo_act_forward(int act, float param, float x)
{
    switch (act) {
    case QO_ACT_RELU: return x > 0.f ? x : 0.f;
    case QO_ACT_CELU: return x > 0.f ? x : expf(x) - 1.f;
    case QO_ACT_SINE: return sinf(x);
    case QO_ACT_SINE_FREQ: return sinf(param * x);
    default: return x;
    }
}

float qo_act_adjoint(int act, float param, float x, float adjz)
{
    switch (act) {
    case QO_ACT_RELU: return x > 0.f ? adjz : 0.f;
    case QO_ACT_CELU: return x > 0.f ? adjz : adjz * expf(x);
    case QO_ACT_SINE: return cosf(x) * adjz;
    case QO_ACT_SINE_FREQ: return param * cosf(param * x) * adjz;
    default: return adjz;
    }
}

/* ------------------------------------------------------------------ fused network */

int qo_network_encoded_channels(const qo_network* net)
{
    int c = 0;
    for (int e = 0; e < net->n_enc; ++e)
        c += net->enc_kind[e] == QO_ENC_IDENTITY ? net->enc_nin[e]
                                                 : qo_hashgrid_num_outputs(net->enc_grid[e]);  /* grid, or a line's child */
    return c;
}

static inline float layer_act_forward(const qo_network* net, int l, int channel, float x)
{
    if (net->act_channel[l])
        return qo_act_forward(net->act_channel[l][channel], net->act_param_channel[l][channel], x);
    return qo_act_forward(net->act[l], net->act_param[l], x);
}

static inline float layer_act_adjoint(const qo_network* net, int l, int channel, float x, float adjz)
{
    if (net->act_channel[l])
        return qo_act_adjoint(net->act_channel[l][channel], net->act_param_channel[l][channel], x, adjz);
    return qo_act_adjoint(net->act[l], net->act_param[l], x, adjz);
}

static inline float maybe_round(const qo_network* net, float v)
{
    return net->round_mode ? qo_round_half(v) : v;
}

/* Encodings of one point into a zero-padded row of cin[0] channels, concatenated in
 * array order (fused_network.cpp:423-437; zero padding network_forward.cuh:77-81). */
static void encode_point(const qo_network* net, const float* x, float* row)
{
    int off = 0;
    for (int e = 0; e < net->n_enc; ++e) {
        if (net->enc_kind[e] == QO_ENC_IDENTITY) {
            for (int i = 0; i < net->enc_nin[e]; ++i) row[off + i] = x[net->enc_start[e] + i];
            off += net->enc_nin[e];
        } else if (net->enc_kind[e] == QO_ENC_LINE) {
            line_forward_point(net->enc_line[e], net->enc_grid[e], net->enc_table[e], x, row + off);
            off += qo_hashgrid_num_outputs(net->enc_grid[e]);
        } else {
            hashgrid_forward_point(net->enc_grid[e], net->enc_table[e], x, row + off);
            off += qo_hashgrid_num_outputs(net->enc_grid[e]);
        }
    }
    for (int i = off; i < net->cin[0]; ++i) row[i] = 0.f;
    if (net->round_mode)
        for (int i = 0; i < off; ++i) row[i] = qo_round_half(row[i]);
}

__attribute__((target_clones("avx2,fma", "default")))
static void layer_forward_row(const float* W, const float* b, const float* in, int cin, int cout,
                              float* pre)
{
    for (int o = 0; o < cout; ++o) {
        const float* w = W + (size_t)o * cin;
        float acc = b ? b[o] : 0.f;     /* bias is the accumulator's initial value */
        for (int i = 0; i < cin; ++i) acc += w[i] * in[i];
        pre[o] = acc;
    }
}

__attribute__((target_clones("avx2,fma", "default")))
static void layer_backward_row(const float* W, const float* dpre, int cin, int cout, float* dx)
{
    for (int i = 0; i < cin; ++i) dx[i] = 0.f;
    for (int o = 0; o < cout; ++o) {
        const float* w = W + (size_t)o * cin;
        const float d = dpre[o];
        for (int i = 0; i < cin; ++i) dx[i] += w[i] * d;
    }
}

__attribute__((target_clones("avx2,fma", "default")))
static void outer_accumulate(float* dW, const float* dpre, const float* in, int cin, int cout)
{
    for (int o = 0; o < cout; ++o) {
        float* w = dW + (size_t)o * cin;
        const float d = dpre[o];
        for (int i = 0; i < cin; ++i) w[i] += d * in[i];
    }
}

static int max_width(const qo_network* net)
{
    int m = net->cin[0];
    for (int l = 0; l < net->n_layers; ++l) {
        if (net->cin[l] > m) m = net->cin[l];
        if (net->cout[l] > m) m = net->cout[l];
    }
    return m;
}

void qo_network_forward(const qo_network* net, const float* X, long N, long x_stride,
                        float* out, int n_out, float* enc_out, float* const* pre)
{
    const int mw = max_width(net);
#pragma omp parallel
    {
        float* cur = (float*)malloc(sizeof(float) * (size_t)mw);
        float* nxt = (float*)malloc(sizeof(float) * (size_t)mw);
#pragma omp for schedule(static)
        for (long n = 0; n < N; ++n) {
            encode_point(net, X + n * x_stride, cur);
            if (enc_out) memcpy(enc_out + n * net->cin[0], cur, sizeof(float) * (size_t)net->cin[0]);
            for (int l = 0; l < net->n_layers; ++l) {
                const int ci = net->cin[l], co = net->cout[l];
                layer_forward_row(net->W[l], net->b[l], cur, ci, co, nxt);
                for (int o = 0; o < co; ++o) {
                    float p = maybe_round(net, nxt[o]);
                    if (pre) pre[l][n * co + o] = p;
                    nxt[o] = maybe_round(net, layer_act_forward(net, l, o, p));
                }
                float* t = cur; cur = nxt; nxt = t;
            }
            for (int o = 0; o < n_out; ++o) out[n * n_out + o] = cur[o];
        }
        free(cur);
        free(nxt);
    }
}

void qo_network_backward(const qo_network* net, const float* X, long N, long x_stride,
                         const float* adj_out, int n_out, int flags,
                         const float* enc_out, float* const* pre,
                         float* adj_x, float* const* dpre_out)
{
    const int mw = max_width(net), L = net->n_layers;
    size_t wtot = 0, btot = 0;
    for (int l = 0; l < L; ++l) {
        wtot += (size_t)net->cin[l] * net->cout[l];
        btot += (size_t)net->cout[l];
    }
    const int want_w = (flags & QO_GRAD_WEIGHTS) != 0;
#pragma omp parallel
    {
        float* cur = (float*)malloc(sizeof(float) * (size_t)mw);
        float* nxt = (float*)malloc(sizeof(float) * (size_t)mw);
        float* inrow = (float*)malloc(sizeof(float) * (size_t)mw);
        float* lw = want_w ? (float*)calloc(wtot, sizeof(float)) : NULL;
        float* lb = want_w ? (float*)calloc(btot, sizeof(float)) : NULL;
#pragma omp for schedule(static)
        for (long n = 0; n < N; ++n) {
            /* dL/dy, zero padded up to the padded last width (test_against_eigen2.cpp:182) */
            const int cl = net->cout[L - 1];
            for (int o = 0; o < cl; ++o)
                cur[o] = o < n_out ? maybe_round(net, adj_out[n * n_out + o]) : 0.f;
            size_t woff = wtot, boff = btot;
            for (int l = L - 1; l >= 0; --l) {
                const int ci = net->cin[l], co = net->cout[l];
                woff -= (size_t)ci * co;
                boff -= (size_t)co;
                for (int o = 0; o < co; ++o) {
                    float d = layer_act_adjoint(net, l, o, pre[l][n * co + o], cur[o]);
                    d = maybe_round(net, d);
                    cur[o] = d;
                    if (dpre_out) dpre_out[l][n * co + o] = d;
                }
                if (want_w) {
                    if (l == 0) {
                        memcpy(inrow, enc_out + n * ci, sizeof(float) * (size_t)ci);
                    } else {
                        const int cp = net->cout[l - 1];
                        for (int i = 0; i < cp; ++i)
                            inrow[i] = maybe_round(net, layer_act_forward(net, l - 1, i, pre[l - 1][n * cp + i]));
                    }
                    if (net->dW[l]) outer_accumulate(lw + woff, cur, inrow, ci, co);
                    if (net->db[l]) for (int o = 0; o < co; ++o) lb[boff + o] += cur[o];
                }
                layer_backward_row(net->W[l], cur, ci, co, nxt);
                if (net->round_mode) for (int i = 0; i < ci; ++i) nxt[i] = qo_round_half(nxt[i]);
                float* t = cur; cur = nxt; nxt = t;
            }
            /* encoding adjoints on the row of encoded-channel adjoints */
            if (flags & (QO_GRAD_INPUT | QO_GRAD_ENCODINGS)) {
                const float* x = X + n * x_stride;
                float* ax = (flags & QO_GRAD_INPUT) ? adj_x + n * net->n_in : NULL;
                int off = 0;
                for (int e = 0; e < net->n_enc; ++e) {
                    if (net->enc_kind[e] == QO_ENC_IDENTITY) {
                        if (ax)
                            for (int i = 0; i < net->enc_nin[e]; ++i)
                                ax[net->enc_start[e] + i] += cur[off + i];
                        off += net->enc_nin[e];
                    } else {
                        float* gt = (flags & QO_GRAD_ENCODINGS) ? net->enc_grad[e] : NULL;
                        if ((ax || gt) && net->enc_kind[e] == QO_ENC_LINE)
                            line_adjoint_point(net->enc_line[e], net->enc_grid[e], net->enc_table[e], x,
                                               cur + off, ax, gt, net->res_factor, 1);
                        else if (ax || gt)
                            hashgrid_adjoint_point(net->enc_grid[e], net->enc_table[e], x,
                                                   cur + off, ax, gt, net->res_factor, 1);
                        off += qo_hashgrid_num_outputs(net->enc_grid[e]);
                    }
                }
            }
        }
        if (want_w) {
#pragma omp critical
            {
                size_t woff = 0, boff = 0;
                for (int l = 0; l < L; ++l) {
                    const size_t nw = (size_t)net->cin[l] * net->cout[l];
                    if (net->dW[l]) for (size_t i = 0; i < nw; ++i) net->dW[l][i] += lw[woff + i];
                    if (net->db[l]) for (int o = 0; o < net->cout[l]; ++o) net->db[l][o] += lb[boff + o];
                    woff += nw;
                    boff += (size_t)net->cout[l];
                }
            }
        }
        free(cur); free(nxt); free(inrow); free(lw); free(lb);
    }
}
