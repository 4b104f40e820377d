/*
 * CPU oracle for the two-layer MACE energy+forces path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT THE PRODUCT.  It is a serial fp64
 * restatement, in plain C, of the reference's CPU algorithm; the GPU engine
 * never calls it.  Only the test-suite, the smoke check and the benchmark's
 * CPU-baseline leg load this file's shared object.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference tree).  Loop nests and summation orders are kept the same as the
 * reference so that differences against it are at rounding level.
 *
 * Third-party arithmetic that is absent from the reference tree:
 *   - sphericart (lab-cosmo/sphericart, git submodule libsymmetrix/external/
 *     sphericart, commit not pinned by the tree).  Called at
 *     libsymmetrix/source/mace.cpp:132-133 as
 *     SphericalHarmonics<double>(l_max).compute_with_gradients.  Restated here
 *     from its published definition: orthonormal real spherical harmonics of
 *     the direction r/|r| (m<0 ~ sin|m|phi, m>0 ~ cos m phi, no Condon-Shortley
 *     sign in the real form) and their Cartesian gradients, closed forms l<=3.
 *     Pinned by the tests against scipy.special.sph_harm_y, the sum rule
 *     sum_m Y_lm^2 = (2l+1)/4pi, r.grad Y = 0 and central differences.
 *   - CBLAS dgemm/dgemv/ddot/dcopy: textbook semantics, written out as loops.
 *
 * Parity pins per function (see tests/test_oracle_*.py):
 *   orc_spline_set_*      reference object code (oracle/_ref, built from
 *                         cubic_spline_set.cpp) + scipy CubicSpline
 *   orc_poly_*            brute-force monomial sums + reference tools.cpp
 *                         partitions via oracle/_ref
 *   orc_mlp_*             numpy closed form + central differences
 *   compute_* / reverse_* the reference's own test method
 *                         (symmetrix/test/test_mace.py:73-84,145-159): adjoint
 *                         of each stage vs central differences; total energy
 *                         vs per-edge finite differences; rotation,
 *                         translation and permutation invariance of E.
 *   compute_* index conventions (which finite differences and invariances
 *                         cannot see): tests/test_oracle_stage_pins.py --
 *                         pair-table index, radial function index, sender
 *                         species of H0_weights, row-major [kp][k] weights of
 *                         A0 / H1 / A1 (rows e K + kp), transposed H2 weights,
 *                         readout layouts, (species, LM, k) of the M0 / M1
 *                         polynomials and their gradient slots, the sender-row
 *                         gather of Phi1, and the forward chain in numpy.
 *   orc_zbl_*, *_scaled   the two known answers of symmetrix/test/test_zbl.py
 *                         through the reference object code; special cases
 *                         fixed by the mathematics (tests/test_oracle_pipeline.py).
 * No function here is left without such a pin.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <stdio.h>

/* ------------------------------------------------------------------ */
/* growable double array with std::vector::resize semantics            */
typedef struct { double *p; size_t n, cap; } vec;

static void vec_resize(vec *v, size_t n)
{
    if (n > v->cap) {
        size_t cap = n;
        double *q = (double *)realloc(v->p, cap * sizeof(double));
        if (!q) { fprintf(stderr, "oracle: out of memory\n"); abort(); }
        v->p = q; v->cap = cap;
    }
    if (n > v->n) memset(v->p + v->n, 0, (n - v->n) * sizeof(double));
    v->n = n;
}
static void vec_fill(vec *v, double x) { for (size_t i = 0; i < v->n; ++i) v->p[i] = x; }
static void vec_free(vec *v) { free(v->p); v->p = NULL; v->n = v->cap = 0; }

/* ------------------------------------------------------------------ */
/* CubicSplineSet: libsymmetrix/source/cubic_spline_set.cpp            */

/* ctor, cubic_spline_set.cpp:5-25.  values/derivs are [num_splines][num_nodes];
 * c is [(4*interval+q)*num_splines + j], (num_nodes-1) intervals. */
void orc_spline_set_build(double h, int num_splines, int num_nodes,
                          const double *values, const double *derivs, double *c)
{
    for (int i = 0; i < num_nodes - 1; ++i) {
        for (int j = 0; j < num_splines; ++j) {
            const double v0 = values[(size_t)j * num_nodes + i];
            const double v1 = values[(size_t)j * num_nodes + i + 1];
            const double d0 = derivs[(size_t)j * num_nodes + i];
            const double d1 = derivs[(size_t)j * num_nodes + i + 1];
            c[(size_t)(4 * i) * num_splines + j] = v0;
            c[(size_t)(4 * i + 1) * num_splines + j] = d0;
            c[(size_t)(4 * i + 2) * num_splines + j] = (-3 * v0 - 2 * h * d0 + 3 * v1 - h * d1) / (h * h);
            c[(size_t)(4 * i + 3) * num_splines + j] = (2 * v0 + h * d0 - 2 * v1 + h * d1) / (h * h * h);
        }
    }
}

/* evaluate_derivs, cubic_spline_set.cpp:50-84 (no bounds check there either). */
void orc_spline_set_evaluate_derivs(double h, int num_splines, const double *c,
                                    double r, double *values, double *derivs)
{
    const int i = (int)(r / h);
    const double x = r - h * i;
    const double xx = x * x;
    const double xxx = xx * x;
    const double two_x = 2 * x;
    const double three_xx = 3 * xx;
    const double *c_i = c + (size_t)4 * i * num_splines;
    for (int j = 0; j < num_splines; ++j) values[j] = c_i[j];
    c_i += num_splines;
    for (int j = 0; j < num_splines; ++j) values[j] += x * c_i[j];
    c_i += num_splines;
    for (int j = 0; j < num_splines; ++j) values[j] += xx * c_i[j];
    c_i += num_splines;
    for (int j = 0; j < num_splines; ++j) values[j] += xxx * c_i[j];
    c_i = c + (size_t)(4 * i + 1) * num_splines;
    for (int j = 0; j < num_splines; ++j) derivs[j] = c_i[j];
    c_i += num_splines;
    for (int j = 0; j < num_splines; ++j) derivs[j] += two_x * c_i[j];
    c_i += num_splines;
    for (int j = 0; j < num_splines; ++j) derivs[j] += three_xx * c_i[j];
}

/* ------------------------------------------------------------------ */
/* CubicSpline (single): libsymmetrix/source/cubic_spline.cpp:15-71.
 * c is [interval][4].  Returns 0, or -1 where the reference throws
 * std::invalid_argument("Out of bounds in CubicSpline::evaluate."). */
void orc_spline_build(double h, int num_nodes, const double *values, const double *derivs, double *c)
{
    for (int i = 0; i < num_nodes - 1; ++i) {
        c[4 * i] = values[i];
        c[4 * i + 1] = derivs[i];
        c[4 * i + 2] = (-3 * values[i] - 2 * h * derivs[i] + 3 * values[i + 1] - h * derivs[i + 1]) / (h * h);
        c[4 * i + 3] = (2 * values[i] + h * derivs[i] - 2 * values[i + 1] + h * derivs[i + 1]) / (h * h * h);
    }
}
int orc_spline_evaluate_deriv(double h, int num_intervals, const double *c, double r, double *f, double *d)
{
    const int i = (int)(r / h);
    if (i < 0 || i >= num_intervals) return -1;
    const double x = r - h * i;
    const double xx = x * x;
    const double xxx = xx * x;
    const double *ci = c + 4 * i;
    *f = ci[0] + ci[1] * x + ci[2] * xx + ci[3] * xxx;
    *d = ci[1] + 2 * ci[2] * x + 3 * ci[3] * xx;
    return 0;
}

/* ------------------------------------------------------------------ */
/* MultivariatePolynomial evaluation on a prebuilt product graph.
 * libsymmetrix/source/multivariate_polynomial.cpp:114-187: forward sweep over
 * the edge list (node num_variables+e = product of its two parents), value =
 * dot(node_coefficients, node_values), adjoints seeded with the coefficients,
 * backward sweep in reverse edge order, gradient = adjoints of the leaves. */
double orc_poly_evaluate_gradient(int num_variables, int num_nodes, const int *edges,
                                  const double *node_coefficients, const double *x,
                                  double *node_values, double *node_adjoints, double *g)
{
    const int num_edges = num_nodes - num_variables;
    for (int i = 0; i < num_variables; ++i) node_values[i] = x[i];
    for (int e = 0; e < num_edges; ++e)
        node_values[num_variables + e] = node_values[edges[2 * e]] * node_values[edges[2 * e + 1]];
    double f = 0.0;
    for (int i = 0; i < num_nodes; ++i) f += node_coefficients[i] * node_values[i];
    for (int i = 0; i < num_nodes; ++i) node_adjoints[i] = node_coefficients[i];
    for (int e = num_edges - 1; e >= 0; --e) {
        const int i0 = edges[2 * e], i1 = edges[2 * e + 1];
        node_adjoints[i0] += node_adjoints[num_variables + e] * node_values[i1];
        node_adjoints[i1] += node_adjoints[num_variables + e] * node_values[i0];
    }
    for (int i = 0; i < num_variables; ++i) g[i] = node_adjoints[i];
    return f;
}

/* ------------------------------------------------------------------ */
/* MultilayerPerceptron::evaluate_gradient for a scalar-output MLP,
 * libsymmetrix/source/multilayer_perceptron.cpp:76-150.  weights[l] is
 * row-major [shape[l+1]][shape[l]]; activation c*x*sigmoid(x) on all but the
 * last layer.  Returns f, writes df/dinput to g[shape[0]]. */
double orc_mlp_evaluate_gradient(int num_layers, const int *shape, const double *const *weights,
                                 double scale, const double *input, double *g)
{
    /* num_layers = number of entries in shape */
    int maxw = 0;
    for (int i = 0; i < num_layers; ++i) if (shape[i] > maxw) maxw = shape[i];
    double *vals = (double *)calloc((size_t)num_layers * maxw, sizeof(double));
    double *act = (double *)calloc((size_t)num_layers * maxw, sizeof(double));
    double *der = (double *)calloc((size_t)2 * maxw, sizeof(double));
    for (int i = 0; i < shape[0]; ++i) vals[i] = input[i];
    for (int l = 0; l < num_layers - 2; ++l) {
        const double *W = weights[l];
        for (int o = 0; o < shape[l + 1]; ++o) {
            double s = 0.0;
            for (int i = 0; i < shape[l]; ++i) s += W[(size_t)o * shape[l] + i] * vals[(size_t)l * maxw + i];
            const double sig = 1.0 / (1.0 + exp(-s));
            vals[(size_t)(l + 1) * maxw + o] = scale * s * sig;
            act[(size_t)(l + 1) * maxw + o] = scale * sig + scale * s * sig * (1 - sig);
        }
    }
    double f = 0.0;
    {
        const int l = num_layers - 2;
        const double *W = weights[l];
        for (int i = 0; i < shape[l]; ++i) f += W[i] * vals[(size_t)l * maxw + i];
    }
    /* differentiate backwards: der holds d f / d node_values[l+1] */
    double *cur = der, *nxt = der + maxw;
    for (int i = 0; i < shape[num_layers - 2]; ++i) cur[i] = weights[num_layers - 2][i];
    for (int l = num_layers - 3; l >= 0; --l) {
        for (int j = 0; j < shape[l + 1]; ++j) cur[j] *= act[(size_t)(l + 1) * maxw + j];
        for (int i = 0; i < shape[l]; ++i) nxt[i] = 0.0;
        for (int j = 0; j < shape[l + 1]; ++j)
            for (int i = 0; i < shape[l]; ++i)
                nxt[i] += cur[j] * weights[l][(size_t)j * shape[l] + i];
        double *t = cur; cur = nxt; nxt = t;
    }
    for (int i = 0; i < shape[0]; ++i) g[i] = cur[i];
    free(vals); free(act); free(der);
    return f;
}

/* ------------------------------------------------------------------ */
/* ZBL: libsymmetrix/source/zbl.cpp:22-125 */
typedef struct {
    double a_exp, a_prefactor, c[4];
    double *covalent_radii; int n_radii; int p;
} orc_zbl;

static void zbl_envelope(double r, double r_max, int p, double *f, double *d)
{
    /* zbl.cpp:73-94: polynomial cutoff of order p and its derivative */
    if (r >= r_max) { *f = 0.0; *d = 0.0; return; }
    const double x = r / r_max;
    *f = 1.0 - ((p + 1.0) * (p + 2.0) / 2.0) * pow(x, p) + p * (p + 2.0) * pow(x, p + 1)
         - (p * (p + 1.0) / 2.0) * pow(x, p + 2);
    *d = (-((p + 1.0) * (p + 2.0) / 2.0) * p * pow(x, p - 1) + p * (p + 2.0) * (p + 1.0) * pow(x, p)
          - (p * (p + 1.0) / 2.0) * (p + 2.0) * pow(x, p + 1)) / r_max;
}

void orc_zbl_compute(const orc_zbl *z, int Zu, int Zv, double r, double *f_out, double *d_out)
{
    /* zbl.cpp:22-71: screened Coulomb pair term times half the envelope, and d/dr */
    const double Zuf = Zu, Zvf = Zv;
    const double a = z->a_prefactor * 0.529 / (pow(Zuf, z->a_exp) + pow(Zvf, z->a_exp));
    const double ra = r / a;
    static const double k[4] = {-3.2, -0.9423, -0.4028, -0.2016};
    const double e0 = z->c[0] * exp(k[0] * ra), e1 = z->c[1] * exp(k[1] * ra);
    const double e2 = z->c[2] * exp(k[2] * ra), e3 = z->c[3] * exp(k[3] * ra);
    const double phi = e0 + e1 + e2 + e3;
    const double dphi = (k[0] * e0 + k[1] * e1 + k[2] * e2 + k[3] * e3) / a;
    const double v = 14.3996 * Zuf * Zvf / r * phi;
    const double dv = 14.3996 * Zuf * Zvf * (r * dphi - phi) / (r * r);
    const double r_max = z->covalent_radii[Zu] + z->covalent_radii[Zv];
    double env, denv;
    zbl_envelope(r, r_max, z->p, &env, &denv);
    *f_out = v * (0.5 * env);
    *d_out = 0.5 * (v * denv + dv * env);
}

/* ------------------------------------------------------------------ */
typedef struct {
    int num_variables, num_nodes;      /* graph size */
    int *edges;                        /* [2*(num_nodes-num_variables)] */
    double *coef;                      /* [T][K][num_nodes] node coefficients */
} orc_poly;

typedef struct {
    /* basic model information, mace.cpp:912-920 */
    int T, K, l_max, num_lm, L_max, num_LM;
    double r_cut;
    int *atomic_numbers; double *atomic_energies;
    /* radial spline sets, mace.cpp:932-941 */
    double spl_h; int spl_nodes; int num_pairs; int nspl0, nspl1;
    double *c0, *c1;                   /* [pair][4*(nodes-1)*nspl] */
    double *H0_weights;                /* [T][K] */
    double *A0_weights;                /* [T][l_max+1][K*K] */
    int A0_scaled, A1_scaled; double A0_spl_h, A1_spl_h; int A0_spl_nodes, A1_spl_nodes;
    double *A0_spl_c, *A1_spl_c;       /* [pair][nodes-1][4] */
    orc_poly *P0; orc_poly P1;         /* P0[num_LM] */
    double *H1_weights;                /* [L_max+1][K*K] */
    int num_paths; int *Phi1_l, *Phi1_l1, *Phi1_l2;
    int num_cg; int *Phi1_lme, *Phi1_lelm1lm2; double *Phi1_cg;
    int num_lme, num_lelm1lm2;
    double *A1_weights[8]; /* per l, [num_e[l]*K][K] */
    double *H2_weights_for_H1;         /* [T][K*K] */
    double *H2_weights_for_M1;         /* [K*K] */
    double *readout_1_weights;         /* [K] */
    double *readout_2_w1, *readout_2_w2; double readout_2_scale;
    int has_zbl; orc_zbl zbl;
    /* state, mace.hpp members */
    vec node_energies, node_forces;
    vec R0, R0_deriv, R1, R1_deriv, Y, Y_grad;
    vec A0, A0_adj, M0, M0_grad, M0_adj, H1, H1_adj;
    vec Phi1r, dPhi1r, Phi1, dPhi1, A1, A1_adj, M1, M1_grad, M1_adj, H2, H2_adj;
} orc_model;

orc_model *orc_model_create(void) { return (orc_model *)calloc(1, sizeof(orc_model)); }

static double *dup_d(const double *p, size_t n)
{
    double *q = (double *)malloc((n ? n : 1) * sizeof(double));
    memcpy(q, p, n * sizeof(double));
    return q;
}
static int *dup_i(const int *p, size_t n)
{
    int *q = (int *)malloc((n ? n : 1) * sizeof(int));
    memcpy(q, p, n * sizeof(int));
    return q;
}

void orc_model_set_basic(orc_model *m, int T, int K, int l_max, int L_max, double r_cut,
                         const int *atomic_numbers, const double *atomic_energies)
{
    m->T = T; m->K = K; m->l_max = l_max; m->num_lm = (l_max + 1) * (l_max + 1);
    m->L_max = L_max; m->num_LM = (L_max + 1) * (L_max + 1); m->r_cut = r_cut;
    m->atomic_numbers = dup_i(atomic_numbers, T);
    m->atomic_energies = dup_d(atomic_energies, T);
    m->P0 = (orc_poly *)calloc(m->num_LM, sizeof(orc_poly));
}

/* values/derivs: [pair][num_splines][num_nodes]; which = 0 (R0) or 1 (R1) */
void orc_model_set_radial(orc_model *m, int which, double h, int num_pairs, int num_splines,
                          int num_nodes, const double *values, const double *derivs)
{
    const size_t per = (size_t)4 * (num_nodes - 1) * num_splines;
    double *c = (double *)malloc(per * num_pairs * sizeof(double));
    for (int p = 0; p < num_pairs; ++p)
        orc_spline_set_build(h, num_splines, num_nodes,
                             values + (size_t)p * num_splines * num_nodes,
                             derivs + (size_t)p * num_splines * num_nodes, c + per * p);
    m->spl_h = h; m->spl_nodes = num_nodes; m->num_pairs = num_pairs;
    if (which == 0) { m->c0 = c; m->nspl0 = num_splines; }
    else { m->c1 = c; m->nspl1 = num_splines; }
}

void orc_model_set_scaling(orc_model *m, int which, double h, int num_pairs, int num_nodes,
                           const double *values, const double *derivs)
{
    double *c = (double *)malloc((size_t)num_pairs * (num_nodes - 1) * 4 * sizeof(double));
    for (int p = 0; p < num_pairs; ++p)
        orc_spline_build(h, num_nodes, values + (size_t)p * num_nodes, derivs + (size_t)p * num_nodes,
                         c + (size_t)p * (num_nodes - 1) * 4);
    if (which == 0) { m->A0_scaled = 1; m->A0_spl_h = h; m->A0_spl_nodes = num_nodes; m->A0_spl_c = c; }
    else { m->A1_scaled = 1; m->A1_spl_h = h; m->A1_spl_nodes = num_nodes; m->A1_spl_c = c; }
}

void orc_model_set_zbl(orc_model *m, double a_exp, double a_prefactor, const double *c,
                       const double *radii, int n_radii, int p)
{
    m->has_zbl = 1; m->zbl.a_exp = a_exp; m->zbl.a_prefactor = a_prefactor;
    memcpy(m->zbl.c, c, 4 * sizeof(double));
    m->zbl.covalent_radii = dup_d(radii, n_radii); m->zbl.n_radii = n_radii; m->zbl.p = p;
}

/* which: 0 -> P0[LM], 1 -> P1.  coef: [T][K][num_nodes] */
void orc_model_set_poly(orc_model *m, int which, int LM, int num_variables, int num_nodes,
                        const int *edges, const double *coef)
{
    orc_poly *P = which == 0 ? &m->P0[LM] : &m->P1;
    P->num_variables = num_variables; P->num_nodes = num_nodes;
    P->edges = dup_i(edges, (size_t)2 * (num_nodes - num_variables));
    P->coef = dup_d(coef, (size_t)m->T * m->K * num_nodes);
}

void orc_model_set_weights(orc_model *m, const double *H0, const double *A0w, const double *H1w,
                           const double *H2H1, const double *H2M1, const double *ro1,
                           const double *ro2w1, const double *ro2w2, double ro2scale)
{
    const int K = m->K, T = m->T;
    m->H0_weights = dup_d(H0, (size_t)T * K);
    m->A0_weights = dup_d(A0w, (size_t)T * (m->l_max + 1) * K * K);
    m->H1_weights = dup_d(H1w, (size_t)(m->L_max + 1) * K * K);
    m->H2_weights_for_H1 = dup_d(H2H1, (size_t)T * K * K);
    m->H2_weights_for_M1 = dup_d(H2M1, (size_t)K * K);
    m->readout_1_weights = dup_d(ro1, K);
    m->readout_2_w1 = dup_d(ro2w1, (size_t)16 * K);
    m->readout_2_w2 = dup_d(ro2w2, 16);
    m->readout_2_scale = ro2scale;
}

void orc_model_set_phi1(orc_model *m, int num_paths, const int *l, const int *l1, const int *l2,
                        int num_cg, const int *lme, const double *cgv, const int *lelm1lm2)
{
    m->num_paths = num_paths;
    m->Phi1_l = dup_i(l, num_paths); m->Phi1_l1 = dup_i(l1, num_paths); m->Phi1_l2 = dup_i(l2, num_paths);
    m->num_cg = num_cg;
    m->Phi1_lme = dup_i(lme, num_cg); m->Phi1_cg = dup_d(cgv, num_cg); m->Phi1_lelm1lm2 = dup_i(lelm1lm2, num_cg);
    /* mace.cpp:984-989 */
    m->num_lme = 0;
    for (int i = 0; i < num_paths; ++i) m->num_lme += 2 * l[i] + 1;
    m->num_lelm1lm2 = 0;
    for (int i = 0; i < num_paths; ++i) m->num_lelm1lm2 += (2 * l1[i] + 1) * (2 * l2[i] + 1);
}

void orc_model_set_A1_weights(orc_model *m, int l, const double *w, int n)
{
    m->A1_weights[l] = dup_d(w, n);
}

void orc_model_free(orc_model *m)
{
    if (!m) return;
    free(m->atomic_numbers); free(m->atomic_energies); free(m->c0); free(m->c1);
    free(m->H0_weights); free(m->A0_weights); free(m->A0_spl_c); free(m->A1_spl_c);
    for (int i = 0; i < m->num_LM; ++i) { free(m->P0[i].edges); free(m->P0[i].coef); }
    free(m->P0); free(m->P1.edges); free(m->P1.coef);
    free(m->H1_weights); free(m->Phi1_l); free(m->Phi1_l1); free(m->Phi1_l2);
    free(m->Phi1_lme); free(m->Phi1_lelm1lm2); free(m->Phi1_cg);
    for (int l = 0; l < 8; ++l) free(m->A1_weights[l]);
    free(m->H2_weights_for_H1); free(m->H2_weights_for_M1); free(m->readout_1_weights);
    free(m->readout_2_w1); free(m->readout_2_w2); free(m->zbl.covalent_radii);
    vec *vs[] = {&m->node_energies, &m->node_forces, &m->R0, &m->R0_deriv, &m->R1, &m->R1_deriv,
                 &m->Y, &m->Y_grad, &m->A0, &m->A0_adj, &m->M0, &m->M0_grad, &m->M0_adj, &m->H1,
                 &m->H1_adj, &m->Phi1r, &m->dPhi1r, &m->Phi1, &m->dPhi1, &m->A1, &m->A1_adj,
                 &m->M1, &m->M1_grad, &m->M1_adj, &m->H2, &m->H2_adj};
    for (size_t i = 0; i < sizeof(vs) / sizeof(vs[0]); ++i) vec_free(vs[i]);
    free(m);
}

static vec *find_vec(orc_model *m, const char *name)
{
    struct { const char *n; vec *v; } tab[] = {
        {"node_energies", &m->node_energies}, {"node_forces", &m->node_forces},
        {"R0", &m->R0}, {"R0_deriv", &m->R0_deriv}, {"R1", &m->R1}, {"R1_deriv", &m->R1_deriv},
        {"Y", &m->Y}, {"Y_grad", &m->Y_grad}, {"A0", &m->A0}, {"A0_adj", &m->A0_adj},
        {"M0", &m->M0}, {"M0_grad", &m->M0_grad}, {"M0_adj", &m->M0_adj}, {"H1", &m->H1},
        {"H1_adj", &m->H1_adj}, {"Phi1r", &m->Phi1r}, {"dPhi1r", &m->dPhi1r}, {"Phi1", &m->Phi1},
        {"Phi1_adj", &m->dPhi1}, {"dPhi1", &m->dPhi1}, {"A1", &m->A1}, {"A1_adj", &m->A1_adj},
        {"M1", &m->M1}, {"M1_grad", &m->M1_grad}, {"M1_adj", &m->M1_adj}, {"H2", &m->H2},
        {"H2_adj", &m->H2_adj}};
    for (size_t i = 0; i < sizeof(tab) / sizeof(tab[0]); ++i)
        if (!strcmp(tab[i].n, name)) return tab[i].v;
    return NULL;
}
/* read/write access to the named intermediates (symmetrix/source/cpp/mace.cpp:14-34) */
double *orc_get(orc_model *m, const char *name, long *n)
{
    vec *v = find_vec(m, name);
    if (!v) { *n = -1; return NULL; }
    *n = (long)v->n; return v->p;
}
int orc_set(orc_model *m, const char *name, const double *p, long n)
{
    vec *v = find_vec(m, name);
    if (!v) return -1;
    v->n = 0; vec_resize(v, (size_t)n); memcpy(v->p, p, (size_t)n * sizeof(double));
    return 0;
}

static inline int pair_index(int T, int a, int b)
{
    /* mace.cpp:81-83 */
    return (a <= b) ? a * (2 * T - a - 1) / 2 + b : b * (2 * T - b - 1) / 2 + a;
}

/* ------------------------------------------------------------------ */
/* mace.cpp:66-116 */
static void compute_R(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                      const int *neigh_types, const double *r, size_t E, int num_spl, const double *c,
                      vec *R, vec *Rd)
{
    vec_resize(R, E * num_spl); vec_resize(Rd, R->n);
    const size_t per = (size_t)4 * (m->spl_nodes - 1) * num_spl;
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        const int ti = node_types[i];
        for (int j = 0; j < num_neigh[i]; ++j) {
            const int tij = pair_index(m->T, ti, neigh_types[ij]);
            orc_spline_set_evaluate_derivs(m->spl_h, num_spl, c + per * tij, r[ij],
                                           R->p + ij * num_spl, Rd->p + ij * num_spl);
            ij += 1;
        }
    }
}
void orc_compute_R0(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                    const int *neigh_types, const double *r, long E)
{ compute_R(m, num_nodes, node_types, num_neigh, neigh_types, r, (size_t)E, m->nspl0, m->c0, &m->R0, &m->R0_deriv); }
void orc_compute_R1(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                    const int *neigh_types, const double *r, long E)
{ compute_R(m, num_nodes, node_types, num_neigh, neigh_types, r, (size_t)E, m->nspl1, m->c1, &m->R1, &m->R1_deriv); }

/* ------------------------------------------------------------------ */
/* Real spherical harmonics l<=3 of the direction of v and their gradients
 * with respect to v (sphericart's normalised variant, closed forms). */
void orc_sph_harm_l3(const double v[3], double Y[16], double dY[3][16])
{
    const double PI = 3.14159265358979323846;
    const double r = sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
    const double x = v[0] / r, y = v[1] / r, z = v[2] / r;
    const double c0 = 0.5 * sqrt(1.0 / PI), c1 = sqrt(3.0 / (4.0 * PI));
    const double c2a = 0.5 * sqrt(15.0 / PI), c2b = 0.25 * sqrt(5.0 / PI), c2c = 0.25 * sqrt(15.0 / PI);
    const double c3a = 0.25 * sqrt(35.0 / (2.0 * PI)), c3b = 0.5 * sqrt(105.0 / PI);
    const double c3c = 0.25 * sqrt(21.0 / (2.0 * PI)), c3d = 0.25 * sqrt(7.0 / PI), c3e = 0.25 * sqrt(105.0 / PI);
    const double xx = x * x, yy = y * y, zz = z * z;
    double g[3][16]; /* derivative of the homogeneous form with respect to the unit vector */
    Y[0] = c0;                          g[0][0] = 0;              g[1][0] = 0;               g[2][0] = 0;
    Y[1] = c1 * y;                      g[0][1] = 0;              g[1][1] = c1;              g[2][1] = 0;
    Y[2] = c1 * z;                      g[0][2] = 0;              g[1][2] = 0;               g[2][2] = c1;
    Y[3] = c1 * x;                      g[0][3] = c1;             g[1][3] = 0;               g[2][3] = 0;
    Y[4] = c2a * x * y;                 g[0][4] = c2a * y;        g[1][4] = c2a * x;         g[2][4] = 0;
    Y[5] = c2a * y * z;                 g[0][5] = 0;              g[1][5] = c2a * z;         g[2][5] = c2a * y;
    Y[6] = c2b * (2 * zz - xx - yy);    g[0][6] = -2 * c2b * x;   g[1][6] = -2 * c2b * y;    g[2][6] = 4 * c2b * z;
    Y[7] = c2a * x * z;                 g[0][7] = c2a * z;        g[1][7] = 0;               g[2][7] = c2a * x;
    Y[8] = c2c * (xx - yy);             g[0][8] = 2 * c2c * x;    g[1][8] = -2 * c2c * y;    g[2][8] = 0;
    Y[9] = c3a * y * (3 * xx - yy);     g[0][9] = 6 * c3a * x * y; g[1][9] = c3a * (3 * xx - 3 * yy); g[2][9] = 0;
    Y[10] = c3b * x * y * z;            g[0][10] = c3b * y * z;   g[1][10] = c3b * x * z;    g[2][10] = c3b * x * y;
    Y[11] = c3c * y * (4 * zz - xx - yy);
    g[0][11] = -2 * c3c * x * y; g[1][11] = c3c * (4 * zz - xx - 3 * yy); g[2][11] = 8 * c3c * y * z;
    Y[12] = c3d * z * (2 * zz - 3 * xx - 3 * yy);
    g[0][12] = -6 * c3d * x * z; g[1][12] = -6 * c3d * y * z; g[2][12] = c3d * (6 * zz - 3 * xx - 3 * yy);
    Y[13] = c3c * x * (4 * zz - xx - yy);
    g[0][13] = c3c * (4 * zz - 3 * xx - yy); g[1][13] = -2 * c3c * x * y; g[2][13] = 8 * c3c * x * z;
    Y[14] = c3e * (xx - yy) * z;        g[0][14] = 2 * c3e * x * z; g[1][14] = -2 * c3e * y * z; g[2][14] = c3e * (xx - yy);
    Y[15] = c3a * x * (xx - 3 * yy);    g[0][15] = c3a * (3 * xx - 3 * yy); g[1][15] = -6 * c3a * x * y; g[2][15] = 0;
    /* chain rule through u = v/|v|: grad_v = (grad_u - u (u.grad_u)) / r, and
     * u.grad_u = l * Y for a homogeneous form of degree l */
    const double u[3] = {x, y, z};
    for (int l = 0; l <= 3; ++l)
        for (int lm = l * l; lm < (l + 1) * (l + 1); ++lm)
            for (int a = 0; a < 3; ++a)
                dY[a][lm] = (g[a][lm] - l * u[a] * Y[lm]) / r;
}

/* mace.cpp:118-148 */
void orc_compute_Y(orc_model *m, const double *xyz, long n3)
{
    if (n3 == 0) return;
    const size_t num = (size_t)n3 / 3;
    const int num_lm = m->num_lm;
    vec_resize(&m->Y, num * num_lm); vec_resize(&m->Y_grad, 3 * num * num_lm);
    const double norm = 2 * sqrt(3.14159265358979323846);
    for (size_t i = 0; i < num; ++i) {
        /* shuffle to (z,x,y), mace.cpp:127-131 */
        const double s[3] = {xyz[3 * i + 2], xyz[3 * i], xyz[3 * i + 1]};
        double Y[16], dY[3][16];
        orc_sph_harm_l3(s, Y, dY);
        for (int lm = 0; lm < num_lm; ++lm) {
            m->Y.p[i * num_lm + lm] = norm * Y[lm];
            /* unshuffle gradient rows, mace.cpp:141-147 */
            m->Y_grad.p[3 * i * num_lm + 0 * num_lm + lm] = norm * dY[1][lm];
            m->Y_grad.p[3 * i * num_lm + 1 * num_lm + lm] = norm * dY[2][lm];
            m->Y_grad.p[3 * i * num_lm + 2 * num_lm + lm] = norm * dY[0][lm];
        }
    }
}

/* row-major C[m x n] = A[m x k] * op(B) ; beta = 0.  transb: B is [n x k] used transposed */
static void gemm_nn(int M, int N, int Kd, const double *A, int lda, const double *B, int ldb, double *C, int ldc)
{
    for (int i = 0; i < M; ++i) {
        double *c = C + (size_t)i * ldc;
        for (int j = 0; j < N; ++j) c[j] = 0.0;
        for (int p = 0; p < Kd; ++p) {
            const double a = A[(size_t)i * lda + p];
            const double *b = B + (size_t)p * ldb;
            for (int j = 0; j < N; ++j) c[j] += a * b[j];
        }
    }
}
static void gemm_nt(int M, int N, int Kd, const double *A, int lda, const double *B, int ldb, double *C, int ldc)
{
    for (int i = 0; i < M; ++i) {
        const double *a = A + (size_t)i * lda;
        for (int j = 0; j < N; ++j) {
            const double *b = B + (size_t)j * ldb;
            double s = 0.0;
            for (int p = 0; p < Kd; ++p) s += a[p] * b[p];
            C[(size_t)i * ldc + j] = s;
        }
    }
}

/* mace.cpp:150-201 */
void orc_compute_A0(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                    const int *neigh_types)
{
    const int K = m->K, num_lm = m->num_lm, l_max = m->l_max;
    vec_resize(&m->A0, (size_t)num_nodes * num_lm * K);
    double *Phi0 = (double *)malloc((size_t)num_lm * K * sizeof(double));
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        for (int q = 0; q < num_lm * K; ++q) Phi0[q] = 0.0;
        for (int j = 0; j < num_neigh[i]; ++j) {
            const double *Y_ij = m->Y.p + ij * num_lm;
            const double *H0_ij = m->H0_weights + (size_t)neigh_types[ij] * K;
            for (int l = 0; l <= l_max; ++l) {
                const double *R0_ij_l = m->R0.p + ij * (l_max + 1) * K + (size_t)l * K;
                for (int mm = -l; mm <= l; ++mm) {
                    const int lm = l * l + l + mm;
                    const double y = Y_ij[lm];
                    double *P = Phi0 + (size_t)lm * K;
                    for (int k = 0; k < K; ++k) P[k] += R0_ij_l[k] * y * H0_ij[k];
                }
            }
            ij += 1;
        }
        for (int l = 0; l <= l_max; ++l)
            gemm_nn(2 * l + 1, K, K, Phi0 + (size_t)l * l * K, K,
                    m->A0_weights + ((size_t)node_types[i] * (l_max + 1) + l) * K * K, K,
                    m->A0.p + ((size_t)i * num_lm + l * l) * K, K);
    }
    free(Phi0);
}

/* mace.cpp:203-271 */
void orc_reverse_A0(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                    const int *neigh_types, const double *xyz, const double *r)
{
    const int K = m->K, num_lm = m->num_lm, l_max = m->l_max;
    double *Phi0_adj = (double *)malloc((size_t)num_lm * K * sizeof(double));
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        for (int l = 0; l <= l_max; ++l)
            gemm_nt(2 * l + 1, K, K, m->A0_adj.p + ((size_t)i * num_lm + l * l) * K, K,
                    m->A0_weights + ((size_t)node_types[i] * (l_max + 1) + l) * K * K, K,
                    Phi0_adj + (size_t)l * l * K, K);
        for (int j = 0; j < num_neigh[i]; ++j) {
            const double *x = xyz + ij * 3;
            const double r_ij = r[ij];
            const double *Y_ij = m->Y.p + ij * num_lm;
            const double *Yg = m->Y_grad.p + ij * 3 * num_lm;
            const double *H0_ij = m->H0_weights + (size_t)neigh_types[ij] * K;
            double *f = m->node_forces.p + ij * 3;
            for (int l = 0; l <= l_max; ++l) {
                const double *R = m->R0.p + ij * (l_max + 1) * K + (size_t)l * K;
                const double *Rd = m->R0_deriv.p + ij * (l_max + 1) * K + (size_t)l * K;
                for (int mm = -l; mm <= l; ++mm) {
                    const int lm = l * l + l + mm;
                    const double y = Y_ij[lm];
                    const double gx = Yg[lm], gy = Yg[num_lm + lm], gz = Yg[2 * num_lm + lm];
                    const double *Pa = Phi0_adj + (size_t)lm * K;
                    for (int k = 0; k < K; ++k) {
                        f[0] += -Pa[k] * (x[0] / r_ij * Rd[k] * y * H0_ij[k] + R[k] * gx * H0_ij[k]);
                        f[1] += -Pa[k] * (x[1] / r_ij * Rd[k] * y * H0_ij[k] + R[k] * gy * H0_ij[k]);
                        f[2] += -Pa[k] * (x[2] / r_ij * Rd[k] * y * H0_ij[k] + R[k] * gz * H0_ij[k]);
                    }
                }
            }
            ij += 1;
        }
    }
    free(Phi0_adj);
}

/* mace.cpp:273-297 and 681-705 (same code for layer 0 and 1) */
static int compute_scaled(orc_model *m, int scaled, double h, int nodes, const double *c, vec *A,
                          int num_nodes, const int *node_types, const int *num_neigh,
                          const int *neigh_types, const double *r)
{
    if (!scaled) return 0;
    const int nK = m->num_lm * m->K;
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        double s = 1.0;
        for (int j = 0; j < num_neigh[i]; ++j) {
            const int tij = pair_index(m->T, node_types[i], neigh_types[ij]);
            double f, d;
            if (orc_spline_evaluate_deriv(h, nodes - 1, c + (size_t)tij * (nodes - 1) * 4, r[ij], &f, &d)) return -1;
            s += f;
            ij += 1;
        }
        double *Ai = A->p + (size_t)i * nK;
        for (int q = 0; q < nK; ++q) Ai[q] /= s;
    }
    return 0;
}
int orc_compute_A0_scaled(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                          const int *neigh_types, const double *r)
{ return compute_scaled(m, m->A0_scaled, m->A0_spl_h, m->A0_spl_nodes, m->A0_spl_c, &m->A0, num_nodes, node_types, num_neigh, neigh_types, r); }
int orc_compute_A1_scaled(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                          const int *neigh_types, const double *r)
{ return compute_scaled(m, m->A1_scaled, m->A1_spl_h, m->A1_spl_nodes, m->A1_spl_c, &m->A1, num_nodes, node_types, num_neigh, neigh_types, r); }

/* mace.cpp:299-346 and 707-757 */
static int reverse_scaled(orc_model *m, int scaled, double h, int nodes, const double *c, vec *A, vec *A_adj,
                          int num_nodes, const int *node_types, const int *num_neigh,
                          const int *neigh_types, const double *xyz, const double *r)
{
    if (!scaled) return 0;
    const int nK = m->num_lm * m->K;
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        const double *Ai = A->p + (size_t)i * nK;
        double *Aa = A_adj->p + (size_t)i * nK;
        double s = 1.0;
        for (int j = 0; j < num_neigh[i]; ++j) {
            const int tij = pair_index(m->T, node_types[i], neigh_types[ij]);
            double f, d;
            if (orc_spline_evaluate_deriv(h, nodes - 1, c + (size_t)tij * (nodes - 1) * 4, r[ij], &f, &d)) return -1;
            s += f;
            ij += 1;
        }
        double dot = 0.0;
        for (int q = 0; q < nK; ++q) dot += Aa[q] * Ai[q];
        ij -= num_neigh[i];
        for (int j = 0; j < num_neigh[i]; ++j) {
            const int tij = pair_index(m->T, node_types[i], neigh_types[ij]);
            double f, d;
            orc_spline_evaluate_deriv(h, nodes - 1, c + (size_t)tij * (nodes - 1) * 4, r[ij], &f, &d);
            double *F = m->node_forces.p + ij * 3;
            F[0] += dot / s * d * xyz[ij * 3] / r[ij];
            F[1] += dot / s * d * xyz[ij * 3 + 1] / r[ij];
            F[2] += dot / s * d * xyz[ij * 3 + 2] / r[ij];
            ij += 1;
        }
        for (int q = 0; q < nK; ++q) Aa[q] /= s;
    }
    return 0;
}
int orc_reverse_A0_scaled(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                          const int *neigh_types, const double *xyz, const double *r)
{ return reverse_scaled(m, m->A0_scaled, m->A0_spl_h, m->A0_spl_nodes, m->A0_spl_c, &m->A0, &m->A0_adj, num_nodes, node_types, num_neigh, neigh_types, xyz, r); }
int orc_reverse_A1_scaled(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                          const int *neigh_types, const double *xyz, const double *r, long n3, int zero_dxyz)
{
    if (!m->A1_scaled) return 0;
    vec_resize(&m->node_forces, (size_t)n3);
    if (zero_dxyz) vec_fill(&m->node_forces, 0.0);
    return reverse_scaled(m, m->A1_scaled, m->A1_spl_h, m->A1_spl_nodes, m->A1_spl_c, &m->A1, &m->A1_adj, num_nodes, node_types, num_neigh, neigh_types, xyz, r);
}

/* mace.cpp:348-370 */
void orc_compute_M0(orc_model *m, int num_nodes, const int *node_types)
{
    const int K = m->K, num_lm = m->num_lm, num_LM = m->num_LM;
    vec_resize(&m->M0, (size_t)num_nodes * num_LM * K);
    vec_resize(&m->M0_grad, (size_t)num_nodes * K * num_LM * num_lm);
    int maxn = 0;
    for (int LM = 0; LM < num_LM; ++LM) if (m->P0[LM].num_nodes > maxn) maxn = m->P0[LM].num_nodes;
    double *nv = (double *)malloc((size_t)maxn * sizeof(double));
    double *na = (double *)malloc((size_t)maxn * sizeof(double));
    double x[64], g[64];
    for (int i = 0; i < num_nodes; ++i) {
        const double *A0_i = m->A0.p + (size_t)i * num_lm * K;
        double *M0_i = m->M0.p + (size_t)i * num_LM * K;
        double *M0_grad_i = m->M0_grad.p + (size_t)i * num_LM * K * num_lm;
        for (int LM = 0; LM < num_LM; ++LM) {
            const orc_poly *P = &m->P0[LM];
            for (int k = 0; k < K; ++k) {
                for (int q = 0; q < num_lm; ++q) x[q] = A0_i[(size_t)q * K + k];
                const double *coef = P->coef + ((size_t)node_types[i] * K + k) * P->num_nodes;
                const double f = orc_poly_evaluate_gradient(P->num_variables, P->num_nodes, P->edges, coef, x, nv, na, g);
                M0_i[(size_t)LM * K + k] = f;
                for (int q = 0; q < num_lm; ++q) M0_grad_i[((size_t)LM * num_lm + q) * K + k] = g[q];
            }
        }
    }
    free(nv); free(na);
}

/* mace.cpp:372-395 */
void orc_reverse_M0(orc_model *m, int num_nodes)
{
    const int K = m->K, num_lm = m->num_lm, num_LM = m->num_LM;
    vec_resize(&m->A0_adj, m->A0.n); vec_fill(&m->A0_adj, 0.0);
    for (int i = 0; i < num_nodes; ++i) {
        double *A0_adj_i = m->A0_adj.p + (size_t)i * num_lm * K;
        const double *M0_adj_i = m->M0_adj.p + (size_t)i * num_LM * K;
        const double *M0_grad_i = m->M0_grad.p + (size_t)i * num_LM * num_lm * K;
        for (int lm = 0; lm < num_lm; ++lm)
            for (int LM = 0; LM < num_LM; ++LM)
                for (int k = 0; k < K; ++k)
                    A0_adj_i[(size_t)lm * K + k] += M0_grad_i[((size_t)LM * num_lm + lm) * K + k] * M0_adj_i[(size_t)LM * K + k];
    }
}

/* mace.cpp:397-423 */
void orc_compute_H1(orc_model *m, int num_nodes)
{
    const int K = m->K, num_LM = m->num_LM;
    vec_resize(&m->H1, m->M0.n);
    for (int i = 0; i < num_nodes; ++i)
        for (int l = 0; l <= m->L_max; ++l)
            gemm_nn(2 * l + 1, K, K, m->M0.p + ((size_t)i * num_LM + l * l) * K, K,
                    m->H1_weights + (size_t)l * K * K, K, m->H1.p + ((size_t)i * num_LM + l * l) * K, K);
}
/* mace.cpp:425-451 */
void orc_reverse_H1(orc_model *m, int num_nodes)
{
    const int K = m->K, num_LM = m->num_LM;
    vec_resize(&m->M0_adj, m->M0.n);
    for (int i = 0; i < num_nodes; ++i)
        for (int l = 0; l <= m->L_max; ++l)
            gemm_nt(2 * l + 1, K, K, m->H1_adj.p + ((size_t)i * num_LM + l * l) * K, K,
                    m->H1_weights + (size_t)l * K * K, K, m->M0_adj.p + ((size_t)i * num_LM + l * l) * K, K);
}

/* mace.cpp:453-502 */
void orc_compute_Phi1(orc_model *m, int num_nodes, const int *num_neigh, const int *neigh_indices)
{
    const int K = m->K, num_lm = m->num_lm, num_LM = m->num_LM, nq = m->num_lelm1lm2, ne = m->num_lme;
    vec_resize(&m->Phi1r, (size_t)num_nodes * nq * K); vec_fill(&m->Phi1r, 0.0);
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        double *Pr = m->Phi1r.p + (size_t)i * nq * K;
        for (int j = 0; j < num_neigh[i]; ++j) {
            const double *R1_ij = m->R1.p + ij * m->nspl1;
            const double *Y_ij = m->Y.p + ij * num_lm;
            const double *H1_ij = m->H1.p + (size_t)neigh_indices[ij] * num_LM * K;
            int q = 0;
            for (int p = 0; p < m->num_paths; ++p) {
                const int l1 = m->Phi1_l1[p], l2 = m->Phi1_l2[p];
                const double *Rp = R1_ij + (size_t)p * K;
                for (int lm1 = l1 * l1; lm1 <= l1 * (l1 + 2); ++lm1) {
                    const double y = Y_ij[lm1];
                    for (int lm2 = l2 * l2; lm2 <= l2 * (l2 + 2); ++lm2) {
                        const double *H = H1_ij + (size_t)lm2 * K;
                        double *o = Pr + (size_t)q * K;
                        for (int k = 0; k < K; ++k) o[k] += Rp[k] * y * H[k];
                        q += 1;
                    }
                }
            }
            ij += 1;
        }
    }
    vec_resize(&m->Phi1, (size_t)num_nodes * ne * K); vec_fill(&m->Phi1, 0.0);
    for (int i = 0; i < num_nodes; ++i) {
        double *P = m->Phi1.p + (size_t)i * ne * K;
        const double *Pr = m->Phi1r.p + (size_t)i * nq * K;
        for (int p = 0; p < m->num_cg; ++p) {
            double *o = P + (size_t)m->Phi1_lme[p] * K;
            const double C = m->Phi1_cg[p];
            const double *s = Pr + (size_t)m->Phi1_lelm1lm2[p] * K;
            for (int k = 0; k < K; ++k) o[k] += C * s[k];
        }
    }
}

/* mace.cpp:504-605 */
void orc_reverse_Phi1(orc_model *m, int num_nodes, const int *num_neigh, const int *neigh_indices,
                      const double *xyz, const double *r, long n3, int zero_dxyz, int zero_H1_adj)
{
    const int K = m->K, num_lm = m->num_lm, num_LM = m->num_LM, nq = m->num_lelm1lm2, ne = m->num_lme;
    vec_resize(&m->dPhi1r, m->Phi1r.n); vec_fill(&m->dPhi1r, 0.0);
    for (int i = 0; i < num_nodes; ++i) {
        double *dr = m->dPhi1r.p + (size_t)i * nq * K;
        const double *d = m->dPhi1.p + (size_t)i * ne * K;
        for (int p = 0; p < m->num_cg; ++p) {
            double *o = dr + (size_t)m->Phi1_lelm1lm2[p] * K;
            const double C = m->Phi1_cg[p];
            const double *s = d + (size_t)m->Phi1_lme[p] * K;
            for (int k = 0; k < K; ++k) o[k] += C * s[k];
        }
    }
    vec_resize(&m->node_forces, (size_t)n3);
    if (zero_dxyz) vec_fill(&m->node_forces, 0.0);
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        const double *dr = m->dPhi1r.p + (size_t)i * nq * K;
        for (int j = 0; j < num_neigh[i]; ++j) {
            double *f = m->node_forces.p + 3 * ij;
            const double *x = xyz + 3 * ij;
            const double r_ij = r[ij];
            const double *R1_ij = m->R1.p + ij * m->nspl1;
            const double *R1d_ij = m->R1_deriv.p + ij * m->nspl1;
            const double *Y_ij = m->Y.p + ij * num_lm;
            const double *Yg = m->Y_grad.p + ij * 3 * num_lm;
            const double *H1_ij = m->H1.p + (size_t)neigh_indices[ij] * num_LM * K;
            int q = 0;
            for (int p = 0; p < m->num_paths; ++p) {
                const int l1 = m->Phi1_l1[p], l2 = m->Phi1_l2[p];
                const double *Rp = R1_ij + (size_t)p * K;
                const double *Rdp = R1d_ij + (size_t)p * K;
                for (int lm1 = l1 * l1; lm1 <= l1 * (l1 + 2); ++lm1) {
                    const double y = Y_ij[lm1];
                    const double gx = Yg[lm1], gy = Yg[num_lm + lm1], gz = Yg[2 * num_lm + lm1];
                    for (int lm2 = l2 * l2; lm2 <= l2 * (l2 + 2); ++lm2) {
                        const double *H = H1_ij + (size_t)lm2 * K;
                        const double *dq = dr + (size_t)q * K;
                        for (int k = 0; k < K; ++k) {
                            f[0] += -dq[k] * (x[0] / r_ij * Rdp[k] * y * H[k] + Rp[k] * gx * H[k]);
                            f[1] += -dq[k] * (x[1] / r_ij * Rdp[k] * y * H[k] + Rp[k] * gy * H[k]);
                            f[2] += -dq[k] * (x[2] / r_ij * Rdp[k] * y * H[k] + Rp[k] * gz * H[k]);
                        }
                        q += 1;
                    }
                }
            }
            ij += 1;
        }
    }
    vec_resize(&m->H1_adj, m->H1.n);
    if (zero_H1_adj) vec_fill(&m->H1_adj, 0.0);
    ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        const double *dr = m->dPhi1r.p + (size_t)i * nq * K;
        for (int j = 0; j < num_neigh[i]; ++j) {
            const double *R1_ij = m->R1.p + ij * m->nspl1;
            const double *Y_ij = m->Y.p + ij * num_lm;
            double *Ha = m->H1_adj.p + (size_t)neigh_indices[ij] * num_LM * K;
            int q = 0;
            for (int p = 0; p < m->num_paths; ++p) {
                const int l1 = m->Phi1_l1[p], l2 = m->Phi1_l2[p];
                const double *Rp = R1_ij + (size_t)p * K;
                for (int lm1 = l1 * l1; lm1 <= l1 * (l1 + 2); ++lm1) {
                    for (int lm2 = l2 * l2; lm2 <= l2 * (l2 + 2); ++lm2) {
                        double *o = Ha + (size_t)lm2 * K;
                        const double *dq = dr + (size_t)q * K;
                        for (int k = 0; k < K; ++k) o[k] += Rp[k] * Y_ij[lm1] * dq[k];
                        q += 1;
                    }
                }
            }
            ij += 1;
        }
    }
}

static void count_e(const orc_model *m, int *num_e)
{
    for (int l = 0; l <= m->l_max; ++l) num_e[l] = 0;
    for (int p = 0; p < m->num_paths; ++p) num_e[m->Phi1_l[p]] += 1;
}

/* mace.cpp:607-642 */
void orc_compute_A1(orc_model *m, int num_nodes)
{
    const int K = m->K, num_lm = m->num_lm;
    int num_e[8]; count_e(m, num_e);
    vec_resize(&m->A1, (size_t)num_nodes * num_lm * K);
    for (int i = 0; i < num_nodes; ++i) {
        const double *P = m->Phi1.p + (size_t)i * m->num_lme * K;
        double *A = m->A1.p + (size_t)i * num_lm * K;
        for (int l = 0; l <= m->l_max; ++l) {
            gemm_nn(2 * l + 1, K, num_e[l] * K, P, num_e[l] * K, m->A1_weights[l], K, A, K);
            P += (size_t)(2 * l + 1) * num_e[l] * K;
            A += (size_t)(2 * l + 1) * K;
        }
    }
}
/* mace.cpp:644-679 */
void orc_reverse_A1(orc_model *m, int num_nodes)
{
    const int K = m->K, num_lm = m->num_lm;
    int num_e[8]; count_e(m, num_e);
    vec_resize(&m->dPhi1, m->Phi1.n);
    for (int i = 0; i < num_nodes; ++i) {
        const double *Aa = m->A1_adj.p + (size_t)i * num_lm * K;
        double *d = m->dPhi1.p + (size_t)i * m->num_lme * K;
        for (int l = 0; l <= m->l_max; ++l) {
            gemm_nt(2 * l + 1, num_e[l] * K, K, Aa, K, m->A1_weights[l], K, d, num_e[l] * K);
            Aa += (size_t)(2 * l + 1) * K;
            d += (size_t)(2 * l + 1) * num_e[l] * K;
        }
    }
}

/* mace.cpp:759-777 */
void orc_compute_M1(orc_model *m, int num_nodes, const int *node_types)
{
    const int K = m->K, num_lm = m->num_lm;
    vec_resize(&m->M1, (size_t)num_nodes * K);
    vec_resize(&m->M1_grad, (size_t)num_nodes * K * num_lm);
    const orc_poly *P = &m->P1;
    double *nv = (double *)malloc((size_t)P->num_nodes * sizeof(double));
    double *na = (double *)malloc((size_t)P->num_nodes * sizeof(double));
    double x[64], g[64];
    for (int i = 0; i < num_nodes; ++i) {
        const double *A1_i = m->A1.p + (size_t)i * num_lm * K;
        for (int k = 0; k < K; ++k) {
            for (int q = 0; q < num_lm; ++q) x[q] = A1_i[(size_t)q * K + k];
            const double *coef = P->coef + ((size_t)node_types[i] * K + k) * P->num_nodes;
            m->M1.p[(size_t)i * K + k] = orc_poly_evaluate_gradient(P->num_variables, P->num_nodes, P->edges, coef, x, nv, na, g);
            for (int q = 0; q < num_lm; ++q) m->M1_grad.p[((size_t)i * num_lm + q) * K + k] = g[q];
        }
    }
    free(nv); free(na);
}
/* mace.cpp:779-794 */
void orc_reverse_M1(orc_model *m, int num_nodes)
{
    const int K = m->K, num_lm = m->num_lm;
    vec_resize(&m->A1_adj, m->A1.n);
    for (int i = 0; i < num_nodes; ++i)
        for (int lm = 0; lm < num_lm; ++lm)
            for (int k = 0; k < K; ++k)
                m->A1_adj.p[((size_t)i * num_lm + lm) * K + k] =
                    m->M1_grad.p[((size_t)i * num_lm + lm) * K + k] * m->M1_adj.p[(size_t)i * K + k];
}

/* mace.cpp:796-832 */
void orc_compute_H2(orc_model *m, int num_nodes, const int *node_types)
{
    const int K = m->K, num_LM = m->num_LM;
    vec_resize(&m->H2, (size_t)num_nodes * K);
    for (int i = 0; i < num_nodes; ++i) {
        double *H2_i = m->H2.p + (size_t)i * K;
        const double *H1_i = m->H1.p + (size_t)i * num_LM * K;
        const double *M1_i = m->M1.p + (size_t)i * K;
        const double *W1 = m->H2_weights_for_H1 + (size_t)node_types[i] * K * K;
        const double *W2 = m->H2_weights_for_M1;
        for (int k = 0; k < K; ++k) H2_i[k] = 0.0;
        for (int kp = 0; kp < K; ++kp) for (int k = 0; k < K; ++k) H2_i[k] += W1[(size_t)kp * K + k] * H1_i[kp];
        for (int kp = 0; kp < K; ++kp) for (int k = 0; k < K; ++k) H2_i[k] += W2[(size_t)kp * K + k] * M1_i[kp];
    }
}
/* mace.cpp:834-874 */
void orc_reverse_H2(orc_model *m, int num_nodes, const int *node_types, int zero_H1_adj)
{
    const int K = m->K, num_LM = m->num_LM;
    vec_resize(&m->H1_adj, m->H1.n); vec_resize(&m->M1_adj, m->M1.n);
    if (zero_H1_adj) vec_fill(&m->H1_adj, 0.0);
    for (int i = 0; i < num_nodes; ++i) {
        const double *H2a = m->H2_adj.p + (size_t)i * K;
        double *H1a = m->H1_adj.p + (size_t)i * num_LM * K;
        double *M1a = m->M1_adj.p + (size_t)i * K;
        const double *W1 = m->H2_weights_for_H1 + (size_t)node_types[i] * K * K;
        const double *W2 = m->H2_weights_for_M1;
        for (int kp = 0; kp < K; ++kp) {
            double s = 0.0, t = 0.0;
            for (int k = 0; k < K; ++k) { s += W1[(size_t)kp * K + k] * H2a[k]; t += W2[(size_t)kp * K + k] * H2a[k]; }
            H1a[kp] += s; M1a[kp] = t;
        }
    }
}

/* mace.cpp:876-903 */
void orc_compute_readouts(orc_model *m, int num_nodes, const int *node_types)
{
    const int K = m->K, num_LM = m->num_LM;
    vec_resize(&m->node_energies, (size_t)num_nodes);
    vec_resize(&m->H1_adj, m->H1.n); vec_fill(&m->H1_adj, 0.0);
    vec_resize(&m->H2_adj, m->H2.n);
    const int shape[3] = {K, 16, 1};
    const double *W[2] = {m->readout_2_w1, m->readout_2_w2};
    for (int i = 0; i < num_nodes; ++i) {
        m->node_energies.p[i] += m->atomic_energies[node_types[i]];
        for (int k = 0; k < K; ++k) {
            m->node_energies.p[i] += m->readout_1_weights[k] * m->H1.p[(size_t)i * num_LM * K + k];
            m->H1_adj.p[(size_t)i * num_LM * K + k] = m->readout_1_weights[k];
        }
        m->node_energies.p[i] += orc_mlp_evaluate_gradient(3, shape, W, m->readout_2_scale,
                                                           m->H2.p + (size_t)i * K, m->H2_adj.p + (size_t)i * K);
    }
}

/* zbl.cpp:96-125 */
void orc_compute_ZBL(orc_model *m, int num_nodes, const int *node_types, const int *num_neigh,
                     const int *neigh_types, const double *r, const double *xyz)
{
    size_t ij = 0;
    for (int i = 0; i < num_nodes; ++i) {
        const int Zi = m->atomic_numbers[node_types[i]];
        for (int j = 0; j < num_neigh[i]; ++j) {
            const int Zj = m->atomic_numbers[neigh_types[ij]];
            double f, d;
            orc_zbl_compute(&m->zbl, Zi, Zj, r[ij], &f, &d);
            m->node_energies.p[i] += f;
            m->node_forces.p[3 * ij] -= d * xyz[3 * ij] / r[ij];
            m->node_forces.p[3 * ij + 1] -= d * xyz[3 * ij + 1] / r[ij];
            m->node_forces.p[3 * ij + 2] -= d * xyz[3 * ij + 2] / r[ij];
            ij += 1;
        }
    }
}

/* mace.cpp:17-64 */
int orc_compute_node_energies_forces(orc_model *m, int num_nodes, const int *node_types,
                                     const int *num_neigh, const int *neigh_indices,
                                     const int *neigh_types, const double *xyz, const double *r, long E)
{
    const long n3 = 3 * E;
    vec_resize(&m->node_energies, (size_t)num_nodes); vec_fill(&m->node_energies, 0.0);
    vec_resize(&m->node_forces, (size_t)n3); vec_fill(&m->node_forces, 0.0);
    if (m->has_zbl) orc_compute_ZBL(m, num_nodes, node_types, num_neigh, neigh_types, r, xyz);
    orc_compute_Y(m, xyz, n3);
    orc_compute_R0(m, num_nodes, node_types, num_neigh, neigh_types, r, E);
    orc_compute_A0(m, num_nodes, node_types, num_neigh, neigh_types);
    if (orc_compute_A0_scaled(m, num_nodes, node_types, num_neigh, neigh_types, r)) return -1;
    orc_compute_M0(m, num_nodes, node_types);
    orc_compute_H1(m, num_nodes);
    orc_compute_R1(m, num_nodes, node_types, num_neigh, neigh_types, r, E);
    orc_compute_Phi1(m, num_nodes, num_neigh, neigh_indices);
    orc_compute_A1(m, num_nodes);
    if (orc_compute_A1_scaled(m, num_nodes, node_types, num_neigh, neigh_types, r)) return -1;
    orc_compute_M1(m, num_nodes, node_types);
    orc_compute_H2(m, num_nodes, node_types);
    orc_compute_readouts(m, num_nodes, node_types);
    orc_reverse_H2(m, num_nodes, node_types, 0);
    orc_reverse_M1(m, num_nodes);
    if (orc_reverse_A1_scaled(m, num_nodes, node_types, num_neigh, neigh_types, xyz, r, n3, 0)) return -1;
    orc_reverse_A1(m, num_nodes);
    orc_reverse_Phi1(m, num_nodes, num_neigh, neigh_indices, xyz, r, n3, 0, 0);
    orc_reverse_H1(m, num_nodes);
    orc_reverse_M0(m, num_nodes);
    if (orc_reverse_A0_scaled(m, num_nodes, node_types, num_neigh, neigh_types, xyz, r)) return -1;
    orc_reverse_A0(m, num_nodes, node_types, num_neigh, neigh_types, xyz, r);
    return 0;
}
