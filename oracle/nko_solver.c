/*
 * CPU oracle (test infrastructure; see nuka_oracle.h): augmented-Lagrangian row math and the UABD
 * tile block-descent solve of one environment with one articulated block, restated from
 * src/phi/backend_cuda/ops/block_descent_tile.cuh and block_descent.cu.
 *
 * Where the reference reduces across a 32-lane warp with a shuffle tree, the oracle adds in index
 * order; the compensated TileSum arithmetic, fmaf uses and branch structure are kept.  Free rigid
 * bodies (6x6 blocks) and mimic couplings are outside this restatement.
 */
#include <stdio.h>

#include "nko_internal.h"

typedef struct { float value, error; } tile_sum;   /* block_descent_tile.cuh:15-31 */
static void tile_add(tile_sum* s, float x) {
    const float sum = s->value + x;
    const float part = sum - s->value;
    s->error += (s->value - (sum - part)) + (x - part);
    s->value = sum;
}
static void tile_add_product(tile_sum* s, float a, float b) {
    const float product = a * b;
    s->error += fmaf(a, b, -product);
    tile_add(s, product);
}

/* ---- nk/solve/augmented_row.hpp ------------------------------------------ */

typedef struct { float dual_scale, residual_scale; } scalar_response;
static scalar_response float_scalar_response(float cap, float compliance) {   /* :226-229 */
    const float product = cap * compliance;
    scalar_response r;
    if (product >= 1.0f) { r.dual_scale = 0.0f; r.residual_scale = 1.0f / compliance; }
    else { r.dual_scale = 1.0f - product; r.residual_scale = cap; }
    return r;
}

/* :232-247 EvaluateScalarImpulse (float response): impulse, curvature */
static void scalar_impulse(float dual, float rho, float residual, float compliance, float lower, float upper,
                           scalar_response response, float* impulse, float* curvature) {
    *impulse = 0.0f; *curvature = 0.0f;
    if (rho <= 0.0f) return;
    if (dual != dual || rho != rho || residual != residual || compliance != compliance || lower != lower || upper != upper) {
        const float invalid = dual + rho + residual + compliance + lower + upper;
        *impulse = invalid; *curvature = invalid;
        return;
    }
    const float k = response.residual_scale;
    const float x = fmaf(k, residual, response.dual_scale * dual);
    *impulse = x < lower ? lower : (x > upper ? upper : x);
    *curvature = x != x ? x : (lower < upper && x >= lower && x <= upper ? k : 0.0f);
}

void nko_scalar_impulse(float dual, float rho, float residual, float compliance, float lower, float upper, float out[2]) {
    scalar_impulse(dual, rho, residual, compliance, lower, upper, float_scalar_response(rho, compliance), &out[0], &out[1]);
}

/* :302-318 ConeArgument */
static float cone_argument(float dual, float rho, float mu, float residual) {
    const int dual_zero = dual == 0.0f;
    const float dual_quotient = (dual + (float)dual_zero) / mu;
    const float d = dual_zero ? dual : dual_quotient;
    const float low = fmaf(-d, mu, dual);
    const int low_zero = low == 0.0f;
    const float low_quotient = (low + (float)low_zero) / mu;
    const float d_low = low_zero ? low : low_quotient;
    const float p = rho * mu;
    const float t = p * residual;
    const float t_low = fmaf(p, residual, -t) + fmaf(rho, mu, -p) * residual;
    const float sum = d + t;
    const float t_part = sum - d;
    const float sum_low = (d - (sum - t_part)) + (t - t_part);
    return sum + (sum_low + d_low + t_low);
}

/* :321-348 EvaluateTangentImpulse; curvature = {xx,yy,zz,xy,xz,yz} */
static void tangent_impulse(v3 dual, float rho, v3 residual, float normal_impulse, float mu_first, float mu_second,
                            v3* impulse, float* c) {
    *impulse = v3_make(0, 0, 0);
    for (int i = 0; i < 6; ++i) c[i] = 0.0f;
    if (rho <= 0.0f) return;
    const float scale = fmaxf(mu_first, mu_second);
    const float mu_y = mu_first <= 0.0f ? 0.0f : mu_first / scale;
    const float mu_z = mu_second <= 0.0f ? 0.0f : mu_second / scale;
    const float q_y = mu_y == 0.0f ? 0.0f : cone_argument(dual.y, rho, mu_y, residual.y);
    const float q_z = mu_z == 0.0f ? 0.0f : cone_argument(dual.z, rho, mu_z, residual.z);
    const float radius = (normal_impulse < 0.0f ? 0.0f : normal_impulse) * fmaxf(scale, 0.0f);
    if (q_y != q_y || q_z != q_z || radius != radius || rho != rho) {
        const float invalid = q_y + q_z + radius + rho;
        *impulse = v3_make(0.0f, invalid, invalid);
        c[1] = invalid; c[2] = invalid; c[5] = invalid;
        return;
    }
    if (radius == 0.0f) return;
    const float norm = hypotf(q_y, q_z);
    if (norm <= radius) {
        *impulse = v3_make(0.0f, mu_y * q_y, mu_z * q_z);
        c[1] = rho * mu_y * mu_y; c[2] = rho * mu_z * mu_z;
        return;
    }
    const float dy = q_y / norm, dz = q_z / norm;
    const float cs = rho * radius / norm;
    *impulse = v3_make(0.0f, mu_y * radius * dy, mu_z * radius * dz);
    c[1] = cs * mu_y * mu_y * dz * dz; c[2] = cs * mu_z * mu_z * dy * dy; c[5] = -cs * mu_y * mu_z * dy * dz;
}

void nko_tangent_impulse(const float dual[3], float rho, const float residual[3], float normal_impulse,
                         float mu_first, float mu_second, float impulse[3], float curvature[6]) {
    v3 f;
    tangent_impulse(v3_make(dual[0], dual[1], dual[2]), rho, v3_make(residual[0], residual[1], residual[2]), normal_impulse,
                    mu_first, mu_second, &f, curvature);
    impulse[0] = f.x; impulse[1] = f.y; impulse[2] = f.z;
}

typedef struct { v3 step; float weight; v3 point; } relaxation;
/* :128-138 RelaxContactImpulse */
static v3 relax_contact_impulse(v3 dual, v3 next, relaxation* last) {
    const v3 step = v3_make(next.x - dual.x, next.y - dual.y, next.z - dual.z);
    const v3 change = v3_make(step.x - last->step.x, step.y - last->step.y, step.z - last->step.z);
    const v3 moved = v3_sub(dual, last->point);
    const float square = change.x * change.x + change.y * change.y + change.z * change.z;
    const float along = -(moved.x * change.x + moved.y * change.y + moved.z * change.z);
    float weight = 1.0f;
    if (last->weight > 0.0f && along > 0.0f && square > 0.0f) weight = fminf(1.0f, along / square);
    last->step = step; last->weight = weight; last->point = dual;
    return v3_make(dual.x + weight * step.x, dual.y + weight * step.y, dual.z + weight * step.z);
}

void nko_relax_contact_impulse(const float dual[3], const float next[3], float last_step[3], float* last_weight,
                               float last_point[3], float out[3]) {
    relaxation r;
    r.step = v3_make(last_step[0], last_step[1], last_step[2]); r.weight = *last_weight;
    r.point = v3_make(last_point[0], last_point[1], last_point[2]);
    const v3 o = relax_contact_impulse(v3_make(dual[0], dual[1], dual[2]), v3_make(next[0], next[1], next[2]), &r);
    last_step[0] = r.step.x; last_step[1] = r.step.y; last_step[2] = r.step.z; *last_weight = r.weight;
    last_point[0] = r.point.x; last_point[1] = r.point.y; last_point[2] = r.point.z;
    out[0] = o.x; out[1] = o.y; out[2] = o.z;
}

/* :119-124 MultiplierMomentumRestart */
static double momentum_restart(v3 point, v3 next, v3 base, v3 scale) {
    return (scale.x > 0.0f ? ((double)point.x - next.x) * ((double)next.x - base.x) / scale.x : 0.0) +
           (scale.y > 0.0f ? ((double)point.y - next.y) * ((double)next.y - base.y) / scale.y : 0.0) +
           (scale.z > 0.0f ? ((double)point.z - next.z) * ((double)next.z - base.z) / scale.z : 0.0);
}

/* ---- block_descent.cu helpers --------------------------------------------- */

float nko_cone_argument(float dual, float rho, float mu, float residual) { return cone_argument(dual, rho, mu, residual); }
double nko_momentum_restart(const float point[3], const float next[3], const float base[3], const float scale[3]) {
    return momentum_restart(v3_make(point[0], point[1], point[2]), v3_make(next[0], next[1], next[2]),
                            v3_make(base[0], base[1], base[2]), v3_make(scale[0], scale[1], scale[2]));
}
/* ---- the compliant (MuJoCo-law) row terms and the elliptic cone.  The product builds rows of the native law only
 * (compliance 0, Coulomb disc): these restatements have no device counterpart and exist so that the reference's known
 * answers for them (tests/constraint/test_solref_solimp.cpp) are held and checked here too. ---- */
static float clampf(float v, float lo, float hi) { return fminf(fmaxf(v, lo), hi); }
/* constraint/solref_solimp.hpp:55-86 ComputeCompliantRowTerms -> k, b, imp, D, R, aref */
void nko_compliant_row_terms(const float solref[2], const float solimp[5], float pos_imp, float pos_aref, float vel, float invweight,
                             float dt, int refsafe, float out[6]) {
    float timeconst = solref[0];
    const float dampratio = solref[1];
    if (refsafe) timeconst = fmaxf(timeconst, 2.0f * dt);
    const float dmin = clampf(solimp[0], 1.0e-4f, 0.9999f), dmax = clampf(solimp[1], 1.0e-4f, 0.9999f);
    const float width = fmaxf(1.0e-15f, solimp[2]);
    const float mid = clampf(solimp[3], 1.0e-4f, 0.9999f);
    const float power = fmaxf(1.0f, solimp[4]);
    const float dmax_sq = dmax * dmax;
    float k = 1.0f / (dmax_sq * timeconst * timeconst * dampratio * dampratio);
    float b = 2.0f / (dmax * timeconst);
    if (solref[0] <= 0.0f) k = -solref[0] / dmax_sq;
    if (solref[1] <= 0.0f) b = -solref[1] / dmax;
    const float x = fabsf(pos_imp) / width;
    const float rising = (1.0f / powf(mid, power - 1.0f)) * powf(x, power);
    const float falling = 1.0f - (1.0f / powf(1.0f - mid, power - 1.0f)) * powf(1.0f - x, power);
    const float y = x < mid ? rising : falling;
    float imp = clampf(dmin + y * (dmax - dmin), dmin, dmax);
    if (x > 1.0f) imp = dmax;
    const float D = 1.0f / fmaxf(invweight * (1.0f - imp) / imp, 1.0e-15f);
    out[0] = k; out[1] = b; out[2] = imp; out[3] = D; out[4] = 1.0f / D; out[5] = -k * imp * pos_aref - b * vel;
}
/* constraint/solref_solimp.hpp:40-44 DiscretizeCompliantRow -> R, bias, reference gain (midpoint damping) */
void nko_discretize_compliant_row(float R, float aref_bias, float damping, float dt, float out[3]) {
    const double scale = 1.0 + 0.5 * (double)dt * damping;
    out[0] = (float)(R / scale); out[1] = (float)(aref_bias / scale); out[2] = (float)((1.0 / (double)dt - 0.5 * damping) / scale);
}
/* augmented_row.hpp:48-55 ComputeEllipticResponse -> residual scale k[3], dual scale s[3] */
static void elliptic_response(float cap, v3 compliance, v3* k, v3* s) {
    const double tangent = fmin((double)compliance.y, (double)compliance.z);
    const double normal_scale = 1.0 / (1.0 + (double)cap * compliance.x);
    const double tangent_scale = 1.0 / (1.0 + (double)cap * tangent);
    *k = v3_make((float)(cap * normal_scale), (float)(cap * tangent_scale * tangent / compliance.y), (float)(cap * tangent_scale * tangent / compliance.z));
    *s = v3_make((float)normal_scale, (float)tangent_scale, (float)tangent_scale);
}
/* augmented_row.hpp:58-80 EvaluateEllipticImpulse -> impulse[3], curvature xx yy zz xy xz yz: the projection onto the
 * friction cone in the metric that makes its cross section a circle */
void nko_elliptic_impulse(const float dual[3], float cap, const float residual[3], const float compliance[3], float mu_first, float out[9]) {
    v3 k, s;
    elliptic_response(cap, v3_make(compliance[0], compliance[1], compliance[2]), &k, &s);
    const v3 x = v3_make(fmaf(k.x, residual[0], s.x * dual[0]), fmaf(k.y, residual[1], s.y * dual[1]), fmaf(k.z, residual[2], s.z * dual[2]));
    const v3 root = v3_make(sqrtf(k.x), sqrtf(k.y), sqrtf(k.z));
    const float m = mu_first * root.x / root.y;
    const float p = x.x / root.x, q1 = x.y / root.y, q2 = x.z / root.z;
    const float t = hypotf(q1, q2);
    for (int i = 0; i < 9; ++i) out[i] = 0.0f;
    if (t <= m * p) { out[0] = x.x; out[1] = x.y; out[2] = x.z; out[3] = k.x; out[4] = k.y; out[5] = k.z; return; }
    if (m * t + p <= 0.0f) return;
    const float a = 1.0f / (1.0f + m * m);
    const float projected = (p + m * t) * a;
    const float u1 = q1 / t, u2 = q2 / t;
    const float b = m * projected / t, along = m * m * a;
    out[0] = projected * root.x; out[1] = m * projected * u1 * root.y; out[2] = m * projected * u2 * root.z;
    out[3] = k.x * a; out[4] = k.y * (along * u1 * u1 + b * u2 * u2); out[5] = k.z * (along * u2 * u2 + b * u1 * u1);
    out[6] = root.x * root.y * m * a * u1; out[7] = root.x * root.z * m * a * u2; out[8] = root.y * root.z * (along - b) * u1 * u2;
}
/* augmented_row.hpp:104-108 EllipticMultiplierStep */
void nko_elliptic_multiplier_step(const float dual[3], const float next[3], float cap, const float compliance[3], float out[3]) {
    v3 k, s;
    elliptic_response(cap, v3_make(compliance[0], compliance[1], compliance[2]), &k, &s);
    out[0] = fabsf(next[0] - dual[0]) / k.x; out[1] = fabsf(next[1] - dual[1]) / k.y; out[2] = fabsf(next[2] - dual[2]) / k.z;
}

static uint32_t residual_bits(float value) { return f2u(value <= FLT_MAX ? fabsf(value) : FLT_MAX); }   /* :735 */
static float along_axis(float impulse, float velocity) { return impulse > 0.0f ? velocity : impulse < 0.0f ? -velocity : 0.0f; }   /* :773-775 */

/* :761-770 MultiplierSteps -> {normal, tangent} */
static void multiplier_steps(v3 dual, v3 next, float scale, float dual_scale, float rho, float mu_first, float mu_second, float* out) {
    const float normal = scale > 0.0f && dual_scale != 0.0f ? fabsf(next.x - dual.x) / scale : 0.0f;
    const float fs = fmaxf(mu_first, mu_second);
    mu_first = mu_first <= 0.0f ? 0.0f : mu_first / fs;
    mu_second = mu_second <= 0.0f ? 0.0f : mu_second / fs;
    const float first = mu_first > 0.0f && rho > 0.0f ? (next.y - dual.y) / (rho * mu_first * mu_first) : 0.0f;
    const float second = mu_second > 0.0f && rho > 0.0f ? (next.z - dual.z) / (rho * mu_second * mu_second) : 0.0f;
    out[0] = normal; out[1] = hypotf(first, second);
}

typedef struct { float t, beta; uint32_t restarts; } dual_momentum;
static void advance_dual_momentum(dual_momentum* m, double restart) {   /* :780-788 */
    if (restart > 0.0) { m->t = 1.0f; ++m->restarts; }
    const float t = 0.5f * (1.0f + sqrtf(fmaf(4.0f * m->t, m->t, 1.0f)));
    m->beta = (m->t - 1.0f) / t;
    m->t = t;
}
static v3 multiplier_metric(float scale, float rho, int contact, float mu_first, float mu_second) {   /* :790-795 */
    const float friction = fmaxf(mu_first, mu_second);
    const float first = contact && mu_first > 0.0f ? mu_first / friction : 0.0f;
    const float second = contact && mu_second > 0.0f ? mu_second / friction : 0.0f;
    return v3_make(scale, rho * first * first, rho * second * second);
}
/* :808-820 ExtrapolateDual */
static v3 extrapolate_dual(v3 base, v3 next, float beta, float lower, float upper, int contact, float mu_first, float mu_second) {
    if (beta == 0.0f) return next;
    v3 y = v3_make(fmaf(beta, next.x - base.x, next.x), fmaf(beta, next.y - base.y, next.y), fmaf(beta, next.z - base.z, next.z));
    y.x = fminf(fmaxf(y.x, lower), upper);
    if (!contact) return v3_make(y.x, 0.0f, 0.0f);
    const float first = mu_first > 0.0f ? y.y / mu_first : 0.0f;
    const float second = mu_second > 0.0f ? y.z / mu_second : 0.0f;
    const float slip = hypotf(first, second), radius = fmaxf(y.x, 0.0f);
    const float scale = slip > radius ? radius / slip : 1.0f;
    return v3_make(y.x, mu_first > 0.0f ? y.y * scale : 0.0f, mu_second > 0.0f ? y.z * scale : 0.0f);
}

/* ---- the tile ------------------------------------------------------------ */

#define NO_BLOCK 0xFFFFFFFFu

typedef struct {
    uint32_t slot, stride, axes, owner[2], unit[2], row[2];
    float unit_value[2];
    float rho, compliance, lower, upper, mu_first, mu_second, normal_bound;
    int elliptic;            /* three axes of a MuJoCo-law contact: the elliptic cone (block_descent_tile.cuh:645, 778) */
    v3 cone_compliance;      /* the compliances of the normal row and of its two tangent rows */
    v3 residual, dual, move, step, base;
    scalar_response response;
    relaxation relax;
} tile_head;

typedef struct {
    nko_world* w;
    uint32_t env, n, width, heads, iteration, incident_count;
    tile_head* head;
    uint32_t* incident;
    float* jac;          /* staged rows: [row][width] */
    float mass[NKO_MAX_DOF][NKO_MAX_DOF + 1];
    float momentum, residual;
    float tolerance;
    int failed;
} tile;

/* TileResponse (block_descent_tile.cuh:678-681) with EvaluateAugmentedResponse (block_descent.cu:1593-1621), Coulomb cone */
static void tile_response(const tile_head* t, v3 move, v3* f, float* c) {
    if (t->elliptic) {   /* block_descent.cu:1595-1601 */
        const float dual[3] = {t->dual.x, t->dual.y, t->dual.z};
        const float residual[3] = {t->residual.x - move.x, t->residual.y - move.y, t->residual.z - move.z};
        const float compliance[3] = {t->cone_compliance.x, t->cone_compliance.y, t->cone_compliance.z};
        float out[9];
        nko_elliptic_impulse(dual, t->rho, residual, compliance, t->mu_first, out);
        *f = v3_make(out[0], out[1], out[2]);
        for (int i = 0; i < 6; ++i) c[i] = out[3 + i];
        return;
    }
    float ni, nc;
    scalar_impulse(t->dual.x, t->rho, t->residual.x - move.x, t->compliance, t->lower, t->upper, t->response, &ni, &nc);
    *f = v3_make(ni, 0.0f, 0.0f);
    c[0] = nc; c[1] = c[2] = c[3] = c[4] = c[5] = 0.0f;
    if (t->axes != 3u) return;
    v3 ft; float ct[6];
    tangent_impulse(t->dual, t->rho, v3_make(0.0f, t->residual.y - move.y, t->residual.z - move.z), t->normal_bound,
                    t->mu_first, t->mu_second, &ft, ct);
    f->y = ft.y; f->z = ft.z;
    c[1] = ct[1]; c[2] = ct[2]; c[5] = ct[5];
}

/* FactorTileBlock + SolveTileBlock (:1622-1666): left-looking Cholesky by rows, fma substitutions */
static int cholesky_solve(float h[NKO_MAX_DOF][NKO_MAX_DOF + 1], uint32_t n, const float* g, float* d) {
    float inverse[NKO_MAX_DOF];
    int valid = 1;
    for (uint32_t k = 0u; k < n; ++k) {
        float pivot = 0.0f;
        float column[NKO_MAX_DOF];
        for (uint32_t i = 0u; i < n; ++i) {
            float value = h[i][k];
            for (uint32_t j = 0u; j < k; ++j) value -= h[i][j] * h[k][j];
            column[i] = value;
            if (i == k) pivot = value;
        }
        if (valid && !(pivot > 0.0f && pivot <= FLT_MAX) && getenv("NKO_TRACE_FAILURES") != NULL)
            fprintf(stderr, "nko: pivot %u of %u is %g (diagonal entry %g)\n", k, n, pivot, h[k][k]);
        valid = valid && pivot > 0.0f && pivot <= FLT_MAX;
        const float root = sqrtf(valid ? pivot : 1.0f);
        const float scale = 1.0f / root;
        for (uint32_t i = 0u; i < n; ++i) h[i][k] = i == k ? root : column[i] * scale;
        inverse[k] = scale;
    }
    if (!valid) return 0;
    float r[NKO_MAX_DOF];
    for (uint32_t i = 0u; i < n; ++i) r[i] = g[i];
    for (uint32_t j = 0u; j < n; ++j) {
        const float y = r[j] * inverse[j];
        r[j] = y;
        for (uint32_t i = j + 1u; i < n; ++i) r[i] = fmaf(-h[i][j], y, r[i]);
    }
    for (uint32_t k = n; k > 0u; --k) {
        const uint32_t j = k - 1u;
        const float x = r[j] * inverse[j];
        r[j] = x;
        for (uint32_t i = 0u; i < j; ++i) r[i] = fmaf(-h[j][i], x, r[i]);
    }
    for (uint32_t i = 0u; i < n; ++i) d[i] = r[i];
    return 1;
}

/* Past a warp of coordinates (TileSpan > 1: more than 32) the reference factors H = U U^T from the last coordinate
 * down, "so a tree's leaves go first".  FactorTileColumns (:212-252): left-looking; the dot of row i with the pivot row
 * over the finished columns k+2.. is split over four partial sums in runs of eight columns, the first of which takes
 * the still unscaled column k+1 last, and the four are added pairwise.  SolveWideTileBlock (:1866-1895): U w = g up
 * the columns, then U^T d = w down the rows.  Only the upper triangle of h is read. */
static int cholesky_solve_wide(float h[NKO_MAX_DOF][NKO_MAX_DOF + 1], uint32_t n, const float* g, float* d) {
    float inverse[NKO_MAX_DOF], raw[2][NKO_MAX_DOF];
    int valid = 1;
    for (uint32_t kk = n; kk > 0u; --kk) {
        const uint32_t k = kk - 1u;
        const float* last = raw[(k + 1u) % 2u];
        float* next = raw[k % 2u];
        const int scaled = k + 1u < n;
        const float scale = scaled ? inverse[k + 1u] : 0.0f;
        float pivot = 0.0f;
        for (uint32_t i = 0u; i <= k; ++i) {
            float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (uint32_t p = 0u; p < 4u; ++p) {
                for (uint32_t m = 0u; m < 16u; ++m) {
                    const uint32_t j = k + 2u + 8u * p + m % 8u + 32u * (m / 8u);
                    if (j < n) part[p] = fmaf(h[i][j], h[k][j], part[p]);
                }
                if (p == 0u && scaled) part[p] = fmaf(last[i] * scale, last[k] * scale, part[p]);
            }
            const float sum = (part[0] + part[1]) + (part[2] + part[3]);
            if (i < k) next[i] = h[i][k] - sum;
            else pivot = h[i][k] - sum;
        }
        if (scaled) for (uint32_t i = 0u; i <= k; ++i) h[i][k + 1u] = last[i] * scale;
        /* a failed pivot leaves every later root at one */
        if (valid && !(pivot > 0.0f && pivot <= FLT_MAX) && getenv("NKO_TRACE_FAILURES") != NULL)
            fprintf(stderr, "nko: pivot %u of %u is %g (diagonal entry %g)\n", k, n, pivot, h[k][k]);
        valid = valid && pivot > 0.0f && pivot <= FLT_MAX;
        const float root = sqrtf(valid ? pivot : 1.0f);
        h[k][k] = root;
        inverse[k] = 1.0f / root;
    }
    if (!valid) return 0;
    float r[NKO_MAX_DOF];
    for (uint32_t i = 0u; i < n; ++i) r[i] = g[i];
    for (uint32_t jj = n; jj > 0u; --jj) {
        const uint32_t j = jj - 1u;
        const float y = r[j] * inverse[j];
        r[j] = y;
        for (uint32_t i = 0u; i < j; ++i) r[i] = fmaf(-h[i][j], y, r[i]);
    }
    for (uint32_t j = 0u; j < n; ++j) {
        const float x = r[j] * inverse[j];
        r[j] = x;
        for (uint32_t i = j + 1u; i < n; ++i) r[i] = fmaf(-h[j][i], x, r[i]);
    }
    for (uint32_t i = 0u; i < n; ++i) d[i] = r[i];
    return 1;
}

/* the reference's tile width decides the route: TileSpan (:71-73) over 32-lane warps */
static int wide_tile(uint32_t n) { return n > 32u; }

/* The block factorisation by itself, for unit pins: h is n x n row-major; on return factor (n x n) holds the
 * triangular factor the route of this width builds (lower L with h = L L^T up to 32 coordinates, upper U with
 * h = U U^T past them) and d the solution of h d = g.  Returns 0 when a pivot fails. */
int nko_tile_cholesky_solve(const float* h_in, uint32_t n, const float* g, float* factor, float* d) {
    static _Thread_local float h[NKO_MAX_DOF][NKO_MAX_DOF + 1];
    if (n == 0u || n > NKO_MAX_DOF) return 0;
    for (uint32_t i = 0u; i < n; ++i) for (uint32_t j = 0u; j < n; ++j) h[i][j] = h_in[(size_t)i * n + j];
    const int valid = wide_tile(n) ? cholesky_solve_wide(h, n, g, d) : cholesky_solve(h, n, g, d);
    for (uint32_t i = 0u; i < n; ++i)
        for (uint32_t j = 0u; j < n; ++j)
            factor[(size_t)i * n + j] = (wide_tile(n) ? j >= i : j <= i) ? h[i][j] : 0.0f;
    return valid;
}

/* AssembleTileBlock (:1507-1618) */
static int assemble_block(tile* c, const float* u, const float* free_v, float h[NKO_MAX_DOF][NKO_MAX_DOF + 1],
                          float* force, float* inertia, int* converged) {
    const uint32_t n = c->n;
    float difference[NKO_MAX_DOF], difference_error[NKO_MAX_DOF], scale[NKO_MAX_DOF], diagonal[NKO_MAX_DOF];
    tile_sum g[NKO_MAX_DOF], inertial[NKO_MAX_DOF];
    for (uint32_t i = 0u; i < n; ++i) {
        difference[i] = u[i] - free_v[i];
        const float part = difference[i] - u[i];
        difference_error[i] = (u[i] - (difference[i] - part)) + (-free_v[i] - part);
    }
    for (uint32_t i = 0u; i < n; ++i) {
        inertial[i].value = inertial[i].error = 0.0f;
        scale[i] = 0.0f; diagonal[i] = 0.0f;
        for (uint32_t k = 0u; k < n; ++k) {
            const float mass = c->mass[i][k];
            h[i][k] = mass;
            tile_add_product(&inertial[i], mass, difference[k]);
            tile_add_product(&inertial[i], mass, difference_error[k]);
            scale[i] += fabsf(mass) * fabsf(difference[k]);
        }
        g[i].value = -inertial[i].value; g[i].error = -inertial[i].error;
    }
    for (uint32_t chunk = 0u; chunk < c->incident_count; chunk += 32u) {
        const uint32_t end = chunk + 32u < c->incident_count ? chunk + 32u : c->incident_count;
        for (int pass = 0; pass < 2; ++pass)
            for (uint32_t k = chunk; k < end; ++k) {
                tile_head* t = &c->head[c->incident[k]];
                const uint32_t incidence = t->owner[0] == 0u ? 0u : 1u;
                const uint32_t unit = t->unit[incidence];
                if ((pass == 0) != (unit != NO_BLOCK)) continue;
                v3 f; float cv[6];
                tile_response(t, t->move, &f, cv);
                const v3 noise = v3_make(fabsf(f.x) + cv[0] * (fabsf(t->residual.x) + fabsf(t->move.x)),
                                         fabsf(f.y) + cv[1] * (fabsf(t->residual.y) + fabsf(t->move.y)),
                                         fabsf(f.z) + cv[2] * (fabsf(t->residual.z) + fabsf(t->move.z)));
                const int contributes = f.x != 0.0f || f.y != 0.0f || f.z != 0.0f || cv[0] != 0.0f || cv[1] != 0.0f || cv[2] != 0.0f ||
                    cv[5] != 0.0f || cv[3] != 0.0f || cv[4] != 0.0f || noise.x != 0.0f || noise.y != 0.0f || noise.z != 0.0f;
                if (!contributes) continue;
                if (unit != NO_BLOCK) {
                    const float v = t->unit_value[incidence];
                    diagonal[unit] += v * cv[0] * v;
                    tile_add_product(&g[unit], v, f.x);
                    scale[unit] += fabsf(v) * noise.x;
                    continue;
                }
                const float* j0r = c->jac + (size_t)t->row[incidence] * c->width;
                const float* j1r = j0r + c->width, *j2r = j0r + 2u * c->width;
                for (uint32_t i = 0u; i < n; ++i) {
                    const float j0 = j0r[i];
                    tile_add_product(&g[i], j0, f.x);
                    scale[i] += fabsf(j0) * noise.x;
                    if (t->axes == 1u) {
                        const float a0 = j0 * cv[0];
                        /* h += a0 j: one product added to the entry, which the reference's compiler contracts to one fused
                         * multiply-add (:1581-1585) */
                        for (uint32_t kk = wide_tile(n) ? i : 0u; kk < n; ++kk) h[i][kk] = fmaf(a0, j0r[kk], h[i][kk]);
                        continue;
                    }
                    const float j1 = j1r[i], j2 = j2r[i];
                    tile_add_product(&g[i], j1, f.y);
                    tile_add_product(&g[i], j2, f.z);
                    scale[i] += fabsf(j1) * noise.y + fabsf(j2) * noise.z;
                    const float a0 = (j0 * cv[0] + j1 * cv[3]) + j2 * cv[4];
                    const float a1 = (j1 * cv[1] + j2 * cv[5]) + j0 * cv[3];
                    const float a2 = (j2 * cv[2] + j1 * cv[5]) + j0 * cv[4];
                    if (wide_tile(n)) {   /* AssembleTileChunk (:170-190): the upper triangle, one fused product per staged row */
                        for (uint32_t kk = i; kk < n; ++kk) h[i][kk] = fmaf(a2, j2r[kk], fmaf(a1, j1r[kk], fmaf(a0, j0r[kk], h[i][kk])));
                        continue;
                    }
                    for (uint32_t kk = 0u; kk < n; ++kk) h[i][kk] += a0 * j0r[kk] + a1 * j1r[kk] + a2 * j2r[kk];
                }
            }
    }
    int finite = 1, settled = 1;
    /* ScaleTileRows (:194-207) reads the wide block's entry (i, k) from the upper triangle */
    if (wide_tile(n)) for (uint32_t i = 0u; i < n; ++i) for (uint32_t k = 0u; k < i; ++k) h[i][k] = h[k][i];
    for (uint32_t i = 0u; i < n; ++i) {
        h[i][i] += diagonal[i];
        force[i] = g[i].value + g[i].error;
        inertia[i] = inertial[i].value + inertial[i].error;
        finite = finite && isfinite(force[i]);
    }
    for (uint32_t i = 0u; i < n; ++i) {
        for (uint32_t k = 0u; k < n; ++k) {
            finite = finite && isfinite(h[i][k]);
            scale[i] += fabsf(h[i][k]) * fabsf(u[k]);
        }
        settled = settled && fabsf(force[i]) <= 8.0f * FLT_EPSILON * scale[i];
    }
    *converged = settled;
    return finite;
}

/* SolveTileMass (:1898-1931): d = M^-1 f by the same Cholesky */
static int solve_tile_mass(tile* c, const float* force, float* d) {
    float m[NKO_MAX_DOF][NKO_MAX_DOF + 1];
    for (uint32_t i = 0u; i < c->n; ++i) for (uint32_t j = 0u; j < c->n; ++j) m[i][j] = c->mass[i][j];
    return wide_tile(c->n) ? cholesky_solve_wide(m, c->n, force, d) : cholesky_solve(m, c->n, force, d);
}

enum { FAIL_NONE = 0, FAIL_EQUATION, FAIL_FACTOR, FAIL_DIRECTION, FAIL_CANDIDATE };

/* TileNewtonDirection (:1935-1992): the narrow form up to 32 coordinates, the wide form (its second assembly
 * reproduces the first bit for bit and is not repeated) past them */
static int newton_direction(tile* c, const float* u, const float* free_v, float* force, float* inertia, float* d, int* converged) {
    float h[NKO_MAX_DOF][NKO_MAX_DOF + 1];
    if (!assemble_block(c, u, free_v, h, force, inertia, converged)) return FAIL_EQUATION;
    if (*converged && c->tolerance > 0.0f) {
        if (!solve_tile_mass(c, force, d)) return FAIL_FACTOR;
        int stationary = 1;
        for (uint32_t i = 0u; i < c->n; ++i) stationary = stationary && fabsf(d[i]) < c->tolerance;
        *converged = stationary;
    }
    if (*converged) return FAIL_NONE;
    if (!(wide_tile(c->n) ? cholesky_solve_wide(h, c->n, force, d) : cholesky_solve(h, c->n, force, d))) return FAIL_FACTOR;
    return FAIL_NONE;
}

/* TileRowSteps (:2018-2044): step = J d, serial fma form */
static void row_steps(tile* c, const float* d) {
    for (uint32_t k = 0u; k < c->incident_count; ++k) {
        tile_head* t = &c->head[c->incident[k]];
        const uint32_t incidence = t->owner[0] == 0u ? 0u : 1u;
        v3 step = v3_make(0, 0, 0);
        if (t->unit[incidence] != NO_BLOCK) step.x = t->unit_value[incidence] * d[t->unit[incidence]];
        else {
            const float* j = c->jac + (size_t)t->row[incidence] * c->width;
            float value = 0.0f;
            for (uint32_t i = 0u; i < c->n; ++i) value = fmaf(j[i], d[i], value);
            step.x = value;
            if (t->axes == 3u) {
                value = 0.0f;
                for (uint32_t i = 0u; i < c->n; ++i) value = fmaf(j[c->width + i], d[i], value);
                step.y = value;
                value = 0.0f;
                for (uint32_t i = 0u; i < c->n; ++i) value = fmaf(j[2u * c->width + i], d[i], value);
                step.z = value;
            }
        }
        t->step = step;
    }
}

/* TileLineDerivatives (:2048-2086) */
static void line_derivatives(tile* c, float alpha, float inertial_slope, float inertial_curvature, float* slope, float* curvature, float* magnitude) {
    tile_sum row_slope = {0.0f, 0.0f};
    float row_curvature = 0.0f, row_magnitude = 0.0f;
    for (uint32_t k = 0u; k < c->incident_count; ++k) {
        const tile_head* t = &c->head[c->incident[k]];
        const v3 trial = v3_make(fmaf(alpha, t->step.x, t->move.x), fmaf(alpha, t->step.y, t->move.y), fmaf(alpha, t->step.z, t->move.z));
        v3 f; float r[6];
        tile_response(t, trial, &f, r);
        tile_add_product(&row_slope, f.x, t->step.x);
        tile_add_product(&row_slope, f.y, t->step.y);
        tile_add_product(&row_slope, f.z, t->step.z);
        row_magnitude += fabsf(f.x * t->step.x) + fabsf(f.y * t->step.y) + fabsf(f.z * t->step.z);
        if (c->w->line_rule != 0)   /* not the reference's: nko_world_set_line_rule */
            row_magnitude += r[0] * (fabsf(t->residual.x) + fabsf(trial.x)) * fabsf(t->step.x) + r[1] * (fabsf(t->residual.y) + fabsf(trial.y)) * fabsf(t->step.y) +
                             r[2] * (fabsf(t->residual.z) + fabsf(trial.z)) * fabsf(t->step.z);
        row_curvature += r[0] * t->step.x * t->step.x + r[1] * t->step.y * t->step.y + r[2] * t->step.z * t->step.z +
                         2.0f * r[5] * t->step.y * t->step.z + 2.0f * r[3] * t->step.x * t->step.y + 2.0f * r[4] * t->step.x * t->step.z;
    }
    tile_sum total = {-row_slope.value, -row_slope.error};
    tile_add_product(&total, alpha, inertial_curvature);
    tile_add(&total, inertial_slope);
    *slope = total.value + total.error;
    *curvature = inertial_curvature + row_curvature;
    *magnitude = fabsf(inertial_slope) + alpha * inertial_curvature + row_magnitude;
}

/* SearchTileLine (:2089-2125) */
static float search_line(tile* c, float inertial_slope, float inertial_curvature) {
    float slope = 0.0f, curvature = 0.0f, magnitude = 0.0f;
    line_derivatives(c, 0.0f, inertial_slope, inertial_curvature, &slope, &curvature, &magnitude);
    const float initial = slope;
    if (!(initial < 0.0f)) return 0.0f;
    float low = 0.0f, high = 0.0f, alpha = 1.0f;
    int bounded = 0;
    for (uint32_t step = 0u; step < 32u; ++step) {
        line_derivatives(c, alpha, inertial_slope, inertial_curvature, &slope, &curvature, &magnitude);
        if (!isfinite(slope) || !isfinite(curvature)) {
            high = alpha; bounded = 1; alpha = 0.5f * (low + high);
            continue;
        }
        if (fabsf(slope) <= fmaxf((float)1.0e-6 * -initial, 8.0f * FLT_EPSILON * magnitude)) return alpha;
        if (slope < 0.0f) low = alpha;
        else { high = alpha; bounded = 1; }
        if (bounded && high - low <= FLT_EPSILON * high) break;
        float next = alpha - slope / curvature;
        if (!(next > low && (!bounded || next < high))) next = bounded ? 0.5f * (low + high) : 2.0f * alpha;
        alpha = next;
    }
    return low;
}

static void apply_moves(tile* c, float alpha) {
    for (uint32_t k = 0u; k < c->incident_count; ++k) {
        tile_head* t = &c->head[c->incident[k]];
        t->move = v3_make(fmaf(alpha, t->step.x, t->move.x), fmaf(alpha, t->step.y, t->move.y), fmaf(alpha, t->step.z, t->move.z));
    }
}

/* DescendTileBlock (:2145-2301) for the articulated block; `free_v` is NULL in the position pass */
static void descend_block(tile* c, float* velocity, const float* free_in) {
    const uint32_t n = c->n;
    int coupled = 0;
    for (uint32_t k = 0u; k < c->incident_count; ++k) {   /* StartTileBlock :1386-1397 */
        tile_head* t = &c->head[c->incident[k]];
        coupled = coupled || (t->owner[0] != NO_BLOCK && t->owner[1] != NO_BLOCK);
        t->normal_bound = t->dual.x;
        t->move = v3_make(0, 0, 0);
    }
    float start[NKO_MAX_DOF], free_v[NKO_MAX_DOF], u[NKO_MAX_DOF];
    for (uint32_t i = 0u; i < n; ++i) {
        start[i] = velocity[i];
        free_v[i] = free_in != NULL ? free_in[i] : 0.0f;
        u[i] = start[i];
    }
    if (c->iteration == 0u && free_in != NULL) {   /* :2165-2209 first-sweep segment search */
        float d[NKO_MAX_DOF], mass_step[NKO_MAX_DOF];
        for (uint32_t i = 0u; i < n; ++i) { d[i] = free_v[i] - u[i]; mass_step[i] = 0.0f; }
        for (uint32_t k = 0u; k < n; ++k) for (uint32_t i = 0u; i < n; ++i) mass_step[i] += c->mass[i][k] * d[k];
        tile_sum curvature = {0.0f, 0.0f};
        for (uint32_t i = 0u; i < n; ++i) tile_add_product(&curvature, d[i], mass_step[i]);
        const float inertial_curvature = curvature.value + curvature.error;
        if (inertial_curvature > 0.0f && isfinite(inertial_curvature)) {
            row_steps(c, d);
            const float alpha = search_line(c, -inertial_curvature, inertial_curvature);
            if (alpha > 0.0f) {
                for (uint32_t i = 0u; i < n; ++i) u[i] = fmaf(alpha, d[i], u[i]);
                apply_moves(c, alpha);
            }
        }
    }
    int failure = FAIL_NONE;
    float primal = FLT_MAX;
    for (uint32_t step = 0u; step < 16u; ++step) {
        float force[NKO_MAX_DOF], inertia[NKO_MAX_DOF], d[NKO_MAX_DOF], mass_step[NKO_MAX_DOF];
        int converged = 0;
        failure = newton_direction(c, u, free_v, force, inertia, d, &converged);
        if (converged) primal = 0.0f;
        if (failure != FAIL_NONE || converged) break;
        for (uint32_t i = 0u; i < n; ++i) mass_step[i] = 0.0f;
        for (uint32_t k = 0u; k < n; ++k) for (uint32_t i = 0u; i < n; ++i) mass_step[i] += c->mass[i][k] * d[k];
        tile_sum decrement = {0, 0}, slope = {0, 0}, curvature = {0, 0};
        for (uint32_t i = 0u; i < n; ++i) {
            tile_add_product(&decrement, force[i], d[i]);
            tile_add_product(&slope, inertia[i], d[i]);
            tile_add_product(&curvature, d[i], mass_step[i]);
        }
        const float total_decrement = decrement.value + decrement.error;
        const float inertial_slope = slope.value + slope.error;
        const float inertial_curvature = curvature.value + curvature.error;
        if (!isfinite(total_decrement) || !isfinite(inertial_slope) || !isfinite(inertial_curvature)) { failure = FAIL_DIRECTION; break; }
        if (!(total_decrement > 0.0f)) break;
        row_steps(c, d);
        const float alpha = search_line(c, inertial_slope, inertial_curvature);
        float after[NKO_MAX_DOF];
        int finite = 1, rounded = 1;
        for (uint32_t i = 0u; i < n; ++i) {
            after[i] = fmaf(alpha, d[i], u[i]);
            finite = finite && isfinite(after[i]);
            rounded = rounded && after[i] == u[i];
        }
        if (!finite) { failure = FAIL_CANDIDATE; break; }
        primal = 0.0f;
        for (uint32_t i = 0u; i < n; ++i) if (!rounded) primal = fmaxf(primal, fabsf(alpha * d[i]));
        if (!(alpha > 0.0f)) break;
        for (uint32_t i = 0u; i < n; ++i) u[i] = after[i];
        apply_moves(c, alpha);
        if (rounded) break;
    }
    for (uint32_t k = 0u; k < c->incident_count; ++k) {   /* EndTileBlock :1400-1409 */
        tile_head* t = &c->head[c->incident[k]];
        t->residual = v3_make(t->residual.x - t->move.x, t->residual.y - t->move.y, t->residual.z - t->move.z);
    }
    if (failure != FAIL_NONE) { c->failed = 1; c->w->env_status[c->env] |= NKO_STATUS_SOLVER_FAILURE; }
    if (failure != FAIL_NONE && getenv("NKO_TRACE_FAILURES") != NULL)
        fprintf(stderr, "nko: env %u sweep %u block descent failure kind %d\n", c->env, c->iteration, failure);
    float moved = failure == FAIL_NONE ? 0.0f : FLT_MAX;
    for (uint32_t i = 0u; i < n; ++i) moved = fmaxf(moved, u2f(residual_bits(u[i] - start[i])));
    c->momentum = fmaxf(c->momentum, moved);
    if (failure != FAIL_NONE) primal = FLT_MAX;
    c->residual = fmaxf(c->residual, fmaxf(primal, coupled ? moved : 0.0f));
    for (uint32_t i = 0u; i < n; ++i) velocity[i] = u[i];
}

/* MeasureTilePrimal (:2378-2489) */
static void measure_primal(tile* c, float* velocity, const float* free_v, const float* lambda_env, int reconstruct) {
    const uint32_t n = c->n;
    double balance[NKO_MAX_DOF];
    float force[NKO_MAX_DOF] = {0.0f}, direction[NKO_MAX_DOF] = {0.0f};
    for (uint32_t i = 0u; i < n; ++i) {
        balance[i] = 0.0;
        for (uint32_t j = 0u; j < n; ++j) balance[i] -= (double)c->mass[i][j] * ((double)velocity[j] - free_v[j]);
    }
    const uint32_t R = c->w->t.rows_per_env;
    for (uint32_t k = 0u; k < c->incident_count; ++k) {
        const tile_head* t = &c->head[c->incident[k]];
        const uint32_t local = t->slot - c->env * R;
        const v3 impulse = v3_make(lambda_env[local], t->axes == 3u ? lambda_env[local + t->stride] : 0.0f,
                                   t->axes == 3u ? lambda_env[local + 2u * t->stride] : 0.0f);
        if (!(impulse.x != 0.0f || impulse.y != 0.0f || impulse.z != 0.0f)) continue;
        const uint32_t incidence = t->owner[0] == 0u ? 0u : 1u;
        const float applied[3] = {impulse.x, impulse.y, impulse.z};
        for (uint32_t axis = 0u; axis < t->axes; ++axis)
            for (uint32_t i = 0u; i < n; ++i) {
                const float jacobian = t->unit[incidence] != NO_BLOCK ? (i == t->unit[incidence] ? t->unit_value[incidence] : 0.0f)
                    : c->jac[(size_t)(t->row[incidence] + axis) * c->width + i];
                balance[i] += (double)jacobian * applied[axis];
            }
    }
    int finite = 1;
    for (uint32_t i = 0u; i < n; ++i) { force[i] = (float)balance[i]; finite = finite && fabs(balance[i]) <= FLT_MAX; }
    int failure = finite ? FAIL_NONE : FAIL_EQUATION;
    if (failure == FAIL_NONE && !solve_tile_mass(c, force, direction)) failure = FAIL_FACTOR;
    float residual = failure == FAIL_NONE ? 0.0f : FLT_MAX;
    if (failure != FAIL_NONE) c->w->env_status[c->env] |= NKO_STATUS_SOLVER_FAILURE;
    if (failure != FAIL_NONE && getenv("NKO_TRACE_FAILURES") != NULL)
        fprintf(stderr, "nko: env %u sweep %u primal measure failure kind %d\n", c->env, c->iteration, failure);
    for (uint32_t i = 0u; i < n && failure == FAIL_NONE; ++i)
        residual = fmaxf(residual, isfinite(direction[i]) ? fabsf(direction[i]) : FLT_MAX);
    c->residual = fmaxf(c->residual, residual);
    if (reconstruct && failure == FAIL_NONE) {
        int ok = 1;
        for (uint32_t i = 0u; i < n; ++i) ok = ok && isfinite(velocity[i] + direction[i]);
        if (!ok) { c->residual = FLT_MAX; return; }
        for (uint32_t i = 0u; i < n; ++i) velocity[i] += direction[i];
        c->momentum = fmaxf(c->momentum, residual);
    }
}

/* InitializeTileResiduals (:890-930), serial product-sum form of SerialSideSpeed */
static void initialize_residuals(tile* c, const float* velocity) {
    const nko_world* w = c->w;
    const uint32_t R = w->t.rows_per_env, md = w->t.max_dof;
    const nko_row* rows = (const nko_row*)w->urows;
    for (uint32_t h = 0u; h < c->heads; ++h) {
        tile_head* t = &c->head[h];
        float res[3] = {0.0f, 0.0f, 0.0f};
        for (uint32_t axis = 0u; axis < t->axes; ++axis) {
            const uint32_t at = t->slot + axis * t->stride;
            const nko_row* row = &rows[at];
            float along_a = 0.0f, along_b = 0.0f;
            if (row->a.kind == NKO_SIDE_ARTIC)
                for (uint32_t i = 0u; i < c->n; ++i) along_a = along_a + w->chain_jacobian[(size_t)at * md + i] * velocity[i];
            if (row->b.kind == NKO_SIDE_ARTIC)
                for (uint32_t i = 0u; i < c->n; ++i) along_b = along_b + w->chain_jacobian_b[(size_t)at * md + i] * velocity[i];
            res[axis] = row->rhs * w->cfg.fixed_dt - (along_a + along_b);
        }
        (void)R;
        t->residual = v3_make(res[0], res[1], res[2]);
    }
}

/* UpdateTileHeadDuals (:2493-2595); returns residual classes {normal, tangent, joint} */
static void update_duals(tile* c, float* lambda_env, dual_momentum* momentum, int velocity, int commit, float* classes) {
    uint32_t steps[4] = {0u, 0u, 0u, 0u};
    double restart = 0.0;
    const uint32_t R = c->w->t.rows_per_env;
    const nko_row* rows = (const nko_row*)c->w->urows;
    for (uint32_t h = 0u; h < c->heads; ++h) {
        tile_head* th = &c->head[h];
        tile_head t = *th;
        if (!commit) t.dual = t.base;
        const uint32_t local = t.slot - c->env * R;
        const int contact = t.axes == 3u;
        float normal, ncurv;
        scalar_impulse(t.dual.x, t.rho, t.residual.x, t.compliance, t.lower, t.upper, t.response, &normal, &ncurv);
        relaxation relax = t.relax;
        if (!commit) memset(&relax, 0, sizeof(relax));
        v3 dual;
        const float t_dual[3] = {t.dual.x, t.dual.y, t.dual.z}, t_residual[3] = {t.residual.x, t.residual.y, t.residual.z};
        const float t_compliance[3] = {t.cone_compliance.x, t.cone_compliance.y, t.cone_compliance.z};
        if (t.elliptic) {   /* :2509-2510 */
            float out[9];
            nko_elliptic_impulse(t_dual, t.rho, t_residual, t_compliance, t.mu_first, out);
            dual = v3_make(out[0], out[1], out[2]);
        } else if (!contact) dual = v3_make(normal, 0.0f, 0.0f);   /* ProjectRowDual block_descent.cu:799-804 */
        else {
            v3 f; float cv[6];
            tangent_impulse(t.dual, t.rho, t.residual, normal, t.mu_first, t.mu_second, &f, cv);
            dual = relax_contact_impulse(t.dual, v3_make(normal, f.y, f.z), &relax);
        }
        float step[2];
        multiplier_steps(t.dual, dual, t.response.residual_scale, t.response.dual_scale, t.rho, contact ? t.mu_first : 0.0f,
                         contact ? t.mu_second : 0.0f, step);
        if (!commit && t.response.residual_scale > 0.0f) step[0] = fabsf(dual.x - t.dual.x) / t.response.residual_scale;
        if (t.elliptic) {   /* :2516-2519 */
            const float next[3] = {dual.x, dual.y, dual.z};
            float delta[3];
            nko_elliptic_multiplier_step(t_dual, next, t.rho, t_compliance, delta);
            step[0] = delta[0]; step[1] = fmaxf(delta[1], delta[2]);
        }
        const v3 physical = commit ? dual : t.dual;
        if (!contact) {
            const int normal_row = (rows[t.slot].flags & NKO_ROW_CONTACT_NORMAL) != 0u;
            const uint32_t kind = normal_row ? 0u : 2u;
            const float rate = -t.residual.x + t.compliance * physical.x;
            const float violation = physical.x > 0.0f ? fabsf(rate) : fmaxf(-rate, 0.0f);
            const float residual = normal_row ? fmaxf(step[0], violation) : step[0];
            if (residual_bits(residual) > steps[kind]) steps[kind] = residual_bits(residual);
        } else {
            if (commit) {
                th->relax = relax;
                lambda_env[local + t.stride] = dual.y;
                lambda_env[local + 2u * t.stride] = dual.z;
            }
            if (t.elliptic) {   /* :2540-2542 */
                if (residual_bits(step[0]) > steps[0]) steps[0] = residual_bits(step[0]);
                if (residual_bits(step[1]) > steps[1]) steps[1] = residual_bits(step[1]);
            } else {
                const v3 v = v3_make(-t.residual.x + t.compliance * physical.x, -t.residual.y, -t.residual.z);
                const uint32_t nb = residual_bits(physical.x > 0.0f ? fabsf(v.x) : fmaxf(-v.x, 0.0f));
                if (nb > steps[0]) steps[0] = nb;
                const uint32_t tb = residual_bits(fmaxf(step[1], fmaxf(along_axis(physical.y, v.y), along_axis(physical.z, v.z))));
                if (tb > steps[1]) steps[1] = tb;
            }
        }
        if (!commit) continue;
        if (velocity) lambda_env[local] = dual.x;
        const int extrapolate = contact || t.response.dual_scale != 0.0f;
        const v3 base = t.base;
        v3 metric = multiplier_metric(t.response.residual_scale, t.rho, contact, t.mu_first, t.mu_second);
        if (t.elliptic) { v3 unused; elliptic_response(t.rho, t.cone_compliance, &metric, &unused); }   /* :2555-2557 */
        if (extrapolate) restart += momentum_restart(t.dual, dual, base, metric);
        if (momentum != NULL) th->move = base;
        th->dual = dual;
        th->base = dual;
    }
    if (momentum != NULL) {
        advance_dual_momentum(momentum, restart);
        for (uint32_t h = 0u; h < c->heads; ++h) {
            tile_head* t = &c->head[h];
            const int contact = t->axes == 3u;
            const int extrapolate = contact || t->response.dual_scale != 0.0f;
            t->dual = extrapolate_dual(t->move, t->base, extrapolate ? momentum->beta : 0.0f, t->lower, t->upper, contact,
                                       t->mu_first, t->mu_second);
        }
    }
    classes[0] = u2f(steps[0]); classes[1] = u2f(steps[1]); classes[2] = u2f(steps[2]);
}

static uint32_t row_bound(const uint32_t* extent, uint32_t env, uint32_t contact_rows) {   /* union_types.cuh:187-193 */
    const uint32_t previous = extent[2u * env], current = extent[2u * env + 1u];
    if (previous == 0u || current == 0u) return contact_rows;
    const uint32_t m = (previous > current ? previous : current) - 1u;
    return m < contact_rows ? m : contact_rows;
}

static void index_incidence(tile* c) {   /* IndexTileIncidence, one block (:1019-1035) */
    c->incident_count = 0u;
    for (uint32_t h = 0u; h < c->heads; ++h)
        if (c->head[h].owner[0] != NO_BLOCK || c->head[h].owner[1] != NO_BLOCK) c->incident[c->incident_count++] = h;
}

/* DescendTile (:2941-3087) */
void nko_env_solve(nko_world* w, uint32_t env) {
    const nko_template* tp = &w->t;
    const uint32_t R = tp->rows_per_env, md = tp->max_dof, n = tp->nv, nl = tp->nl;
    if (R == 0u || n == 0u) return;
    const float dt = w->cfg.fixed_dt;
    const nko_row* rows = (const nko_row*)w->urows;
    float* lambda_env = w->lambda + (size_t)env * R;
    float* velocity = w->solver_velocity + (size_t)env * md;
    float* free_v = w->solver_free + (size_t)env * md;
    const size_t lbase = (size_t)env * nl;
    tile* c = (tile*)calloc(1, sizeof(tile));
    c->w = w; c->env = env; c->n = n; c->width = (n + 3u) & ~3u; c->tolerance = w->cfg.solver_velocity_tolerance;
    /* InitializeTile (:1327-1350): free velocity and the carried constraint velocity */
    for (uint32_t d = 0u; d < n; ++d) {
        const uint32_t link = tp->dof_link[d], comp = tp->dof_component[d];
        const float value = comp == NKO_INVALID ? w->qdot[lbase + link] : w->link_velocity[(lbase + link) * 6u + comp];
        const float carried = velocity[d] - free_v[d];
        free_v[d] = value;
        velocity[d] = value + (isfinite(carried) ? carried : 0.0f);
    }
    /* ListTileHeads (:1250-1296) */
    const uint32_t bound = row_bound(w->contact_row_extent, env, tp->contact_rows_per_env);
    const uint32_t total = bound + (R - tp->contact_rows_per_env);
    c->head = (tile_head*)calloc(total ? total : 1u, sizeof(tile_head));
    c->incident = (uint32_t*)calloc(total ? total : 1u, sizeof(uint32_t));
    for (uint32_t index = 0u; index < total; ++index) {
        const uint32_t slot = env * R + (index < bound ? index : tp->contact_rows_per_env + (index - bound));
        const uint32_t flags = rows[slot].flags;
        if ((flags & NKO_ROW_ACTIVE) != 0u && (flags & NKO_ROW_BLOCK_TANGENT) == 0u) c->head[c->heads++].slot = slot;
    }
    /* InitializeTileHead (:743-797) */
    uint32_t staged_rows = 0u;
    for (uint32_t h = 0u; h < c->heads; ++h) {
        tile_head* t = &c->head[h];
        const uint32_t slot = t->slot;
        const nko_row* row = &rows[slot];
        t->stride = row->group_normal_count;
        t->axes = (row->flags & NKO_ROW_BLOCK_NORMAL) != 0u ? 3u : 1u;
        const uint32_t owner = row->a.kind == NKO_SIDE_ARTIC ? 0u : NO_BLOCK;
        const uint32_t other = row->b.kind == NKO_SIDE_ARTIC ? 0u : NO_BLOCK;
        /* TileInertialResponse (:709-739) */
        const int shared = row->a.kind == row->b.kind && row->a.index == row->b.index;
        float response = 0.0f, shares[2] = {0.0f, 0.0f};
        int valid = 1;
        const nko_row_side* sides[2] = {&row->a, &row->b};
        for (uint32_t i = 0u; i < (shared ? 1u : 2u); ++i) {
            float contribution = 0.0f;
            if (sides[i]->kind == NKO_SIDE_ARTIC) {
                const float* jacobian = (i == 0u ? w->chain_jacobian : w->chain_jacobian_b) + (size_t)slot * md;
                contribution = nko_mass_coupling(w->m_factor + (size_t)env * md * md, md, jacobian,
                                                 shared ? w->chain_jacobian_b + (size_t)slot * md : NULL);
            }
            valid = valid && contribution >= 0.0f && isfinite(contribution);
            response += contribution;
            shares[i] = contribution;
        }
        const float coupling = shares[0] * shares[1], largest = fmaxf(shares[0], shares[1]);
        if (!(valid && isfinite(response))) response = NAN;
        const float coupled = coupling > 0.0f ? (response + sqrtf(response * response + 12.0f * coupling)) / (6.0f * coupling) : FLT_MAX;
        const float cap = (float)1.0e2 / largest;
        float rho = response > 0.0f ? fminf(cap, coupled) : 0.0f;
        if (!(response == 0.0f || (response > 0.0f && rho > 0.0f && rho <= FLT_MAX))) {
            w->env_status[env] |= NKO_STATUS_SOLVER_FAILURE;
            if (getenv("NKO_TRACE_FAILURES") != NULL)
                fprintf(stderr, "nko: env %u head %u inertial response %g (shares %g %g) rejected\n", env, h, response, shares[0], shares[1]);
            rho = NAN;
        }
        w->solver_penalty[slot] = rho;
        t->owner[0] = owner; t->owner[1] = other == owner ? NO_BLOCK : other;
        t->rho = rho; t->compliance = row->compliance_alpha;
        t->response = float_scalar_response(rho, t->compliance);
        t->lower = row->lower; t->upper = row->upper; t->mu_first = row->mu; t->mu_second = row->friction_secondary;
        t->normal_bound = 0.0f;
        t->elliptic = t->axes == 3u && (row->flags & NKO_ROW_MUJOCO) != 0u;   /* :778-780 */
        t->cone_compliance = v3_make(t->compliance, t->axes == 3u ? rows[slot + t->stride].compliance_alpha : 0.0f,
                                     t->axes == 3u ? rows[slot + 2u * t->stride].compliance_alpha : 0.0f);
        const uint32_t local = slot - env * R;
        t->dual = v3_make(lambda_env[local], t->axes == 3u ? lambda_env[local + t->stride] : 0.0f, t->axes == 3u ? lambda_env[local + 2u * t->stride] : 0.0f);
        t->base = t->dual;
        staged_rows += 2u * t->axes;
    }
    /* FindTileRowSupport (:801-833) + PlaceTileRows + CopyTileRows (:836-869) */
    c->jac = (float*)calloc((size_t)(staged_rows ? staged_rows : 1u) * c->width, sizeof(float));
    uint32_t next_row = 0u;
    for (uint32_t h = 0u; h < c->heads; ++h) {
        tile_head* t = &c->head[h];
        for (uint32_t incidence = 0u; incidence < 2u; ++incidence) {
            t->unit[incidence] = NO_BLOCK; t->row[incidence] = NO_BLOCK; t->unit_value[incidence] = 0.0f;
            if (t->owner[incidence] == NO_BLOCK) continue;
            const nko_row* head = &rows[t->slot];
            uint32_t supported = 0u, unit = 0u;
            float unit_value = 0.0f;
            for (uint32_t i = 0u; i < n; ++i) {   /* TileBlock::Jacobian :555-573 */
                float value = 0.0f;
                if (head->a.kind == NKO_SIDE_ARTIC) value += w->chain_jacobian[(size_t)t->slot * md + i];
                if (head->b.kind == NKO_SIDE_ARTIC) value += w->chain_jacobian_b[(size_t)t->slot * md + i];
                if (value != 0.0f) { ++supported; unit = i; unit_value = value; }
            }
            const int single = t->axes == 1u && supported <= 1u;
            if (single) { t->unit[incidence] = unit; t->unit_value[incidence] = unit_value; continue; }
            t->row[incidence] = next_row;
            for (uint32_t axis = 0u; axis < t->axes; ++axis) {
                const uint32_t row_slot = t->slot + axis * t->stride;
                const nko_row* ar = &rows[row_slot];
                float* out = c->jac + (size_t)(next_row + axis) * c->width;
                for (uint32_t i = 0u; i < n; ++i) {
                    float value = 0.0f;
                    if (ar->a.kind == NKO_SIDE_ARTIC) value += w->chain_jacobian[(size_t)row_slot * md + i];
                    if (ar->b.kind == NKO_SIDE_ARTIC) value += w->chain_jacobian_b[(size_t)row_slot * md + i];
                    out[i] = value;
                }
            }
            next_row += t->axes;
        }
    }
    index_incidence(c);
    initialize_residuals(c, velocity);
    /* StageTileMass (:2127-2142) */
    for (uint32_t i = 0u; i < n; ++i) for (uint32_t j = 0u; j < n; ++j) c->mass[i][j] = w->m[(size_t)env * md * md + (size_t)i * md + j];
    float residual4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t sweeps = 0u;
    dual_momentum momentum = {1.0f, 0.0f, 0u};
    const float tol = c->tolerance;
    while (sweeps < w->cfg.solver_vel_iters) {
        c->iteration = sweeps++;
        c->momentum = 0.0f; c->residual = 0.0f;
        descend_block(c, velocity, free_v);
        float rowsr[3];
        update_duals(c, lambda_env, &momentum, 1, 1, rowsr);
        if (sweeps == w->cfg.solver_vel_iters || fmaxf(fmaxf(rowsr[0], rowsr[1]), fmaxf(rowsr[2], c->residual)) < tol)
            measure_primal(c, velocity, free_v, lambda_env, 0);
        if (fmaxf(fmaxf(rowsr[0], rowsr[1]), rowsr[2]) < tol && c->residual >= tol && c->residual < FLT_MAX) {
            measure_primal(c, velocity, free_v, lambda_env, 1);
            if (c->residual < FLT_MAX) {
                initialize_residuals(c, velocity);
                update_duals(c, lambda_env, NULL, 1, 0, rowsr);
                c->residual = 0.0f;
                measure_primal(c, velocity, free_v, lambda_env, 0);
            }
        }
        residual4[0] = rowsr[0]; residual4[1] = rowsr[1]; residual4[2] = rowsr[2]; residual4[3] = c->residual;
        const float largest = fmaxf(fmaxf(rowsr[0], rowsr[1]), fmaxf(rowsr[2], c->residual));
        if (largest < tol || largest == FLT_MAX) break;
    }
    for (uint32_t k = 0u; k < 4u; ++k) w->solver_residual[(size_t)env * 4u + k] = residual4[k];
    w->vbd_velocity_sweep_count[env] = sweeps;
    /* FinishTile (:2607-2650) */
    {
        int invalid = 0;
        for (uint32_t d = 0u; d < n; ++d) invalid = invalid || !(fabsf(velocity[d]) <= FLT_MAX);
        if (!invalid)
            for (uint32_t d = 0u; d < md; ++d) {
                const float value = d < n ? velocity[d] : 0.0f;
                w->qdot_flat[(size_t)env * md + d] = value;
                if (d >= n) continue;
                const uint32_t link = tp->dof_link[d], comp = tp->dof_component[d];
                if (comp == NKO_INVALID) w->qdot[lbase + link] = value;
                else w->link_velocity[(lbase + link) * 6u + comp] = value;
            }
        else w->env_status[env] |= NKO_STATUS_SOLVER_FAILURE;
    }
    /* joint limit impulses (FinishTile :2658-2668) */
    if (tp->joint_limit_rows >= 2u * nl)
        for (uint32_t l = 0u; l < nl; ++l) {
            const size_t lower = (size_t)env * R + tp->contact_rows_per_env + (size_t)l * 2u;
            w->joint_limit_impulse[2u * (lbase + l)] = (rows[lower].flags & NKO_ROW_ACTIVE) != 0u ? w->lambda[lower] : 0.0f;
            w->joint_limit_impulse[2u * (lbase + l) + 1u] = (rows[lower + 1u].flags & NKO_ROW_ACTIVE) != 0u ? w->lambda[lower + 1u] : 0.0f;
        }
    /* split-impulse position pass (:3059-3077, MarkTilePositions :2673-2708) */
    if (w->cfg.solver_pos_iters != 0u) {
        float pseudo[NKO_MAX_DOF];
        int push = 0, coupled = 0;
        const uint32_t S = tp->slots;
        for (uint32_t h = 0u; h < c->heads; ++h) {
            tile_head* t = &c->head[h];
            const uint32_t slot = t->slot, local = slot - env * R;
            const nko_row* row = &rows[slot];
            const float penetration = w->row_penetration[slot];
            const int speculative = (row->flags & NKO_ROW_SPECULATIVE) != 0u;
            const float slop = speculative ? 0.0f : w->cfg.solver_pos_slop;
            const int position = (row->flags & (NKO_ROW_FRICTION | NKO_ROW_VELOCITY_ONLY | NKO_ROW_MUJOCO)) == 0u &&
                (speculative || penetration > slop || t->dual.x != 0.0f);
            float bias = 0.0f, rounding = 0.0f;
            if (position) {   /* PositionRowBias block_descent.cu:1734-1753 */
                const float pen = fmaxf(penetration - slop, 0.0f);
                if (speculative) {
                    /* MapRowContactsKernel :1756-1767: the contact slot whose normal rows hold this row */
                    uint32_t contact = 0u, first = 0u, points = 1u;
                    for (uint32_t s = 0u; s < S; ++s) {
                        const uint32_t f = w->ucontact_row_range[((size_t)env * S + s) * 2u], p = w->ucontact_row_range[((size_t)env * S + s) * 2u + 1u];
                        if (p > 0u && slot >= f && slot < f + p) { contact = env * S + s; first = f; points = p; }
                    }
                    const size_t point = (size_t)contact * 4u + (slot - first) % points;
                    const double depth = (double)w->ucontact_depth[point] - slop;
                    const double reserve = (double)w->row_penetration[slot] - w->ucontact_depth[point];
                    const double correction = w->cfg.solver_pos_beta * fmax(depth, 0.0) + reserve;
                    const double target = fmin(depth, 0.0) + correction;
                    double vel = 0.0;   /* RowVelocity :1051-1082 against qdot_flat */
                    if (row->a.kind == NKO_SIDE_ARTIC) {
                        double value = 0.0;
                        for (uint32_t d = 0u; d < md; ++d) value += (double)w->chain_jacobian[(size_t)slot * md + d] * w->qdot_flat[(size_t)env * md + d];
                        vel += value;
                    }
                    if (row->b.kind == NKO_SIDE_ARTIC) {
                        double value = 0.0;
                        for (uint32_t d = 0u; d < md; ++d) value += (double)w->chain_jacobian_b[(size_t)slot * md + d] * w->qdot_flat[(size_t)env * md + d];
                        vel += value;
                    }
                    const double limit = fmin(correction / dt, (double)w->cfg.solver_baumgarte_max_velocity);
                    const double absorbed = target > 0.0 ? 0.0 : fmax(reserve, 0.0) / dt;
                    bias = (float)fmin(target / dt - vel, limit);
                    rounding = (float)absorbed;
                } else {
                    const float correction = w->cfg.solver_pos_beta * pen + fmaxf(pen - pen, 0.0f);
                    bias = fminf(correction / dt, w->cfg.solver_baumgarte_max_velocity);
                }
            }
            (void)local;
            if (!position) t->owner[0] = t->owner[1] = NO_BLOCK;
            coupled = coupled || (t->owner[0] != NO_BLOCK && t->owner[1] != NO_BLOCK);
            t->axes = 1u;
            t->elliptic = 0;   /* :2691 */
            t->compliance = 0.0f; t->lower = 0.0f; t->upper = FLT_MAX;
            t->response = float_scalar_response(t->rho, 0.0f);
            t->residual = v3_make(bias, 0.0f, 0.0f);
            t->dual = v3_make(0, 0, 0);
            push = push || bias > rounding;
        }
        for (uint32_t d = 0u; d < n; ++d) pseudo[d] = 0.0f;
        if (push) {
            index_incidence(c);
            const uint32_t positions = coupled ? w->cfg.solver_pos_iters : 1u;
            for (uint32_t iteration = 0u; iteration < positions; ++iteration) {
                c->iteration = sweeps + iteration;
                descend_block(c, pseudo, NULL);
                if (iteration + 1u < positions) {
                    float unused[3];
                    update_duals(c, lambda_env, NULL, 0, 1, unused);
                }
            }
        }
        /* FinishTilePositions (:2720-2744) */
        for (uint32_t d = 0u; d < n; ++d) {
            const uint32_t link = tp->dof_link[d], comp = tp->dof_component[d];
            if (comp == NKO_INVALID) w->qdot_pseudo[lbase + link] = pseudo[d];
            else w->link_velocity_pseudo[(lbase + link) * 6u + comp] = pseudo[d];
        }
    }
    free(c->head); free(c->incident); free(c->jac); free(c);
}
