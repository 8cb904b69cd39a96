/*
 * CPU oracle (test infrastructure; see nuka_oracle.h): the free rigid body of a world whose template says free_body.
 *
 * The reference steps such a body with its own ops - BodyIntegrateVelocityKernel before the contact solve, a six by six
 * block of the tile in it (block_descent_rigid.cuh, block_descent_tile.cuh:541-603), BodyIntegratePositionKernel with the
 * free-rotation solve after it.  The body's coordinates are its linear velocity and its angular velocity about the
 * centre of mass, both in world axes.  Here the body is the one link of the template: `base_pose` is the body's pose,
 * `body_linear_velocity` / `body_angular_velocity` (per body row, as in the reference: the link's own row holds them)
 * its state, and the six coordinates pass through the link's twist words (`link_velocity`: linear first, then angular)
 * to the row assembly and the block descent, which take the block's mass matrix and factor from `m` / `m_factor` as
 * they do for an articulation.
 */
#include "nko_internal.h"

/* math/symmetric_mat3.hpp:31-47 FromRotatedDiagonal: R diag(d) R^T of the rotation of q, as xx yy zz xy xz yz */
static void from_rotated_diagonal(v3 d, quat q, float out[6]) {
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    const float s = norm_sq > 1.0e-12f ? 2.0f / norm_sq : 0.0f;
    const v3 x = v3_make(1.0f - s * (q.y * q.y + q.z * q.z), s * (q.x * q.y - q.w * q.z), s * (q.x * q.z + q.w * q.y));
    const v3 y = v3_make(s * (q.x * q.y + q.w * q.z), 1.0f - s * (q.x * q.x + q.z * q.z), s * (q.y * q.z - q.w * q.x));
    const v3 z = v3_make(s * (q.x * q.z - q.w * q.y), s * (q.y * q.z + q.w * q.x), 1.0f - s * (q.x * q.x + q.y * q.y));
    out[0] = d.x * x.x * x.x + d.y * x.y * x.y + d.z * x.z * x.z;
    out[1] = d.x * y.x * y.x + d.y * y.y * y.y + d.z * y.z * y.z;
    out[2] = d.x * z.x * z.x + d.y * z.y * z.y + d.z * z.z * z.z;
    out[3] = d.x * x.x * y.x + d.y * x.y * y.y + d.z * x.z * y.z;
    out[4] = d.x * x.x * z.x + d.y * x.y * z.y + d.z * x.z * z.z;
    out[5] = d.x * y.x * z.x + d.y * y.y * z.y + d.z * y.z * z.z;
}

/* math/symmetric_mat3.hpp:25-29 Multiply */
static v3 sym_multiply(const float* m, v3 v) {
    return v3_make(m[0] * v.x + m[3] * v.y + m[4] * v.z, m[3] * v.x + m[1] * v.y + m[5] * v.z, m[4] * v.x + m[5] * v.y + m[2] * v.z);
}

/* nk/solve/vertex_block.hpp:139-153 Invert (floor 0): cofactors in double, rounded once */
static int sym_invert(const float* m, float out[6]) {
    const double xx = m[0], yy = m[1], zz = m[2], xy = m[3], xz = m[4], yz = m[5];
    const double cxx = yy * zz - yz * yz, cyy = xx * zz - xz * xz;
    const double czz = xx * yy - xy * xy, cxy = xz * yz - xy * zz;
    const double cxz = xy * yz - xz * yy, cyz = xy * xz - xx * yz;
    const double det = xx * cxx + xy * cxy + xz * cxz;
    if (!(det > 0.0 && det <= DBL_MAX)) return 0;
    const double inv = 1.0 / det;
    const double values[6] = {cxx * inv, cyy * inv, czz * inv, cxy * inv, cxz * inv, cyz * inv};
    for (uint32_t i = 0u; i < 6u; ++i) {
        if (!(values[i] >= -FLT_MAX && values[i] <= FLT_MAX)) return 0;
        out[i] = (float)values[i];
    }
    return 1;
}

/* rigid_types.cuh:10-14 BodyCenterOfMass, :16-21 BodyWorldInverseInertia */
static v3 body_center_of_mass(xform pose, xform frame) { return v3_add(pose.p, nko_rotate_normalized(pose.r, frame.p)); }
static void body_world_inverse_inertia(xform pose, xform frame, v3 inv_i, float out[6]) {
    from_rotated_diagonal(inv_i, nko_quat_mul(pose.r, frame.r), out);
}
void nko_body_center_of_mass(const nko_world* w, uint32_t env, float out[3]) {
    const v3 c = body_center_of_mass(xform_load(w->base_pose + (size_t)env * 7u), xform_load(w->t.link_inertial_frame));
    out[0] = c.x; out[1] = c.y; out[2] = c.z;
}

/* The free-rotation step (rigid_types.cuh:38-121 SolveFreeRotation): Euler's equations in the principal frame by the
 * implicit midpoint rule, m1 - m0 = dt (m_mid x w_mid), solved for the end-of-step angular momentum.  The unknown is the
 * momentum scaled to unit size, g(u) = u - u0 + c o (mid_y mid_z, mid_z mid_x, mid_x mid_y) with mid = (u0 + u) / 2 and
 * c = dt (a_y - a_z, a_z - a_x, a_x - a_y), a = scaled inverse moments; Newton steps on g, each halved while the residual
 * does not fall, at most twelve, to a residual of 1e-6.  `midpoint` is the angular velocity at the middle of the step. */
typedef struct { v3 midpoint; float residual; uint32_t iterations, status; } gyro_result;
enum { GYRO_CONVERGED = 0, GYRO_NOT_CONVERGED = 1, GYRO_INVALID_INPUT = 2 };   /* op_schema.hpp:53-54 */
typedef struct { float start[3], coupling[3]; } midpoint_rule;

static void rule_residual(const midpoint_rule* r, const float u[3], float g[3]) {
    const float mid[3] = {(r->start[0] + u[0]) * 0.5f, (r->start[1] + u[1]) * 0.5f, (r->start[2] + u[2]) * 0.5f};
    for (int k = 0; k < 3; ++k) g[k] = u[k] - r->start[k] + r->coupling[k] * mid[(k + 1) % 3] * mid[(k + 2) % 3];
}
/* dg/du: the identity and half the coupling times the other two midpoint components */
static void rule_jacobian(const midpoint_rule* r, const float u[3], float j[3][3]) {
    const float mid[3] = {(r->start[0] + u[0]) * 0.5f, (r->start[1] + u[1]) * 0.5f, (r->start[2] + u[2]) * 0.5f};
    for (int k = 0; k < 3; ++k) {
        j[k][k] = 1.0f;
        j[k][(k + 1) % 3] = 0.5f * r->coupling[k] * mid[(k + 2) % 3];
        j[k][(k + 2) % 3] = 0.5f * r->coupling[k] * mid[(k + 1) % 3];
    }
}
static float largest3(const float v[3]) { return fmaxf(fabsf(v[0]), fmaxf(fabsf(v[1]), fabsf(v[2]))); }
static int all_finite3(const float v[3]) { return isfinite(v[0]) && isfinite(v[1]) && isfinite(v[2]); }
/* x of a x = b by elimination with row pivoting, columns left to right; 0 when a pivot is below 1e-12 or not finite */
static int solve3(float a[3][3], float b[3], float x[3]) {
    for (int column = 0; column < 3; ++column) {
        int best = column;
        for (int row = column + 1; row < 3; ++row)
            if (fabsf(a[row][column]) > fabsf(a[best][column])) best = row;
        if (!isfinite(a[best][column]) || fabsf(a[best][column]) < 1.0e-12f) return 0;
        for (int k = column; k < 3; ++k) { const float held = a[column][k]; a[column][k] = a[best][k]; a[best][k] = held; }
        { const float held = b[column]; b[column] = b[best]; b[best] = held; }
        for (int row = column + 1; row < 3; ++row) {
            const float ratio = a[row][column] / a[column][column];
            for (int k = column + 1; k < 3; ++k) a[row][k] -= ratio * a[column][k];
            b[row] -= ratio * b[column];
        }
    }
    x[2] = b[2] / a[2][2];
    x[1] = (b[1] - a[1][2] * x[2]) / a[1][1];
    x[0] = (b[0] - a[0][1] * x[1] - a[0][2] * x[2]) / a[0][0];
    return 1;
}
static gyro_result solve_free_rotation(v3 w0, v3 inv_i, float dt) {
    gyro_result out;
    memset(&out, 0, sizeof(out));
    const float rate[3] = {w0.x, w0.y, w0.z}, inverse[3] = {inv_i.x, inv_i.y, inv_i.z};
    float momentum[3];
    int usable = all_finite3(rate) && all_finite3(inverse);
    for (int k = 0; k < 3; ++k) { usable = usable && inverse[k] > 0.0f; momentum[k] = rate[k] / inverse[k]; }
    if (!usable || !all_finite3(momentum)) { out.status = GYRO_INVALID_INPUT; out.residual = INFINITY; return out; }
    const float size = largest3(momentum);
    if (size == 0.0f) return out;   /* nothing turns */
    const float to_unit = 1.0f / size;
    const float a[3] = {inverse[0] * size, inverse[1] * size, inverse[2] * size};
    midpoint_rule rule;
    for (int k = 0; k < 3; ++k) { rule.start[k] = momentum[k] * to_unit; rule.coupling[k] = dt * (a[(k + 1) % 3] - a[(k + 2) % 3]); }
    float u[3] = {rule.start[0], rule.start[1], rule.start[2]};
    const uint32_t most_steps = 12u, most_halvings = 8u;
    for (uint32_t step = 0u; step <= most_steps; ++step) {
        float g[3];
        rule_residual(&rule, u, g);
        out.residual = all_finite3(g) ? largest3(g) : INFINITY;
        if (out.residual <= 1.0e-6f) {
            out.midpoint = v3_make(a[0] * ((rule.start[0] + u[0]) * 0.5f), a[1] * ((rule.start[1] + u[1]) * 0.5f), a[2] * ((rule.start[2] + u[2]) * 0.5f));
            return out;
        }
        if (step == most_steps || !isfinite(out.residual)) break;
        float j[3][3], change[3];
        rule_jacobian(&rule, u, j);
        ++out.iterations;
        if (!solve3(j, g, change)) break;
        int fell = 0;
        float length = 1.0f;
        for (uint32_t halving = 0u; halving < most_halvings && !fell; ++halving, length *= 0.5f) {
            const float trial[3] = {u[0] - change[0] * length, u[1] - change[1] * length, u[2] - change[2] * length};
            float at_trial[3];
            rule_residual(&rule, trial, at_trial);
            if (all_finite3(at_trial) && largest3(at_trial) < out.residual) { u[0] = trial[0]; u[1] = trial[1]; u[2] = trial[2]; fell = 1; }
        }
        if (!fell) break;
    }
    out.status = GYRO_NOT_CONVERGED;
    return out;
}
/* the free-rotation solve alone, for the tests: returns the status, writes the midpoint angular velocity (principal
 * frame), the residual and the Newton steps taken */
uint32_t nko_solve_free_rotation(const float w0[3], const float inv_i[3], float dt, float midpoint[3], float* residual, uint32_t* iterations) {
    const gyro_result g = solve_free_rotation(v3_make(w0[0], w0[1], w0[2]), v3_make(inv_i[0], inv_i[1], inv_i[2]), dt);
    midpoint[0] = g.midpoint.x; midpoint[1] = g.midpoint.y; midpoint[2] = g.midpoint.z;
    *residual = g.residual; *iterations = g.iterations;
    return g.status;
}

static v3 inverse_inertia_of(const nko_template* t) {   /* cook: body_inv_inertia = 1 / principal moment, 0 for none */
    const float* d = t->body_diag_inertia;
    return v3_make(d[0] > 0.0f ? 1.0f / d[0] : 0.0f, d[1] > 0.0f ? 1.0f / d[1] : 0.0f, d[2] > 0.0f ? 1.0f / d[2] : 0.0f);
}

/* BodyIntegrateVelocityKernel (articulation.cu:1019-1049): the world inverse inertia at the step's pose, gravity and the
 * applied force on the linear velocity, the applied torque on the angular velocity (no gyroscopic term here: the
 * position update carries it).  `link_wrench` holds the applied force and torque about the centre of mass, world axes,
 * and is cleared.  Then the block the tile will descend on (InitializeRigidBlock, block_descent_rigid.cuh:4-48): mass
 * matrix diag(m, m, m) and the inverse of the world inverse inertia, its L D L^T factor for the heads' inertial
 * response, and the six coordinates in the link's twist words. */
void nko_env_body_integrate_velocity(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const float dt = w->cfg.fixed_dt;
    const size_t body = (size_t)env * t->nb + t->link_body[0];   /* the body's row among the environment's bodies */
    float* lin = w->body_linear_velocity + body * 3u, *ang = w->body_angular_velocity + body * 3u;
    float* wrench = w->link_wrench + (size_t)env * 6u;
    float* inverse = w->body_world_inv_inertia + body * 6u;
    const v3 force = v3_make(wrench[0], wrench[1], wrench[2]), torque = v3_make(wrench[3], wrench[4], wrench[5]);
    for (uint32_t i = 0u; i < 6u; ++i) wrench[i] = 0.0f;
    const float inv_mass = t->body_mass > 0.0f ? 1.0f / t->body_mass : 0.0f;
    const uint32_t md = t->max_dof;
    float* M = w->m + (size_t)env * md * md, *F = w->m_factor + (size_t)env * md * md;
    for (uint32_t i = 0u; i < md * md; ++i) { M[i] = 0.0f; F[i] = 0.0f; }
    if (inv_mass <= 0.0f) {
        for (uint32_t i = 0u; i < 6u; ++i) inverse[i] = 0.0f;
    } else {
        const xform pose = xform_load(w->base_pose + (size_t)env * 7u), frame = xform_load(t->link_inertial_frame);
        body_world_inverse_inertia(pose, frame, inverse_inertia_of(t), inverse);
        const v3 g = v3_make(w->cfg.gravity[0], w->cfg.gravity[1], w->cfg.gravity[2]);
        const v3 dv = v3_scale(v3_add(g, v3_scale(force, inv_mass)), dt);
        lin[0] += dv.x; lin[1] += dv.y; lin[2] += dv.z;
        const v3 dw = v3_scale(sym_multiply(inverse, torque), dt);
        ang[0] += dw.x; ang[1] += dw.y; ang[2] += dw.z;
    }
    float inertia[6];
    const float mass = (float)(1.0 / (double)inv_mass);
    const int valid = inv_mass > 0.0f && sym_invert(inverse, inertia) && inertia[0] > 0.0f && inertia[1] > 0.0f && inertia[2] > 0.0f &&
                      (double)inertia[0] * inertia[1] > (double)inertia[3] * inertia[3] && isfinite(lin[0]) && isfinite(lin[1]) &&
                      isfinite(lin[2]) && isfinite(ang[0]) && isfinite(ang[1]) && isfinite(ang[2]);
    if (!valid) { w->env_status[env] |= NKO_STATUS_SOLVER_FAILURE; for (uint32_t i = 0u; i < 6u; ++i) inertia[i] = i < 3u ? 1.0f : 0.0f; }
    const float rotational[3][3] = {{inertia[0], inertia[3], inertia[4]}, {inertia[3], inertia[1], inertia[5]}, {inertia[4], inertia[5], inertia[2]}};
    for (uint32_t r = 0u; r < 6u; ++r)
        for (uint32_t c = 0u; c < 6u; ++c) {
            float value = 0.0f;
            if (r < 3u && c < 3u && r == c) value = valid ? mass : 1.0f;
            if (r >= 3u && c >= 3u) value = rotational[r - 3u][c - 3u];
            M[(size_t)r * md + c] = value;
        }
    nko_factor_mass(M, F, 6u, md);
    float* twist = w->link_velocity + (size_t)env * 6u;
    for (uint32_t i = 0u; i < 3u; ++i) { twist[i] = lin[i]; twist[3u + i] = ang[i]; }
    for (uint32_t i = 0u; i < md; ++i) { w->articulation_qdd[(size_t)env * md + i] = 0.0f; w->articulation_bias[(size_t)env * md + i] = 0.0f; }
}

/* BodyIntegratePositionKernel (articulation.cu:1058-1117): the solve's velocities from the link's twist words; the
 * angular momentum is carried through the step in world axes while the pose turns by the midpoint angular velocity of
 * the free-rotation solve (and by the position pass's pseudo velocity, which moves the pose only); the centre of mass
 * moves with the linear velocity. */
void nko_env_body_integrate_position(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const float dt = w->cfg.fixed_dt;
    const int pos_pass = w->cfg.solver_pos_iters > 0u && t->rows_per_env > 0u;
    const size_t body = (size_t)env * t->nb + t->link_body[0];
    float* lin = w->body_linear_velocity + body * 3u, *ang = w->body_angular_velocity + body * 3u;
    float* twist = w->link_velocity + (size_t)env * 6u;
    if (t->rows_per_env > 0u) for (uint32_t i = 0u; i < 3u; ++i) { lin[i] = twist[i]; ang[i] = twist[3u + i]; }
    w->body_gyro_residual[body] = 0.0f; w->body_gyro_iterations[body] = 0u; w->body_gyro_status[body] = 0u;
    if (!(t->body_mass > 0.0f)) return;
    xform pose = xform_load(w->base_pose + (size_t)env * 7u);
    const xform frame = xform_load(t->link_inertial_frame);
    const v3 inv_i = inverse_inertia_of(t);
    const quat principal = nko_quat_normalize_rsqrt(nko_quat_mul(pose.r, frame.r), 1.0e-12f);
    const quat inverse = quat_make(principal.w, -principal.x, -principal.y, -principal.z);
    const v3 w0 = nko_rotate_normalized(inverse, v3_make(ang[0], ang[1], ang[2]));
    const gyro_result gyro = solve_free_rotation(w0, inv_i, dt);
    w->body_gyro_residual[body] = gyro.residual; w->body_gyro_iterations[body] = gyro.iterations; w->body_gyro_status[body] = gyro.status;
    if (gyro.status != 0u) { w->env_status[env] |= NKO_STATUS_GYRO_FAILURE; return; }
    const v3 momentum = nko_rotate_normalized(principal, v3_make(w0.x / inv_i.x, w0.y / inv_i.y, w0.z / inv_i.z));
    v3 v = v3_make(lin[0], lin[1], lin[2]);
    const v3 wm = nko_rotate_normalized(principal, gyro.midpoint);
    const v3 center = body_center_of_mass(pose, frame);
    const quat dq = quat_make(1.0f, 0.5f * dt * wm.x, 0.5f * dt * wm.y, 0.5f * dt * wm.z);
    quat q = nko_quat_normalize_rsqrt(nko_quat_mul(dq, pose.r), 1.0e-12f);
    if (pos_pass) {
        const float* pseudo = w->link_velocity_pseudo + (size_t)env * 6u;
        v = v3_add(v, v3_make(pseudo[0], pseudo[1], pseudo[2]));
        const quat turn = quat_make(1.0f, 0.5f * dt * pseudo[3], 0.5f * dt * pseudo[4], 0.5f * dt * pseudo[5]);
        q = nko_quat_normalize_rsqrt(nko_quat_mul(turn, q), 1.0e-12f);
    }
    pose.r = q;
    const v3 offset = nko_rotate_normalized(q, frame.p);
    pose.p = v3_sub(v3_add(center, v3_scale(v, dt)), offset);
    xform_store(w->base_pose + (size_t)env * 7u, pose);
    float* world_inverse = w->body_world_inv_inertia + body * 6u;
    body_world_inverse_inertia(pose, frame, inv_i, world_inverse);
    const v3 turned = sym_multiply(world_inverse, momentum);
    ang[0] = turned.x; ang[1] = turned.y; ang[2] = turned.z;
    for (uint32_t i = 0u; i < 3u; ++i) { twist[i] = lin[i]; twist[3u + i] = ang[i]; }
}
