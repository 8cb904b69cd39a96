// A free rigid body (ModelView::free_body): the reference's rigid-body ops around the contact solve.
//
// The reference steps such a body with BodyIntegrateVelocityKernel before the solve (articulation.cu:1019-1049), a six
// by six block of the tile in it (block_descent_rigid.cuh:4-48, block_descent_tile.cuh:541-603) and
// BodyIntegratePositionKernel with the free-rotation solve after it (articulation.cu:1058-1117, rigid_types.cuh:38-121).
// Here the body is the template's one link: `base_pose` is its pose, `body_linear_velocity` / `body_angular_velocity`
// (per body row, as in the reference: the link's own row holds them) its state, and the six coordinates - linear
// velocity, then angular velocity about the centre of mass, world axes - pass through the link's twist words to the row
// assembly and the block descent, which take the block's mass matrix and its factor from `m` / `m_factor` as for an
// articulation.  One thread an environment: the work is a few hundred operations on a body.
#include <cfloat>

#include "nk_device_math.h"
#include "nk_ops.h"

namespace nkh {
namespace {

// math/symmetric_mat3.hpp:31-47 FromRotatedDiagonal: R diag(d) R^T of the rotation of q, as xx yy zz xy xz yz
__device__ void from_rotated_diagonal(V3 d, Q4 q, float* out) {
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    const float s = norm_sq > 1.0e-12f ? 2.0f / norm_sq : 0.0f;
    const V3 x{1.0f - s * (q.y * q.y + q.z * q.z), s * (q.x * q.y - q.w * q.z), s * (q.x * q.z + q.w * q.y)};
    const V3 y{s * (q.x * q.y + q.w * q.z), 1.0f - s * (q.x * q.x + q.z * q.z), s * (q.y * q.z - q.w * q.x)};
    const V3 z{s * (q.x * q.z - q.w * q.y), s * (q.y * q.z + q.w * q.x), 1.0f - s * (q.x * q.x + q.y * q.y)};
    out[0] = d.x * x.x * x.x + d.y * x.y * x.y + d.z * x.z * x.z;
    out[1] = d.x * y.x * y.x + d.y * y.y * y.y + d.z * y.z * y.z;
    out[2] = d.x * z.x * z.x + d.y * z.y * z.y + d.z * z.z * z.z;
    out[3] = d.x * x.x * y.x + d.y * x.y * y.y + d.z * x.z * y.z;
    out[4] = d.x * x.x * z.x + d.y * x.y * z.y + d.z * x.z * z.z;
    out[5] = d.x * y.x * z.x + d.y * y.y * z.y + d.z * y.z * z.z;
}
// math/symmetric_mat3.hpp:25-29 Multiply
__device__ V3 sym_multiply(const float* m, V3 v) {
    return V3{m[0] * v.x + m[3] * v.y + m[4] * v.z, m[3] * v.x + m[1] * v.y + m[5] * v.z, m[4] * v.x + m[5] * v.y + m[2] * v.z};
}
// nk/solve/vertex_block.hpp:139-153 Invert (floor 0): cofactors in double, rounded once
__device__ bool sym_invert(const float* m, float* out) {
    const double xx = m[0], yy = m[1], zz = m[2], xy = m[3], xz = m[4], yz = m[5];
    const double cxx = yy * zz - yz * yz, cyy = xx * zz - xz * xz;
    const double czz = xx * yy - xy * xy, cxy = xz * yz - xy * zz;
    const double cxz = xy * yz - xz * yy, cyz = xy * xz - xx * yz;
    const double det = xx * cxx + xy * cxy + xz * cxz;
    if (!(det > 0.0 && det <= DBL_MAX)) return false;
    const double inv = 1.0 / det;
    const double values[6] = {cxx * inv, cyy * inv, czz * inv, cxy * inv, cxz * inv, cyz * inv};
    bool ok = true;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        ok = ok && values[i] >= -double(FLT_MAX) && values[i] <= double(FLT_MAX);
        out[i] = float(values[i]);
    }
    return ok;
}
// rigid_types.cuh:10-14, 16-21
__device__ V3 body_center_of_mass(Xf pose, Xf frame) { return add3(pose.p, rotate_normalized(pose.r, frame.p)); }
__device__ void body_world_inverse_inertia(Xf pose, Xf frame, V3 inv_i, float* out) { from_rotated_diagonal(inv_i, qmul(pose.r, frame.r), out); }

__device__ bool finite3(V3 v) { return isfinite(v.x) && isfinite(v.y) && isfinite(v.z); }

// The free-rotation step (rigid_types.cuh:38-121 SolveFreeRotation): Euler's equations in the principal frame by the
// implicit midpoint rule, m1 - m0 = dt (m_mid x w_mid), solved for the end-of-step angular momentum.  The unknown is the
// momentum scaled to unit size, `g(u) = u - u0 + c o (mid_y mid_z, mid_z mid_x, mid_x mid_y)` with mid = (u0 + u) / 2
// and c = dt (a_y - a_z, a_z - a_x, a_x - a_y), a = scaled inverse moments; Newton steps on g with a halved step while
// the residual does not fall, at most twelve, to a residual of 1e-6.  Returns the angular velocity at the middle of the
// step, which turns the pose.
struct FreeRotation { V3 midpoint; float residual; uint32_t iterations, status; };
enum : uint32_t { kGyroConverged = 0u, kGyroNotConverged = 1u, kGyroInvalidInput = 2u };   // op_schema.hpp:53-54

struct MidpointRule {
    float start[3], coupling[3];
    __device__ void residual(const float (&u)[3], float (&g)[3]) const {
        const float mid[3] = {(start[0] + u[0]) * 0.5f, (start[1] + u[1]) * 0.5f, (start[2] + u[2]) * 0.5f};
#pragma unroll
        for (int k = 0; k < 3; ++k) g[k] = u[k] - start[k] + coupling[k] * mid[(k + 1) % 3] * mid[(k + 2) % 3];
    }
    // dg/du: the identity and half the coupling times the other two midpoint components
    __device__ void jacobian(const float (&u)[3], float (&j)[3][3]) const {
        const float mid[3] = {(start[0] + u[0]) * 0.5f, (start[1] + u[1]) * 0.5f, (start[2] + u[2]) * 0.5f};
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            j[k][k] = 1.0f;
            j[k][(k + 1) % 3] = 0.5f * coupling[k] * mid[(k + 2) % 3];
            j[k][(k + 2) % 3] = 0.5f * coupling[k] * mid[(k + 1) % 3];
        }
    }
};
__device__ float largest3(const float (&v)[3]) { return fmaxf(fabsf(v[0]), fmaxf(fabsf(v[1]), fabsf(v[2]))); }
__device__ bool all_finite3(const float (&v)[3]) { return isfinite(v[0]) && isfinite(v[1]) && isfinite(v[2]); }
// x of a x = b by elimination with row pivoting, columns left to right; false when a pivot is below 1e-12 or not finite
__device__ bool solve3(float (&a)[3][3], float (&b)[3], float (&x)[3]) {
    for (int column = 0; column < 3; ++column) {
        int best = column;
        for (int row = column + 1; row < 3; ++row)
            if (fabsf(a[row][column]) > fabsf(a[best][column])) best = row;
        if (!isfinite(a[best][column]) || fabsf(a[best][column]) < 1.0e-12f) return false;
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
    return true;
}
__device__ FreeRotation solve_free_rotation(V3 w0, V3 inv_i, float dt) {
    FreeRotation out{V3{0.0f, 0.0f, 0.0f}, 0.0f, 0u, kGyroConverged};
    const float rate[3] = {w0.x, w0.y, w0.z}, inverse[3] = {inv_i.x, inv_i.y, inv_i.z};
    float momentum[3];
    bool usable = all_finite3(rate) && all_finite3(inverse);
#pragma unroll
    for (int k = 0; k < 3; ++k) { usable = usable && inverse[k] > 0.0f; momentum[k] = rate[k] / inverse[k]; }
    if (!usable || !all_finite3(momentum)) { out.status = kGyroInvalidInput; out.residual = INFINITY; return out; }
    const float size = largest3(momentum);
    if (size == 0.0f) return out;   // nothing turns
    const float to_unit = 1.0f / size;
    const float a[3] = {inverse[0] * size, inverse[1] * size, inverse[2] * size};
    MidpointRule rule;
#pragma unroll
    for (int k = 0; k < 3; ++k) { rule.start[k] = momentum[k] * to_unit; rule.coupling[k] = dt * (a[(k + 1) % 3] - a[(k + 2) % 3]); }
    float u[3] = {rule.start[0], rule.start[1], rule.start[2]};
    constexpr uint32_t kMostSteps = 12u, kMostHalvings = 8u;
    for (uint32_t step = 0u; step <= kMostSteps; ++step) {
        float g[3];
        rule.residual(u, g);
        out.residual = all_finite3(g) ? largest3(g) : INFINITY;
        if (out.residual <= 1.0e-6f) {
            out.midpoint = V3{a[0] * ((rule.start[0] + u[0]) * 0.5f), a[1] * ((rule.start[1] + u[1]) * 0.5f), a[2] * ((rule.start[2] + u[2]) * 0.5f)};
            return out;
        }
        if (step == kMostSteps || !isfinite(out.residual)) break;
        float j[3][3], change[3];
        rule.jacobian(u, j);
        ++out.iterations;
        if (!solve3(j, g, change)) break;
        bool fell = false;
        float length = 1.0f;
        for (uint32_t halving = 0u; halving < kMostHalvings && !fell; ++halving, length *= 0.5f) {
            const float trial[3] = {u[0] - change[0] * length, u[1] - change[1] * length, u[2] - change[2] * length};
            float at_trial[3];
            rule.residual(trial, at_trial);
            if (all_finite3(at_trial) && largest3(at_trial) < out.residual) { u[0] = trial[0]; u[1] = trial[1]; u[2] = trial[2]; fell = true; }
        }
        if (!fell) break;
    }
    out.status = kGyroNotConverged;
    return out;
}

// BodyIntegrateVelocityKernel (articulation.cu:1019-1049): the world inverse inertia at the step's pose, gravity and the
// applied force on the linear velocity, the applied torque on the angular velocity (`link_wrench`: force and torque
// about the centre of mass in world axes, cleared here).  Then the block the solve descends on (InitializeRigidBlock,
// block_descent_rigid.cuh:4-48): the mass matrix diag(m, m, m) with the inverse of the world inverse inertia, its
// L D L^T factor (FactorMass, articulation_mass.cuh:269-335, right-looking) for the heads' inertial response, and the six
// coordinates in the link's twist words.
__global__ void __launch_bounds__(256) BodyIntegrateVelocityKernel(ModelView m, DataView d, IntegrateVelocityParams p, uint32_t env_count) {
    const uint32_t env = blockIdx.x * blockDim.x + threadIdx.x;
    if (env >= env_count) return;
    const size_t body = size_t{env} * m.bodies_per_env + m.link_body[0];   // the body's row among the environment's bodies
    float* lin = d.body_linear_velocity + body * 3u, *ang = d.body_angular_velocity + body * 3u;
    float* wrench = d.link_wrench + size_t{env} * 6u;
    float* inverse = d.body_world_inv_inertia + body * 6u;
    const V3 force{wrench[0], wrench[1], wrench[2]}, torque{wrench[3], wrench[4], wrench[5]};
    if (p.clear_body_forces != 0u)
        for (uint32_t i = 0u; i < 6u; ++i) wrench[i] = 0.0f;
    const float inv_mass = d.body_inv_mass[body];
    const uint32_t md = m.max_dof;
    float* M = d.m + size_t{env} * md * md, *F = d.m_factor + size_t{env} * md * md;
    V3 v{lin[0], lin[1], lin[2]}, w{ang[0], ang[1], ang[2]};
    float world_inverse[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (inv_mass > 0.0f) {
        const Xf pose = load_xf(d.base_pose + size_t{env} * 7u), frame = load_xf(d.body_inertial_frame + body * 7u);
        const float* inv_i = d.body_inv_inertia + body * 3u;
        body_world_inverse_inertia(pose, frame, V3{inv_i[0], inv_i[1], inv_i[2]}, world_inverse);
        const V3 g{p.gravity[0], p.gravity[1], p.gravity[2]};
        v = add3(v, scale3(add3(g, scale3(force, inv_mass)), p.dt));
        w = add3(w, scale3(sym_multiply(world_inverse, torque), p.dt));
    }
    for (uint32_t i = 0u; i < 6u; ++i) inverse[i] = world_inverse[i];
    lin[0] = v.x; lin[1] = v.y; lin[2] = v.z; ang[0] = w.x; ang[1] = w.y; ang[2] = w.z;
    float inertia[6];
    const float mass = float(1.0 / double(inv_mass));
    const bool valid = inv_mass > 0.0f && sym_invert(world_inverse, inertia) && inertia[0] > 0.0f && inertia[1] > 0.0f && inertia[2] > 0.0f &&
                       double(inertia[0]) * inertia[1] > double(inertia[3]) * inertia[3] && finite3(v) && finite3(w);
    if (!valid) {
        atomicOr(d.env_status + env, uint32_t(kEnvStatusSolverFailure));
        for (uint32_t i = 0u; i < 6u; ++i) inertia[i] = i < 3u ? 1.0f : 0.0f;
    }
    // the block is diag(m, m, m) and a symmetric three by three: the factor of the first is itself, the second's follows
    // the right-looking order of FactorMass with its pivot floor
    float a[3][3] = {{inertia[0], inertia[3], inertia[4]}, {inertia[3], inertia[1], inertia[5]}, {inertia[4], inertia[5], inertia[2]}};
    float work[3][3] = {{0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f}};
    const float linear = valid ? mass : 1.0f;
    for (uint32_t r = 0u; r < md; ++r)
        for (uint32_t c = 0u; c < md; ++c) {
            float value = 0.0f;
            if (r < 3u && c < 3u && r == c) value = linear;
            if (r >= 3u && r < 6u && c >= 3u && c < 6u) value = a[r - 3u][c - 3u];
            M[size_t{r} * md + c] = value;
        }
    for (uint32_t k = 0u; k < 3u; ++k) {
        const float diagonal = fmaxf(a[k][k], 1.0e-6f);
        for (uint32_t i = k + 1u; i < 3u; ++i) work[i][k] = a[i][k] / diagonal;
        work[k][k] = diagonal;
        for (uint32_t i = k + 1u; i < 3u; ++i) {
            const float l = work[i][k];
            for (uint32_t j = k + 1u; j <= i; ++j) a[i][j] -= l * work[j][k] * diagonal;
        }
    }
    for (uint32_t r = 0u; r < md; ++r)
        for (uint32_t c = 0u; c <= r; ++c) {
            float value = r == c ? 1.0e-6f : 0.0f;   // rows past the coordinates (articulation_mass.cuh:333)
            if (r < 3u) value = r == c ? fmaxf(linear, 1.0e-6f) : 0.0f;
            else if (r < 6u) value = c >= 3u ? work[r - 3u][c - 3u] : 0.0f;
            F[size_t{r} * md + c] = value;
        }
    float* twist = d.link_velocity + size_t{env} * 6u;
    twist[0] = v.x; twist[1] = v.y; twist[2] = v.z; twist[3] = w.x; twist[4] = w.y; twist[5] = w.z;
    for (uint32_t i = 0u; i < md; ++i) { d.articulation_qdd[size_t{env} * md + i] = 0.0f; d.articulation_bias[size_t{env} * md + i] = 0.0f; }
}

// BodyIntegratePositionKernel (articulation.cu:1058-1117): the solve's velocities from the link's twist words; the
// angular momentum goes through the step in world axes while the pose turns by the midpoint angular velocity of the
// free-rotation solve (and by the position pass's pseudo velocity, which moves the pose only); the centre of mass moves
// with the linear velocity.
__global__ void __launch_bounds__(256) BodyIntegratePositionKernel(ModelView m, DataView d, IntegratePositionParams p, uint32_t env_count) {
    const uint32_t env = blockIdx.x * blockDim.x + threadIdx.x;
    if (env >= env_count) return;
    const size_t body = size_t{env} * m.bodies_per_env + m.link_body[0];
    float* lin = d.body_linear_velocity + body * 3u, *ang = d.body_angular_velocity + body * 3u;
    float* twist = d.link_velocity + size_t{env} * 6u;
    if (m.rows_per_env > 0u)
        for (uint32_t i = 0u; i < 3u; ++i) { lin[i] = twist[i]; ang[i] = twist[3u + i]; }
    d.body_gyro_residual[body] = 0.0f; d.body_gyro_iterations[body] = 0u; d.body_gyro_status[body] = 0u;
    if (!(d.body_inv_mass[body] > 0.0f)) return;
    Xf pose = load_xf(d.base_pose + size_t{env} * 7u);
    const Xf frame = load_xf(d.body_inertial_frame + body * 7u);
    const V3 inv_i{d.body_inv_inertia[body * 3u], d.body_inv_inertia[body * 3u + 1u], d.body_inv_inertia[body * 3u + 2u]};
    const Q4 principal = qnormalize_le(qmul(pose.r, frame.r), 1.0e-12f);
    const Q4 inverse{principal.w, -principal.x, -principal.y, -principal.z};
    const V3 w0 = rotate_normalized(inverse, V3{ang[0], ang[1], ang[2]});
    const FreeRotation gyro = solve_free_rotation(w0, inv_i, p.dt);
    d.body_gyro_residual[body] = gyro.residual; d.body_gyro_iterations[body] = gyro.iterations; d.body_gyro_status[body] = gyro.status;
    if (gyro.status != 0u) { atomicOr(d.env_status + env, uint32_t(kEnvStatusGyroFailure)); return; }
    const V3 momentum = rotate_normalized(principal, V3{w0.x / inv_i.x, w0.y / inv_i.y, w0.z / inv_i.z});
    V3 v{lin[0], lin[1], lin[2]};
    const V3 wm = rotate_normalized(principal, gyro.midpoint);
    const V3 center = body_center_of_mass(pose, frame);
    const Q4 dq{1.0f, 0.5f * p.dt * wm.x, 0.5f * p.dt * wm.y, 0.5f * p.dt * wm.z};
    Q4 q = qnormalize_le(qmul(dq, pose.r), 1.0e-12f);
    if (p.pos_pass != 0u) {
        const float* pseudo = d.link_velocity_pseudo + size_t{env} * 6u;
        v = add3(v, V3{pseudo[0], pseudo[1], pseudo[2]});
        const Q4 turn{1.0f, 0.5f * p.dt * pseudo[3], 0.5f * p.dt * pseudo[4], 0.5f * p.dt * pseudo[5]};
        q = qnormalize_le(qmul(turn, q), 1.0e-12f);
    }
    pose.r = q;
    const V3 offset = rotate_normalized(q, frame.p);
    pose.p = sub3(add3(center, scale3(v, p.dt)), offset);
    store_xf(d.base_pose + size_t{env} * 7u, pose);
    float world_inverse[6];
    body_world_inverse_inertia(pose, frame, inv_i, world_inverse);
    for (uint32_t i = 0u; i < 6u; ++i) d.body_world_inv_inertia[body * 6u + i] = world_inverse[i];
    const V3 turned = sym_multiply(world_inverse, momentum);
    ang[0] = turned.x; ang[1] = turned.y; ang[2] = turned.z;
    for (uint32_t i = 0u; i < 3u; ++i) { twist[i] = lin[i]; twist[3u + i] = ang[i]; }
}

}  // namespace

Status BodyIntegrateVelocity(const ModelView& m, const DataView& d, const IntegrateVelocityParams& p, hipStream_t stream) {
    if (m.links_per_env != 1u || m.dof != 6u || m.max_dof < 6u || p.articulation_count == 0u) return Status::InvalidArgument;
    const uint32_t E = p.articulation_count;
    hipLaunchKernelGGL(BodyIntegrateVelocityKernel, dim3((E + 255u) / 256u), dim3(256), 0, stream, m, d, p, E);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}
Status BodyIntegratePosition(const ModelView& m, const DataView& d, const IntegratePositionParams& p, hipStream_t stream) {
    if (m.links_per_env != 1u || m.dof != 6u || p.env_count == 0u) return Status::InvalidArgument;
    hipLaunchKernelGGL(BodyIntegratePositionKernel, dim3((p.env_count + 255u) / 256u), dim3(256), 0, stream, m, d, p, p.env_count);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

}  // namespace nkh
