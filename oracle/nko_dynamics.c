/*
 * CPU oracle (test infrastructure; see nuka_oracle.h): small-vector math, forward kinematics,
 * RNEA bias + CRBA + LDL^T forward dynamics, position integration, link twists.
 * Operation order follows the cited reference lines; no FMA contraction (build with -ffp-contract=off).
 */
#include "nko_internal.h"

/* ---- math -------------------------------------------------------------- */

/* math/cuda_vec_ops.cuh:207-213 QuatMul */
quat nko_quat_mul(quat a, quat b) {
    return quat_make(a.w * b.w - a.x * b.x - a.y * b.y - a.z * b.z,
                     a.w * b.x + a.x * b.w + a.y * b.z - a.z * b.y,
                     a.w * b.y - a.x * b.z + a.y * b.w + a.z * b.x,
                     a.w * b.z + a.x * b.y - a.y * b.x + a.z * b.w);
}

/* math/cuda_vec_ops.cuh:254-261 QuatNormalizeRsqrt (rsqrtf restated as 1/sqrtf) */
quat nko_quat_normalize_rsqrt(quat q, float eps) {
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq <= eps) return quat_make(1.0f, 0.0f, 0.0f, 0.0f);
    const float inv = nko_rsqrt(norm_sq);
    return quat_make(q.w * inv, q.x * inv, q.y * inv, q.z * inv);
}

/* math/cuda_vec_ops.cuh:263-284 QuatNormalizeForwardRsqrt (strict <) */
static quat quat_normalize_forward(quat q, float eps) {
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq < eps) return quat_make(1.0f, 0.0f, 0.0f, 0.0f);
    const float inv = nko_rsqrt(norm_sq);
    q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    return q;
}

/* math/cuda_vec_ops.cuh:297-312 RotateByQuatNormalized */
v3 nko_rotate_normalized(quat q, v3 v) {
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq > 1.0e-12f) {
        const float inv = nko_rsqrt(norm_sq);
        q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    }
    const v3 qv = v3_make(q.x, q.y, q.z);
    const v3 t = v3_cross(qv, v);
    const v3 t2 = v3_make(2.0f * t.x, 2.0f * t.y, 2.0f * t.z);
    const v3 wt = v3_make(q.w * t2.x, q.w * t2.y, q.w * t2.z);
    const v3 qvt = v3_cross(qv, t2);
    return v3_make(v.x + wt.x + qvt.x, v.y + wt.y + qvt.y, v.z + wt.z + qvt.z);
}

/* articulation.cu:220-233 RotateByQuatInverse */
v3 nko_rotate_inverse(quat q, v3 v) {
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq > 1.0e-12f) {
        const float inv = nko_rsqrt(norm_sq);
        q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    }
    const v3 qv = v3_make(-q.x, -q.y, -q.z);
    const v3 t = v3_scale(v3_cross(qv, v), 2.0f);
    return v3_add(v, v3_add(v3_scale(t, q.w), v3_cross(qv, t)));
}

/* articulation.cu:709-721 RotateByQuatForward */
v3 nko_rotate_forward(quat q, v3 v) {
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq > 1.0e-12f) {
        const float inv = nko_rsqrt(norm_sq);
        q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    }
    const v3 qv = v3_make(q.x, q.y, q.z);
    const v3 t = v3_scale(v3_cross(qv, v), 2.0f);
    return v3_add(v, v3_add(v3_scale(t, q.w), v3_cross(qv, t)));
}

/* prims_types.cuh:92-96 PrimRotate (no normalisation) */
v3 nko_prim_rotate(quat q, v3 v) {
    const v3 qv = v3_make(q.x, q.y, q.z);
    const v3 t = v3_scale(v3_cross(qv, v), 2.0f);
    return v3_add(v3_add(v, v3_scale(t, q.w)), v3_cross(qv, t));
}

/* articulation.cu:1136-1158 RotateByQuat + ComposeTransform (FK composition) */
xform nko_compose_frame(xform parent, xform local) {
    quat q = parent.r;
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq > 1.0e-12f) {
        const float inv = nko_rsqrt(norm_sq);
        q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    }
    const v3 qv = v3_make(q.x, q.y, q.z);
    const v3 t = v3_scale(v3_cross(qv, local.p), 2.0f);
    const v3 wt = v3_scale(t, q.w);
    const v3 qvt = v3_cross(qv, t);
    xform out;
    out.p = v3_add(parent.p, v3_add(v3_add(local.p, wt), qvt));
    out.r = nko_quat_normalize_rsqrt(nko_quat_mul(parent.r, local.r), 1.0e-12f);
    return out;
}

/* collision/analytical_manifold.hpp:130-171 RotateByQuatHD + QuatMulHD + ComposeTransformHD */
xform nko_compose_hd(xform parent, xform child) {
    quat q = parent.r;
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq > 1.0e-12f) {
        const float inv = 1.0f / sqrtf(norm_sq);
        q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    }
    const v3 qv = v3_make(q.x, q.y, q.z), v = child.p;
    const v3 t = v3_make(2.0f * (qv.y * v.z - qv.z * v.y), 2.0f * (qv.z * v.x - qv.x * v.z),
                         2.0f * (qv.x * v.y - qv.y * v.x));
    const v3 qvt = v3_cross(qv, t);
    xform out;
    out.p = v3_add(parent.p, v3_make(v.x + q.w * t.x + qvt.x, v.y + q.w * t.y + qvt.y, v.z + q.w * t.z + qvt.z));
    out.r = nko_quat_mul(parent.r, child.r);
    return out;
}

/* articulation_types.cuh:100-114 JointDofCountDevice */
uint32_t nko_joint_dof(uint8_t type) {
    switch (type) {
        case NKO_REVOLUTE: case NKO_PRISMATIC: return 1u;
        case NKO_FLOATING: return 6u;
        case NKO_SPHERICAL: return 3u;
        default: return 0u;
    }
}

/* ---- cook: spatial inertia (runtime/articulation/articulation_state.cpp:113-165, 307-343) ---- */

static void rotation_from_quat_host(quat q, float* out) {
    const float n = sqrtf(q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z);
    if (n > 0.0f) { const float inv = 1.0f / n; q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv; }
    const float xx = q.x * q.x, yy = q.y * q.y, zz = q.z * q.z, xy = q.x * q.y, xz = q.x * q.z, yz = q.y * q.z;
    const float wx = q.w * q.x, wy = q.w * q.y, wz = q.w * q.z;
    out[0] = 1.0f - 2.0f * (yy + zz); out[1] = 2.0f * (xy - wz); out[2] = 2.0f * (xz + wy);
    out[3] = 2.0f * (xy + wz); out[4] = 1.0f - 2.0f * (xx + zz); out[5] = 2.0f * (yz - wx);
    out[6] = 2.0f * (xz - wy); out[7] = 2.0f * (yz + wx); out[8] = 1.0f - 2.0f * (xx + yy);
}

void nko_make_spatial_inertia(float mass, const float diag[3], const float inertial_frame[7], float I[36]) {
    memset(I, 0, 36 * sizeof(float));
    if (mass <= 0.0f) return;
    const xform frame = xform_load(inertial_frame);
    float r[9], com[9];
    rotation_from_quat_host(frame.r, r);
    for (uint32_t row = 0u; row < 3u; ++row)
        for (uint32_t col = 0u; col < 3u; ++col) {
            float value = 0.0f;
            for (uint32_t k = 0u; k < 3u; ++k) value += r[row * 3u + k] * diag[k] * r[col * 3u + k];
            com[row * 3u + col] = value;
        }
    const v3 c = frame.p;
    const float c_dot = v3_dot(c, c);
    const float parallel[9] = {c_dot - c.x * c.x, -c.x * c.y, -c.x * c.z, -c.y * c.x, c_dot - c.y * c.y, -c.y * c.z,
                               -c.z * c.x, -c.z * c.y, c_dot - c.z * c.z};
    const float cross[9] = {0.0f, -c.z, c.y, c.z, 0.0f, -c.x, -c.y, c.x, 0.0f};
    for (uint32_t row = 0u; row < 3u; ++row)
        for (uint32_t col = 0u; col < 3u; ++col) {
            I[row * 6u + col] = com[row * 3u + col] + mass * parallel[row * 3u + col];
            I[row * 6u + 3u + col] += mass * cross[row * 3u + col];
            I[(3u + row) * 6u + col] += -mass * cross[row * 3u + col];
            I[(3u + row) * 6u + 3u + col] = row == col ? mass : 0.0f;
        }
}

/* ---- spatial algebra (math/cuda_spatial_ops.cuh) ------------------------ */

static void mat66_mul_vec6(const float* m, const float* v, float* out) {   /* :78-88 */
    for (uint32_t row = 0u; row < 6u; ++row) {
        float value = 0.0f;
        for (uint32_t col = 0u; col < 6u; ++col) value += m[row * 6u + col] * v[col];
        out[row] = value;
    }
}
static void transform_force_transpose(const float* X, const float* in, float* out) {   /* :125-135 */
    for (uint32_t row = 0u; row < 6u; ++row) {
        float value = 0.0f;
        for (uint32_t col = 0u; col < 6u; ++col) value += X[col * 6u + row] * in[col];
        out[row] = value;
    }
}
static void transform_inertia_to_parent(const float* X, const float* child, float* delta) {   /* :140-162 */
    float temp[36];
    for (uint32_t row = 0u; row < 6u; ++row)
        for (uint32_t col = 0u; col < 6u; ++col) {
            float value = 0.0f;
            for (uint32_t k = 0u; k < 6u; ++k) value += child[row * 6u + k] * X[k * 6u + col];
            temp[row * 6u + col] = value;
        }
    for (uint32_t row = 0u; row < 6u; ++row)
        for (uint32_t col = 0u; col < 6u; ++col) {
            float value = 0.0f;
            for (uint32_t k = 0u; k < 6u; ++k) value += X[k * 6u + row] * temp[k * 6u + col];
            delta[row * 6u + col] = value;
        }
}
static float dot6(const float* a, const float* b) {   /* :56-62 */
    float sum = 0.0f;
    for (uint32_t i = 0u; i < 6u; ++i) sum += a[i] * b[i];
    return sum;
}
static void motion_cross(const float* l, const float* r, float* out) {   /* :170-185 */
    const v3 lw = v3_make(l[0], l[1], l[2]), lv = v3_make(l[3], l[4], l[5]);
    const v3 rw = v3_make(r[0], r[1], r[2]), rv = v3_make(r[3], r[4], r[5]);
    const v3 ang = v3_cross(lw, rw), lin = v3_add(v3_cross(lw, rv), v3_cross(lv, rw));
    out[0] = ang.x; out[1] = ang.y; out[2] = ang.z; out[3] = lin.x; out[4] = lin.y; out[5] = lin.z;
}
static void force_cross(const float* m, const float* f, float* out) {   /* :236-250 */
    const v3 w = v3_make(m[0], m[1], m[2]), v = v3_make(m[3], m[4], m[5]);
    const v3 n = v3_make(f[0], f[1], f[2]), ff = v3_make(f[3], f[4], f[5]);
    const v3 ang = v3_add(v3_cross(w, n), v3_cross(v, ff)), lin = v3_cross(w, ff);
    out[0] = ang.x; out[1] = ang.y; out[2] = ang.z; out[3] = lin.x; out[4] = lin.y; out[5] = lin.z;
}

/* ---- joint frames ------------------------------------------------------- */

static v3 joint_unit_axis(v3 axis) {   /* kinematics.cuh:9-12 */
    const float l = v3_dot(axis, axis);
    return l > 1.0e-12f ? v3_scale(axis, nko_rsqrt(l)) : v3_make(0.0f, 0.0f, 0.0f);
}

/* kinematics.cuh:25-42 JointRelativeFrame */
static xform joint_relative_frame(uint8_t type, v3 axis, xform local, v3 parent_offset, float coordinate) {
    xform result = local;
    result.p = v3_add(local.p, parent_offset);
    axis = joint_unit_axis(axis);
    if (type == NKO_REVOLUTE) {
        const float half = 0.5f * coordinate;
        const float sine = sinf(half);
        const quat turn = quat_make(cosf(half), axis.x * sine, axis.y * sine, axis.z * sine);
        result.r = nko_quat_normalize_rsqrt(nko_quat_mul(local.r, turn), 1.0e-12f);
    } else if (type == NKO_PRISMATIC) {
        result.p = v3_add(result.p, nko_rotate_normalized(local.r, v3_scale(axis, coordinate)));
    }
    return result;
}

static void mat3_from_quat(quat q, float* m) {   /* articulation.cu:91-124 RotationFromQuat */
    const float norm_sq = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (norm_sq <= 1.0e-12f) {
        const float id[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
        memcpy(m, id, sizeof(id));
        return;
    }
    const float inv = nko_rsqrt(norm_sq);
    q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    const float xx = q.x * q.x, yy = q.y * q.y, zz = q.z * q.z, xy = q.x * q.y, xz = q.x * q.z, yz = q.y * q.z;
    const float wx = q.w * q.x, wy = q.w * q.y, wz = q.w * q.z;
    m[0] = 1.0f - 2.0f * (yy + zz); m[1] = 2.0f * (xy - wz); m[2] = 2.0f * (xz + wy);
    m[3] = 2.0f * (xy + wz); m[4] = 1.0f - 2.0f * (xx + zz); m[5] = 2.0f * (yz - wx);
    m[6] = 2.0f * (xz - wy); m[7] = 2.0f * (yz + wx); m[8] = 1.0f - 2.0f * (xx + yy);
}

static void mat3_axis_angle(v3 axis, float angle, float* m) {   /* articulation.cu:126-147 */
    const float l = v3_dot(axis, axis);
    if (l <= 1.0e-12f) {
        const float id[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
        memcpy(m, id, sizeof(id));
        return;
    }
    axis = v3_scale(axis, nko_rsqrt(l));
    const float c = cosf(angle), s = sinf(angle), t = 1.0f - c;
    m[0] = t * axis.x * axis.x + c; m[1] = t * axis.x * axis.y - s * axis.z; m[2] = t * axis.x * axis.z + s * axis.y;
    m[3] = t * axis.x * axis.y + s * axis.z; m[4] = t * axis.y * axis.y + c; m[5] = t * axis.y * axis.z - s * axis.x;
    m[6] = t * axis.x * axis.z - s * axis.y; m[7] = t * axis.y * axis.z + s * axis.x; m[8] = t * axis.z * axis.z + c;
}

static void mat3_mul(const float* a, const float* b, float* out) {   /* articulation.cu:71-82 */
    for (uint32_t row = 0u; row < 3u; ++row)
        for (uint32_t col = 0u; col < 3u; ++col)
            out[row * 3u + col] = a[row * 3u] * b[col] + a[row * 3u + 1u] * b[col + 3u] + a[row * 3u + 2u] * b[col + 6u];
}

/* articulation.cu:149-171 MakeMotionTransform: X = [[E,0],[-E skew(t),E]] */
static void make_motion_transform(const float* E, v3 t, float* X) {
    memset(X, 0, 36 * sizeof(float));
    for (uint32_t row = 0u; row < 3u; ++row)
        for (uint32_t col = 0u; col < 3u; ++col) {
            X[row * 6u + col] = E[row * 3u + col];
            X[(row + 3u) * 6u + col + 3u] = E[row * 3u + col];
        }
    const float skew[9] = {0.0f, -t.z, t.y, t.z, 0.0f, -t.x, -t.y, t.x, 0.0f};
    float ll[9];
    mat3_mul(E, skew, ll);
    for (uint32_t row = 0u; row < 3u; ++row)
        for (uint32_t col = 0u; col < 3u; ++col) X[(row + 3u) * 6u + col] = -ll[row * 3u + col];
}

/* articulation.cu:259-277 JointTransform */
void nko_joint_transform(const nko_world* w, uint32_t env, uint32_t link, float X[36]) {
    const nko_template* t = &w->t;
    const uint8_t type = t->joint_type[link];
    const v3 axis = v3_make(t->joint_axis[3u * link], t->joint_axis[3u * link + 1u], t->joint_axis[3u * link + 2u]);
    const xform local = xform_load(t->link_local_pose + 7u * link);
    const v3 offset = v3_make(t->parent_offset[3u * link], t->parent_offset[3u * link + 1u], t->parent_offset[3u * link + 2u]);
    const float q = w->q[(size_t)env * t->nl + link];
    float joint[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
    v3 translation = v3_add(local.p, offset);
    if (type == NKO_REVOLUTE) mat3_axis_angle(axis, q, joint);
    else if (type == NKO_PRISMATIC) translation = joint_relative_frame(type, axis, local, offset, q).p;
    float lr[9], rot[9], E[9];
    mat3_from_quat(local.r, lr);
    mat3_mul(lr, joint, rot);
    for (uint32_t r = 0u; r < 3u; ++r) for (uint32_t c = 0u; c < 3u; ++c) E[r * 3u + c] = rot[c * 3u + r];
    make_motion_transform(E, translation, X);
}

/* articulation.cu:194-211 MotionSubspaceForJoint */
void nko_motion_subspace(uint8_t type, v3 axis, float s[6]) {
    for (uint32_t i = 0u; i < 6u; ++i) s[i] = 0.0f;
    const float l = v3_dot(axis, axis);
    if (l > 1.0e-12f) axis = v3_scale(axis, nko_rsqrt(l));
    if (type == NKO_REVOLUTE) { s[0] = axis.x; s[1] = axis.y; s[2] = axis.z; }
    else if (type == NKO_PRISMATIC) { s[3] = axis.x; s[4] = axis.y; s[5] = axis.z; }
}

/* ---- FK (articulation.cu:1561-1596 UpdateWorldLinkPosesKernel) ---------- */
void nko_env_fk(const nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl;
    float* pose = w->link_pose + (size_t)env * nl * 7u;
    for (uint32_t depth = 0u; depth <= t->max_depth; ++depth)
        for (uint32_t link = 0u; link < nl; ++link) {
            if (t->link_tree_depth[link] != depth) continue;
            const v3 axis = v3_make(t->joint_axis[3u * link], t->joint_axis[3u * link + 1u], t->joint_axis[3u * link + 2u]);
            const v3 offset = v3_make(t->parent_offset[3u * link], t->parent_offset[3u * link + 1u], t->parent_offset[3u * link + 2u]);
            const xform relative = joint_relative_frame(t->joint_type[link], axis, xform_load(t->link_local_pose + 7u * link),
                                                        offset, w->q[(size_t)env * nl + link]);
            const uint32_t parent = t->parent_link[link];
            xform out;
            if (parent == NKO_INVALID)
                out = t->joint_type[link] == NKO_FLOATING ? xform_load(w->base_pose + (size_t)env * 7u) : relative;
            else
                out = nko_compose_frame(xform_load(pose + 7u * parent), relative);
            xform_store(pose + 7u * link, out);
        }
}

/* ---- LDL^T (articulation_mass.cuh:269-335 FactorMass, right-looking) ---- */
void nko_factor_mass(const float* mass, float* factor, uint32_t n, uint32_t stride) {
    float a[NKO_MAX_DOF][NKO_MAX_DOF], work[NKO_MAX_DOF][NKO_MAX_DOF];
    for (uint32_t i = 0u; i < n; ++i)
        for (uint32_t j = 0u; j <= i; ++j) { a[i][j] = mass[(size_t)i * stride + j]; work[i][j] = 0.0f; }
    for (uint32_t k = 0u; k < n; ++k) {
        const float diagonal = fmaxf(a[k][k], 1.0e-6f);
        for (uint32_t i = k + 1u; i < n; ++i) work[i][k] = a[i][k] / diagonal;
        work[k][k] = diagonal;
        for (uint32_t i = k + 1u; i < n; ++i) {
            const float l = work[i][k];
            for (uint32_t j = k + 1u; j <= i; ++j) a[i][j] -= l * work[j][k] * diagonal;
        }
    }
    for (uint32_t i = 0u; i < stride; ++i)
        for (uint32_t j = 0u; j <= i; ++j)
            factor[(size_t)i * stride + j] = i < n ? work[i][j] : (i == j ? 1.0e-6f : 0.0f);
}

/* articulation_mass.cuh:357-396 SolveMassBlock: forward by rows, divide, backward serial */
void nko_solve_mass(const float* factor, float* value, uint32_t n, uint32_t stride) {
    float x[NKO_MAX_DOF];
    for (uint32_t i = 0u; i < n; ++i) x[i] = value[i];
    for (uint32_t j = 0u; j < n; ++j) {
        const float solved = x[j];
        for (uint32_t i = j + 1u; i < n; ++i) x[i] -= factor[(size_t)i * stride + j] * solved;
    }
    for (uint32_t i = 0u; i < n; ++i) value[i] = x[i] / factor[(size_t)i * stride + i];
    for (uint32_t end = n; end > 0u; --end) {
        const uint32_t i = end - 1u;
        float sum = value[i];
        for (uint32_t j = i + 1u; j < n; ++j) sum -= factor[(size_t)j * stride + i] * value[j];
        value[i] = sum;
    }
}

/* articulation_mass.cuh:414-441 ForwardMass + MassDot + MassCoupling<float> */
float nko_mass_coupling(const float* factor, uint32_t n, const float* v, const float* extra) {
    float y[NKO_MAX_DOF];
    for (uint32_t i = 0u; i < n; ++i) {
        float a = v[i] + (extra == NULL ? 0.0f : extra[i]);
        for (uint32_t j = 0u; j < i; ++j) a -= factor[(size_t)i * n + j] * y[j];
        y[i] = a;
    }
    float response = 0.0f;
    for (uint32_t i = 0u; i < n; ++i) response += y[i] * y[i] / factor[(size_t)i * n + i];
    return response;
}

/* ---- dynamics (articulation.cu:309-376, 505-645; articulation_mass.cuh:124-253) ---- */
void nko_env_dynamics(nko_world* w, uint32_t env, uint32_t integrate_velocity) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl, stride = t->max_dof, dof = t->nv;
    const size_t lbase = (size_t)env * nl;
    float* xup = (float*)malloc(sizeof(float) * nl * (36u + 6u + 6u + 6u + 36u));
    float* S = xup + (size_t)nl * 36u;
    float* vbias = S + (size_t)nl * 6u;
    float* pf = vbias + (size_t)nl * 6u;
    float* comp = pf + (size_t)nl * 6u;
    float* lv = w->link_velocity + lbase * 6u;
    float* la = w->link_acceleration + lbase * 6u;
    const float* q = w->q + lbase;
    float* qd = w->qdot + lbase;
    const v3 gravity = v3_make(w->cfg.gravity[0], w->cfg.gravity[1], w->cfg.gravity[2]);
    const quat base_rot = xform_load(w->base_pose + (size_t)env * 7u).r;
    const float dt = w->cfg.fixed_dt;

    /* PrepareArticulationKinematics: joint transforms and subspaces (:318-332) */
    for (uint32_t l = 0u; l < nl; ++l) {
        if (t->parent_link[l] == NKO_INVALID && t->joint_type[l] == NKO_FLOATING) {
            const float id[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
            make_motion_transform(id, v3_make(0.0f, 0.0f, 0.0f), xup + 36u * l);
            for (uint32_t i = 0u; i < 6u; ++i) { S[6u * l + i] = 0.0f; vbias[6u * l + i] = 0.0f; }
            continue;
        }
        nko_joint_transform(w, env, l, xup + 36u * l);
        nko_motion_subspace(t->joint_type[l], v3_make(t->joint_axis[3u * l], t->joint_axis[3u * l + 1u], t->joint_axis[3u * l + 2u]),
                            S + 6u * l);
    }
    /* velocity sweep root to leaf (:334-363); a floating root's twist is state */
    for (uint32_t depth = 0u; depth <= t->max_depth; ++depth)
        for (uint32_t l = 0u; l < nl; ++l) {
            if (t->link_tree_depth[l] != depth) continue;
            const uint32_t parent = t->parent_link[l];
            if (parent == NKO_INVALID && t->joint_type[l] == NKO_FLOATING) continue;
            float vp[6] = {0, 0, 0, 0, 0, 0}, tp[6], jv[6], v[6];
            if (parent != NKO_INVALID) memcpy(vp, lv + 6u * parent, sizeof(vp));
            mat66_mul_vec6(xup + 36u * l, vp, tp);
            for (uint32_t i = 0u; i < 6u; ++i) jv[i] = S[6u * l + i] * qd[l];
            for (uint32_t i = 0u; i < 6u; ++i) v[i] = tp[i] + jv[i];
            memcpy(lv + 6u * l, v, sizeof(v));
            motion_cross(v, jv, vbias + 6u * l);
        }
    /* p = v x* (I v) - external wrench (:364-374, 279-295) */
    for (uint32_t l = 0u; l < nl; ++l) {
        float iv[6];
        mat66_mul_vec6(t->link_inertia + 36u * l, lv + 6u * l, iv);
        force_cross(lv + 6u * l, iv, pf + 6u * l);
        const float* wr = w->link_wrench + (lbase + l) * 6u;
        if (wr[0] != 0.0f || wr[1] != 0.0f || wr[2] != 0.0f || wr[3] != 0.0f || wr[4] != 0.0f || wr[5] != 0.0f) {
            const quat rot = xform_load(w->link_pose + (lbase + l) * 7u).r;
            const v3 force = nko_rotate_inverse(rot, v3_make(wr[0], wr[1], wr[2]));
            const v3 torque = nko_rotate_inverse(rot, v3_make(wr[3], wr[4], wr[5]));
            const v3 com = xform_load(t->link_inertial_frame + 7u * l).p;
            const v3 moment = v3_add(torque, v3_cross(com, force));
            pf[6u * l] -= moment.x; pf[6u * l + 1u] -= moment.y; pf[6u * l + 2u] -= moment.z;
            pf[6u * l + 3u] -= force.x; pf[6u * l + 4u] -= force.y; pf[6u * l + 5u] -= force.z;
        }
    }
    /* bias accelerations with gravity as base acceleration (:526-547) */
    for (uint32_t depth = 0u; depth <= t->max_depth; ++depth)
        for (uint32_t l = 0u; l < nl; ++l) {
            if (t->link_tree_depth[l] != depth) continue;
            float a[6];
            const uint32_t parent = t->parent_link[l];
            if (parent != NKO_INVALID) mat66_mul_vec6(xup + 36u * l, la + 6u * parent, a);
            else if (t->joint_type[l] == NKO_FLOATING) {
                const v3 g = nko_rotate_inverse(base_rot, gravity);
                a[0] = a[1] = a[2] = 0.0f; a[3] = -g.x; a[4] = -g.y; a[5] = -g.z;
            } else {
                const float world[6] = {0.0f, 0.0f, 0.0f, -gravity.x, -gravity.y, -gravity.z};
                mat66_mul_vec6(xup + 36u * l, world, a);
            }
            for (uint32_t i = 0u; i < 6u; ++i) a[i] += vbias[6u * l + i];
            memcpy(la + 6u * l, a, sizeof(a));
        }
    /* p += I a (:548-555; gravity compensation is zero here) */
    for (uint32_t l = 0u; l < nl; ++l) {
        float f[6];
        mat66_mul_vec6(t->link_inertia + 36u * l, la + 6u * l, f);
        for (uint32_t i = 0u; i < 6u; ++i) pf[6u * l + i] += f[i];
        for (uint32_t i = 0u; i < 6u; ++i) pf[6u * l + i] -= 0.0f;
    }
    /* leaf to root in child CSR order (:557-569) */
    for (uint32_t remaining = t->max_depth + 1u; remaining > 0u; --remaining)
        for (uint32_t l = 0u; l < nl; ++l) {
            if (t->link_tree_depth[l] != remaining - 1u) continue;
            for (uint32_t i = t->link_child_range[2u * l]; i < t->link_child_range[2u * l + 1u]; ++i) {
                const uint32_t child = t->link_children[i];
                float f[6];
                transform_force_transpose(xup + 36u * child, pf + 6u * child, f);
                for (uint32_t c = 0u; c < 6u; ++c) pf[6u * l + c] += f[c];
            }
        }
    /* generalized bias and right-hand side (:570-585) */
    float velocity[NKO_MAX_DOF], acceleration[NKO_MAX_DOF];
    float* bias = w->articulation_bias + (size_t)env * stride;
    for (uint32_t d = 0u; d < stride; ++d) {
        if (d >= dof) { bias[d] = 0.0f; continue; }
        const uint32_t link = t->dof_link[d], component = t->dof_component[d];
        const int scalar = component == NKO_INVALID;
        velocity[d] = scalar ? qd[link] : lv[6u * link + component];
        bias[d] = scalar ? dot6(S + 6u * link, pf + 6u * link) : pf[6u * link + component];
        if (scalar) bias[d] += w->joint_gravity_force[lbase + link];
        const int fold = w->fold_drive_damping && t->joint_drive_rows > 0u;   /* pipeline.cpp:380-381, 400 */
        const float damping = scalar ? t->joint_damping[link] + (fold ? w->drive_dissipation[lbase + link] : 0.0f) : 0.0f;
        const float spring = scalar ? t->joint_stiffness[link] * (q[link] - t->joint_spring_reference[link]) : 0.0f;
        acceleration[d] = (scalar ? w->tau[lbase + link] : 0.0f) - bias[d] - damping * velocity[d] - spring;
    }
    /* CRBA (articulation_mass.cuh:124-253) */
    float* M = w->m + (size_t)env * stride * stride;
    for (size_t i = 0u; i < (size_t)stride * stride; ++i) M[i] = 0.0f;
    for (uint32_t l = 0u; l < nl; ++l) memcpy(comp + 36u * l, t->link_inertia + 36u * l, 36u * sizeof(float));
    for (uint32_t depth = t->max_depth; depth > 0u; --depth)
        for (uint32_t l = 0u; l < nl; ++l) {
            if (t->link_tree_depth[l] + 1u != depth) continue;
            for (uint32_t i = t->link_child_range[2u * l]; i < t->link_child_range[2u * l + 1u]; ++i) {
                const uint32_t child = t->link_children[i];
                float delta[36];
                transform_inertia_to_parent(xup + 36u * child, comp + 36u * child, delta);
                for (uint32_t e = 0u; e < 36u; ++e) comp[36u * l + e] += delta[e];
            }
        }
    const int floating_root = nl > 0u && t->parent_link[0] == NKO_INVALID && t->joint_type[0] == NKO_FLOATING;
    if (floating_root && stride >= 6u)
        for (uint32_t e = 0u; e < 36u; ++e) M[(size_t)(e / 6u) * stride + e % 6u] = comp[e];
    for (uint32_t l = 0u; l < nl; ++l) {
        if (nko_joint_dof(t->joint_type[l]) == 0u) continue;
        if (l == 0u && floating_root) continue;
        const uint32_t dof_i = t->link_dof[l];
        if (dof_i >= stride) continue;
        float force[6];
        mat66_mul_vec6(comp + 36u * l, S + 6u * l, force);
        float diagonal = dot6(S + 6u * l, force);
        diagonal += t->joint_armature[l];
        if (w->fold_drive_damping && t->joint_drive_rows > 0u) diagonal += dt * w->drive_dissipation[lbase + l];   /* :206-208 */
        M[(size_t)dof_i * stride + dof_i] = diagonal;
        uint32_t walk = l;
        for (;;) {
            const uint32_t parent = t->parent_link[walk];
            if (parent == NKO_INVALID) break;
            float pushed[6];
            transform_force_transpose(xup + 36u * walk, force, pushed);
            memcpy(force, pushed, sizeof(force));
            walk = parent;
            if (nko_joint_dof(t->joint_type[walk]) == 0u) continue;
            const uint32_t dof_j = t->link_dof[walk];
            if (dof_j >= stride) continue;
            if (walk == 0u && floating_root) {
                for (uint32_t b = 0u; b < 6u && b < stride; ++b) {
                    M[(size_t)dof_i * stride + b] = force[b];
                    M[(size_t)b * stride + dof_i] = force[b];
                }
                continue;
            }
            const float entry = dot6(S + 6u * walk, force);
            M[(size_t)dof_i * stride + dof_j] = entry;
            M[(size_t)dof_j * stride + dof_i] = entry;
        }
    }
    /* factor and solve (:587-596) */
    float* factor = w->m_factor + (size_t)env * stride * stride;
    nko_factor_mass(M, factor, dof, stride);
    nko_solve_mass(factor, acceleration, dof, stride);
    float* qdd_flat = w->articulation_qdd + (size_t)env * stride;
    for (uint32_t d = 0u; d < stride; ++d) qdd_flat[d] = d < dof ? acceleration[d] : 0.0f;
    /* write back (:597-615) */
    for (uint32_t l = 0u; l < nl; ++l) {
        w->qddot[lbase + l] = 0.0f;
        if (integrate_velocity) memset(w->link_wrench + (lbase + l) * 6u, 0, 6u * sizeof(float));
    }
    for (uint32_t d = 0u; d < dof; ++d) {
        const uint32_t link = t->dof_link[d], component = t->dof_component[d];
        if (component == NKO_INVALID) {
            w->qddot[lbase + link] = acceleration[d];
            if (integrate_velocity) qd[link] = velocity[d] + dt * acceleration[d];
        } else if (integrate_velocity) {
            const uint32_t i = component % 3u, j = (i + 1u) % 3u, k = (i + 2u) % 3u;
            const float transport = component < 3u ? 0.0f :
                velocity[d - component + j] * velocity[d - i + k] - velocity[d - component + k] * velocity[d - i + j];
            lv[6u * link + component] = velocity[d] + dt * (acceleration[d] + transport);
        }
    }
    /* final link accelerations (:617-644) */
    for (uint32_t depth = 0u; depth <= t->max_depth; ++depth)
        for (uint32_t l = 0u; l < nl; ++l) {
            if (t->link_tree_depth[l] != depth) continue;
            float a[6];
            const uint32_t parent = t->parent_link[l];
            if (t->joint_type[l] == NKO_FLOATING) {
                const v3 g = nko_rotate_inverse(base_rot, gravity);
                for (uint32_t c = 0u; c < 6u; ++c) a[c] = acceleration[c];
                a[3] -= g.x; a[4] -= g.y; a[5] -= g.z;
            } else {
                if (parent != NKO_INVALID) mat66_mul_vec6(xup + 36u * l, la + 6u * parent, a);
                else {
                    const float world[6] = {0.0f, 0.0f, 0.0f, -gravity.x, -gravity.y, -gravity.z};
                    mat66_mul_vec6(xup + 36u * l, world, a);
                }
                for (uint32_t c = 0u; c < 6u; ++c) a[c] += vbias[6u * l + c] + S[6u * l + c] * w->qddot[lbase + l];
            }
            memcpy(la + 6u * l, a, sizeof(a));
        }
    free(xup);
}

/* ---- IntegratePosition (articulation.cu:732-791) ------------------------ */
void nko_env_integrate_position(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl;
    const size_t lbase = (size_t)env * nl;
    const float dt = w->cfg.fixed_dt;
    const int pos_pass = w->cfg.solver_pos_iters > 0u && t->rows_per_env > 0u;
    for (uint32_t l = 0u; l < nl; ++l) {
        if (pos_pass) w->q[lbase + l] += (w->qdot[lbase + l] + w->qdot_pseudo[lbase + l]) * dt;
        else w->q[lbase + l] += w->qdot[lbase + l] * dt;
        if (t->parent_link[l] == NKO_INVALID && t->joint_type[l] == NKO_FLOATING) {
            float* rv = w->link_velocity + (lbase + l) * 6u;
            xform pose = xform_load(w->base_pose + (size_t)env * 7u);
            float v[6];
            for (uint32_t i = 0u; i < 6u; ++i) v[i] = pos_pass ? rv[i] + w->link_velocity_pseudo[(lbase + l) * 6u + i] : rv[i];
            const v3 lin_world = nko_rotate_forward(pose.r, v3_make(v[3], v[4], v[5]));
            pose.p = v3_add(pose.p, v3_scale(lin_world, dt));
            const quat dq = quat_make(1.0f, 0.5f * v[0] * dt, 0.5f * v[1] * dt, 0.5f * v[2] * dt);
            pose.r = quat_normalize_forward(nko_quat_mul(pose.r, dq), 1.0e-24f);
            const v3 turned = nko_rotate_inverse(quat_normalize_forward(dq, 1.0e-24f), v3_make(rv[3], rv[4], rv[5]));
            rv[3] = turned.x; rv[4] = turned.y; rv[5] = turned.z;
            xform_store(w->base_pose + (size_t)env * 7u, pose);
        }
    }
}

/* ---- FkLinkVelocities (articulation.cu:647-689) -------------------------- */
void nko_env_link_velocities(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl;
    const size_t lbase = (size_t)env * nl;
    float* lv = w->link_velocity + lbase * 6u;
    for (uint32_t depth = 0u; depth <= t->max_depth; ++depth)
        for (uint32_t l = 0u; l < nl; ++l) {
            if (t->link_tree_depth[l] != depth) continue;
            const uint32_t parent = t->parent_link[l];
            if (parent == NKO_INVALID && t->joint_type[l] == NKO_FLOATING) continue;
            float pv[6] = {0, 0, 0, 0, 0, 0}, X[36], s[6], v[6];
            if (parent != NKO_INVALID) memcpy(pv, lv + 6u * parent, sizeof(pv));
            nko_joint_transform(w, env, l, X);
            nko_motion_subspace(t->joint_type[l], v3_make(t->joint_axis[3u * l], t->joint_axis[3u * l + 1u], t->joint_axis[3u * l + 2u]), s);
            mat66_mul_vec6(X, pv, v);
            for (uint32_t c = 0u; c < 6u; ++c) v[c] += s[c] * w->qdot[lbase + l];
            memcpy(lv + 6u * l, v, sizeof(v));
        }
}

/* ---- ApplyDrives (articulation.cu:836-940 ApplyAffineDriveKernel) --------
 * Controllers hand the row solver an affine effort `command - dissipation * qdot` and its bounds; the dissipation
 * is folded into the articulation mass and bias when the velocity feedback is solved implicitly.  Gravity
 * compensation (ProjectGravityCompensationKernel :393-423) is not authored on this path: joint_gravity_force
 * stays as uploaded (zero by default).  The inverse-dynamics modes (ComputedTorque, Osc) are not built. */
void nko_env_apply_drives(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl, mode = t->drive_mode;
    const size_t lbase = (size_t)env * nl;
    const int implicit = w->fold_drive_damping;
    const float dt = w->cfg.fixed_dt;
    for (uint32_t l = 0u; l < nl; ++l) {
        const size_t link = lbase + l;
        w->drive_command[link] = w->drive_dissipation[link] = 0.0f;
        w->drive_lower[link] = w->drive_upper[link] = 0.0f;
        w->tau[link] = 0.0f;
        if (nko_joint_dof(t->joint_type[l]) != 1u) continue;
        const int position_control = mode == NKO_DRIVE_PD_POSITION;
        const int velocity_control = mode == NKO_DRIVE_VELOCITY;
        const float kp = w->drive_stiffness[link], kd = w->drive_damping[link];
        if ((position_control && (!isfinite(w->drive_target[link]) || !isfinite(kp) || kp < 0.0f || !isfinite(kd) ||
                                  (implicit && kd < 0.0f))) ||
            ((position_control || velocity_control) && !isfinite(w->velocity_target[link])) ||
            (velocity_control && (!isfinite(kp) || kp < 0.0f)) ||
            (mode == NKO_DRIVE_ACTUATOR && !isfinite(w->actuator_noload_speed[link]))) {
            w->env_status[env] |= NKO_STATUS_CONTROL_FAILURE;
            continue;
        }
        const float velocity = w->qdot[link];
        const float limit = w->drive_force_limit[link];
        float lower = limit > 0.0f ? -limit : -FLT_MAX;
        float upper = limit > 0.0f ? limit : FLT_MAX;
        float bias = 0.0f, damping = 0.0f;
        switch (mode) {
            case NKO_DRIVE_PD_POSITION:
                damping = kd + (implicit ? dt * kp : 0.0f);
                bias = kp * (w->drive_target[link] - w->q[link]) + damping * w->velocity_target[link];
                break;
            case NKO_DRIVE_VELOCITY:
                damping = kp;
                bias = damping * w->velocity_target[link];
                break;
            case NKO_DRIVE_TORQUE:
            case NKO_DRIVE_ACTUATOR:
                bias = w->drive_target[link];
                if (mode == NKO_DRIVE_ACTUATOR && limit > 0.0f && w->actuator_noload_speed[link] > 0.0f) {
                    const float speed_bias = limit * velocity / w->actuator_noload_speed[link];
                    lower = fminf(fmaxf(-limit - speed_bias, -limit), limit);
                    upper = fminf(fmaxf(limit - speed_bias, -limit), limit);
                }
                break;
            default: break;
        }
        const float effort = bias - damping * velocity;
        const float gravity_force = w->joint_gravity_force[link];
        const int saturated = effort < lower || effort > upper;
        const float joint_limit = w->drive_joint_force_limit[link];
        if (implicit && joint_limit > 0.0f) {
            bias = fminf(fmaxf(fminf(fmaxf(effort, lower), upper) + gravity_force, -joint_limit), joint_limit);
            damping = saturated ? 0.0f : damping;
            bias += damping * velocity;
            lower = -FLT_MAX;
            upper = FLT_MAX;
        } else if (!implicit || saturated) {
            bias = effort + gravity_force;
            damping = 0.0f;
            lower += gravity_force;
            upper += gravity_force;
            if (joint_limit > 0.0f) {
                lower = fminf(fmaxf(lower, -joint_limit), joint_limit);
                upper = fminf(fmaxf(upper, -joint_limit), joint_limit);
            }
        } else {
            bias += gravity_force;
            lower += gravity_force + damping * velocity;
            upper += gravity_force + damping * velocity;
        }
        const float feedforward = w->joint_f[link];
        if (!isfinite(bias) || !isfinite(damping) || damping < 0.0f || !isfinite(limit) || !isfinite(feedforward) ||
            !isfinite(velocity) || !isfinite(w->q[link])) {
            w->env_status[env] |= NKO_STATUS_CONTROL_FAILURE;
            continue;
        }
        w->drive_command[link] = bias;
        w->drive_dissipation[link] = damping;
        w->drive_lower[link] = lower;
        w->drive_upper[link] = upper;
        w->tau[link] = feedforward;
    }
}

/* ---- ReadoutDrives (articulation.cu:999-1016) ---------------------------- */
void nko_env_readout_drives(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl, R = t->rows_per_env;
    const uint32_t first_drive_row = t->contact_rows_per_env + t->joint_limit_rows + t->joint_friction_rows;
    const float dt = w->cfg.fixed_dt;
    for (uint32_t l = 0u; l < nl; ++l) {
        const size_t link = (size_t)env * nl + l;
        w->actuator_effort_requested[link] = w->actuator_effort[link] = w->actuator_saturated[link] = 0.0f;
        if (nko_joint_dof(t->joint_type[l]) != 1u) continue;
        const size_t row = (size_t)env * R + first_drive_row + l;
        const float effort = w->drive_command[link] - w->drive_dissipation[link] * w->qdot[link];
        w->actuator_effort_requested[link] = effort;
        w->actuator_effort[link] = w->lambda[row] / dt - w->drive_dissipation[link] * w->qdot[link];
        w->actuator_saturated[link] =
            w->drive_command[link] < w->drive_lower[link] || w->drive_command[link] > w->drive_upper[link] ? 1.0f : 0.0f;
        w->tau[link] += w->actuator_effort[link];
    }
}

/* ArticulationReferenceWeightsKernel and BodyReferenceWeightsKernel (articulation.cu:425-500): the mass matrix at the
 * current pose (armature included, no damping folded in), its factor, the diagonal of its inverse, and for every link
 * the mean translational and rotational response of its centre of mass to a unit force and a unit moment. */
void nko_env_reference_weights(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl, nb = t->nb, md = t->max_dof, dof = t->nv;
    float* weights = w->body_invweight0 + (size_t)env * nb * 2u;
    for (uint32_t b = 0u; b < nb; ++b) weights[2u * b] = weights[2u * b + 1u] = 0.0f;   /* static rows: inverse mass zero */
    if (t->free_body) {   /* BodyReferenceWeightsKernel (articulation.cu:425-432): the inverse mass, the mean inverse principal moment */
        const uint32_t body = t->link_body[0];
        const float* d = t->body_diag_inertia;
        const float inverse[3] = {d[0] > 0.0f ? 1.0f / d[0] : 0.0f, d[1] > 0.0f ? 1.0f / d[1] : 0.0f, d[2] > 0.0f ? 1.0f / d[2] : 0.0f};
        weights[2u * body] = t->body_mass > 0.0f ? 1.0f / t->body_mass : 0.0f;
        weights[2u * body + 1u] = (inverse[0] + inverse[1] + inverse[2]) / 3.0f;
        return;
    }
    if (dof == 0u) return;
    nko_env_dynamics(w, env, 0u);   /* m, m_factor at the current pose; the caller has switched the damping fold off */
    const float* factor = w->m_factor + (size_t)env * md * md;
    float* diagonal = w->dof_invweight0 + (size_t)env * md;
    float row[NKO_MAX_DOF], solution[NKO_MAX_DOF];
    for (uint32_t d = 0u; d < dof; ++d) {
        for (uint32_t i = 0u; i < dof; ++i) solution[i] = i == d ? 1.0f : 0.0f;
        nko_solve_mass(factor, solution, dof, md);
        diagonal[d] = solution[d];
    }
    if (t->joint_type[0] == NKO_FLOATING) {
        const float rotation = (diagonal[0] + diagonal[1] + diagonal[2]) / 3.0f;
        const float translation = (diagonal[3] + diagonal[4] + diagonal[5]) / 3.0f;
        for (uint32_t i = 0u; i < 3u; ++i) { diagonal[i] = rotation; diagonal[i + 3u] = translation; }
    }
    for (uint32_t link = 0u; link < nl; ++link) {
        const xform pose = xform_load(w->link_pose + ((size_t)env * nl + link) * 7u);
        const v3 com = v3_make(t->link_inertial_frame[7u * link], t->link_inertial_frame[7u * link + 1u], t->link_inertial_frame[7u * link + 2u]);
        const v3 point = v3_add(pose.p, nko_rotate_normalized(pose.r, com));
        float weight[2] = {0.0f, 0.0f};
        for (uint32_t axis = 0u; axis < 6u; ++axis) {
            for (uint32_t d = 0u; d < dof; ++d) row[d] = 0.0f;
            const v3 unit = v3_make(axis % 3u == 0u ? 1.0f : 0.0f, axis % 3u == 1u ? 1.0f : 0.0f, axis % 3u == 2u ? 1.0f : 0.0f);
            const v3 none = v3_make(0.0f, 0.0f, 0.0f);
            uint32_t walk = link;
            while (walk != NKO_INVALID) {
                if (nko_joint_dof(t->joint_type[walk]) != 0u)
                    nko_accumulate_chain(w, env, walk, t->link_dof[walk], point, axis < 3u ? unit : none, axis < 3u ? none : unit, row);
                walk = t->parent_link[walk];
            }
            for (uint32_t d = 0u; d < dof; ++d) solution[d] = row[d];
            nko_solve_mass(factor, solution, dof, md);
            for (uint32_t d = 0u; d < dof; ++d) weight[axis / 3u] += row[d] * solution[d];
        }
        const uint32_t body = t->link_body[link];
        if (body < nb) { weights[2u * body] = weight[0] / 3.0f; weights[2u * body + 1u] = weight[1] / 3.0f; }
    }
}

/* ActuatorVelocityDerivative (articulation.cu:942-948): what a servo's effort changes per unit joint velocity, none while
 * its own force limit clamps it */
static float actuator_velocity_derivative(const nko_world* w, size_t link) {
    if (w->drive_force_limit[link] > 0.0f && fabsf(w->drive_command[link] - w->joint_gravity_force[link]) > w->drive_force_limit[link]) return 0.0f;
    return w->t.drive_mode == NKO_DRIVE_PD_POSITION ? w->drive_damping[link] : w->t.drive_mode == NKO_DRIVE_VELOCITY ? w->drive_stiffness[link] : 0.0f;
}

/* ArticulationDampingKernel (articulation.cu:950-1000): contacts are solved with the plain mass; afterwards the step's
 * velocity change goes through (M + dt D)^-1 M, D the joint damping and, for the implicit integrators, the unclamped
 * servo velocity gains. */
void nko_env_articulation_damping(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t nl = t->nl, stride = t->max_dof, dof = t->nv;
    const size_t lbase = (size_t)env * nl, base = (size_t)env * stride;
    const float dt = w->cfg.fixed_dt;
    const int actuator_derivative = t->integrator == 2u, readout_drives = t->joint_drive_rows > 0u;
    float change[NKO_MAX_DOF], damping[NKO_MAX_DOF];
    int damped = 0;
    for (uint32_t d = 0u; d < dof; ++d) {
        const uint32_t link = t->dof_link[d], component = t->dof_component[d];
        const int scalar = component == NKO_INVALID;
        float value = scalar ? t->joint_damping[link] : 0.0f;
        if (scalar && actuator_derivative) value += actuator_velocity_derivative(w, lbase + link);
        const float velocity = scalar ? w->qdot[lbase + link] : w->link_velocity[(lbase + link) * 6u + component];
        damping[d] = dt * value;
        change[d] = damping[d] * (velocity - w->step_qdot_flat[base + d]);
        damped |= value != 0.0f;
    }
    if (!damped) return;
    float* mass = (float*)malloc(sizeof(float) * (size_t)stride * stride * 2u);
    float* factor = mass + (size_t)stride * stride;
    memcpy(mass, w->m + base * stride, sizeof(float) * (size_t)stride * stride);
    for (uint32_t d = 0u; d < dof; ++d) mass[(size_t)d * stride + d] = mass[(size_t)d * stride + d] + damping[d];   /* FactorMass: `add` joins the diagonal */
    nko_factor_mass(mass, factor, dof, stride);
    nko_solve_mass(factor, change, dof, stride);
    for (uint32_t d = 0u; d < dof; ++d) {
        const uint32_t link = t->dof_link[d], component = t->dof_component[d];
        float* velocity = component == NKO_INVALID ? &w->qdot[lbase + link] : &w->link_velocity[(lbase + link) * 6u + component];
        *velocity -= change[d];
        w->qdot_flat[base + d] = *velocity;
        if (component == NKO_INVALID && actuator_derivative && readout_drives) {
            const float derivative = actuator_velocity_derivative(w, lbase + link);
            const float correction = derivative * (*velocity - w->step_qdot_flat[base + d]);
            w->actuator_effort_requested[lbase + link] -= correction;
            w->actuator_effort[lbase + link] -= correction;
            w->tau[lbase + link] -= correction;
        }
    }
    free(mass);
}
