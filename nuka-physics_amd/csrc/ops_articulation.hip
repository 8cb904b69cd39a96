// Articulation ops for gfx950: forward kinematics, forward dynamics (RNEA bias + CRBA + LDL^T solve), position
// integration and link twists.  One 64-lane wavefront owns one environment (the forward dynamics runs two, its bias
// forces and its mass matrix side by side): lanes are links in the tree sweeps, matrix entries in the 6x6 inertia
// pushes, and matrix rows in the factorisation; every per-link quantity of the environment lives in LDS between the
// sweeps and reaches HBM once, in contiguous env-major blocks.
//
// Replaces src/phi/backend_cuda/ops/articulation.cu (UpdateWorldLinkPosesKernel :1561-1596,
// ArticulationDynamicsKernel :505-645, IntegratePositionArticulationKernel :764-791, FkLinkVelocitiesKernel
// :647-689) and articulation_mass.cuh (ComputeArticulationMass :124-253, FactorMass :269-335,
// SolveMassBlock :357-396).
#include "nk_device_math.h"
#include "nk_body_pose.h"
#include "backend.h"
#include "nk_ops.h"

namespace nkh {

namespace {

constexpr int kWave = 64;

// Orders one wavefront's LDS writes before its later reads: its lanes run in step and the LDS takes a wavefront's
// accesses in order, so only the compiler could move them - a fence of wavefront scope holds it without a wait
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ V3 load3(const float* p) { return V3{p[0], p[1], p[2]}; }

// kinematics.cuh:25-42 JointRelativeFrame (revolute / prismatic / fixed)
__device__ Xf joint_relative_frame(uint8_t type, V3 axis, Xf local, V3 parent_offset, float coordinate) {
    Xf result = local;
    result.p = add3(local.p, parent_offset);
    const float l = dot3(axis, axis);
    axis = l > 1.0e-12f ? scale3(axis, rsqrt_exact(l)) : V3{0.0f, 0.0f, 0.0f};
    if (type == kRevolute) {
        const float half = 0.5f * coordinate;
        const float sine = sinf(half);
        const Q4 turn{cosf(half), axis.x * sine, axis.y * sine, axis.z * sine};
        result.r = qnormalize_le(qmul(local.r, turn), 1.0e-12f);
    } else if (type == kPrismatic) {
        result.p = add3(result.p, rotate_normalized(local.r, scale3(axis, coordinate)));
    }
    return result;
}

// articulation.cu:91-124
__device__ void mat3_from_quat(Q4 q, float* m) {
    const float n = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (n <= 1.0e-12f) {
        m[0] = 1; m[1] = 0; m[2] = 0; m[3] = 0; m[4] = 1; m[5] = 0; m[6] = 0; m[7] = 0; m[8] = 1;
        return;
    }
    const float inv = rsqrt_exact(n);
    q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    const float xx = q.x * q.x, yy = q.y * q.y, zz = q.z * q.z, xy = q.x * q.y, xz = q.x * q.z, yz = q.y * q.z;
    const float wx = q.w * q.x, wy = q.w * q.y, wz = q.w * q.z;
    m[0] = 1.0f - 2.0f * (yy + zz); m[1] = 2.0f * (xy - wz); m[2] = 2.0f * (xz + wy);
    m[3] = 2.0f * (xy + wz); m[4] = 1.0f - 2.0f * (xx + zz); m[5] = 2.0f * (yz - wx);
    m[6] = 2.0f * (xz - wy); m[7] = 2.0f * (yz + wx); m[8] = 1.0f - 2.0f * (xx + yy);
}

// articulation.cu:126-147
__device__ void mat3_axis_angle(V3 axis, float angle, float* m) {
    const float l = dot3(axis, axis);
    if (l <= 1.0e-12f) {
        m[0] = 1; m[1] = 0; m[2] = 0; m[3] = 0; m[4] = 1; m[5] = 0; m[6] = 0; m[7] = 0; m[8] = 1;
        return;
    }
    axis = scale3(axis, rsqrt_exact(l));
    const float c = cosf(angle), s = sinf(angle), t = 1.0f - c;
    m[0] = t * axis.x * axis.x + c; m[1] = t * axis.x * axis.y - s * axis.z; m[2] = t * axis.x * axis.z + s * axis.y;
    m[3] = t * axis.x * axis.y + s * axis.z; m[4] = t * axis.y * axis.y + c; m[5] = t * axis.y * axis.z - s * axis.x;
    m[6] = t * axis.x * axis.z - s * axis.y; m[7] = t * axis.y * axis.z + s * axis.x; m[8] = t * axis.z * axis.z + c;
}

__device__ void mat3_mul(const float* a, const float* b, float* out) {
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 3; ++c) out[r * 3 + c] = a[r * 3] * b[c] + a[r * 3 + 1] * b[c + 3] + a[r * 3 + 2] * b[c + 6];
}

// articulation.cu:149-171: X = [[E, 0], [-E skew(t), E]] written to a 36-float LDS tile
__device__ void store_motion_transform(const float* E, V3 t, float* X) {
    const float skew[9] = {0.0f, -t.z, t.y, t.z, 0.0f, -t.x, -t.y, t.x, 0.0f};
    float ll[9];
    mat3_mul(E, skew, ll);
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 3; ++c) {
            X[r * 6 + c] = E[r * 3 + c];
            X[r * 6 + c + 3] = 0.0f;
            X[(r + 3) * 6 + c] = -ll[r * 3 + c];
            X[(r + 3) * 6 + c + 3] = E[r * 3 + c];
        }
}

// articulation.cu:259-277 JointTransform
__device__ void joint_transform(const ModelView& m, uint32_t link, float q, float* X) {
    const uint8_t type = m.joint_type[link];
    const V3 axis = load3(m.joint_axis + 3u * link);
    const Xf local = load_xf(m.link_local_pose + 7u * link);
    const V3 offset = load3(m.parent_offset + 3u * link);
    float joint[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
    V3 translation = add3(local.p, offset);
    if (type == kRevolute) mat3_axis_angle(axis, q, joint);
    else if (type == kPrismatic) translation = joint_relative_frame(type, axis, local, offset, q).p;
    float lr[9], rot[9], E[9];
    mat3_from_quat(local.r, lr);
    mat3_mul(lr, joint, rot);
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 3; ++c) E[r * 3 + c] = rot[c * 3 + r];
    store_motion_transform(E, translation, X);
}

// articulation.cu:194-211
__device__ void motion_subspace(uint8_t type, V3 axis, float* s) {
#pragma unroll
    for (int i = 0; i < 6; ++i) s[i] = 0.0f;
    const float l = dot3(axis, axis);
    if (l > 1.0e-12f) axis = scale3(axis, rsqrt_exact(l));
    if (type == kRevolute) { s[0] = axis.x; s[1] = axis.y; s[2] = axis.z; }
    else if (type == kPrismatic) { s[3] = axis.x; s[4] = axis.y; s[5] = axis.z; }
}

// ---- FkWorldPoses ---------------------------------------------------------------------------------------
// One wavefront, one environment; `pose` holds nl * 7 words of LDS
__device__ __forceinline__ void world_poses_of_env(const ModelView& m, const DataView& d, uint32_t env, uint32_t lane, float* pose) {
    const uint32_t nl = m.links_per_env;
    const float* q = d.q + size_t{env} * nl;
    // A link's frame in its parent does not wait on the tree: every lane computes its own link's before the sweep, which
    // then only composes a depth at a time (links past the 64th compute theirs when their depth comes).
    struct Placed { uint32_t depth, parent; Xf frame; };
    auto place = [&](uint32_t l) {
        const uint8_t type = m.joint_type[l];
        const uint32_t parent = m.parent_link[l];
        const Xf relative = joint_relative_frame(type, load3(m.joint_axis + 3u * l), load_xf(m.link_local_pose + 7u * l),
                                                 load3(m.parent_offset + 3u * l), q[l]);
        return Placed{m.link_tree_depth[l], parent, parent == kInvalid && type == kFloatingBase ? load_xf(d.base_pose + size_t{env} * 7u) : relative};
    };
    auto compose = [&](uint32_t l, const Placed& t) {
        store_xf(pose + 7u * l, t.parent == kInvalid ? t.frame : compose_frame(load_xf(pose + 7u * t.parent), t.frame));
    };
    Placed own{kInvalid, kInvalid, Xf{}};
    if (lane < nl) own = place(lane);
    for (uint32_t depth = 0u; depth <= m.max_depth; ++depth) {
        if (own.depth == depth) compose(lane, own);
        for (uint32_t l = lane + kWave; l < nl; l += kWave) {
            const Placed t = place(l);
            if (t.depth == depth) compose(l, t);
        }
        wave_sync();
    }
    float* out = d.link_pose + size_t{env} * nl * 7u;
    for (uint32_t e = lane; e < nl * 7u; e += kWave) out[e] = pose[e];
}
__global__ void __launch_bounds__(kWave) FkWorldPosesKernel(ModelView m, DataView d, uint32_t env_count) {
    extern __shared__ float lds[];
    if (blockIdx.x >= env_count) return;
    world_poses_of_env(m, d, blockIdx.x, threadIdx.x, lds);
}

// ---- ArticulationDynamics -------------------------------------------------------------------------------
// Two wavefronts an environment.  The bias forces (velocities, bias accelerations, the leaf-to-root force pass) and the
// mass matrix with its factor (composite inertias, columns, LDL^T) do not depend on each other, and each is a chain of
// tree sweeps that keeps a few lanes busy: the first wavefront takes the one, the second the other, side by side, and
// they meet before the solve.  Each keeps to its own words of LDS in between.
__host__ __device__ inline uint32_t DynamicsLdsFloats(uint32_t nl, uint32_t n, uint32_t sweep_passes) {
    return nl * (36u + 36u + 5u * 6u) + n * (n + 1u) + 2u * n + 64u + nl * 7u + sweep_passes * kSweepLinks;
}

// Compiled per padded DoF width N (a multiple of 4): the LDL^T factorisation and the solve keep one matrix row per
// lane in registers, fully unrolled, and pass pivots and multipliers between lanes as scalar lane reads.
// The tree sweeps run six lanes a link - a lane a row of the link's 6x6 products - and ten links a pass, a depth at a
// time from the cooked pass list (ModelView::sweep_links): a pass costs about a third of the instructions of a lane a
// link carrying all six rows, and each row sums in the order the whole product does.
template <int N>
__global__ void __launch_bounds__(2 * kWave) ArticulationDynamicsKernel(ModelView m, DataView d, ArticulationDynamicsParams p,
                                                                       uint32_t env_count) {
    extern __shared__ float lds[];
    const uint32_t env = blockIdx.x, lane = threadIdx.x % kWave, nl = m.links_per_env, n = m.dof, stride = m.max_dof;
    const bool forces = threadIdx.x < uint32_t(kWave);   // the first wavefront: bias forces; the second: mass matrix, factor, solve
    if (env >= env_count) return;
    float* xup = lds;
    float* S = xup + nl * 36u;
    float* vb = S + nl * 6u;
    float* v = vb + nl * 6u;
    float* ic = v + nl * 6u;          // composite inertias (second wavefront)
    float* a = ic + nl * 36u;         // link accelerations: bias pass (first wavefront), and again the final pass (second)
    float* pf = a + nl * 6u;          // bias forces (first wavefront)
    float* A = pf + nl * 6u;          // n x (n + 1): mass matrix, then its factor (second wavefront)
    float* vel = A + n * (n + 1u);
    float* acc = vel + n;
    float* tmp = acc + n;             // 36 floats of the inertia push, padded to 64
    // the tree as the sweeps read it, a word a link each: parent, joint type, first coordinate, child range, children, rate
    uint32_t* t_parent = reinterpret_cast<uint32_t*>(tmp + 64u);
    uint32_t* t_type = t_parent + nl;
    uint32_t* t_dof = t_type + nl;
    uint32_t* t_child_begin = t_dof + nl;
    uint32_t* t_child_end = t_child_begin + nl;
    uint32_t* t_children = t_child_end + nl;
    float* t_rate = reinterpret_cast<float*>(t_children + nl);
    uint32_t* sweep = reinterpret_cast<uint32_t*>(t_rate + nl);   // sweep_passes x kSweepLinks links, kInvalid where a pass ends early
    const uint32_t passes = m.sweep_passes;
    const uint32_t ld = n + 1u;
    const size_t lbase = size_t{env} * nl;
    const float* q = d.q + lbase;
    float* qd = d.qdot + lbase;
    const V3 gravity{p.gravity[0], p.gravity[1], p.gravity[2]};
    const Q4 base_rot = load_xf(d.base_pose + size_t{env} * 7u).r;
    const uint32_t slot = lane / 6u, srow = lane - 6u * slot;   // of the sweeps: lanes 60..63 sit them out
    const uint32_t ri = srow % 3u, rj = (ri + 1u) % 3u, rk = (ri + 2u) % 3u;
    auto link_of_pass = [&](uint32_t pass) { return lane < 6u * kSweepLinks ? sweep[pass * kSweepLinks + slot] : kInvalid; };
    const V3 gravity_in_base = rotate_inverse(base_rot, gravity);
    const float gravity_in_base_row = srow < 3u ? 0.0f : (srow == 3u ? gravity_in_base.x : srow == 4u ? gravity_in_base.y : gravity_in_base.z);

    if (!forces) {   // what the mass matrix starts from and the sweeps' tables, while the first wavefront builds the joint transforms
        for (uint32_t e = lane; e < nl * 36u; e += kWave) ic[e] = m.link_inertia[e];
        for (uint32_t e = lane; e < n * ld; e += kWave) A[e] = 0.0f;
        for (uint32_t l = lane; l < nl; l += kWave) {
            t_parent[l] = m.parent_link[l]; t_type[l] = m.joint_type[l]; t_dof[l] = m.link_dof[l];
            t_child_begin[l] = m.link_child_range[2u * l]; t_child_end[l] = m.link_child_range[2u * l + 1u];
            t_children[l] = m.link_children[l]; t_rate[l] = qd[l];
        }
        for (uint32_t e = lane; e < passes * kSweepLinks; e += kWave) sweep[e] = m.sweep_links[e];
    }
    // link twists of the state enter LDS (a floating root's twist is state; the rest is rebuilt)
    for (uint32_t e = lane; forces && e < nl * 6u; e += kWave) v[e] = d.link_velocity[lbase * 6u + e];
    // joint transforms and motion subspaces (articulation.cu:318-332)
    for (uint32_t l = lane; forces && l < nl; l += kWave) {
        if (m.parent_link[l] == kInvalid && m.joint_type[l] == kFloatingBase) {
            const float id[9] = {1, 0, 0, 0, 1, 0, 0, 0, 1};
            store_motion_transform(id, V3{0.0f, 0.0f, 0.0f}, xup + 36u * l);
#pragma unroll
            for (int i = 0; i < 6; ++i) { S[6u * l + i] = 0.0f; vb[6u * l + i] = 0.0f; }
            continue;
        }
        joint_transform(m, l, q[l], xup + 36u * l);
        motion_subspace(m.joint_type[l], load3(m.joint_axis + 3u * l), S + 6u * l);
    }
    __syncthreads();
    const bool floating_root = m.floating_root != 0u;
    float row[N];   // the second wavefront's row of the mass matrix, then of its factor
    if (forces) {
        // velocities root to leaf (:334-363)
        for (uint32_t pass = 0u; pass < passes; ++pass) {
            const uint32_t l = link_of_pass(pass);
            const bool moves = l != kInvalid && !(t_parent[l] == kInvalid && t_type[l] == kFloatingBase);   // a floating root's twist is state
            if (moves) {
                const uint32_t parent = t_parent[l];
                const float* X = xup + 36u * l + 6u * srow;
                float through = 0.0f;
#pragma unroll
                for (int c = 0; c < 6; ++c) through += X[c] * (parent != kInvalid ? v[6u * parent + c] : 0.0f);
                v[6u * l + srow] = through + S[6u * l + srow] * t_rate[l];
            }
            wave_sync();
            if (moves) {   // the link's twist crossed with its joint's own twist, row by row (motion_cross)
                const float* vl = v + 6u * l, *s6 = S + 6u * l;
                const float rate = t_rate[l];
                const float first = vl[rj] * (s6[(srow < 3u ? 0u : 3u) + rk] * rate) - vl[rk] * (s6[(srow < 3u ? 0u : 3u) + rj] * rate);
                const float second = vl[3u + rj] * (s6[rk] * rate) - vl[3u + rk] * (s6[rj] * rate);
                vb[6u * l + srow] = srow < 3u ? first : first + second;
            }
        }
        wave_sync();
        // p = v x* (I v) - external wrench (:364-374, 279-295)
        for (uint32_t l = lane; l < nl; l += kWave) {
            float vl[6], iv[6], bf[6];
#pragma unroll
            for (int i = 0; i < 6; ++i) vl[i] = v[6u * l + i];
            mat66_vec(m.link_inertia + 36u * l, vl, iv);
            force_cross(vl, iv, bf);
            if (p.apply_link_wrench != 0u) {
                const float* wr = d.link_wrench + (lbase + l) * 6u;
                if (wr[0] != 0.0f || wr[1] != 0.0f || wr[2] != 0.0f || wr[3] != 0.0f || wr[4] != 0.0f || wr[5] != 0.0f) {
                    const Q4 rot = load_xf(d.link_pose + (lbase + l) * 7u).r;
                    const V3 force = rotate_inverse(rot, V3{wr[0], wr[1], wr[2]});
                    const V3 torque = rotate_inverse(rot, V3{wr[3], wr[4], wr[5]});
                    const V3 moment = add3(torque, cross3(load_xf(m.link_inertial_frame + 7u * l).p, force));
                    bf[0] -= moment.x; bf[1] -= moment.y; bf[2] -= moment.z; bf[3] -= force.x; bf[4] -= force.y; bf[5] -= force.z;
                }
            }
#pragma unroll
            for (int i = 0; i < 6; ++i) pf[6u * l + i] = bf[i];
        }
        wave_sync();
        // bias accelerations with gravity as base acceleration (:526-547)
        for (uint32_t pass = 0u; pass < passes; ++pass) {
            const uint32_t l = link_of_pass(pass);
            if (l != kInvalid) {
                const uint32_t parent = t_parent[l];
                float al;
                if (parent == kInvalid && t_type[l] == kFloatingBase) al = srow < 3u ? 0.0f : -gravity_in_base_row;
                else {
                    const float* X = xup + 36u * l + 6u * srow;
                    al = 0.0f;
#pragma unroll
                    for (int c = 0; c < 6; ++c) al += X[c] * (parent != kInvalid ? a[6u * parent + c] : (c < 3 ? 0.0f : (c == 3 ? -gravity.x : c == 4 ? -gravity.y : -gravity.z)));
                }
                a[6u * l + srow] = al + vb[6u * l + srow];
            }
            wave_sync();
        }
        // p += I a (:548-555)
        for (uint32_t l = lane; l < nl; l += kWave) {
            float al[6], f[6];
#pragma unroll
            for (int i = 0; i < 6; ++i) al[i] = a[6u * l + i];
            mat66_vec(m.link_inertia + 36u * l, al, f);
#pragma unroll
            for (int i = 0; i < 6; ++i) pf[6u * l + i] += f[i];
        }
        wave_sync();
        // leaf to root, children in CSR order (:557-569): the passes backwards, a lane a row of every child's X^T p
        for (uint32_t pass = passes; pass-- > 0u;) {
            const uint32_t l = link_of_pass(pass);
            if (l != kInvalid) {
                float total = pf[6u * l + srow];
                for (uint32_t i = t_child_begin[l]; i < t_child_end[l]; ++i) {
                    const uint32_t child = t_children[i];
                    const float* X = xup + 36u * child + srow, *pc = pf + 6u * child;
                    float pushed = 0.0f;
#pragma unroll
                    for (int c = 0; c < 6; ++c) pushed += X[6 * c] * pc[c];
                    total += pushed;
                }
                pf[6u * l + srow] = total;
            }
            wave_sync();
        }
        // generalized bias and right-hand side, lane = DoF (:570-585)
        float* bias = d.articulation_bias + size_t{env} * stride;
        if (lane < stride) {
            if (lane >= n) bias[lane] = 0.0f;
            else {
                const uint32_t link = m.dof_link[lane], component = m.dof_component[lane];
                const bool scalar = component == kInvalid;
                const float velocity = scalar ? qd[link] : v[6u * link + component];
                float b = scalar ? dot6(S + 6u * link, pf + 6u * link) : pf[6u * link + component];
                if (scalar) b += d.joint_gravity_force[lbase + link];   // zero unless uploaded
                const float damping = scalar ? m.joint_damping[link] + (p.fold_drive_damping != 0u ? d.drive_dissipation[lbase + link] : 0.0f) : 0.0f;
                const float spring = scalar ? m.joint_stiffness[link] * (q[link] - m.joint_spring_reference[link]) : 0.0f;
                vel[lane] = velocity;
                bias[lane] = b;
                acc[lane] = (scalar ? d.tau[lbase + link] : 0.0f) - b - damping * velocity - spring;
            }
        }
        __syncthreads();   // the second wavefront has the mass matrix in LDS
        // the dense mass tile reaches HBM once, in row-major runs (row and column of a lane's word step with it: a
        // division by the stride a word costs more than the word)
        float* M = d.m + size_t{env} * stride * stride;
        const uint32_t rows_a_step = uint32_t(kWave) / stride, columns_a_step = uint32_t(kWave) % stride;
        {
            uint32_t i = lane / stride, j = lane % stride;
            for (uint32_t e = lane; e < stride * stride; e += kWave) {
                M[e] = i < n && j < n ? A[i * ld + j] : 0.0f;
                i += rows_a_step; j += columns_a_step;
                if (j >= stride) { j -= stride; ++i; }
            }
        }
        __syncthreads();   // ... and may now overwrite it with the factor
    } else {
        // CRBA: composite inertias leaf to root; the push X^T Ic X runs entry-parallel on 36 lanes (articulation_mass.cuh:146-165)
        // deepest parents first, parents of one depth in link order, a parent's children in list order: the cooked visiting
        // list, sixty-four visits at a time - a lane reads one visit's child and parent, the visits take theirs as lane reads
        for (uint32_t first = 0u; first < nl; first += kWave) {
            uint32_t my_child = kInvalid, my_parent = 0u;
            if (first + lane < nl) {
                my_child = m.link_push_order[first + lane];
                if (my_child != kInvalid) my_parent = m.parent_link[my_child];
            }
            for (uint32_t visit = 0u; visit < uint32_t(kWave); ++visit) {
                const uint32_t child = uint32_t(__builtin_amdgcn_readlane(int(my_child), int(visit)));
                if (child == kInvalid) break;
                const uint32_t l = uint32_t(__builtin_amdgcn_readlane(int(my_parent), int(visit)));
                const float* X = xup + 36u * child;
                const float* C = ic + 36u * child;
                const uint32_t entry_row = lane / 6u, entry_col = lane % 6u;
                if (lane < 36u) {
                    float value = 0.0f;
#pragma unroll
                    for (int k = 0; k < 6; ++k) value += C[entry_row * 6u + k] * X[k * 6u + entry_col];
                    tmp[lane] = value;
                }
                wave_sync();
                if (lane < 36u) {
                    float value = 0.0f;
#pragma unroll
                    for (int k = 0; k < 6; ++k) value += X[k * 6u + entry_row] * tmp[k * 6u + entry_col];
                    ic[36u * l + lane] += value;
                }
                wave_sync();
            }
        }
        if (floating_root && lane < 36u) A[(lane / 6u) * ld + lane % 6u] = ic[lane];
        wave_sync();
        // mass columns: each jointed link pushes Ic S to the root (:183-252)
        for (uint32_t l = lane; l < nl; l += kWave) {
            if (joint_dof(uint8_t(t_type[l])) == 0u) continue;
            if (l == 0u && floating_root) continue;
            const uint32_t dof_i = t_dof[l];
            float force[6], sl[6];
#pragma unroll
            for (int i = 0; i < 6; ++i) sl[i] = S[6u * l + i];
            mat66_vec(ic + 36u * l, sl, force);
            float diagonal = dot6(sl, force);
            diagonal += m.joint_armature[l];
            if (p.fold_drive_damping != 0u) diagonal += p.dt * d.drive_dissipation[lbase + l];   // articulation_mass.cuh:206-208
            A[dof_i * ld + dof_i] = diagonal;
            uint32_t walk = l;
            for (;;) {
                const uint32_t parent = t_parent[walk];   // the walk reads the tree from LDS: a table load a hop would be its latency
                if (parent == kInvalid) break;
                float pushed[6];
                mat66t_vec(xup + 36u * walk, force, pushed);
#pragma unroll
                for (int i = 0; i < 6; ++i) force[i] = pushed[i];
                walk = parent;
                if (joint_dof(uint8_t(t_type[walk])) == 0u) continue;
                const uint32_t dof_j = t_dof[walk];
                if (walk == 0u && floating_root) {
#pragma unroll
                    for (int b = 0; b < 6; ++b) { A[dof_i * ld + b] = force[b]; A[b * ld + dof_i] = force[b]; }
                    continue;
                }
                const float entry = dot6(S + 6u * walk, force);
                A[dof_i * ld + dof_j] = entry;
                A[dof_j * ld + dof_i] = entry;
            }
        }
        __syncthreads();   // the mass matrix stands in LDS: the first wavefront carries it to HBM while this one factors it
        // LDL^T, right-looking, lane = row in registers; the strict lower triangle becomes L and the diagonal D (:269-335).
        // Rows and columns n..N-1 are those of the identity.  Entry (i, j) loses (L_ik L_jk) D_k for k = 0, 1, ... as the
        // serial loop does (the products in the reference's order: fused into one multiply-add an entry the factor
        // differs in its last place, and of 4096 humanoids one then ends its eight sweeps 2e-4 from the oracle's);
        // what a lane computes above its diagonal is never read.
        {
            // (every word read whether or not the lane keeps it, from a place inside the matrix: a read under a condition
            // compiles to a branch a word)
            const uint32_t ll = local_lane(lane);
            const uint32_t from = (ll < n ? ll : 0u) * ld;
#pragma unroll
            for (int k = 0; k < N; ++k) {
                const float word = A[from + (uint32_t(k) < n ? uint32_t(k) : 0u)];
                row[k] = ll < n && uint32_t(k) < n ? word : (ll == uint32_t(k) ? 1.0f : 0.0f);
            }
        }
        {
            const uint32_t ll = local_lane(lane);
#pragma unroll
            for (int k = 0; k < N; ++k) {
                const float diagonal = fmaxf(lane_value(row[k], k), 1.0e-6f);
                const float lik = row[k] / diagonal;
                row[k] = ll > uint32_t(k) ? lik : (ll == uint32_t(k) ? diagonal : row[k]);
#pragma unroll
                for (int j0 = k + 1; j0 < N; j0 += 8) {
                    float l[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) l[t] = j0 + t < N ? lane_value(lik, j0 + t) : 0.0f;
#pragma unroll
                    for (int t = 0; t < 8; ++t)
                        if (j0 + t < N) row[j0 + t] -= lik * l[t] * diagonal;
                }
            }
            __syncthreads();   // the first wavefront has read the mass matrix: its words take the factor
            if (ll < n) {
#pragma unroll
                for (int k = 0; k < N; ++k)
                    if (uint32_t(k) < n) A[ll * ld + k] = row[k];
            }
        }
    }
    __syncthreads();   // the factor stands in LDS, and the right-hand side (first wavefront) meets it (second)
    if (forces) {
        float* factor = d.m_factor + size_t{env} * stride * stride;
        const uint32_t rows_a_step = uint32_t(kWave) / stride, columns_a_step = uint32_t(kWave) % stride;
        uint32_t i = lane / stride, j = lane % stride;
        for (uint32_t e = lane; e < stride * stride; e += kWave) {
            if (j <= i) factor[e] = i < n ? A[i * ld + j] : (i == j ? 1.0e-6f : 0.0f);
            i += rows_a_step; j += columns_a_step;
            if (j >= stride) { j -= stride; ++i; }
        }
        return;
    }
    // solve L D L^T x = rhs: forward by rows, scale, backward by columns (:357-396)
    float x = lane < n ? acc[lane] : 0.0f;
    {
        const uint32_t ll = local_lane(lane);
        float col[N];
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const float word = A[(uint32_t(i) < n ? uint32_t(i) : 0u) * ld + (ll < n ? ll : 0u)];
            col[i] = ll < uint32_t(i) && uint32_t(i) < n ? word : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const float solved = lane_value(x, j);
            if (ll > uint32_t(j) && ll < n) x -= row[j] * solved;
        }
        if (ll < n) x = x / A[ll * ld + ll];
#pragma unroll
        for (int i = N - 1; i >= 0; --i) {
            const float value = lane_value(x, i);
            if (ll < uint32_t(i)) x -= col[i] * value;
        }
    }
    if (lane < stride) d.articulation_qdd[size_t{env} * stride + lane] = lane < n ? x : 0.0f;
    if (lane < n) acc[lane] = x;
    wave_sync();
    // write back accelerations and the unconstrained velocity update (:597-615)
    for (uint32_t l = lane; l < nl; l += kWave) {
        const uint8_t type = m.joint_type[l];
        float qdd = 0.0f;
        if (joint_dof(type) == 1u) {
            const uint32_t dof = m.link_dof[l];
            qdd = acc[dof];
            if (p.integrate_velocity != 0u) qd[l] = vel[dof] + p.dt * qdd;
        }
        d.qddot[lbase + l] = qdd;
        if (p.integrate_velocity != 0u) {
            float* wr = d.link_wrench + (lbase + l) * 6u;
#pragma unroll
            for (int i = 0; i < 6; ++i) wr[i] = 0.0f;
        }
    }
    if (floating_root && p.integrate_velocity != 0u && lane < 6u) {
        const uint32_t component = lane, i = component % 3u, j = (i + 1u) % 3u, k = (i + 2u) % 3u;
        const float transport = component < 3u ? 0.0f : vel[j] * vel[3u + k] - vel[k] * vel[3u + j];
        v[component] = vel[lane] + p.dt * (acc[lane] + transport);
    }
    wave_sync();
    // final link accelerations (:617-644)
    for (uint32_t pass = 0u; pass < passes; ++pass) {
        const uint32_t l = link_of_pass(pass);
        if (l != kInvalid) {
            const uint32_t parent = t_parent[l], type = t_type[l];
            float al;
            if (type == kFloatingBase) al = srow < 3u ? acc[srow] : acc[srow] - gravity_in_base_row;
            else {
                const float* X = xup + 36u * l + 6u * srow;
                al = 0.0f;
#pragma unroll
                for (int c = 0; c < 6; ++c) al += X[c] * (parent != kInvalid ? a[6u * parent + c] : (c < 3 ? 0.0f : (c == 3 ? -gravity.x : c == 4 ? -gravity.y : -gravity.z)));
                const float qdd = joint_dof(uint8_t(type)) == 1u ? acc[t_dof[l]] : 0.0f;
                al += vb[6u * l + srow] + S[6u * l + srow] * qdd;
            }
            a[6u * l + srow] = al;
        }
        wave_sync();
    }
    for (uint32_t e = lane; e < nl * 6u; e += kWave) {
        d.link_velocity[lbase * 6u + e] = v[e];
        d.link_acceleration[lbase * 6u + e] = a[e];
    }
}

// ---- IntegratePosition: one thread per (env, link) (articulation.cu:732-791) ------------------------------
__device__ __forceinline__ void integrate_position_of_link(const ModelView& m, const DataView& d, const IntegratePositionParams& p,
                                                            uint32_t env, uint32_t l) {
    const uint32_t gid = env * m.links_per_env + l;
    const float dt = p.dt;
    if (p.pos_pass != 0u) d.q[gid] += (d.qdot[gid] + d.qdot_pseudo[gid]) * dt;
    else d.q[gid] += d.qdot[gid] * dt;
    if (m.parent_link[l] == kInvalid && m.joint_type[l] == kFloatingBase) {
        float* rv = d.link_velocity + size_t{gid} * 6u;
        Xf pose = load_xf(d.base_pose + size_t{env} * 7u);
        float vv[6];
#pragma unroll
        for (int i = 0; i < 6; ++i) vv[i] = p.pos_pass != 0u ? rv[i] + d.link_velocity_pseudo[size_t{gid} * 6u + i] : rv[i];
        const V3 lin_world = rotate_forward(pose.r, V3{vv[3], vv[4], vv[5]});
        pose.p = add3(pose.p, scale3(lin_world, dt));
        const Q4 dq{1.0f, 0.5f * vv[0] * dt, 0.5f * vv[1] * dt, 0.5f * vv[2] * dt};
        pose.r = qnormalize_lt(qmul(pose.r, dq), 1.0e-24f);
        const V3 turned = rotate_inverse(qnormalize_lt(dq, 1.0e-24f), V3{rv[3], rv[4], rv[5]});
        rv[3] = turned.x; rv[4] = turned.y; rv[5] = turned.z;
        store_xf(d.base_pose + size_t{env} * 7u, pose);
    }
}
__global__ void IntegratePositionKernel(ModelView m, DataView d, IntegratePositionParams p) {
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= p.total_link_count) return;
    integrate_position_of_link(m, d, p, gid / m.links_per_env, gid % m.links_per_env);
}

// ---- FkLinkVelocities (articulation.cu:647-689) ---------------------------------------------------------
// One wavefront, one environment; `v` holds nl * 6 words of LDS
__device__ __forceinline__ void link_velocities_of_env(const ModelView& m, const DataView& d, uint32_t env, uint32_t lane, float* v) {
    const uint32_t nl = m.links_per_env;
    const size_t lbase = size_t{env} * nl;
    for (uint32_t e = lane; e < nl * 6u; e += kWave) v[e] = d.link_velocity[lbase * 6u + e];
    wave_sync();
    // the joint transform and the joint's own twist do not wait on the tree: a lane prepares its link's before the sweep
    struct Jointed { uint32_t depth, parent; bool state; float X[36], own[6]; };
    auto prepare = [&](uint32_t l, Jointed& t) {
        const uint8_t type = m.joint_type[l];
        t.depth = m.link_tree_depth[l]; t.parent = m.parent_link[l];
        t.state = t.parent == kInvalid && type == kFloatingBase;   // a floating root's twist is state
        if (t.state) return;
        float s[6];
        joint_transform(m, l, d.q[lbase + l], t.X);
        motion_subspace(type, load3(m.joint_axis + 3u * l), s);
        const float qdl = d.qdot[lbase + l];
#pragma unroll
        for (int c = 0; c < 6; ++c) t.own[c] = s[c] * qdl;
    };
    auto propagate = [&](uint32_t l, const Jointed& t) {
        if (t.state) return;
        float pv[6] = {0, 0, 0, 0, 0, 0}, vl[6];
        if (t.parent != kInvalid) {
#pragma unroll
            for (int i = 0; i < 6; ++i) pv[i] = v[6u * t.parent + i];
        }
        mat66_vec(t.X, pv, vl);
#pragma unroll
        for (int c = 0; c < 6; ++c) v[6u * l + c] = vl[c] + t.own[c];
    };
    Jointed own;
    own.depth = kInvalid; own.parent = kInvalid; own.state = true;
    if (lane < nl) prepare(lane, own);
    for (uint32_t depth = 0u; depth <= m.max_depth; ++depth) {
        if (own.depth == depth) propagate(lane, own);
        for (uint32_t l = lane + kWave; l < nl; l += kWave) {
            Jointed t;
            prepare(l, t);
            if (t.depth == depth) propagate(l, t);
        }
        wave_sync();
    }
    for (uint32_t e = lane; e < nl * 6u; e += kWave) d.link_velocity[lbase * 6u + e] = v[e];
}
__global__ void __launch_bounds__(kWave) FkLinkVelocitiesKernel(ModelView m, DataView d, uint32_t env_count) {
    extern __shared__ float lds[];
    if (blockIdx.x >= env_count) return;
    link_velocities_of_env(m, d, blockIdx.x, threadIdx.x, lds);
}

// What follows the solve in a step - positions integrated, world poses, link twists, the bodies' poses - as one kernel,
// one wavefront an environment: four kernels that each take about the time of a launch become one, running the same
// device code in the same order (IntegratePosition, FkWorldPoses, FkLinkVelocities, SyncLinkBodyPose).  A plan takes this
// route when its op list holds the four in a row (backend.hip); an op dispatched by itself runs its own kernel.
__global__ void __launch_bounds__(2 * kWave) StepTailKernel(ModelView m, DataView d, IntegratePositionParams p, uint32_t env_count,
                                                            uint32_t sync_bodies) {
    extern __shared__ float lds[];
    const uint32_t env = blockIdx.x, lane = threadIdx.x % kWave, nl = m.links_per_env;
    const bool twists = threadIdx.x >= uint32_t(kWave);   // world poses and link twists do not depend on each other: a wavefront each
    if (env >= env_count) return;
    if (!twists) for (uint32_t l = lane; l < nl; l += kWave) integrate_position_of_link(m, d, p, env, l);
    __syncthreads();   // the new coordinates, base pose and root twist are in memory for both wavefronts
    if (twists) { link_velocities_of_env(m, d, env, lane, lds + nl * 7u); return; }
    world_poses_of_env(m, d, env, lane, lds);
    if (sync_bodies == 0u) return;
    wave_sync();
    for (uint32_t b = lane; b < m.bodies_per_env; b += kWave) sync_body_pose(m, d, env, b, lds);
}

}  // namespace

// ---- op entry points ------------------------------------------------------------------------------------
Status OpFkWorldPoses(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const FkWorldPosesParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->articulation_count == 0u || p->total_link_count == 0u) return Status::Ok;
    if (m.links_per_env == 0u || p->total_link_count != p->articulation_count * m.links_per_env) return Status::InvalidArgument;
    const size_t lds = size_t{m.links_per_env} * 7u * sizeof(float);
    hipLaunchKernelGGL(FkWorldPosesKernel, dim3(p->articulation_count), dim3(kWave), lds, stream, m, d, p->articulation_count);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

// The four ops after the solve as one launch; Unsupported when any of them would not run its kernel as dispatched
// (the caller then dispatches them one by one).
Status OpStepTail(const ModelView& m, const DataView& d, const IntegratePositionParams* integrate, const FkWorldPosesParams* poses,
                  const FkLinkVelocitiesParams* twists, const SyncLinkBodyPoseParams* bodies, hipStream_t stream) {
    if (integrate == nullptr || poses == nullptr || twists == nullptr) return Status::Unsupported;
    const uint32_t E = poses->articulation_count, links = E * m.links_per_env;
    if (E == 0u || m.links_per_env == 0u || integrate->dt <= 0.0f || integrate->total_link_count != links ||
        poses->total_link_count != links || poses->selected_env_count != 0u || twists->articulation_count != E ||
        twists->total_link_count != links) return Status::Unsupported;
    if (bodies != nullptr && (bodies->env_count != E || bodies->bodies_per_env != m.bodies_per_env || bodies->bodies_per_env == 0u ||
                              bodies->selected_env_count != 0u)) return Status::Unsupported;
    const size_t lds = size_t{m.links_per_env} * 13u * sizeof(float);
    hipLaunchKernelGGL(StepTailKernel, dim3(E), dim3(2 * kWave), lds, stream, m, d, *integrate, E, bodies != nullptr ? 1u : 0u);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

using DynamicsKernel = void (*)(ModelView, DataView, ArticulationDynamicsParams, uint32_t);
static const DynamicsKernel kDynamicsKernels[16] = {
    ArticulationDynamicsKernel<4>, ArticulationDynamicsKernel<8>, ArticulationDynamicsKernel<12>, ArticulationDynamicsKernel<16>,
    ArticulationDynamicsKernel<20>, ArticulationDynamicsKernel<24>, ArticulationDynamicsKernel<28>, ArticulationDynamicsKernel<32>,
    ArticulationDynamicsKernel<36>, ArticulationDynamicsKernel<40>, ArticulationDynamicsKernel<44>, ArticulationDynamicsKernel<48>,
    ArticulationDynamicsKernel<52>, ArticulationDynamicsKernel<56>, ArticulationDynamicsKernel<60>, ArticulationDynamicsKernel<64>};

Status OpArticulationDynamics(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const ArticulationDynamicsParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->articulation_count == 0u || p->total_link_count == 0u) return Status::Ok;
    if (m.dof > kMaxDof || m.dof == 0u || p->max_dof != m.max_dof ||
        p->total_link_count != p->articulation_count * m.links_per_env) return Status::InvalidArgument;
    const size_t lds = size_t{DynamicsLdsFloats(m.links_per_env, m.dof, m.sweep_passes)} * sizeof(float);
    if (lds > 160u * 1024u) return Status::InvalidArgument;
    hipLaunchKernelGGL(kDynamicsKernels[((m.dof + 3u) & ~3u) / 4u - 1u], dim3(p->articulation_count), dim3(2 * kWave), lds, stream, m, d,
                       *p, p->articulation_count);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

namespace {
// SolveMassBlock (articulation_mass.cuh:357-396) by one thread: forward by columns, divide, backward
__device__ void solve_mass_serial(const float* factor, float* value, uint32_t n, uint32_t stride) {
    for (uint32_t j = 0u; j < n; ++j) {
        const float solved = value[j];
        for (uint32_t i = j + 1u; i < n; ++i) value[i] -= factor[size_t{i} * stride + j] * solved;
    }
    for (uint32_t i = 0u; i < n; ++i) value[i] = value[i] / factor[size_t{i} * stride + i];
    for (uint32_t end = n; end > 0u; --end) {
        const uint32_t i = end - 1u;
        float sum = value[i];
        for (uint32_t j = i + 1u; j < n; ++j) sum -= factor[size_t{j} * stride + i] * value[j];
        value[i] = sum;
    }
}

// AccumulateChainJointForce (articulation_types.cuh:193-238): what a force f and a moment at `point` add to the
// generalized force of the joint of `link`
__device__ void accumulate_chain(const ModelView& m, const DataView& d, uint32_t env, uint32_t link, V3 point, V3 f, V3 moment, float* out) {
    const uint32_t dof_index = m.link_dof[link], stride = m.max_dof;
    const uint8_t type = m.joint_type[link];
    if (type == kFloatingBase) {
        const Xf base = load_xf(d.base_pose + size_t{env} * 7u);
        const V3 lever = sub3(point, base.p);
        const V3 e[3] = {rotate_normalized(base.r, V3{1, 0, 0}), rotate_normalized(base.r, V3{0, 1, 0}), rotate_normalized(base.r, V3{0, 0, 1})};
        for (uint32_t b = 0u; b < 3u; ++b) {
            const float angular = dot3(cross3(e[b], lever), f) + dot3(e[b], moment), linear = dot3(e[b], f);
            if (dof_index + b < stride) out[dof_index + b] += angular;
            if (dof_index + 3u + b < stride) out[dof_index + 3u + b] += linear;
        }
        return;
    }
    const Xf pose = load_xf(d.link_pose + (size_t{env} * m.links_per_env + link) * 7u);
    const V3 axis_world = rotate_normalized(pose.r, load3(m.joint_axis + 3u * link));
    float entry;
    if (type == kPrismatic) entry = dot3(axis_world, f);
    else entry = dot3(cross3(axis_world, sub3(point, pose.p)), f) + dot3(axis_world, moment);
    if (dof_index < stride) out[dof_index] += entry;
}

// ArticulationReferenceWeightsKernel (articulation.cu:434-501), one thread an environment as in the reference: the
// diagonal of M^-1 (a floating base's six entries averaged over its rotations and its translations), and for every
// link the mean response of its centre of mass to a unit force and to a unit moment along the three world axes.
// `m_factor` holds the factor of the mass matrix at the current pose (no drive damping folded in).
__global__ void __launch_bounds__(kWave) ReferenceWeightsKernel(ModelView m, DataView d, uint32_t env_count) {
    const uint32_t env = blockIdx.x * kWave + threadIdx.x;
    if (env >= env_count) return;
    const uint32_t nl = m.links_per_env, nb = m.bodies_per_env, md = m.max_dof, dof = m.dof;
    float* weights = d.body_invweight0 + size_t{env} * nb * 2u;
    for (uint32_t b = 0u; b < nb; ++b) weights[2u * b] = weights[2u * b + 1u] = 0.0f;   // static rows move under nothing
    const float* factor = d.m_factor + size_t{env} * md * md;
    float* diagonal = d.dof_invweight0 + size_t{env} * md;
    float row[kMaxDof], solution[kMaxDof];
    for (uint32_t k = 0u; k < dof; ++k) {
        for (uint32_t i = 0u; i < dof; ++i) solution[i] = i == k ? 1.0f : 0.0f;
        solve_mass_serial(factor, solution, dof, md);
        diagonal[k] = solution[k];
    }
    if (m.joint_type[0] == kFloatingBase) {
        const float rotation = (diagonal[0] + diagonal[1] + diagonal[2]) / 3.0f;
        const float translation = (diagonal[3] + diagonal[4] + diagonal[5]) / 3.0f;
        for (uint32_t i = 0u; i < 3u; ++i) { diagonal[i] = rotation; diagonal[i + 3u] = translation; }
    }
    for (uint32_t link = 0u; link < nl; ++link) {
        const Xf pose = load_xf(d.link_pose + (size_t{env} * nl + link) * 7u);
        const V3 point = add3(pose.p, rotate_normalized(pose.r, load3(m.link_inertial_frame + 7u * link)));
        float weight[2] = {0.0f, 0.0f};
        for (uint32_t axis = 0u; axis < 6u; ++axis) {
            for (uint32_t k = 0u; k < dof; ++k) row[k] = 0.0f;
            const V3 unit{axis % 3u == 0u ? 1.0f : 0.0f, axis % 3u == 1u ? 1.0f : 0.0f, axis % 3u == 2u ? 1.0f : 0.0f};
            const V3 none{0.0f, 0.0f, 0.0f};
            for (uint32_t walk = link; walk != kInvalid; walk = m.parent_link[walk])
                if (joint_dof(m.joint_type[walk]) != 0u) accumulate_chain(m, d, env, walk, point, axis < 3u ? unit : none, axis < 3u ? none : unit, row);
            for (uint32_t k = 0u; k < dof; ++k) solution[k] = row[k];
            solve_mass_serial(factor, solution, dof, md);
            for (uint32_t k = 0u; k < dof; ++k) weight[axis / 3u] += row[k] * solution[k];
        }
        const uint32_t body = m.link_body[link];
        if (body < nb) { weights[2u * body] = weight[0] / 3.0f; weights[2u * body + 1u] = weight[1] / 3.0f; }
    }
}
}  // namespace

// ReferenceWeights (op_schema.hpp:123-130; articulation.cu:425-500): the mass matrix at the current poses without
// drive damping, its factor, and the reference weights from it.  World creation and reset dispatch it after the poses
// are refreshed (nk/pipeline/world.cpp:553-561).
// BodyReferenceWeightsKernel (articulation.cu:425-432): a free body's weights are its inverse mass and the mean of its
// inverse principal moments; rows without mass weigh nothing
__global__ void __launch_bounds__(256) BodyReferenceWeightsKernel(DataView d, uint32_t count) {
    const uint32_t body = blockIdx.x * 256u + threadIdx.x;
    if (body >= count) return;
    const float* inverse = d.body_inv_inertia + size_t{body} * 3u;
    d.body_invweight0[2u * body] = d.body_inv_mass[body];
    d.body_invweight0[2u * body + 1u] = (inverse[0] + inverse[1] + inverse[2]) / 3.0f;
}

Status OpReferenceWeights(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const ReferenceWeightsParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (m.free_body != 0u) {
        if (p->total_body_count == 0u) return Status::Ok;
        hipLaunchKernelGGL(BodyReferenceWeightsKernel, dim3((p->total_body_count + 255u) / 256u), dim3(256), 0, stream, d, p->total_body_count);
        return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
    }
    if (p->articulation_count == 0u || p->total_link_count == 0u) return Status::Ok;
    if (p->articulations_per_env != 1u || p->max_dof != m.max_dof || p->bodies_per_env != m.bodies_per_env ||
        p->total_link_count != p->articulation_count * m.links_per_env) return Status::InvalidArgument;
    ArticulationDynamicsParams mass{};   // no velocity update, no wrench, nothing folded into the diagonal
    mass.max_dof = p->max_dof; mass.integrate_velocity = 0u; mass.articulation_count = p->articulation_count;
    mass.total_link_count = p->total_link_count; mass.max_links = m.links_per_env; mass.links_per_env = m.links_per_env;
    mass.bodies_per_env = m.bodies_per_env;
    if (m.dof != 0u) {
        const Status status = OpArticulationDynamics(m, d, &mass, stream);
        if (status != Status::Ok) return status;
    }
    hipLaunchKernelGGL(ReferenceWeightsKernel, dim3((p->articulation_count + kWave - 1u) / kWave), dim3(kWave), 0, stream, m, d,
                       p->articulation_count);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

namespace {
// ActuatorVelocityDerivative (articulation.cu:942-948): what a servo's effort changes per unit joint velocity, none
// while its own force limit clamps it
__device__ float actuator_velocity_derivative(const DataView& d, uint32_t mode, size_t link) {
    if (d.drive_force_limit[link] > 0.0f && fabsf(d.drive_command[link] - d.joint_gravity_force[link]) > d.drive_force_limit[link]) return 0.0f;
    return mode == kDrivePdPosition ? d.drive_damping[link] : mode == kDriveVelocity ? d.drive_stiffness[link] : 0.0f;
}

// ArticulationDampingKernel (articulation.cu:950-1000), one wavefront an environment: contacts were solved with the plain
// mass; the step's velocity change now goes through (M + dt D)^-1 M, D the joint damping and, for the implicit
// integrators, the unclamped servo velocity gains.  M + dt D is factored as L D L^T in LDS, lane = row; every entry takes
// its pivots' updates in pivot order (FactorMass, articulation_mass.cuh:269-335), and the solve runs forward by
// columns, divides, and substitutes back serially (SolveMassBlock :357-396).
__global__ void __launch_bounds__(kWave) ArticulationDampingKernel(ModelView m, DataView d, ArticulationDampingParams p) {
    extern __shared__ float lds[];
    const uint32_t env = blockIdx.x, lane = threadIdx.x, n = m.dof, stride = m.max_dof, nl = m.links_per_env, ld = n + 1u;
    float* A = lds;               // n x (n + 1)
    float* change = A + n * ld;   // n
    const size_t lbase = size_t{env} * nl, base = size_t{env} * stride;
    const bool coordinate = lane < n;
    uint32_t link = 0u, component = kInvalid;
    float value = 0.0f, velocity = 0.0f, damping = 0.0f;
    if (coordinate) {
        link = m.dof_link[lane]; component = m.dof_component[lane];
        const bool scalar = component == kInvalid;
        value = scalar ? m.joint_damping[link] : 0.0f;
        if (scalar && p.actuator_derivative != 0u) value += actuator_velocity_derivative(d, p.mode, lbase + link);
        velocity = scalar ? d.qdot[lbase + link] : d.link_velocity[(lbase + link) * 6u + component];
        damping = p.dt * value;
        change[lane] = damping * (velocity - d.step_qdot_flat[base + lane]);
    }
    if (!__any(coordinate && value != 0.0f)) return;
    if (coordinate)
        for (uint32_t j = 0u; j <= lane; ++j) A[lane * ld + j] = d.m[(base + lane) * stride + j] + (j == lane ? damping : 0.0f);
    for (uint32_t k = 0u; k < n; ++k) {
        __syncthreads();
        const float diagonal = fmaxf(A[k * ld + k], 1.0e-6f);
        __syncthreads();
        float l = 0.0f;
        if (coordinate && lane > k) { l = A[lane * ld + k] / diagonal; A[lane * ld + k] = l; }
        if (lane == k) A[k * ld + k] = diagonal;
        __syncthreads();
        if (coordinate && lane > k)
            for (uint32_t j = k + 1u; j <= lane; ++j) A[lane * ld + j] -= l * A[j * ld + k] * diagonal;
    }
    for (uint32_t j = 0u; j < n; ++j) {   // forward by columns
        __syncthreads();
        const float solved = change[j];
        if (coordinate && lane > j) change[lane] -= A[lane * ld + j] * solved;
    }
    __syncthreads();
    if (coordinate) change[lane] = change[lane] / A[lane * ld + lane];
    __syncthreads();
    if (lane == 0u)
        for (uint32_t end = n; end > 0u; --end) {
            const uint32_t i = end - 1u;
            float sum = change[i];
            for (uint32_t j = i + 1u; j < n; ++j) sum -= A[j * ld + i] * change[j];
            change[i] = sum;
        }
    __syncthreads();
    if (!coordinate) return;
    velocity -= change[lane];
    if (component == kInvalid) d.qdot[lbase + link] = velocity; else d.link_velocity[(lbase + link) * 6u + component] = velocity;
    d.qdot_flat[base + lane] = velocity;
    if (component == kInvalid && p.actuator_derivative != 0u && p.readout_drives != 0u) {
        const float derivative = actuator_velocity_derivative(d, p.mode, lbase + link);
        const float correction = derivative * (velocity - d.step_qdot_flat[base + lane]);
        d.actuator_effort_requested[lbase + link] -= correction;
        d.actuator_effort[lbase + link] -= correction;
        d.tau[lbase + link] -= correction;
    }
}
}  // namespace

// ArticulationDamping (op_schema.hpp:132-141): the op a MuJoCo integrator adds after the constraint solve.
Status OpArticulationDamping(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const ArticulationDampingParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->articulation_count == 0u || p->total_link_count == 0u || m.dof == 0u) return Status::Ok;
    if (m.dof > kMaxDof || p->max_dof != m.max_dof || p->total_link_count != p->articulation_count * m.links_per_env) return Status::InvalidArgument;
    const size_t lds = size_t{m.dof} * (m.dof + 2u) * sizeof(float);
    hipLaunchKernelGGL(ArticulationDampingKernel, dim3(p->articulation_count), dim3(kWave), lds, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

Status OpIntegratePosition(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const IntegratePositionParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->dt <= 0.0f || p->total_link_count == 0u) return Status::Ok;
    if (m.free_body != 0u) return BodyIntegratePosition(m, d, *p, stream);
    const uint32_t blocks = (p->total_link_count + 255u) / 256u;
    hipLaunchKernelGGL(IntegratePositionKernel, dim3(blocks), dim3(256), 0, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

Status OpFkLinkVelocities(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const FkLinkVelocitiesParams*>(params);
    if (p == nullptr) return Status::InvalidArgument;
    if (p->articulation_count == 0u || p->total_link_count == 0u) return Status::Ok;
    const size_t lds = size_t{m.links_per_env} * 6u * sizeof(float);
    hipLaunchKernelGGL(FkLinkVelocitiesKernel, dim3(p->articulation_count), dim3(kWave), lds, stream, m, d, p->articulation_count);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

void InitArticulationKernels() {
    for (DynamicsKernel kernel : kDynamicsKernels) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
    }
}

// ApplyAffineDriveKernel (articulation.cu:836-940): one thread per link turns the controller fields into an affine
// effort `command - dissipation * qdot` and its bounds for the drive row, and overwrites tau with the feedforward
// load.  Gravity compensation (ProjectGravityCompensationKernel :393-423) is not authored on this path:
// joint_gravity_force stays as uploaded.  The inverse-dynamics modes (ComputedTorque, Osc) are not built.
__global__ void __launch_bounds__(256) ApplyAffineDriveKernel(ModelView m, DataView d, ApplyDrivesParams p) {
    const uint32_t link = blockIdx.x * blockDim.x + threadIdx.x;
    if (link >= p.total_link_count) return;
    d.drive_command[link] = d.drive_dissipation[link] = 0.0f;
    d.drive_lower[link] = d.drive_upper[link] = 0.0f;
    d.tau[link] = 0.0f;
    const uint32_t local = link % p.links_per_env;
    if (joint_dof(m.joint_type[local]) != 1u) return;
    const uint32_t mode = p.mode;
    const bool implicit = p.defer_velocity_damping != 0u;
    const bool position_control = mode == kDrivePdPosition, velocity_control = mode == kDriveVelocity;
    const float kp = d.drive_stiffness[link], kd = d.drive_damping[link];
    if ((position_control && (!isfinite(d.drive_target[link]) || !isfinite(kp) || kp < 0.0f || !isfinite(kd) || (implicit && kd < 0.0f))) ||
        ((position_control || velocity_control) && !isfinite(d.velocity_target[link])) ||
        (velocity_control && (!isfinite(kp) || kp < 0.0f)) ||
        (mode == kDriveActuator && !isfinite(d.actuator_noload_speed[link]))) {
        atomicOr(d.env_status + link / p.links_per_env, kEnvStatusControlFailure);
        return;
    }
    const float velocity = d.qdot[link];
    const float limit = d.drive_force_limit[link];
    float lower = limit > 0.0f ? -limit : -FLT_MAX;
    float upper = limit > 0.0f ? limit : FLT_MAX;
    float bias = 0.0f, damping = 0.0f;
    if (mode == kDrivePdPosition) {
        // an implicit spring is evaluated at the end of the step, adding dt kp to the damping
        damping = kd + (implicit ? p.dt * kp : 0.0f);
        bias = kp * (d.drive_target[link] - d.q[link]) + damping * d.velocity_target[link];
    } else if (mode == kDriveVelocity) {
        damping = kp;
        bias = damping * d.velocity_target[link];
    } else {   // torque, actuator
        bias = d.drive_target[link];
        if (mode == kDriveActuator && limit > 0.0f && d.actuator_noload_speed[link] > 0.0f) {
            const float speed_bias = limit * velocity / d.actuator_noload_speed[link];
            lower = fminf(fmaxf(-limit - speed_bias, -limit), limit);
            upper = fminf(fmaxf(limit - speed_bias, -limit), limit);
        }
    }
    const float effort = bias - damping * velocity;
    const float gravity_force = d.joint_gravity_force[link];
    const bool saturated = effort < lower || effort > upper;
    const float joint_limit = d.drive_joint_force_limit[link];
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
    } else {   // the row clamps the command bias = effort + damping * velocity
        bias += gravity_force;
        lower += gravity_force + damping * velocity;
        upper += gravity_force + damping * velocity;
    }
    const float feedforward = d.joint_f[link];
    if (!isfinite(bias) || !isfinite(damping) || damping < 0.0f || !isfinite(limit) || !isfinite(feedforward) || !isfinite(velocity) ||
        !isfinite(d.q[link])) {
        atomicOr(d.env_status + link / p.links_per_env, kEnvStatusControlFailure);
        return;
    }
    d.drive_command[link] = bias;
    d.drive_dissipation[link] = damping;
    d.drive_lower[link] = lower;
    d.drive_upper[link] = upper;
    d.tau[link] = feedforward;
}

// ReadoutDrivesKernel (articulation.cu:999-1016)
__global__ void __launch_bounds__(256) ReadoutDrivesKernel(ModelView m, DataView d, ReadoutDrivesParams p) {
    const uint32_t link = blockIdx.x * blockDim.x + threadIdx.x;
    if (link >= p.total_link_count) return;
    d.actuator_effort_requested[link] = d.actuator_effort[link] = d.actuator_saturated[link] = 0.0f;
    const uint32_t env = link / p.links_per_env, local = link - env * p.links_per_env;
    if (joint_dof(m.joint_type[local]) != 1u) return;
    const size_t row = size_t{env} * p.rows_per_env + p.first_drive_row + local;
    const float effort = d.drive_command[link] - d.drive_dissipation[link] * d.qdot[link];
    d.actuator_effort_requested[link] = effort;
    const float applied = d.lambda[row] / p.dt - d.drive_dissipation[link] * d.qdot[link];
    d.actuator_effort[link] = applied;
    d.actuator_saturated[link] = d.drive_command[link] < d.drive_lower[link] || d.drive_command[link] > d.drive_upper[link] ? 1.0f : 0.0f;
    d.tau[link] += applied;
}

// OpApplyDrives (articulation.cu:1604-1620).  Without drive rows in the cooked world tau is the applied generalized
// force and the op only validates; IntegrateVelocity acts on a free body only (ops_rigid.hip).
Status OpApplyDrives(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const ApplyDrivesParams*>(params);
    if (p == nullptr || p->mode > kDriveActuator) return Status::InvalidArgument;
    // a world cooked without drive rows leaves `tau` as the applied generalized force: nothing to turn into rows
    if (m.joint_drive_rows == 0u) return p->mode == kDriveTorque ? Status::Ok : Status::Unsupported;
    if (p->mode == kDriveComputedTorque || p->mode == kDriveOsc) return Status::Unsupported;
    if (p->total_link_count == 0u) return Status::Ok;
    if (p->links_per_env == 0u || p->links_per_env != m.links_per_env) return Status::InvalidArgument;
    hipLaunchKernelGGL(ApplyAffineDriveKernel, dim3((p->total_link_count + 255u) / 256u), dim3(256), 0, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}
// OpReadoutDrives (articulation.cu:1654-1667)
Status OpReadoutDrives(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const ReadoutDrivesParams*>(params);
    if (p == nullptr || p->dt <= 0.0f) return Status::InvalidArgument;
    if (p->total_link_count == 0u) return Status::Ok;
    if (p->links_per_env == 0u || p->links_per_env != m.links_per_env || p->first_drive_row + p->links_per_env > p->rows_per_env)
        return Status::InvalidArgument;
    hipLaunchKernelGGL(ReadoutDrivesKernel, dim3((p->total_link_count + 255u) / 256u), dim3(256), 0, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}
Status OpIntegrateVelocity(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const IntegrateVelocityParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->dt <= 0.0f) return Status::Ok;
    if (m.free_body != 0u && p->total_body_count > 0u) return BodyIntegrateVelocity(m, d, *p, stream);
    return Status::Ok;
}

}  // namespace nkh
