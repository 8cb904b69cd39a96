// Test infrastructure: extern "C" entry points around the reference's own host-compilable headers, compiled
// from /root/reference/src where they lie (never copied).  Used only to pin the CPU oracle's restatement of
// the row math (nk/solve/augmented_row.hpp), the analytic manifolds (collision/analytical_manifold.hpp),
// the compliant-row discretisation (constraint/solref_solimp.hpp), contact identity and filters.
#include <cstdint>
#include <cstring>

#include "collision/analytical_manifold.hpp"
#include "collision/contact_query.hpp"
#include "collision/shape_kind.hpp"
#include "constraint/solref_solimp.hpp"
#include "nk/contact/contact_identity.hpp"
#include "nk/solve/augmented_row.hpp"
#include "scene/contact_filter.hpp"

using namespace nuka;

static math::Transform MakeTransform(const float* p) {
    math::Transform t;
    t.position = {p[0], p[1], p[2]};
    t.rotation.w = p[3]; t.rotation.x = p[4]; t.rotation.y = p[5]; t.rotation.z = p[6];
    return t;
}

extern "C" {

void ref_scalar_impulse(float dual, float rho, float residual, float compliance, float lower, float upper, float* out) {
    const auto term = nk::augmented::EvaluateScalarImpulse(dual, rho, residual, compliance, lower, upper,
        nk::augmented::ComputeFloatScalarResponse(rho, compliance));
    out[0] = term.impulse; out[1] = term.curvature;
}

void ref_tangent_impulse(const float* dual, float rho, const float* residual, float normal_impulse, float mu_first,
                         float mu_second, float* impulse, float* curvature) {
    const auto term = nk::augmented::EvaluateTangentImpulse({dual[0], dual[1], dual[2]}, rho,
        {residual[0], residual[1], residual[2]}, normal_impulse, mu_first, mu_second);
    impulse[0] = term.impulse.x; impulse[1] = term.impulse.y; impulse[2] = term.impulse.z;
    curvature[0] = term.curvature.xx; curvature[1] = term.curvature.yy; curvature[2] = term.curvature.zz;
    curvature[3] = term.curvature.xy; curvature[4] = term.curvature.xz; curvature[5] = term.curvature.yz;
}

void ref_relax_contact_impulse(const float* dual, const float* next, float* last_step, float* last_weight,
                               float* last_point, float* out) {
    nk::augmented::ContactRelaxation last{{last_step[0], last_step[1], last_step[2]}, *last_weight,
                                          {last_point[0], last_point[1], last_point[2]}};
    const auto r = nk::augmented::RelaxContactImpulse({dual[0], dual[1], dual[2]}, {next[0], next[1], next[2]}, &last);
    last_step[0] = last.step.x; last_step[1] = last.step.y; last_step[2] = last.step.z; *last_weight = last.weight;
    last_point[0] = last.point.x; last_point[1] = last.point.y; last_point[2] = last.point.z;
    out[0] = r.x; out[1] = r.y; out[2] = r.z;
}

float ref_cone_argument(float dual, float rho, float mu, float residual) {
    return nk::augmented::ConeArgument(dual, rho, mu, residual);
}

double ref_momentum_restart(const float* point, const float* next, const float* base, const float* scale) {
    return nk::augmented::MultiplierMomentumRestart({point[0], point[1], point[2]}, {next[0], next[1], next[2]},
                                                    {base[0], base[1], base[2]}, {scale[0], scale[1], scale[2]});
}

double ref_tangent_potential(const float* dual, float rho, const float* residual, float normal_impulse, float mu_first,
                             float mu_second) {
    return nk::augmented::EvaluateTangent({dual[0], dual[1], dual[2]}, rho, {residual[0], residual[1], residual[2]},
                                          normal_impulse, mu_first, mu_second).potential;
}

float ref_tangent_potential_change(const float* dual, float rho, const float* residual, const float* drop,
                                   float normal_impulse, float mu_first, float mu_second) {
    return nk::augmented::TangentPotentialChange({dual[0], dual[1], dual[2]}, rho, {residual[0], residual[1], residual[2]},
                                                 {drop[0], drop[1], drop[2]}, normal_impulse, mu_first, mu_second);
}

static collision::amf::PrimParams Prim(const float* pose, const float* params) {
    collision::amf::PrimParams p;
    p.frame = collision::amf::BuildPrimFrameDevice(MakeTransform(pose));
    p.radius = params[0]; p.half_height = params[1]; p.half_extents = {params[0], params[1], params[2]};
    return p;
}

// Same, with the two prim frames given as cx, cy, cz, t (12 floats): the pipeline bakes its frames in a device-only
// helper, so the manifold math is compared on frames the caller supplies.
static collision::amf::PrimParams PrimFromFrame(const float* f, const float* params) {
    collision::amf::PrimParams p;
    p.frame.cx = {f[0], f[1], f[2]}; p.frame.cy = {f[3], f[4], f[5]}; p.frame.cz = {f[6], f[7], f[8]};
    p.frame.t = {f[9], f[10], f[11]};
    p.radius = params[0]; p.half_height = params[1]; p.half_extents = {params[0], params[1], params[2]};
    return p;
}

uint32_t ref_primitive_pair_frames(uint32_t kind_a, const float* frame_a, const float* params_a, uint32_t kind_b,
                                   const float* frame_b, const float* params_b, float query, float* points,
                                   float* normals, float* penetration, uint64_t* keys) {
    constraint::ContactManifold m;
    collision::amf::PrimitivePair(kind_a, PrimFromFrame(frame_a, params_a), kind_b, PrimFromFrame(frame_b, params_b),
                                  query, &m);
    for (uint32_t i = 0; i < m.point_count; ++i) {
        points[3 * i] = m.points[i].position.x; points[3 * i + 1] = m.points[i].position.y; points[3 * i + 2] = m.points[i].position.z;
        normals[3 * i] = m.points[i].normal.x; normals[3 * i + 1] = m.points[i].normal.y; normals[3 * i + 2] = m.points[i].normal.z;
        penetration[i] = m.points[i].penetration; keys[i] = m.points[i].stable_key;
    }
    return m.point_count;
}

uint32_t ref_primitive_pair(uint32_t kind_a, const float* pose_a, const float* params_a, uint32_t kind_b,
                            const float* pose_b, const float* params_b, float query, float* points, float* normals,
                            float* penetration, uint64_t* keys) {
    constraint::ContactManifold m;
    collision::amf::PrimitivePair(kind_a, Prim(pose_a, params_a), kind_b, Prim(pose_b, params_b), query, &m);
    for (uint32_t i = 0; i < m.point_count; ++i) {
        points[3 * i] = m.points[i].position.x; points[3 * i + 1] = m.points[i].position.y; points[3 * i + 2] = m.points[i].position.z;
        normals[3 * i] = m.points[i].normal.x; normals[3 * i + 1] = m.points[i].normal.y; normals[3 * i + 2] = m.points[i].normal.z;
        penetration[i] = m.points[i].penetration; keys[i] = m.points[i].stable_key;
    }
    return m.point_count;
}

void ref_compose_transform(const float* parent, const float* child, float* out) {
    const auto t = collision::amf::ComposeTransformHD(MakeTransform(parent), MakeTransform(child));
    out[0] = t.position.x; out[1] = t.position.y; out[2] = t.position.z;
    out[3] = t.rotation.w; out[4] = t.rotation.x; out[5] = t.rotation.y; out[6] = t.rotation.z;
}

void ref_make_contact_id(uint32_t a, uint32_t b, const float* local_a, const float* local_b, const float* normal,
                         uint32_t feature, uint32_t manifold_slot, uint64_t* out) {
    nk::CanonicalContactDescriptor d;
    d.a.handle = a; d.b.handle = b;
    d.local_point_a = {local_a[0], local_a[1], local_a[2]}; d.local_point_b = {local_b[0], local_b[1], local_b[2]};
    d.normal = {normal[0], normal[1], normal[2]};
    d.feature_a = d.feature_b = feature; d.manifold_slot = manifold_slot;
    const auto id = nk::MakeContactId(d);
    out[0] = id.pair; out[1] = id.feature;
}

// constraint/solref_solimp.hpp ComputeCompliantRowTerms -> k, b, imp, D, R, aref; DiscretizeCompliantRow -> R, bias, gain
void ref_compliant_row_terms(const float* solref, const float* solimp, float pos_imp, float pos_aref, float vel, float invweight,
                             float dt, int refsafe, float* out) {
    const auto t = constraint::ComputeCompliantRowTerms(solref, solimp, pos_imp, pos_aref, vel, invweight, dt, refsafe != 0);
    out[0] = t.k; out[1] = t.b; out[2] = t.imp; out[3] = t.D; out[4] = t.R; out[5] = t.aref;
}
void ref_discretize_row(float R, float aref_bias, float damping, float dt, float* out) {
    constraint::CompliantContactRow row;
    row.R = R; row.aref_bias = aref_bias; row.damping = damping;
    const auto d = constraint::DiscretizeCompliantRow(row, dt);
    out[0] = d.R; out[1] = d.bias; out[2] = d.reference_gain;
}
// nk/solve/augmented_row.hpp EvaluateEllipticImpulse -> impulse[3], curvature xx yy zz xy xz yz; EllipticMultiplierStep
void ref_elliptic_impulse(const float* dual, float cap, const float* residual, const float* compliance, float mu_first, float* out) {
    const auto t = nk::augmented::EvaluateEllipticImpulse({dual[0], dual[1], dual[2]}, cap, {residual[0], residual[1], residual[2]},
                                                          {compliance[0], compliance[1], compliance[2]}, mu_first);
    out[0] = t.impulse.x; out[1] = t.impulse.y; out[2] = t.impulse.z;
    out[3] = t.curvature.xx; out[4] = t.curvature.yy; out[5] = t.curvature.zz;
    out[6] = t.curvature.xy; out[7] = t.curvature.xz; out[8] = t.curvature.yz;
}
void ref_elliptic_multiplier_step(const float* dual, const float* next, float cap, const float* compliance, float* out) {
    const auto d = nk::augmented::EllipticMultiplierStep({dual[0], dual[1], dual[2]}, {next[0], next[1], next[2]}, cap,
                                                         {compliance[0], compliance[1], compliance[2]});
    out[0] = d.x; out[1] = d.y; out[2] = d.z;
}

void ref_discretize_zero_row(float dt, float* out) {
    const auto d = constraint::DiscretizeCompliantRow(constraint::CompliantContactRow{}, dt);
    out[0] = d.R; out[1] = d.bias; out[2] = d.reference_gain;
}

void ref_merge_friction(float mu_a, float mu_b, float* out) {
    scene::ContactParamsIn a, b;
    a.mu1 = a.mu2 = mu_a; b.mu1 = b.mu2 = mu_b;
    const auto m = scene::MergeContactParams(a, b);
    out[0] = m.mu1; out[1] = m.mu2; out[2] = float(m.condim); out[3] = m.margin;
}

// MergeContactParams of two default-authored profiles that differ in friction: every field the slot material key hashes.
void ref_merged_profile(float mu_a, float mu_b, float* out) {
    scene::ContactParamsIn a, b;
    a.mu1 = a.mu2 = mu_a; b.mu1 = b.mu2 = mu_b;
    const auto m = scene::MergeContactParams(a, b);
    out[0] = m.mu1; out[1] = m.mu2; out[2] = m.friction_spin; out[3] = m.friction_roll; out[4] = m.solref[0]; out[5] = m.solref[1];
    for (int i = 0; i < 5; ++i) out[6 + i] = m.solimp[i];
    out[11] = m.margin; out[12] = m.gap; out[13] = float(m.condim); out[14] = m.friction_stiffness;
    out[15] = m.solreffriction[0]; out[16] = m.solreffriction[1];
}

// MergeContactParams of two profiles packed mu1 mu2 solref[2] solimp[5] margin gap priority solmix condim; out without
// priority and solmix
void ref_merge_params(const float* pa, const float* pb, float* out) {
    scene::ContactParamsIn a, b;
    const float* in[2] = {pa, pb};
    scene::ContactParamsIn* side[2] = {&a, &b};
    for (int s = 0; s < 2; ++s) {
        side[s]->mu1 = in[s][0]; side[s]->mu2 = in[s][1];
        side[s]->solref[0] = in[s][2]; side[s]->solref[1] = in[s][3];
        for (int i = 0; i < 5; ++i) side[s]->solimp[i] = in[s][4 + i];
        side[s]->margin = in[s][9]; side[s]->gap = in[s][10];
        side[s]->priority = int32_t(in[s][11]); side[s]->solmix = in[s][12]; side[s]->condim = uint8_t(in[s][13]);
    }
    const auto m = scene::MergeContactParams(a, b);
    out[0] = m.mu1; out[1] = m.mu2; out[2] = m.solref[0]; out[3] = m.solref[1];
    for (int i = 0; i < 5; ++i) out[4 + i] = m.solimp[i];
    out[9] = m.margin; out[10] = m.gap; out[11] = float(m.condim);
}

int ref_shape_filter_admits(uint32_t ta, uint32_t aa, uint32_t ga, uint32_t tb, uint32_t ab, uint32_t gb) {
    return collision::ShapeFilterAdmits(ta, aa, ga, tb, ab, gb) ? 1 : 0;
}

double ref_contact_projection_roundoff(const float* start, const float* end, const float* axis) {
    return collision::ContactProjectionRoundoff({start[0], start[1], start[2]}, {end[0], end[1], end[2]},
                                                {axis[0], axis[1], axis[2]});
}

float ref_contact_query_reach(float thickness, float margin) { return collision::ContactQueryReach(thickness, margin); }
float ref_contact_motion_radius(float base, float dt, float sa, float sb, float relaxation) {
    return collision::ContactMotionRadius(base, dt, sa, sb, relaxation);
}
float ref_rigid_contact_query_margin() { return collision::kRigidContactQueryMargin; }

}  // extern "C"
