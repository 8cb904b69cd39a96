// Host side of the library above the PHI seam: the template cook, the device arena with its named env-major
// fields, the pipeline (the ordered op list of one step with its parameter PODs), the world that steps it eagerly or
// as a captured plan, and the C ABI.  Counterpart, for the articulation-step path only, of src/nk/{model,data,
// pipeline} and src/c_abi/{device,world,buffer}.cpp.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdio>
#include <cstring>
#include <exception>
#include <memory>
#include <atomic>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/nuka_hip.h"
#include "backend.h"
#include "scene_loader.h"
#include "nk_types.h"

namespace nkh {
namespace {

thread_local std::string g_last_error;   // nuka.h:42-44

nuka_result_t Error(nuka_result_t code, const std::string& message) {
    g_last_error = message;
    return code;
}

// ---- host math for the cook (runtime/articulation/articulation_state.cpp:113-165, 307-343) ---------------
void MakeSpatialInertia(float mass, const float* diag, const float* frame, float* I) {
    std::memset(I, 0, 36 * sizeof(float));
    if (mass <= 0.0f) return;
    float qw = frame[3], qx = frame[4], qy = frame[5], qz = frame[6];
    const float norm = std::sqrt(qw * qw + qx * qx + qy * qy + qz * qz);
    if (norm > 0.0f) { const float inv = 1.0f / norm; qw *= inv; qx *= inv; qy *= inv; qz *= inv; }
    const float xx = qx * qx, yy = qy * qy, zz = qz * qz, xy = qx * qy, xz = qx * qz, yz = qy * qz, wx = qw * qx, wy = qw * qy, wz = qw * qz;
    const float r[9] = {1.0f - 2.0f * (yy + zz), 2.0f * (xy - wz), 2.0f * (xz + wy), 2.0f * (xy + wz), 1.0f - 2.0f * (xx + zz),
                        2.0f * (yz - wx), 2.0f * (xz - wy), 2.0f * (yz + wx), 1.0f - 2.0f * (xx + yy)};
    const float cx = frame[0], cy = frame[1], cz = frame[2];
    const float c_dot = cx * cx + cy * cy + cz * cz;
    const float parallel[9] = {c_dot - cx * cx, -cx * cy, -cx * cz, -cy * cx, c_dot - cy * cy, -cy * cz, -cz * cx, -cz * cy, c_dot - cz * cz};
    const float cross[9] = {0.0f, -cz, cy, cz, 0.0f, -cx, -cy, cx, 0.0f};
    for (int row = 0; row < 3; ++row)
        for (int col = 0; col < 3; ++col) {
            float com = 0.0f;
            for (int k = 0; k < 3; ++k) com += r[row * 3 + k] * diag[k] * r[col * 3 + k];
            I[row * 6 + col] = com + mass * parallel[row * 3 + col];
            I[row * 6 + 3 + col] += mass * cross[row * 3 + col];
            I[(3 + row) * 6 + col] += -mass * cross[row * 3 + col];
            I[(3 + row) * 6 + 3 + col] = row == col ? mass : 0.0f;
        }
}

uint32_t JointWidth(uint8_t type) { return type <= kPrismatic ? 1u : type == kFloatingBase ? 6u : 0u; }

struct HostModel {
    ModelView counts{};   // scalar members only
    std::vector<uint8_t> joint_type, joint_limit_flags, joint_law;
    std::vector<uint32_t> parent_link, link_body, link_tree_depth, link_child_range, link_children, link_push_order, sweep_links, link_dof, dof_link, dof_component,
        link_geom_kind, body_to_link, body_to_articulation, body_collidable_link, body_collidable_body, pairable_rows;
    std::vector<uint64_t> link_dof_mask, excluded_pairs;
    std::vector<float> joint_axis, parent_offset, link_local_pose, link_inertial_frame, link_inertia, joint_damping, joint_armature,
        joint_stiffness, joint_spring_reference, joint_limit_lower, joint_limit_upper, joint_frictionloss, link_geom_local, shape_table, body_collidable_local, body_init_pose, profile_mu,
        profile_solref, profile_solimp, profile_margin, profile_mix,   // profile_mix: [profile][3] priority, solmix, condim
        joint_limit_margin, joint_limit_reference, joint_friction_reference;
    std::vector<uint32_t> profile_law;
    std::vector<float> link_mass, link_diag_inertia;   // kept for nuka_world_set_param: a new mass rebuilds the spatial inertia
};

struct NotSupported : std::runtime_error { using std::runtime_error::runtime_error; };

std::vector<float> CopyOrZero(const float* src, size_t n) {
    return src != nullptr ? std::vector<float>(src, src + n) : std::vector<float>(n, 0.0f);
}

// The cook: tree tables (fields.yaml:845-848), DoF maps (articulation_mass.cuh:64-90), spatial inertias, collidable rows
// (prims_types.cuh:27-54) and owner tables (nk/solve/collidable_owner.hpp).
void Cook(const nuka_template_desc_t& d, HostModel* out) {
    const uint32_t nl = d.link_count, nb = d.body_count;
    if (nl == 0u) throw std::invalid_argument("template has no links");
    if (!d.joint_type || !d.parent_link || !d.joint_axis || !d.link_local_pose || !d.link_inertial_frame || !d.link_mass ||
        !d.link_diag_inertia) throw std::invalid_argument("template link arrays are required");
    if (nb > 0u && (!d.body_role || !d.body_link || !d.body_local || !d.shape_kind || !d.shape_params || !d.shape_contype ||
                    !d.shape_conaffinity || !d.shape_group || !d.shape_profile)) throw std::invalid_argument("template body arrays are required");
    HostModel& m = *out;
    m.joint_type.assign(d.joint_type, d.joint_type + nl);
    m.parent_link.assign(d.parent_link, d.parent_link + nl);
    m.joint_axis.assign(d.joint_axis, d.joint_axis + 3u * nl);
    m.parent_offset = CopyOrZero(d.parent_offset, 3u * nl);
    m.link_local_pose.assign(d.link_local_pose, d.link_local_pose + 7u * nl);
    m.link_inertial_frame.assign(d.link_inertial_frame, d.link_inertial_frame + 7u * nl);
    m.joint_damping = CopyOrZero(d.joint_damping, nl);
    m.joint_armature = CopyOrZero(d.joint_armature, nl);
    m.joint_stiffness = CopyOrZero(d.joint_stiffness, nl);
    m.joint_spring_reference = CopyOrZero(d.joint_spring_reference, nl);
    m.joint_limit_lower = CopyOrZero(d.joint_limit_lower, nl);
    m.joint_limit_upper = CopyOrZero(d.joint_limit_upper, nl);
    m.joint_frictionloss = CopyOrZero(d.joint_frictionloss, nl);
    // MuJoCo-sourced joints (scene/cook/cook_to_model.cpp:662-693)
    m.joint_law = d.joint_law != nullptr ? std::vector<uint8_t>(d.joint_law, d.joint_law + nl) : std::vector<uint8_t>(nl, 0u);
    m.joint_limit_margin = CopyOrZero(d.joint_limit_margin, nl);
    {
        const float reference[7] = {0.02f, 1.0f, 0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
        m.joint_limit_reference.resize(7u * nl); m.joint_friction_reference.resize(7u * nl);
        for (uint32_t l = 0u; l < nl; ++l)
            for (uint32_t k = 0u; k < 7u; ++k) {
                m.joint_limit_reference[7u * l + k] = d.joint_limit_reference != nullptr ? d.joint_limit_reference[7u * l + k] : reference[k];
                m.joint_friction_reference[7u * l + k] = d.joint_friction_reference != nullptr ? d.joint_friction_reference[7u * l + k] : reference[k];
                if (!std::isfinite(m.joint_limit_reference[7u * l + k]) || !std::isfinite(m.joint_friction_reference[7u * l + k]))
                    throw std::invalid_argument("invalid joint solref or solimp");
            }
        for (uint32_t l = 0u; l < nl; ++l)
            if (m.joint_law[l] > 1u || !std::isfinite(m.joint_limit_margin[l])) throw std::invalid_argument("invalid joint law or limit margin");
    }
    m.joint_limit_flags = d.joint_limit_flags != nullptr ? std::vector<uint8_t>(d.joint_limit_flags, d.joint_limit_flags + nl) : std::vector<uint8_t>(nl, 0u);
    m.link_inertia.resize(36u * nl);
    m.link_mass.assign(d.link_mass, d.link_mass + nl);
    m.link_diag_inertia.assign(d.link_diag_inertia, d.link_diag_inertia + 3u * nl);
    m.link_dof.resize(nl);
    m.link_body.assign(nl, kInvalid);
    m.link_geom_kind.assign(nl, 0u);
    m.link_geom_local.resize(7u * nl);
    uint32_t nv = 0u;
    for (uint32_t l = 0u; l < nl; ++l) {
        const uint8_t type = m.joint_type[l];
        if (type > kFloatingBase) throw std::invalid_argument("joint type not supported on this path");
        if (type == kFloatingBase && (l != 0u || m.parent_link[l] != kInvalid)) throw std::invalid_argument("a floating base must be link 0");
        if (m.parent_link[l] != kInvalid && m.parent_link[l] >= l) throw std::invalid_argument("parents must precede children");
        if (l > 0u && m.parent_link[l] == kInvalid) throw std::invalid_argument("one articulation (one root) per environment");
        MakeSpatialInertia(d.link_mass[l], d.link_diag_inertia + 3u * l, d.link_inertial_frame + 7u * l, m.link_inertia.data() + 36u * l);
        m.link_dof[l] = nv;
        nv += JointWidth(type);
        const float id[7] = {0, 0, 0, 1, 0, 0, 0};
        std::memcpy(m.link_geom_local.data() + 7u * l, id, sizeof(id));
    }
    if (nv == 0u || nv > kMaxDof) throw std::invalid_argument("articulation DoF must be in 1..64");
    m.dof_link.resize(nv);
    m.dof_component.resize(nv);
    m.link_dof_mask.assign(nl, 0ull);
    m.link_tree_depth.resize(nl);
    uint32_t max_depth = 0u;
    for (uint32_t l = 0u; l < nl; ++l) {
        const uint32_t width = JointWidth(m.joint_type[l]);
        uint64_t own = 0ull;
        for (uint32_t c = 0u; c < width; ++c) {
            m.dof_link[m.link_dof[l] + c] = l;
            m.dof_component[m.link_dof[l] + c] = width == 1u ? kInvalid : c;
            own |= 1ull << (m.link_dof[l] + c);
        }
        const uint32_t parent = m.parent_link[l];
        m.link_dof_mask[l] = own | (parent == kInvalid ? 0ull : m.link_dof_mask[parent]);
        m.link_tree_depth[l] = parent == kInvalid ? 0u : m.link_tree_depth[parent] + 1u;
        max_depth = std::max(max_depth, m.link_tree_depth[l]);
    }
    m.link_child_range.resize(2u * nl);
    m.link_children.clear();
    for (uint32_t l = 0u; l < nl; ++l) {
        m.link_child_range[2u * l] = uint32_t(m.link_children.size());
        for (uint32_t c = 0u; c < nl; ++c) if (m.parent_link[c] == l) m.link_children.push_back(c);
        m.link_child_range[2u * l + 1u] = uint32_t(m.link_children.size());
    }
    m.link_children.resize(nl, 0u);
    // the composite-inertia pass adds every child to its parent, deepest parents first, parents of one depth in link
    // order, a parent's children in list order: that visiting order as one list (ended by kInvalid)
    m.link_push_order.clear();
    for (uint32_t depth = max_depth; depth > 0u; --depth)
        for (uint32_t l = 0u; l < nl; ++l) {
            if (m.link_tree_depth[l] + 1u != depth) continue;
            for (uint32_t i = m.link_child_range[2u * l]; i < m.link_child_range[2u * l + 1u]; ++i) m.link_push_order.push_back(m.link_children[i]);
        }
    m.link_push_order.resize(nl, kInvalid);
    // the dynamics' tree sweeps: the links of one depth, ten a pass (a pass that ends early is filled with kInvalid)
    m.sweep_links.clear();
    for (uint32_t depth = 0u; depth <= max_depth; ++depth) {
        uint32_t in_pass = 0u;
        for (uint32_t l = 0u; l < nl; ++l) {
            if (m.link_tree_depth[l] != depth) continue;
            m.sweep_links.push_back(l);
            in_pass = (in_pass + 1u) % kSweepLinks;
        }
        while (in_pass != 0u) { m.sweep_links.push_back(kInvalid); in_pass = (in_pass + 1u) % kSweepLinks; }
    }
    m.counts.sweep_passes = uint32_t(m.sweep_links.size() / kSweepLinks);
    m.shape_table.assign(size_t{nb} * kShapeStride, 0.0f);
    m.body_to_link.assign(nb, kInvalid);
    m.body_to_articulation.assign(nb, kInvalid);
    m.body_collidable_link.assign(nb, kInvalid);
    m.body_collidable_body.assign(nb, kInvalid);
    m.body_collidable_local.resize(size_t{nb} * 7u);
    m.body_init_pose.resize(size_t{nb} * 7u);
    m.profile_mu.assign(d.profile_mu, d.profile_mu + 2u * d.profile_count);
    // the MuJoCo-law terms of each profile, at the defaults of ContactParamsIn (scene/contact_filter.hpp:20-37) where not authored
    m.profile_law.assign(d.profile_count, 0u);
    m.profile_solref.resize(2u * d.profile_count); m.profile_solimp.resize(5u * d.profile_count); m.profile_margin.assign(2u * d.profile_count, 0.0f);
    {
        const float solimp[5] = {0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
        for (uint32_t i = 0u; i < d.profile_count; ++i) {
            if (d.profile_law != nullptr) m.profile_law[i] = d.profile_law[i];
            m.profile_solref[2u * i] = d.profile_solref != nullptr ? d.profile_solref[2u * i] : 0.02f;
            m.profile_solref[2u * i + 1u] = d.profile_solref != nullptr ? d.profile_solref[2u * i + 1u] : 1.0f;
            for (uint32_t k = 0u; k < 5u; ++k) m.profile_solimp[5u * i + k] = d.profile_solimp != nullptr ? d.profile_solimp[5u * i + k] : solimp[k];
            for (uint32_t k = 0u; k < 2u; ++k) if (d.profile_margin != nullptr) m.profile_margin[2u * i + k] = d.profile_margin[2u * i + k];
            m.profile_mix.push_back(d.profile_priority != nullptr ? float(d.profile_priority[i]) : 0.0f);
            m.profile_mix.push_back(d.profile_solmix != nullptr ? d.profile_solmix[i] : 1.0f);
            m.profile_mix.push_back(d.profile_condim != nullptr ? float(d.profile_condim[i]) : 3.0f);
            if (d.profile_condim != nullptr && d.profile_condim[i] != 1u && d.profile_condim[i] != 3u)
                throw NotSupported("contact dimensions other than 1 and 3 (torsional and rolling friction) are not built on this path");
            if (!std::isfinite(m.profile_mix[3u * i + 1u]) || std::fabs(m.profile_mix[3u * i]) > 16777216.0f) throw std::invalid_argument("invalid profile solmix or priority");
            if (m.profile_law[i] > 1u) throw std::invalid_argument("unknown profile law");
            for (uint32_t k = 0u; k < 2u; ++k) if (!std::isfinite(m.profile_solref[2u * i + k]) || !std::isfinite(m.profile_margin[2u * i + k])) throw std::invalid_argument("invalid profile solref or margin");
            for (uint32_t k = 0u; k < 5u; ++k) if (!std::isfinite(m.profile_solimp[5u * i + k])) throw std::invalid_argument("invalid profile solimp");
        }
    }
    auto bits = [](uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; };
    for (uint32_t b = 0u; b < nb; ++b) {
        const uint32_t role = d.body_role[b], link = d.body_link[b];
        float* row = m.shape_table.data() + size_t{b} * kShapeStride;
        row[0] = bits(d.shape_kind[b]);
        for (int k = 0; k < 4; ++k) row[1 + k] = d.shape_params[4u * b + k];
        row[5] = bits(d.shape_contype[b]); row[6] = bits(d.shape_conaffinity[b]); row[7] = bits(0u);
        row[8] = bits(role == 0u ? 0xFFFFFFFFu : b); row[9] = bits(d.shape_group[b]);
        row[10] = bits(0u); row[11] = bits(0u); row[12] = bits(d.shape_profile[b]);
        const float id[7] = {0, 0, 0, 1, 0, 0, 0};
        std::memcpy(m.body_collidable_local.data() + 7u * b, id, sizeof(id));
        std::memcpy(m.body_init_pose.data() + 7u * b, id, sizeof(id));
        if (role == 0u) std::memcpy(m.body_init_pose.data() + 7u * b, d.body_local + 7u * b, 7u * sizeof(float));
        else if (role == 1u) {
            if (link >= nl || m.link_body[link] != kInvalid) throw std::invalid_argument("each link owns at most one body row");
            m.link_body[link] = b; m.body_to_link[b] = link; m.body_to_articulation[b] = 0u;
            std::memcpy(m.link_geom_local.data() + 7u * link, d.body_local + 7u * b, 7u * sizeof(float));
            m.link_geom_kind[link] = d.shape_kind[b] != kInvalid ? 1u : 0u;
        } else if (role != 2u) throw std::invalid_argument("unknown collidable role");
    }
    for (uint32_t b = 0u; b < nb; ++b) {
        if (d.body_role[b] != 2u) continue;
        const uint32_t link = d.body_link[b];
        if (link >= nl || m.link_body[link] == kInvalid) throw std::invalid_argument("an extra collidable needs its link's body row");
        m.body_collidable_link[b] = link;
        m.body_collidable_body[b] = m.link_body[link];
        std::memcpy(m.body_collidable_local.data() + 7u * b, d.body_local + 7u * b, 7u * sizeof(float));
    }
    // Excluded pairs (scene/cook/cook_to_model.cpp:1468-1490): the authored ones and every two rows of one link, as
    // sorted (a << 32 | b) keys with a < b.
    m.excluded_pairs.clear();
    if (d.excluded_pairs != nullptr)
        for (uint32_t k = 0u; k < d.excluded_pair_count; ++k) {
            const uint32_t a = d.excluded_pairs[2u * k], b = d.excluded_pairs[2u * k + 1u];
            if (a >= nb || b >= nb || a == b) throw std::invalid_argument("excluded pair names no two collidable rows");
            m.excluded_pairs.push_back((uint64_t{std::min(a, b)} << 32u) | uint64_t{std::max(a, b)});
        }
    for (uint32_t i = 0u; i < nb; ++i)
        for (uint32_t j = i + 1u; j < nb; ++j)
            if (d.body_role[i] != 0u && d.body_role[j] != 0u && d.body_link[i] == d.body_link[j])
                m.excluded_pairs.push_back((uint64_t{i} << 32u) | uint64_t{j});
    std::sort(m.excluded_pairs.begin(), m.excluded_pairs.end());
    m.excluded_pairs.erase(std::unique(m.excluded_pairs.begin(), m.excluded_pairs.end()), m.excluded_pairs.end());
    // Manifolds built here: the analytic pairs of the reference's PrimitivePair (collision/analytical_manifold.hpp:934-971).  Any other admitted pair is refused at cook time instead of
    // silently producing no contact.
    const auto points_of = [](uint32_t ka, uint32_t kb) -> uint32_t {   // most points of the pair's manifold, 0 for none
        if (ka > kb) std::swap(ka, kb);
        if (kb == kShapePlane) return ka == kShapeSphere ? 1u : ka == kShapeCapsule ? 2u : ka == kShapeBox ? 4u : 0u;
        if (kb == kShapeCylinder) return ka == kShapeSphere ? 1u : ka == kShapePlane ? 4u : 0u;
        if (ka == kShapeSphere) return kb <= kShapeBox ? 1u : 0u;                      // sphere x sphere, capsule, box
        if (ka == kShapeBox && kb == kShapeBox) return 4u;
        return ka == kShapeCapsule && kb == kShapeCapsule ? 1u : 0u;
    };
    uint32_t admitted = 0u, max_points = 1u;
    bool link_pairs = false;   // some admitted pair joins the shapes of two links
    for (uint32_t i = 0u; i < nb; ++i) {
        const uint32_t kind = d.shape_kind[i];
        if (kind != kInvalid && kind != kShapeSphere && kind != kShapeCapsule && kind != kShapeBox && kind != kShapePlane && kind != kShapeCylinder)
            throw NotSupported("shape kind not supported on this path (sphere, capsule, box, plane, cylinder)");
        if ((kind == kShapeSphere || kind == kShapeCapsule || kind == kShapeCylinder) && !(d.shape_params[4u * i] >= 0.0f))
            throw std::invalid_argument("negative shape radius");
        if ((kind == kShapeCapsule || kind == kShapeCylinder) && !(d.shape_params[4u * i + 1u] >= 0.0f))
            throw std::invalid_argument("negative shape half length");
        for (uint32_t j = i + 1u; j < nb; ++j) {
            if (d.body_role[i] == 0u && d.body_role[j] == 0u) continue;
            if (kind == kInvalid || d.shape_kind[j] == kInvalid) continue;
            if (((d.shape_contype[i] & d.shape_conaffinity[j]) | (d.shape_contype[j] & d.shape_conaffinity[i])) == 0u) continue;
            const int32_t ga = int32_t(d.shape_group[i]), gb = int32_t(d.shape_group[j]);   // shape_kind.hpp:26-33
            if (ga != 0 && gb != 0 && (ga > 0 ? ga != gb && gb > 0 : ga == gb)) continue;
            if (std::binary_search(m.excluded_pairs.begin(), m.excluded_pairs.end(), (uint64_t{i} << 32u) | uint64_t{j})) continue;
            const uint32_t points = points_of(kind, d.shape_kind[j]);
            if (points == 0u) throw NotSupported("admitted collidable pair has no analytic manifold (capsule or cylinder against box, capsule x cylinder, cylinder x cylinder)");
            max_points = std::max(max_points, points);
            ++admitted;
            if (d.body_role[i] != 0u && d.body_role[j] != 0u) link_pairs = true;
        }
    }
    const uint32_t slots = d.max_contacts_per_env != 0u ? d.max_contacts_per_env : admitted;
    ModelView& c = m.counts;
    c.links_per_env = nl; c.bodies_per_env = nb; c.dof = nv; c.max_dof = nv; c.max_depth = max_depth;
    c.contact_slots = slots;
    c.contact_rows_per_env = slots * kPointsPerSlot * kRowsPerPoint;   // nk_row.hpp:59-63
    // joint row slots (scene/cook/cook_to_model.cpp:696-719; nk/pipeline/world.cpp:61, 96)
    bool any_limit = false, any_friction = false;
    for (uint32_t l = 0u; l < nl; ++l) {
        const uint8_t flags = m.joint_limit_flags[l];
        if (((flags & 1u) != 0u && !std::isfinite(m.joint_limit_lower[l])) || ((flags & 2u) != 0u && !std::isfinite(m.joint_limit_upper[l])) ||
            ((flags & 3u) == 3u && m.joint_limit_lower[l] > m.joint_limit_upper[l])) throw std::invalid_argument("invalid authored joint limit");
        if (!std::isfinite(m.joint_frictionloss[l]) || m.joint_frictionloss[l] < 0.0f) throw std::invalid_argument("invalid joint frictionloss");
        any_limit = any_limit || flags != 0u;
        any_friction = any_friction || m.joint_frictionloss[l] > 0.0f;
    }
    if (d.drive_rows != 0u && (d.drive_mode == kDriveComputedTorque || d.drive_mode == kDriveOsc))
        throw NotSupported("inverse-dynamics drive modes are not built on this path");
    if (d.drive_rows != 0u && d.drive_mode > kDriveActuator) throw std::invalid_argument("unknown drive mode");
    c.joint_limit_rows = any_limit ? nl * 2u : 0u;
    c.joint_friction_rows = any_friction ? nl : 0u;
    c.joint_drive_rows = d.drive_rows != 0u ? nl : 0u;
    c.drive_mode = d.drive_rows != 0u ? d.drive_mode : uint32_t(kDriveTorque);
    c.rows_per_env = c.contact_rows_per_env + c.joint_limit_rows + c.joint_friction_rows + c.joint_drive_rows;
    c.profile_count = d.profile_count;
    c.any_mujoco = 0u;
    for (uint32_t law : m.profile_law) if (law == 1u) c.any_mujoco = 1u;
    for (uint8_t law : m.joint_law) if (law == 1u) c.any_mujoco = 1u;
    if (d.integrator > 2u) throw std::invalid_argument("unknown integrator");
    c.integrator = d.integrator;
    if (d.contact_cone > 1u) throw std::invalid_argument("unknown contact cone");
    c.contact_cone = d.contact_cone;
    c.contact_impratio = d.contact_impratio > 0.0f ? d.contact_impratio : 1.0f;
    c.floating_root = m.joint_type[0] == kFloatingBase ? 1u : 0u;
    // a free rigid body: the template's one link, stepped by the rigid-body ops
    c.free_body = d.struct_size >= sizeof(nuka_template_desc_t) && d.free_body != 0u ? 1u : 0u;
    if (c.free_body != 0u) {
        if (nl != 1u || c.floating_root == 0u) throw std::invalid_argument("a free body is a template of one link with a floating root");
        if (c.joint_limit_rows + c.joint_friction_rows + c.joint_drive_rows != 0u || c.integrator != 0u)
            throw std::invalid_argument("a free body has no joint rows, drives or joint integrator");
        if (m.link_body[0] == kInvalid) throw std::invalid_argument("a free body needs its own body row: its state lives there");
        if (!(d.link_mass[0] > 0.0f) || !std::isfinite(d.link_mass[0])) throw std::invalid_argument("a free body needs a positive mass");
        for (uint32_t k = 0u; k < 3u; ++k)
            if (!(d.link_diag_inertia[k] > 0.0f) || !std::isfinite(d.link_diag_inertia[k])) throw std::invalid_argument("a free body needs positive principal moments");
    }
    c.max_points_per_slot = max_points;
    // the coordinates a contact can act on: those on the way to the root from a link that carries a shape that can pair
    c.contact_dof_end = 0u;
    for (uint32_t b = 0u; b < nb; ++b) {
        if (d.body_role[b] == 0u || d.shape_kind[b] == kInvalid || d.body_link[b] >= nl) continue;
        const uint64_t mask = m.link_dof_mask[d.body_link[b]];
        for (uint32_t k = 0u; k < nv; ++k) if ((mask >> k) & 1ull) c.contact_dof_end = std::max(c.contact_dof_end, k + 1u);
    }
    c.rows_from_links = link_pairs ? 0u : 1u;
    for (uint32_t l = 0u; l < nl; ++l) {
        const uint8_t type = m.joint_type[l];
        if (!(type == kRevolute || type == kPrismatic || type == kFixed || (type == kFloatingBase && l == 0u))) c.rows_from_links = 0u;
    }
    c.excluded_pair_count = uint32_t(m.excluded_pairs.size());
    // rows whose type and affinity masks are both empty pass the filter with no partner (shape_kind.hpp:26-33): the pair
    // query walks the grid of the other rows only, in the same ascending order
    m.pairable_rows.clear();
    for (uint32_t b = 0u; b < nb; ++b) if ((d.shape_contype[b] | d.shape_conaffinity[b]) != 0u) m.pairable_rows.push_back(b);
    c.pairable_count = uint32_t(m.pairable_rows.size());
    m.pairable_rows.resize(nb, kInvalid);
}

enum Dtype : uint8_t { kF32 = 0, kU32 = 1, kU64 = 2, kU8 = 3 };
struct Field { const char* name; Dtype dtype; uint32_t elem_bytes; size_t count; size_t offset; bool is_template; };

#define NKH_DATA_FIELDS(X) \
    X(q, kF32, E * nl) X(qdot, kF32, E * nl) X(qddot, kF32, E * nl) X(tau, kF32, E * nl) X(base_pose, kF32, E * 7) \
    X(link_pose, kF32, E * nl * 7) X(link_velocity, kF32, E * nl * 6) X(link_acceleration, kF32, E * nl * 6) \
    X(link_wrench, kF32, E * nl * 6) X(articulation_bias, kF32, E * md) X(articulation_qdd, kF32, E * md) \
    X(m, kF32, E * md * md) X(m_factor, kF32, E * md * md) X(qdot_flat, kF32, E * md) X(qdot_pseudo, kF32, E * nl) \
    X(link_velocity_pseudo, kF32, E * nl * 6) X(body_pose, kF32, E * nb * 7) X(body_aabb_lo, kF32, E * nb * 3) \
    X(body_aabb_hi, kF32, E * nb * 3) X(candidate_pairs, kU32, E * S * 2) X(pair_count, kU32, E) X(ucontact_count, kU32, E * S) \
    X(ucontact_a, kU32, E * S * 4) X(ucontact_b, kU32, E * S * 4) X(ucontact_law, kU32, E * S) \
    X(ucontact_row_range, kU32, E * S * 2) X(ucontact_point, kF32, E * S * 12) X(ucontact_normal, kF32, E * S * 12) \
    X(ucontact_depth, kF32, E * S * 4) X(ucontact_id_pair, kU64, E * S * 4) X(ucontact_id_feature, kU64, E * S * 4) \
    X(urows, kF32, E * R * 26) X(lambda, kF32, E * R) X(row_penetration, kF32, E * R) X(row_cj_point, kF32, E * R * 3) \
    X(row_cj_point_b, kF32, E * R * 3) X(chain_jacobian, kF32, E * R * md) X(chain_jacobian_b, kF32, E * R * md) \
    X(row_cj_link, kU32, E * R) X(row_cj_link_b, kU32, E * R) X(row_count, kU32, E) X(contact_count, kU32, E) \
    X(contact_row_extent, kU32, E * 2) X(env_status, kU32, E) X(vbd_velocity_sweep_count, kU32, E) \
    X(solver_residual, kF32, E * 4) X(solver_penalty, kF32, E * R) X(solver_velocity, kF32, E * md) X(solver_free, kF32, E * md) \
    X(solver_cost, kU32, E) X(tile_order, kU32, E) X(row_unit, kU32, E * R) X(row_unit_value, kF32, E * R) \
    X(solver_mass_factor, kF32, E * mf) \
    X(body_invweight0, kF32, E * nb * 2) X(dof_invweight0, kF32, E * md) X(row_invweight, kF32, E * R) \
    X(row_reference_velocity_gain, kF32, E * R) X(step_qdot_flat, kF32, E * md) \
    X(contact_material, kU64, E * S) X(contact_cache_pair, kU64, E * S * 4) X(contact_cache_feature, kU64, E * S * 4) \
    X(contact_cache_material, kU64, E * S * 4) X(contact_cache_lambda, kF32, E * S * 16) X(contact_cache_normal, kF32, E * S * 12) \
    X(contact_cache_age, kU32, E * S * 4) X(contact_cache_current_owner, kU32, E * S * 4) X(contact_cache_old_keep, kU32, E * S * 4) \
    X(contact_cache_extent, kU32, E * 2) X(contact_warm_start_counts, kU32, E * 2) X(contact_cache_match, kU32, E * S * 4) \
    X(reset_env_ids, kU32, E) \
    X(drive_target, kF32, E * nl) X(drive_stiffness, kF32, E * nl) X(drive_damping, kF32, E * nl) X(drive_force_limit, kF32, E * nl) \
    X(drive_joint_force_limit, kF32, E * nl) X(velocity_target, kF32, E * nl) X(actuator_noload_speed, kF32, E * nl) \
    X(joint_f, kF32, E * nl) X(joint_gravity_force, kF32, E * nl) X(drive_command, kF32, E * nl) X(drive_dissipation, kF32, E * nl) \
    X(drive_lower, kF32, E * nl) X(drive_upper, kF32, E * nl) X(joint_limit_impulse, kF32, E * nl * 2) \
    X(actuator_effort_requested, kF32, E * nl) X(actuator_effort, kF32, E * nl) X(actuator_saturated, kF32, E * nl) \
    X(contact_point, kF32, E * S * 3) X(contact_normal, kF32, E * S * 3) X(contact_force, kF32, E * S * 3) \
    X(ucontact_impulse, kF32, E * S * 12) X(link_contact_wrench, kF32, E * nl * 6) X(contact_side_a_kind, kU32, E * S) \
    X(contact_side_b_kind, kU32, E * S) X(contact_side_a_index, kU32, E * S) X(contact_side_b_index, kU32, E * S) \
    X(contact_link, kU32, E * S) \
    X(step_env_status, kU32, E) X(step_link_impulse, kF32, E * nl * 3) X(step_link_moment, kF32, E * nl * 3) \
    X(step_joint_limit_impulse, kF32, E * nl * 2) \
    X(body_linear_velocity, kF32, E * fb * 3) X(body_angular_velocity, kF32, E * fb * 3) X(body_world_inv_inertia, kF32, E * fb * 6) \
    X(body_gyro_residual, kF32, E * fb) X(body_gyro_iterations, kU32, E * fb) X(body_gyro_status, kU32, E * fb) \
    X(body_inv_mass, kF32, E * fb) X(body_inv_inertia, kF32, E * fb * 3) X(body_inertial_frame, kF32, E * fb * 7)

#define NKH_MODEL_FIELDS(X) \
    X(joint_type, kU8) X(parent_link, kU32) X(joint_axis, kF32) X(parent_offset, kF32) X(link_local_pose, kF32) \
    X(link_inertial_frame, kF32) X(link_inertia, kF32) X(joint_damping, kF32) X(joint_armature, kF32) X(joint_stiffness, kF32) \
    X(joint_spring_reference, kF32) X(joint_limit_lower, kF32) X(joint_limit_upper, kF32) X(joint_frictionloss, kF32) \
    X(joint_limit_flags, kU8) X(joint_law, kU8) X(joint_limit_margin, kF32) X(joint_limit_reference, kF32) \
    X(joint_friction_reference, kF32) X(link_body, kU32) X(link_tree_depth, kU32) X(link_child_range, kU32) X(link_children, kU32) X(link_push_order, kU32) X(sweep_links, kU32) \
    X(link_dof, kU32) X(dof_link, kU32) X(dof_component, kU32) X(link_dof_mask, kU64) X(link_geom_kind, kU32) \
    X(link_geom_local, kF32) X(shape_table, kF32) X(body_to_link, kU32) X(body_to_articulation, kU32) \
    X(body_collidable_link, kU32) X(body_collidable_body, kU32) X(body_collidable_local, kF32) X(pairable_rows, kU32) X(profile_mu, kF32) \
    X(profile_law, kU32) X(profile_solref, kF32) X(profile_solimp, kF32) X(profile_margin, kF32) X(profile_mix, kF32) \
    X(excluded_pairs, kU64)

uint32_t DtypeBytes(Dtype t) { return t == kU64 ? 8u : t == kU8 ? 1u : 4u; }

struct DeviceRecord {   // src/c_abi/internal.hpp:57-69
    void* backend = nullptr;
    int gpu_index = 0;
};

struct World {   // src/c_abi/internal.hpp:153-165 WorldRecord + nk::World
    DeviceRecord* device = nullptr;
    uint64_t id = 0u;   // creation number, unique in the process
    nuka_phi_backend* backend = nullptr;
    const nuka_phi_backend_i* be = nullptr;
    HostModel host;
    nuka_hip_world_desc_t cfg{};
    uint32_t env_count = 0u;
    nuka_phi_buffer* arena = nullptr;
    nuka_phi_buffer* initial = nullptr;   // the state after creation, for nuka_world_reset
    size_t arena_bytes = 0u;
    std::vector<Field> fields;
    ModelView model{};
    DataView data{};
    // the pipeline: ops in step order with their parameter PODs (src/nk/pipeline/pipeline.cpp:187-1020)
    std::vector<nuka_phi_op_call> calls;
    FkWorldPosesParams p_fk{};
    FkLinkVelocitiesParams p_fk_velocity{};
    ApplyDrivesParams p_drives{};
    ReadoutDrivesParams p_readout_drives{};
    ReadoutContactWrenchParams p_readout_contacts{};
    bool contact_readout_demanded = false;   // nk/pipeline/pipeline.hpp:60 kReadoutContactWrench
    ArticulationDynamicsParams p_dynamics{}, p_dynamics_probe{};
    IntegrateVelocityParams p_int_vel{};
    IntegratePositionParams p_int_pos{};
    SyncLinkBodyPoseParams p_sync{};
    BuildAabbsParams p_aabbs{};
    LbvhBuildParams p_lbvh{};
    LbvhQueryPairsParams p_query{};
    NarrowphasePrimitivesParams p_narrow{};
    AssembleRowsParams p_assemble{};
    ContactWarmStartParams p_warm0{}, p_warm1{};
    BlockDescentSolveParams p_solve{};
    SnapshotStepVelocityParams p_snapshot{};
    ArticulationDampingParams p_damping{};
    ReferenceWeightsParams p_reference_weights{};   // dispatched at creation, outside the step (nk/pipeline/world.cpp:553-561)
    NarrowphaseHeightfieldParams p_heightfield{};
    std::vector<AccumulateStepParams> p_accumulate;   // one per substep (pipeline.cpp:128-152)
    nuka_execution_mode_t mode = NUKA_EXECUTION_EAGER;
    nuka_phi_plan* plan = nullptr;
    std::vector<float> drive_stiffness, drive_force_limit;   // per template link: what nuka_world_get_param reports
    uint64_t capture_attempts = 0u, graph_replays = 0u;      // nuka_world_get_execution_info
    uint64_t param_version = 0u;   // counts the calls that may have changed a live parameter: a checkpoint taken at the current count holds the current values
    bool from_scene = false;                            // created from a scene file: the names below are the file's
    std::vector<std::string> link_names, joint_names;   // per template link; a joint's name sits at its child link
    nuka_phi_execution_error last_error{};

    ~World() {
        if (be != nullptr && plan != nullptr) be->plan_free(backend, plan);
        if (arena != nullptr) reinterpret_cast<nuka_phi_buffer_head*>(arena)->iface->free(arena);
        if (initial != nullptr) reinterpret_cast<nuka_phi_buffer_head*>(initial)->iface->free(initial);
    }
};

// Checkpoint of the persistent physics (src/include/nuka/nuka.h:388-392): the fields the reference keeps in its
// persistent arena (fields.yaml: q, qdot, qddot, tau, base_pose, link_pose, link_velocity, body_pose, lambda and the
// contact cache) plus the applied link wrench.  Everything else is per-step scratch; a restore puts the scratch a
// step reads before writing into its cleared state - row and cache extents of zero make the next assembly clear
// every row, carried solver velocities of zero start the solve from the free velocity, status words are cleared -
// the lifecycle of a reset (op_schema.hpp:936 RestoreStateParams).
constexpr uint32_t kMaxCheckpointSegments = 64u;
struct CheckpointSegments {
    uint32_t count;
    uint32_t units[kMaxCheckpointSegments];          // 16-byte units
    char* live[kMaxCheckpointSegments];
    char* kept[kMaxCheckpointSegments];
};
// What nuka_world_set_param can change after creation (src/c_abi/checkpoint.cpp:18-24 keeps link_inertia and
// joint_armature beside the state; here every live parameter), in the order of the parameter table: a few words a link,
// held on the host.
struct LiveParams {
    std::vector<double> values;   // [parameter][element], flattened
    bool operator==(const LiveParams& o) const { return values == o.values; }
};
struct Checkpoint {
    World* owner = nullptr;
    uint64_t owner_id = 0u;        // the world's creation number: a destroyed world's address may be used again
    uint64_t layout_hash = 0u;     // of the owner, taken at capture
    nuka_phi_buffer* store = nullptr;
    CheckpointSegments segments{};
    uint64_t bytes = 0u;
    LiveParams params;
    uint64_t param_version = ~0ull;   // the owner's count when `params` was last known to equal its live parameters
};
bool OwnedBy(const Checkpoint* cp, const World* w) { return cp->owner == w && cp->owner_id == w->id; }

// blockIdx.y picks the segment, blockIdx.x strides over its 16-byte units.
__global__ void __launch_bounds__(256) CheckpointCopyKernel(CheckpointSegments s, uint32_t restore) {
    const uint32_t seg = blockIdx.y;
    if (s.kept[seg] == nullptr) {   // a scratch field a restore clears; a capture leaves it alone
        if (restore == 0u) return;
        uint4* cleared = reinterpret_cast<uint4*>(s.live[seg]);
        for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < s.units[seg]; i += gridDim.x * blockDim.x) cleared[i] = uint4{0u, 0u, 0u, 0u};
        return;
    }
    const uint4* src = reinterpret_cast<const uint4*>(restore != 0u ? s.kept[seg] : s.live[seg]);
    uint4* dst = reinterpret_cast<uint4*>(restore != 0u ? s.live[seg] : s.kept[seg]);
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < s.units[seg]; i += gridDim.x * blockDim.x) dst[i] = src[i];
}

// ResetEnvs (op_schema.hpp:904-926): the selected environments get their slice of every persistent field back from
// the snapshot taken at creation, and their per-step history cleared.  blockIdx.x = selected environment,
// blockIdx.y = field; words of four bytes, since an environment's slice of a field need not be 16-byte aligned.
struct ResetSegments {
    uint32_t count;
    uint32_t words_per_env[kMaxCheckpointSegments];
    uint32_t* live[kMaxCheckpointSegments];
    const uint32_t* initial[kMaxCheckpointSegments];   // null: clear
};
__global__ void __launch_bounds__(256) ResetEnvsKernel(ResetSegments s, const uint32_t* ids, uint32_t env_count) {
    const uint32_t env = ids[blockIdx.x], seg = blockIdx.y;
    if (env >= env_count) return;
    const size_t first = size_t{env} * s.words_per_env[seg];
    for (uint32_t i = threadIdx.x; i < s.words_per_env[seg]; i += blockDim.x)
        s.live[seg][first + i] = s.initial[seg] != nullptr ? s.initial[seg][first + i] : 0u;
}

// Staging of nuka_world_reset_envs_static: the environment ids of one call.  A file-scope device array, so the call
// takes no device memory of its own; every GPU the library runs on holds its own copy, at its own address, until the
// process ends.  In host code the array's name is only a stand-in: its device address on a GPU is asked for once, with
// that GPU current, when a device handle is created there, and kept in g_static_reset_ids.
constexpr int kMaxGpus = 64;
static __device__ __align__(256) uint32_t scratch[NUKA_RESET_ENVS_STATIC_MAX];
uint32_t* g_static_reset_ids[kMaxGpus] = {};
uint32_t g_static_reset_host[NUKA_RESET_ENVS_STATIC_MAX];   // the sorted, deduplicated ids of the call in flight
std::mutex g_static_reset_mutex;                            // guards the host staging above

bool CheckpointKeeps(const char* name) {
    for (const char* kept : {"q", "qdot", "qddot", "tau", "base_pose", "link_pose", "link_velocity", "body_pose", "lambda", "link_wrench",
                             "body_linear_velocity", "body_angular_velocity",
                             "drive_target", "drive_stiffness", "drive_damping", "drive_force_limit", "drive_joint_force_limit",
                             "velocity_target", "actuator_noload_speed",
                             "contact_cache_pair", "contact_cache_feature", "contact_cache_material", "contact_cache_lambda",
                             "contact_cache_normal", "contact_cache_age"})
        if (std::strcmp(name, kept) == 0) return true;
    return false;
}
bool CheckpointClears(const char* name) {
    for (const char* cleared : {"contact_row_extent", "contact_cache_extent", "solver_velocity", "solver_free", "env_status"})
        if (std::strcmp(name, cleared) == 0) return true;
    return false;
}

const nuka_phi_buffer_i* Iface(nuka_phi_buffer* b) { return reinterpret_cast<nuka_phi_buffer_head*>(b)->iface; }

void BuildPipeline(World& w) {
    const ModelView& m = w.model;
    const uint32_t E = w.env_count, nl = m.links_per_env, nb = m.bodies_per_env;
    const nuka_hip_world_desc_t& cfg = w.cfg;
    const bool has_contacts = m.rows_per_env > 0u;
    // A step of several substeps runs the interval below that many times at dt / substeps (pipeline.cpp:63-69).
    const uint32_t substeps = std::max(1u, cfg.solver_substeps);
    const float dt = cfg.fixed_dt / float(substeps);
    const float contact_margin = cfg.solver_contact_margin;
    const float query_reach = std::fmax(0.02f, 2.0f * (2.0f * 0.0f + contact_margin));   // contact_query.hpp:20-22
    w.p_fk = {};
    w.p_fk.articulation_count = E; w.p_fk.total_link_count = E * nl; w.p_fk.articulations_per_env = 1u;
    w.p_fk_velocity = {E, E * nl};
    w.p_drives = {};
    w.p_drives.dt = dt; w.p_drives.total_link_count = E * nl; w.p_drives.links_per_env = nl;
    w.p_drives.mode = m.drive_mode; w.p_drives.articulation_count = E; w.p_drives.bodies_per_env = nb;
    const bool drives = m.joint_drive_rows > 0u;
    // pipeline.cpp:380-381; a MuJoCo integrator keeps the damping explicit in the solve and applies it afterwards (:264-265)
    const bool fold = drives && cfg.solver_fold_drive_damping != 0xFFFFFFFFu && m.integrator == 0u;
    w.p_drives.defer_velocity_damping = fold ? 1u : 0u;
    std::memcpy(w.p_drives.gravity, cfg.gravity, sizeof(cfg.gravity));
    w.p_readout_drives = {dt, E * nl, nl, m.rows_per_env, m.contact_rows_per_env + m.joint_limit_rows + m.joint_friction_rows};
    ArticulationDynamicsParams& dyn = w.p_dynamics;   // pipeline.cpp:388-402
    dyn = {};
    dyn.dt = dt; dyn.max_dof = m.max_dof; dyn.integrate_velocity = 1u; dyn.fold_drive_damping = fold ? 1u : 0u; dyn.reuse_mass = 0u;
    std::memcpy(dyn.gravity, cfg.gravity, sizeof(cfg.gravity));
    dyn.articulation_count = E; dyn.total_link_count = E * nl; dyn.apply_link_wrench = 1u; dyn.max_links = nl;
    dyn.links_per_env = nl; dyn.bodies_per_env = nb;
    w.p_dynamics_probe = dyn;
    w.p_dynamics_probe.integrate_velocity = 0u;
    w.p_int_vel = {};
    w.p_int_vel.dt = dt; w.p_int_vel.total_link_count = E * nl; w.p_int_vel.articulation_count = E;
    std::memcpy(w.p_int_vel.gravity, cfg.gravity, sizeof(cfg.gravity));
    w.p_snapshot = {E, E, m.max_dof, nl, E * nb, 0u};
    w.p_reference_weights = {m.max_dof, E, E * nl, 1u, nb, E * nb};
    w.p_int_pos = {};
    w.p_int_pos.dt = dt; w.p_int_pos.total_link_count = E * nl; w.p_int_pos.articulation_count = E; w.p_int_pos.env_count = E;
    w.p_int_pos.pos_pass = (has_contacts && cfg.solver_pos_iters > 0u) ? 1u : 0u;
    w.p_sync = {};
    w.p_sync.env_count = E; w.p_sync.links_per_env = nl; w.p_sync.bodies_per_env = nb;
    w.p_aabbs = {};   // pipeline.cpp:613-615
    w.p_aabbs.env_count = E; w.p_aabbs.bodies_per_env = nb; w.p_aabbs.margin = std::fmax(contact_margin, 0.0005f);
    w.p_aabbs.dt = dt; w.p_aabbs.query_reach = query_reach;
    w.p_lbvh = {};
    w.p_lbvh.env_count = E; w.p_lbvh.bodies_per_env = nb;
    w.p_query = {};
    w.p_query.env_count = E; w.p_query.bodies_per_env = nb; w.p_query.max_contacts_per_env = m.contact_slots;
    w.p_query.rigid_slot_cap = m.contact_slots; w.p_query.max_pairs = m.contact_slots;
    w.p_narrow = {};
    w.p_narrow.env_count = E; w.p_narrow.bodies_per_env = nb; w.p_narrow.union_slot_count = m.contact_slots;
    w.p_narrow.rigid_slot_cap = m.contact_slots; w.p_narrow.contact_margin = contact_margin; w.p_narrow.dt = dt;
    w.p_narrow.query_reach = query_reach; w.p_narrow.base_link_count = nl; w.p_narrow.articulations_per_env = 1u;
    w.p_narrow.max_contacts_per_pair = 4u;
    w.p_heightfield = {};   // has_heightfield 0: the op has nothing to add
    w.p_heightfield.env_count = E; w.p_heightfield.bodies_per_env = nb; w.p_heightfield.rigid_slot_cap = m.contact_slots;
    w.p_heightfield.slot_stride = m.contact_slots; w.p_heightfield.contact_margin = contact_margin;
    AssembleRowsParams& as = w.p_assemble;   // pipeline.cpp:861-897
    as = {};
    as.env_count = E; as.articulation_count = E; as.total_link_count = E * nl; as.max_dof = m.max_dof;
    as.union_slot_count = m.contact_slots; as.rows_per_env = m.rows_per_env; as.contact_rows_per_env = m.contact_rows_per_env;
    as.full_row_slot_count = m.contact_slots; as.bodies_per_env = nb; as.base_link_count = nl;
    as.position_pass = cfg.solver_pos_iters > 0u ? 1u : 0u;
    as.dt = dt; as.overlap_recovery_velocity = cfg.solver_overlap_recovery_velocity; as.contact_margin = contact_margin;
    as.joint_limit_rows_per_env = m.joint_limit_rows; as.joint_friction_rows_per_env = m.joint_friction_rows;
    as.joint_drive_rows_per_env = m.joint_drive_rows; as.baumgarte_max_velocity = cfg.solver_baumgarte_max_velocity;
    // the MuJoCo law's world-wide terms (pipeline.cpp:880-886); a pair's solref and solimp come from its profiles
    as.solref[0] = 0.02f; as.solref[1] = 1.0f;
    as.solimp[0] = 0.9f; as.solimp[1] = 0.95f; as.solimp[2] = 0.001f; as.solimp[3] = 0.5f; as.solimp[4] = 2.0f;
    as.impratio = m.contact_impratio; as.refsafe = true; as.cone = m.contact_cone;
    w.p_warm0 = {};
    w.p_warm0.env_count = E; w.p_warm0.slot_count = m.contact_slots; w.p_warm0.rows_per_env = m.rows_per_env;
    w.p_warm0.full_row_slot_count = m.contact_slots; w.p_warm0.decay_steps = 2u;
    w.p_warm1 = w.p_warm0;
    w.p_warm1.phase = 1u;
    BlockDescentSolveParams& bd = w.p_solve;   // pipeline.cpp:471-497
    bd = {};
    bd.dt = dt; bd.env_count = E; bd.rows_per_env = m.rows_per_env; bd.total_body_count = E * nb; bd.articulation_count = E;
    bd.max_dof = m.max_dof; bd.max_independent_dof = m.dof; bd.base_link_count = nl; bd.contact_rows_per_env = m.contact_rows_per_env;
    bd.contact_slots_per_env = m.contact_slots; bd.iterations = cfg.solver_vel_iters;
    bd.position_iterations = has_contacts ? cfg.solver_pos_iters : 0u;
    bd.position_beta = cfg.solver_pos_beta; bd.position_slop = cfg.solver_pos_slop;
    bd.position_max_velocity = cfg.solver_baumgarte_max_velocity; bd.velocity_tolerance = cfg.solver_velocity_tolerance;
    bd.joint_limit_rows_per_env = m.joint_limit_rows;

    // op order of one interval (pipeline.cpp:374, 428-430, 442, 605-639, 699, 746, 908-923, 967, 981-986)
    w.calls.clear();
    auto add = [&](NkOp op, const void* params) {
        if (!BackendSupportsOp(op)) throw std::runtime_error(std::string("backend does not support op ") + OpName(op));
        w.calls.push_back({uint16_t(op), params});
    };
    add(NkOp::SnapshotStepVelocity, &w.p_snapshot);
    if (m.free_body != 0u) {
        // a world of free bodies (pipeline.cpp:434-443, 600-606): the bodies' velocity update, with the block the solve
        // descends on, then the poses of their collidable rows
        w.p_int_vel.total_body_count = E * nb > 0u ? E * nb : E;
        w.p_int_pos.total_body_count = w.p_int_vel.total_body_count;
        add(NkOp::IntegrateVelocity, &w.p_int_vel);
        add(NkOp::FkWorldPoses, &w.p_fk);
    } else {
        add(NkOp::FkWorldPoses, &w.p_fk);
        add(NkOp::ApplyDrives, &w.p_drives);
        add(NkOp::ArticulationDynamics, &w.p_dynamics);
        add(NkOp::IntegrateVelocity, &w.p_int_vel);
    }
    if (has_contacts) {   // rows of any kind: contact slots, joint limits, joint friction, drives (pipeline.cpp:207)
        if (m.contact_slots > 0u) {
            add(NkOp::SyncLinkBodyPose, &w.p_sync);
            add(NkOp::BuildAabbs, &w.p_aabbs);
            add(NkOp::LbvhBuild, &w.p_lbvh);
            add(NkOp::LbvhQueryPairs, &w.p_query);
            add(NkOp::NarrowphasePrimitives, &w.p_narrow);
            add(NkOp::NarrowphaseHeightfield, &w.p_heightfield);
        }
        add(NkOp::AssembleRows, &w.p_assemble);
        if (m.contact_slots > 0u) add(NkOp::ContactWarmStart, &w.p_warm0);
        add(NkOp::BlockDescentSolve, &w.p_solve);
        if (m.contact_slots > 0u) add(NkOp::ContactWarmStart, &w.p_warm1);
    }
    if (drives) add(NkOp::ReadoutDrives, &w.p_readout_drives);   // pipeline.cpp:929-937
    w.p_damping = {dt, m.max_dof, E, E * nl, m.integrator == 2u ? 1u : 0u, m.drive_mode, drives ? 1u : 0u};
    if (m.integrator != 0u) add(NkOp::ArticulationDamping, &w.p_damping);   // pipeline.cpp:939-951
    add(NkOp::IntegratePosition, &w.p_int_pos);
    add(NkOp::FkWorldPoses, &w.p_fk);
    if (m.free_body == 0u) add(NkOp::FkLinkVelocities, &w.p_fk_velocity);   // a free body's twist words hold its six coordinates
    if (nb > 0u) add(NkOp::SyncLinkBodyPose, &w.p_sync);
    // a pure readout, part of the step only once a consumer has asked for one of its fields (pipeline.cpp:990-1005)
    w.p_readout_contacts = {};
    w.p_readout_contacts.dt = dt; w.p_readout_contacts.env_count = E; w.p_readout_contacts.base_link_count = nl;
    w.p_readout_contacts.max_contacts_per_env = m.contact_slots; w.p_readout_contacts.rows_per_env = m.rows_per_env;
    w.p_readout_contacts.full_row_slot_count = m.contact_slots; w.p_readout_contacts.contact_rows_per_env = m.contact_rows_per_env;
    const bool reads_contacts = w.contact_readout_demanded && has_contacts && m.contact_slots > 0u;
    if (reads_contacts) add(NkOp::ReadoutContactWrench, &w.p_readout_contacts);
    if (substeps == 1u) return;
    // pipeline.cpp:118-180: the interval once per substep, each followed by the accumulation of the step's outputs
    const std::vector<nuka_phi_op_call> interval = w.calls;
    w.calls.clear();
    w.p_accumulate.assign(substeps, AccumulateStepParams{});
    for (uint32_t step = 0u; step < substeps; ++step) {
        AccumulateStepParams& outputs = w.p_accumulate[step];
        outputs.env_count = E; outputs.links_per_env = nl;
        outputs.flags = kAccumulateOutputs | kFinalizeLinkWrench;
        if (reads_contacts) outputs.flags |= kAccumulateLinkWrench;
        if (m.joint_limit_rows != 0u) outputs.flags |= kAccumulateJointLimit;
        outputs.first = step == 0u ? 1u : 0u; outputs.last = step + 1u == substeps ? 1u : 0u;
        outputs.substep_dt = dt; outputs.inv_outer_dt = 1.0f / cfg.fixed_dt;
        for (const nuka_phi_op_call& call : interval) w.calls.push_back(call);
        add(NkOp::AccumulateStep, &outputs);
    }
}

void InvalidatePlan(World& w) {
    if (w.plan != nullptr) { w.be->plan_free(w.backend, w.plan); w.plan = nullptr; }
}

nuka_result_t MapStatus(uint8_t status) {
    switch (static_cast<Status>(status)) {
        case Status::Ok: return NUKA_RESULT_OK;
        case Status::Unsupported: return NUKA_RESULT_NOT_SUPPORTED;
        case Status::OutOfMemory: return NUKA_RESULT_OUT_OF_MEMORY;
        case Status::InvalidArgument: return NUKA_RESULT_INVALID_ARG;
        default: return NUKA_RESULT_DEVICE_ERROR;
    }
}

// nk::World::Step (src/nk/pipeline/world.cpp:663-686): every op through the backend's dispatch
nuka_result_t StepEager(World& w) {
    for (const nuka_phi_op_call& call : w.calls) {
        const uint8_t status = w.be->dispatch(w.backend, reinterpret_cast<const nuka_phi_model_view*>(&w.model),
                                              reinterpret_cast<const nuka_phi_data_view*>(&w.data), &call);
        if (status != uint8_t(Status::Ok)) {
            w.last_error = {};
            w.last_error.status = status; w.last_error.failed_op = call.op;
            std::snprintf(w.last_error.message, sizeof(w.last_error.message), "step failed in op %s", OpName(static_cast<NkOp>(call.op)));
            return Error(MapStatus(status), w.last_error.message);
        }
    }
    return NUKA_RESULT_OK;
}

// nk::World::PrepareGraph (world.cpp:688-705)
nuka_result_t PreparePlan(World& w) {
    if (w.plan != nullptr) return NUKA_RESULT_OK;
    nuka_phi_execution_error error{};
    ++w.capture_attempts;
    w.plan = w.be->plan_create(w.backend, reinterpret_cast<const nuka_phi_model_view*>(&w.model),
                               reinterpret_cast<const nuka_phi_data_view*>(&w.data), w.calls.data(), int(w.calls.size()), &error);
    if (w.plan == nullptr) { w.last_error = error; return Error(MapStatus(error.status), std::string("graph capture failed: ") + error.message); }
    return NUKA_RESULT_OK;
}

nuka_result_t StepN(World& w, uint32_t n) {
    if (w.mode == NUKA_EXECUTION_GRAPH) {
        const nuka_result_t prepared = PreparePlan(w);
        if (prepared != NUKA_RESULT_OK) return prepared;
        uint32_t submitted = 0u;
        nuka_phi_execution_error error{};
        const uint8_t status = w.be->plan_execute_repeated(w.backend, w.plan, n, &submitted, &error);
        w.graph_replays += submitted;
        if (status != uint8_t(Status::Ok)) { w.last_error = error; return Error(MapStatus(status), std::string("graph launch failed: ") + error.message); }
        return NUKA_RESULT_OK;
    }
    for (uint32_t i = 0u; i < n; ++i) {
        const nuka_result_t r = StepEager(w);
        if (r != NUKA_RESULT_OK) return r;
    }
    return NUKA_RESULT_OK;
}

template <typename T>
size_t Place(std::vector<Field>& fields, const char* name, Dtype dtype, size_t count, size_t* cursor, bool is_template) {
    (void)sizeof(T);
    const size_t offset = *cursor;
    fields.push_back({name, dtype, DtypeBytes(dtype), count, offset, is_template});
    *cursor = (offset + count * DtypeBytes(dtype) + 255u) & ~size_t{255u};
    return offset;
}

}  // namespace
}  // namespace nkh

using namespace nkh;

extern "C" {

const char* nuka_result_message(nuka_result_t result) {
    switch (result) {
        case NUKA_RESULT_OK: return "ok";
        case NUKA_RESULT_INVALID_ARG: return "invalid argument";
        case NUKA_RESULT_NULL_HANDLE: return "null handle";
        case NUKA_RESULT_DEVICE_ERROR: return "device error";
        case NUKA_RESULT_OUT_OF_MEMORY: return "out of memory";
        case NUKA_RESULT_NOT_SUPPORTED: return "not supported";
        default: return "internal error";
    }
}

const char* nuka_last_error_message(void) {
    static thread_local std::string held;
    held.swap(g_last_error);
    g_last_error.clear();
    return held.c_str();
}

nuka_result_t nuka_device_create(const nuka_device_desc_t* desc, nuka_device_handle* out) {
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out = nullptr;
    if (desc == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "desc is null");
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count == 0) {
        (void)hipGetLastError();
        return Error(NUKA_RESULT_DEVICE_ERROR, "no HIP device: the library has no CPU fallback");
    }
    const uint32_t index = desc->gpu_index;
    if (index >= uint32_t(count)) return Error(NUKA_RESULT_DEVICE_ERROR, "no HIP device with this gpu_index");
    void* backend = CreateBackend(int(index), desc->cuda_stream);
    if (backend == nullptr) return Error(NUKA_RESULT_DEVICE_ERROR, "backend creation failed");
    // CreateBackend has made this GPU current: its copy of the static staging array is looked up once
    if (index < uint32_t(kMaxGpus) && g_static_reset_ids[index] == nullptr) {
        void* address = nullptr;
        if (hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)) != hipSuccess || address == nullptr) {
            (void)hipGetLastError();
            auto* made = reinterpret_cast<nuka_phi_backend*>(backend);
            reinterpret_cast<nuka_phi_backend_head*>(made)->iface->free(made);
            return Error(NUKA_RESULT_DEVICE_ERROR, "the static staging array has no address on this device");
        }
        g_static_reset_ids[index] = static_cast<uint32_t*>(address);
    }
    auto* record = new DeviceRecord{backend, int(index)};
    *out = reinterpret_cast<nuka_device_handle>(record);
    return NUKA_RESULT_OK;
}

void nuka_device_destroy(nuka_device_handle device) {
    auto* record = reinterpret_cast<DeviceRecord*>(device);
    if (record == nullptr) return;
    auto* backend = reinterpret_cast<nuka_phi_backend*>(record->backend);
    reinterpret_cast<nuka_phi_backend_head*>(backend)->iface->free(backend);
    delete record;
}

nuka_phi_backend* nuka_device_backend(nuka_device_handle device) {
    auto* record = reinterpret_cast<DeviceRecord*>(device);
    return record != nullptr ? reinterpret_cast<nuka_phi_backend*>(record->backend) : nullptr;
}

namespace nkh {
namespace {
nuka_result_t CreateWorld(nuka_device_handle device, const nuka_template_desc_t* tmpl, const nuka_hip_world_desc_t* desc,
                          const scene_file::Scene* scene, nuka_world_handle* out) {
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out = nullptr;
    if (device == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "device is null");
    if (tmpl == nullptr || desc == nullptr || desc->env_count == 0u) return Error(NUKA_RESULT_INVALID_ARG, "template, desc and env_count are required");
    // a caller built against the header before the joint-row members passes the shorter size; those members read as zero
    constexpr size_t kTemplateBase = offsetof(nuka_template_desc_t, joint_limit_lower);
    constexpr size_t kTemplateJointRows = offsetof(nuka_template_desc_t, excluded_pairs);
    constexpr size_t kTemplateExcluded = offsetof(nuka_template_desc_t, profile_law);
    constexpr size_t kTemplateLaw = offsetof(nuka_template_desc_t, profile_priority);
    constexpr size_t kTemplateMerge = offsetof(nuka_template_desc_t, joint_law);
    constexpr size_t kWorldBase = offsetof(nuka_hip_world_desc_t, solver_fold_drive_damping);
    constexpr size_t kWorldDrives = offsetof(nuka_hip_world_desc_t, solver_substeps);
    if ((tmpl->struct_size != sizeof(nuka_template_desc_t) && tmpl->struct_size != kTemplateMerge && tmpl->struct_size != kTemplateLaw && tmpl->struct_size != kTemplateExcluded && tmpl->struct_size != kTemplateJointRows &&
         tmpl->struct_size != kTemplateBase) ||
        (desc->struct_size != sizeof(nuka_hip_world_desc_t) && desc->struct_size != kWorldDrives && desc->struct_size != kWorldBase))
        return Error(NUKA_RESULT_INVALID_ARG, "struct_size mismatch");
    nuka_template_desc_t template_copy{};
    std::memcpy(&template_copy, tmpl, tmpl->struct_size);
    nuka_hip_world_desc_t desc_copy{};
    std::memcpy(&desc_copy, desc, desc->struct_size);
    tmpl = &template_copy;
    desc = &desc_copy;
    try {
        auto world = std::make_unique<World>();
        World& w = *world;
        static std::atomic<uint64_t> created{0u};
        w.id = ++created;
        w.device = reinterpret_cast<DeviceRecord*>(device);
        w.backend = reinterpret_cast<nuka_phi_backend*>(w.device->backend);
        w.be = reinterpret_cast<nuka_phi_backend_head*>(w.backend)->iface;
        Cook(*tmpl, &w.host);
        w.cfg = *desc;
        nuka_hip_world_desc_t& cfg = w.cfg;   // nuka.h:160-173 defaults; pipeline.hpp SolverConfig; op_schema.hpp:598, 663
        if (cfg.fixed_dt <= 0.0f) cfg.fixed_dt = 1.0f / 240.0f;
        if (cfg.solver_vel_iters == 0u) cfg.solver_vel_iters = 10u;
        if (cfg.solver_pos_iters == 0u) cfg.solver_pos_iters = 4u;
        if (cfg.solver_pos_iters == 0xFFFFFFFFu) cfg.solver_pos_iters = 0u;
        if (cfg.solver_pos_beta <= 0.0f) cfg.solver_pos_beta = 0.3f;
        if (cfg.solver_pos_slop <= 0.0f) cfg.solver_pos_slop = 1.0e-3f;
        if (cfg.solver_velocity_tolerance <= 0.0f) cfg.solver_velocity_tolerance = 1.0e-5f;
        if (cfg.solver_baumgarte_max_velocity <= 0.0f) cfg.solver_baumgarte_max_velocity = 3.0e38f;
        if (cfg.solver_substeps == 0u) cfg.solver_substeps = 1u;
        if (cfg.solver_substeps > 64u) throw std::invalid_argument("solver_substeps must be at most 64");
        if (cfg.contact_detection_substeps > 1u) throw NotSupported("substeps that share one contact detection are not built on this path");
        w.env_count = desc->env_count;
        const ModelView& hc = w.host.counts;
        const size_t E = w.env_count, nl = hc.links_per_env, nb = hc.bodies_per_env, md = hc.max_dof, S = hc.contact_slots, R = hc.rows_per_env;
        const size_t mf = SolverMassFactorFloats(hc);
        const size_t fb = hc.free_body != 0u ? nb : 0u;   // the rigid-body fields have their rows in a world of free bodies only
        if (E * std::max<size_t>(R, 1u) > 0xFFFFFFFFull / 2u || E * nl * 7u > 0xFFFFFFFFull) throw std::invalid_argument("world too large for 32-bit row indices");
        if (hc.rows_per_env > 0u && SolverHeadCapacity(hc, std::max(hc.contact_slots, 1u), 150u * 1024u) == 0u) throw std::invalid_argument("solver tile does not fit LDS");
        // arena layout: template tables first, then the env-major fields, each on a 256-byte boundary (buffer.hpp:39)
        size_t cursor = 0u;
#define X(name, dtype) Place<int>(w.fields, #name, dtype, w.host.name.size(), &cursor, true);
        NKH_MODEL_FIELDS(X)
#undef X
#define X(name, dtype, count) Place<int>(w.fields, #name, dtype, size_t(count), &cursor, false);
        NKH_DATA_FIELDS(X)
#undef X
        w.arena_bytes = cursor;
        uint8_t status = 0u;
        nuka_phi_buffer_type* type = BackendDeviceBufferType(w.device->backend);
        w.arena = reinterpret_cast<nuka_phi_buffer_type_head*>(type)->iface->alloc(type, w.arena_bytes, &status);
        if (w.arena == nullptr) return Error(NUKA_RESULT_OUT_OF_MEMORY, "arena allocation failed");
        w.initial = reinterpret_cast<nuka_phi_buffer_type_head*>(type)->iface->alloc(type, w.arena_bytes, &status);
        if (w.initial == nullptr) return Error(NUKA_RESULT_OUT_OF_MEMORY, "reset snapshot allocation failed");
        if (Iface(w.arena)->memset(w.arena, 0u, 0u, w.arena_bytes) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "arena clear failed");
        char* base = static_cast<char*>(Iface(w.arena)->base(w.arena));
        w.model = hc;
        size_t f = 0u;
#define X(name, dtype) { const Field& fld = w.fields[f++]; \
            w.model.name = reinterpret_cast<decltype(w.model.name)>(base + fld.offset); \
            if (fld.count > 0u && Iface(w.arena)->upload(w.arena, w.host.name.data(), fld.offset, fld.count * fld.elem_bytes) != uint8_t(Status::Ok)) \
                return Error(NUKA_RESULT_DEVICE_ERROR, "template upload failed"); }
        NKH_MODEL_FIELDS(X)
#undef X
#define X(name, dtype, count) { const Field& fld = w.fields[f++]; w.data.name = reinterpret_cast<decltype(w.data.name)>(base + fld.offset); }
        NKH_DATA_FIELDS(X)
#undef X
        // initial state: identity poses, cooked static poses, no rows
        {
            std::vector<float> base_pose(E * 7u, 0.0f), link_pose(E * nl * 7u, 0.0f), body_pose(E * nb * 7u, 0.0f);
            for (size_t e = 0u; e < E; ++e) {
                base_pose[e * 7u + 3u] = 1.0f;
                for (size_t l = 0u; l < nl; ++l) link_pose[(e * nl + l) * 7u + 3u] = 1.0f;
                for (size_t b = 0u; b < nb; ++b) std::memcpy(&body_pose[(e * nb + b) * 7u], &w.host.body_init_pose[b * 7u], 7u * sizeof(float));
            }
            std::vector<uint32_t> invalid(E * R, kInvalid);
            auto put = [&](void* field, const void* src, size_t bytes) {
                if (bytes == 0u) return true;
                return Iface(w.arena)->upload(w.arena, src, size_t(static_cast<char*>(field) - base), bytes) == uint8_t(Status::Ok);
            };
            // the bodies' inertial parameters (fields.yaml:17, 108, 568): a free body's in its own row - 1 / mass, 1 / principal
            // moments, the inertial frame - and zero mass (a body the rigid-body ops leave alone) in every other row
            std::vector<float> inv_mass(E * fb, 0.0f), inv_inertia(E * fb * 3u, 0.0f), inertial_frame(E * fb * 7u, 0.0f);
            for (size_t e = 0u; e < E; ++e)
                for (size_t b = 0u; b < fb; ++b) {
                    inertial_frame[(e * nb + b) * 7u + 3u] = 1.0f;
                    if (hc.free_body == 0u || b != w.host.link_body[0]) continue;
                    inv_mass[e * nb + b] = 1.0f / w.host.link_mass[0];
                    for (size_t k = 0u; k < 3u; ++k) inv_inertia[(e * nb + b) * 3u + k] = 1.0f / w.host.link_diag_inertia[k];
                    std::memcpy(&inertial_frame[(e * nb + b) * 7u], w.host.link_inertial_frame.data(), 7u * sizeof(float));
                }
            if (!put(w.data.body_inv_mass, inv_mass.data(), inv_mass.size() * 4u) || !put(w.data.body_inv_inertia, inv_inertia.data(), inv_inertia.size() * 4u) ||
                !put(w.data.body_inertial_frame, inertial_frame.data(), inertial_frame.size() * 4u))
                return Error(NUKA_RESULT_DEVICE_ERROR, "initial state upload failed");
            if (!put(w.data.base_pose, base_pose.data(), base_pose.size() * 4u) || !put(w.data.link_pose, link_pose.data(), link_pose.size() * 4u) ||
                !put(w.data.body_pose, body_pose.data(), body_pose.size() * 4u) || !put(w.data.row_cj_link, invalid.data(), invalid.size() * 4u) ||
                !put(w.data.row_cj_link_b, invalid.data(), invalid.size() * 4u) || !put(w.data.row_unit, invalid.data(), invalid.size() * 4u))
                return Error(NUKA_RESULT_DEVICE_ERROR, "initial state upload failed");
        }
        w.drive_stiffness.assign(nl, 0.0f);
        w.drive_force_limit.assign(nl, 0.0f);
        if (scene != nullptr) { w.drive_stiffness = scene->drive_stiffness; w.drive_force_limit = scene->drive_force_limit; }
        if (scene != nullptr) {   // the state and drive parameters the scene file authors, in every environment
            auto tile = [&](const std::vector<float>& per_link) {
                std::vector<float> all(E * nl);
                for (size_t e = 0u; e < E; ++e) std::copy(per_link.begin(), per_link.end(), all.begin() + e * nl);
                return all;
            };
            auto put = [&](void* field, const std::vector<float>& values) {
                return Iface(w.arena)->upload(w.arena, values.data(), size_t(static_cast<char*>(field) - base), values.size() * 4u) == uint8_t(Status::Ok);
            };
            std::vector<float> base_pose(E * 7u);
            for (size_t e = 0u; e < E; ++e) std::copy(scene->base_pose.begin(), scene->base_pose.end(), base_pose.begin() + e * 7u);
            bool ok = put(w.data.q, tile(scene->initial_q)) && put(w.data.drive_stiffness, tile(scene->drive_stiffness)) &&
                      put(w.data.drive_damping, tile(scene->drive_damping)) && put(w.data.drive_force_limit, tile(scene->drive_force_limit)) &&
                      put(w.data.drive_joint_force_limit, tile(scene->drive_joint_force_limit));
            if (hc.floating_root != 0u) ok = ok && put(w.data.base_pose, base_pose);
            if (hc.drive_mode == kDrivePdPosition) ok = ok && put(w.data.drive_target, tile(scene->initial_q));   // hold the authored pose
            if (!ok) return Error(NUKA_RESULT_DEVICE_ERROR, "scene state upload failed");
        }
        if (scene != nullptr) { w.from_scene = true; w.link_names = scene->link_names; w.joint_names = scene->joint_names; }
        BuildPipeline(w);
        // nk/pipeline/world.cpp:553-561: creation exposes the poses of the initial state and the reference weights at
        // them.  Only the MuJoCo contact law reads the weights; other worlds first compute their poses in their first step.
        if (hc.any_mujoco != 0u) {
            const nuka_phi_op_call at_creation[3] = {{uint16_t(NkOp::FkWorldPoses), &w.p_fk}, {uint16_t(NkOp::SyncLinkBodyPose), &w.p_sync},
                                                     {uint16_t(NkOp::ReferenceWeights), &w.p_reference_weights}};
            for (const nuka_phi_op_call& call : at_creation) {
                if (call.op == uint16_t(NkOp::SyncLinkBodyPose) && nb == 0u) continue;
                const uint8_t status = w.be->dispatch(w.backend, reinterpret_cast<const nuka_phi_model_view*>(&w.model),
                                                      reinterpret_cast<const nuka_phi_data_view*>(&w.data), &call);
                if (status != uint8_t(Status::Ok)) return Error(MapStatus(status), "reference weights failed");
            }
            if (w.be->synchronize(w.backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "device error in the reference weights");
        }
        if (Iface(w.initial)->copy_from(w.initial, w.arena, 0u, 0u, w.arena_bytes) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "snapshot failed");
        if (w.be->synchronize(w.backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "device error during world creation");
        *out = reinterpret_cast<nuka_world_handle>(world.release());
        return NUKA_RESULT_OK;
    } catch (const std::invalid_argument& e) {
        return Error(NUKA_RESULT_INVALID_ARG, e.what());
    } catch (const NotSupported& e) {
        return Error(NUKA_RESULT_NOT_SUPPORTED, e.what());
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    } catch (const std::exception& e) {
        return Error(NUKA_RESULT_INTERNAL, e.what());
    }
}
}  // namespace
}  // namespace nkh

nuka_result_t nuka_world_create_from_template(nuka_device_handle device, const nuka_template_desc_t* tmpl,
                                              const nuka_hip_world_desc_t* desc, nuka_world_handle* out) {
    return CreateWorld(device, tmpl, desc, nullptr, out);
}

nuka_result_t nuka_scene_load_mjcf(const char* path, uint32_t flags, nuka_scene_handle* out) {
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out = nullptr;
    if (path == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "path is null");
    if ((flags & ~uint32_t(NUKA_SCENE_PLANE_CONTACTS_ONLY | NUKA_SCENE_GROUND_PLANE | NUKA_SCENE_NATIVE_CONTACT_LAW | NUKA_SCENE_NATIVE_JOINT_LAW)) != 0u) return Error(NUKA_RESULT_INVALID_ARG, "unknown scene flag");
    try {
        *out = reinterpret_cast<nuka_scene_handle>(scene_file::LoadMjcf(path, flags).release());
        return NUKA_RESULT_OK;
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    } catch (const std::exception& e) {
        return Error(NUKA_RESULT_INVALID_ARG, e.what());
    }
}

nuka_result_t nuka_scene_load_urdf(const char* path, uint32_t flags, nuka_scene_handle* out) {
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out = nullptr;
    if (path == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "path is null");
    if ((flags & ~uint32_t(NUKA_SCENE_PLANE_CONTACTS_ONLY | NUKA_SCENE_FIXED_BASE | NUKA_SCENE_GROUND_PLANE)) != 0u) return Error(NUKA_RESULT_INVALID_ARG, "unknown scene flag");
    try {
        *out = reinterpret_cast<nuka_scene_handle>(scene_file::LoadUrdf(path, flags).release());
        return NUKA_RESULT_OK;
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    } catch (const std::exception& e) {
        return Error(NUKA_RESULT_INVALID_ARG, e.what());
    }
}

void nuka_scene_destroy(nuka_scene_handle scene) { delete reinterpret_cast<scene_file::Scene*>(scene); }

const nuka_template_desc_t* nuka_scene_template(nuka_scene_handle scene) {
    return scene != nullptr ? &reinterpret_cast<scene_file::Scene*>(scene)->desc : nullptr;
}

nuka_result_t nuka_scene_get_info(nuka_scene_handle scene, nuka_scene_info_t* out) {
    const auto* s = reinterpret_cast<const scene_file::Scene*>(scene);
    if (s == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "scene is null");
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out = {s->desc.link_count, s->desc.body_count, s->actuator_count, s->dropped_geom_count, s->floating_root ? 1u : 0u, s->drive_mode,
            s->timestep, {s->gravity[0], s->gravity[1], s->gravity[2]}};
    return NUKA_RESULT_OK;
}

const char* nuka_scene_link_name(nuka_scene_handle scene, uint32_t link) {
    const auto* s = reinterpret_cast<const scene_file::Scene*>(scene);
    return s != nullptr && link < s->link_names.size() ? s->link_names[link].c_str() : nullptr;
}

const char* nuka_scene_joint_name(nuka_scene_handle scene, uint32_t link) {
    const auto* s = reinterpret_cast<const scene_file::Scene*>(scene);
    return s != nullptr && link < s->joint_names.size() ? s->joint_names[link].c_str() : nullptr;
}

nuka_result_t nuka_scene_initial_state(nuka_scene_handle scene, float* q, float* base_pose, float* drive_stiffness, float* drive_damping,
                                       float* drive_force_limit, float* drive_joint_force_limit) {
    const auto* s = reinterpret_cast<const scene_file::Scene*>(scene);
    if (s == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "scene is null");
    auto copy = [](float* out, const std::vector<float>& values) { if (out != nullptr) std::copy(values.begin(), values.end(), out); };
    copy(q, s->initial_q);
    copy(drive_stiffness, s->drive_stiffness);
    copy(drive_damping, s->drive_damping);
    copy(drive_force_limit, s->drive_force_limit);
    copy(drive_joint_force_limit, s->drive_joint_force_limit);
    if (base_pose != nullptr) std::copy(s->base_pose.begin(), s->base_pose.end(), base_pose);
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_hip_world_create_from_scene_handle(nuka_device_handle device, nuka_scene_handle scene,
                                                      const nuka_hip_world_desc_t* desc, nuka_world_handle* out) {
    const auto* s = reinterpret_cast<const scene_file::Scene*>(scene);
    if (s == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "scene is null");
    if (desc == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "desc is null");
    if (desc->struct_size != sizeof(nuka_hip_world_desc_t)) return Error(NUKA_RESULT_INVALID_ARG, "struct_size mismatch");
    nuka_hip_world_desc_t with_file = *desc;
    if (with_file.fixed_dt <= 0.0f) with_file.fixed_dt = s->timestep;
    if (with_file.gravity[0] == 0.0f && with_file.gravity[1] == 0.0f && with_file.gravity[2] == 0.0f)
        std::copy(s->gravity, s->gravity + 3, with_file.gravity);
    return CreateWorld(device, &s->desc, &with_file, s, out);
}

// nuka_world_create_from_scene (nuka.h:175-177; src/c_abi/world.cpp:493-527, 590-635): the reference's descriptor, the
// scene file read by its extension (LoadSceneByExtension, world.cpp:60-82).
nuka_result_t nuka_world_create_from_scene(nuka_device_handle device, const nuka_world_desc_t* desc, nuka_world_handle* out) {
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out = nullptr;
    if (desc == nullptr || desc->scene_path == nullptr || !(desc->fixed_dt > 0.0f) || desc->env_count == 0u)
        return Error(NUKA_RESULT_INVALID_ARG, "desc, scene_path, a positive fixed_dt and env_count are required");
    if (desc->determinism > 1u) return Error(NUKA_RESULT_INVALID_ARG, "determinism is 0 or 1");
    if (desc->control_mode > 5u) return Error(NUKA_RESULT_INVALID_ARG, "unknown control mode");
    if (device == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "device is null");
    if (desc->control_mode == 3u || desc->control_mode == 4u)
        return Error(NUKA_RESULT_NOT_SUPPORTED, "the computed-torque and OSC control modes are not built");
    const bool terrain = desc->terrain_step_height != 0.0f || desc->terrain_step_width != 0.0f || desc->terrain_platform_width != 0.0f ||
                         desc->terrain_grid_width != 0.0f || desc->terrain_grid_height_max != 0.0f || desc->contact_family != 0u ||
                         desc->heightfield_terrain_type != 0u || desc->heightfield_nrow != 0u || desc->heightfield_ncol != 0u ||
                         desc->heightfield_cell != 0.0f || (desc->heightfield_image_path != nullptr && desc->heightfield_image_path[0] != '\0') ||
                         desc->heightfield_radius_x != 0.0f || desc->heightfield_radius_y != 0.0f || desc->heightfield_elevation_z != 0.0f ||
                         desc->heightfield_base_z != 0.0f || desc->curric_levels != 0u || desc->curric_types != 0u ||
                         desc->terrain_feature_cell != 0.0f;
    if (terrain) return Error(NUKA_RESULT_NOT_SUPPORTED, "terrain and heightfield members must be zero: no heightfield path is built");
    if (desc->instance_count > 1u) return Error(NUKA_RESULT_NOT_SUPPORTED, "one articulation per environment: instance_count must be 0 or 1");
    if (desc->cloth_integrator != 0u || desc->ogc_contact_capacity != 0u)
        return Error(NUKA_RESULT_NOT_SUPPORTED, "cloth_integrator and ogc_contact_capacity must be zero: no particle path is built");
    const std::string path(desc->scene_path);
    const size_t dot = path.find_last_of('.');
    const size_t slash = path.find_last_of("/\\");
    const std::string extension = dot == std::string::npos || (slash != std::string::npos && dot < slash) ? std::string() : path.substr(dot);
    const bool mjcf = extension == ".xml" || extension == ".mjcf", urdf = extension == ".urdf";
    if (!mjcf && !urdf) return Error(NUKA_RESULT_NOT_SUPPORTED, "scene files are read as MJCF (.xml, .mjcf) or URDF (.urdf)");
    {
        std::FILE* probe = std::fopen(path.c_str(), "rb");
        if (probe == nullptr) return Error(NUKA_RESULT_FILE_NOT_FOUND, "cannot open " + path);
        std::fclose(probe);
    }
    std::unique_ptr<scene_file::Scene> scene;
    try {
        scene = mjcf ? scene_file::LoadMjcf(path.c_str(), 0u) : scene_file::LoadUrdf(path.c_str(), 0u);
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    } catch (const scene_file::Unsupported& e) {
        return Error(NUKA_RESULT_NOT_SUPPORTED, e.what());
    } catch (const std::exception& e) {
        return Error(NUKA_RESULT_PARSE_ERROR, e.what());
    }
    nuka_template_desc_t tmpl = scene->desc;
    tmpl.drive_mode = desc->control_mode;
    nuka_hip_world_desc_t options{};
    options.struct_size = sizeof(options);
    options.env_count = desc->env_count;
    options.fixed_dt = desc->fixed_dt;
    const bool no_gravity = desc->gravity_x == 0.0f && desc->gravity_y == 0.0f && desc->gravity_z == 0.0f;
    options.gravity[0] = desc->gravity_x; options.gravity[1] = desc->gravity_y; options.gravity[2] = no_gravity ? -9.81f : desc->gravity_z;
    options.solver_vel_iters = desc->solver_vel_iters;
    options.solver_pos_iters = desc->solver_pos_iters;
    options.solver_contact_margin = desc->solver_contact_margin;
    options.solver_baumgarte_max_velocity = desc->solver_baumgarte_max_velocity;
    options.solver_overlap_recovery_velocity = desc->solver_overlap_recovery_velocity;
    options.solver_substeps = desc->solver_substeps;
    options.contact_detection_substeps = desc->contact_detection_substeps;
    return CreateWorld(device, &tmpl, &options, scene.get(), out);
}

void nuka_world_destroy(nuka_world_handle world) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return;
    (void)w->be->synchronize(w->backend, nullptr);
    delete w;
}

nuka_result_t nuka_world_step(nuka_world_handle world) { return nuka_world_step_n(world, 1u); }

nuka_result_t nuka_world_step_n(nuka_world_handle world, uint32_t step_count) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    try {
        return StepN(*w, step_count);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "nuka_world_step_n: %s\n", e.what());
        return Error(NUKA_RESULT_INTERNAL, e.what());
    }
}

nuka_result_t nuka_world_set_execution_mode(nuka_world_handle world, nuka_execution_mode_t mode) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (mode != NUKA_EXECUTION_EAGER && mode != NUKA_EXECUTION_GRAPH) return Error(NUKA_RESULT_INVALID_ARG, "unknown execution mode");
    if (mode == NUKA_EXECUTION_GRAPH) {   // capture without advancing state; fail explicitly if unavailable (nuka.h:275-277)
        const nuka_result_t prepared = PreparePlan(*w);
        if (prepared != NUKA_RESULT_OK) return prepared;
    }
    w->mode = mode;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_set_velocity_iterations(nuka_world_handle world, uint32_t iterations) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (iterations == 0u || iterations > 65535u) return Error(NUKA_RESULT_INVALID_ARG, "iterations must be in 1..65535");
    if (w->be->synchronize(w->backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "device error");
    ++w->param_version;
    w->cfg.solver_vel_iters = iterations;
    w->p_solve.iterations = iterations;
    InvalidatePlan(*w);   // a changed value invalidates the execution graph (nuka.h:287-288)
    if (w->mode == NUKA_EXECUTION_GRAPH) return PreparePlan(*w);
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_velocity_iterations(nuka_world_handle world, uint32_t* out_iterations) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out_iterations == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out_iterations = w->p_solve.iterations;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_synchronize(nuka_world_handle world) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    nuka_phi_execution_error error{};
    if (w->be->synchronize(w->backend, &error) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, error.message);
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_reset(nuka_world_handle world) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (Iface(w->arena)->copy_from(w->arena, w->initial, 0u, 0u, w->arena_bytes) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "reset copy failed");
    return nuka_world_synchronize(world);
}

namespace nkh {
namespace {
// The arena slices a masked reset copies back or clears, one segment per field.
nuka_result_t ResetSegmentsOf(World* w, ResetSegments* out) {
    ResetSegments segments{};
    char* arena = static_cast<char*>(Iface(w->arena)->base(w->arena));
    const char* initial = static_cast<const char*>(Iface(w->initial)->base(w->initial));
    for (const Field& f : w->fields) {
        if (f.is_template || f.count == 0u || !(CheckpointKeeps(f.name) || CheckpointClears(f.name))) continue;
        if (segments.count == kMaxCheckpointSegments) return NUKA_RESULT_INTERNAL;
        const uint32_t at = segments.count++;
        segments.words_per_env[at] = uint32_t(f.count * f.elem_bytes / 4u / w->env_count);
        segments.live[at] = reinterpret_cast<uint32_t*>(arena + f.offset);
        segments.initial[at] = CheckpointKeeps(f.name) ? reinterpret_cast<const uint32_t*>(initial + f.offset) : nullptr;
    }
    *out = segments;
    return NUKA_RESULT_OK;
}
}  // namespace
}  // namespace nkh

nuka_result_t nuka_world_reset_envs(nuka_world_handle world, const uint32_t* env_ids, uint32_t count) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (count == 0u) return NUKA_RESULT_OK;
    if (env_ids == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "env_ids is null");
    // an invalid id changes nothing; duplicates are dropped so that no two workgroups write one slice
    std::vector<uint8_t> seen(w->env_count, 0u);
    std::vector<uint32_t> unique;
    for (uint32_t i = 0u; i < count; ++i) {
        if (env_ids[i] >= w->env_count) return Error(NUKA_RESULT_INVALID_ARG, "environment id out of range");
        if (seen[env_ids[i]] == 0u) { seen[env_ids[i]] = 1u; unique.push_back(env_ids[i]); }
    }
    ResetSegments segments{};
    if (ResetSegmentsOf(w, &segments) != NUKA_RESULT_OK) return Error(NUKA_RESULT_INTERNAL, "too many reset segments");
    if (nuka_world_synchronize(world) != NUKA_RESULT_OK) return NUKA_RESULT_DEVICE_ERROR;
    if (hipMemcpyAsync(w->data.reset_env_ids, unique.data(), unique.size() * sizeof(uint32_t), hipMemcpyHostToDevice,
                       BackendStream(w->device->backend)) != hipSuccess) return Error(NUKA_RESULT_DEVICE_ERROR, "id upload failed");
    hipLaunchKernelGGL(ResetEnvsKernel, dim3(uint32_t(unique.size()), segments.count), dim3(256), 0, BackendStream(w->device->backend),
                       segments, w->data.reset_env_ids, w->env_count);
    if (hipGetLastError() != hipSuccess) return Error(NUKA_RESULT_DEVICE_ERROR, "reset launch failed");
    return nuka_world_synchronize(world);   // the host copy of the ids must outlive the upload
}

// nuka_world_reset_envs for callers that cannot allocate: same kernel, same result, but the ids are staged in the
// static device array (at most NUKA_RESET_ENVS_STATIC_MAX of them) and in a static host array, so the call takes no
// device or host memory.  The array is shared by every call on one GPU: calls that overlap there race.
nuka_result_t nuka_world_reset_envs_static(nuka_world_handle world, const uint32_t* env_ids, uint32_t count) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (count == 0u) return NUKA_RESULT_OK;
    if (env_ids == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "env_ids is null");
    if (count > NUKA_RESET_ENVS_STATIC_MAX)
        return Error(NUKA_RESULT_INVALID_ARG, "more environment ids than NUKA_RESET_ENVS_STATIC_MAX in one static reset");
    const int gpu = w->device->gpu_index;
    uint32_t* staged = gpu >= 0 && gpu < kMaxGpus ? g_static_reset_ids[gpu] : nullptr;
    if (staged == nullptr) return Error(NUKA_RESULT_DEVICE_ERROR, "no static staging array on this device");
    for (uint32_t i = 0u; i < count; ++i)
        if (env_ids[i] >= w->env_count) return Error(NUKA_RESULT_INVALID_ARG, "environment id out of range");
    ResetSegments segments{};
    if (ResetSegmentsOf(w, &segments) != NUKA_RESULT_OK) return Error(NUKA_RESULT_INTERNAL, "too many reset segments");
    std::lock_guard<std::mutex> lock(g_static_reset_mutex);
    // duplicates are dropped so that no two workgroups write one slice; the order of the ids does not matter
    std::memcpy(g_static_reset_host, env_ids, size_t{count} * sizeof(uint32_t));
    std::sort(g_static_reset_host, g_static_reset_host + count);
    const uint32_t unique = uint32_t(std::unique(g_static_reset_host, g_static_reset_host + count) - g_static_reset_host);
    if (nuka_world_synchronize(world) != NUKA_RESULT_OK) return NUKA_RESULT_DEVICE_ERROR;
    hipStream_t stream = BackendStream(w->device->backend);
    // only the first `unique` words are read by this call; what an earlier, longer call left behind them is ignored
    if (hipMemcpyAsync(staged, g_static_reset_host, size_t{unique} * sizeof(uint32_t), hipMemcpyHostToDevice, stream) != hipSuccess)
        return Error(NUKA_RESULT_DEVICE_ERROR, "id upload failed");
    hipLaunchKernelGGL(ResetEnvsKernel, dim3(unique, segments.count), dim3(256), 0, stream, segments, staged, w->env_count);
    if (hipGetLastError() != hipSuccess) return Error(NUKA_RESULT_DEVICE_ERROR, "reset launch failed");
    return nuka_world_synchronize(world);   // the host staging is free again once the upload has run
}

nuka_result_t nuka_world_dispatch_op(nuka_world_handle world, uint16_t op, uint32_t variant) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (op >= uint16_t(NkOp::Count)) return Error(NUKA_RESULT_INVALID_ARG, "unknown op");
    const void* params = nullptr;
    for (const nuka_phi_op_call& call : w->calls) if (call.op == op) { params = call.params; break; }
    if (op == uint16_t(NkOp::ArticulationDynamics) && variant == 1u) params = &w->p_dynamics_probe;
    if (op == uint16_t(NkOp::ContactWarmStart) && variant == 1u) params = &w->p_warm1;
    if (op == uint16_t(NkOp::ReferenceWeights)) params = &w->p_reference_weights;
    if (params == nullptr) return Error(NUKA_RESULT_NOT_SUPPORTED, "op is not part of this world's pipeline");
    const nuka_phi_op_call call{op, params};
    const uint8_t status = w->be->dispatch(w->backend, reinterpret_cast<const nuka_phi_model_view*>(&w->model),
                                           reinterpret_cast<const nuka_phi_data_view*>(&w->data), &call);
    if (status != uint8_t(Status::Ok)) return Error(MapStatus(status), std::string("dispatch failed: ") + OpName(static_cast<NkOp>(op)));
    return NUKA_RESULT_OK;
}

// ---- the views by field name (include/nuka_phi.h) -----------------------------------------------------------------
namespace nkh {
namespace {
struct ViewField { const char* name; const char* reference_name; uint8_t owner, dtype, per; uint32_t scalars; size_t offset; };
// Members that stand for a field of fields.yaml under another name there, and members of the backend's own (no
// counterpart: nullptr).  Every other member carries the reference's name.
const char* ReferenceName(const char* name) {
    static const char* const renamed[][2] = {{"dof_link", "dof_to_link"}, {"dof_component", "dof_to_component"}};
    static const char* const own[] = {"joint_law", "link_push_order", "sweep_links", "link_dof", "link_dof_mask", "pairable_rows", "profile_mu",
                                      "profile_law", "profile_solref", "profile_solimp", "profile_margin", "profile_mix", "articulation_qdd",
                                      "solver_penalty", "solver_velocity", "solver_free", "solver_cost", "tile_order", "row_unit",
                                      "row_unit_value", "solver_mass_factor", "contact_cache_match"};
    for (const auto& pair : renamed) if (std::strcmp(name, pair[0]) == 0) return pair[1];
    for (const char* mine : own) if (std::strcmp(name, mine) == 0) return nullptr;
    return name;
}
// The model tables' element groups: entity and scalars a group (the data fields' follow from their counts).
struct ModelShape { const char* name; uint8_t per; uint32_t scalars; };
constexpr ModelShape kModelShapes[] = {
    {"joint_type", NUKA_HIP_PER_LINK, 1u}, {"parent_link", NUKA_HIP_PER_LINK, 1u}, {"joint_axis", NUKA_HIP_PER_LINK, 3u}, {"parent_offset", NUKA_HIP_PER_LINK, 3u},
    {"link_local_pose", NUKA_HIP_PER_LINK, 7u}, {"link_inertial_frame", NUKA_HIP_PER_LINK, 7u}, {"link_inertia", NUKA_HIP_PER_LINK, 36u},
    {"joint_damping", NUKA_HIP_PER_LINK, 1u}, {"joint_armature", NUKA_HIP_PER_LINK, 1u}, {"joint_stiffness", NUKA_HIP_PER_LINK, 1u},
    {"joint_spring_reference", NUKA_HIP_PER_LINK, 1u}, {"joint_limit_lower", NUKA_HIP_PER_LINK, 1u}, {"joint_limit_upper", NUKA_HIP_PER_LINK, 1u},
    {"joint_frictionloss", NUKA_HIP_PER_LINK, 1u}, {"joint_limit_flags", NUKA_HIP_PER_LINK, 1u}, {"joint_law", NUKA_HIP_PER_LINK, 1u},
    {"joint_limit_margin", NUKA_HIP_PER_LINK, 1u}, {"joint_limit_reference", NUKA_HIP_PER_LINK, 7u}, {"joint_friction_reference", NUKA_HIP_PER_LINK, 7u},
    {"link_body", NUKA_HIP_PER_LINK, 1u}, {"link_tree_depth", NUKA_HIP_PER_LINK, 1u}, {"link_child_range", NUKA_HIP_PER_LINK, 2u},
    {"link_children", NUKA_HIP_PER_LINK, 1u}, {"link_push_order", NUKA_HIP_PER_LINK, 1u}, {"sweep_links", NUKA_HIP_PER_SCALAR, 0u},
    {"link_dof", NUKA_HIP_PER_LINK, 1u}, {"dof_link", NUKA_HIP_PER_DOF, 1u}, {"dof_component", NUKA_HIP_PER_DOF, 1u}, {"link_dof_mask", NUKA_HIP_PER_LINK, 1u},
    {"link_geom_kind", NUKA_HIP_PER_LINK, 1u}, {"link_geom_local", NUKA_HIP_PER_LINK, 7u}, {"shape_table", NUKA_HIP_PER_SCALAR, 0u},
    {"body_to_link", NUKA_HIP_PER_BODY, 1u}, {"body_to_articulation", NUKA_HIP_PER_BODY, 1u}, {"body_collidable_link", NUKA_HIP_PER_BODY, 1u},
    {"body_collidable_body", NUKA_HIP_PER_BODY, 1u}, {"body_collidable_local", NUKA_HIP_PER_BODY, 7u}, {"pairable_rows", NUKA_HIP_PER_BODY, 1u},
    {"profile_mu", NUKA_HIP_PER_SCALAR, 0u}, {"profile_law", NUKA_HIP_PER_SCALAR, 0u}, {"profile_solref", NUKA_HIP_PER_SCALAR, 0u},
    {"profile_solimp", NUKA_HIP_PER_SCALAR, 0u}, {"profile_margin", NUKA_HIP_PER_SCALAR, 0u}, {"profile_mix", NUKA_HIP_PER_SCALAR, 0u},
    {"excluded_pairs", NUKA_HIP_PER_SCALAR, 0u}};
// A data field's entity and group from its count, evaluated at counts that are distinct primes past any group size:
// the primes that divide the count name the entity, what is left is the group.
void DataShape(size_t count, uint8_t* per, uint32_t* scalars) {
    constexpr size_t kEnvs = 2u, kLinks = 101u, kBodies = 103u, kDof = 107u, kSlots = 109u, kRows = 113u, kOwn = 127u;
    size_t rest = count / kEnvs;
    auto takes = [&](size_t prime) { if (rest % prime != 0u) return false; rest /= prime; return true; };
    if (takes(kOwn)) { *per = NUKA_HIP_PER_SCALAR; *scalars = 0u; return; }
    if (takes(kLinks)) *per = NUKA_HIP_PER_LINK;
    else if (takes(kBodies)) *per = NUKA_HIP_PER_BODY;
    else if (takes(kSlots)) *per = NUKA_HIP_PER_CONTACT_SLOT;
    else if (takes(kRows)) *per = takes(kDof) ? NUKA_HIP_PER_ROW_DOF : NUKA_HIP_PER_ROW_SLOT;
    else if (takes(kDof)) *per = takes(kDof) ? NUKA_HIP_PER_DOF2 : NUKA_HIP_PER_DOF;
    else *per = NUKA_HIP_PER_ENV;
    *scalars = uint32_t(rest);
}
extern "C++" const std::vector<ViewField>& ViewFields() {   // (a C++ return type: not a C function, though the file's entry points around it are)
    static const std::vector<ViewField> fields = [] {
        std::vector<ViewField> out;
#define X(field, dtype) { uint8_t per = NUKA_HIP_PER_SCALAR; uint32_t scalars = 0u; \
            for (const ModelShape& shape : kModelShapes) if (std::strcmp(shape.name, #field) == 0) { per = shape.per; scalars = shape.scalars; } \
            out.push_back({#field, ReferenceName(#field), 0u, uint8_t(dtype), per, scalars, offsetof(ModelView, field)}); }
        NKH_MODEL_FIELDS(X)
#undef X
        const size_t E = 2u, nl = 101u, nb = 103u, md = 107u, S = 109u, R = 113u, mf = 127u, fb = nb;
#define X(field, dtype, count) { uint8_t per = 0u; uint32_t scalars = 0u; DataShape(size_t(count), &per, &scalars); \
            out.push_back({#field, ReferenceName(#field), 1u, uint8_t(dtype), per, scalars, offsetof(DataView, field)}); }
        NKH_DATA_FIELDS(X)
#undef X
        return out;
    }();
    return fields;
}
}  // namespace
}  // namespace nkh

uint32_t nuka_hip_view_field_count(void) { return uint32_t(nkh::ViewFields().size()); }
int nuka_hip_view_field(uint32_t index, nuka_hip_view_field_t* out) {
    const auto& fields = nkh::ViewFields();
    if (out == nullptr || index >= fields.size()) return -1;
    const nkh::ViewField& f = fields[index];
    *out = {f.name, f.reference_name, f.owner, f.dtype, f.per, f.scalars};
    return 0;
}
size_t nuka_hip_model_view_bytes(void) { return sizeof(nkh::ModelView); }
size_t nuka_hip_data_view_bytes(void) { return sizeof(nkh::DataView); }
int nuka_hip_bind_views(const char* const* names, void* const* pointers, uint32_t count, nuka_phi_model_view* model, nuka_phi_data_view* data,
                        char* missing, size_t missing_bytes) {
    if (model == nullptr || data == nullptr || (count != 0u && (names == nullptr || pointers == nullptr))) return -1;
    int unset = 0;
    size_t written = 0u;
    if (missing != nullptr && missing_bytes != 0u) missing[0] = '\0';
    for (const nkh::ViewField& f : nkh::ViewFields()) {
        void** member = reinterpret_cast<void**>(reinterpret_cast<char*>(f.owner == 0u ? static_cast<void*>(model) : static_cast<void*>(data)) + f.offset);
        for (uint32_t i = 0u; i < count; ++i) {
            if (names[i] == nullptr) continue;
            if (std::strcmp(names[i], f.name) == 0 || (f.reference_name != nullptr && std::strcmp(names[i], f.reference_name) == 0)) *member = pointers[i];
        }
        if (*member != nullptr) continue;
        ++unset;
        const size_t length = std::strlen(f.name);
        if (missing != nullptr && written + length + 2u <= missing_bytes) {
            if (written != 0u) missing[written++] = ',';
            std::memcpy(missing + written, f.name, length + 1u);
            written += length;
        }
    }
    return unset;
}
int nuka_hip_model_view_set_count(nuka_phi_model_view* model, const char* name, uint32_t value) {
    if (model == nullptr || name == nullptr) return -1;
    auto* m = reinterpret_cast<nkh::ModelView*>(model);
#define COUNT(member) if (std::strcmp(name, #member) == 0) { m->member = value; return 0; }
    COUNT(links_per_env) COUNT(bodies_per_env) COUNT(dof) COUNT(max_dof) COUNT(max_depth) COUNT(contact_slots) COUNT(rows_per_env)
    COUNT(contact_rows_per_env) COUNT(profile_count) COUNT(floating_root) COUNT(max_points_per_slot) COUNT(excluded_pair_count)
    COUNT(sweep_passes) COUNT(pairable_count) COUNT(contact_dof_end) COUNT(rows_from_links) COUNT(joint_limit_rows) COUNT(joint_friction_rows) COUNT(joint_drive_rows)
    COUNT(drive_mode) COUNT(any_mujoco) COUNT(contact_cone) COUNT(integrator) COUNT(free_body)
#undef COUNT
    return -1;
}

const char* nuka_field_names(void) {
#define X(name, ...) #name ","
    return NKH_MODEL_FIELDS(X) NKH_DATA_FIELDS(X) "";
#undef X
}

nuka_state_field_t nuka_field_from_name(const char* name) {
    if (name == nullptr) return NUKA_HIP_FIELD_NONE;
    uint32_t index = 0u;
#define X(field, ...) if (std::strcmp(name, #field) == 0) return nuka_state_field_t(uint32_t(NUKA_HIP_FIELD_BASE) + index); ++index;
    NKH_MODEL_FIELDS(X)
    NKH_DATA_FIELDS(X)
#undef X
    return NUKA_HIP_FIELD_NONE;
}

namespace nkh {
namespace {
// The public field ids this library serves: the world's field behind each and the element stride of its view
// (src/c_abi/dlpack_table.hpp:101-330; element sizes of src/nk/model/fields.yaml).
struct PublicField { nuka_state_field_t id; const char* name; uint32_t stride; };
constexpr PublicField kPublicFields[] = {
    {NUKA_FIELD_RIGID_BODY_TRANSFORM, "body_pose", 28u}, {NUKA_FIELD_ARTICULATION_LINK_POSE, "link_pose", 28u},
    {NUKA_FIELD_JOINT_POSITION, "q", 4u}, {NUKA_FIELD_JOINT_VELOCITY, "qdot", 4u}, {NUKA_FIELD_CONTACT_POINTS, "contact_point", 12u},
    {NUKA_FIELD_DRIVE_TARGET, "drive_target", 4u}, {NUKA_FIELD_LINK_VELOCITY, "link_velocity", 24u},
    {NUKA_FIELD_DRIVE_STIFFNESS, "drive_stiffness", 4u}, {NUKA_FIELD_DRIVE_DAMPING, "drive_damping", 4u},
    {NUKA_FIELD_DRIVE_FORCE_LIMIT, "drive_force_limit", 4u}, {NUKA_FIELD_BASE_POSE, "base_pose", 28u},
    {NUKA_FIELD_TORQUE_INPUT, "drive_target", 4u}, {NUKA_FIELD_VELOCITY_TARGET, "velocity_target", 4u},
    {NUKA_FIELD_ACTUATOR_NOLOAD_SPEED, "actuator_noload_speed", 4u}, {NUKA_FIELD_LINK_CONTACT_WRENCH, "link_contact_wrench", 24u},
    {NUKA_FIELD_CONTACT_NORMAL, "contact_normal", 12u}, {NUKA_FIELD_CONTACT_FORCE, "contact_force", 12u},
    {NUKA_FIELD_CONTACT_LINK, "contact_link", 4u}, {NUKA_FIELD_JOINT_FEEDFORWARD, "joint_f", 4u},
    {NUKA_FIELD_JOINT_LIMIT_IMPULSE, "joint_limit_impulse", 8u}, {NUKA_FIELD_ACTUATOR_EFFORT_REQUESTED, "actuator_effort_requested", 4u},
    {NUKA_FIELD_ACTUATOR_EFFORT, "actuator_effort", 4u}, {NUKA_FIELD_ACTUATOR_SATURATED, "actuator_saturated", 4u},
    {NUKA_FIELD_CONTACT_SIDE_A_KIND, "contact_side_a_kind", 4u}, {NUKA_FIELD_CONTACT_SIDE_B_KIND, "contact_side_b_kind", 4u},
    {NUKA_FIELD_CONTACT_SIDE_A_INDEX, "contact_side_a_index", 4u}, {NUKA_FIELD_CONTACT_SIDE_B_INDEX, "contact_side_b_index", 4u},
    {NUKA_FIELD_ENV_STATUS, "env_status", 4u}, {NUKA_FIELD_CONTACT_WARM_START_COUNTS, "contact_warm_start_counts", 8u},
    {NUKA_FIELD_VBD_VELOCITY_SWEEP_COUNT, "vbd_velocity_sweep_count", 4u}, {NUKA_FIELD_UCONTACT_ROW_RANGE, "ucontact_row_range", 8u},
    {NUKA_FIELD_LINK_WRENCH, "link_wrench", 24u}, {NUKA_FIELD_UCONTACT_COUNT, "ucontact_count", 4u},
    {NUKA_FIELD_UCONTACT_POINT, "ucontact_point", 48u}, {NUKA_FIELD_SOLVER_RESIDUAL, "solver_residual", 16u},
    {NUKA_FIELD_UCONTACT_NORMAL, "ucontact_normal", 48u}, {NUKA_FIELD_UCONTACT_DEPTH, "ucontact_depth", 16u},
    {NUKA_FIELD_UCONTACT_LAW, "ucontact_law", 4u}, {NUKA_FIELD_UCONTACT_SIDE_A, "ucontact_a", 16u},
    {NUKA_FIELD_UCONTACT_SIDE_B, "ucontact_b", 16u}, {NUKA_FIELD_UCONTACT_IMPULSE, "ucontact_impulse", 48u},
    {NUKA_FIELD_JOINT_GRAVITY_FORCE, "joint_gravity_force", 4u}, {NUKA_FIELD_ROW_PENETRATION, "row_penetration", 4u},
    {NUKA_FIELD_ROW_LAMBDA, "lambda", 4u},
    {NUKA_FIELD_BODY_LINEAR_VELOCITY, "body_linear_velocity", 12u}, {NUKA_FIELD_BODY_ANGULAR_VELOCITY, "body_angular_velocity", 12u},
};

// The world's field a public or library id stands for and the stride of its view; null when the id is not served.
const Field* ResolveField(const World& w, nuka_state_field_t field, uint32_t* stride) {
    const uint32_t id = uint32_t(field);
    if (id >= uint32_t(NUKA_HIP_FIELD_BASE)) {
        const uint32_t index = id - uint32_t(NUKA_HIP_FIELD_BASE);
        if (index >= w.fields.size()) return nullptr;
        *stride = w.fields[index].elem_bytes;
        return &w.fields[index];
    }
    for (const PublicField& entry : kPublicFields) {
        if (uint32_t(entry.id) != id) continue;
        for (const Field& f : w.fields)
            if (std::strcmp(f.name, entry.name) == 0) { *stride = entry.stride; return &f; }
    }
    return nullptr;
}
}  // namespace
}  // namespace nkh

namespace nkh {
namespace {
// nk::World::DemandReadout (src/nk/pipeline/world.cpp:905-975): the first request for a contact readout field waits
// for the device, runs the readout once on the current solution and makes it part of every later step.
nuka_result_t DemandReadout(World& w, const Field& f) {
    static const char* const kContactReadout[] = {"contact_point", "contact_normal", "contact_force", "ucontact_impulse",
        "link_contact_wrench", "contact_side_a_kind", "contact_side_b_kind", "contact_side_a_index", "contact_side_b_index", "contact_link"};
    bool wanted = false;
    for (const char* name : kContactReadout) wanted = wanted || std::strcmp(f.name, name) == 0;
    if (!wanted || w.contact_readout_demanded || w.model.contact_slots == 0u) return NUKA_RESULT_OK;
    if (w.be->synchronize(w.backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "device error before the readout");
    const nuka_phi_op_call call{uint16_t(NkOp::ReadoutContactWrench), &w.p_readout_contacts};
    const uint8_t status = w.be->dispatch(w.backend, reinterpret_cast<const nuka_phi_model_view*>(&w.model),
                                          reinterpret_cast<const nuka_phi_data_view*>(&w.data), &call);
    if (status != uint8_t(Status::Ok)) return Error(MapStatus(status), "contact readout failed");
    if (w.be->synchronize(w.backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "device error in the readout");
    w.contact_readout_demanded = true;
    InvalidatePlan(w);
    BuildPipeline(w);
    return NUKA_RESULT_OK;
}
}  // namespace
}  // namespace nkh

nuka_result_t nuka_world_get_buffer_view(nuka_world_handle world, nuka_state_field_t field, nuka_buffer_view_t* out) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    uint32_t stride = 0u;
    const Field* resolved = ResolveField(*w, field, &stride);
    if (resolved == nullptr) return Error(NUKA_RESULT_NOT_SUPPORTED, "this world serves no field of that id");
    const Field& f = *resolved;
    if (const nuka_result_t demanded = DemandReadout(*w, f); demanded != NUKA_RESULT_OK) return demanded;
    out->device_ptr = static_cast<char*>(Iface(w->arena)->base(w->arena)) + f.offset;
    out->element_count = f.count * f.elem_bytes / stride;
    out->element_stride_bytes = stride;
    out->dtype = uint8_t(f.dtype);
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_upload_field(nuka_world_handle world, nuka_state_field_t field, const void* bytes, size_t nbytes, size_t byte_offset) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    uint32_t stride = 0u;
    const Field* resolved = ResolveField(*w, field, &stride);
    if (resolved == nullptr) return Error(NUKA_RESULT_NOT_SUPPORTED, "this world serves no field of that id");
    const Field& f = *resolved;
    const size_t size = f.count * f.elem_bytes;
    if (byte_offset > size || nbytes > size - byte_offset || (bytes == nullptr && nbytes > 0u)) return Error(NUKA_RESULT_INVALID_ARG, "range exceeds the field");
    if (nbytes == 0u) return NUKA_RESULT_OK;
    return MapStatus(Iface(w->arena)->upload(w->arena, bytes, f.offset + byte_offset, nbytes));
}

nuka_result_t nuka_world_download_field(nuka_world_handle world, nuka_state_field_t field, void* bytes, size_t nbytes, size_t byte_offset) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    uint32_t stride = 0u;
    const Field* resolved = ResolveField(*w, field, &stride);
    if (resolved == nullptr) return Error(NUKA_RESULT_NOT_SUPPORTED, "this world serves no field of that id");
    const Field& f = *resolved;
    const size_t size = f.count * f.elem_bytes;
    if (byte_offset > size || nbytes > size - byte_offset || (bytes == nullptr && nbytes > 0u)) return Error(NUKA_RESULT_INVALID_ARG, "range exceeds the field");
    if (nbytes == 0u) return NUKA_RESULT_OK;
    if (const nuka_result_t demanded = DemandReadout(*w, f); demanded != NUKA_RESULT_OK) return demanded;
    return MapStatus(Iface(w->arena)->download(w->arena, bytes, f.offset + byte_offset, nbytes));
}

nuka_result_t nuka_world_get_info(nuka_world_handle world, nuka_world_info_t* out) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    const ModelView& m = w->model;
    *out = {w->env_count, m.links_per_env, m.bodies_per_env, m.dof, m.max_dof, m.contact_slots, m.rows_per_env, uint32_t(w->calls.size()),
            SolverSweepWidth(m), SolverBlocksPerUnit(m, w->env_count)};
    return NUKA_RESULT_OK;
}

nuka_version_t nuka_get_version(void) { return {0u, 1u, 0u}; }   // src/c_abi/error.cpp:69-72

nuka_result_t nuka_get_runtime_info(nuka_runtime_info_t* out) {   // src/c_abi/cuda_interop.cpp:40-56
    if (out == nullptr || out->struct_size != sizeof(*out) || out->schema_version != NUKA_RUNTIME_INFO_VERSION) return NUKA_RESULT_INVALID_ARG;
    *out = {};
    out->struct_size = sizeof(*out);
    out->schema_version = NUKA_RUNTIME_INFO_VERSION;
    int runtime_version = 0, driver_version = 0;
    if (hipRuntimeGetVersion(&runtime_version) != hipSuccess || hipDriverGetVersion(&driver_version) != hipSuccess) return NUKA_RESULT_DEVICE_ERROR;
    out->cuda_runtime_version = runtime_version;
    out->cuda_driver_version = driver_version;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_stream(nuka_world_handle world, void** out_stream) {   // cuda_interop.cpp:20-28
    if (out_stream == nullptr) return NUKA_RESULT_INVALID_ARG;
    *out_stream = nullptr;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    *out_stream = BackendStream(w->device->backend);
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_record_event(nuka_world_handle world, void* cuda_event) {   // cuda_interop.cpp:30-38
    if (cuda_event == nullptr) return NUKA_RESULT_INVALID_ARG;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    return hipEventRecord(static_cast<hipEvent_t>(cuda_event), BackendStream(w->device->backend)) == hipSuccess
               ? NUKA_RESULT_OK : Error(NUKA_RESULT_DEVICE_ERROR, "event record failed");
}

nuka_result_t nuka_world_get_solver_options(nuka_world_handle world, nuka_solver_options_t* out) {   // world.cpp:759-768
    if (out == nullptr) return NUKA_RESULT_INVALID_ARG;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    // the template's integrator 0 (native) and 1 (MuJoCo's Euler) are both Euler steps; 2 runs implicitfast
    *out = {w->model.contact_cone, w->model.integrator == 2u ? 3u : 0u, w->model.contact_impratio, 1u};
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_dof_name(nuka_world_handle world, uint32_t link_index, char* out, size_t cap, size_t* out_len) {   // world.cpp:1170-1225
    if (out_len != nullptr) *out_len = 0u;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (!w->from_scene) return Error(NUKA_RESULT_NOT_SUPPORTED, "the world was not created from a scene file: its links have no names");
    const uint32_t nl = w->model.links_per_env;
    if (uint64_t{link_index} >= uint64_t{nl} * w->env_count) return Error(NUKA_RESULT_INVALID_ARG, "link index out of range");
    const uint32_t l = link_index % nl;
    std::string name = l < w->joint_names.size() ? w->joint_names[l] : std::string();
    if (name.empty() && l < w->link_names.size()) name = w->link_names[l];
    if (out_len != nullptr) *out_len = name.size();
    if (out == nullptr) return NUKA_RESULT_OK;   // size query
    if (name.size() + 1u > cap) return Error(NUKA_RESULT_INVALID_ARG, "the buffer cannot hold the name and its terminator");
    std::memcpy(out, name.c_str(), name.size() + 1u);
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_kinematic_link(nuka_world_handle world, uint32_t link_index, nuka_kinematic_link_t* out) {   // world.cpp:1227-1276
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out == nullptr) return NUKA_RESULT_INVALID_ARG;
    const HostModel& h = w->host;
    if (link_index >= w->model.links_per_env) return Error(NUKA_RESULT_INVALID_ARG, "link index out of range");
    nuka_kinematic_link_t result{};
    result.parent_index = h.parent_link[link_index];
    result.articulation_index = 0u;
    result.local_pose[3] = 1.0f;
    if (result.parent_index == kInvalid) {
        result.joint_type = NUKA_KINEMATIC_ROOT;
    } else {
        switch (h.joint_type[link_index]) {
            case kFixed: result.joint_type = NUKA_KINEMATIC_FIXED; break;
            case kRevolute: result.joint_type = NUKA_KINEMATIC_REVOLUTE; break;
            case kPrismatic: result.joint_type = NUKA_KINEMATIC_PRISMATIC; break;
            default: return Error(NUKA_RESULT_NOT_SUPPORTED, "joint type without a kinematic record");
        }
        const float* local = h.link_local_pose.data() + 7u * link_index;
        for (int k = 0; k < 3; ++k) result.local_pose[k] = local[k] + h.parent_offset[3u * link_index + k];
        for (int k = 3; k < 7; ++k) result.local_pose[k] = local[k];
        for (int k = 0; k < 3; ++k) result.axis[k] = h.joint_axis[3u * link_index + k];
    }
    *out = result;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_link_binding(nuka_world_handle world, uint32_t link_index, nuka_link_binding_t* out) {   // world.cpp:1278-1294
    if (out == nullptr) return NUKA_RESULT_INVALID_ARG;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    const HostModel& h = w->host;
    if (link_index >= w->model.links_per_env) return Error(NUKA_RESULT_INVALID_ARG, "link index out of range");
    out->body_index = h.link_body[link_index];
    out->articulation_index = 0u;
    out->is_root = h.parent_link[link_index] == kInvalid ? 1u : 0u;
    out->is_floating = out->is_root != 0u && h.joint_type[link_index] == kFloatingBase ? 1u : 0u;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_colliders(nuka_world_handle world, uint32_t env_index, nuka_collider_t* out, uint32_t capacity,
                                       uint32_t* out_count) {   // world.cpp:1345-1413
    if (out_count == nullptr) return NUKA_RESULT_INVALID_ARG;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    const HostModel& h = w->host;
    const uint32_t nb = w->model.bodies_per_env, nl = w->model.links_per_env;
    *out_count = nb;
    if (out == nullptr) return NUKA_RESULT_OK;
    if (capacity < nb || env_index >= w->env_count) return Error(NUKA_RESULT_INVALID_ARG, "capacity below the shape rows, or environment out of range");
    try {
        std::vector<float> body_pose(size_t{nb} * 7u), link_pose(size_t{nl} * 7u);
        const nuka_result_t synced = nuka_world_synchronize(world);
        if (synced != NUKA_RESULT_OK) return synced;
        auto fetch = [&](const float* field, std::vector<float>& host, uint32_t per_env) {
            if (per_env == 0u) return true;
            const char* base = static_cast<const char*>(Iface(w->arena)->base(w->arena));
            const size_t offset = size_t(reinterpret_cast<const char*>(field) - base) + size_t{env_index} * per_env * sizeof(float);
            return Iface(w->arena)->download(w->arena, host.data(), offset, size_t{per_env} * sizeof(float)) == uint8_t(Status::Ok);
        };
        if (!fetch(w->data.body_pose, body_pose, nb * 7u) || !fetch(w->data.link_pose, link_pose, nl * 7u)) return Error(NUKA_RESULT_INTERNAL, "pose download failed");
        // parent * child: the child's origin carried by the parent, the rotations multiplied and normalised (math/transform.hpp:37-42)
        auto compose = [](const float* parent, const float* child, float* result) {
            const float w0 = parent[3], x0 = parent[4], y0 = parent[5], z0 = parent[6];
            const float v[3] = {child[0], child[1], child[2]};
            const float t[3] = {2.0f * (y0 * v[2] - z0 * v[1]), 2.0f * (z0 * v[0] - x0 * v[2]), 2.0f * (x0 * v[1] - y0 * v[0])};
            result[0] = parent[0] + v[0] + w0 * t[0] + (y0 * t[2] - z0 * t[1]);
            result[1] = parent[1] + v[1] + w0 * t[1] + (z0 * t[0] - x0 * t[2]);
            result[2] = parent[2] + v[2] + w0 * t[2] + (x0 * t[1] - y0 * t[0]);
            const float w1 = child[3], x1 = child[4], y1 = child[5], z1 = child[6];
            float q[4] = {w0 * w1 - x0 * x1 - y0 * y1 - z0 * z1, w0 * x1 + x0 * w1 + y0 * z1 - z0 * y1,
                          w0 * y1 - x0 * z1 + y0 * w1 + z0 * x1, w0 * z1 + x0 * y1 - y0 * x1 + z0 * w1};
            const float norm = std::sqrt(q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3]);
            for (int k = 0; k < 4; ++k) result[3 + k] = norm > 0.0f ? q[k] / norm : (k == 0 ? 1.0f : 0.0f);
        };
        for (uint32_t row = 0u; row < nb; ++row) {
            const float* shape = h.shape_table.data() + size_t{row} * kShapeStride;
            nuka_collider_t& collider = out[row];
            std::memcpy(&collider.kind, shape, sizeof(uint32_t));
            std::memcpy(collider.params, shape + 1, 4u * sizeof(float));
            int32_t body_id;
            std::memcpy(&body_id, shape + 8, sizeof(body_id));
            float pose[7] = {0.0f, 0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 0.0f};
            bool is_static = true;
            if (body_id >= 0) {
                const uint32_t body = uint32_t(body_id);
                const uint32_t link = body < h.body_to_link.size() ? h.body_to_link[body] : kInvalid;
                const uint32_t owner = body < h.body_collidable_link.size() ? h.body_collidable_link[body] : kInvalid;
                if (link != kInvalid || owner != kInvalid) {
                    // a link's own row hangs off the link by the link's shape frame, a further row of a link by its own
                    if (owner != kInvalid) compose(link_pose.data() + 7u * owner, h.body_collidable_local.data() + 7u * body, pose);
                    else compose(link_pose.data() + 7u * link, h.link_geom_local.data() + 7u * link, pose);
                    is_static = false;
                } else {
                    std::memcpy(pose, body_pose.data() + 7u * body, sizeof(pose));
                }
            } else if (row < nb) {
                std::memcpy(pose, body_pose.data() + 7u * row, sizeof(pose));
            }
            collider.is_static = is_static ? 1u : 0u;
            std::memcpy(collider.pose, pose, sizeof(pose));
        }
        return NUKA_RESULT_OK;
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    }
}

nuka_result_t nuka_device_get_resource_info(nuka_device_handle device, nuka_device_resource_info_t* out) {   // src/c_abi/device.cpp:101-108
    auto* record = reinterpret_cast<DeviceRecord*>(device);
    if (record == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "device is null");
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    auto* backend = reinterpret_cast<nuka_phi_backend*>(record->backend);
    const nuka_phi_resource_info info = reinterpret_cast<nuka_phi_backend_head*>(backend)->iface->resource_info(backend);
    *out = {info.free_bytes, info.total_bytes, info.thread_stack_limit_bytes, info.graph_used_bytes, info.graph_reserved_bytes,
            info.compute_units, info.threads_per_unit};
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_resource_info(nuka_world_handle world, nuka_world_resource_info_t* out) {   // src/c_abi/world.cpp:917-929
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    uint64_t model = 0u, persistent = 0u, scratch = 0u;
    for (const Field& f : w->fields) {
        const uint64_t bytes = (uint64_t{f.count} * f.elem_bytes + 255u) & ~uint64_t{255u};   // as the arena places it
        (f.is_template ? model : CheckpointKeeps(f.name) ? persistent : scratch) += bytes;
    }
    const ModelView& m = w->model;
    *out = {model, persistent, scratch, w->env_count, m.contact_slots, m.rows_per_env, m.dof, m.bodies_per_env, 0u};
    return NUKA_RESULT_OK;
}

uint32_t nuka_world_resource_field_count(nuka_world_handle world) {   // world.cpp:931-936
    auto* w = reinterpret_cast<World*>(world);
    return w == nullptr ? 0u : uint32_t(w->fields.size());
}

nuka_result_t nuka_world_get_resource_fields(nuka_world_handle world, nuka_resource_field_t* out) {   // world.cpp:938-959
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    uint32_t index = 0u;
    for (const bool template_pass : {true, false})   // the model's fields first, as the reference lists them
        for (const Field& f : w->fields) {
            if (f.is_template != template_pass) continue;
            nuka_resource_field_t& field = out[index++];
            const char* reference_name = ReferenceName(f.name);
            std::snprintf(field.name, sizeof(field.name), "%s", reference_name != nullptr && reference_name[0] != '\0' ? reference_name : f.name);
            field.offset = f.offset;
            field.bytes = uint64_t{f.count} * f.elem_bytes;
            field.owner = f.is_template ? 0u : 1u;
            field.arena = f.is_template || CheckpointKeeps(f.name) ? 0u : 1u;
        }
    return NUKA_RESULT_OK;
}

namespace nkh {
namespace {
struct ExecutionWindow {   // world.cpp:910-914
    nuka_phi_event* start;
    nuka_phi_event* end;
    uint64_t replays;
    uint64_t owner_id;
};
}  // namespace
}  // namespace nkh

nuka_result_t nuka_world_begin_execution_window(nuka_world_handle world, void** window) {   // world.cpp:961-969
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (window == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "window is null");
    *window = nullptr;
    auto interval = std::make_unique<nkh::ExecutionWindow>();
    interval->start = w->be->event_new(w->backend);
    interval->end = w->be->event_new(w->backend);
    if (interval->start == nullptr || interval->end == nullptr) {
        if (interval->start != nullptr) w->be->event_free(w->backend, interval->start);
        if (interval->end != nullptr) w->be->event_free(w->backend, interval->end);
        return Error(NUKA_RESULT_DEVICE_ERROR, "event creation failed");
    }
    interval->replays = w->graph_replays;
    interval->owner_id = w->id;
    w->be->event_record(w->backend, interval->start);
    *window = interval.release();
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_end_execution_window(nuka_world_handle world, void* window, nuka_execution_window_t* out) {   // world.cpp:971-990
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    auto* interval = static_cast<nkh::ExecutionWindow*>(window);
    if (interval == nullptr || out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "window and out are required");
    if (interval->owner_id != w->id) return Error(NUKA_RESULT_INVALID_ARG, "the window was opened on another world");
    w->be->event_record(w->backend, interval->end);
    const uint8_t waited = w->be->synchronize(w->backend, nullptr);   // the elapsed time exists once the end event has completed
    nuka_phi_plan_metrics metrics{};
    if (w->plan != nullptr) metrics = w->be->plan_metrics(w->backend, w->plan);
    *out = {double(w->be->event_elapsed_ms(w->backend, interval->start, interval->end)), w->graph_replays - interval->replays, metrics.nodes,
            metrics.kernels, metrics.clears, metrics.copies};
    w->be->event_free(w->backend, interval->start);
    w->be->event_free(w->backend, interval->end);
    delete interval;
    return waited == uint8_t(Status::Ok) ? NUKA_RESULT_OK : Error(NUKA_RESULT_DEVICE_ERROR, "device error inside the window");
}

nuka_result_t nuka_world_time_steps(nuka_world_handle world, nuka_checkpoint_handle from, uint32_t step_count, float* out_total_ms) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out_total_ms == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    if (from != nullptr && !OwnedBy(reinterpret_cast<Checkpoint*>(from), w)) return Error(NUKA_RESULT_INVALID_ARG, "checkpoint belongs to another world");
    nuka_phi_event* start = w->be->event_new(w->backend);
    nuka_phi_event* stop = w->be->event_new(w->backend);
    if (start == nullptr || stop == nullptr) return Error(NUKA_RESULT_DEVICE_ERROR, "event creation failed");
    w->be->event_record(w->backend, start);
    nuka_result_t r = NUKA_RESULT_OK;
    if (from == nullptr) r = StepN(*w, step_count);
    else
        for (uint32_t s = 0u; s < step_count && r == NUKA_RESULT_OK; ++s) {
            r = nuka_world_checkpoint_restore(world, from);
            if (r == NUKA_RESULT_OK) r = StepN(*w, 1u);
        }
    w->be->event_record(w->backend, stop);
    w->be->event_wait(w->backend, stop);
    *out_total_ms = w->be->event_elapsed_ms(w->backend, start, stop);
    w->be->event_free(w->backend, start);
    w->be->event_free(w->backend, stop);
    return r;
}

nuka_result_t nuka_world_profile_ops(nuka_world_handle world, nuka_checkpoint_handle from, uint32_t step_count, float* out_ms,
                                     uint16_t* out_ops) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out_ms == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    if (from != nullptr && !OwnedBy(reinterpret_cast<Checkpoint*>(from), w)) return Error(NUKA_RESULT_INVALID_ARG, "checkpoint belongs to another world");
    const size_t n = w->calls.size();
    std::vector<nuka_phi_event*> events(n + 1u, nullptr);
    for (auto& e : events) e = w->be->event_new(w->backend);
    for (size_t i = 0u; i < n; ++i) { out_ms[i] = 0.0f; if (out_ops != nullptr) out_ops[i] = w->calls[i].op; }
    nuka_result_t result = NUKA_RESULT_OK;
    for (uint32_t s = 0u; s < step_count && result == NUKA_RESULT_OK; ++s) {
        if (from != nullptr && (result = nuka_world_checkpoint_restore(world, from)) != NUKA_RESULT_OK) break;
        w->be->event_record(w->backend, events[0]);
        for (size_t i = 0u; i < n; ++i) {
            const uint8_t status = w->be->dispatch(w->backend, reinterpret_cast<const nuka_phi_model_view*>(&w->model),
                                                   reinterpret_cast<const nuka_phi_data_view*>(&w->data), &w->calls[i]);
            if (status != uint8_t(Status::Ok)) { result = Error(MapStatus(status), "profile dispatch failed"); break; }
            w->be->event_record(w->backend, events[i + 1u]);
        }
        w->be->event_wait(w->backend, events[n]);
        if (result == NUKA_RESULT_OK)
            for (size_t i = 0u; i < n; ++i) out_ms[i] += w->be->event_elapsed_ms(w->backend, events[i], events[i + 1u]);
    }
    (void)w->be->synchronize(w->backend, nullptr);
    for (auto* e : events) w->be->event_free(w->backend, e);
    return result;
}

nuka_result_t nuka_device_copy_bandwidth(nuka_device_handle device, size_t bytes, uint32_t repeats, float* out_gb_per_s) {
    auto* record = reinterpret_cast<DeviceRecord*>(device);
    if (record == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "device is null");
    if (out_gb_per_s == nullptr || bytes == 0u || repeats == 0u) return Error(NUKA_RESULT_INVALID_ARG, "bytes, repeats and out are required");
    auto* backend = reinterpret_cast<nuka_phi_backend*>(record->backend);
    const nuka_phi_backend_i* be = reinterpret_cast<nuka_phi_backend_head*>(backend)->iface;
    nuka_phi_buffer_type* type = BackendDeviceBufferType(record->backend);
    uint8_t status = 0u;
    nuka_phi_buffer* a = reinterpret_cast<nuka_phi_buffer_type_head*>(type)->iface->alloc(type, bytes, &status);
    nuka_phi_buffer* b = reinterpret_cast<nuka_phi_buffer_type_head*>(type)->iface->alloc(type, bytes, &status);
    if (a == nullptr || b == nullptr) {
        if (a != nullptr) Iface(a)->free(a);
        if (b != nullptr) Iface(b)->free(b);
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "copy buffers");
    }
    (void)Iface(a)->memset(a, 1u, 0u, bytes);
    (void)Iface(b)->copy_from(b, a, 0u, 0u, bytes);
    nuka_phi_event* start = be->event_new(backend);
    nuka_phi_event* stop = be->event_new(backend);
    be->event_record(backend, start);
    for (uint32_t i = 0u; i < repeats; ++i) (void)Iface(b)->copy_from(b, a, 0u, 0u, bytes);
    be->event_record(backend, stop);
    be->event_wait(backend, stop);
    const float ms = be->event_elapsed_ms(backend, start, stop);
    be->event_free(backend, start);
    be->event_free(backend, stop);
    Iface(a)->free(a);
    Iface(b)->free(b);
    *out_gb_per_s = ms > 0.0f ? float(2.0 * double(bytes) * repeats / (double(ms) * 1.0e6)) : 0.0f;
    return NUKA_RESULT_OK;
}

namespace nkh {
namespace {
// A checkpoint's storage and segment table for `w`, nothing copied yet.
nuka_result_t NewCheckpoint(World* w, std::unique_ptr<Checkpoint>* out) {
    auto cp = std::unique_ptr<Checkpoint>(new (std::nothrow) Checkpoint{});
    if (!cp) return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    cp->owner = w;
    cp->owner_id = w->id;
    size_t total = 0u;
    for (const Field& f : w->fields) {
        if (f.is_template || f.count == 0u || !(CheckpointKeeps(f.name) || CheckpointClears(f.name))) continue;
        if (cp->segments.count == kMaxCheckpointSegments) return Error(NUKA_RESULT_INTERNAL, "too many checkpoint segments");
        if (CheckpointKeeps(f.name)) total += (f.count * f.elem_bytes + 255u) & ~size_t{255u};
        ++cp->segments.count;
    }
    uint8_t status = 0u;
    nuka_phi_buffer_type* type = BackendDeviceBufferType(w->device->backend);
    cp->store = reinterpret_cast<nuka_phi_buffer_type_head*>(type)->iface->alloc(type, total, &status);
    if (cp->store == nullptr) return Error(NUKA_RESULT_OUT_OF_MEMORY, "checkpoint allocation failed");
    char* arena = static_cast<char*>(Iface(w->arena)->base(w->arena));
    char* kept = static_cast<char*>(Iface(cp->store)->base(cp->store));
    uint32_t at = 0u;
    size_t offset = 0u;
    for (const Field& f : w->fields) {
        if (f.is_template || f.count == 0u || !(CheckpointKeeps(f.name) || CheckpointClears(f.name))) continue;
        const size_t padded = (f.count * f.elem_bytes + 255u) & ~size_t{255u};    // arena fields are 256-byte aligned and padded
        cp->segments.live[at] = arena + f.offset;
        cp->segments.units[at] = uint32_t(padded / 16u);
        if (CheckpointKeeps(f.name)) { cp->segments.kept[at] = kept + offset; offset += padded; }
        else cp->segments.kept[at] = nullptr;
        ++at;
    }
    cp->bytes = total;
    *out = std::move(cp);
    return NUKA_RESULT_OK;
}

// What a checkpoint file has to agree on with the world that reads it: the environment count and every kept field's
// name and size, FNV-1a hashed.
uint64_t CheckpointLayoutHash(const World& w) {
    uint64_t hash = 14695981039346656037ull;
    auto mix = [&hash](const void* bytes, size_t count) {
        const auto* p = static_cast<const uint8_t*>(bytes);
        for (size_t i = 0u; i < count; ++i) { hash ^= p[i]; hash *= 1099511628211ull; }
    };
    const uint64_t envs = w.env_count;
    mix(&envs, sizeof(envs));
    for (const Field& f : w.fields) {
        if (f.is_template || f.count == 0u || !CheckpointKeeps(f.name)) continue;
        const uint64_t bytes = f.count * f.elem_bytes;
        mix(f.name, std::strlen(f.name) + 1u);
        mix(&bytes, sizeof(bytes));
    }
    return hash;
}
struct CheckpointFileHeader { char magic[8]; uint64_t layout_hash, bytes, param_values; };
constexpr char kCheckpointMagic[8] = {'N', 'K', 'H', 'C', 'K', 'P', 'T', '2'};

// Every live parameter of the world as the public getters report it.
nuka_result_t ReadLiveParams(World* w, LiveParams* out) {
    out->values.clear();
    uint32_t count = 0u;
    if (const nuka_result_t r = nuka_world_param_count(reinterpret_cast<nuka_world_handle>(w), &count); r != NUKA_RESULT_OK) return r;
    std::vector<nuka_param_info_t> infos(count);
    for (auto& info : infos) { info.struct_size = sizeof(info); info.schema_version = NUKA_PARAM_INFO_VERSION; }
    if (const nuka_result_t r = nuka_world_get_param_infos(reinterpret_cast<nuka_world_handle>(w), infos.data(), count); r != NUKA_RESULT_OK) return r;
    for (uint32_t p = 0u; p < count; ++p)
        for (uint32_t e = 0u; e < infos[p].count; ++e) {
            double value = 0.0;
            if (const nuka_result_t r = nuka_world_get_param(reinterpret_cast<nuka_world_handle>(w), p, e, &value); r != NUKA_RESULT_OK) return r;
            out->values.push_back(value);
        }
    return NUKA_RESULT_OK;
}
// Brings the world's live parameters to `wanted` through the public setter (which keeps the device tables, the reset
// snapshot and the host mirrors in step); nothing happens when they already agree, as on every restore of a
// checkpoint taken since the last parameter change.
nuka_result_t ApplyLiveParams(World* w, const LiveParams& wanted) {
    LiveParams current;
    if (const nuka_result_t r = ReadLiveParams(w, &current); r != NUKA_RESULT_OK) return r;
    if (current == wanted) return NUKA_RESULT_OK;
    if (current.values.size() != wanted.values.size()) return Error(NUKA_RESULT_INVALID_ARG, "the checkpoint holds another number of parameters");
    uint32_t count = 0u;
    if (const nuka_result_t r = nuka_world_param_count(reinterpret_cast<nuka_world_handle>(w), &count); r != NUKA_RESULT_OK) return r;
    std::vector<nuka_param_info_t> infos(count);
    for (auto& info : infos) { info.struct_size = sizeof(info); info.schema_version = NUKA_PARAM_INFO_VERSION; }
    if (const nuka_result_t r = nuka_world_get_param_infos(reinterpret_cast<nuka_world_handle>(w), infos.data(), count); r != NUKA_RESULT_OK) return r;
    size_t at = 0u;
    for (uint32_t p = 0u; p < count; ++p)
        for (uint32_t e = 0u; e < infos[p].count; ++e, ++at)
            if (current.values[at] != wanted.values[at])
                if (const nuka_result_t r = nuka_world_set_param(reinterpret_cast<nuka_world_handle>(w), p, e, wanted.values[at]); r != NUKA_RESULT_OK) return r;
    return NUKA_RESULT_OK;
}
}  // namespace
}  // namespace nkh

nuka_result_t nuka_world_checkpoint_capture(nuka_world_handle world, nuka_checkpoint_handle* out) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out = nullptr;
    std::unique_ptr<Checkpoint> cp;
    if (const nuka_result_t made = NewCheckpoint(w, &cp); made != NUKA_RESULT_OK) return made;
    hipLaunchKernelGGL(CheckpointCopyKernel, dim3(256, cp->segments.count), dim3(256), 0, BackendStream(w->device->backend), cp->segments, 0u);
    if (hipGetLastError() != hipSuccess || nuka_world_synchronize(world) != NUKA_RESULT_OK) {
        Iface(cp->store)->free(cp->store);
        return Error(NUKA_RESULT_DEVICE_ERROR, "checkpoint capture failed");
    }
    cp->layout_hash = CheckpointLayoutHash(*w);
    if (const nuka_result_t r = ReadLiveParams(w, &cp->params); r != NUKA_RESULT_OK) { Iface(cp->store)->free(cp->store); return r; }
    cp->param_version = w->param_version;
    *out = reinterpret_cast<nuka_checkpoint_handle>(cp.release());
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_checkpoint_write(nuka_checkpoint_handle checkpoint, const char* path) {
    auto* cp = reinterpret_cast<Checkpoint*>(checkpoint);
    if (cp == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "checkpoint is null");
    if (path == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "path is null");
    try {
        std::vector<uint8_t> bytes(cp->bytes);
        if (cp->bytes > 0u && Iface(cp->store)->download(cp->store, bytes.data(), 0u, cp->bytes) != uint8_t(Status::Ok))
            return Error(NUKA_RESULT_DEVICE_ERROR, "checkpoint download failed");
        CheckpointFileHeader header{};
        std::memcpy(header.magic, kCheckpointMagic, sizeof(header.magic));
        header.layout_hash = cp->layout_hash;   // taken at capture: the world may be gone by now
        header.bytes = cp->bytes;
        header.param_values = cp->params.values.size();
        std::FILE* file = std::fopen(path, "wb");
        if (file == nullptr) return Error(NUKA_RESULT_INVALID_ARG, std::string("cannot open ") + path);
        const bool ok = std::fwrite(&header, sizeof(header), 1u, file) == 1u && (bytes.empty() || std::fwrite(bytes.data(), bytes.size(), 1u, file) == 1u) &&
                        (cp->params.values.empty() || std::fwrite(cp->params.values.data(), cp->params.values.size() * sizeof(double), 1u, file) == 1u);
        if (std::fclose(file) != 0 || !ok) return Error(NUKA_RESULT_INTERNAL, std::string("write failed: ") + path);
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    }
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_checkpoint_read(nuka_world_handle world, const char* path, nuka_checkpoint_handle* out) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (path == nullptr || out == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "path and out are required");
    *out = nullptr;
    std::FILE* file = std::fopen(path, "rb");
    if (file == nullptr) return Error(NUKA_RESULT_INVALID_ARG, std::string("cannot open ") + path);
    nuka_result_t result = NUKA_RESULT_OK;
    try {
        CheckpointFileHeader header{};
        std::unique_ptr<Checkpoint> cp;
        if (std::fread(&header, sizeof(header), 1u, file) != 1u || std::memcmp(header.magic, kCheckpointMagic, sizeof(header.magic)) != 0)
            result = Error(NUKA_RESULT_INVALID_ARG, "not a checkpoint file");
        else if (header.layout_hash != CheckpointLayoutHash(*w))
            result = Error(NUKA_RESULT_INVALID_ARG, "the checkpoint was written by a world of another layout");
        else if ((result = NewCheckpoint(w, &cp)) == NUKA_RESULT_OK) {
            std::vector<uint8_t> bytes(cp->bytes);
            if (header.bytes != cp->bytes || (!bytes.empty() && std::fread(bytes.data(), bytes.size(), 1u, file) != 1u))
                result = Error(NUKA_RESULT_INVALID_ARG, "truncated checkpoint file");
            else if (!bytes.empty() && Iface(cp->store)->upload(cp->store, bytes.data(), 0u, bytes.size()) != uint8_t(Status::Ok))
                result = Error(NUKA_RESULT_DEVICE_ERROR, "checkpoint upload failed");
            if (result == NUKA_RESULT_OK) {
                cp->layout_hash = header.layout_hash;
                cp->params.values.resize(header.param_values < (1u << 24u) ? header.param_values : 0u);
                if (cp->params.values.size() != header.param_values ||
                    (!cp->params.values.empty() && std::fread(cp->params.values.data(), cp->params.values.size() * sizeof(double), 1u, file) != 1u))
                    result = Error(NUKA_RESULT_INVALID_ARG, "truncated checkpoint file");
            }
            if (result == NUKA_RESULT_OK && nuka_world_synchronize(world) != NUKA_RESULT_OK) result = NUKA_RESULT_DEVICE_ERROR;
            if (result != NUKA_RESULT_OK) Iface(cp->store)->free(cp->store);
            else *out = reinterpret_cast<nuka_checkpoint_handle>(cp.release());
        }
    } catch (const std::bad_alloc&) {
        result = Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    }
    std::fclose(file);
    return result;
}

nuka_result_t nuka_world_get_execution_info(nuka_world_handle world, nuka_world_execution_info_t* out) {   // src/c_abi/world.cpp:890-909
    if (out == nullptr || out->struct_size != sizeof(*out) || out->schema_version != NUKA_EXECUTION_INFO_VERSION)
        return Error(NUKA_RESULT_INVALID_ARG, "struct_size or schema_version mismatch");
    *out = {};
    out->struct_size = sizeof(*out);
    out->schema_version = NUKA_EXECUTION_INFO_VERSION;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    out->mode = w->mode;
    out->graph_ready = w->plan != nullptr ? 1u : 0u;
    out->capture_attempts = w->capture_attempts;
    out->graph_replays = w->graph_replays;
    out->last_result = MapStatus(w->last_error.status);
    out->failed_op = w->last_error.failed_op;
    out->native_error = w->last_error.native_code;
    std::snprintf(out->message, sizeof(out->message), "%s", w->last_error.message);
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_checkpoint_restore(nuka_world_handle world, nuka_checkpoint_handle checkpoint) {
    auto* w = reinterpret_cast<World*>(world);
    auto* cp = reinterpret_cast<Checkpoint*>(checkpoint);
    if (w == nullptr || cp == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world or checkpoint is null");
    if (!OwnedBy(cp, w)) return Error(NUKA_RESULT_INVALID_ARG, "checkpoint belongs to another world");
    // no parameter call since the checkpoint's values were last seen to be the world's: nothing to compare, the restore
    // only enqueues its copy
    if (cp->param_version != w->param_version) {
        if (const nuka_result_t r = ApplyLiveParams(w, cp->params); r != NUKA_RESULT_OK) return r;
        cp->param_version = w->param_version;
    }
    hipLaunchKernelGGL(CheckpointCopyKernel, dim3(256, cp->segments.count), dim3(256), 0, BackendStream(w->device->backend), cp->segments, 1u);
    return hipGetLastError() == hipSuccess ? NUKA_RESULT_OK : Error(NUKA_RESULT_DEVICE_ERROR, "checkpoint restore failed");
}

void nuka_checkpoint_destroy(nuka_checkpoint_handle checkpoint) {
    auto* cp = reinterpret_cast<Checkpoint*>(checkpoint);
    if (cp == nullptr) return;
    if (cp->store != nullptr) Iface(cp->store)->free(cp->store);
    delete cp;
}

nuka_result_t nuka_checkpoint_byte_size(nuka_checkpoint_handle checkpoint, uint64_t* out_bytes) {
    auto* cp = reinterpret_cast<Checkpoint*>(checkpoint);
    if (cp == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "checkpoint is null");
    if (out_bytes == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out_bytes = cp->bytes;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_checkpoint_equal(nuka_checkpoint_handle a, nuka_checkpoint_handle b, uint32_t* out_equal) {
    auto* x = reinterpret_cast<Checkpoint*>(a);
    auto* y = reinterpret_cast<Checkpoint*>(b);
    if (x == nullptr || y == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "checkpoint is null");
    if (out_equal == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out_equal = 0u;
    bool same_layout = x->bytes == y->bytes && x->segments.count == y->segments.count;
    for (uint32_t s = 0u; same_layout && s < x->segments.count; ++s)
        same_layout = x->segments.units[s] == y->segments.units[s] && (x->segments.kept[s] == nullptr) == (y->segments.kept[s] == nullptr);
    if (!same_layout) return NUKA_RESULT_OK;
    try {
        std::vector<uint8_t> left(x->bytes), right(y->bytes);
        if (x->bytes > 0u && (Iface(x->store)->download(x->store, left.data(), 0u, x->bytes) != uint8_t(Status::Ok) ||
                              Iface(y->store)->download(y->store, right.data(), 0u, y->bytes) != uint8_t(Status::Ok)))
            return Error(NUKA_RESULT_DEVICE_ERROR, "checkpoint download failed");
        *out_equal = left == right && x->params == y->params ? 1u : 0u;
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    }
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_state_hash(nuka_world_handle world, uint64_t* out_hash) {
    if (out_hash == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    *out_hash = 0u;
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (nuka_world_synchronize(world) != NUKA_RESULT_OK) return NUKA_RESULT_DEVICE_ERROR;
    uint64_t hash = 14695981039346656037ull;   // FNV-1a (src/c_abi/checkpoint.cpp:47-57)
    auto mix = [&hash](const void* bytes, size_t count) {
        const auto* p = static_cast<const uint8_t*>(bytes);
        for (size_t i = 0u; i < count; ++i) { hash ^= p[i]; hash *= 1099511628211ull; }
    };
    constexpr char domain[] = "NukaHipStateHashV1";
    mix(domain, sizeof(domain));
    uint64_t byte_count = 0u;
    for (const Field& f : w->fields) if (!f.is_template && CheckpointKeeps(f.name)) byte_count += f.count * f.elem_bytes;
    mix(&byte_count, sizeof(byte_count));
    try {
        std::vector<uint8_t> bytes;
        for (const Field& f : w->fields) {
            if (f.is_template || f.count == 0u || !CheckpointKeeps(f.name)) continue;
            bytes.resize(f.count * f.elem_bytes);
            if (Iface(w->arena)->download(w->arena, bytes.data(), f.offset, bytes.size()) != uint8_t(Status::Ok))
                return Error(NUKA_RESULT_DEVICE_ERROR, "state download failed");
            mix(bytes.data(), bytes.size());
        }
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    }
    LiveParams params;   // a world that differs in a live parameter alone is another state
    if (const nuka_result_t r = ReadLiveParams(w, &params); r != NUKA_RESULT_OK) return r;
    if (!params.values.empty()) mix(params.values.data(), params.values.size() * sizeof(double));
    *out_hash = hash;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_forward_kinematics(nuka_world_handle world) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    const nuka_phi_op_call fk{uint16_t(NkOp::FkWorldPoses), &w->p_fk}, sync{uint16_t(NkOp::SyncLinkBodyPose), &w->p_sync};
    for (const nuka_phi_op_call* call : {&fk, &sync}) {
        if (call == &sync && w->model.bodies_per_env == 0u) break;
        const uint8_t status = w->be->dispatch(w->backend, reinterpret_cast<const nuka_phi_model_view*>(&w->model),
                                               reinterpret_cast<const nuka_phi_data_view*>(&w->data), call);
        if (status != uint8_t(Status::Ok)) return Error(MapStatus(status), std::string("dispatch failed: ") + OpName(static_cast<NkOp>(call->op)));
    }
    return NUKA_RESULT_OK;
}

extern "C++" {
namespace nkh {
namespace {
// src/c_abi/params.cpp:24-57
enum Param : uint32_t { kGravityZ, kVelocityIterations, kLinkMass, kJointDamping, kJointArmature, kJointFrictionloss, kDriveStiffness, kDriveForceLimit, kParamCount };
struct ParamDef { const char* key; const char* unit; const char* scene_field; nuka_param_type_t type; double min_value, max_value; };
constexpr double kFloatMin = 1.1754943508222875e-38, kFloatMax = 3.4028234663852886e38;
constexpr ParamDef kParams[kParamCount] = {
    {"gravity_z", "m/s^2", "", NUKA_PARAM_F32, -1000.0, 1000.0},
    {"velocity_iterations", "", "", NUKA_PARAM_U32, 1.0, 65535.0},
    {"link_mass", "kg", "body.mass", NUKA_PARAM_F32, kFloatMin, kFloatMax},
    {"joint_damping", "N*m*s/rad", "joint.damping", NUKA_PARAM_F32, 0.0, kFloatMax},
    {"joint_armature", "kg*m^2", "joint.armature", NUKA_PARAM_F32, 0.0, kFloatMax},
    {"joint_frictionloss", "N*m", "joint.frictionloss", NUKA_PARAM_F32, 0.0, kFloatMax},
    {"drive_stiffness", "N*m/rad", "actuator.gain", NUKA_PARAM_F32, 0.0, kFloatMax},
    {"drive_force_limit", "N*m", "actuator.force_limit", NUKA_PARAM_F32, 0.0, kFloatMax},
};
uint32_t ParamElements(const World& w, uint32_t p) { return p >= kLinkMass ? w.model.links_per_env : 1u; }
nuka_param_tier_t ParamTier(const World& w, uint32_t p) {   // params.cpp:66-72
    return p == kJointFrictionloss && w.model.joint_friction_rows == 0u ? NUKA_PARAM_REBUILD : NUKA_PARAM_LIVE;
}

const Field* FindField(const World& w, const char* name) {
    for (const Field& f : w.fields) if (std::strcmp(f.name, name) == 0) return &f;
    return nullptr;
}

// One value of a template table: the live arena and the snapshot a reset copies back.
bool PutTemplate(World& w, const char* name, size_t first, const float* values, size_t count) {
    const Field* f = FindField(w, name);
    if (f == nullptr || (first + count) > f->count) return false;
    const size_t offset = f->offset + first * sizeof(float), bytes = count * sizeof(float);
    return Iface(w.arena)->upload(w.arena, values, offset, bytes) == uint8_t(Status::Ok) &&
           Iface(w.initial)->upload(w.initial, values, offset, bytes) == uint8_t(Status::Ok);
}

// One link's column of an environment-major field, in the live arena and in the reset snapshot.
__global__ void __launch_bounds__(256) FillLinkColumnKernel(float* live, float* initial, uint32_t env_count, uint32_t links, uint32_t link, float value) {
    for (uint32_t env = blockIdx.x * blockDim.x + threadIdx.x; env < env_count; env += gridDim.x * blockDim.x) {
        live[size_t{env} * links + link] = value;
        initial[size_t{env} * links + link] = value;
    }
}
bool PutColumn(World& w, const char* name, uint32_t link, float value) {
    const Field* f = FindField(w, name);
    if (f == nullptr || f->count != size_t{w.env_count} * w.model.links_per_env) return false;
    char* live = static_cast<char*>(Iface(w.arena)->base(w.arena));
    char* initial = static_cast<char*>(Iface(w.initial)->base(w.initial));
    hipLaunchKernelGGL(FillLinkColumnKernel, dim3(std::min((w.env_count + 255u) / 256u, 1024u)), dim3(256), 0, BackendStream(w.device->backend),
                       reinterpret_cast<float*>(live + f->offset), reinterpret_cast<float*>(initial + f->offset), w.env_count, w.model.links_per_env, link, value);
    return hipGetLastError() == hipSuccess;
}

nuka_result_t SetParam(World& w, nuka_world_handle handle, uint32_t p, uint32_t element, double value) {   // params.cpp:149-190
    const ParamDef& def = kParams[p];
    if (element >= ParamElements(w, p) || !std::isfinite(value) || value < def.min_value || value > def.max_value ||
        (def.type == NUKA_PARAM_U32 && value != std::floor(value))) return Error(NUKA_RESULT_INVALID_ARG, std::string("value or element out of range for ") + def.key);
    if (ParamTier(w, p) != NUKA_PARAM_LIVE) return Error(NUKA_RESULT_NOT_SUPPORTED, std::string(def.key) + " changes through a rebuild in this world");
    const float f = float(value);
    if (p == kVelocityIterations) return nuka_world_set_velocity_iterations(handle, uint32_t(value));
    if (p == kGravityZ) {   // nk::World::SetGravity (src/nk/pipeline/world.cpp:804-828): the parameter blocks are rebuilt, a captured graph dropped
        if (f == w.cfg.gravity[2]) return NUKA_RESULT_OK;
        if (w.be->synchronize(w.backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "device error");
        w.cfg.gravity[2] = f;
        InvalidatePlan(w);
        BuildPipeline(w);
        return w.mode == NUKA_EXECUTION_GRAPH ? PreparePlan(w) : NUKA_RESULT_OK;
    }
    const bool scalar_joint = w.host.joint_type[element] <= kPrismatic;
    if ((p == kJointDamping || p == kJointArmature || p == kJointFrictionloss) && !scalar_joint)
        return Error(NUKA_RESULT_NOT_SUPPORTED, "the link's joint has no scalar coordinate");
    if ((p == kDriveStiffness || p == kDriveForceLimit) && (!scalar_joint || w.model.joint_drive_rows == 0u))
        return Error(NUKA_RESULT_NOT_SUPPORTED, "the link has no drive in this world");
    if (w.be->synchronize(w.backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, "device error");
    bool ok = false;
    switch (p) {
        case kLinkMass: {   // the centre of mass and the rotational inertia about it stay (params.cpp:112-121)
            if (w.model.free_body != 0u) return Error(NUKA_RESULT_NOT_SUPPORTED, "a free body's mass changes through a rebuild in this world");
            float inertia[36];
            MakeSpatialInertia(f, w.host.link_diag_inertia.data() + 3u * element, w.host.link_inertial_frame.data() + 7u * element, inertia);
            ok = PutTemplate(w, "link_inertia", size_t{36u} * element, inertia, 36u);
            if (ok) { std::memcpy(w.host.link_inertia.data() + 36u * element, inertia, sizeof(inertia)); w.host.link_mass[element] = f; }
            break;
        }
        case kJointDamping: ok = PutTemplate(w, "joint_damping", element, &f, 1u); if (ok) w.host.joint_damping[element] = f; break;
        case kJointArmature: ok = PutTemplate(w, "joint_armature", element, &f, 1u); if (ok) w.host.joint_armature[element] = f; break;
        case kJointFrictionloss: ok = PutTemplate(w, "joint_frictionloss", element, &f, 1u); if (ok) w.host.joint_frictionloss[element] = f; break;
        case kDriveStiffness:   // the cook derives a position drive's damping from its gain the same way (params.cpp:135-141)
            ok = PutColumn(w, "drive_stiffness", element, f) && PutColumn(w, "drive_damping", element, 2.0f * std::sqrt(f));
            if (ok) w.drive_stiffness[element] = f;
            break;
        case kDriveForceLimit: ok = PutColumn(w, "drive_force_limit", element, f); if (ok) w.drive_force_limit[element] = f; break;
        default: break;
    }
    if (!ok || w.be->synchronize(w.backend, nullptr) != uint8_t(Status::Ok)) return Error(NUKA_RESULT_DEVICE_ERROR, std::string("write of ") + def.key + " failed");
    return NUKA_RESULT_OK;
}
}  // namespace
}  // namespace nkh
}  // extern "C++"

nuka_result_t nuka_world_param_count(nuka_world_handle world, uint32_t* out_count) {
    if (out_count == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    if (world == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    *out_count = kParamCount;
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_param_infos(nuka_world_handle world, nuka_param_info_t* infos, uint32_t capacity) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (infos == nullptr || capacity < kParamCount) return Error(NUKA_RESULT_INVALID_ARG, "infos must hold every parameter");
    for (uint32_t i = 0u; i < kParamCount; ++i)
        if (infos[i].struct_size != sizeof(nuka_param_info_t) || infos[i].schema_version != NUKA_PARAM_INFO_VERSION)
            return Error(NUKA_RESULT_INVALID_ARG, "struct_size or schema_version mismatch");
    for (uint32_t i = 0u; i < kParamCount; ++i) {
        const ParamDef& def = kParams[i];
        nuka_param_info_t& info = infos[i];
        info = {};
        info.struct_size = sizeof(info);
        info.schema_version = NUKA_PARAM_INFO_VERSION;
        std::snprintf(info.key, sizeof(info.key), "%s", def.key);
        std::snprintf(info.unit, sizeof(info.unit), "%s", def.unit);
        std::snprintf(info.scene_field, sizeof(info.scene_field), "%s", def.scene_field);
        info.type = def.type;
        info.tier = ParamTier(*w, i);
        info.count = ParamElements(*w, i);
        info.min_value = def.min_value;
        info.max_value = def.max_value;
    }
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_get_param(nuka_world_handle world, uint32_t param, uint32_t element, double* out_value) {
    if (out_value == nullptr) return Error(NUKA_RESULT_INVALID_ARG, "out is null");
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (param >= kParamCount || element >= ParamElements(*w, param)) return Error(NUKA_RESULT_INVALID_ARG, "unknown parameter or element");
    switch (param) {   // params.cpp:74-90
        case kGravityZ: *out_value = w->cfg.gravity[2]; break;
        case kVelocityIterations: *out_value = w->p_solve.iterations; break;
        case kLinkMass: *out_value = w->host.link_inertia[size_t{36u} * element + 3u * 6u + 3u]; break;   // (3,3) of the row-major 6x6
        case kJointDamping: *out_value = w->host.joint_damping[element]; break;
        case kJointArmature: *out_value = w->host.joint_armature[element]; break;
        case kJointFrictionloss: *out_value = w->host.joint_frictionloss[element]; break;
        case kDriveStiffness: *out_value = w->drive_stiffness[element]; break;
        default: *out_value = w->drive_force_limit[element]; break;
    }
    return NUKA_RESULT_OK;
}

nuka_result_t nuka_world_set_param(nuka_world_handle world, uint32_t param, uint32_t element, double value) {
    auto* w = reinterpret_cast<World*>(world);
    if (w == nullptr) return Error(NUKA_RESULT_NULL_HANDLE, "world is null");
    if (param >= kParamCount) return Error(NUKA_RESULT_INVALID_ARG, "unknown parameter");
    ++w->param_version;
    try {
        return SetParam(*w, world, param, element, value);
    } catch (const std::bad_alloc&) {
        return Error(NUKA_RESULT_OUT_OF_MEMORY, "host allocation failed");
    } catch (const std::exception& e) {
        return Error(NUKA_RESULT_INTERNAL, e.what());
    }
}

nuka_result_t nuka_world_set_link_mass(nuka_world_handle world, uint32_t link_index, float mass) {
    return nuka_world_set_param(world, kLinkMass, link_index, mass);
}

nuka_result_t nuka_world_set_gravity_z(nuka_world_handle world, float gravity_z) {
    return nuka_world_set_param(world, kGravityZ, 0u, gravity_z);
}

}  // extern "C"
