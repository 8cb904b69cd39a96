/*
 * CPU oracle (test infrastructure; see nuka_oracle.h): template cook, env-major storage, the named
 * field table and the per-op drivers that loop environments (OpenMP when built with -fopenmp).
 */
#include <stdio.h>

#include "nko_internal.h"
#include <stddef.h>

#define ALLOC(type, count) ((type*)calloc((size_t)(count) + 1u, sizeof(type)))

static void copy_or_zero(float* dst, const float* src, size_t n) {
    if (src != NULL) memcpy(dst, src, n * sizeof(float));
    else memset(dst, 0, n * sizeof(float));
}

/* Tree tables (fields.yaml:845-848; articulation_types.cuh:40-50): BFS depth, children CSR in link order;
 * DOF maps as BuildDofMaps (articulation_mass.cuh:64-90). */
static int cook_template(nko_template* t, const nko_template_desc* d) {
    const uint32_t nl = d->link_count, nb = d->body_count;
    memset(t, 0, sizeof(*t));
    t->nl = nl; t->nb = nb; t->n_profiles = d->profile_count;
    t->joint_type = ALLOC(uint8_t, nl); t->parent_link = ALLOC(uint32_t, nl);
    t->joint_axis = ALLOC(float, nl * 3u); t->parent_offset = ALLOC(float, nl * 3u);
    t->link_local_pose = ALLOC(float, nl * 7u); t->link_inertial_frame = ALLOC(float, nl * 7u);
    t->link_inertia = ALLOC(float, nl * 36u);
    t->joint_damping = ALLOC(float, nl); t->joint_armature = ALLOC(float, nl);
    t->joint_stiffness = ALLOC(float, nl); t->joint_spring_reference = ALLOC(float, nl);
    t->joint_limit_lower = ALLOC(float, nl); t->joint_limit_upper = ALLOC(float, nl);
    t->joint_frictionloss = ALLOC(float, nl); t->joint_limit_flags = ALLOC(uint8_t, nl);
    t->link_body = ALLOC(uint32_t, nl); t->link_tree_depth = ALLOC(uint32_t, nl);
    t->link_child_range = ALLOC(uint32_t, nl * 2u); t->link_children = ALLOC(uint32_t, nl);
    t->link_dof = ALLOC(uint32_t, nl);
    t->link_geom_local = ALLOC(float, nl * 7u); t->link_geom_kind = ALLOC(uint32_t, nl);
    memcpy(t->joint_type, d->joint_type, nl);
    memcpy(t->parent_link, d->parent_link, nl * sizeof(uint32_t));
    memcpy(t->joint_axis, d->joint_axis, nl * 3u * sizeof(float));
    copy_or_zero(t->parent_offset, d->parent_offset, nl * 3u);
    memcpy(t->link_local_pose, d->link_local_pose, nl * 7u * sizeof(float));
    memcpy(t->link_inertial_frame, d->link_inertial_frame, nl * 7u * sizeof(float));
    copy_or_zero(t->joint_damping, d->joint_damping, nl);
    copy_or_zero(t->joint_armature, d->joint_armature, nl);
    copy_or_zero(t->joint_stiffness, d->joint_stiffness, nl);
    copy_or_zero(t->joint_spring_reference, d->joint_spring_reference, nl);
    const int has_joint_rows = d->struct_size >= offsetof(nko_template_desc, excluded_pairs);
    const int has_excluded = d->struct_size >= offsetof(nko_template_desc, profile_law);
    copy_or_zero(t->joint_limit_lower, has_joint_rows ? d->joint_limit_lower : NULL, nl);
    copy_or_zero(t->joint_limit_upper, has_joint_rows ? d->joint_limit_upper : NULL, nl);
    copy_or_zero(t->joint_frictionloss, has_joint_rows ? d->joint_frictionloss : NULL, nl);
    if (has_joint_rows && d->joint_limit_flags != NULL) memcpy(t->joint_limit_flags, d->joint_limit_flags, nl);
    t->drive_mode = has_joint_rows ? d->drive_mode : NKO_DRIVE_TORQUE;
    uint32_t nv = 0u;
    for (uint32_t l = 0u; l < nl; ++l) {
        nko_make_spatial_inertia(d->link_mass[l], d->link_diag_inertia + 3u * l, d->link_inertial_frame + 7u * l, t->link_inertia + 36u * l);
        t->link_dof[l] = nv;
        nv += nko_joint_dof(t->joint_type[l]);
        t->link_body[l] = NKO_INVALID;
        const float id[7] = {0, 0, 0, 1, 0, 0, 0};
        memcpy(t->link_geom_local + 7u * l, id, sizeof(id));
    }
    if (nv > NKO_MAX_DOF) return -1;
    t->nv = nv; t->max_dof = nv;
    t->floating = nl > 0u && t->joint_type[0] == NKO_FLOATING && t->parent_link[0] == NKO_INVALID;
    t->free_body = d->struct_size >= sizeof(nko_template_desc) && d->free_body != 0u;
    if (t->free_body) {
        if (nl != 1u || !t->floating) return -1;   /* one free body an environment, the template's one link */
        t->body_mass = d->link_mass[0];
        for (uint32_t k = 0u; k < 3u; ++k) t->body_diag_inertia[k] = d->link_diag_inertia[k];
    }
    t->dof_link = ALLOC(uint32_t, nv); t->dof_component = ALLOC(uint32_t, nv);
    for (uint32_t l = 0u; l < nl; ++l) {
        const uint32_t width = nko_joint_dof(t->joint_type[l]);
        for (uint32_t c = 0u; c < width; ++c) {
            t->dof_link[t->link_dof[l] + c] = l;
            t->dof_component[t->link_dof[l] + c] = width == 1u ? NKO_INVALID : c;
        }
    }
    for (uint32_t l = 0u; l < nl; ++l) {
        uint32_t depth = 0u, walk = l;
        while (t->parent_link[walk] != NKO_INVALID) { walk = t->parent_link[walk]; ++depth; if (depth > nl) return -1; }
        t->link_tree_depth[l] = depth;
        if (depth > t->max_depth) t->max_depth = depth;
    }
    uint32_t cursor = 0u;
    for (uint32_t l = 0u; l < nl; ++l) {
        t->link_child_range[2u * l] = cursor;
        for (uint32_t c = 0u; c < nl; ++c) if (t->parent_link[c] == l) t->link_children[cursor++] = c;
        t->link_child_range[2u * l + 1u] = cursor;
    }
    /* collidable rows (scene/cook/cook_to_model.cpp:612-640; prims_types.cuh:27-54) */
    t->shape_table = ALLOC(float, nb * 13u);
    t->body_to_link = ALLOC(uint32_t, nb); t->body_to_articulation = ALLOC(uint32_t, nb);
    t->body_collidable_link = ALLOC(uint32_t, nb); t->body_collidable_body = ALLOC(uint32_t, nb);
    t->body_collidable_local = ALLOC(float, nb * 7u); t->body_init_pose = ALLOC(float, nb * 7u);
    t->profile_mu = ALLOC(float, t->n_profiles * 2u);
    if (t->n_profiles) memcpy(t->profile_mu, d->profile_mu, t->n_profiles * 2u * sizeof(float));
    {   /* MuJoCo-law profile terms, defaults of ContactParamsIn (contact_filter.hpp:20-37) where not authored */
        const int has = d->struct_size >= offsetof(nko_template_desc, profile_priority);
        const int has_mix = d->struct_size >= offsetof(nko_template_desc, joint_law);
        t->profile_mix = ALLOC(float, t->n_profiles * 3u);
        t->profile_law = ALLOC(uint32_t, t->n_profiles); t->profile_solref = ALLOC(float, t->n_profiles * 2u);
        t->profile_solimp = ALLOC(float, t->n_profiles * 5u); t->profile_margin = ALLOC(float, t->n_profiles * 2u);
        const float solimp[5] = {0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
        for (uint32_t i = 0u; i < t->n_profiles; ++i) {
            t->profile_law[i] = has && d->profile_law ? d->profile_law[i] : 0u;
            t->profile_solref[2u * i] = has && d->profile_solref ? d->profile_solref[2u * i] : 0.02f;
            t->profile_solref[2u * i + 1u] = has && d->profile_solref ? d->profile_solref[2u * i + 1u] : 1.0f;
            for (uint32_t k = 0u; k < 5u; ++k) t->profile_solimp[5u * i + k] = has && d->profile_solimp ? d->profile_solimp[5u * i + k] : solimp[k];
            for (uint32_t k = 0u; k < 2u; ++k) t->profile_margin[2u * i + k] = has && d->profile_margin ? d->profile_margin[2u * i + k] : 0.0f;
            t->profile_mix[3u * i] = has_mix && d->profile_priority ? (float)d->profile_priority[i] : 0.0f;
            t->profile_mix[3u * i + 1u] = has_mix && d->profile_solmix ? d->profile_solmix[i] : 1.0f;
            t->profile_mix[3u * i + 2u] = has_mix && d->profile_condim ? (float)d->profile_condim[i] : 3.0f;
            t->any_mujoco = t->any_mujoco || t->profile_law[i] == 1u;
        }
        t->cone = has ? d->contact_cone : 0u;
        t->impratio = has && d->contact_impratio > 0.0f ? d->contact_impratio : 1.0f;
    }
    {   /* MuJoCo-sourced joints: limit margin and the solref / solimp of the limit and friction rows */
        const int has_joints = d->struct_size >= sizeof(nko_template_desc);
        const float reference[7] = {0.02f, 1.0f, 0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
        t->joint_law = ALLOC(uint8_t, nl); t->joint_limit_margin = ALLOC(float, nl);
        t->joint_limit_reference = ALLOC(float, nl * 7u); t->joint_friction_reference = ALLOC(float, nl * 7u);
        for (uint32_t l = 0u; l < nl; ++l) {
            t->joint_law[l] = has_joints && d->joint_law ? d->joint_law[l] : 0u;
            t->joint_limit_margin[l] = has_joints && d->joint_limit_margin ? d->joint_limit_margin[l] : 0.0f;
            for (uint32_t k = 0u; k < 7u; ++k) {
                t->joint_limit_reference[7u * l + k] = has_joints && d->joint_limit_reference ? d->joint_limit_reference[7u * l + k] : reference[k];
                t->joint_friction_reference[7u * l + k] = has_joints && d->joint_friction_reference ? d->joint_friction_reference[7u * l + k] : reference[k];
            }
            t->any_mujoco = t->any_mujoco || t->joint_law[l] == 1u;
        }
        t->integrator = has_joints ? d->integrator : 0u;
    }
    for (uint32_t b = 0u; b < nb; ++b) {
        const uint32_t role = d->body_role[b], link = d->body_link[b];
        float* row = t->shape_table + 13u * b;
        row[0] = u2f(d->shape_kind[b]);
        for (uint32_t k = 0u; k < 4u; ++k) row[1u + k] = d->shape_params[4u * b + k];
        row[5] = u2f(d->shape_contype[b]); row[6] = u2f(d->shape_conaffinity[b]); row[7] = u2f(0u);
        row[8] = u2f(role == 0u ? 0xFFFFFFFFu : b); row[9] = u2f(d->shape_group[b]);
        row[10] = u2f(0u); row[11] = u2f(0u); row[12] = u2f(d->shape_profile[b]);
        t->body_to_link[b] = NKO_INVALID; t->body_to_articulation[b] = NKO_INVALID;
        t->body_collidable_link[b] = NKO_INVALID; t->body_collidable_body[b] = NKO_INVALID;
        const float id[7] = {0, 0, 0, 1, 0, 0, 0};
        memcpy(t->body_collidable_local + 7u * b, id, sizeof(id));
        memcpy(t->body_init_pose + 7u * b, id, sizeof(id));
        if (role == 0u) memcpy(t->body_init_pose + 7u * b, d->body_local + 7u * b, 7u * sizeof(float));
        else if (role == 1u) {
            if (link >= nl || t->link_body[link] != NKO_INVALID) return -1;
            t->link_body[link] = b; t->body_to_link[b] = link; t->body_to_articulation[b] = 0u;
            memcpy(t->link_geom_local + 7u * link, d->body_local + 7u * b, 7u * sizeof(float));
            t->link_geom_kind[link] = d->shape_kind[b] != NKO_INVALID ? 1u : 0u;
        }
    }
    for (uint32_t b = 0u; b < nb; ++b) {
        if (d->body_role[b] != 2u) continue;
        const uint32_t link = d->body_link[b];
        if (link >= nl || t->link_body[link] == NKO_INVALID) return -1;
        t->body_collidable_link[b] = link;
        t->body_collidable_body[b] = t->link_body[link];
        memcpy(t->body_collidable_local + 7u * b, d->body_local + 7u * b, 7u * sizeof(float));
    }
    /* excluded pairs (scene/cook/cook_to_model.cpp:1468-1490): the authored ones and every two rows of one link,
     * as sorted (a << 32 | b) keys with a < b */
    {
        const uint32_t authored = has_excluded && d->excluded_pairs != NULL ? d->excluded_pair_count : 0u;
        size_t cap = authored;
        for (uint32_t i = 0u; i < nb; ++i)
            for (uint32_t j = i + 1u; j < nb; ++j)
                if (d->body_role[i] != 0u && d->body_role[j] != 0u && d->body_link[i] == d->body_link[j]) ++cap;
        t->excluded_pairs = ALLOC(uint64_t, cap ? cap : 1u);
        uint32_t n = 0u;
        for (uint32_t k = 0u; k < authored; ++k) {
            const uint32_t a = d->excluded_pairs[2u * k], b = d->excluded_pairs[2u * k + 1u];
            if (a >= nb || b >= nb || a == b) return -1;
            t->excluded_pairs[n++] = ((uint64_t)(a < b ? a : b) << 32u) | (uint64_t)(a < b ? b : a);
        }
        for (uint32_t i = 0u; i < nb; ++i)
            for (uint32_t j = i + 1u; j < nb; ++j)
                if (d->body_role[i] != 0u && d->body_role[j] != 0u && d->body_link[i] == d->body_link[j])
                    t->excluded_pairs[n++] = ((uint64_t)i << 32u) | (uint64_t)j;
        for (uint32_t i = 1u; i < n; ++i) {   /* insertion sort, then drop repeats */
            const uint64_t key = t->excluded_pairs[i]; uint32_t j = i;
            while (j > 0u && t->excluded_pairs[j - 1u] > key) { t->excluded_pairs[j] = t->excluded_pairs[j - 1u]; --j; }
            t->excluded_pairs[j] = key;
        }
        uint32_t unique = 0u;
        for (uint32_t i = 0u; i < n; ++i) if (unique == 0u || t->excluded_pairs[unique - 1u] != t->excluded_pairs[i]) t->excluded_pairs[unique++] = t->excluded_pairs[i];
        t->excluded_count = unique;
    }
    for (uint32_t i = 0u; i < nb; ++i) {
        const uint32_t kind = d->shape_kind[i];
        if (kind != NKO_INVALID && kind != NKO_SPHERE && kind != NKO_CAPSULE && kind != NKO_BOX && kind != NKO_PLANE && kind != NKO_CYLINDER) return -1;
    }
    uint32_t slots = d->max_contacts_per_env;
    if (slots == 0u) {   /* admitted pairs of the template */
        for (uint32_t i = 0u; i < nb; ++i)
            for (uint32_t j = i + 1u; j < nb; ++j) {
                const int si = d->body_role[i] == 0u, sj = d->body_role[j] == 0u;
                if (si && sj) continue;
                if (d->shape_kind[i] == NKO_INVALID || d->shape_kind[j] == NKO_INVALID) continue;
                if (!nko_shape_filter_admits(d->shape_contype[i], d->shape_conaffinity[i], d->shape_group[i],
                                             d->shape_contype[j], d->shape_conaffinity[j], d->shape_group[j])) continue;
                if (nko_template_pair_excluded(t, i, j)) continue;
                ++slots;
            }
    }
    t->slots = slots;
    t->contact_rows_per_env = slots * 16u;   /* nk_row.hpp:59-63: 4 points x 4 rows per rigid slot */
    /* joint row slots (cook_to_model.cpp:696-719, nk/pipeline/world.cpp:61, 96) */
    int any_limit = 0, any_friction = 0;
    for (uint32_t l = 0u; l < nl; ++l) {
        const uint8_t flags = t->joint_limit_flags[l];
        if (((flags & 1u) && !isfinite(t->joint_limit_lower[l])) || ((flags & 2u) && !isfinite(t->joint_limit_upper[l])) ||
            ((flags & 3u) == 3u && t->joint_limit_lower[l] > t->joint_limit_upper[l])) return -1;
        if (!isfinite(t->joint_frictionloss[l]) || t->joint_frictionloss[l] < 0.0f) return -1;
        any_limit = any_limit || flags != 0u;
        any_friction = any_friction || t->joint_frictionloss[l] > 0.0f;
    }
    t->joint_limit_rows = any_limit ? nl * 2u : 0u;
    t->joint_friction_rows = any_friction ? nl : 0u;
    t->joint_drive_rows = has_joint_rows && d->drive_rows != 0u ? nl : 0u;
    t->rows_per_env = t->contact_rows_per_env + t->joint_limit_rows + t->joint_friction_rows + t->joint_drive_rows;
    if (t->free_body && t->link_body[0] == NKO_INVALID) return -1;   /* the body's state lives in its own body row */
    return 0;
}

static void free_template(nko_template* t) {
    free(t->joint_type); free(t->parent_link); free(t->joint_axis); free(t->parent_offset); free(t->link_local_pose);
    free(t->link_inertial_frame); free(t->link_inertia); free(t->joint_damping); free(t->joint_armature);
    free(t->joint_stiffness); free(t->joint_spring_reference); free(t->joint_limit_lower); free(t->joint_limit_upper);
    free(t->joint_frictionloss); free(t->joint_limit_flags); free(t->link_body); free(t->link_tree_depth);
    free(t->link_child_range); free(t->link_children); free(t->link_dof); free(t->dof_link); free(t->dof_component);
    free(t->link_geom_local); free(t->link_geom_kind); free(t->shape_table); free(t->excluded_pairs); free(t->body_to_link);
    free(t->body_to_articulation); free(t->body_collidable_link); free(t->body_collidable_body);
    free(t->body_collidable_local); free(t->body_init_pose); free(t->profile_mu);
    free(t->joint_law); free(t->joint_limit_margin); free(t->joint_limit_reference); free(t->joint_friction_reference);
    free(t->profile_mix); free(t->profile_law); free(t->profile_solref); free(t->profile_solimp); free(t->profile_margin);
}

nko_world* nko_world_create(const nko_template_desc* tmpl, const nko_world_desc* desc) {
    if (tmpl == NULL || desc == NULL || desc->env_count == 0u) return NULL;
    nko_world* w = (nko_world*)calloc(1, sizeof(nko_world));
    if (cook_template(&w->t, tmpl) != 0) { free_template(&w->t); free(w); return NULL; }
    w->cfg = *desc;
    /* C-ABI defaults (nuka.h:160-173; pipeline.hpp SolverConfig; op_schema.hpp:598, 663) */
    if (w->cfg.fixed_dt <= 0.0f) w->cfg.fixed_dt = 1.0f / 240.0f;
    if (w->cfg.solver_vel_iters == 0u) w->cfg.solver_vel_iters = 10u;
    if (w->cfg.solver_pos_iters == 0u) w->cfg.solver_pos_iters = 4u;
    if (w->cfg.solver_pos_iters == 0xFFFFFFFFu) w->cfg.solver_pos_iters = 0u;
    if (w->cfg.solver_pos_beta <= 0.0f) w->cfg.solver_pos_beta = 0.3f;
    if (w->cfg.solver_pos_slop <= 0.0f) w->cfg.solver_pos_slop = 1.0e-3f;
    if (w->cfg.solver_velocity_tolerance <= 0.0f) w->cfg.solver_velocity_tolerance = 1.0e-5f;
    if (w->cfg.solver_baumgarte_max_velocity <= 0.0f) w->cfg.solver_baumgarte_max_velocity = 3.0e38f;
    /* pipeline.hpp:48-49: velocity feedback of a drive is solved implicitly unless switched off */
    w->fold_drive_damping = 1;
    if (desc->struct_size >= offsetof(nko_world_desc, solver_substeps) && desc->solver_fold_drive_damping == 0xFFFFFFFFu) w->fold_drive_damping = 0;
    if (w->t.integrator != 0u) w->fold_drive_damping = 0;   /* pipeline.cpp:380-381: a MuJoCo integrator keeps the damping explicit in the solve */
    /* pipeline.cpp:63-69: every op of the interval runs at dt / substeps */
    w->substeps = desc->struct_size >= sizeof(nko_world_desc) && desc->solver_substeps > 1u ? desc->solver_substeps : 1u;
    w->outer_dt = w->cfg.fixed_dt;
    w->cfg.fixed_dt = w->cfg.fixed_dt / (float)w->substeps;
    w->env_count = desc->env_count;
    w->threads = 1;
    const nko_template* t = &w->t;
    const size_t E = w->env_count, nl = t->nl, nb = t->nb, md = t->max_dof, S = t->slots, R = t->rows_per_env;
    w->q = ALLOC(float, E * nl); w->qdot = ALLOC(float, E * nl); w->qddot = ALLOC(float, E * nl); w->tau = ALLOC(float, E * nl);
    w->base_pose = ALLOC(float, E * 7u); w->link_pose = ALLOC(float, E * nl * 7u);
    w->link_velocity = ALLOC(float, E * nl * 6u); w->link_acceleration = ALLOC(float, E * nl * 6u); w->link_wrench = ALLOC(float, E * nl * 6u);
    w->articulation_bias = ALLOC(float, E * md); w->articulation_qdd = ALLOC(float, E * md);
    w->m = ALLOC(float, E * md * md); w->m_factor = ALLOC(float, E * md * md); w->qdot_flat = ALLOC(float, E * md);
    w->qdot_pseudo = ALLOC(float, E * nl); w->link_velocity_pseudo = ALLOC(float, E * nl * 6u);
    w->body_pose = ALLOC(float, E * nb * 7u); w->body_aabb_lo = ALLOC(float, E * nb * 3u); w->body_aabb_hi = ALLOC(float, E * nb * 3u);
    w->body_linear_velocity = ALLOC(float, E * nb * 3u); w->body_angular_velocity = ALLOC(float, E * nb * 3u);
    w->body_world_inv_inertia = ALLOC(float, E * nb * 6u); w->body_gyro_residual = ALLOC(float, E * nb);
    w->body_gyro_iterations = ALLOC(uint32_t, E * nb); w->body_gyro_status = ALLOC(uint32_t, E * nb);
    w->candidate_pairs = ALLOC(uint32_t, E * S * 2u); w->pair_count = ALLOC(uint32_t, E);
    w->ucontact_count = ALLOC(uint32_t, E * S); w->ucontact_a = ALLOC(uint32_t, E * S * 4u); w->ucontact_b = ALLOC(uint32_t, E * S * 4u);
    w->ucontact_law = ALLOC(uint32_t, E * S); w->ucontact_row_range = ALLOC(uint32_t, E * S * 2u);
    w->ucontact_point = ALLOC(float, E * S * 12u); w->ucontact_normal = ALLOC(float, E * S * 12u); w->ucontact_depth = ALLOC(float, E * S * 4u);
    w->ucontact_id_pair = ALLOC(uint64_t, E * S * 4u); w->ucontact_id_feature = ALLOC(uint64_t, E * S * 4u);
    w->urows = ALLOC(float, E * R * 26u); w->lambda = ALLOC(float, E * R); w->row_penetration = ALLOC(float, E * R);
    w->row_cj_point = ALLOC(float, E * R * 3u); w->row_cj_point_b = ALLOC(float, E * R * 3u);
    w->chain_jacobian = ALLOC(float, E * R * md); w->chain_jacobian_b = ALLOC(float, E * R * md);
    w->row_cj_link = ALLOC(uint32_t, E * R); w->row_cj_link_b = ALLOC(uint32_t, E * R);
    w->row_count = ALLOC(uint32_t, E); w->contact_count = ALLOC(uint32_t, E); w->contact_row_extent = ALLOC(uint32_t, E * 2u);
    w->step_env_status = ALLOC(uint32_t, E); w->step_link_impulse = ALLOC(float, E * nl * 3u);
    w->step_link_moment = ALLOC(float, E * nl * 3u); w->step_joint_limit_impulse = ALLOC(float, E * nl * 2u);
    w->env_status = ALLOC(uint32_t, E); w->vbd_velocity_sweep_count = ALLOC(uint32_t, E);
    w->solver_residual = ALLOC(float, E * 4u);
    w->solver_velocity = ALLOC(float, E * md); w->solver_free = ALLOC(float, E * md); w->solver_penalty = ALLOC(float, E * R);
    w->body_invweight0 = ALLOC(float, E * nb * 2u); w->dof_invweight0 = ALLOC(float, E * md);
    w->row_invweight = ALLOC(float, E * R); w->row_reference_velocity_gain = ALLOC(float, E * R);
    w->step_qdot_flat = ALLOC(float, E * md);
    w->contact_material = ALLOC(uint64_t, E * S); w->contact_cache_pair = ALLOC(uint64_t, E * S * 4u);
    w->contact_cache_feature = ALLOC(uint64_t, E * S * 4u); w->contact_cache_material = ALLOC(uint64_t, E * S * 4u);
    w->contact_cache_lambda = ALLOC(float, E * S * 16u); w->contact_cache_normal = ALLOC(float, E * S * 12u);
    w->contact_cache_age = ALLOC(uint32_t, E * S * 4u); w->contact_cache_current_owner = ALLOC(uint32_t, E * S * 4u);
    w->contact_cache_old_keep = ALLOC(uint32_t, E * S * 4u); w->contact_cache_extent = ALLOC(uint32_t, E * 2u);
    w->contact_warm_start_counts = ALLOC(uint32_t, E * 2u); w->contact_cache_match = ALLOC(uint32_t, E * S * 4u);
    w->drive_target = ALLOC(float, E * nl); w->drive_stiffness = ALLOC(float, E * nl); w->drive_damping = ALLOC(float, E * nl);
    w->drive_force_limit = ALLOC(float, E * nl); w->drive_joint_force_limit = ALLOC(float, E * nl);
    w->velocity_target = ALLOC(float, E * nl); w->actuator_noload_speed = ALLOC(float, E * nl); w->joint_f = ALLOC(float, E * nl);
    w->joint_gravity_force = ALLOC(float, E * nl);
    w->drive_command = ALLOC(float, E * nl); w->drive_dissipation = ALLOC(float, E * nl); w->drive_lower = ALLOC(float, E * nl);
    w->drive_upper = ALLOC(float, E * nl); w->joint_limit_impulse = ALLOC(float, E * nl * 2u);
    w->actuator_effort_requested = ALLOC(float, E * nl); w->actuator_effort = ALLOC(float, E * nl);
    w->actuator_saturated = ALLOC(float, E * nl);
    w->contact_point = ALLOC(float, E * S * 3u); w->contact_normal = ALLOC(float, E * S * 3u); w->contact_force = ALLOC(float, E * S * 3u);
    w->ucontact_impulse = ALLOC(float, E * S * 12u); w->link_contact_wrench = ALLOC(float, E * nl * 6u);
    w->contact_side_a_kind = ALLOC(uint32_t, E * S); w->contact_side_b_kind = ALLOC(uint32_t, E * S);
    w->contact_side_a_index = ALLOC(uint32_t, E * S); w->contact_side_b_index = ALLOC(uint32_t, E * S);
    w->contact_link = ALLOC(uint32_t, E * S);
    for (size_t i = 0u; i < E * R; ++i) { w->row_cj_link[i] = NKO_INVALID; w->row_cj_link_b[i] = NKO_INVALID; }
    for (size_t e = 0u; e < E; ++e) {
        const float id[7] = {0, 0, 0, 1, 0, 0, 0};
        memcpy(w->base_pose + e * 7u, id, sizeof(id));
        for (size_t l = 0u; l < nl; ++l) memcpy(w->link_pose + (e * nl + l) * 7u, id, sizeof(id));
        for (size_t b = 0u; b < nb; ++b) memcpy(w->body_pose + (e * nb + b) * 7u, t->body_init_pose + 7u * b, sizeof(id));
    }
    /* nk/pipeline/world.cpp:553-561: creation exposes the poses of the rest state and the reference weights at them */
    if (t->any_mujoco) {
        nko_fk_world_poses(w);
        if (t->nb > 0u) nko_sync_link_body_pose(w);
        nko_reference_weights(w);
    }
    return w;
}

void nko_world_destroy(nko_world* w) {
    if (w == NULL) return;
    free_template(&w->t);
    free(w->q); free(w->qdot); free(w->qddot); free(w->tau); free(w->base_pose); free(w->link_pose); free(w->link_velocity);
    free(w->link_acceleration); free(w->link_wrench); free(w->articulation_bias); free(w->articulation_qdd); free(w->m);
    free(w->m_factor); free(w->qdot_flat); free(w->qdot_pseudo); free(w->link_velocity_pseudo); free(w->body_pose);
    free(w->body_aabb_lo); free(w->body_aabb_hi); free(w->candidate_pairs); free(w->pair_count); free(w->ucontact_count);
    free(w->ucontact_a); free(w->ucontact_b); free(w->ucontact_law); free(w->ucontact_row_range); free(w->ucontact_point);
    free(w->ucontact_normal); free(w->ucontact_depth); free(w->ucontact_id_pair); free(w->ucontact_id_feature); free(w->urows);
    free(w->lambda); free(w->row_penetration); free(w->row_cj_point); free(w->row_cj_point_b); free(w->chain_jacobian);
    free(w->chain_jacobian_b); free(w->row_cj_link); free(w->row_cj_link_b); free(w->row_count); free(w->contact_count);
    free(w->contact_row_extent); free(w->env_status); free(w->vbd_velocity_sweep_count); free(w->solver_residual);
    free(w->solver_velocity); free(w->solver_free); free(w->solver_penalty);
    free(w->body_invweight0); free(w->dof_invweight0); free(w->row_invweight); free(w->row_reference_velocity_gain); free(w->step_qdot_flat);
    free(w->step_env_status); free(w->step_link_impulse); free(w->step_link_moment); free(w->step_joint_limit_impulse);
    free(w->contact_material); free(w->contact_cache_pair); free(w->contact_cache_feature); free(w->contact_cache_material);
    free(w->contact_cache_lambda); free(w->contact_cache_normal); free(w->contact_cache_age); free(w->contact_cache_current_owner);
    free(w->contact_cache_old_keep); free(w->contact_cache_extent); free(w->contact_warm_start_counts); free(w->contact_cache_match);
    free(w->drive_target); free(w->drive_stiffness); free(w->drive_damping); free(w->drive_force_limit);
    free(w->drive_joint_force_limit); free(w->velocity_target); free(w->actuator_noload_speed); free(w->joint_f);
    free(w->joint_gravity_force); free(w->drive_command); free(w->drive_dissipation); free(w->drive_lower); free(w->drive_upper);
    free(w->joint_limit_impulse); free(w->actuator_effort_requested); free(w->actuator_effort); free(w->actuator_saturated);
    free(w->contact_point); free(w->contact_normal); free(w->contact_force); free(w->ucontact_impulse); free(w->link_contact_wrench);
    free(w->contact_side_a_kind); free(w->contact_side_b_kind); free(w->contact_side_a_index); free(w->contact_side_b_index);
    free(w->contact_link);
    free(w);
}

#define FIELD_LIST(X) \
    X(q, float, E * nl) X(qdot, float, E * nl) X(qddot, float, E * nl) X(tau, float, E * nl) \
    X(base_pose, float, E * 7u) X(link_pose, float, E * nl * 7u) X(link_velocity, float, E * nl * 6u) \
    X(link_acceleration, float, E * nl * 6u) X(link_wrench, float, E * nl * 6u) \
    X(articulation_bias, float, E * md) X(articulation_qdd, float, E * md) X(m, float, E * md * md) \
    X(m_factor, float, E * md * md) X(qdot_flat, float, E * md) X(qdot_pseudo, float, E * nl) \
    X(link_velocity_pseudo, float, E * nl * 6u) X(body_pose, float, E * nb * 7u) X(body_aabb_lo, float, E * nb * 3u) \
    X(body_aabb_hi, float, E * nb * 3u) X(candidate_pairs, uint32_t, E * S * 2u) X(pair_count, uint32_t, E) \
    X(ucontact_count, uint32_t, E * S) X(ucontact_a, uint32_t, E * S * 4u) X(ucontact_b, uint32_t, E * S * 4u) \
    X(ucontact_law, uint32_t, E * S) X(ucontact_row_range, uint32_t, E * S * 2u) X(ucontact_point, float, E * S * 12u) \
    X(ucontact_normal, float, E * S * 12u) X(ucontact_depth, float, E * S * 4u) X(ucontact_id_pair, uint64_t, E * S * 4u) \
    X(ucontact_id_feature, uint64_t, E * S * 4u) X(urows, float, E * R * 26u) X(lambda, float, E * R) \
    X(row_penetration, float, E * R) X(row_cj_point, float, E * R * 3u) X(row_cj_point_b, float, E * R * 3u) \
    X(chain_jacobian, float, E * R * md) X(chain_jacobian_b, float, E * R * md) X(row_cj_link, uint32_t, E * R) \
    X(row_cj_link_b, uint32_t, E * R) X(row_count, uint32_t, E) X(contact_count, uint32_t, E) \
    X(contact_row_extent, uint32_t, E * 2u) X(env_status, uint32_t, E) X(vbd_velocity_sweep_count, uint32_t, E) \
    X(solver_residual, float, E * 4u) X(solver_penalty, float, E * R) \
    X(body_invweight0, float, E * nb * 2u) X(dof_invweight0, float, E * md) X(row_invweight, float, E * R) \
    X(row_reference_velocity_gain, float, E * R) X(step_qdot_flat, float, E * md) \
    X(contact_material, uint64_t, E * S) X(contact_cache_pair, uint64_t, E * S * 4u) X(contact_cache_feature, uint64_t, E * S * 4u) \
    X(contact_cache_material, uint64_t, E * S * 4u) X(contact_cache_lambda, float, E * S * 16u) \
    X(contact_cache_normal, float, E * S * 12u) X(contact_cache_age, uint32_t, E * S * 4u) \
    X(contact_cache_current_owner, uint32_t, E * S * 4u) X(contact_cache_old_keep, uint32_t, E * S * 4u) \
    X(contact_cache_extent, uint32_t, E * 2u) X(contact_warm_start_counts, uint32_t, E * 2u) \
    X(drive_target, float, E * nl) X(drive_stiffness, float, E * nl) X(drive_damping, float, E * nl) \
    X(drive_force_limit, float, E * nl) X(drive_joint_force_limit, float, E * nl) X(velocity_target, float, E * nl) \
    X(actuator_noload_speed, float, E * nl) X(joint_f, float, E * nl) X(joint_gravity_force, float, E * nl) \
    X(drive_command, float, E * nl) X(drive_dissipation, float, E * nl) X(drive_lower, float, E * nl) \
    X(drive_upper, float, E * nl) X(joint_limit_impulse, float, E * nl * 2u) X(actuator_effort_requested, float, E * nl) \
    X(actuator_effort, float, E * nl) X(actuator_saturated, float, E * nl) \
    X(contact_point, float, E * S * 3u) X(contact_normal, float, E * S * 3u) X(contact_force, float, E * S * 3u) \
    X(ucontact_impulse, float, E * S * 12u) X(link_contact_wrench, float, E * nl * 6u) \
    X(contact_side_a_kind, uint32_t, E * S) X(contact_side_b_kind, uint32_t, E * S) X(contact_side_a_index, uint32_t, E * S) \
    X(contact_side_b_index, uint32_t, E * S) X(contact_link, uint32_t, E * S) \
    X(body_linear_velocity, float, E * nb * 3u) X(body_angular_velocity, float, E * nb * 3u) X(body_world_inv_inertia, float, E * nb * 6u) \
    X(body_gyro_residual, float, E * nb) X(body_gyro_iterations, uint32_t, E * nb) X(body_gyro_status, uint32_t, E * nb)

#define TEMPLATE_LIST(X) \
    X(link_inertia, float, nl * 36u) X(link_tree_depth, uint32_t, nl) X(link_child_range, uint32_t, nl * 2u) \
    X(link_children, uint32_t, nl) X(link_dof, uint32_t, nl) X(dof_link, uint32_t, md) X(dof_component, uint32_t, md) \
    X(link_body, uint32_t, nl) X(shape_table, float, nb * 13u) X(body_to_link, uint32_t, nb) \
    X(body_collidable_link, uint32_t, nb) X(body_collidable_body, uint32_t, nb)

int nko_world_field(nko_world* w, const char* name, void** ptr, size_t* bytes) {
    const nko_template* t = &w->t;
    const size_t E = w->env_count, nl = t->nl, nb = t->nb, md = t->max_dof, S = t->slots, R = t->rows_per_env;
#define X(field, type, count) if (strcmp(name, #field) == 0) { *ptr = w->field; *bytes = (size_t)(count) * sizeof(type); return 0; }
    FIELD_LIST(X)
#undef X
#define X(field, type, count) if (strcmp(name, #field) == 0) { *ptr = w->t.field; *bytes = (size_t)(count) * sizeof(type); return 0; }
    TEMPLATE_LIST(X)
#undef X
    (void)E; (void)nl; (void)nb; (void)md; (void)S; (void)R;
    return -1;
}

const char* nko_world_field_names(void) {
#define X(field, type, count) #field ","
    return FIELD_LIST(X) TEMPLATE_LIST(X) "";
#undef X
}

void nko_world_set_threads(nko_world* w, int threads) { w->threads = threads > 0 ? threads : 1; }
void nko_world_set_line_rule(nko_world* w, int rule) { w->line_rule = rule != 0 ? 1 : 0; }
/* bytes of the scalar type of this build: 4, or 8 for the double-precision build */
uint32_t nko_real_bytes(void) { return (uint32_t)sizeof(float); }
uint32_t nko_world_dof(const nko_world* w) { return w->t.nv; }
uint32_t nko_world_rows_per_env(const nko_world* w) { return w->t.rows_per_env; }

#define FOR_ENVS(body) \
    { const int threads_ = w->threads; (void)threads_; \
      _Pragma("omp parallel for schedule(dynamic, 8) num_threads(threads_)") \
      for (long env_ = 0; env_ < (long)w->env_count; ++env_) { const uint32_t env = (uint32_t)env_; body; } }

void nko_fk_world_poses(nko_world* w) { FOR_ENVS(nko_env_fk(w, env)) }
void nko_apply_drives(nko_world* w) { FOR_ENVS(nko_env_apply_drives(w, env)) }
void nko_readout_drives(nko_world* w) { FOR_ENVS(nko_env_readout_drives(w, env)) }
void nko_readout_contact_wrench(nko_world* w) { w->readout_in_step = 1; FOR_ENVS(nko_env_readout_contact_wrench(w, env)) }
void nko_articulation_dynamics(nko_world* w, uint32_t integrate_velocity) { FOR_ENVS(nko_env_dynamics(w, env, integrate_velocity)) }
void nko_sync_link_body_pose(nko_world* w) { FOR_ENVS(nko_env_sync_body_pose(w, env)) }
void nko_build_aabbs(nko_world* w) { FOR_ENVS(nko_env_aabbs(w, env)) }
void nko_query_pairs(nko_world* w) { FOR_ENVS(nko_env_pairs(w, env)) }
void nko_narrowphase(nko_world* w) { FOR_ENVS(nko_env_narrowphase(w, env)) }
void nko_assemble_rows(nko_world* w) { FOR_ENVS(nko_env_assemble_rows(w, env)) }
/* assemble_rows.cu:1393-1455: phase 0 seeds the rows from the cache, phase 1 rebuilds the cache from the solution */
void nko_contact_warm_start(nko_world* w, uint32_t phase) {
    if (phase == 0u) { FOR_ENVS(nko_env_warm_start_prepare(w, env)) }
    else { FOR_ENVS(nko_env_warm_start_commit(w, env)) }
}
void nko_block_descent_solve(nko_world* w) { FOR_ENVS(nko_env_solve(w, env)) }
void nko_integrate_position(nko_world* w) { FOR_ENVS(nko_env_integrate_position(w, env)) }
void nko_body_integrate_velocity(nko_world* w) { FOR_ENVS(nko_env_body_integrate_velocity(w, env)) }
void nko_body_integrate_position(nko_world* w) { FOR_ENVS(nko_env_body_integrate_position(w, env)) }
void nko_fk_link_velocities(nko_world* w) { FOR_ENVS(nko_env_link_velocities(w, env)) }
void nko_articulation_damping(nko_world* w) { FOR_ENVS(nko_env_articulation_damping(w, env)) }
void nko_reference_weights(nko_world* w) {
    const int fold = w->fold_drive_damping;
    w->fold_drive_damping = 0;   /* ComputeArticulationMass without drive damping (articulation.cu:452-453) */
    FOR_ENVS(nko_env_reference_weights(w, env))
    w->fold_drive_damping = fold;
}

/* Op order of one step (src/nk/pipeline/pipeline.cpp:374-986) for an articulated world with ground contact. */
/* OpSnapshotStepVelocity (assemble_rows.cu:1457-1477, PackQdotFlatMultiKernel :200-214): the generalized velocity the
 * step starts from, which the compliant rows' reference acceleration is taken at (pipeline.cpp:367-375) */
void nko_snapshot_step_velocity(nko_world* w) {
    const nko_template* t = &w->t;
    for (size_t env = 0u; env < w->env_count; ++env)
        for (uint32_t d = 0u; d < t->max_dof; ++d) {
            float value = 0.0f;
            if (d < t->nv) {
                const uint32_t link = t->dof_link[d], component = t->dof_component[d];
                value = component == NKO_INVALID ? w->qdot[env * t->nl + link] : w->link_velocity[(env * t->nl + link) * 6u + component];
            }
            w->step_qdot_flat[env * t->max_dof + d] = value;
        }
}

/* pipeline.cpp:434-443, 600-606, 955-986 for a world of free bodies: the velocity update, the contact pipeline on the
 * bodies' poses, the solve on their six by six blocks, the position update */
static void step_free_body(nko_world* w) {
    for (size_t e = 0u; e < w->env_count; ++e)   /* the six coordinates as the state holds them */
        for (uint32_t i = 0u; i < 3u; ++i) {
            const size_t body = e * w->t.nb + w->t.link_body[0];
            w->link_velocity[e * 6u + i] = w->body_linear_velocity[body * 3u + i];
            w->link_velocity[e * 6u + 3u + i] = w->body_angular_velocity[body * 3u + i];
        }
    if (w->t.rows_per_env > 0u) nko_snapshot_step_velocity(w);
    nko_body_integrate_velocity(w);
    nko_fk_world_poses(w);
    if (w->t.rows_per_env > 0u) {
        if (w->t.slots > 0u) {
            nko_sync_link_body_pose(w);
            nko_build_aabbs(w);
            nko_query_pairs(w);
            nko_narrowphase(w);
        }
        nko_assemble_rows(w);
        nko_contact_warm_start(w, 0u);
        nko_block_descent_solve(w);
        nko_contact_warm_start(w, 1u);
    }
    nko_body_integrate_position(w);
    nko_fk_world_poses(w);
    if (w->t.nb > 0u) nko_sync_link_body_pose(w);
    if (w->readout_in_step && w->t.rows_per_env > 0u && w->t.slots > 0u) nko_readout_contact_wrench(w);
}

static void step_interval(nko_world* w) {
    if (w->t.free_body) { step_free_body(w); return; }
    if (w->t.rows_per_env > 0u || w->t.integrator != 0u) nko_snapshot_step_velocity(w);   /* pipeline.cpp:367 */
    nko_fk_world_poses(w);
    if (w->t.joint_drive_rows > 0u) nko_apply_drives(w);
    nko_articulation_dynamics(w, 1u);
    if (w->t.rows_per_env > 0u) {
        if (w->t.slots > 0u) {
            nko_sync_link_body_pose(w);
            nko_build_aabbs(w);
            nko_query_pairs(w);
            nko_narrowphase(w);
        }
        nko_assemble_rows(w);
        nko_contact_warm_start(w, 0u);
        nko_block_descent_solve(w);
        nko_contact_warm_start(w, 1u);
    }
    if (w->t.joint_drive_rows > 0u) nko_readout_drives(w);   /* pipeline.cpp:929-937 */
    if (w->t.integrator != 0u) nko_articulation_damping(w);  /* pipeline.cpp:939-951 */
    nko_integrate_position(w);
    nko_fk_world_poses(w);
    nko_fk_link_velocities(w);
    if (w->t.nb > 0u) nko_sync_link_body_pose(w);
    /* pipeline.cpp:990-1005: a readout a consumer has asked for closes every interval */
    if (w->readout_in_step && w->t.rows_per_env > 0u && w->t.slots > 0u) nko_readout_contact_wrench(w);
}

/* AccumulateStepKernel (ops/readout.cu:222-300) for the outputs this path has: status words or-ed over the substeps,
 * joint limit impulses summed, link contact wrenches averaged as impulses and moments about the world origin, the
 * applied link wrenches cleared after the last substep. */
static void accumulate_step(nko_world* w, int first, int last) {
    const size_t E = w->env_count, nl = w->t.nl;
    const float substep_dt = w->cfg.fixed_dt, inv_outer_dt = 1.0f / w->outer_dt;
    const int wrenches = w->readout_in_step && w->t.rows_per_env > 0u && w->t.slots > 0u;
    for (size_t e = 0u; e < E; ++e) {
        const uint32_t status = w->env_status[e];
        const uint32_t combined = first ? status : (w->step_env_status[e] | status);
        w->step_env_status[e] = combined;
        if (last) w->env_status[e] = combined;
    }
    for (size_t i = 0u; i < E * nl; ++i) {
        if (wrenches) {
            float* wrench = w->link_contact_wrench + i * 6u;
            const v3 impulse = v3_scale(v3_make(wrench[0], wrench[1], wrench[2]), substep_dt);
            const v3 origin = v3_make(w->link_pose[i * 7u], w->link_pose[i * 7u + 1u], w->link_pose[i * 7u + 2u]);
            const v3 moment = v3_add(v3_scale(v3_make(wrench[3], wrench[4], wrench[5]), substep_dt), v3_cross(origin, impulse));
            float* si = w->step_link_impulse + i * 3u, *sm = w->step_link_moment + i * 3u;
            v3 total_impulse = impulse, total_moment = moment;
            if (!first) {
                total_impulse = v3_add(v3_make(si[0], si[1], si[2]), impulse);
                total_moment = v3_add(v3_make(sm[0], sm[1], sm[2]), moment);
            }
            si[0] = total_impulse.x; si[1] = total_impulse.y; si[2] = total_impulse.z;
            sm[0] = total_moment.x; sm[1] = total_moment.y; sm[2] = total_moment.z;
            if (last) {
                const v3 force = v3_scale(total_impulse, inv_outer_dt);
                const v3 torque = v3_scale(v3_sub(total_moment, v3_cross(origin, total_impulse)), inv_outer_dt);
                wrench[0] = force.x; wrench[1] = force.y; wrench[2] = force.z; wrench[3] = torque.x; wrench[4] = torque.y; wrench[5] = torque.z;
            }
        }
        if (w->t.joint_limit_rows != 0u)
            for (size_t side = 0u; side < 2u; ++side) {
                const size_t slot = i * 2u + side;
                const float impulse = w->joint_limit_impulse[slot];
                const float total = first ? impulse : w->step_joint_limit_impulse[slot] + impulse;
                w->step_joint_limit_impulse[slot] = total;
                if (last) w->joint_limit_impulse[slot] = total;
            }
        if (last) for (size_t k = 0u; k < 6u; ++k) w->link_wrench[i * 6u + k] = 0.0f;
    }
}

void nko_world_step(nko_world* w) {
    if (w->substeps <= 1u) {
        step_interval(w);
    } else {
        for (uint32_t s = 0u; s < w->substeps; ++s) {
            step_interval(w);
            accumulate_step(w, s == 0u, s + 1u == w->substeps);
        }
    }
    ++w->step_index;
}
