/*
 * CPU oracle (test infrastructure; see nuka_oracle.h): collidable poses, AABBs, candidate pairs in
 * canonical order, sphere/box x plane manifolds, pair-driven row assembly and chain Jacobians.
 */
#include "nko_internal.h"

#define SHAPE_STRIDE 13u   /* phi/op_schema.hpp:26 kShapeTableRowStride */

typedef struct {
    uint32_t kind; float p[4]; uint32_t contype, conaffinity; int32_t body_id; uint32_t group, profile;
} shape_row;

/* prims_types.cuh:55-72 LoadPrimShape */
static shape_row load_shape(const float* table, uint32_t row) {
    const float* q = table + (size_t)row * SHAPE_STRIDE;
    shape_row s;
    s.kind = f2u(q[0]);
    s.p[0] = q[1]; s.p[1] = q[2]; s.p[2] = q[3]; s.p[3] = q[4];
    s.contype = f2u(q[5]); s.conaffinity = f2u(q[6]);
    s.body_id = (int32_t)f2u(q[8]); s.group = f2u(q[9]); s.profile = f2u(q[12]);
    return s;
}

/* ---- SyncLinkBodyPose (ops/sync_body_pose.cu:23-52, 54-83) -------------- */
void nko_env_sync_body_pose(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const size_t lbase = (size_t)env * t->nl, bbase = (size_t)env * t->nb;
    for (uint32_t l = 0u; l < t->nl; ++l) {
        const uint32_t b = t->link_body[l];
        if (b >= t->nb) continue;
        xform world = xform_load(w->link_pose + (lbase + l) * 7u);
        if (t->link_geom_kind[l] != 0u) world = nko_compose_hd(world, xform_load(t->link_geom_local + 7u * l));
        xform_store(w->body_pose + (bbase + b) * 7u, world);
    }
    for (uint32_t b = 0u; b < t->nb; ++b) {
        const uint32_t link = t->body_collidable_link[b];
        if (link != NKO_INVALID) {
            if (link >= t->nl) continue;
            xform_store(w->body_pose + (bbase + b) * 7u,
                        nko_compose_hd(xform_load(w->link_pose + (lbase + link) * 7u), xform_load(t->body_collidable_local + 7u * b)));
            continue;
        }
        const uint32_t owner = t->body_collidable_body[b];
        if (owner == NKO_INVALID || owner >= t->nb) continue;
        xform_store(w->body_pose + (bbase + b) * 7u,
                    nko_compose_hd(xform_load(w->body_pose + (bbase + owner) * 7u), xform_load(t->body_collidable_local + 7u * b)));
    }
}

/* broadphase.cu:154-170 RotAbs */
static v3 rot_abs(quat q, v3 v) {
    const v3 cx = nko_prim_rotate(q, v3_make(1, 0, 0)), cy = nko_prim_rotate(q, v3_make(0, 1, 0)), cz = nko_prim_rotate(q, v3_make(0, 0, 1));
    return v3_make(fabsf(cx.x) * v.x + fabsf(cy.x) * v.y + fabsf(cz.x) * v.z,
                   fabsf(cx.y) * v.x + fabsf(cy.y) * v.y + fabsf(cz.y) * v.z,
                   fabsf(cx.z) * v.x + fabsf(cy.z) * v.y + fabsf(cz.z) * v.z);
}

/* collision/contact_query.hpp:17-31 */
static float contact_query_reach(float thickness, float margin) { return fmaxf(0.02f, 2.0f * (2.0f * thickness + margin)); }
static float contact_motion_radius(float base, float dt, float sa, float sb, float relax) { return base + dt * (sa + sb) * (2.0f / relax); }

/* ---- BuildAabbs (broadphase.cu:173-270). Link-owned collidables keep zero body velocity and
 * zero previous motion on this path (nothing writes them for inv_mass 0 rows), so speed = 0; a free
 * body's row carries the body's velocities. ---- */
void nko_env_aabbs(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const size_t bbase = (size_t)env * t->nb;
    const float margin = fmaxf(w->cfg.solver_contact_margin, 0.0005f);   /* pipeline.cpp:613 */
    const float reach = contact_query_reach(0.0f, w->cfg.solver_contact_margin);   /* pipeline.cpp:202 */
    for (uint32_t b = 0u; b < t->nb; ++b) {
        const shape_row s = load_shape(t->shape_table, b);
        const xform xf = xform_load(w->body_pose + (bbase + b) * 7u);
        float* lo = w->body_aabb_lo + (bbase + b) * 3u;
        float* hi = w->body_aabb_hi + (bbase + b) * 3u;
        v3 he = v3_make(0, 0, 0);
        if (s.kind == NKO_SPHERE) he = v3_make(s.p[0], s.p[0], s.p[0]);
        else if (s.kind == NKO_CAPSULE) he = rot_abs(xf.r, v3_make(s.p[0], s.p[0], s.p[0] + s.p[1]));
        else if (s.kind == NKO_BOX) he = rot_abs(xf.r, v3_make(s.p[0], s.p[1], s.p[2]));
        else if (s.kind == NKO_CYLINDER) {   /* per world axis hh |a_i| + r sqrt(1 - a_i^2) for the cylinder's axis a */
            const v3 qv = v3_make(xf.r.x, xf.r.y, xf.r.z), ez = v3_make(0, 0, 1);
            const v3 tz = v3_scale(v3_cross(qv, ez), 2.0f);
            const v3 a = v3_add(v3_add(ez, v3_scale(tz, xf.r.w)), v3_cross(qv, tz));
            he = v3_make(s.p[1] * fabsf(a.x) + s.p[0] * sqrtf(fmaxf(0.0f, 1.0f - a.x * a.x)),
                         s.p[1] * fabsf(a.y) + s.p[0] * sqrtf(fmaxf(0.0f, 1.0f - a.y * a.y)),
                         s.p[1] * fabsf(a.z) + s.p[0] * sqrtf(fmaxf(0.0f, 1.0f - a.z * a.z)));
        } else if (s.kind == NKO_PLANE) {
            lo[0] = lo[1] = lo[2] = -FLT_MAX; hi[0] = hi[1] = hi[2] = FLT_MAX;
            continue;
        } else {
            lo[0] = lo[1] = lo[2] = FLT_MAX; hi[0] = hi[1] = hi[2] = -FLT_MAX;
            continue;
        }
        /* :262-264: a free body's own row moves with it - its speed, and its turning rate over the shape's radius */
        float speed = 0.0f;
        if (t->free_body && b == t->link_body[0]) {
            const float* lv = w->body_linear_velocity + (bbase + b) * 3u, *av = w->body_angular_velocity + (bbase + b) * 3u;
            const float radius = sqrtf(he.x * he.x + he.y * he.y + he.z * he.z) + sqrtf(0.0f);
            speed = fmaxf(0.0f, sqrtf(lv[0] * lv[0] + lv[1] * lv[1] + lv[2] * lv[2]) + sqrtf(av[0] * av[0] + av[1] * av[1] + av[2] * av[2]) * radius);
        }
        const float m = fmaxf(margin, fminf(contact_motion_radius(margin, w->cfg.fixed_dt, speed, 0.0f, 0.9f), reach));
        const v3 c = xf.p;
        lo[0] = c.x - he.x - m; lo[1] = c.y - he.y - m; lo[2] = c.z - he.z - m;
        hi[0] = c.x + he.x + m; hi[1] = c.y + he.y + m; hi[2] = c.z + he.z + m;
    }
}

/* collision/shape_kind.hpp:26-33 ShapeFilterAdmits */
static int shape_filter_admits(uint32_t ta, uint32_t aa, uint32_t ga_, uint32_t tb, uint32_t ab, uint32_t gb_) {
    if (((ta & ab) | (tb & aa)) == 0u) return 0;
    const int32_t ga = (int32_t)ga_, gb = (int32_t)gb_;
    return !(ga != 0 && gb != 0 && (ga > 0 ? (ga != gb && gb > 0) : ga == gb));
}

/* ---- candidate pairs (broadphase.cu:408-474 EnvAllPairsKernel, 478-542 canonical sort).
 * Emission order is a race in the reference and is erased by the stable sort on (a, b); the
 * oracle enumerates i<j ascending, which already is that order.  Overflow keeps the first
 * `capacity` emitted pairs in the reference (racy); the oracle keeps the smallest keys. ---- */
/* broadphase.cu:87-99 IsExcluded: binary search of the sorted (a << 32 | b) keys, a < b */
int nko_template_pair_excluded(const nko_template* t, uint32_t a, uint32_t b) {
    const uint64_t key = ((uint64_t)a << 32u) | (uint64_t)b;
    uint32_t lo = 0u, hi = t->excluded_count;
    while (lo < hi) {
        const uint32_t mid = lo + (hi - lo) / 2u;
        if (t->excluded_pairs[mid] < key) lo = mid + 1u; else hi = mid;
    }
    return lo < t->excluded_count && t->excluded_pairs[lo] == key;
}
int nko_pair_excluded(const nko_world* w, uint32_t a, uint32_t b) { return nko_template_pair_excluded(&w->t, a < b ? a : b, a < b ? b : a); }

void nko_env_pairs(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const size_t bbase = (size_t)env * t->nb;
    uint32_t* pairs = w->candidate_pairs + (size_t)env * t->slots * 2u;
    uint32_t count = 0u;
    w->env_status[env] &= ~(uint32_t)NKO_STATUS_PAIR_OVERFLOW;
    for (uint32_t i = 0u; i < t->nb; ++i)
        for (uint32_t j = i + 1u; j < t->nb; ++j) {
            const float* alo = w->body_aabb_lo + (bbase + i) * 3u, *ahi = w->body_aabb_hi + (bbase + i) * 3u;
            const float* blo = w->body_aabb_lo + (bbase + j) * 3u, *bhi = w->body_aabb_hi + (bbase + j) * 3u;
            if (ahi[0] < blo[0] || alo[0] > bhi[0]) continue;
            if (ahi[1] < blo[1] || alo[1] > bhi[1]) continue;
            if (ahi[2] < blo[2] || alo[2] > bhi[2]) continue;
            const shape_row sa = load_shape(t->shape_table, i), sb = load_shape(t->shape_table, j);
            if (sa.body_id < 0 && sb.body_id < 0) continue;
            if (!shape_filter_admits(sa.contype, sa.conaffinity, sa.group, sb.contype, sb.conaffinity, sb.group)) continue;
            if (nko_template_pair_excluded(t, i, j)) continue;
            if (count < t->slots) { pairs[2u * count] = i; pairs[2u * count + 1u] = j; ++count; }
            else w->env_status[env] |= NKO_STATUS_PAIR_OVERFLOW;
        }
    w->pair_count[env] = count;
}

/* ---- manifolds (collision/analytical_manifold.hpp) ----------------------- */
typedef struct { v3 cx, cy, cz, t; float radius, half_height; v3 half; } prim;

static prim make_prim(shape_row s, xform xf) {   /* narrowphase_prims.cu:34-46 MakePrim */
    prim p;
    p.cx = nko_prim_rotate(xf.r, v3_make(1, 0, 0)); p.cy = nko_prim_rotate(xf.r, v3_make(0, 1, 0));
    p.cz = nko_prim_rotate(xf.r, v3_make(0, 0, 1)); p.t = xf.p;
    p.radius = s.p[0]; p.half_height = s.p[1]; p.half = v3_make(s.p[0], s.p[1], s.p[2]);
    return p;
}
static v3 norm_or(v3 v, v3 fallback) {   /* analytical_manifold.hpp:194-198 Norm */
    const float len = sqrtf(v.x * v.x + v.y * v.y + v.z * v.z);
    if (len < 1.0e-12f) return fallback;
    return v3_make(v.x / len, v.y / len, v.z / len);
}
typedef struct { uint32_t count; v3 position[4]; v3 normal[4]; float penetration[4]; uint64_t key[4]; } manifold;

/* analytical_manifold.hpp:451-463 SpherePlane */
static void sphere_plane(const prim* sph, const prim* plane, float query, manifold* out) {
    out->count = 0u;
    const v3 n = norm_or(plane->cz, v3_make(0, 0, 1));
    const float signed_dist = v3_dot(v3_sub(sph->t, plane->t), n);
    const float pen = sph->radius - signed_dist;
    if (pen <= -query) return;
    out->position[0] = v3_sub(sph->t, v3_scale(n, sph->radius - 0.5f * pen));
    out->normal[0] = n; out->penetration[0] = pen; out->key[0] = 0u; out->count = 1u;
}

/* analytical_manifold.hpp:273-311 ReduceAndEmit: the four deepest candidates (ties to the smaller feature id),
 * emitted in ascending feature order */
static void reduce_and_emit(v3* position, float* pen, uint32_t* feature, int ncand, v3 n, manifold* out) {
    out->count = 0u;
    if (ncand <= 0) return;
    const int keep = ncand < 4 ? ncand : 4;
    for (int s = 0; s < keep; ++s) {
        int best = s;
        for (int i = s + 1; i < ncand; ++i)
            if (pen[i] > pen[best] || (pen[i] == pen[best] && feature[i] < feature[best])) best = i;
        const v3 tp = position[s]; position[s] = position[best]; position[best] = tp;
        const float tf = pen[s]; pen[s] = pen[best]; pen[best] = tf;
        const uint32_t tk = feature[s]; feature[s] = feature[best]; feature[best] = tk;
    }
    for (int i = 1; i < keep; ++i) {
        const v3 kp = position[i]; const float kf = pen[i]; const uint32_t kk = feature[i];
        int j = i - 1;
        while (j >= 0 && feature[j] > kk) { position[j + 1] = position[j]; pen[j + 1] = pen[j]; feature[j + 1] = feature[j]; --j; }
        position[j + 1] = kp; pen[j + 1] = kf; feature[j + 1] = kk;
    }
    for (int i = 0; i < keep; ++i) {
        out->position[i] = position[i]; out->normal[i] = n; out->penetration[i] = pen[i]; out->key[i] = feature[i];
    }
    out->count = (uint32_t)keep;
}

/* analytical_manifold.hpp:337-405 ReduceAndEmitSpread: up to four candidates as they are; of more, the deepest
 * and then, three times, the one farthest from those kept (ties to the lower index); ascending feature order */
static void reduce_and_emit_spread(v3* position, float* pen, uint32_t* feature, int n, v3 normal, manifold* out) {
    out->count = 0u;
    if (n <= 0) return;
    int kept[4];
    int count = n;
    if (n <= 4) {
        for (int i = 0; i < n; ++i) kept[i] = i;
    } else {
        int used[24] = {0};
        int seed = 0;
        for (int i = 1; i < n; ++i) if (pen[i] > pen[seed]) seed = i;
        kept[0] = seed; used[seed] = 1;
        count = 1;
        for (int s = 1; s < 4; ++s) {
            int best = -1; float best_mind = -1.0f;
            for (int i = 0; i < n; ++i) {
                if (used[i]) continue;
                float mind = 3.4e38f;
                for (int t = 0; t < s; ++t) {
                    const v3 d = v3_sub(position[i], position[kept[t]]);
                    const float dd = v3_dot(d, d);
                    if (dd < mind) mind = dd;
                }
                if (mind > best_mind) { best_mind = mind; best = i; }
            }
            if (best < 0) break;
            kept[s] = best; used[best] = 1; count = s + 1;
        }
        /* the reference sorts and emits four entries once more than four candidates exist; with n > 4 every
         * round finds one, so count is 4 here */
    }
    for (int i = 1; i < count; ++i) {
        const int key = kept[i]; int j = i - 1;
        while (j >= 0 && feature[kept[j]] > feature[key]) { kept[j + 1] = kept[j]; --j; }
        kept[j + 1] = key;
    }
    for (int i = 0; i < count; ++i) {
        out->position[i] = position[kept[i]]; out->normal[i] = normal; out->penetration[i] = pen[kept[i]]; out->key[i] = feature[kept[i]];
    }
    out->count = (uint32_t)count;
}

/* analytical_manifold.hpp:69-93 PrimFrame */
static v3 frame_local_to_world(const prim* f, v3 l) {
    return v3_make(f->cx.x * l.x + f->cy.x * l.y + f->cz.x * l.z + f->t.x,
                   f->cx.y * l.x + f->cy.y * l.y + f->cz.y * l.z + f->t.y,
                   f->cx.z * l.x + f->cy.z * l.y + f->cz.z * l.z + f->t.z);
}
static v3 frame_world_to_local(const prim* f, v3 w) {
    const v3 d = v3_make(w.x - f->t.x, w.y - f->t.y, w.z - f->t.z);
    return v3_make(d.x * f->cx.x + d.y * f->cx.y + d.z * f->cx.z,
                   d.x * f->cy.x + d.y * f->cy.y + d.z * f->cy.z,
                   d.x * f->cz.x + d.y * f->cz.y + d.z * f->cz.z);
}
static v3 frame_dir_to_world(const prim* f, v3 l) {
    return v3_make(f->cx.x * l.x + f->cy.x * l.y + f->cz.x * l.z,
                   f->cx.y * l.x + f->cy.y * l.y + f->cz.y * l.z,
                   f->cx.z * l.x + f->cy.z * l.y + f->cz.z * l.z);
}

/* collision/primitive_surface.hpp:28-122 QueryPrimitiveSurface: signed distance (positive outside), outward normal,
 * closest surface point and feature of a point in the primitive's own frame */
typedef struct { float distance; v3 normal, point; uint32_t feature; int valid; } surface;
static surface query_surface(uint32_t kind, v3 par, v3 pos) {
    surface r; r.distance = 0.0f; r.normal = v3_make(1, 0, 0); r.point = v3_make(0, 0, 0); r.feature = 0u; r.valid = 0;
    if (kind == NKO_SPHERE || kind == NKO_CAPSULE) {
        if (!(par.x >= 0.0f)) return r;
        v3 offset = pos;
        if (kind == NKO_CAPSULE) {
            if (!(par.y >= 0.0f)) return r;
            const float axis = fmaxf(-par.y, fminf(pos.z, par.y));
            offset.z -= axis;
            r.feature = pos.z < -par.y ? 0u : pos.z > par.y ? 2u : 1u;
        }
        const float length = sqrtf(v3_dot(offset, offset));
        if (length > 0.0f) r.normal = v3_make(offset.x / length, offset.y / length, offset.z / length);
        r.distance = length - par.x;
    } else if (kind == NKO_BOX) {
        if (!(par.x >= 0.0f && par.y >= 0.0f && par.z >= 0.0f)) return r;
        const v3 closest = v3_make(fmaxf(-par.x, fminf(pos.x, par.x)), fmaxf(-par.y, fminf(pos.y, par.y)), fmaxf(-par.z, fminf(pos.z, par.z)));
        const v3 offset = v3_sub(pos, closest);
        const float length = sqrtf(v3_dot(offset, offset));
        if (length > 0.0f) {
            r.distance = length;
            r.normal = v3_make(offset.x / length, offset.y / length, offset.z / length);
            if (offset.x != 0.0f) r.feature |= 1u << (pos.x < 0.0f ? 0u : 1u);
            if (offset.y != 0.0f) r.feature |= 1u << (pos.y < 0.0f ? 2u : 3u);
            if (offset.z != 0.0f) r.feature |= 1u << (pos.z < 0.0f ? 4u : 5u);
        } else {
            const v3 dist = v3_make(fabsf(pos.x) - par.x, fabsf(pos.y) - par.y, fabsf(pos.z) - par.z);
            if (dist.x >= dist.y && dist.x >= dist.z) {
                r.distance = dist.x; r.normal = v3_make(pos.x < 0.0f ? -1.0f : 1.0f, 0, 0); r.feature = 1u << (pos.x < 0.0f ? 0u : 1u);
            } else if (dist.y >= dist.z) {
                r.distance = dist.y; r.normal = v3_make(0, pos.y < 0.0f ? -1.0f : 1.0f, 0); r.feature = 1u << (pos.y < 0.0f ? 2u : 3u);
            } else {
                r.distance = dist.z; r.normal = v3_make(0, 0, pos.z < 0.0f ? -1.0f : 1.0f); r.feature = 1u << (pos.z < 0.0f ? 4u : 5u);
            }
        }
    } else if (kind == NKO_PLANE) {
        r.distance = pos.z; r.normal = v3_make(0, 0, 1);
    } else if (kind == NKO_CYLINDER) {
        if (!(par.x >= 0.0f && par.y >= 0.0f)) return r;
        /* features: 0 bottom cap, 1 side, 2 top cap, 3 bottom rim, 4 top rim */
        const float rho = sqrtf(pos.x * pos.x + pos.y * pos.y);
        const v3 radial = rho > 0.0f ? v3_make(pos.x / rho, pos.y / rho, 0.0f) : v3_make(1, 0, 0);
        const v3 axial = v3_make(0, 0, pos.z < 0.0f ? -1.0f : 1.0f);
        const float side = rho - par.x;
        const float cap = fabsf(pos.z) - par.y;
        if (side > 0.0f && cap > 0.0f) {
            r.distance = sqrtf(side * side + cap * cap);
            const v3 sum = v3_add(v3_scale(radial, side), v3_scale(axial, cap));
            r.normal = v3_make(sum.x / r.distance, sum.y / r.distance, sum.z / r.distance);
            r.feature = pos.z < 0.0f ? 3u : 4u;
        } else if (side > cap) {
            r.distance = side; r.normal = radial; r.feature = 1u;
        } else {
            r.distance = cap; r.normal = axial; r.feature = pos.z < 0.0f ? 0u : 2u;
        }
    } else return r;
    r.point = v3_sub(pos, v3_scale(r.normal, r.distance));
    r.valid = 1;
    return r;
}

static void emit_one(manifold* out, v3 position, v3 normal, float pen, uint64_t key) {
    out->position[0] = position; out->normal[0] = normal; out->penetration[0] = pen; out->key[0] = key; out->count = 1u;
}

/* analytical_manifold.hpp:416-429 SphereSphere: the normal points from b to a, the point lies midway between the surfaces */
static void sphere_sphere(const prim* a, const prim* b, float query, manifold* out) {
    out->count = 0u;
    const v3 delta = v3_sub(a->t, b->t);
    const float dist = sqrtf(delta.x * delta.x + delta.y * delta.y + delta.z * delta.z);
    const float pen = (a->radius + b->radius) - dist;
    if (pen <= -query) return;
    const v3 n = norm_or(delta, v3_make(0, 1, 0));
    emit_one(out, v3_add(b->t, v3_scale(n, b->radius - 0.5f * pen)), n, pen, 0u);
}

/* analytical_manifold.hpp:434-448 SphereBox (a = sphere) */
static void sphere_box(const prim* sph, const prim* box, float query, manifold* out) {
    out->count = 0u;
    const surface s = query_surface(NKO_BOX, box->half, frame_world_to_local(box, sph->t));
    if (!s.valid) return;
    const float pen = sph->radius - s.distance;
    if (pen <= -query) return;
    const v3 normal = frame_dir_to_world(box, s.normal);
    emit_one(out, v3_sub(frame_local_to_world(box, s.point), v3_scale(normal, 0.5f * pen)), normal, pen, 0u);
}

/* analytical_manifold.hpp:469-493 BoxPlane */
static void box_plane(const prim* box, const prim* plane, float query, manifold* out) {
    out->count = 0u;
    const v3 n = norm_or(plane->cz, v3_make(0, 0, 1));
    v3 position[8]; float pen[8]; uint32_t feature[8];
    int ncand = 0;
    for (uint32_t c = 0u; c < 8u; ++c) {
        const float sx = (c & 1u) ? 1.0f : -1.0f, sy = (c & 2u) ? 1.0f : -1.0f, sz = (c & 4u) ? 1.0f : -1.0f;
        const v3 corner = frame_local_to_world(box, v3_make(sx * box->half.x, sy * box->half.y, sz * box->half.z));
        const float sd = v3_dot(v3_sub(corner, plane->t), n);
        if (sd < query) {
            position[ncand] = v3_sub(corner, v3_scale(n, 0.5f * sd));
            pen[ncand] = -sd; feature[ncand] = c; ++ncand;
        }
    }
    reduce_and_emit(position, pen, feature, ncand, n, out);
}

/* analytical_manifold.hpp:738-759 CapsulePlane: both ends of the segment along the capsule's local z */
static void capsule_plane(const prim* cap, const prim* plane, float query, manifold* out) {
    out->count = 0u;
    const v3 n = norm_or(plane->cz, v3_make(0, 0, 1));
    const v3 axis = cap->cz;
    const v3 ends[2] = {v3_add(cap->t, v3_scale(axis, cap->half_height)), v3_sub(cap->t, v3_scale(axis, cap->half_height))};
    v3 position[2]; float pen[2]; uint32_t feature[2];
    int ncand = 0;
    for (uint32_t k = 0u; k < 2u; ++k) {
        const float sd = v3_dot(v3_sub(ends[k], plane->t), n) - cap->radius;
        if (sd < query) {
            position[ncand] = v3_sub(ends[k], v3_scale(n, cap->radius + 0.5f * sd));
            pen[ncand] = -sd; feature[ncand] = k; ++ncand;
        }
    }
    reduce_and_emit(position, pen, feature, ncand, n, out);
}

/* analytical_manifold.hpp:764-778 CapsuleSphere (a = capsule): the normal points from the sphere to the capsule */
static void capsule_sphere(const prim* cap, const prim* sph, float query, manifold* out) {
    out->count = 0u;
    const surface s = query_surface(NKO_CAPSULE, v3_make(cap->radius, cap->half_height, 0.0f), frame_world_to_local(cap, sph->t));
    if (!s.valid) return;
    const float pen = sph->radius - s.distance;
    if (pen <= -query) return;
    const v3 normal = v3_scale(frame_dir_to_world(cap, s.normal), -1.0f);
    emit_one(out, v3_add(frame_local_to_world(cap, s.point), v3_scale(normal, 0.5f * pen)), normal, pen, 0u);
}

/* analytical_manifold.hpp:780-815 CylinderPlane: the lower cap's octagon and deepest point when a cap faces the
 * plane, else each cap's deepest point */
static void cylinder_plane(const prim* cyl, const prim* plane, float query, manifold* out) {
    out->count = 0u;
    static const float kS = 0.70710678f;
    const float rc[8] = {1.0f, kS, 0.0f, -kS, -1.0f, -kS, 0.0f, kS};
    const float rs[8] = {0.0f, kS, 1.0f, kS, 0.0f, -kS, -1.0f, -kS};
    const v3 n = norm_or(plane->cz, v3_make(0, 0, 1));
    const v3 axis = cyl->cz;
    const float d = v3_dot(axis, n);
    const int on_cap = (d < 0.0f ? -d : d) >= 0.95f;
    const v3 down = norm_or(v3_sub(v3_scale(axis, d), n), cyl->cx);
    v3 position[10]; float pen[10]; uint32_t feature[10];
    int ncand = 0;
    for (int cap = 0; cap < 2; ++cap) {
        if (on_cap && (cap == 0) == (d > 0.0f)) continue;
        const v3 center = v3_add(cyl->t, v3_scale(axis, cap == 0 ? cyl->half_height : -cyl->half_height));
        for (int k = -1; k < (on_cap ? 8 : 0); ++k) {
            const v3 dir = k < 0 ? down : v3_add(v3_scale(cyl->cx, rc[k]), v3_scale(cyl->cy, rs[k]));
            const v3 p = v3_add(center, v3_scale(dir, cyl->radius));
            const float sd = v3_dot(v3_sub(p, plane->t), n);
            if (sd >= query) continue;
            position[ncand] = v3_sub(p, v3_scale(n, sd * 0.5f));
            pen[ncand] = -sd;
            feature[ncand] = (uint32_t)(k < 0 ? cap : 2 + cap * 8 + k);
            ++ncand;
        }
    }
    reduce_and_emit_spread(position, pen, feature, ncand, n, out);
}

/* analytical_manifold.hpp:819-834 CylinderSphere (a = cylinder) */
static void cylinder_sphere(const prim* cyl, const prim* sph, float query, manifold* out) {
    out->count = 0u;
    const surface s = query_surface(NKO_CYLINDER, v3_make(cyl->radius, cyl->half_height, 0.0f), frame_world_to_local(cyl, sph->t));
    if (!s.valid) return;
    const float pen = sph->radius - s.distance;
    if (pen <= -query) return;
    const v3 normal = v3_scale(frame_dir_to_world(cyl, s.normal), -1.0f);
    emit_one(out, v3_add(frame_local_to_world(cyl, s.point), v3_scale(normal, 0.5f * pen)), normal, pen, (uint64_t)s.feature);
}

/* analytical_manifold.hpp:841-896 ClosestPtSegmentSegment (fixed branch order) */
static float clamp01(float v) { return v < 0.0f ? 0.0f : (v > 1.0f ? 1.0f : v); }
static float closest_segment_segment(v3 p1, v3 q1, v3 p2, v3 q2, v3* c1_out, v3* c2_out) {
    const v3 d1 = v3_sub(q1, p1), d2 = v3_sub(q2, p2), r = v3_sub(p1, p2);
    const float a = v3_dot(d1, d1), e = v3_dot(d2, d2), f = v3_dot(d2, r);
    float s = 0.0f, t = 0.0f;
    const float eps = 1.0e-12f;
    if (a <= eps && e <= eps) { s = 0.0f; t = 0.0f; }
    else if (a <= eps) { s = 0.0f; t = clamp01(f / e); }
    else {
        const float c = v3_dot(d1, r);
        if (e <= eps) { t = 0.0f; s = clamp01(-c / a); }
        else {
            const float b = v3_dot(d1, d2);
            const float denom = a * e - b * b;
            if (denom > eps) s = clamp01((b * f - c * e) / denom); else s = 0.0f;
            t = (b * s + f) / e;
            if (t < 0.0f) { t = 0.0f; s = clamp01(-c / a); }
            else if (t > 1.0f) { t = 1.0f; s = clamp01((b - c) / a); }
        }
    }
    const v3 c1 = v3_add(p1, v3_scale(d1, s)), c2 = v3_add(p2, v3_scale(d2, t));
    *c1_out = c1; *c2_out = c2;
    const v3 dv = v3_sub(c1, c2);
    return v3_dot(dv, dv);
}

/* analytical_manifold.hpp:905-932 CapsuleCapsule: closest points of the two axes, inflated by the radii */
static void capsule_capsule(const prim* a, const prim* b, float query, manifold* out) {
    out->count = 0u;
    const v3 axa = a->cz, axb = b->cz;
    const v3 a0 = v3_add(a->t, v3_scale(axa, a->half_height)), a1 = v3_sub(a->t, v3_scale(axa, a->half_height));
    const v3 b0 = v3_add(b->t, v3_scale(axb, b->half_height)), b1 = v3_sub(b->t, v3_scale(axb, b->half_height));
    v3 ca, cb;
    const float dist = sqrtf(closest_segment_segment(a0, a1, b0, b1, &ca, &cb));
    const float pen = (a->radius + b->radius) - dist;
    if (pen <= -query) return;
    const v3 n = norm_or(v3_sub(ca, cb), norm_or(v3_cross(axa, axb), v3_make(0, 1, 0)));
    const v3 sa = v3_sub(ca, v3_scale(n, a->radius)), sb = v3_add(cb, v3_scale(n, b->radius));
    emit_one(out, v3_scale(v3_add(sa, sb), 0.5f), n, pen, 0u);
}

/* analytical_manifold.hpp:224-260 ClipAgainstPlane: Sutherland-Hodgman against one half-space, edges in fixed order;
 * an intersection inherits the feature of the edge's first vertex */
typedef struct { v3 v[8]; uint32_t feat[8]; int count; } clip_poly;
static void clip_add(clip_poly* p, v3 v, uint32_t f) { if (p->count < 8) { p->v[p->count] = v; p->feat[p->count] = f; ++p->count; } }
static clip_poly clip_against_plane(const clip_poly* in, v3 plane_pt, v3 plane_n) {
    clip_poly out; out.count = 0;
    for (int i = 0; i < in->count; ++i) {
        const int j = (i + 1) % in->count;
        const v3 cur = in->v[i], nxt = in->v[j];
        const float dc = v3_dot(v3_sub(cur, plane_pt), plane_n), dn = v3_dot(v3_sub(nxt, plane_pt), plane_n);
        const int cur_in = dc <= 0.0f, nxt_in = dn <= 0.0f;
        if (cur_in) clip_add(&out, cur, in->feat[i]);
        if (cur_in != nxt_in) {
            const float t = dc / (dc - dn);
            clip_add(&out, v3_make(cur.x + (nxt.x - cur.x) * t, cur.y + (nxt.y - cur.y) * t, cur.z + (nxt.z - cur.z) * t), in->feat[i]);
        }
    }
    return out;
}
static v3 v3_neg(v3 a) { return v3_make(-a.x, -a.y, -a.z); }
static float comp(v3 v, int k) { return k == 0 ? v.x : (k == 1 ? v.y : v.z); }

/* analytical_manifold.hpp:503-736 BoxBox: the axis of least penetration among the 15 separating-axis candidates in
 * fixed order (faces preferred by a 1e-5 bias); an edge pair gives one point between the closest edge points, a face
 * gives the incident face clipped against the reference face's sides, reduced by ReduceAndEmitSpread */
static void box_box(const prim* A, const prim* B, float query, manifold* out) {
    out->count = 0u;
    const v3 dpos = v3_sub(B->t, A->t);
    const v3 ax[3] = {A->cx, A->cy, A->cz}, bx[3] = {B->cx, B->cy, B->cz};
    float AbsR[3][3];
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) { const float r = v3_dot(ax[i], bx[j]); AbsR[i][j] = (r < 0.0f ? -r : r) + 1.0e-6f; }
    const float ea[3] = {A->half.x, A->half.y, A->half.z}, eb[3] = {B->half.x, B->half.y, B->half.z};
    const float dA[3] = {v3_dot(dpos, ax[0]), v3_dot(dpos, ax[1]), v3_dot(dpos, ax[2])};
    float min_pen = 3.4e38f;
    int best_axis = -1;
    v3 best_n = v3_make(0, 1, 0);
    const float bias = 1.0e-5f;
    for (int i = 0; i < 3; ++i) {
        const float ra = ea[i], rb = eb[0] * AbsR[i][0] + eb[1] * AbsR[i][1] + eb[2] * AbsR[i][2];
        const float s = dA[i] < 0.0f ? -dA[i] : dA[i];
        const float pen = (ra + rb) - s;
        if (pen <= -query) return;
        if (pen < min_pen - bias) { min_pen = pen; best_axis = i; best_n = dA[i] < 0.0f ? v3_neg(ax[i]) : ax[i]; }
    }
    for (int j = 0; j < 3; ++j) {
        const float ra = ea[0] * AbsR[0][j] + ea[1] * AbsR[1][j] + ea[2] * AbsR[2][j], rb = eb[j];
        const float dBj = v3_dot(dpos, bx[j]);
        const float s = dBj < 0.0f ? -dBj : dBj;
        const float pen = (ra + rb) - s;
        if (pen <= -query) return;
        if (pen < min_pen - bias) { min_pen = pen; best_axis = 3 + j; best_n = dBj < 0.0f ? v3_neg(bx[j]) : bx[j]; }
    }
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) {
            v3 L = v3_cross(ax[i], bx[j]);
            const float Llen = sqrtf(L.x * L.x + L.y * L.y + L.z * L.z);
            if (Llen < 1.0e-6f) continue;
            L = v3_make(L.x / Llen, L.y / Llen, L.z / Llen);
            const float ra = ea[0] * fabsf(v3_dot(ax[0], L)) + ea[1] * fabsf(v3_dot(ax[1], L)) + ea[2] * fabsf(v3_dot(ax[2], L));
            const float rb = eb[0] * fabsf(v3_dot(bx[0], L)) + eb[1] * fabsf(v3_dot(bx[1], L)) + eb[2] * fabsf(v3_dot(bx[2], L));
            const float s = v3_dot(dpos, L);
            const float pen = (ra + rb) - (s < 0.0f ? -s : s);
            if (pen <= -query) return;
            if (pen < min_pen - bias) { min_pen = pen; best_axis = 6 + i * 3 + j; best_n = s < 0.0f ? v3_neg(L) : L; }
        }
    if (best_axis < 0) return;
    if (best_axis >= 6) {   /* edge against edge: one point between the closest points of the two edges */
        const int i = (best_axis - 6) / 3, j = (best_axis - 6) % 3;
        v3 pa = A->t, pb = B->t;
        for (int k = 0; k < 3; ++k) {
            if (k == i) continue;
            const float sgn = v3_dot(ax[k], best_n) >= 0.0f ? 1.0f : -1.0f;
            pa = v3_add(pa, v3_scale(ax[k], sgn * ea[k]));
        }
        for (int k = 0; k < 3; ++k) {
            if (k == j) continue;
            const float sgn = v3_dot(bx[k], best_n) >= 0.0f ? -1.0f : 1.0f;
            pb = v3_add(pb, v3_scale(bx[k], sgn * eb[k]));
        }
        const v3 r = v3_sub(pa, pb);
        const float aa = 1.0f, bb = v3_dot(ax[i], bx[j]), cc = 1.0f;
        const float dd = v3_dot(ax[i], r), ee = v3_dot(bx[j], r);
        const float denom = aa * cc - bb * bb;
        float sN = 0.0f, tN = 0.0f;
        if (denom > 1.0e-9f) { sN = (bb * ee - cc * dd) / denom; tN = (aa * ee - bb * dd) / denom; }
        const float sCl = sN < -ea[i] ? -ea[i] : (sN > ea[i] ? ea[i] : sN);
        const float tCl = tN < -eb[j] ? -eb[j] : (tN > eb[j] ? eb[j] : tN);
        const v3 ca = v3_add(pa, v3_scale(ax[i], sCl)), cb = v3_add(pb, v3_scale(bx[j], tCl));
        emit_one(out, v3_scale(v3_add(ca, cb), 0.5f), best_n, min_pen, 0xE0000000ull | ((uint64_t)i << 4) | (uint64_t)j);
        return;
    }
    const int ref_is_A = best_axis < 3;
    const int ref_axis = ref_is_A ? best_axis : best_axis - 3;
    const prim* Rf = ref_is_A ? A : B;
    const prim* If = ref_is_A ? B : A;
    const v3 rax[3] = {Rf->cx, Rf->cy, Rf->cz}, iax[3] = {If->cx, If->cy, If->cz};
    const v3 rhe = Rf->half, ihe = If->half;
    v3 refN = rax[ref_axis];
    if (v3_dot(v3_sub(If->t, Rf->t), refN) < 0.0f) refN = v3_neg(refN);
    int inc_axis = 0; float best_dot = 3.4e38f, inc_sign = 1.0f;
    for (int k = 0; k < 3; ++k) {
        const float d = v3_dot(iax[k], refN);
        const float ad = d < 0.0f ? -d : d;
        if (-ad < best_dot) { best_dot = -ad; inc_axis = k; inc_sign = d < 0.0f ? 1.0f : -1.0f; }
    }
    const int iu = (inc_axis + 1) % 3, iv = (inc_axis + 2) % 3;
    const v3 inc_face_center = v3_add(If->t, v3_scale(iax[inc_axis], inc_sign * comp(ihe, inc_axis)));
    const v3 iu_w = iax[iu], iv_w = iax[iv];
    const float iu_e = comp(ihe, iu), iv_e = comp(ihe, iv);
    clip_poly poly; poly.count = 0;
    const float su[4] = {-1.0f, 1.0f, 1.0f, -1.0f}, sv[4] = {-1.0f, -1.0f, 1.0f, 1.0f};
    for (uint32_t k = 0u; k < 4u; ++k)
        clip_add(&poly, v3_add(v3_add(inc_face_center, v3_scale(iu_w, su[k] * iu_e)), v3_scale(iv_w, sv[k] * iv_e)), ((uint32_t)inc_axis << 4) | k);
    const int ru = (ref_axis + 1) % 3, rv = (ref_axis + 2) % 3;
    const v3 ru_w = rax[ru], rv_w = rax[rv];
    const float ru_e = comp(rhe, ru), rv_e = comp(rhe, rv);
    const v3 ref_face_center = v3_add(Rf->t, v3_scale(refN, comp(rhe, ref_axis)));
    poly = clip_against_plane(&poly, v3_add(ref_face_center, v3_scale(ru_w, ru_e)), ru_w);
    poly = clip_against_plane(&poly, v3_sub(ref_face_center, v3_scale(ru_w, ru_e)), v3_neg(ru_w));
    poly = clip_against_plane(&poly, v3_add(ref_face_center, v3_scale(rv_w, rv_e)), rv_w);
    poly = clip_against_plane(&poly, v3_sub(ref_face_center, v3_scale(rv_w, rv_e)), v3_neg(rv_w));
    v3 position[8]; float pen[8]; uint32_t feature[8];
    int ncand = 0;
    for (int k = 0; k < poly.count; ++k) {
        const float depth = v3_dot(v3_sub(ref_face_center, poly.v[k]), refN);
        if (depth >= -query) {
            const v3 onref = v3_add(poly.v[k], v3_scale(refN, depth));
            position[ncand] = v3_scale(v3_add(poly.v[k], onref), 0.5f);
            pen[ncand] = depth; feature[ncand] = (uint32_t)k; ++ncand;
        }
    }
    const v3 normalA = ref_is_A ? v3_neg(refN) : refN;
    if (ncand == 0) {
        emit_one(out, v3_add(inc_face_center, v3_scale(refN, min_pen * 0.5f)), normalA, min_pen, (uint64_t)inc_axis << 4);
        return;
    }
    reduce_and_emit_spread(position, pen, feature, ncand, normalA, out);
}

/* analytical_manifold.hpp:934-971 PrimitivePair, every analytic pair; a flipped pair negates the
 * normals.  Returns 0 for a pair that has no analytic manifold. */
static int primitive_pair(uint32_t ka, const prim* a, uint32_t kb, const prim* b, float query, manifold* out) {
    out->count = 0u;
    if (ka == NKO_SPHERE && kb == NKO_SPHERE) { sphere_sphere(a, b, query, out); return 1; }
    if (ka == NKO_SPHERE && kb == NKO_BOX) { sphere_box(a, b, query, out); return 1; }
    if (ka == NKO_SPHERE && kb == NKO_PLANE) { sphere_plane(a, b, query, out); return 1; }
    if (ka == NKO_BOX && kb == NKO_PLANE) { box_plane(a, b, query, out); return 1; }
    if (ka == NKO_BOX && kb == NKO_BOX) { box_box(a, b, query, out); return 1; }
    if (ka == NKO_CAPSULE && kb == NKO_PLANE) { capsule_plane(a, b, query, out); return 1; }
    if (ka == NKO_CAPSULE && kb == NKO_SPHERE) { capsule_sphere(a, b, query, out); return 1; }
    if (ka == NKO_CAPSULE && kb == NKO_CAPSULE) { capsule_capsule(a, b, query, out); return 1; }
    if (ka == NKO_CYLINDER && kb == NKO_PLANE) { cylinder_plane(a, b, query, out); return 1; }
    if (ka == NKO_CYLINDER && kb == NKO_SPHERE) { cylinder_sphere(a, b, query, out); return 1; }
    int flipped = 1;
    if (ka == NKO_BOX && kb == NKO_SPHERE) sphere_box(b, a, query, out);
    else if (ka == NKO_PLANE && kb == NKO_SPHERE) sphere_plane(b, a, query, out);
    else if (ka == NKO_PLANE && kb == NKO_BOX) box_plane(b, a, query, out);
    else if (ka == NKO_PLANE && kb == NKO_CAPSULE) capsule_plane(b, a, query, out);
    else if (ka == NKO_SPHERE && kb == NKO_CAPSULE) capsule_sphere(b, a, query, out);
    else if (ka == NKO_PLANE && kb == NKO_CYLINDER) cylinder_plane(b, a, query, out);
    else if (ka == NKO_SPHERE && kb == NKO_CYLINDER) cylinder_sphere(b, a, query, out);
    else flipped = 0;
    for (uint32_t i = 0u; i < out->count; ++i) out->normal[i] = v3_make(-out->normal[i].x, -out->normal[i].y, -out->normal[i].z);
    return flipped;
}
int nko_pair_has_manifold(uint32_t ka, uint32_t kb) {
    static const uint32_t kinds[5] = {NKO_SPHERE, NKO_CAPSULE, NKO_BOX, NKO_PLANE, NKO_CYLINDER};
    int known_a = 0, known_b = 0;
    for (int i = 0; i < 5; ++i) { known_a |= ka == kinds[i]; known_b |= kb == kinds[i]; }
    if (!known_a || !known_b) return 0;
    if (ka == NKO_PLANE && kb == NKO_PLANE) return 0;
    if ((ka == NKO_CYLINDER && (kb == NKO_CYLINDER || kb == NKO_BOX || kb == NKO_CAPSULE)) ||
        (kb == NKO_CYLINDER && (ka == NKO_BOX || ka == NKO_CAPSULE))) return 0;
    if ((ka == NKO_CAPSULE && kb == NKO_BOX) || (ka == NKO_BOX && kb == NKO_CAPSULE)) return 0;
    return 1;
}

uint32_t nko_sphere_plane(const float sphere_pose[7], float radius, const float plane_pose[7], float query,
                          float point[3], float normal[3], float* penetration) {
    shape_row s; memset(&s, 0, sizeof(s)); s.p[0] = radius;
    shape_row pl; memset(&pl, 0, sizeof(pl));
    const prim a = make_prim(s, xform_load(sphere_pose)), b = make_prim(pl, xform_load(plane_pose));
    manifold m; sphere_plane(&a, &b, query, &m);
    if (m.count) {
        point[0] = m.position[0].x; point[1] = m.position[0].y; point[2] = m.position[0].z;
        normal[0] = m.normal[0].x; normal[1] = m.normal[0].y; normal[2] = m.normal[0].z; *penetration = m.penetration[0];
    }
    return m.count;
}

uint32_t nko_box_plane(const float box_pose[7], const float half[3], const float plane_pose[7], float query,
                       float points[12], float normal[3], float penetration[4], uint32_t feature[4]) {
    shape_row s; memset(&s, 0, sizeof(s)); s.p[0] = half[0]; s.p[1] = half[1]; s.p[2] = half[2];
    shape_row pl; memset(&pl, 0, sizeof(pl));
    const prim a = make_prim(s, xform_load(box_pose)), b = make_prim(pl, xform_load(plane_pose));
    manifold m; box_plane(&a, &b, query, &m);
    for (uint32_t i = 0u; i < m.count; ++i) {
        points[3u * i] = m.position[i].x; points[3u * i + 1u] = m.position[i].y; points[3u * i + 2u] = m.position[i].z;
        penetration[i] = m.penetration[i]; feature[i] = (uint32_t)m.key[i];
        normal[0] = m.normal[i].x; normal[1] = m.normal[i].y; normal[2] = m.normal[i].z;
    }
    return m.count;
}

uint32_t nko_primitive_pair_frames(uint32_t kind_a, const float frame_a[12], const float params_a[4], uint32_t kind_b,
                                   const float frame_b[12], const float params_b[4], float query, float points[12],
                                   float normals[12], float penetration[4], uint64_t keys[4]) {
    prim pr[2];
    const float* f[2] = {frame_a, frame_b};
    const float* s[2] = {params_a, params_b};
    for (int k = 0; k < 2; ++k) {
        pr[k].cx = v3_make(f[k][0], f[k][1], f[k][2]); pr[k].cy = v3_make(f[k][3], f[k][4], f[k][5]);
        pr[k].cz = v3_make(f[k][6], f[k][7], f[k][8]); pr[k].t = v3_make(f[k][9], f[k][10], f[k][11]);
        pr[k].radius = s[k][0]; pr[k].half_height = s[k][1]; pr[k].half = v3_make(s[k][0], s[k][1], s[k][2]);
    }
    manifold m; primitive_pair(kind_a, &pr[0], kind_b, &pr[1], query, &m);
    for (uint32_t i = 0u; i < m.count; ++i) {
        points[3u * i] = m.position[i].x; points[3u * i + 1u] = m.position[i].y; points[3u * i + 2u] = m.position[i].z;
        normals[3u * i] = m.normal[i].x; normals[3u * i + 1u] = m.normal[i].y; normals[3u * i + 2u] = m.normal[i].z;
        penetration[i] = m.penetration[i]; keys[i] = m.key[i];
    }
    return m.count;
}

void nko_prim_frame(const float pose[7], float frame[12]) {
    shape_row s; memset(&s, 0, sizeof(s));
    const prim p = make_prim(s, xform_load(pose));
    const v3 c[4] = {p.cx, p.cy, p.cz, p.t};
    for (int i = 0; i < 4; ++i) { frame[3 * i] = c[i].x; frame[3 * i + 1] = c[i].y; frame[3 * i + 2] = c[i].z; }
}

/* ---- contact identity (nk/contact/contact_identity.hpp:98-157) ----------- */
static int32_t quantize_coord(float value) {
    const float scaled = value * 4096.0f;
    const float rounded = scaled >= 0.0f ? scaled + 0.5f : scaled - 0.5f;
    return (int32_t)rounded;
}
static uint64_t hash_word(uint64_t hash, uint64_t word) { hash ^= word; hash *= 1099511628211ull; return hash; }
static uint64_t feature_token(uint32_t feature, v3 p) {
    if (feature != 0xffffffffu) return 0x8000000000000000ull | (uint64_t)feature;
    uint64_t h = 1469598103934665603ull;
    h = hash_word(h, (uint32_t)quantize_coord(p.x)); h = hash_word(h, (uint32_t)quantize_coord(p.y));
    h = hash_word(h, (uint32_t)quantize_coord(p.z));
    return h & 0x7fffffffffffffffull;
}
/* MakeContactId for two CollidableRefs of type 0 with a < b (:108-157): pair word, then the feature hash over
 * both sides' tokens, the manifold slot and the two (zero) element words. */
static void contact_id(uint32_t a, uint32_t b, v3 la, v3 lb, uint32_t feature, uint32_t manifold_slot, uint64_t out[2]) {
    uint64_t h = 1469598103934665603ull;
    h = hash_word(h, feature_token(feature, la)); h = hash_word(h, feature_token(feature, lb));
    h = hash_word(h, manifold_slot); h = hash_word(h, 0u); h = hash_word(h, 0u);
    out[0] = ((uint64_t)(a & 0x0fffffffu) << 32u) | (uint64_t)(b & 0x0fffffffu);
    out[1] = h;
}
static v3 inverse_transform_point(xform xf, v3 wp) {   /* prims_types.cuh:98-105 */
    const v3 v = v3_sub(wp, xf.p);
    const v3 qv = v3_make(-xf.r.x, -xf.r.y, -xf.r.z);
    const v3 t = v3_scale(v3_cross(qv, v), 2.0f);
    return v3_add(v3_add(v, v3_scale(t, xf.r.w)), v3_cross(qv, t));
}

/* ---- NarrowphasePrimitives (narrowphase_prims.cu:181-366, analytic route) ---- */
void nko_env_narrowphase(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const size_t bbase = (size_t)env * t->nb;
    const float separation = fmaxf(w->cfg.solver_contact_margin, 0.0005f);   /* :425 */
    const float reach = contact_query_reach(0.0f, w->cfg.solver_contact_margin);
    const uint32_t live = w->pair_count[env];
    uint32_t contacts = 0u;
    for (uint32_t slot = 0u; slot < t->slots; ++slot) {
        const size_t gid = (size_t)env * t->slots + slot;
        manifold m; m.count = 0u;
        uint32_t a = 0u, b = 0u;
        uint32_t law = 2u;   /* kContactLawSpeculative unless a side's profile is MuJoCo-sourced (:232, 268-276) */
        if (slot < live) {
            a = w->candidate_pairs[gid * 2u]; b = w->candidate_pairs[gid * 2u + 1u];
            const shape_row sa = load_shape(t->shape_table, a), sb = load_shape(t->shape_table, b);
            const xform xa = xform_load(w->body_pose + (bbase + a) * 7u), xb = xform_load(w->body_pose + (bbase + b) * 7u);
            const prim pa = make_prim(sa, xa), pb = make_prim(sb, xb);
            const int has_a = sa.profile < t->n_profiles, has_b = sb.profile < t->n_profiles;
            if ((has_a && t->profile_law[sa.profile] == 1u) || (has_b && t->profile_law[sb.profile] == 1u)) law = 0u;   /* kContactLawCompliant */
            float query_margin = separation;
            if (law == 0u) {   /* :277-281: the profiles' margin + gap */
                const float margin_a = has_a ? t->profile_margin[2u * sa.profile] + t->profile_margin[2u * sa.profile + 1u] : 0.0f;
                const float margin_b = has_b ? t->profile_margin[2u * sb.profile] + t->profile_margin[2u * sb.profile + 1u] : 0.0f;
                query_margin = margin_a + margin_b;
            }
            /* :236-250 query band; both speeds are zero for link-owned collidables, a free body's own row moves with it */
            float speeds[2] = {0.0f, 0.0f};
            const uint32_t ends[2] = {a, b};
            for (uint32_t side = 0u; side < 2u && t->free_body; ++side) {
                if (ends[side] != t->link_body[0]) continue;
                const size_t at = bbase + ends[side];
                const float* center = w->body_pose + at * 7u, *lo = w->body_aabb_lo + at * 3u, *hi = w->body_aabb_hi + at * 3u;
                const v3 extent = v3_make(fmaxf(fabsf(lo[0] - center[0]), fabsf(hi[0] - center[0])), fmaxf(fabsf(lo[1] - center[1]), fabsf(hi[1] - center[1])),
                                          fmaxf(fabsf(lo[2] - center[2]), fabsf(hi[2] - center[2])));
                const float* lv = w->body_linear_velocity + at * 3u, *av = w->body_angular_velocity + at * 3u;
                speeds[side] = fmaxf(0.0f, sqrtf(lv[0] * lv[0] + lv[1] * lv[1] + lv[2] * lv[2]) +
                                           sqrtf((av[0] * av[0] + av[1] * av[1] + av[2] * av[2]) * (extent.x * extent.x + extent.y * extent.y + extent.z * extent.z)));
            }
            const float query = fmaxf(query_margin, fminf(contact_motion_radius(2.0f * separation, w->cfg.fixed_dt, speeds[0], speeds[1], 0.9f), reach));
            primitive_pair(sa.kind, &pa, sb.kind, &pb, query, &m);
            if (law != 0u) for (uint32_t i = 0u; i < m.count; ++i) m.penetration[i] += separation;   /* :295-296 */
        }
        w->ucontact_count[gid] = m.count;
        w->ucontact_law[gid] = law;
        for (uint32_t i = 0u; i < m.count; ++i) {
            const size_t at = gid * 4u + i;
            w->ucontact_point[3u * at] = m.position[i].x; w->ucontact_point[3u * at + 1u] = m.position[i].y; w->ucontact_point[3u * at + 2u] = m.position[i].z;
            w->ucontact_normal[3u * at] = m.normal[i].x; w->ucontact_normal[3u * at + 1u] = m.normal[i].y; w->ucontact_normal[3u * at + 2u] = m.normal[i].z;
            w->ucontact_depth[at] = m.penetration[i];
            w->ucontact_a[at] = a; w->ucontact_b[at] = b;
            /* MakeContactId with CollidableRef type 0: a < b already canonical (:108-157) */
            const uint32_t feature = m.key[i] == 0u ? 0xffffffffu : (uint32_t)m.key[i];
            const v3 la = inverse_transform_point(xform_load(w->body_pose + (bbase + a) * 7u), m.position[i]);
            const v3 lb = inverse_transform_point(xform_load(w->body_pose + (bbase + b) * 7u), m.position[i]);
            uint64_t id[2];
            contact_id(a, b, la, lb, feature, i, id);
            w->ucontact_id_pair[at] = id[0];
            w->ucontact_id_feature[at] = id[1];
        }
        contacts += m.count;
    }
    w->contact_count[env] = contacts;
}

/* contact_query.hpp:33-40 ContactProjectionRoundoff */
static double projection_roundoff(v3 start, v3 end, v3 axis) {
    const double gamma = 3.0 * FLT_EPSILON / (1.0 - 3.0 * FLT_EPSILON);
    return gamma * (fabs((double)axis.x) * (fabs((double)start.x) + fabs((double)end.x)) +
                    fabs((double)axis.y) * (fabs((double)start.y) + fabs((double)end.y)) +
                    fabs((double)axis.z) * (fabs((double)start.z) + fabs((double)end.z)));
}

/* ---- exported restatements for the unit pins ---- */
double nko_contact_projection_roundoff(const float start[3], const float end[3], const float axis[3]) {
    return projection_roundoff(v3_make(start[0], start[1], start[2]), v3_make(end[0], end[1], end[2]), v3_make(axis[0], axis[1], axis[2]));
}
float nko_contact_query_reach(float thickness, float margin) { return contact_query_reach(thickness, margin); }
float nko_contact_motion_radius(float base, float dt, float sa, float sb, float relax) { return contact_motion_radius(base, dt, sa, sb, relax); }
int nko_shape_filter_admits(uint32_t ta, uint32_t aa, uint32_t ga_, uint32_t tb, uint32_t ab, uint32_t gb_) {
    return shape_filter_admits(ta, aa, ga_, tb, ab, gb_);
}
void nko_compose_transform(const float parent[7], const float child[7], float out[7]) {
    xform_store(out, nko_compose_hd(xform_load(parent), xform_load(child)));
}
void nko_make_contact_id(uint32_t a, uint32_t b, const float local_a[3], const float local_b[3], uint32_t feature,
                         uint32_t manifold_slot, uint64_t out[2]) {
    contact_id(a, b, v3_make(local_a[0], local_a[1], local_a[2]), v3_make(local_b[0], local_b[1], local_b[2]), feature, manifold_slot, out);
}

/* math/cuda_vec_ops.cuh:150-183 NormalizeOrUp + ContactTangentBasis */
void nko_contact_tangent_basis(const float normal[3], float t1[3], float t2[3]) {
    v3 n = v3_make(normal[0], normal[1], normal[2]);
    const float l = v3_dot(n, n);
    if (l > 1.0e-10f) { const float inv = nko_rsqrt(l); n = v3_make(n.x * inv, n.y * inv, n.z * inv); }
    else n = v3_make(0.0f, 0.0f, 1.0f);
    v3 reference = v3_make(1.0f, 0.0f, 0.0f);
    if (fabsf(n.x) > 0.9f) reference = v3_make(0.0f, 1.0f, 0.0f);
    const float proj = v3_dot(reference, n);
    v3 ta = v3_make(reference.x - proj * n.x, reference.y - proj * n.y, reference.z - proj * n.z);
    const float len_sq = v3_dot(ta, ta);
    if (len_sq > 1.0e-12f) { const float s = nko_rsqrt(len_sq); ta = v3_make(ta.x * s, ta.y * s, ta.z * s); }
    else ta = v3_make(1.0f, 0.0f, 0.0f);
    const v3 tb = v3_cross(n, ta);
    t1[0] = ta.x; t1[1] = ta.y; t1[2] = ta.z; t2[0] = tb.x; t2[1] = tb.y; t2[2] = tb.z;
}

/* union_types.cuh:187-193 ContactRowBound */
static uint32_t contact_row_bound(const uint32_t* extent, uint32_t env, uint32_t contact_rows) {
    const uint32_t previous = extent[2u * env], current = extent[2u * env + 1u];
    if (previous == 0u || current == 0u) return contact_rows;
    const uint32_t m = (previous > current ? previous : current) - 1u;
    return m < contact_rows ? m : contact_rows;
}

/* nk/solve/collidable_owner.hpp:25-62 ResolveCollidableOwner (one articulation per env) */
static uint32_t resolve_side(const nko_template* t, uint32_t env, uint32_t collidable, int32_t body_id,
                             uint32_t* index, uint32_t* link) {
    *index = NKO_INVALID; *link = NKO_INVALID;
    if (collidable >= t->nb) return NKO_INVALID;
    uint32_t body = collidable;
    if (body_id < 0) return NKO_SIDE_STATIC;
    const uint32_t proxy = t->body_collidable_body[body];
    if (proxy != NKO_INVALID) {
        if (proxy >= t->nb) return NKO_INVALID;
        body = proxy;
        if (t->body_collidable_body[body] != NKO_INVALID) return NKO_INVALID;
    }
    const uint32_t l = t->body_to_link[body];
    if (l == NKO_INVALID) { *index = env * t->nb + body; return NKO_SIDE_RIGID; }
    if (l >= t->nl) return NKO_INVALID;
    if (t->body_to_articulation[body] >= 1u) return NKO_INVALID;
    *link = env * t->nl + l; *index = env;
    return NKO_SIDE_ARTIC;
}

/* articulation_types.cuh:193-238 AccumulateChainJointForce */
void nko_accumulate_chain(const nko_world* w, uint32_t env, uint32_t link_local, uint32_t dof_index, v3 point, v3 f, v3 zero, float* out) {
    const nko_template* t = &w->t;
    const uint32_t stride = t->max_dof;
    const uint8_t type = t->joint_type[link_local];
    if (type == NKO_FLOATING && t->free_body) {
        /* a free body's six coordinates: its linear velocity, then its angular velocity about the centre of mass, in world
         * axes - the row's jlin and jang = (point - com) x jlin (assemble_rows.cu:537-538, 680-681; TileBlock::Jacobian,
         * block_descent_tile.cuh:556-563) */
        float com[3];
        nko_body_center_of_mass(w, env, com);
        const v3 jang = v3_add(v3_cross(v3_sub(point, v3_make(com[0], com[1], com[2])), f), zero);
        const float lin[3] = {f.x, f.y, f.z}, ang[3] = {jang.x, jang.y, jang.z};
        for (uint32_t b = 0u; b < 3u; ++b) {
            if (dof_index + b < stride) out[dof_index + b] += lin[b];
            if (dof_index + 3u + b < stride) out[dof_index + 3u + b] += ang[b];
        }
        return;
    }
    if (type == NKO_FLOATING) {
        const xform base = xform_load(w->base_pose + (size_t)env * 7u);
        const v3 lever = v3_sub(point, base.p);
        const v3 ex = nko_rotate_normalized(base.r, v3_make(1, 0, 0)), ey = nko_rotate_normalized(base.r, v3_make(0, 1, 0)),
                 ez = nko_rotate_normalized(base.r, v3_make(0, 0, 1));
        const float ang[3] = {v3_dot(v3_cross(ex, lever), f) + v3_dot(ex, zero), v3_dot(v3_cross(ey, lever), f) + v3_dot(ey, zero),
                              v3_dot(v3_cross(ez, lever), f) + v3_dot(ez, zero)};
        const float lin[3] = {v3_dot(ex, f), v3_dot(ey, f), v3_dot(ez, f)};
        for (uint32_t b = 0u; b < 3u; ++b) {
            if (dof_index + b < stride) out[dof_index + b] += ang[b];
            if (dof_index + 3u + b < stride) out[dof_index + 3u + b] += lin[b];
        }
        return;
    }
    const xform pose = xform_load(w->link_pose + ((size_t)env * t->nl + link_local) * 7u);
    const v3 axis_world = nko_rotate_normalized(pose.r, v3_make(t->joint_axis[3u * link_local], t->joint_axis[3u * link_local + 1u],
                                                                 t->joint_axis[3u * link_local + 2u]));
    float entry;
    if (type == NKO_PRISMATIC) entry = v3_dot(axis_world, f);
    else {
        const v3 lever = v3_sub(point, pose.p);
        entry = v3_dot(v3_cross(axis_world, lever), f) + v3_dot(axis_world, zero);
    }
    if (dof_index < stride) out[dof_index] += entry;
}

/* assemble_rows.cu:122-169 ComputeContactChainJacobianKernel for one row side */
static void chain_jacobian_row(const nko_world* w, uint32_t env, uint32_t link_global, v3 point, v3 dir, float* out) {
    const nko_template* t = &w->t;
    if (link_global == NKO_INVALID) return;
    for (uint32_t k = 0u; k < t->max_dof; ++k) out[k] = 0.0f;
    uint32_t link = link_global - env * t->nl;
    while (link != NKO_INVALID) {
        if (nko_joint_dof(t->joint_type[link]) != 0u) nko_accumulate_chain(w, env, link, t->link_dof[link], point, dir, v3_make(0, 0, 0), out);
        link = t->parent_link[link];
    }
}

/* One shape's contact parameters as MergeContactParams takes them: mu1, mu2, solref[2], solimp[5], margin, gap; a
 * shape without a profile has the defaults (assemble_rows.cu:41-52 DefaultProfile, mu 1). */
static void profile_terms(const nko_template* t, uint32_t profile, float out[14]) {
    const float defaults[14] = {1.0f, 1.0f, 0.02f, 1.0f, 0.9f, 0.95f, 0.001f, 0.5f, 2.0f, 0.0f, 0.0f, 0.0f, 1.0f, 3.0f};
    memcpy(out, defaults, sizeof(defaults));
    if (profile >= t->n_profiles) return;
    out[0] = t->profile_mu[2u * profile]; out[1] = t->profile_mu[2u * profile + 1u];
    out[2] = t->profile_solref[2u * profile]; out[3] = t->profile_solref[2u * profile + 1u];
    for (uint32_t k = 0u; k < 5u; ++k) out[4u + k] = t->profile_solimp[5u * profile + k];
    out[9] = t->profile_margin[2u * profile]; out[10] = t->profile_margin[2u * profile + 1u];
    for (uint32_t k = 0u; k < 3u; ++k) out[11u + k] = t->profile_mix[3u * profile + k];
}
/* scene/contact_filter.hpp:89-137 MergeContactParams with arithmetic friction mixing: the side of higher priority gives
 * friction and condim and all of the mixing weight; at equal priority friction and condim take the larger and the weight
 * is solmix_a / (solmix_a + solmix_b), a side whose solmix is below mjMINVAL deferring to the other.  solref is mixed, or
 * the minimum when either is in direct form; solimp is mixed; margins and gaps add. */
void nko_merge_contact_params(const float a[14], const float b[14], float out[12]) {
    float mix;
    if (a[11] != b[11]) {
        const float* w = a[11] > b[11] ? a : b;
        mix = a[11] > b[11] ? 1.0f : 0.0f;
        out[11] = w[13]; out[0] = w[0]; out[1] = w[1];
    } else {
        out[11] = a[13] > b[13] ? a[13] : b[13];
        out[0] = a[0] > b[0] ? a[0] : b[0];
        out[1] = a[1] > b[1] ? a[1] : b[1];
        const int a_ok = a[12] >= 1e-15f, b_ok = b[12] >= 1e-15f;
        if (a_ok && b_ok) mix = a[12] / (a[12] + b[12]);
        else if (!a_ok && !b_ok) mix = 0.5f;
        else if (!a_ok) mix = 0.0f;
        else mix = 1.0f;
    }
    const float imix = 1.0f - mix;
    if (a[2] > 0.0f && b[2] > 0.0f) { out[2] = mix * a[2] + imix * b[2]; out[3] = mix * a[3] + imix * b[3]; }
    else { out[2] = a[2] < b[2] ? a[2] : b[2]; out[3] = a[3] < b[3] ? a[3] : b[3]; }
    for (int i = 0; i < 5; ++i) out[4 + i] = mix * a[4 + i] + imix * b[4 + i];
    out[9] = a[9] + b[9];
    out[10] = a[10] + b[10];
}
/* math/cuda_vec_ops.cuh:187-196 MuJoCoContactFrame */
static void mujoco_contact_frame(const float normal[3], v3 axis, float t1[3], float t2[3]) {
    v3 n = v3_make(normal[0], normal[1], normal[2]);
    const float l = v3_dot(n, n);
    if (l > 1.0e-10f) { const float inv = nko_rsqrt(l); n = v3_make(n.x * inv, n.y * inv, n.z * inv); }
    else n = v3_make(0.0f, 0.0f, 1.0f);
    v3 tangent = v3_sub(axis, v3_scale(n, v3_dot(n, axis)));
    if (v3_dot(tangent, tangent) < 0.25f) {
        const v3 reference = n.y > -0.5f && n.y < 0.5f ? v3_make(0.0f, 1.0f, 0.0f) : v3_make(0.0f, 0.0f, 1.0f);
        tangent = v3_sub(reference, v3_scale(n, v3_dot(n, reference)));
    }
    const v3 a = v3_scale(tangent, nko_rsqrt(v3_dot(tangent, tangent)));
    const v3 b = v3_cross(n, a);
    t1[0] = a.x; t1[1] = a.y; t1[2] = a.z; t2[0] = b.x; t2[1] = b.y; t2[2] = b.z;
}

/* ---- AssembleRows (assemble_rows.cu:325-394 ranges/clear, 406-801 emit, 1587-1605 chain J) ---- */
/* EmitJointRowsKernel (assemble_rows.cu:803-1026): stable per-link slots after the contact rows - lower and upper
 * limit (2 per link), dry friction (1 per link), drive (1 per link).  Every row acts on one coordinate: J = +-e_joint
 * over a zeroed Jacobian row.  Only the native (non-MuJoCo) law is built. */
void nko_env_joint_rows(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t R = t->rows_per_env, CR = t->contact_rows_per_env, nl = t->nl, md = t->max_dof;
    const uint32_t limit_rows = t->joint_limit_rows, friction_rows = t->joint_friction_rows, drive_rows = t->joint_drive_rows;
    if (limit_rows + friction_rows + drive_rows == 0u) return;
    const float dt = w->cfg.fixed_dt;
    const int position_pass = w->cfg.solver_pos_iters > 0u;
    nko_row* rows = (nko_row*)w->urows;
    const size_t lbase = (size_t)env * nl;
    for (uint32_t slot = 0u; slot < limit_rows + friction_rows + drive_rows; ++slot) {
        const size_t rs = (size_t)env * R + CR + slot;
        float* J = w->chain_jacobian + rs * md;
        for (uint32_t k = 0u; k < md; ++k) J[k] = 0.0f;   /* :1000-1004 */
        nko_row row; memset(&row, 0, sizeof(row));
        w->row_cj_link[rs] = NKO_INVALID; w->row_cj_link_b[rs] = NKO_INVALID;
        w->row_penetration[rs] = 0.0f;
        if (slot < limit_rows) {   /* EmitJointLimitRow :805-882 */
            const uint32_t l = slot / 2u, side = slot & 1u;
            const size_t link = lbase + l;
            const int scalar = nko_joint_dof(t->joint_type[l]) == 1u;
            if (scalar && (t->joint_limit_flags[l] & (1u << side)) != 0u && dt > 0.0f) {
                const float sign = side == 0u ? 1.0f : -1.0f;
                const float bound = side == 0u ? t->joint_limit_lower[l] : t->joint_limit_upper[l];
                const float signed_distance = side == 0u ? w->q[link] - bound : bound - w->q[link];
                const float target_velocity = -(position_pass ? fmaxf(signed_distance, 0.0f) : signed_distance) / dt;
                const float capped_velocity = fminf(target_velocity, w->cfg.solver_baumgarte_max_velocity);
                row.flags = NKO_ROW_ACTIVE | (side == 0u ? NKO_ROW_JOINT_LIMIT_LOWER : NKO_ROW_JOINT_LIMIT_UPPER);
                row.group_first = (uint32_t)rs; row.group_normal_count = 1u; row.env = env;
                row.rhs = capped_velocity / dt;
                row.lower = 0.0f; row.upper = FLT_MAX;
                row.a.kind = NKO_SIDE_ARTIC; row.a.index = env;
                J[t->link_dof[l]] = sign;
                w->row_penetration[rs] = fmaxf(-signed_distance, 0.0f);
                if (t->joint_law[l] == 1u) {   /* :860-877: the limit as a compliant row inside its margin, on the nearer bound only */
                    const float pos = signed_distance - t->joint_limit_margin[l];
                    const float* reference = t->joint_limit_reference + 7u * l;
                    const float invweight = w->dof_invweight0[(size_t)env * md + t->link_dof[l]];
                    float terms[6], discrete[3];
                    nko_compliant_row_terms(reference, reference + 2u, pos, pos, 0.0f, invweight, dt, 1, terms);
                    nko_discretize_compliant_row(terms[4], terms[5], terms[1], dt, discrete);
                    row.flags |= NKO_ROW_MUJOCO;
                    const int lower_nearest = w->q[link] - t->joint_limit_lower[l] < t->joint_limit_upper[l] - w->q[link];
                    if (pos >= 0.0f || lower_nearest != (side == 0u)) {
                        row.flags &= ~NKO_ROW_ACTIVE;
                        w->lambda[rs] = 0.0f;
                    }
                    row.rhs = discrete[1]; row.compliance_alpha = discrete[0];
                    w->row_reference_velocity_gain[rs] = discrete[2];
                    w->row_invweight[rs] = invweight;
                }
                if (row.flags & NKO_ROW_ACTIVE) w->row_count[env] += 1u;
            } else w->lambda[rs] = 0.0f;
        } else if (slot < limit_rows + friction_rows) {   /* EmitJointFrictionRows :886-934 */
            const uint32_t l = slot - limit_rows;
            w->lambda[rs] = 0.0f;
            const float friction = t->joint_frictionloss[l];
            if (nko_joint_dof(t->joint_type[l]) == 1u && friction > 0.0f && dt > 0.0f) {
                row.flags = NKO_ROW_ACTIVE | NKO_ROW_VELOCITY_ONLY;
                row.group_first = (uint32_t)rs; row.group_normal_count = 1u; row.env = env;
                row.lower = -friction * dt; row.upper = friction * dt;
                row.a.kind = NKO_SIDE_ARTIC; row.a.index = env;
                J[t->link_dof[l]] = 1.0f;
                if (t->joint_law[l] == 1u) {   /* :921-931: dry friction regularised by its own solref / solimp */
                    const float* reference = t->joint_friction_reference + 7u * l;
                    const float invweight = w->dof_invweight0[(size_t)env * md + t->link_dof[l]];
                    float terms[6], discrete[3];
                    nko_compliant_row_terms(reference, reference + 2u, 0.0f, 0.0f, 0.0f, invweight, dt, 1, terms);
                    nko_discretize_compliant_row(terms[4], terms[5], terms[1], dt, discrete);
                    row.flags |= NKO_ROW_MUJOCO;
                    row.compliance_alpha = discrete[0];
                    w->row_reference_velocity_gain[rs] = discrete[2];
                    w->row_invweight[rs] = invweight;
                }
                w->row_count[env] += 1u;
            }
        } else {   /* EmitJointDriveRows :938-971 */
            const uint32_t l = slot - limit_rows - friction_rows;
            const size_t link = lbase + l;
            w->lambda[rs] = 0.0f;
            const float effort = fminf(fmaxf(w->drive_command[link], w->drive_lower[link]), w->drive_upper[link]);
            if (nko_joint_dof(t->joint_type[l]) == 1u && effort != 0.0f) {
                row.flags = NKO_ROW_ACTIVE | NKO_ROW_VELOCITY_ONLY;
                row.group_first = (uint32_t)rs; row.group_normal_count = 1u; row.env = env;
                row.a.kind = NKO_SIDE_ARTIC; row.a.index = env;
                J[t->link_dof[l]] = 1.0f;
                row.lower = row.upper = effort * dt;
                w->lambda[rs] = row.lower;   /* the row admits one impulse */
                w->row_count[env] += 1u;
            }
        }
        rows[rs] = row;
    }
}

void nko_env_assemble_rows(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t R = t->rows_per_env, S = t->slots, CR = t->contact_rows_per_env;
    if (R == 0u) return;
    const float dt = w->cfg.fixed_dt;
    nko_row* rows = (nko_row*)w->urows + (size_t)env * R;
    float* lambda = w->lambda + (size_t)env * R;
    float* pen = w->row_penetration + (size_t)env * R;
    uint32_t* cj_link = w->row_cj_link + (size_t)env * R, *cj_link_b = w->row_cj_link_b + (size_t)env * R;
    float* cj_point = w->row_cj_point + (size_t)env * R * 3u, *cj_point_b = w->row_cj_point_b + (size_t)env * R * 3u;
    uint32_t* extent = w->contact_row_extent;
    /* InitializePairDrivenRangesKernel :336-360 */
    w->row_count[env] = 0u;
    extent[2u * env] = extent[2u * env + 1u];
    extent[2u * env + 1u] = 1u;
    uint32_t carry = 0u;
    const uint32_t range_bound = contact_row_bound(extent, env, CR);
    for (uint32_t slot = 0u; slot < S; ++slot) {
        const uint32_t points = w->ucontact_count[(size_t)env * S + slot];
        w->ucontact_row_range[((size_t)env * S + slot) * 2u] = env * R + carry * 4u;
        w->ucontact_row_range[((size_t)env * S + slot) * 2u + 1u] = points;
        if (carry * 4u < range_bound) w->contact_material[(size_t)env * S + slot] = 0u;   /* :358 */
        carry += points;
    }
    /* ClearPairDrivenRowsKernel :366-394 */
    {
        const uint32_t bound = contact_row_bound(extent, env, CR);
        for (uint32_t local = 0u; local < R; ++local)
            if (local < bound) {
                lambda[local] = 0.0f; pen[local] = 0.0f; cj_link[local] = NKO_INVALID; cj_link_b[local] = NKO_INVALID;
                if (rows[local].flags != 0u) rows[local].flags = 0u;
            }
    }
    /* PackQdotFlatMultiKernel :200-214 */
    for (uint32_t d = 0u; d < t->max_dof; ++d) {
        float v = 0.0f;
        if (d < t->nv) {
            const uint32_t link = t->dof_link[d], c = t->dof_component[d];
            v = c == NKO_INVALID ? w->qdot[(size_t)env * t->nl + link] : w->link_velocity[((size_t)env * t->nl + link) * 6u + c];
        }
        w->qdot_flat[(size_t)env * t->max_dof + d] = v;
    }
    /* EmitPairDrivenRowsKernel :453-801, speculative law, condim 3 */
    uint32_t active_rows = 0u;
    for (uint32_t slot = 0u; slot < S; ++slot) {
        const size_t gid = (size_t)env * S + slot;
        const uint32_t base = w->ucontact_row_range[gid * 2u] - env * R, P = w->ucontact_row_range[gid * 2u + 1u];
        const uint32_t n_active_in = w->ucontact_count[gid];
        if (n_active_in > 0u) {
            const uint32_t e = base + P * 4u + 1u;   /* :464-472 extent past the slot's rows */
            if (e > extent[2u * env + 1u]) extent[2u * env + 1u] = e;
        }
        if (n_active_in == 0u) continue;
        uint32_t n_active = n_active_in;
        const uint32_t local_a = w->ucontact_a[gid * 4u], local_b = w->ucontact_b[gid * 4u];
        shape_row sa, sb; memset(&sa, 0, sizeof(sa)); memset(&sb, 0, sizeof(sb)); sa.body_id = sb.body_id = -1;
        if (local_a < t->nb) sa = load_shape(t->shape_table, local_a);
        if (local_b < t->nb) sb = load_shape(t->shape_table, local_b);
        uint32_t idx_a, idx_b, link_a, link_b;
        uint32_t kind_a = resolve_side(t, env, local_a, sa.body_id, &idx_a, &link_a);
        uint32_t kind_b = resolve_side(t, env, local_b, sb.body_id, &idx_b, &link_b);
        if (kind_a == NKO_INVALID || kind_b == NKO_INVALID) {
            w->env_status[env] |= NKO_STATUS_INVALID_ENDPOINT;
            n_active = 0u; kind_a = kind_b = NKO_SIDE_STATIC;
        }
        if (kind_a == NKO_SIDE_STATIC) idx_a = NKO_INVALID;
        if (kind_b == NKO_SIDE_STATIC) idx_b = NKO_INVALID;
        const int position_pass = w->cfg.solver_pos_iters > 0u;
        const uint32_t law = w->ucontact_law[gid];
        const int mujoco = law == 0u;   /* kContactLawCompliant (:480) */
        /* the two sides' profiles merged (:540-594; contact_filter.hpp:89-137), a side without one at the defaults */
        float side_a[14], side_b[14], merged[12];
        profile_terms(t, sa.profile, side_a); profile_terms(t, sb.profile, side_b);
        nko_merge_contact_params(side_a, side_b, merged);
        if (mujoco) { merged[0] = fmaxf(1.0e-5f, merged[0]); merged[1] = fmaxf(1.0e-5f, merged[1]); }   /* :573-576 */
        const float mu1 = merged[0], mu2 = merged[1];
        const int friction_rows = merged[11] == 3.0f;   /* condim 3: a normal and two tangents, else the normal alone (:721, 763) */
        const float* solref = merged + 2, *solimp = merged + 4;
        const float margin = merged[9];
        const uint32_t weight_a = kind_a == NKO_SIDE_ARTIC ? t->link_body[link_a - env * t->nl] : local_a;
        const uint32_t weight_b = kind_b == NKO_SIDE_ARTIC ? t->link_body[link_b - env * t->nl] : local_b;
        const float* invweight0 = w->body_invweight0 + (size_t)env * t->nb * 2u;
        const float invweight = mujoco ? invweight0[2u * weight_a] + invweight0[2u * weight_b] : 0.0f;   /* :597 */
        const int pyramidal = mujoco && t->cone == 0u && friction_rows;   /* :598 */
        const float impratio = t->impratio;
        v3 frame_axis = v3_make(0, 0, 0);   /* :601-605: a capsule on a plane aligns the pyramid with the capsule's axis */
        if (pyramidal && sa.kind == 1u && sb.kind == 3u) frame_axis = nko_prim_rotate(xform_load(w->body_pose + ((size_t)env * t->nb + local_a) * 7u).r, v3_make(0, 0, 1));
        if (pyramidal && sb.kind == 1u && sa.kind == 3u) frame_axis = nko_prim_rotate(xform_load(w->body_pose + ((size_t)env * t->nb + local_b) * 7u).r, v3_make(0, 0, 1));
        w->contact_material[gid] = n_active > 0u ? nko_contact_material_merged(merged, law, t->cone) : 0u;   /* :620-623 */
        for (uint32_t p = 0u; p < P; ++p) {
            /* velocity_only keeps every point; a compliant point lives inside its margin (:625-626) */
            const int live = p < n_active && p < 4u && (!mujoco || w->ucontact_depth[gid * 4u + p] + margin > 0.0f);
            const size_t mp = gid * 4u + p;
            const uint32_t normal_row = base + p, t1_row = base + P + p, t2_row = base + 2u * P + p;
            v3 n = v3_make(0, 0, 1), point = v3_make(0, 0, 0), t0 = v3_make(1, 0, 0), t1v = v3_make(0, 1, 0);
            if (live) {
                const v3 raw = v3_make(w->ucontact_normal[3u * mp], w->ucontact_normal[3u * mp + 1u], w->ucontact_normal[3u * mp + 2u]);
                const float len = sqrtf(raw.x * raw.x + raw.y * raw.y + raw.z * raw.z);   /* :193-197 NormalizedHostExpr */
                n = len < 1e-12f ? v3_make(0, 0, 0) : v3_make(raw.x / len, raw.y / len, raw.z / len);
                point = v3_make(w->ucontact_point[3u * mp], w->ucontact_point[3u * mp + 1u], w->ucontact_point[3u * mp + 2u]);
                float a[3], b[3];
                nko_contact_tangent_basis(&w->ucontact_normal[3u * mp], a, b);
                t0 = v3_make(a[0], a[1], a[2]); t1v = v3_make(b[0], b[1], b[2]);
            }
            if (pyramidal) {   /* :651-690: four scalar edges n +- mu t of the friction pyramid */
                if (live) {
                    float a[3], b[3];
                    mujoco_contact_frame(&w->ucontact_normal[3u * mp], frame_axis, a, b);
                    t0 = v3_make(a[0], a[1], a[2]); t1v = v3_make(b[0], b[1], b[2]);
                }
                const float d0 = w->ucontact_depth[mp];
                const float edge_invweight = (invweight + mu1 * mu1 * invweight) * 2.0f * mu1 * mu1 / impratio;
                const float pos = -d0 - margin;
                float terms[6], discrete[3];
                nko_compliant_row_terms(solref, solimp, pos, pos, 0.0f, edge_invweight, dt, 1, terms);
                nko_discretize_compliant_row(terms[4], terms[5], terms[1], dt, discrete);
                for (uint32_t edge = 0u; edge < 4u; ++edge) {
                    const uint32_t rs = base + edge * P + p;
                    nko_row row; memset(&row, 0, sizeof(row));
                    lambda[rs] = 0.0f; pen[rs] = 0.0f; cj_link[rs] = NKO_INVALID; cj_link_b[rs] = NKO_INVALID;
                    if (live) {
                        const float mu = edge < 2u ? mu1 : mu2;
                        const v3 tangent = edge < 2u ? t0 : t1v;
                        const v3 dir = v3_add(n, v3_scale(tangent, (edge & 1u) ? -mu : mu));
                        row.flags = NKO_ROW_ACTIVE | NKO_ROW_MUJOCO | NKO_ROW_PYRAMIDAL | (edge == 0u ? NKO_ROW_CONTACT_NORMAL : 0u);
                        row.group_first = env * R + rs; row.group_normal_count = 1u; row.env = env;
                        row.rhs = discrete[1]; row.compliance_alpha = discrete[0];
                        row.lower = 0.0f; row.upper = FLT_MAX; row.mu = mu1; row.friction_secondary = mu2;
                        row.a.kind = kind_a; row.a.index = idx_a; row.a.jlin = dir;
                        row.b.kind = kind_b; row.b.index = idx_b; row.b.jlin = v3_scale(dir, -1.0f);
                        if (kind_a == NKO_SIDE_ARTIC) { cj_link[rs] = link_a; cj_point[3u * rs] = point.x; cj_point[3u * rs + 1u] = point.y; cj_point[3u * rs + 2u] = point.z; }
                        if (kind_b == NKO_SIDE_ARTIC) { cj_link_b[rs] = link_b; cj_point_b[3u * rs] = point.x; cj_point_b[3u * rs + 1u] = point.y; cj_point_b[3u * rs + 2u] = point.z; }
                        w->row_reference_velocity_gain[(size_t)env * R + rs] = discrete[2];
                        w->row_invweight[(size_t)env * R + rs] = edge_invweight;
                        ++active_rows;
                    }
                    rows[rs] = row;
                }
                continue;
            }
            {   /* normal row :692-755 */
                nko_row row; memset(&row, 0, sizeof(row));
                row.a.kind = row.b.kind = NKO_SIDE_STATIC; row.a.index = row.b.index = NKO_INVALID;
                lambda[normal_row] = 0.0f; pen[normal_row] = 0.0f; cj_link[normal_row] = NKO_INVALID; cj_link_b[normal_row] = NKO_INVALID;
                if (live) {
                    const float d0 = w->ucontact_depth[mp];
                    const v3 extent_v = v3_make(fabsf(point.x) + fabsf(n.x * d0), fabsf(point.y) + fabsf(n.y * d0), fabsf(point.z) + fabsf(n.z * d0));
                    const double roundoff = projection_roundoff(extent_v, extent_v, n);
                    const float clearance = roundoff > 0.0 ? nextafterf((float)roundoff, FLT_MAX) : 0.0f;
                    const float depth = d0 + clearance;
                    pen[normal_row] = mujoco ? fmaxf(d0, 0.0f) : depth;
                    row.flags = NKO_ROW_ACTIVE | NKO_ROW_CONTACT_NORMAL | (friction_rows ? NKO_ROW_BLOCK_NORMAL : 0u) | (mujoco ? NKO_ROW_MUJOCO : NKO_ROW_SPECULATIVE);
                    row.group_first = env * R + base; row.group_normal_count = P; row.env = env;
                    row.rhs = (fminf(depth, 0.0f) + (position_pass ? 0.0f : fminf(fmaxf(d0, 0.0f), w->cfg.solver_overlap_recovery_velocity * dt))) / (dt * dt);
                    row.compliance_alpha = 0.0f;   /* DiscretizeCompliantRow of a zero row: R = 0 (solref_solimp.hpp:40-44) */
                    if (mujoco) {   /* :714-731: the spring-damper reference of the merged solref / solimp at this depth */
                        const float pos = -d0 - margin;
                        float terms[6], discrete[3];
                        nko_compliant_row_terms(solref, solimp, pos, pos, 0.0f, invweight, dt, 1, terms);
                        nko_discretize_compliant_row(terms[4], terms[5], terms[1], dt, discrete);
                        row.rhs = discrete[1]; row.compliance_alpha = discrete[0];
                        w->row_reference_velocity_gain[(size_t)env * R + normal_row] = discrete[2];
                        w->row_invweight[(size_t)env * R + normal_row] = invweight;
                    }
                    row.lower = 0.0f; row.upper = FLT_MAX; row.mu = mu1; row.friction_secondary = mu2;
                    row.a.kind = kind_a; row.a.index = idx_a; row.a.jlin = n;
                    row.b.kind = kind_b; row.b.index = idx_b; row.b.jlin = v3_make(-n.x, -n.y, -n.z);
                    if (kind_a == NKO_SIDE_ARTIC) { cj_link[normal_row] = link_a; cj_point[3u * normal_row] = point.x; cj_point[3u * normal_row + 1u] = point.y; cj_point[3u * normal_row + 2u] = point.z; }
                    if (kind_b == NKO_SIDE_ARTIC) { cj_link_b[normal_row] = link_b; cj_point_b[3u * normal_row] = point.x; cj_point_b[3u * normal_row + 1u] = point.y; cj_point_b[3u * normal_row + 2u] = point.z; }
                    ++active_rows;
                    rows[normal_row] = row;
                } else rows[normal_row].flags = 0u;
            }
            const uint32_t trow[2] = {t1_row, t2_row};
            const v3 tdir[2] = {t0, t1v};
            for (uint32_t k = 0u; k < 2u; ++k) {   /* tangent rows :758-797 */
                const uint32_t rs = trow[k];
                nko_row row; memset(&row, 0, sizeof(row));
                row.a.kind = row.b.kind = NKO_SIDE_STATIC; row.a.index = row.b.index = NKO_INVALID;
                lambda[rs] = 0.0f; pen[rs] = 0.0f; cj_link[rs] = NKO_INVALID; cj_link_b[rs] = NKO_INVALID;
                if (live && friction_rows) {
                    const v3 dir = tdir[k];
                    row.flags = NKO_ROW_ACTIVE | NKO_ROW_BLOCK_TANGENT;
                    row.group_first = env * R + base; row.group_normal_count = P; row.env = env;
                    if (mujoco) {   /* :771-782: the tangent rows' compliance, which shapes the elliptic cone's metric */
                        const float mu = k == 0u ? mu1 : mu2;
                        const float tangent_invweight = invweight / impratio * (mu1 * mu1) / (mu * mu);
                        float terms[6], discrete[3];
                        nko_compliant_row_terms(solref, solimp, -w->ucontact_depth[mp] - margin, 0.0f, 0.0f, tangent_invweight, dt, 1, terms);
                        nko_discretize_compliant_row(terms[4], terms[5], terms[1], dt, discrete);
                        row.flags |= NKO_ROW_MUJOCO;
                        row.compliance_alpha = discrete[0];
                        w->row_reference_velocity_gain[(size_t)env * R + rs] = discrete[2];
                        w->row_invweight[(size_t)env * R + rs] = tangent_invweight;
                    }
                    row.lower = -FLT_MAX; row.upper = FLT_MAX; row.mu = mu1; row.friction_secondary = mu2;
                    row.a.kind = kind_a; row.a.index = idx_a; row.a.jlin = dir;
                    row.b.kind = kind_b; row.b.index = idx_b; row.b.jlin = v3_make(-dir.x, -dir.y, -dir.z);
                    if (kind_a == NKO_SIDE_ARTIC) { cj_link[rs] = link_a; cj_point[3u * rs] = point.x; cj_point[3u * rs + 1u] = point.y; cj_point[3u * rs + 2u] = point.z; }
                    if (kind_b == NKO_SIDE_ARTIC) { cj_link_b[rs] = link_b; cj_point_b[3u * rs] = point.x; cj_point_b[3u * rs + 1u] = point.y; cj_point_b[3u * rs + 2u] = point.z; }
                    ++active_rows;
                    rows[rs] = row;
                } else rows[rs].flags = 0u;
            }
        }
    }
    w->row_count[env] += active_rows;
    nko_env_joint_rows(w, env);
    /* chain Jacobians for both sides, then the shared-owner merge (:1587-1605, 172-186) */
    for (uint32_t r = 0u; r < R; ++r) {
        float* ja = w->chain_jacobian + ((size_t)env * R + r) * t->max_dof;
        float* jb = w->chain_jacobian_b + ((size_t)env * R + r) * t->max_dof;
        chain_jacobian_row(w, env, cj_link[r], v3_make(cj_point[3u * r], cj_point[3u * r + 1u], cj_point[3u * r + 2u]), rows[r].a.jlin, ja);
        chain_jacobian_row(w, env, cj_link_b[r], v3_make(cj_point_b[3u * r], cj_point_b[3u * r + 1u], cj_point_b[3u * r + 2u]), rows[r].b.jlin, jb);
        if ((rows[r].flags & NKO_ROW_ACTIVE) && rows[r].a.kind == NKO_SIDE_ARTIC && rows[r].b.kind == NKO_SIDE_ARTIC &&
            rows[r].a.index == rows[r].b.index)
            for (uint32_t i = 0u; i < t->max_dof; ++i) { ja[i] += jb[i]; jb[i] = 0.0f; }
    }
    /* PrepareContactRowsKernel (:1134-1140): a compliant row's reference acceleration includes the damping of the
     * velocity the step started from, ContactReferenceVelocity (:1072-1100) side A then side B */
    const float* start = w->step_qdot_flat + (size_t)env * t->max_dof;
    for (uint32_t r = 0u; r < R; ++r) {
        if ((rows[r].flags & NKO_ROW_ACTIVE) == 0u || (rows[r].flags & NKO_ROW_MUJOCO) == 0u) continue;
        float velocity = 0.0f;
        if (rows[r].a.kind == NKO_SIDE_ARTIC)
            for (uint32_t i = 0u; i < t->max_dof; ++i) velocity += w->chain_jacobian[((size_t)env * R + r) * t->max_dof + i] * start[i];
        if (rows[r].b.kind == NKO_SIDE_ARTIC)
            for (uint32_t i = 0u; i < t->max_dof; ++i) velocity += w->chain_jacobian_b[((size_t)env * R + r) * t->max_dof + i] * start[i];
        rows[r].rhs += w->row_reference_velocity_gain[(size_t)env * R + r] * velocity;
    }
}

/* ---- ReadoutContactWrench (ops/readout.cu:59-220, 559-626) ---------------
 * Per slot: first manifold point and normal, the summed {normal, tangent, tangent} force, each point's world impulse
 * (nk/contact/row_readout.hpp:17-48), the sides' owners, the contact's link.  Per link: the world wrench of the
 * active rows ending on it, added by ascending row then side A before B (contact_index.cuh:85-110 key order). */
void nko_env_readout_contact_wrench(nko_world* w, uint32_t env) {
    const nko_template* t = &w->t;
    const uint32_t S = t->slots, R = t->rows_per_env, nl = t->nl;
    const float dt = w->cfg.fixed_dt, inv_dt = dt > 0.0f ? 1.0f / dt : 0.0f;
    const nko_row* rows = (const nko_row*)w->urows;
    for (uint32_t s = 0u; s < S; ++s) {
        const size_t slot = (size_t)env * S + s;
        const uint32_t points = w->ucontact_count[slot];
        for (uint32_t k = 0u; k < 3u; ++k) {
            w->contact_point[slot * 3u + k] = points > 0u ? w->ucontact_point[slot * 12u + k] : 0.0f;
            w->contact_normal[slot * 3u + k] = points > 0u ? w->ucontact_normal[slot * 12u + k] : 0.0f;
        }
        const uint32_t first = w->ucontact_row_range[slot * 2u], pts = w->ucontact_row_range[slot * 2u + 1u];
        float fn = 0.0f, ft1 = 0.0f, ft2 = 0.0f;
        for (uint32_t i = 0u; i < pts; ++i) {
            fn += w->lambda[first + i]; ft1 += w->lambda[first + i + pts]; ft2 += w->lambda[first + i + 2u * pts];
        }
        for (uint32_t i = 0u; i < 4u; ++i) {
            v3 impulse = v3_make(0, 0, 0);
            if (i < pts && (rows[first + i].flags & NKO_ROW_ACTIVE) != 0u)
                for (uint32_t axis = 0u; axis < 3u; ++axis) {
                    const uint32_t index = first + i + axis * pts;
                    impulse = v3_add(impulse, v3_scale(rows[index].a.jlin, w->lambda[index]));
                }
            float* out = w->ucontact_impulse + (slot * 4u + i) * 3u;
            out[0] = impulse.x; out[1] = impulse.y; out[2] = impulse.z;
        }
        w->contact_force[slot * 3u] = fn * inv_dt; w->contact_force[slot * 3u + 1u] = ft1 * inv_dt; w->contact_force[slot * 3u + 2u] = ft2 * inv_dt;
        const int active = pts > 0u && (rows[first].flags & NKO_ROW_ACTIVE) != 0u;
        const uint32_t kind_a = active ? rows[first].a.kind : NKO_SIDE_STATIC, kind_b = active ? rows[first].b.kind : NKO_SIDE_STATIC;
        w->contact_side_a_kind[slot] = kind_a; w->contact_side_b_kind[slot] = kind_b;
        w->contact_side_a_index[slot] = !active || kind_a == NKO_SIDE_STATIC ? NKO_INVALID : kind_a == NKO_SIDE_ARTIC ? w->row_cj_link[first] : rows[first].a.index;
        w->contact_side_b_index[slot] = !active || kind_b == NKO_SIDE_STATIC ? NKO_INVALID : kind_b == NKO_SIDE_ARTIC ? w->row_cj_link_b[first] : rows[first].b.index;
        uint32_t link = NKO_INVALID;
        for (uint32_t i = 0u; i < pts && link == NKO_INVALID; ++i) link = w->row_cj_link[first + i];
        for (uint32_t i = 0u; i < pts && link == NKO_INVALID; ++i) link = w->row_cj_link_b[first + i];
        w->contact_link[slot] = link;
    }
    for (uint32_t l = 0u; l < nl; ++l) {
        const uint32_t link = env * nl + l;
        const v3 origin = v3_make(w->link_pose[(size_t)link * 7u], w->link_pose[(size_t)link * 7u + 1u], w->link_pose[(size_t)link * 7u + 2u]);
        v3 force = v3_make(0, 0, 0), torque = v3_make(0, 0, 0);
        for (uint32_t r = 0u; r < R; ++r) {
            const size_t rs = (size_t)env * R + r;
            if ((rows[rs].flags & NKO_ROW_ACTIVE) == 0u) continue;
            for (uint32_t side = 0u; side < 2u; ++side) {
                if ((side == 0u ? w->row_cj_link[rs] : w->row_cj_link_b[rs]) != link) continue;
                const v3 dir = side == 0u ? rows[rs].a.jlin : rows[rs].b.jlin;
                const float* point = (side == 0u ? w->row_cj_point : w->row_cj_point_b) + rs * 3u;
                const v3 f = v3_scale(dir, w->lambda[rs] * inv_dt);
                force = v3_add(force, f);
                torque = v3_add(torque, v3_cross(v3_sub(v3_make(point[0], point[1], point[2]), origin), f));
            }
        }
        float* out = w->link_contact_wrench + (size_t)link * 6u;
        out[0] = force.x; out[1] = force.y; out[2] = force.z; out[3] = torque.x; out[4] = torque.y; out[5] = torque.z;
    }
}
