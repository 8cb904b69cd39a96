// Contact detection and row assembly for gfx950: collidable poses, AABBs, candidate pairs in canonical (a, b)
// order, the analytic manifolds of sphere, capsule, box, plane and cylinder pairs, pair-driven contact rows and chain
// Jacobians.
//
// Elementwise stages run one thread per (env, item) on contiguous env-major fields; the stages with an order
// inside an environment (pair emission, row-range prefix, Jacobian rows) run one wavefront per environment so the
// order comes from lane ranks and prefix counts - no atomics, no sort, identical output every run.
//
// Replaces src/phi/backend_cuda/ops/sync_body_pose.cu, broadphase.cu (BuildAabbsKernel :173-270, EnvAllPairsKernel
// :408-474 plus the canonical radix sort :478-542, 630-680), narrowphase_prims.cu (PairDrivenNarrowphaseKernel<false>
// :181-366) and assemble_rows.cu (:122-214, 325-801, 1479-1605).
#include "nk_device_math.h"
#include "nk_body_pose.h"
#include "nk_ops.h"

namespace nkh {

namespace {

constexpr int kWave = 64;

struct ShapeRow { uint32_t kind; float p[4]; uint32_t contype, conaffinity; int32_t body_id; uint32_t group, profile; };

// prims_types.cuh:55-72
__device__ __forceinline__ ShapeRow load_shape(const float* table, uint32_t row) {
    const float* q = table + size_t{row} * kShapeStride;
    ShapeRow s;
    s.kind = __float_as_uint(q[0]);
    s.p[0] = q[1]; s.p[1] = q[2]; s.p[2] = q[3]; s.p[3] = q[4];
    s.contype = __float_as_uint(q[5]); s.conaffinity = __float_as_uint(q[6]);
    s.body_id = int32_t(__float_as_uint(q[8])); s.group = __float_as_uint(q[9]); s.profile = __float_as_uint(q[12]);
    return s;
}

// collision/contact_query.hpp:17-31
__device__ __forceinline__ float motion_radius(float base, float dt, float sa, float sb, float relax) {
    return base + dt * (sa + sb) * (2.0f / relax);
}

// ---- SyncLinkBodyPose (sync_body_pose.cu:23-83): link-owned rows only; static rows keep their cooked pose ----
__global__ void SyncLinkBodyPoseKernel(ModelView m, DataView d, uint32_t total_bodies) {
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total_bodies) return;
    const uint32_t env = gid / m.bodies_per_env;
    sync_body_pose(m, d, env, gid % m.bodies_per_env, d.link_pose + size_t{env} * m.links_per_env * 7u);
}

// broadphase.cu:154-170
__device__ V3 rot_abs(Q4 q, V3 v) {
    const V3 cx = rotate_raw(q, V3{1, 0, 0}), cy = rotate_raw(q, V3{0, 1, 0}), cz = rotate_raw(q, V3{0, 0, 1});
    return V3{fabsf(cx.x) * v.x + fabsf(cy.x) * v.y + fabsf(cz.x) * v.z, fabsf(cx.y) * v.x + fabsf(cy.y) * v.y + fabsf(cz.y) * v.z,
              fabsf(cx.z) * v.x + fabsf(cy.z) * v.y + fabsf(cz.z) * v.z};
}

// ---- BuildAabbs (broadphase.cu:173-270).  Link-owned collidables carry no body velocity on this path, so the
// motion term of the margin is zero; a free body's row carries the body's velocities. ----
__device__ __forceinline__ void build_aabb_of_body(const ModelView& m, const DataView& d, const BuildAabbsParams& p, uint32_t gid) {
    const uint32_t b = gid % p.bodies_per_env;
    const ShapeRow s = load_shape(m.shape_table, b);
    const Xf xf = load_xf(d.body_pose + size_t{gid} * 7u);
    float* lo = d.body_aabb_lo + size_t{gid} * 3u;
    float* hi = d.body_aabb_hi + size_t{gid} * 3u;
    V3 he{0, 0, 0};
    if (s.kind == kShapeSphere) he = V3{s.p[0], s.p[0], s.p[0]};
    else if (s.kind == kShapeCapsule) he = rot_abs(xf.r, V3{s.p[0], s.p[0], s.p[0] + s.p[1]});
    else if (s.kind == kShapeBox) he = rot_abs(xf.r, V3{s.p[0], s.p[1], s.p[2]});
    else if (s.kind == kShapeCylinder) {   // per world axis hh |a_i| + r sqrt(1 - a_i^2) for the cylinder's axis a
        const V3 qv{xf.r.x, xf.r.y, xf.r.z}, ez{0, 0, 1};
        const V3 tz = scale3(cross3(qv, ez), 2.0f);
        const V3 a = add3(add3(ez, scale3(tz, xf.r.w)), cross3(qv, tz));
        he = V3{s.p[1] * fabsf(a.x) + s.p[0] * sqrtf(fmaxf(0.0f, 1.0f - a.x * a.x)),
                s.p[1] * fabsf(a.y) + s.p[0] * sqrtf(fmaxf(0.0f, 1.0f - a.y * a.y)),
                s.p[1] * fabsf(a.z) + s.p[0] * sqrtf(fmaxf(0.0f, 1.0f - a.z * a.z))};
    } else if (s.kind == kShapePlane) {
        lo[0] = lo[1] = lo[2] = -FLT_MAX; hi[0] = hi[1] = hi[2] = FLT_MAX;
        return;
    } else {
        lo[0] = lo[1] = lo[2] = FLT_MAX; hi[0] = hi[1] = hi[2] = -FLT_MAX;
        return;
    }
    // (:262-264) a free body's own row moves with it - its speed, and its turning rate over the shape's radius
    float speed = 0.0f;
    if (m.free_body != 0u && b == m.link_body[0]) {
        const float* lv = d.body_linear_velocity + size_t{gid} * 3u, *av = d.body_angular_velocity + size_t{gid} * 3u;
        const float radius = sqrtf(he.x * he.x + he.y * he.y + he.z * he.z) + sqrtf(0.0f);
        speed = fmaxf(0.0f, sqrtf(lv[0] * lv[0] + lv[1] * lv[1] + lv[2] * lv[2]) + sqrtf(av[0] * av[0] + av[1] * av[1] + av[2] * av[2]) * radius);
    }
    const float mg = fmaxf(p.margin, fminf(motion_radius(p.margin, p.dt, speed, 0.0f, 0.9f), p.query_reach));
    const V3 c = xf.p;
    lo[0] = c.x - he.x - mg; lo[1] = c.y - he.y - mg; lo[2] = c.z - he.z - mg;
    hi[0] = c.x + he.x + mg; hi[1] = c.y + he.y + mg; hi[2] = c.z + he.z + mg;
}
__global__ void BuildAabbsKernel(ModelView m, DataView d, BuildAabbsParams p) {
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= p.env_count * p.bodies_per_env) return;
    build_aabb_of_body(m, d, p, gid);
}

// collision/shape_kind.hpp:26-33
__device__ __forceinline__ bool shape_filter_admits(uint32_t ta, uint32_t aa, uint32_t ga_, uint32_t tb, uint32_t ab, uint32_t gb_) {
    if (((ta & ab) | (tb & aa)) == 0u) return false;
    const int32_t ga = int32_t(ga_), gb = int32_t(gb_);
    return !(ga != 0 && gb != 0 && (ga > 0 ? (ga != gb && gb > 0) : ga == gb));
}

// broadphase.cu:87-99 IsExcluded: binary search of the sorted (a << 32 | b) keys, a < b
__device__ bool pair_excluded(const ModelView& m, uint32_t a, uint32_t b) {
    const uint64_t key = (uint64_t{a} << 32u) | uint64_t{b};
    uint32_t lo = 0u, hi = m.excluded_pair_count;
    while (lo < hi) {
        const uint32_t mid = lo + (hi - lo) / 2u;
        if (m.excluded_pairs[mid] < key) lo = mid + 1u; else hi = mid;
    }
    return lo < m.excluded_pair_count && m.excluded_pairs[lo] == key;
}

// ---- candidate pairs: one wavefront per env walks the (i, j) grid in row-major order; the ballot rank of an
// emitting lane is its slot, which is the ascending (a, b) order the reference reaches by sorting.  The grid runs over
// the rows that can pass the shape filter at all (a row with empty type and affinity masks pairs with nothing): a
// humanoid's 31 shapeless link rows leave a grid of 13 x 13 out of 44 x 44. ----
__device__ __forceinline__ void query_pairs_of_env(const ModelView& m, const DataView& d, const LbvhQueryPairsParams& p, uint32_t env,
                                                    uint32_t lane) {
    const uint32_t N = m.pairable_count;
    const size_t bbase = size_t{env} * p.bodies_per_env;
    const uint32_t capacity = min(p.rigid_slot_cap, p.max_pairs);
    uint32_t* pairs = d.candidate_pairs + size_t{env} * p.max_contacts_per_env * 2u;
    uint32_t count = 0u;
    bool overflow = false;
    for (uint32_t base = 0u; base < N * N; base += kWave) {
        const uint32_t item = base + lane, at_i = item / N, at_j = item % N;
        bool emit = false;
        uint32_t i = 0u, j = 0u;
        if (at_i < at_j && at_i < N) {
            i = m.pairable_rows[at_i]; j = m.pairable_rows[at_j];
            const float* alo = d.body_aabb_lo + (bbase + i) * 3u, *ahi = d.body_aabb_hi + (bbase + i) * 3u;
            const float* blo = d.body_aabb_lo + (bbase + j) * 3u, *bhi = d.body_aabb_hi + (bbase + j) * 3u;
            const bool overlap = !(ahi[0] < blo[0] || alo[0] > bhi[0] || ahi[1] < blo[1] || alo[1] > bhi[1] ||
                                   ahi[2] < blo[2] || alo[2] > bhi[2]);
            if (overlap) {
                const ShapeRow sa = load_shape(m.shape_table, i), sb = load_shape(m.shape_table, j);
                emit = !(sa.body_id < 0 && sb.body_id < 0) &&
                       shape_filter_admits(sa.contype, sa.conaffinity, sa.group, sb.contype, sb.conaffinity, sb.group) &&
                       !pair_excluded(m, i, j);
            }
        }
        const uint64_t mask = __ballot(emit);
        if (emit) {
            const uint32_t slot = count + __popcll(mask & ((uint64_t{1} << lane) - 1u));
            if (slot < capacity) { pairs[2u * slot] = i; pairs[2u * slot + 1u] = j; }
            else overflow = true;
        }
        count += __popcll(mask);
    }
    overflow = __any(overflow);
    if (lane == 0u) {
        d.pair_count[env] = min(count, capacity);
        const uint32_t status = d.env_status[env] & ~kEnvStatusPairOverflow;
        d.env_status[env] = overflow ? status | kEnvStatusPairOverflow : status;
    }
}
__global__ void __launch_bounds__(kWave) QueryPairsKernel(ModelView m, DataView d, LbvhQueryPairsParams p) {
    query_pairs_of_env(m, d, p, blockIdx.x, threadIdx.x);
}

// ---- manifolds (collision/analytical_manifold.hpp) ------------------------------------------------------
struct Prim { V3 cx, cy, cz, t; float radius, half_height; V3 half; };
struct Manifold { uint32_t count; V3 position[4]; V3 normal; float penetration[4]; uint32_t key[4]; };

__device__ Prim make_prim(const ShapeRow& s, Xf xf) {   // narrowphase_prims.cu:34-46
    Prim p;
    p.cx = rotate_raw(xf.r, V3{1, 0, 0}); p.cy = rotate_raw(xf.r, V3{0, 1, 0}); p.cz = rotate_raw(xf.r, V3{0, 0, 1});
    p.t = xf.p; p.radius = s.p[0]; p.half_height = s.p[1]; p.half = V3{s.p[0], s.p[1], s.p[2]};
    return p;
}
__device__ V3 norm_or(V3 v, V3 fallback) {   // analytical_manifold.hpp:194-198 Norm
    const float len = sqrtf(v.x * v.x + v.y * v.y + v.z * v.z);
    if (len < 1.0e-12f) return fallback;
    return V3{v.x / len, v.y / len, v.z / len};
}
// analytical_manifold.hpp:69-93 PrimFrame
__device__ V3 frame_local_to_world(const Prim& f, V3 l) {
    return V3{f.cx.x * l.x + f.cy.x * l.y + f.cz.x * l.z + f.t.x, f.cx.y * l.x + f.cy.y * l.y + f.cz.y * l.z + f.t.y,
              f.cx.z * l.x + f.cy.z * l.y + f.cz.z * l.z + f.t.z};
}
__device__ V3 frame_world_to_local(const Prim& f, V3 w) {
    const V3 d = sub3(w, f.t);
    return V3{dot3(d, f.cx), dot3(d, f.cy), dot3(d, f.cz)};
}
__device__ V3 frame_dir_to_world(const Prim& f, V3 l) {
    return V3{f.cx.x * l.x + f.cy.x * l.y + f.cz.x * l.z, f.cx.y * l.x + f.cy.y * l.y + f.cz.y * l.z,
              f.cx.z * l.x + f.cy.z * l.y + f.cz.z * l.z};
}

// analytical_manifold.hpp:273-311 ReduceAndEmit: the four deepest candidates (ties to the smaller feature id), emitted
// in ascending feature order
__device__ void reduce_and_emit(V3* position, float* pen, uint32_t* feature, int ncand, V3 n, Manifold* out) {
    out->count = 0u;
    if (ncand <= 0) return;
    const int keep = ncand < 4 ? ncand : 4;
    for (int s = 0; s < keep; ++s) {
        int best = s;
        for (int i = s + 1; i < ncand; ++i)
            if (pen[i] > pen[best] || (pen[i] == pen[best] && feature[i] < feature[best])) best = i;
        const V3 tp = position[s]; position[s] = position[best]; position[best] = tp;
        const float tf = pen[s]; pen[s] = pen[best]; pen[best] = tf;
        const uint32_t tk = feature[s]; feature[s] = feature[best]; feature[best] = tk;
    }
    for (int i = 1; i < keep; ++i) {
        const V3 kp = position[i]; const float kf = pen[i]; const uint32_t kk = feature[i];
        int j = i - 1;
        while (j >= 0 && feature[j] > kk) { position[j + 1] = position[j]; pen[j + 1] = pen[j]; feature[j + 1] = feature[j]; --j; }
        position[j + 1] = kp; pen[j + 1] = kf; feature[j + 1] = kk;
    }
    for (int i = 0; i < keep; ++i) { out->position[i] = position[i]; out->penetration[i] = pen[i]; out->key[i] = feature[i]; }
    out->normal = n;
    out->count = uint32_t(keep);
}

// analytical_manifold.hpp:337-405 ReduceAndEmitSpread: up to four candidates as they are; of more, the deepest and then,
// three times, the one farthest from those kept (ties to the lower index); ascending feature order
__device__ void reduce_and_emit_spread(const V3* position, const float* pen, const uint32_t* feature, int n, V3 normal, Manifold* out) {
    out->count = 0u;
    if (n <= 0) return;
    int kept[4] = {0, 1, 2, 3};
    int count = n;
    if (n > 4) {
        uint32_t used = 0u;
        int seed = 0;
        for (int i = 1; i < n; ++i) if (pen[i] > pen[seed]) seed = i;
        kept[0] = seed; used |= 1u << seed;
        for (int s = 1; s < 4; ++s) {
            int best = -1; float best_mind = -1.0f;
            for (int i = 0; i < n; ++i) {
                if ((used >> i) & 1u) continue;
                float mind = 3.4e38f;
                for (int t = 0; t < s; ++t) {
                    const V3 d = sub3(position[i], position[kept[t]]);
                    const float dd = dot3(d, d);
                    if (dd < mind) mind = dd;
                }
                if (mind > best_mind) { best_mind = mind; best = i; }
            }
            kept[s] = best; used |= 1u << best;   // more than four candidates: every round finds one
        }
        count = 4;
    }
    for (int i = 1; i < count; ++i) {
        const int key = kept[i]; int j = i - 1;
        while (j >= 0 && feature[kept[j]] > feature[key]) { kept[j + 1] = kept[j]; --j; }
        kept[j + 1] = key;
    }
    for (int i = 0; i < count; ++i) { out->position[i] = position[kept[i]]; out->penetration[i] = pen[kept[i]]; out->key[i] = feature[kept[i]]; }
    out->normal = normal;
    out->count = uint32_t(count);
}

// collision/primitive_surface.hpp:28-122 QueryPrimitiveSurface: signed distance (positive outside), outward normal,
// closest surface point and feature of a point in the primitive's own frame
struct Surface { float distance; V3 normal, point; uint32_t feature; bool valid; };
__device__ __forceinline__ Surface query_surface(uint32_t kind, V3 par, V3 pos) {
    Surface r{0.0f, V3{1, 0, 0}, V3{0, 0, 0}, 0u, false};
    if (kind == kShapeSphere || kind == kShapeCapsule) {
        if (!(par.x >= 0.0f)) return r;
        V3 offset = pos;
        if (kind == kShapeCapsule) {
            if (!(par.y >= 0.0f)) return r;
            offset.z -= fmaxf(-par.y, fminf(pos.z, par.y));
            r.feature = pos.z < -par.y ? 0u : pos.z > par.y ? 2u : 1u;
        }
        const float length = sqrtf(dot3(offset, offset));
        if (length > 0.0f) r.normal = V3{offset.x / length, offset.y / length, offset.z / length};
        r.distance = length - par.x;
    } else if (kind == kShapeBox) {
        if (!(par.x >= 0.0f && par.y >= 0.0f && par.z >= 0.0f)) return r;
        const V3 closest{fmaxf(-par.x, fminf(pos.x, par.x)), fmaxf(-par.y, fminf(pos.y, par.y)), fmaxf(-par.z, fminf(pos.z, par.z))};
        const V3 offset = sub3(pos, closest);
        const float length = sqrtf(dot3(offset, offset));
        if (length > 0.0f) {
            r.distance = length;
            r.normal = V3{offset.x / length, offset.y / length, offset.z / length};
            if (offset.x != 0.0f) r.feature |= 1u << (pos.x < 0.0f ? 0u : 1u);
            if (offset.y != 0.0f) r.feature |= 1u << (pos.y < 0.0f ? 2u : 3u);
            if (offset.z != 0.0f) r.feature |= 1u << (pos.z < 0.0f ? 4u : 5u);
        } else {
            const V3 dist{fabsf(pos.x) - par.x, fabsf(pos.y) - par.y, fabsf(pos.z) - par.z};
            if (dist.x >= dist.y && dist.x >= dist.z) {
                r.distance = dist.x; r.normal = V3{pos.x < 0.0f ? -1.0f : 1.0f, 0, 0}; r.feature = 1u << (pos.x < 0.0f ? 0u : 1u);
            } else if (dist.y >= dist.z) {
                r.distance = dist.y; r.normal = V3{0, pos.y < 0.0f ? -1.0f : 1.0f, 0}; r.feature = 1u << (pos.y < 0.0f ? 2u : 3u);
            } else {
                r.distance = dist.z; r.normal = V3{0, 0, pos.z < 0.0f ? -1.0f : 1.0f}; r.feature = 1u << (pos.z < 0.0f ? 4u : 5u);
            }
        }
    } else if (kind == kShapeCylinder) {   // features: 0 bottom cap, 1 side, 2 top cap, 3 bottom rim, 4 top rim
        if (!(par.x >= 0.0f && par.y >= 0.0f)) return r;
        const float rho = sqrtf(pos.x * pos.x + pos.y * pos.y);
        const V3 radial = rho > 0.0f ? V3{pos.x / rho, pos.y / rho, 0.0f} : V3{1, 0, 0};
        const V3 axial{0, 0, pos.z < 0.0f ? -1.0f : 1.0f};
        const float side = rho - par.x, cap = fabsf(pos.z) - par.y;
        if (side > 0.0f && cap > 0.0f) {
            r.distance = sqrtf(side * side + cap * cap);
            const V3 sum = add3(scale3(radial, side), scale3(axial, cap));
            r.normal = V3{sum.x / r.distance, sum.y / r.distance, sum.z / r.distance};
            r.feature = pos.z < 0.0f ? 3u : 4u;
        } else if (side > cap) {
            r.distance = side; r.normal = radial; r.feature = 1u;
        } else {
            r.distance = cap; r.normal = axial; r.feature = pos.z < 0.0f ? 0u : 2u;
        }
    } else return r;
    r.point = sub3(pos, scale3(r.normal, r.distance));
    r.valid = true;
    return r;
}

__device__ __forceinline__ void emit_one(Manifold* out, V3 position, V3 normal, float pen, uint32_t key) {
    out->position[0] = position; out->normal = normal; out->penetration[0] = pen; out->key[0] = key; out->count = 1u;
}
__device__ __forceinline__ void sphere_sphere(const Prim& a, const Prim& b, float query, Manifold* out) {   // :416-429
    out->count = 0u;
    const V3 delta = sub3(a.t, b.t);
    const float dist = sqrtf(delta.x * delta.x + delta.y * delta.y + delta.z * delta.z);
    const float pen = (a.radius + b.radius) - dist;
    if (pen <= -query) return;
    const V3 n = norm_or(delta, V3{0, 1, 0});
    emit_one(out, add3(b.t, scale3(n, b.radius - 0.5f * pen)), n, pen, 0u);
}
__device__ __forceinline__ void sphere_box(const Prim& sph, const Prim& box, float query, Manifold* out) {   // :434-448
    out->count = 0u;
    const Surface s = query_surface(kShapeBox, box.half, frame_world_to_local(box, sph.t));
    if (!s.valid) return;
    const float pen = sph.radius - s.distance;
    if (pen <= -query) return;
    const V3 normal = frame_dir_to_world(box, s.normal);
    emit_one(out, sub3(frame_local_to_world(box, s.point), scale3(normal, 0.5f * pen)), normal, pen, 0u);
}
__device__ __forceinline__ void sphere_plane(const Prim& sph, const Prim& plane, float query, Manifold* out) {   // :451-463
    out->count = 0u;
    const V3 n = norm_or(plane.cz, V3{0, 0, 1});
    const float signed_dist = dot3(sub3(sph.t, plane.t), n);
    const float pen = sph.radius - signed_dist;
    if (pen <= -query) return;
    emit_one(out, sub3(sph.t, scale3(n, sph.radius - 0.5f * pen)), n, pen, 0u);
}
__device__ void box_plane(const Prim& box, const Prim& plane, float query, Manifold* out) {   // :469-493
    out->count = 0u;
    const V3 n = norm_or(plane.cz, V3{0, 0, 1});
    V3 position[8]; float pen[8]; uint32_t feature[8];
    int ncand = 0;
    for (uint32_t c = 0u; c < 8u; ++c) {
        const float sx = (c & 1u) ? 1.0f : -1.0f, sy = (c & 2u) ? 1.0f : -1.0f, sz = (c & 4u) ? 1.0f : -1.0f;
        const V3 corner = frame_local_to_world(box, V3{sx * box.half.x, sy * box.half.y, sz * box.half.z});
        const float sd = dot3(sub3(corner, plane.t), n);
        if (sd < query) {
            position[ncand] = sub3(corner, scale3(n, 0.5f * sd));
            pen[ncand] = -sd; feature[ncand] = c; ++ncand;
        }
    }
    reduce_and_emit(position, pen, feature, ncand, n, out);
}
__device__ void capsule_plane(const Prim& cap, const Prim& plane, float query, Manifold* out) {   // :738-759
    out->count = 0u;
    const V3 n = norm_or(plane.cz, V3{0, 0, 1});
    const V3 ends[2] = {add3(cap.t, scale3(cap.cz, cap.half_height)), sub3(cap.t, scale3(cap.cz, cap.half_height))};
    V3 position[2]; float pen[2]; uint32_t feature[2];
    int ncand = 0;
    for (uint32_t k = 0u; k < 2u; ++k) {
        const float sd = dot3(sub3(ends[k], plane.t), n) - cap.radius;
        if (sd < query) {
            position[ncand] = sub3(ends[k], scale3(n, cap.radius + 0.5f * sd));
            pen[ncand] = -sd; feature[ncand] = k; ++ncand;
        }
    }
    reduce_and_emit(position, pen, feature, ncand, n, out);
}
__device__ __forceinline__ void capsule_sphere(const Prim& cap, const Prim& sph, float query, Manifold* out) {   // :764-778
    out->count = 0u;
    const Surface s = query_surface(kShapeCapsule, V3{cap.radius, cap.half_height, 0.0f}, frame_world_to_local(cap, sph.t));
    if (!s.valid) return;
    const float pen = sph.radius - s.distance;
    if (pen <= -query) return;
    const V3 normal = scale3(frame_dir_to_world(cap, s.normal), -1.0f);
    emit_one(out, add3(frame_local_to_world(cap, s.point), scale3(normal, 0.5f * pen)), normal, pen, 0u);
}
// :780-815: the lower cap's octagon and deepest point when a cap faces the plane, else each cap's deepest point
__device__ void cylinder_plane(const Prim& cyl, const Prim& plane, float query, Manifold* out) {
    out->count = 0u;
    constexpr float kS = 0.70710678f;
    const float rc[8] = {1.0f, kS, 0.0f, -kS, -1.0f, -kS, 0.0f, kS};
    const float rs[8] = {0.0f, kS, 1.0f, kS, 0.0f, -kS, -1.0f, -kS};
    const V3 n = norm_or(plane.cz, V3{0, 0, 1});
    const V3 axis = cyl.cz;
    const float d = dot3(axis, n);
    const bool on_cap = fabsf(d) >= 0.95f;
    const V3 down = norm_or(sub3(scale3(axis, d), n), cyl.cx);
    V3 position[10]; float pen[10]; uint32_t feature[10];
    int ncand = 0;
    for (int cap = 0; cap < 2; ++cap) {
        if (on_cap && (cap == 0) == (d > 0.0f)) continue;
        const V3 center = add3(cyl.t, scale3(axis, cap == 0 ? cyl.half_height : -cyl.half_height));
        for (int k = -1; k < (on_cap ? 8 : 0); ++k) {
            const V3 dir = k < 0 ? down : add3(scale3(cyl.cx, rc[k]), scale3(cyl.cy, rs[k]));
            const V3 p = add3(center, scale3(dir, cyl.radius));
            const float sd = dot3(sub3(p, plane.t), n);
            if (sd >= query) continue;
            position[ncand] = sub3(p, scale3(n, sd * 0.5f));
            pen[ncand] = -sd;
            feature[ncand] = uint32_t(k < 0 ? cap : 2 + cap * 8 + k);
            ++ncand;
        }
    }
    reduce_and_emit_spread(position, pen, feature, ncand, n, out);
}
__device__ __forceinline__ void cylinder_sphere(const Prim& cyl, const Prim& sph, float query, Manifold* out) {   // :819-834
    out->count = 0u;
    const Surface s = query_surface(kShapeCylinder, V3{cyl.radius, cyl.half_height, 0.0f}, frame_world_to_local(cyl, sph.t));
    if (!s.valid) return;
    const float pen = sph.radius - s.distance;
    if (pen <= -query) return;
    const V3 normal = scale3(frame_dir_to_world(cyl, s.normal), -1.0f);
    emit_one(out, add3(frame_local_to_world(cyl, s.point), scale3(normal, 0.5f * pen)), normal, pen, s.feature);
}
// :841-896 ClosestPtSegmentSegment (fixed branch order)
__device__ __forceinline__ float clamp01(float v) { return v < 0.0f ? 0.0f : (v > 1.0f ? 1.0f : v); }
__device__ __forceinline__ float closest_segment_segment(V3 p1, V3 q1, V3 p2, V3 q2, V3* c1_out, V3* c2_out) {
    const V3 d1 = sub3(q1, p1), d2 = sub3(q2, p2), r = sub3(p1, p2);
    const float a = dot3(d1, d1), e = dot3(d2, d2), f = dot3(d2, r);
    float s = 0.0f, t = 0.0f;
    const float eps = 1.0e-12f;
    if (a <= eps && e <= eps) { s = 0.0f; t = 0.0f; }
    else if (a <= eps) { s = 0.0f; t = clamp01(f / e); }
    else {
        const float c = dot3(d1, r);
        if (e <= eps) { t = 0.0f; s = clamp01(-c / a); }
        else {
            const float b = dot3(d1, d2);
            const float denom = a * e - b * b;
            s = denom > eps ? clamp01((b * f - c * e) / denom) : 0.0f;
            t = (b * s + f) / e;
            if (t < 0.0f) { t = 0.0f; s = clamp01(-c / a); }
            else if (t > 1.0f) { t = 1.0f; s = clamp01((b - c) / a); }
        }
    }
    const V3 c1 = add3(p1, scale3(d1, s)), c2 = add3(p2, scale3(d2, t));
    *c1_out = c1; *c2_out = c2;
    const V3 dv = sub3(c1, c2);
    return dot3(dv, dv);
}
__device__ __forceinline__ void capsule_capsule(const Prim& a, const Prim& b, float query, Manifold* out) {   // :905-932
    out->count = 0u;
    const V3 a0 = add3(a.t, scale3(a.cz, a.half_height)), a1 = sub3(a.t, scale3(a.cz, a.half_height));
    const V3 b0 = add3(b.t, scale3(b.cz, b.half_height)), b1 = sub3(b.t, scale3(b.cz, b.half_height));
    V3 ca, cb;
    const float dist = sqrtf(closest_segment_segment(a0, a1, b0, b1, &ca, &cb));
    const float pen = (a.radius + b.radius) - dist;
    if (pen <= -query) return;
    const V3 n = norm_or(sub3(ca, cb), norm_or(cross3(a.cz, b.cz), V3{0, 1, 0}));
    const V3 sa = sub3(ca, scale3(n, a.radius)), sb = add3(cb, scale3(n, b.radius));
    emit_one(out, scale3(add3(sa, sb), 0.5f), n, pen, 0u);
}
// :224-260 ClipAgainstPlane: Sutherland-Hodgman against one half-space, edges in fixed order; an intersection
// inherits the feature of the edge's first vertex
struct ClipPoly { V3 v[8]; uint32_t feat[8]; int count; };
__device__ __forceinline__ void clip_add(ClipPoly* p, V3 v, uint32_t f) { if (p->count < 8) { p->v[p->count] = v; p->feat[p->count] = f; ++p->count; } }
__device__ void clip_against_plane(const ClipPoly& in, V3 plane_pt, V3 plane_n, ClipPoly* out) {
    out->count = 0;
    for (int i = 0; i < in.count; ++i) {
        const int j = i + 1 == in.count ? 0 : i + 1;
        const V3 cur = in.v[i], nxt = in.v[j];
        const float dc = dot3(sub3(cur, plane_pt), plane_n), dn = dot3(sub3(nxt, plane_pt), plane_n);
        const bool cur_in = dc <= 0.0f, nxt_in = dn <= 0.0f;
        if (cur_in) clip_add(out, cur, in.feat[i]);
        if (cur_in != nxt_in) {
            const float t = dc / (dc - dn);
            clip_add(out, V3{cur.x + (nxt.x - cur.x) * t, cur.y + (nxt.y - cur.y) * t, cur.z + (nxt.z - cur.z) * t}, in.feat[i]);
        }
    }
}
__device__ __forceinline__ V3 neg3(V3 a) { return V3{-a.x, -a.y, -a.z}; }
__device__ __forceinline__ float comp3(V3 v, int k) { return k == 0 ? v.x : (k == 1 ? v.y : v.z); }
__device__ __forceinline__ V3 axis3(const Prim& f, int k) { return k == 0 ? f.cx : (k == 1 ? f.cy : f.cz); }

// :503-736 BoxBox: the axis of least penetration among the 15 separating-axis candidates in fixed order (faces preferred
// by a 1e-5 bias); an edge pair gives one point between the closest edge points, a face gives the incident face clipped
// against the reference face's sides, reduced by ReduceAndEmitSpread
__device__ void box_box(const Prim& A, const Prim& B, float query, Manifold* out) {
    out->count = 0u;
    const V3 dpos = sub3(B.t, A.t);
    float AbsR[3][3];
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) AbsR[i][j] = fabsf(dot3(axis3(A, i), axis3(B, j))) + 1.0e-6f;
    const float ea[3] = {A.half.x, A.half.y, A.half.z}, eb[3] = {B.half.x, B.half.y, B.half.z};
    float min_pen = 3.4e38f;
    int best_axis = -1;
    V3 best_n{0, 1, 0};
    const float bias = 1.0e-5f;
    for (int i = 0; i < 3; ++i) {
        const float d = dot3(dpos, axis3(A, i));
        const float pen = (ea[i] + (eb[0] * AbsR[i][0] + eb[1] * AbsR[i][1] + eb[2] * AbsR[i][2])) - fabsf(d);
        if (pen <= -query) return;
        if (pen < min_pen - bias) { min_pen = pen; best_axis = i; best_n = d < 0.0f ? neg3(axis3(A, i)) : axis3(A, i); }
    }
    for (int j = 0; j < 3; ++j) {
        const float d = dot3(dpos, axis3(B, j));
        const float pen = ((ea[0] * AbsR[0][j] + ea[1] * AbsR[1][j] + ea[2] * AbsR[2][j]) + eb[j]) - fabsf(d);
        if (pen <= -query) return;
        if (pen < min_pen - bias) { min_pen = pen; best_axis = 3 + j; best_n = d < 0.0f ? neg3(axis3(B, j)) : axis3(B, j); }
    }
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) {
            V3 L = cross3(axis3(A, i), axis3(B, j));
            const float Llen = sqrtf(L.x * L.x + L.y * L.y + L.z * L.z);
            if (Llen < 1.0e-6f) continue;
            L = V3{L.x / Llen, L.y / Llen, L.z / Llen};
            const float ra = ea[0] * fabsf(dot3(A.cx, L)) + ea[1] * fabsf(dot3(A.cy, L)) + ea[2] * fabsf(dot3(A.cz, L));
            const float rb = eb[0] * fabsf(dot3(B.cx, L)) + eb[1] * fabsf(dot3(B.cy, L)) + eb[2] * fabsf(dot3(B.cz, L));
            const float s = dot3(dpos, L);
            const float pen = (ra + rb) - fabsf(s);
            if (pen <= -query) return;
            if (pen < min_pen - bias) { min_pen = pen; best_axis = 6 + i * 3 + j; best_n = s < 0.0f ? neg3(L) : L; }
        }
    if (best_axis < 0) return;
    if (best_axis >= 6) {   // edge against edge: one point between the closest points of the two edges
        const int i = (best_axis - 6) / 3, j = (best_axis - 6) % 3;
        V3 pa = A.t, pb = B.t;
        for (int k = 0; k < 3; ++k) {
            if (k != i) pa = add3(pa, scale3(axis3(A, k), (dot3(axis3(A, k), best_n) >= 0.0f ? 1.0f : -1.0f) * ea[k]));
            if (k != j) pb = add3(pb, scale3(axis3(B, k), (dot3(axis3(B, k), best_n) >= 0.0f ? -1.0f : 1.0f) * eb[k]));
        }
        const V3 da = axis3(A, i), db = axis3(B, j), r = sub3(pa, pb);
        const float bb = dot3(da, db), dd = dot3(da, r), ee = dot3(db, r);
        const float denom = 1.0f - bb * bb;
        float sN = 0.0f, tN = 0.0f;
        if (denom > 1.0e-9f) { sN = (bb * ee - dd) / denom; tN = (ee - bb * dd) / denom; }
        const float sCl = fminf(fmaxf(sN, -ea[i]), ea[i]), tCl = fminf(fmaxf(tN, -eb[j]), eb[j]);
        const V3 ca = add3(pa, scale3(da, sCl)), cb = add3(pb, scale3(db, tCl));
        emit_one(out, scale3(add3(ca, cb), 0.5f), best_n, min_pen, 0xE0000000u | (uint32_t(i) << 4) | uint32_t(j));
        return;
    }
    const bool ref_is_A = best_axis < 3;
    const int ref_axis = ref_is_A ? best_axis : best_axis - 3;
    const Prim& Rf = ref_is_A ? A : B;
    const Prim& If = ref_is_A ? B : A;
    V3 refN = axis3(Rf, ref_axis);
    if (dot3(sub3(If.t, Rf.t), refN) < 0.0f) refN = neg3(refN);
    int inc_axis = 0; float best_dot = 3.4e38f, inc_sign = 1.0f;
    for (int k = 0; k < 3; ++k) {
        const float d = dot3(axis3(If, k), refN);
        if (-fabsf(d) < best_dot) { best_dot = -fabsf(d); inc_axis = k; inc_sign = d < 0.0f ? 1.0f : -1.0f; }
    }
    const int iu = (inc_axis + 1) % 3, iv = (inc_axis + 2) % 3;
    const V3 inc_face_center = add3(If.t, scale3(axis3(If, inc_axis), inc_sign * comp3(If.half, inc_axis)));
    const V3 iu_w = axis3(If, iu), iv_w = axis3(If, iv);
    const float iu_e = comp3(If.half, iu), iv_e = comp3(If.half, iv);
    ClipPoly poly, next;
    poly.count = 0;
    for (uint32_t k = 0u; k < 4u; ++k) {
        const float su = (k == 1u || k == 2u) ? 1.0f : -1.0f, sv = k >= 2u ? 1.0f : -1.0f;
        clip_add(&poly, add3(add3(inc_face_center, scale3(iu_w, su * iu_e)), scale3(iv_w, sv * iv_e)), (uint32_t(inc_axis) << 4) | k);
    }
    const int ru = (ref_axis + 1) % 3, rv = (ref_axis + 2) % 3;
    const V3 ru_w = axis3(Rf, ru), rv_w = axis3(Rf, rv);
    const float ru_e = comp3(Rf.half, ru), rv_e = comp3(Rf.half, rv);
    const V3 ref_face_center = add3(Rf.t, scale3(refN, comp3(Rf.half, ref_axis)));
    clip_against_plane(poly, add3(ref_face_center, scale3(ru_w, ru_e)), ru_w, &next);
    clip_against_plane(next, sub3(ref_face_center, scale3(ru_w, ru_e)), neg3(ru_w), &poly);
    clip_against_plane(poly, add3(ref_face_center, scale3(rv_w, rv_e)), rv_w, &next);
    clip_against_plane(next, sub3(ref_face_center, scale3(rv_w, rv_e)), neg3(rv_w), &poly);
    V3 position[8]; float pen[8]; uint32_t feature[8];
    int ncand = 0;
    for (int k = 0; k < poly.count; ++k) {
        const float depth = dot3(sub3(ref_face_center, poly.v[k]), refN);
        if (depth >= -query) {
            const V3 onref = add3(poly.v[k], scale3(refN, depth));
            position[ncand] = scale3(add3(poly.v[k], onref), 0.5f);
            pen[ncand] = depth; feature[ncand] = uint32_t(k); ++ncand;
        }
    }
    const V3 normalA = ref_is_A ? neg3(refN) : refN;
    if (ncand == 0) {
        emit_one(out, add3(inc_face_center, scale3(refN, min_pen * 0.5f)), normalA, min_pen, uint32_t(inc_axis) << 4);
        return;
    }
    reduce_and_emit_spread(position, pen, feature, ncand, normalA, out);
}
// :934-971 PrimitivePair; a flipped pair negates the normal
__device__ void primitive_pair(uint32_t ka, const Prim& a, uint32_t kb, const Prim& b, float query, Manifold* out) {
    out->count = 0u;
    if (ka == kShapeSphere && kb == kShapeSphere) { sphere_sphere(a, b, query, out); return; }
    if (ka == kShapeSphere && kb == kShapeBox) { sphere_box(a, b, query, out); return; }
    if (ka == kShapeSphere && kb == kShapePlane) { sphere_plane(a, b, query, out); return; }
    if (ka == kShapeBox && kb == kShapePlane) { box_plane(a, b, query, out); return; }
    if (ka == kShapeBox && kb == kShapeBox) { box_box(a, b, query, out); return; }
    if (ka == kShapeCapsule && kb == kShapePlane) { capsule_plane(a, b, query, out); return; }
    if (ka == kShapeCapsule && kb == kShapeSphere) { capsule_sphere(a, b, query, out); return; }
    if (ka == kShapeCapsule && kb == kShapeCapsule) { capsule_capsule(a, b, query, out); return; }
    if (ka == kShapeCylinder && kb == kShapePlane) { cylinder_plane(a, b, query, out); return; }
    if (ka == kShapeCylinder && kb == kShapeSphere) { cylinder_sphere(a, b, query, out); return; }
    if (ka == kShapeBox && kb == kShapeSphere) sphere_box(b, a, query, out);
    else if (ka == kShapePlane && kb == kShapeSphere) sphere_plane(b, a, query, out);
    else if (ka == kShapePlane && kb == kShapeBox) box_plane(b, a, query, out);
    else if (ka == kShapePlane && kb == kShapeCapsule) capsule_plane(b, a, query, out);
    else if (ka == kShapeSphere && kb == kShapeCapsule) capsule_sphere(b, a, query, out);
    else if (ka == kShapePlane && kb == kShapeCylinder) cylinder_plane(b, a, query, out);
    else if (ka == kShapeSphere && kb == kShapeCylinder) cylinder_sphere(b, a, query, out);
    out->normal = V3{-out->normal.x, -out->normal.y, -out->normal.z};
}

// The pairs whose manifold is one point at most: a sphere against anything, capsule against capsule.  A world whose
// admitted pairs are all of these (ModelView::max_points_per_slot == 1) runs the narrowphase on this dispatch alone:
// nothing in it indexes a local array by a run-time value, so the manifold stays in registers and the kernel takes no
// scratch memory (the general dispatch clips polygons and reduces candidate lists in local arrays).
__device__ __forceinline__ void primitive_pair_single(uint32_t ka, const Prim& a, uint32_t kb, const Prim& b, float query, Manifold* out) {
    out->count = 0u;
    if (ka == kShapeSphere && kb == kShapeSphere) { sphere_sphere(a, b, query, out); return; }
    if (ka == kShapeSphere && kb == kShapeBox) { sphere_box(a, b, query, out); return; }
    if (ka == kShapeSphere && kb == kShapePlane) { sphere_plane(a, b, query, out); return; }
    if (ka == kShapeCapsule && kb == kShapeSphere) { capsule_sphere(a, b, query, out); return; }
    if (ka == kShapeCapsule && kb == kShapeCapsule) { capsule_capsule(a, b, query, out); return; }
    if (ka == kShapeCylinder && kb == kShapeSphere) { cylinder_sphere(a, b, query, out); return; }
    if (ka == kShapeBox && kb == kShapeSphere) sphere_box(b, a, query, out);
    else if (ka == kShapePlane && kb == kShapeSphere) sphere_plane(b, a, query, out);
    else if (ka == kShapeSphere && kb == kShapeCapsule) capsule_sphere(b, a, query, out);
    else if (ka == kShapeSphere && kb == kShapeCylinder) cylinder_sphere(b, a, query, out);
    out->normal = V3{-out->normal.x, -out->normal.y, -out->normal.z};
}

// nk/contact/contact_identity.hpp:98-157
__device__ __forceinline__ int32_t quantize_coord(float value) {
    const float scaled = value * 4096.0f;
    return int32_t(scaled >= 0.0f ? scaled + 0.5f : scaled - 0.5f);
}
__device__ __forceinline__ uint64_t hash_word(uint64_t hash, uint64_t word) { hash ^= word; return hash * 1099511628211ull; }
__device__ uint64_t feature_token(uint32_t feature, V3 p) {
    if (feature != 0xffffffffu) return 0x8000000000000000ull | uint64_t{feature};
    uint64_t h = 1469598103934665603ull;
    h = hash_word(h, uint32_t(quantize_coord(p.x))); h = hash_word(h, uint32_t(quantize_coord(p.y)));
    h = hash_word(h, uint32_t(quantize_coord(p.z)));
    return h & 0x7fffffffffffffffull;
}
__device__ V3 inverse_transform_point(Xf xf, V3 wp) {   // prims_types.cuh:98-105
    const V3 v = sub3(wp, xf.p);
    const V3 qv{-xf.r.x, -xf.r.y, -xf.r.z};
    const V3 t = scale3(cross3(qv, v), 2.0f);
    return add3(add3(v, scale3(t, xf.r.w)), cross3(qv, t));
}

// ---- NarrowphasePrimitives: one thread per (env, slot) (narrowphase_prims.cu:181-366, analytic route) ----
template <bool kSinglePoint>
__device__ __forceinline__ uint32_t NarrowphaseSlot(const ModelView& m, const DataView& d, const NarrowphasePrimitivesParams& p, uint32_t env,
                                                    uint32_t slot) {
    constexpr uint32_t kPoints = kSinglePoint ? 1u : 4u;
    const size_t gid = size_t{env} * p.union_slot_count + slot;
    const size_t bbase = size_t{env} * p.bodies_per_env;
    const float separation = fmaxf(p.contact_margin, 0.0005f);
    const uint32_t live = d.pair_count[env];
    Manifold mf; mf.count = 0u; mf.normal = V3{0, 0, 1};
    uint32_t a = 0u, b = 0u, law = kContactLawSpeculative;
    Xf xa{}, xb{};
    if (slot < live) {
        a = d.candidate_pairs[gid * 2u]; b = d.candidate_pairs[gid * 2u + 1u];
        const ShapeRow sa = load_shape(m.shape_table, a), sb = load_shape(m.shape_table, b);
        xa = load_xf(d.body_pose + (bbase + a) * 7u); xb = load_xf(d.body_pose + (bbase + b) * 7u);
        const Prim pa = make_prim(sa, xa), pb = make_prim(sb, xb);
        // a MuJoCo-sourced profile on either side makes the contact compliant; its query band is the profiles' margin
        // and gap, and its depth stays the geometric one (narrowphase_prims.cu:232, 268-281, 295-296)
        const bool has_a = sa.profile < m.profile_count, has_b = sb.profile < m.profile_count;
        float query_margin = separation;
        if ((has_a && m.profile_law[sa.profile] == 1u) || (has_b && m.profile_law[sb.profile] == 1u)) {
            law = kContactLawCompliant;
            const float margin_a = has_a ? m.profile_margin[2u * sa.profile] + m.profile_margin[2u * sa.profile + 1u] : 0.0f;
            const float margin_b = has_b ? m.profile_margin[2u * sb.profile] + m.profile_margin[2u * sb.profile + 1u] : 0.0f;
            query_margin = margin_a + margin_b;
        }
        // (:236-250) the gap both sides can close within the step: link-owned rows carry no body velocity, a free body's own
        // row moves with it
        float speeds[2] = {0.0f, 0.0f};
        if (m.free_body != 0u) {
            const uint32_t ends[2] = {a, b};
            for (uint32_t side = 0u; side < 2u; ++side) {
                if (ends[side] != m.link_body[0]) continue;
                const size_t at = bbase + ends[side];
                const float* center = d.body_pose + at * 7u, *lo = d.body_aabb_lo + at * 3u, *hi = d.body_aabb_hi + at * 3u;
                const V3 extent{fmaxf(fabsf(lo[0] - center[0]), fabsf(hi[0] - center[0])), fmaxf(fabsf(lo[1] - center[1]), fabsf(hi[1] - center[1])),
                                fmaxf(fabsf(lo[2] - center[2]), fabsf(hi[2] - center[2]))};
                const float* lv = d.body_linear_velocity + at * 3u, *av = d.body_angular_velocity + at * 3u;
                speeds[side] = fmaxf(0.0f, sqrtf(lv[0] * lv[0] + lv[1] * lv[1] + lv[2] * lv[2]) +
                                           sqrtf((av[0] * av[0] + av[1] * av[1] + av[2] * av[2]) * (extent.x * extent.x + extent.y * extent.y + extent.z * extent.z)));
            }
        }
        const float query = fmaxf(query_margin, fminf(motion_radius(2.0f * separation, p.dt, speeds[0], speeds[1], 0.9f), p.query_reach));
        if constexpr (kSinglePoint) primitive_pair_single(sa.kind, pa, sb.kind, pb, query, &mf);
        else primitive_pair(sa.kind, pa, sb.kind, pb, query, &mf);
        if (law != kContactLawCompliant) {
#pragma unroll
            for (uint32_t i = 0u; i < kPoints; ++i) if (i < mf.count) mf.penetration[i] += separation;
        }
    }
    d.ucontact_count[gid] = mf.count;
    d.ucontact_law[gid] = law;
#pragma unroll
    for (uint32_t i = 0u; i < kPoints; ++i) {
        if (i >= mf.count) break;
        const size_t at = gid * 4u + i;
        d.ucontact_point[3u * at] = mf.position[i].x; d.ucontact_point[3u * at + 1u] = mf.position[i].y; d.ucontact_point[3u * at + 2u] = mf.position[i].z;
        d.ucontact_normal[3u * at] = mf.normal.x; d.ucontact_normal[3u * at + 1u] = mf.normal.y; d.ucontact_normal[3u * at + 2u] = mf.normal.z;
        d.ucontact_depth[at] = mf.penetration[i];
        d.ucontact_a[at] = a; d.ucontact_b[at] = b;
        const uint32_t feature = mf.key[i] == 0u ? 0xffffffffu : mf.key[i];
        uint64_t h = 1469598103934665603ull;
        h = hash_word(h, feature_token(feature, inverse_transform_point(xa, mf.position[i])));
        h = hash_word(h, feature_token(feature, inverse_transform_point(xb, mf.position[i])));
        h = hash_word(h, i); h = hash_word(h, 0u); h = hash_word(h, 0u);
        d.ucontact_id_pair[at] = (uint64_t{a & 0x0fffffffu} << 32u) | uint64_t{b & 0x0fffffffu};
        d.ucontact_id_feature[at] = h;
    }
    return mf.count;
}

// One wavefront per environment; its lanes take the environment's slots in strides of 64, and the per-environment
// contact count is a wave sum (no atomics).
template <bool kSinglePoint>
__device__ __forceinline__ void narrowphase_of_env(const ModelView& m, const DataView& d, const NarrowphasePrimitivesParams& p, uint32_t env,
                                                   uint32_t lane) {
    uint32_t contacts = 0u;
    for (uint32_t first = 0u; first < p.rigid_slot_cap; first += 64u) {
        const uint32_t slot = first + lane;
        if (slot < p.rigid_slot_cap) contacts += NarrowphaseSlot<kSinglePoint>(m, d, p, env, slot);
    }
    contacts = wave_sum_u(contacts);
    if (lane == 0u) d.contact_count[env] = contacts;
}
template <bool kSinglePoint>
__global__ void __launch_bounds__(64) NarrowphaseKernel(ModelView m, DataView d, NarrowphasePrimitivesParams p) {
    narrowphase_of_env<kSinglePoint>(m, d, p, blockIdx.x, threadIdx.x);
}
// Worlds of at most 32 slots an environment: `width` lanes (a power of two, at least the slots) an environment and
// 64 / width environments a wavefront, so that a world of one or two slots does not leave 62 lanes of every wavefront
// idle.  The same slot code; an environment's contact count is the sum over its lanes (integers: any order).
template <bool kSinglePoint>
__global__ void __launch_bounds__(64) NarrowphasePackedKernel(ModelView m, DataView d, NarrowphasePrimitivesParams p, uint32_t width) {
    const uint32_t lane = threadIdx.x;
    const uint32_t env = blockIdx.x * (64u / width) + lane / width, slot = lane % width;
    uint32_t contacts = 0u;
    if (env < p.env_count && slot < p.rigid_slot_cap) contacts = NarrowphaseSlot<kSinglePoint>(m, d, p, env, slot);
    for (uint32_t o = width >> 1u; o != 0u; o >>= 1u) contacts += uint32_t(__shfl_xor(int(contacts), int(o), 64));
    if (slot == 0u && env < p.env_count) d.contact_count[env] = contacts;
}

// What stands between the dynamics and the row assembly - the bodies' poses, their boxes, the candidate pairs, the
// manifolds - as one kernel, one wavefront an environment: four kernels of about a launch's time each become one, running
// the same device code in the same order.  Single-point worlds only (the general manifolds keep their candidate lists in
// scratch memory).  A plan takes this route when its op list holds the ops in a row (backend.hip).
__global__ void __launch_bounds__(kWave) CollisionHeadKernel(ModelView m, DataView d, BuildAabbsParams boxes, LbvhQueryPairsParams query,
                                                             NarrowphasePrimitivesParams narrow) {
    const uint32_t env = blockIdx.x, lane = threadIdx.x, nb = m.bodies_per_env;
    const float* link_pose = d.link_pose + size_t{env} * m.links_per_env * 7u;
    for (uint32_t b = lane; b < nb; b += kWave) sync_body_pose(m, d, env, b, link_pose);
    __syncthreads();   // the poses are in memory for every lane
    for (uint32_t b = lane; b < nb; b += kWave) build_aabb_of_body(m, d, boxes, env * nb + b);
    __syncthreads();
    query_pairs_of_env(m, d, query, env, lane);
    __syncthreads();
    narrowphase_of_env<true>(m, d, narrow, env, lane);
}
// math/cuda_vec_ops.cuh:150-183
__device__ void contact_tangent_basis(V3 normal, V3* t1, V3* t2) {
    V3 n = normal;
    const float l = dot3(n, n);
    if (l > 1.0e-10f) { const float inv = rsqrt_exact(l); n = V3{n.x * inv, n.y * inv, n.z * inv}; }
    else n = V3{0.0f, 0.0f, 1.0f};
    V3 reference{1.0f, 0.0f, 0.0f};
    if (fabsf(n.x) > 0.9f) reference = V3{0.0f, 1.0f, 0.0f};
    const float proj = dot3(reference, n);
    V3 ta{reference.x - proj * n.x, reference.y - proj * n.y, reference.z - proj * n.z};
    const float len_sq = dot3(ta, ta);
    if (len_sq > 1.0e-12f) { const float s = rsqrt_exact(len_sq); ta = V3{ta.x * s, ta.y * s, ta.z * s}; }
    else ta = V3{1.0f, 0.0f, 0.0f};
    *t1 = ta;
    *t2 = cross3(n, ta);
}

// union_types.cuh:187-193
__device__ __forceinline__ uint32_t contact_row_bound(uint32_t previous, uint32_t current, uint32_t contact_rows) {
    if (previous == 0u || current == 0u) return contact_rows;
    return min(max(previous, current) - 1u, contact_rows);
}

// nk/solve/collidable_owner.hpp:25-62 for one articulation per environment
__device__ uint32_t resolve_side(const ModelView& m, uint32_t env, uint32_t collidable, int32_t body_id, uint32_t* index,
                                 uint32_t* link) {
    *index = kInvalid; *link = kInvalid;
    if (collidable >= m.bodies_per_env) return kInvalid;
    uint32_t body = collidable;
    if (body_id < 0) return kSideStatic;
    const uint32_t proxy = m.body_collidable_body[body];
    if (proxy != kInvalid) {
        if (proxy >= m.bodies_per_env) return kInvalid;
        body = proxy;
        if (m.body_collidable_body[body] != kInvalid) return kInvalid;
    }
    const uint32_t l = m.body_to_link[body];
    if (l == kInvalid) { *index = env * m.bodies_per_env + body; return kSideRigid; }
    if (l >= m.links_per_env || m.body_to_articulation[body] >= 1u) return kInvalid;
    *link = env * m.links_per_env + l; *index = env;
    return kSideArtic;
}

struct RowSide { uint32_t kind, index; V3 jlin, jang; };
struct Row { uint32_t flags, group_first, group_normal_count, env; float rhs, compliance_alpha, lower, upper, mu, friction_secondary; RowSide a, b; };
static_assert(sizeof(Row) == kRowWords * sizeof(float), "row layout must stay 26 words");

// HashMergedContactProfile (assemble_rows.cu:88-105) of two default-authored profiles that differ in friction only
// (scene/contact_filter.hpp:16-31, 72-130: equal priorities and mixing weights leave every other term at its default),
// then the contact law for velocity-only laws (:620-622).
__device__ __forceinline__ uint64_t profile_word(uint64_t hash, uint32_t word) { hash ^= uint64_t{word}; hash *= 0x100000001b3ull; return hash; }
__device__ uint64_t contact_material_key(float mu1, float mu2, uint32_t law) {
    uint64_t h = 0x4e554b4150524f46ull;
    h = profile_word(h, 2u);   // profile schema version
    h = profile_word(h, 1u);   // reference-safe flag
    h = profile_word(h, __float_as_uint(mu1)); h = profile_word(h, __float_as_uint(mu2));
    h = profile_word(h, __float_as_uint(0.005f)); h = profile_word(h, __float_as_uint(0.0001f));
    h = profile_word(h, __float_as_uint(0.02f)); h = profile_word(h, __float_as_uint(1.0f));
    h = profile_word(h, __float_as_uint(0.9f)); h = profile_word(h, __float_as_uint(0.95f)); h = profile_word(h, __float_as_uint(0.001f));
    h = profile_word(h, __float_as_uint(0.5f)); h = profile_word(h, __float_as_uint(2.0f));
    h = profile_word(h, __float_as_uint(0.0f)); h = profile_word(h, __float_as_uint(0.0f));
    h = profile_word(h, 3u);
    if (h == 0ull) h = 0x9e3779b97f4a7c15ull;
    if (law == 1u || law == 2u) { h ^= uint64_t{law}; h *= 1099511628211ull; }
    return h;
}

// The same hash of any merged profile (mu1, mu2, solref[2], solimp[5], margin, gap, condim; no friction slope), then
// the law word for the velocity-only laws and the cone for the compliant law (:620-623).
__device__ uint64_t merged_material_key(const float (&merged)[12], uint32_t law, uint32_t cone) {
    uint64_t h = 0x4e554b4150524f46ull;
    h = profile_word(h, 2u);
    h = profile_word(h, 1u);
    h = profile_word(h, __float_as_uint(merged[0])); h = profile_word(h, __float_as_uint(merged[1]));
    h = profile_word(h, __float_as_uint(0.005f)); h = profile_word(h, __float_as_uint(0.0001f));
    for (int i = 2; i < 11; ++i) h = profile_word(h, __float_as_uint(merged[i]));
    h = profile_word(h, uint32_t(merged[11]));
    if (h == 0ull) h = 0x9e3779b97f4a7c15ull;
    if (law == kContactLawVelocity || law == kContactLawSpeculative) { h ^= uint64_t{law}; h *= 1099511628211ull; }
    if (law == kContactLawCompliant) { h ^= uint64_t{cone}; h *= 1099511628211ull; }
    return h;
}
// One shape's contact parameters as the merge takes them: mu1, mu2, solref[2], solimp[5], margin, gap, priority,
// solmix, condim; a shape without a profile has the defaults of scene/contact_filter.hpp:20-37.
__device__ void profile_terms(const ModelView& m, uint32_t profile, float (&out)[14]) {
    out[0] = 1.0f; out[1] = 1.0f; out[2] = 0.02f; out[3] = 1.0f; out[4] = 0.9f; out[5] = 0.95f; out[6] = 0.001f; out[7] = 0.5f; out[8] = 2.0f;
    out[9] = 0.0f; out[10] = 0.0f; out[11] = 0.0f; out[12] = 1.0f; out[13] = 3.0f;
    if (profile >= m.profile_count) return;
    out[0] = m.profile_mu[2u * profile]; out[1] = m.profile_mu[2u * profile + 1u];
    out[2] = m.profile_solref[2u * profile]; out[3] = m.profile_solref[2u * profile + 1u];
    for (uint32_t k = 0u; k < 5u; ++k) out[4u + k] = m.profile_solimp[5u * profile + k];
    out[9] = m.profile_margin[2u * profile]; out[10] = m.profile_margin[2u * profile + 1u];
    for (uint32_t k = 0u; k < 3u; ++k) out[11u + k] = m.profile_mix[3u * profile + k];
}
// MergeContactParams (scene/contact_filter.hpp:89-137) with arithmetic friction mixing: the side of higher priority
// gives friction and condim and all of the mixing weight; at equal priority friction and condim take the larger and
// the weight is solmix_a / (solmix_a + solmix_b), a side whose solmix is below 1e-15 deferring to the other.  solref
// is mixed, or the minimum when either is in direct form; solimp is mixed; margins and gaps add.
__device__ void merge_contact_params(const float (&a)[14], const float (&b)[14], float (&out)[12]) {
    float mix;
    if (a[11] != b[11]) {
        const bool first = a[11] > b[11];
        mix = first ? 1.0f : 0.0f;
        out[11] = first ? a[13] : b[13]; out[0] = first ? a[0] : b[0]; out[1] = first ? a[1] : b[1];
    } else {
        out[11] = a[13] > b[13] ? a[13] : b[13];
        out[0] = a[0] > b[0] ? a[0] : b[0];
        out[1] = a[1] > b[1] ? a[1] : b[1];
        const bool a_ok = a[12] >= 1e-15f, b_ok = b[12] >= 1e-15f;
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
// ComputeCompliantRow (constraint/solref_solimp.hpp:55-86) followed by DiscretizeCompliantRow (:40-44): the row's
// regularisation R, its reference acceleration and the gain on the start velocity, for the step dt with the
// damping taken at the midpoint.
struct CompliantRow { float R, bias, gain; };
__device__ __forceinline__ float clampf(float v, float lo, float hi) { return fminf(fmaxf(v, lo), hi); }
__device__ CompliantRow compliant_row(const float* solref, const float* solimp, float pos_imp, float pos_aref, float vel, float invweight,
                                      float dt, bool refsafe) {
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
    const float R = 1.0f / D, aref = -k * imp * pos_aref - b * vel;
    const double scale = 1.0 + 0.5 * double(dt) * b;
    return CompliantRow{float(R / scale), float(aref / scale), float((1.0 / double(dt) - 0.5 * b) / scale)};
}
// math/cuda_vec_ops.cuh:187-196 MuJoCoContactFrame: the first tangent along `axis` where that is far enough from the
// normal, else along a world axis
__device__ void mujoco_contact_frame(V3 normal, V3 axis, V3* t1, V3* t2) {
    V3 n = normal;
    const float l = dot3(n, n);
    if (l > 1.0e-10f) { const float inv = rsqrt_exact(l); n = V3{n.x * inv, n.y * inv, n.z * inv}; }
    else n = V3{0.0f, 0.0f, 1.0f};
    V3 tangent = sub3(axis, scale3(n, dot3(n, axis)));
    if (dot3(tangent, tangent) < 0.25f) {
        const V3 reference = n.y > -0.5f && n.y < 0.5f ? V3{0.0f, 1.0f, 0.0f} : V3{0.0f, 0.0f, 1.0f};
        tangent = sub3(reference, scale3(n, dot3(n, reference)));
    }
    const V3 a = scale3(tangent, rsqrt_exact(dot3(tangent, tangent)));
    *t1 = a;
    *t2 = cross3(n, a);
}

__device__ __forceinline__ float uniform_value(float v, uint32_t lane) {   // `lane` is the same in every lane
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), int(lane)));
}

// ---- AssembleRows: one wavefront per environment (assemble_rows.cu:325-394, 200-214, 406-801, 122-186) ----
// four waves a SIMD (128 registers a lane): sixteen environments a compute unit are resident at once at 4096 environments
__global__ void __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(4, 4))) AssembleRowsKernel(ModelView m, DataView d, AssembleRowsParams p) {
    extern __shared__ uint32_t lds_u[];
    const uint32_t env = blockIdx.x, lane = threadIdx.x;
    const uint32_t R = p.rows_per_env, S = p.union_slot_count, CR = p.contact_rows_per_env, md = p.max_dof, nl = m.links_per_env;
    uint32_t* range_first = lds_u;        // S
    uint32_t* range_points = lds_u + S;   // S
    // what the chain Jacobian pass needs of each row, kept here so that it does not read back what this block wrote
    uint32_t* row_link_a = lds_u + 2u * S;             // CR (contact rows only; joint rows need no chain walk)
    uint32_t* row_link_b = row_link_a + CR;             // CR
    uint32_t* row_merge = row_link_b + CR;              // CR: both sides articulated with the same owner
    float* row_point = reinterpret_cast<float*>(row_merge + CR);   // 3 CR
    float* row_dir = row_point + 3u * CR;                // 3 CR, side A's direction (side B's is its negative)
    float* row_gain = row_dir + 3u * CR;                 // CR: a compliant row's gain on the start velocity along it, else 0
    // nl: the coordinates on each link's path to the root (2 S + 10 CR words come before: an even count, so 8-byte aligned);
    // the chain Jacobian pass asks for a link's mask once a row and side and would wait on the table each time
    uint64_t* link_mask = reinterpret_cast<uint64_t*>(row_gain + CR);
    for (uint32_t l = lane; l < nl; l += kWave) link_mask[l] = m.link_dof_mask[l];
    Row* rows = reinterpret_cast<Row*>(d.urows) + size_t{env} * R;
    float* lambda = d.lambda + size_t{env} * R;
    float* pen = d.row_penetration + size_t{env} * R;
    uint32_t* cj_link = d.row_cj_link + size_t{env} * R, *cj_link_b = d.row_cj_link_b + size_t{env} * R;
    float* cj_point = d.row_cj_point + size_t{env} * R * 3u, *cj_point_b = d.row_cj_point_b + size_t{env} * R * 3u;
    // row ranges: exclusive prefix of the slots' point counts, four rows a point (:336-360)
    const uint32_t previous_extent = d.contact_row_extent[2u * env + 1u];
    uint32_t carry = 0u, extent = 1u;
    for (uint32_t base = 0u; base < S; base += kWave) {
        const uint32_t slot = base + lane;
        const uint32_t points = slot < S ? d.ucontact_count[size_t{env} * S + slot] : 0u;
        uint32_t through = points;
#pragma unroll
        for (int o = 1; o < kWave; o <<= 1) {
            const uint32_t other = __shfl_up(through, o, kWave);
            if (int(lane) >= o) through += other;
        }
        if (slot < S) {
            const uint32_t first = (carry + through - points) * kRowsPerPoint;
            range_first[slot] = first; range_points[slot] = points;
            d.ucontact_row_range[(size_t{env} * S + slot) * 2u] = env * R + first;
            d.ucontact_row_range[(size_t{env} * S + slot) * 2u + 1u] = points;
            if (first < contact_row_bound(previous_extent, 1u, CR)) d.contact_material[size_t{env} * S + slot] = 0ull;   // :358
            if (points > 0u) extent = max(extent, first + points * kRowsPerPoint + 1u);
        }
        carry += __shfl(through, kWave - 1, kWave);
    }
    extent = wave_max_u(extent);
    // rows below the previous and current extents are cleared (:366-394)
    const uint32_t clear_bound = contact_row_bound(previous_extent, 1u, CR);
    for (uint32_t local = lane; local < min(clear_bound, CR); local += kWave) {
        lambda[local] = 0.0f; pen[local] = 0.0f; cj_link[local] = kInvalid; cj_link_b[local] = kInvalid;
        rows[local].flags = 0u;
    }
    for (uint32_t local = lane; local < CR; local += kWave) { row_link_a[local] = kInvalid; row_link_b[local] = kInvalid; row_merge[local] = 0u; row_gain[local] = 0.0f; }
    if (lane == 0u) {
        d.contact_row_extent[2u * env] = previous_extent;
        d.contact_row_extent[2u * env + 1u] = extent;
    }
    // padded generalized velocity tile (:200-214)
    if (lane < md) {
        float value = 0.0f;
        if (lane < m.dof) {
            const uint32_t link = m.dof_link[lane], c = m.dof_component[lane];
            value = c == kInvalid ? d.qdot[size_t{env} * nl + link] : d.link_velocity[(size_t{env} * nl + link) * 6u + c];
        }
        d.qdot_flat[size_t{env} * md + lane] = value;
    }
    __syncthreads();
    // contact rows (:453-801; speculative law, condim 3): a lane a slot where every slot has one point at most, else a
    // lane a (slot, point) - a slot's points share nothing but the slot's own values, which each of their lanes works
    // out for itself
    uint32_t active_rows = 0u;
    bool invalid_endpoint = false;
    const uint32_t fan = m.max_points_per_slot > 1u ? 4u : 1u;
    for (uint32_t item = lane; item < S * fan; item += kWave) {
        const uint32_t slot = item / fan, own_point = item - slot * fan;
        const size_t gid = size_t{env} * S + slot;
        const uint32_t base = range_first[slot], P = range_points[slot];
        if (P == 0u || (fan > 1u && own_point >= P)) continue;
        const bool slot_lane = own_point == 0u;   // the one lane that writes what belongs to the slot as a whole
        uint32_t n_active = P;
        const uint32_t local_a = d.ucontact_a[gid * 4u], local_b = d.ucontact_b[gid * 4u];
        ShapeRow sa{}, sb{};
        sa.body_id = sb.body_id = -1; sa.profile = sb.profile = kInvalid;
        if (local_a < m.bodies_per_env) sa = load_shape(m.shape_table, local_a);
        if (local_b < m.bodies_per_env) sb = load_shape(m.shape_table, local_b);
        uint32_t idx_a, idx_b, link_a, link_b;
        uint32_t kind_a = resolve_side(m, env, local_a, sa.body_id, &idx_a, &link_a);
        uint32_t kind_b = resolve_side(m, env, local_b, sb.body_id, &idx_b, &link_b);
        if (kind_a == kInvalid || kind_b == kInvalid) {
            invalid_endpoint = true;
            n_active = 0u; kind_a = kind_b = kSideStatic;
        }
        if (kind_a == kSideStatic) idx_a = kInvalid;
        if (kind_b == kSideStatic) idx_b = kInvalid;
        // the two sides' profiles merged (:540-594; scene/contact_filter.hpp:100-137); a side without one has the defaults
        const uint32_t law = d.ucontact_law[gid];
        const bool mujoco = law == kContactLawCompliant;   // :480
        float side_a[14], side_b[14], merged[12];
        profile_terms(m, sa.profile, side_a); profile_terms(m, sb.profile, side_b);
        merge_contact_params(side_a, side_b, merged);
        if (mujoco) { merged[0] = fmaxf(1.0e-5f, merged[0]); merged[1] = fmaxf(1.0e-5f, merged[1]); }   // :573-576
        const float mu1 = merged[0], mu2 = merged[1];
        const float* solref = merged + 2, *solimp = merged + 4;
        const float margin = merged[9];
        if (slot_lane) d.contact_material[gid] = n_active > 0u ? merged_material_key(merged, law, m.contact_cone) : 0ull;   // :620-623
        // a compliant row's weight is the sum of its two bodies' reference weights, a link's through its own collidable row (:595-597)
        float invweight = 0.0f;
        if (mujoco) {
            const float* weights = d.body_invweight0 + size_t{env} * m.bodies_per_env * 2u;
            const uint32_t weight_a = kind_a == kSideArtic ? m.link_body[link_a - env * nl] : local_a;
            const uint32_t weight_b = kind_b == kSideArtic ? m.link_body[link_b - env * nl] : local_b;
            invweight = (weight_a < m.bodies_per_env ? weights[2u * weight_a] : 0.0f) + (weight_b < m.bodies_per_env ? weights[2u * weight_b] : 0.0f);
        }
        const bool friction_rows = merged[11] == 3.0f;   // condim 3: a normal and two tangents, else the normal alone (:721, 763)
        const bool pyramidal = mujoco && m.contact_cone == 0u && friction_rows;   // :598
        const float impratio = m.contact_impratio;
        V3 frame_axis{0, 0, 0};   // :601-605: a capsule on a plane aligns the pyramid with the capsule's axis
        if (pyramidal && sa.kind == 1u && sb.kind == 3u) frame_axis = make_prim(sa, load_xf(d.body_pose + (size_t{env} * m.bodies_per_env + local_a) * 7u)).cz;
        if (pyramidal && sb.kind == 1u && sa.kind == 3u) frame_axis = make_prim(sb, load_xf(d.body_pose + (size_t{env} * m.bodies_per_env + local_b) * 7u)).cz;
        for (uint32_t pt = fan > 1u ? own_point : 0u; pt < (fan > 1u ? own_point + 1u : P); ++pt) {
            const size_t mp = gid * 4u + pt;
            // the velocity laws keep every point; a compliant point lives inside its margin (:625-626)
            const bool live = pt < n_active && pt < 4u && (!mujoco || d.ucontact_depth[mp] + margin > 0.0f);
            // the rows' directions as four values selected by the row's place, not an array indexed by it: an array
            // indexed at run time lives in scratch memory, and every row would wait on it
            V3 n{0, 0, 1}, point{0, 0, 0}, dir0{0, 0, 0}, dir1{0, 0, 0}, dir2{0, 0, 0}, dir3{0, 0, 0};
            V3 t0{1, 0, 0}, t1{0, 1, 0};
            float d0 = 0.0f;
            if (live) {
                const V3 raw{d.ucontact_normal[3u * mp], d.ucontact_normal[3u * mp + 1u], d.ucontact_normal[3u * mp + 2u]};
                const float len = sqrtf(raw.x * raw.x + raw.y * raw.y + raw.z * raw.z);
                n = len < 1e-12f ? V3{0, 0, 0} : V3{raw.x / len, raw.y / len, raw.z / len};
                point = V3{d.ucontact_point[3u * mp], d.ucontact_point[3u * mp + 1u], d.ucontact_point[3u * mp + 2u]};
                if (pyramidal) mujoco_contact_frame(raw, frame_axis, &t0, &t1);
                else contact_tangent_basis(raw, &t0, &t1);
                d0 = d.ucontact_depth[mp];
            }
            // a pyramid has four scalar rows a point along n +- mu t (:651-690); the other cones a normal and two tangents
            const uint32_t row_count = pyramidal ? 4u : 3u;
            const bool emits[2] = {live, live && friction_rows};   // the normal row; the tangent rows
            CompliantRow edge{};
            float edge_invweight = 0.0f;
            if (pyramidal) {
                edge_invweight = (invweight + mu1 * mu1 * invweight) * 2.0f * mu1 * mu1 / impratio;
                const float pos = -d0 - margin;
                edge = compliant_row(solref, solimp, pos, pos, 0.0f, edge_invweight, p.dt, p.refsafe);
                dir0 = add3(n, scale3(t0, mu1)); dir1 = add3(n, scale3(t0, -mu1));
                dir2 = add3(n, scale3(t1, mu2)); dir3 = add3(n, scale3(t1, -mu2));
            } else { dir0 = n; dir1 = t0; dir2 = t1; }
            for (uint32_t axis = 0u; axis < row_count; ++axis) {
                const uint32_t rs = base + axis * P + pt;
                lambda[rs] = 0.0f; pen[rs] = 0.0f; cj_link[rs] = kInvalid; cj_link_b[rs] = kInvalid;
                row_gain[rs] = 0.0f;
                if (!(pyramidal ? live : emits[axis == 0u ? 0 : 1])) {
                    if (pyramidal) rows[rs] = Row{}; else rows[rs].flags = 0u;
                    continue;
                }
                Row row{};
                const V3 dir = axis == 0u ? dir0 : axis == 1u ? dir1 : axis == 2u ? dir2 : dir3;
                row.group_first = env * R + base; row.group_normal_count = P; row.env = env;
                row.mu = mu1; row.friction_secondary = mu2;
                row.a.kind = kind_a; row.a.index = idx_a; row.a.jlin = dir; row.a.jang = V3{0, 0, 0};
                row.b.kind = kind_b; row.b.index = idx_b; row.b.jlin = V3{-dir.x, -dir.y, -dir.z}; row.b.jang = V3{0, 0, 0};
                float gain = 0.0f, weight = 0.0f;
                if (pyramidal) {
                    row.flags = kRowActive | kRowMuJoCo | kRowPyramidal | (axis == 0u ? uint32_t(kRowContactNormal) : 0u);
                    row.group_first = env * R + rs; row.group_normal_count = 1u;
                    row.rhs = edge.bias; row.compliance_alpha = edge.R;
                    row.lower = 0.0f; row.upper = FLT_MAX;
                    gain = edge.gain; weight = edge_invweight;
                } else if (axis == 0u) {
                    // speculative rows reserve the rounding of their projected endpoint positions (:703-713)
                    const V3 ext{fabsf(point.x) + fabsf(n.x * d0), fabsf(point.y) + fabsf(n.y * d0), fabsf(point.z) + fabsf(n.z * d0)};
                    const double gamma = 3.0 * double(FLT_EPSILON) / (1.0 - 3.0 * double(FLT_EPSILON));
                    const double roundoff = gamma * (fabs(double(n.x)) * (fabs(double(ext.x)) + fabs(double(ext.x))) +
                                                     fabs(double(n.y)) * (fabs(double(ext.y)) + fabs(double(ext.y))) +
                                                     fabs(double(n.z)) * (fabs(double(ext.z)) + fabs(double(ext.z))));
                    const float clearance = roundoff > 0.0 ? nextafterf(float(roundoff), FLT_MAX) : 0.0f;
                    const float depth = d0 + clearance;
                    pen[rs] = mujoco ? fmaxf(d0, 0.0f) : depth;
                    row.flags = kRowActive | kRowContactNormal | (friction_rows ? uint32_t(kRowBlockNormal) : 0u) | (mujoco ? uint32_t(kRowMuJoCo) : uint32_t(kRowSpeculative));
                    row.rhs = (fminf(depth, 0.0f) + (p.position_pass != 0u ? 0.0f
                               : fminf(fmaxf(d0, 0.0f), p.overlap_recovery_velocity * p.dt))) / (p.dt * p.dt);
                    if (mujoco) {   // :714-731: the spring-damper reference of the merged solref / solimp at this depth
                        const float pos = -d0 - margin;
                        const CompliantRow c = compliant_row(solref, solimp, pos, pos, 0.0f, invweight, p.dt, p.refsafe);
                        row.rhs = c.bias; row.compliance_alpha = c.R;
                        gain = c.gain; weight = invweight;
                    }
                    row.lower = 0.0f; row.upper = FLT_MAX;
                } else {
                    row.flags = kRowActive | kRowBlockTangent;
                    if (mujoco) {   // :771-782: the tangent rows' compliance, which shapes the elliptic cone's metric
                        const float mu = axis == 1u ? mu1 : mu2;
                        weight = invweight / impratio * (mu1 * mu1) / (mu * mu);
                        const CompliantRow c = compliant_row(solref, solimp, -d0 - margin, 0.0f, 0.0f, weight, p.dt, p.refsafe);
                        row.flags |= kRowMuJoCo;
                        row.compliance_alpha = c.R;
                        gain = c.gain;
                    }
                    row.lower = -FLT_MAX; row.upper = FLT_MAX;
                }
                if (mujoco) {
                    d.row_reference_velocity_gain[size_t{env} * R + rs] = gain;
                    d.row_invweight[size_t{env} * R + rs] = weight;
                    row_gain[rs] = gain;
                }
                row_point[3u * rs] = point.x; row_point[3u * rs + 1u] = point.y; row_point[3u * rs + 2u] = point.z;
                row_dir[3u * rs] = dir.x; row_dir[3u * rs + 1u] = dir.y; row_dir[3u * rs + 2u] = dir.z;
                if (kind_a == kSideArtic) row_link_a[rs] = link_a;
                if (kind_b == kSideArtic) row_link_b[rs] = link_b;
                row_merge[rs] = kind_a == kSideArtic && kind_b == kSideArtic && idx_a == idx_b ? 1u : 0u;
                if (kind_a == kSideArtic) { cj_link[rs] = link_a; cj_point[3u * rs] = point.x; cj_point[3u * rs + 1u] = point.y; cj_point[3u * rs + 2u] = point.z; }
                if (kind_b == kSideArtic) { cj_link_b[rs] = link_b; cj_point_b[3u * rs] = point.x; cj_point_b[3u * rs + 1u] = point.y; cj_point_b[3u * rs + 2u] = point.z; }
                rows[rs] = row;
                ++active_rows;
            }
        }
    }
    // joint rows (EmitJointRowsKernel, assemble_rows.cu:803-1026): stable per-link slots after the contact rows - lower
    // and upper limit (two a link), dry friction, drive.  Each acts on one coordinate, J = +-e_joint; the rest of
    // its Jacobian row is never written and stays at the zeros it was allocated with.  A MuJoCo-sourced joint gets its
    // limit and friction rows as compliant rows (margin, solref, solimp at the coordinate's reference weight).
    {
        const uint32_t limit_rows = p.joint_limit_rows_per_env, friction_rows = p.joint_friction_rows_per_env;
        const uint32_t joint_slots = limit_rows + friction_rows + p.joint_drive_rows_per_env;
        const size_t lbase = size_t{env} * nl;
        for (uint32_t slot = lane; slot < joint_slots; slot += kWave) {
            const uint32_t rs = CR + slot;
            Row row{};
            cj_link[rs] = kInvalid; cj_link_b[rs] = kInvalid; pen[rs] = 0.0f;
            float jacobian = 0.0f, impulse = 0.0f, joint_gain = 0.0f, joint_weight = 0.0f;
            uint32_t l;
            if (slot < limit_rows) {   // EmitJointLimitRow :805-882
                l = slot / 2u;
                const uint32_t side = slot & 1u;
                if (joint_dof(m.joint_type[l]) == 1u && (m.joint_limit_flags[l] & (1u << side)) != 0u && p.dt > 0.0f) {
                    const float bound = side == 0u ? m.joint_limit_lower[l] : m.joint_limit_upper[l];
                    const float q = d.q[lbase + l];
                    const float signed_distance = side == 0u ? q - bound : bound - q;
                    // with a position pass the row only stops further violation; that pass removes it
                    const float target_velocity = -(p.position_pass != 0u ? fmaxf(signed_distance, 0.0f) : signed_distance) / p.dt;
                    row.flags = kRowActive | (side == 0u ? kRowJointLimitLower : kRowJointLimitUpper);
                    row.rhs = fminf(target_velocity, p.baumgarte_max_velocity) / p.dt;
                    row.lower = 0.0f; row.upper = FLT_MAX;
                    jacobian = side == 0u ? 1.0f : -1.0f;
                    pen[rs] = fmaxf(-signed_distance, 0.0f);
                    impulse = lambda[rs];   // an active limit row keeps its multiplier
                    if (m.joint_law[l] == 1u) {   // :860-877: a compliant row inside its margin, on the nearer bound only
                        const float pos = signed_distance - m.joint_limit_margin[l];
                        const float* reference = m.joint_limit_reference + 7u * l;
                        const float invweight = d.dof_invweight0[size_t{env} * md + m.link_dof[l]];
                        const CompliantRow c = compliant_row(reference, reference + 2u, pos, pos, 0.0f, invweight, p.dt, p.refsafe);
                        row.flags |= kRowMuJoCo;
                        const bool lower_nearest = q - m.joint_limit_lower[l] < m.joint_limit_upper[l] - q;
                        if (pos >= 0.0f || lower_nearest != (side == 0u)) { row.flags &= ~uint32_t(kRowActive); impulse = 0.0f; }
                        row.rhs = c.bias; row.compliance_alpha = c.R;
                        joint_gain = c.gain; joint_weight = invweight;
                    }
                }
            } else if (slot < limit_rows + friction_rows) {   // EmitJointFrictionRows :886-934
                l = slot - limit_rows;
                const float friction = m.joint_frictionloss[l];
                if (joint_dof(m.joint_type[l]) == 1u && friction > 0.0f && p.dt > 0.0f) {
                    row.flags = kRowActive | kRowVelocityOnly;
                    row.lower = -friction * p.dt; row.upper = friction * p.dt;
                    jacobian = 1.0f;
                    if (m.joint_law[l] == 1u) {   // :921-931: dry friction regularised by its own solref / solimp
                        const float* reference = m.joint_friction_reference + 7u * l;
                        const float invweight = d.dof_invweight0[size_t{env} * md + m.link_dof[l]];
                        const CompliantRow c = compliant_row(reference, reference + 2u, 0.0f, 0.0f, 0.0f, invweight, p.dt, p.refsafe);
                        row.flags |= kRowMuJoCo;
                        row.compliance_alpha = c.R;
                        joint_gain = c.gain; joint_weight = invweight;
                    }
                }
            } else {   // EmitJointDriveRows :938-971
                l = slot - limit_rows - friction_rows;
                const float effort = fminf(fmaxf(d.drive_command[lbase + l], d.drive_lower[lbase + l]), d.drive_upper[lbase + l]);
                if (joint_dof(m.joint_type[l]) == 1u && effort != 0.0f) {
                    row.flags = kRowActive | kRowVelocityOnly;
                    row.lower = row.upper = effort * p.dt;
                    jacobian = 1.0f;
                    impulse = row.lower;   // the row admits one impulse, so the first sweep already descends against it
                }
            }
            if (row.flags != 0u) {
                row.group_first = env * R + rs; row.group_normal_count = 1u; row.env = env;
                row.a.kind = kSideArtic; row.a.index = env;
                if ((row.flags & kRowActive) != 0u) ++active_rows;
                if ((row.flags & kRowMuJoCo) != 0u) {
                    d.row_reference_velocity_gain[size_t{env} * R + rs] = joint_gain;
                    d.row_invweight[size_t{env} * R + rs] = joint_weight;
                    // PrepareContactRowsKernel (:1134-1140): the row's one entry times the start velocity of its coordinate
                    if ((row.flags & kRowActive) != 0u)
                        row.rhs += joint_gain * (0.0f + jacobian * d.step_qdot_flat[size_t{env} * md + m.link_dof[l]]);
                }
            }
            lambda[rs] = impulse;
            if (joint_dof(m.joint_type[l]) == 1u) d.chain_jacobian[(size_t{env} * R + rs) * md + m.link_dof[l]] = jacobian;
            // the solve takes a row on one coordinate from here instead of scanning its Jacobian row for it
            d.row_unit[size_t{env} * R + rs] = row.flags != 0u ? m.link_dof[l] : kInvalid;
            d.row_unit_value[size_t{env} * R + rs] = jacobian;
            rows[rs] = row;
        }
    }
    active_rows = uint32_t(wave_sum(float(active_rows)));
    invalid_endpoint = __any(invalid_endpoint);
    if (lane == 0u) {
        d.row_count[env] = active_rows;
        if (invalid_endpoint) d.env_status[env] |= kEnvStatusInvalidEndpoint;
    }
    __syncthreads();
    // chain Jacobians, lane = DoF: every row entry is the joint's own column when the joint lies on the path from
    // the row's link to the root, which the cooked per-link DoF mask answers (assemble_rows.cu:122-169,
    // articulation_types.cuh:193-238); both sides, then the shared-owner merge (:172-186).
    if (md == 0u) return;
    V3 axis_world{0, 0, 0}, origin{0, 0, 0};
    uint32_t mode = 0u;   // 0 none, 1 revolute, 2 prismatic, 3 base angular, 4 base linear
    if (lane < m.dof) {
        const uint32_t link = m.dof_link[lane], component = m.dof_component[lane];
        if (component == kInvalid) {
            const Xf pose = load_xf(d.link_pose + (size_t{env} * nl + link) * 7u);
            axis_world = rotate_normalized(pose.r, V3{m.joint_axis[3u * link], m.joint_axis[3u * link + 1u], m.joint_axis[3u * link + 2u]});
            origin = pose.p;
            mode = m.joint_type[link] == kPrismatic ? 2u : 1u;
        } else {
            const Xf base = load_xf(d.base_pose + size_t{env} * 7u);
            const uint32_t k = component % 3u;
            const V3 unit{k == 0u ? 1.0f : 0.0f, k == 1u ? 1.0f : 0.0f, k == 2u ? 1.0f : 0.0f};
            if (m.free_body != 0u) {
                // a free body's coordinates: linear velocity, then angular velocity about the centre of mass, world axes -
                // the row's jlin and jang = (point - com) x jlin (assemble_rows.cu:537-538, 680-681)
                axis_world = unit;
                const float* frame = d.body_inertial_frame + (size_t{env} * m.bodies_per_env + m.link_body[0]) * 7u;
                origin = add3(base.p, rotate_normalized(base.r, V3{frame[0], frame[1], frame[2]}));
                mode = component < 3u ? 4u : 3u;
            } else {
                axis_world = rotate_normalized(base.r, unit);
                origin = base.p;
                mode = component < 3u ? 3u : 4u;
            }
        }
    }
    // only the rows below this step's extent can have a link; the rows up to the previous extent were cleared above
    const uint32_t bound = min(extent - 1u, CR);
    const float start_velocity = m.any_mujoco != 0u && lane < md ? d.step_qdot_flat[size_t{env} * md + lane] : 0.0f;
    // Sixty-four rows at a time: every lane first fetches one row's endpoints, point, direction, gain and its links' masks
    // (one round of LDS reads, all in flight together), then the rows go by in turn with their values handed round as
    // lane reads - a row no longer waits on its own chain of dependent reads.
    auto uniform_word = [](uint32_t v, uint32_t from) { return uint32_t(__builtin_amdgcn_readlane(int(v), int(from))); };
    for (uint32_t first = 0u; first < bound; first += kWave) {
        const uint32_t mine = first + lane;
        uint32_t my_link[2] = {kInvalid, kInvalid}, my_merge = 0u, my_mask[2][2] = {{0u, 0u}, {0u, 0u}};
        float my_point[3] = {0.0f, 0.0f, 0.0f}, my_dir[3] = {0.0f, 0.0f, 0.0f}, my_gain = 0.0f;
        if (mine < bound) {
            my_link[0] = row_link_a[mine]; my_link[1] = row_link_b[mine]; my_merge = row_merge[mine]; my_gain = row_gain[mine];
#pragma unroll
            for (int k = 0; k < 3; ++k) { my_point[k] = row_point[3u * mine + k]; my_dir[k] = row_dir[3u * mine + k]; }
#pragma unroll
            for (int side = 0; side < 2; ++side) {
                if (my_link[side] == kInvalid) continue;
                const uint64_t mask = link_mask[my_link[side] - env * nl];
                my_mask[side][0] = uint32_t(mask); my_mask[side][1] = uint32_t(mask >> 32u);
            }
        }
        const uint32_t count = min(uint32_t(kWave), bound - first);
        for (uint32_t i = 0u; i < count; ++i) {
            const uint32_t r = first + i;
            const uint32_t links[2] = {uniform_word(my_link[0], i), uniform_word(my_link[1], i)};
            if (links[0] == kInvalid && links[1] == kInvalid) continue;
            const V3 point{uniform_value(my_point[0], i), uniform_value(my_point[1], i), uniform_value(my_point[2], i)};
            const V3 dir_a{uniform_value(my_dir[0], i), uniform_value(my_dir[1], i), uniform_value(my_dir[2], i)};
            float entries[2] = {0.0f, 0.0f};
#pragma unroll
            for (int side = 0; side < 2; ++side) {
                if (links[side] == kInvalid) continue;
                const uint64_t mask = (uint64_t(uniform_word(my_mask[side][1], i)) << 32u) | uint64_t(uniform_word(my_mask[side][0], i));
                const V3 dir = side == 0 ? dir_a : V3{-dir_a.x, -dir_a.y, -dir_a.z};
                // a turning coordinate (hinge, base angular) takes the moment of the direction about its axis, a sliding
                // one (prismatic, base linear) the direction along it: both evaluated, one selected, so that lanes of
                // different kinds do not take turns
                const float turning = dot3(cross3(axis_world, sub3(point, origin)), dir) + dot3(axis_world, V3{0, 0, 0});
                const float sliding = dot3(axis_world, dir);
                const bool on_path = lane < m.dof && ((mask >> lane) & 1ull) != 0ull;
                entries[side] = !on_path || mode == 0u ? 0.0f : ((mode & 1u) != 0u ? turning : sliding);
            }
            if (uniform_word(my_merge, i) != 0u) { entries[0] += entries[1]; entries[1] = 0.0f; }   // shared owner (:172-186)
            if (lane < md) {
                if (links[0] != kInvalid) d.chain_jacobian[(size_t{env} * R + r) * md + lane] = entries[0];
                if (links[1] != kInvalid) d.chain_jacobian_b[(size_t{env} * R + r) * md + lane] = entries[1];
            }
            // PrepareContactRowsKernel (:1134-1140): a compliant row's reference acceleration includes the damping of the
            // velocity the step started from along the row, ContactReferenceVelocity (:1072-1100): side A's coordinates
            // in order, then side B's
            const float gain = uniform_value(my_gain, i);
            if (gain != 0.0f) {
                float velocity = 0.0f;
                for (uint32_t side = 0u; side < 2u; ++side) {
                    if (links[side] == kInvalid) continue;
                    const float term = entries[side] * start_velocity;
                    for (uint32_t k = 0u; k < md; ++k) velocity += uniform_value(term, k);
                }
                if (lane == 0u) rows[r].rhs += gain * velocity;
            }
        }
    }
}

}  // namespace

Status OpSyncLinkBodyPose(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const SyncLinkBodyPoseParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->env_count == 0u || p->bodies_per_env == 0u) return Status::Ok;
    if (p->selected_env_count != 0u) return Status::Unsupported;
    const uint32_t total = p->env_count * p->bodies_per_env;
    hipLaunchKernelGGL(SyncLinkBodyPoseKernel, dim3((total + 255u) / 256u), dim3(256), 0, stream, m, d, total);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

Status OpBuildAabbs(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const BuildAabbsParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->env_count == 0u || p->bodies_per_env == 0u) return Status::Ok;
    const uint32_t total = p->env_count * p->bodies_per_env;
    hipLaunchKernelGGL(BuildAabbsKernel, dim3((total + 255u) / 256u), dim3(256), 0, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

// The pair query reads the body AABBs directly, so no tree is built (the reference skips its LBVH the same way for
// small worlds, broadphase.cu:581-582).
Status OpLbvhBuild(const ModelView&, const DataView&, const void* params, hipStream_t) {
    return params == nullptr ? Status::Failed : Status::Ok;
}

Status OpLbvhQueryPairs(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const LbvhQueryPairsParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->env_count == 0u) return Status::Ok;
    if (p->excluded_count != 0u) return Status::Unsupported;
    hipLaunchKernelGGL(QueryPairsKernel, dim3(p->env_count), dim3(kWave), 0, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

Status OpNarrowphasePrimitives(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const NarrowphasePrimitivesParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->env_count == 0u || p->union_slot_count == 0u || p->rigid_slot_cap == 0u) return Status::Ok;
    if (p->rigid_slot_cap <= 32u) {
        uint32_t width = 1u;
        while (width < p->rigid_slot_cap) width <<= 1u;
        const uint32_t blocks = (p->env_count + 64u / width - 1u) / (64u / width);
        if (m.max_points_per_slot <= 1u) hipLaunchKernelGGL(NarrowphasePackedKernel<true>, dim3(blocks), dim3(64), 0, stream, m, d, *p, width);
        else hipLaunchKernelGGL(NarrowphasePackedKernel<false>, dim3(blocks), dim3(64), 0, stream, m, d, *p, width);
    } else if (m.max_points_per_slot <= 1u) hipLaunchKernelGGL(NarrowphaseKernel<true>, dim3(p->env_count), dim3(64), 0, stream, m, d, *p);
    else hipLaunchKernelGGL(NarrowphaseKernel<false>, dim3(p->env_count), dim3(64), 0, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

// SyncLinkBodyPose, BuildAabbs, LbvhBuild (no tree is built on this path), LbvhQueryPairs and NarrowphasePrimitives as one
// launch; Unsupported when any of them would not run its kernel as dispatched, or the world has many-point manifolds.
Status OpCollisionHead(const ModelView& m, const DataView& d, const SyncLinkBodyPoseParams* bodies, const BuildAabbsParams* boxes,
                       const LbvhQueryPairsParams* query, const NarrowphasePrimitivesParams* narrow, hipStream_t stream) {
    if (bodies == nullptr || boxes == nullptr || query == nullptr || narrow == nullptr || m.max_points_per_slot > 1u) return Status::Unsupported;
    const uint32_t E = bodies->env_count, nb = m.bodies_per_env;
    if (E == 0u || nb == 0u || bodies->bodies_per_env != nb || bodies->selected_env_count != 0u || boxes->env_count != E ||
        boxes->bodies_per_env != nb || query->env_count != E || query->bodies_per_env != nb || query->excluded_count != 0u ||
        narrow->env_count != E || narrow->bodies_per_env != nb || narrow->union_slot_count == 0u || narrow->rigid_slot_cap == 0u)
        return Status::Unsupported;
    hipLaunchKernelGGL(CollisionHeadKernel, dim3(E), dim3(kWave), 0, stream, m, d, *boxes, *query, *narrow);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

Status OpNarrowphaseHeightfield(const ModelView&, const DataView&, const void* params, hipStream_t) {
    return params == nullptr ? Status::Ok : Status::Ok;   // no heightfield on this path: a no-op, as in the reference
}


Status OpAssembleRows(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const AssembleRowsParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->env_count == 0u || p->rows_per_env == 0u) return Status::Ok;
    if (p->max_dof > kMaxDof) return Status::InvalidArgument;
    const size_t lds = (size_t{p->union_slot_count} * 2u + size_t{p->contact_rows_per_env} * 10u + size_t{m.links_per_env} * 2u) * sizeof(uint32_t);
    if (lds > 150u * 1024u) return Status::InvalidArgument;
    hipLaunchKernelGGL(AssembleRowsKernel, dim3(p->env_count), dim3(kWave), lds, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

namespace {

// ---- ContactWarmStart (assemble_rows.cu:1393-1455): one wavefront per environment ------------------------------
// The reference indexes equal keys (pair, feature, material) through a hash table sized for the whole batch
// (contact_cache.cuh:167-284).  An environment holds at most a few hundred entries, so here a wavefront lists them
// in LDS (current points first, then cache entries, both in point order) and compares keys directly: the head of a
// key is its first entry, the warm point of a key is its lowest cache point that has not decayed.
struct CacheEntries {
    uint64_t* pair; uint64_t* feature; uint64_t* material;   // 2P each
    uint32_t* point;                                          // 2P: point index; cache entries carry bit 31
};
constexpr uint32_t kCacheFlag = 0x80000000u;

__device__ __forceinline__ uint32_t prefix_rank(uint64_t mask, uint32_t lane) { return uint32_t(__popcll(mask & ((uint64_t{1} << lane) - 1ull))); }

__device__ __forceinline__ bool row_offsets(const DataView& d, uint32_t env, uint32_t S, uint32_t slot, uint32_t point, uint32_t* rn,
                                            uint32_t* r1, uint32_t* r2) {
    const uint32_t first = d.ucontact_row_range[(size_t{env} * S + slot) * 2u], points = d.ucontact_row_range[(size_t{env} * S + slot) * 2u + 1u];
    if (point >= points) return false;
    *rn = first + point; *r1 = first + points + point; *r2 = first + 2u * points + point;
    return true;
}

// Phase 0: BuildIndex (contact_cache.cuh:286-338) and PrepareContactWarmStartKernel (assemble_rows.cu:1229-1272)
__global__ void __launch_bounds__(kWave) WarmStartPrepareKernel(DataView d, ContactWarmStartParams p) {
    extern __shared__ uint64_t lds64[];
    const uint32_t env = blockIdx.x, lane = threadIdx.x, S = p.slot_count, P = S * 4u;
    const size_t base = size_t{env} * P;
    CacheEntries e{lds64, lds64 + 2u * P, lds64 + 4u * P, reinterpret_cast<uint32_t*>(lds64 + 6u * P)};
    uint32_t count = 0u;
    for (uint32_t first = 0u; first < P; first += kWave) {   // current points that exist, in point order
        const uint32_t i = first + lane;
        const bool valid = i < P && (i & 3u) < d.ucontact_count[size_t{env} * S + i / 4u];
        if (i < P) { d.contact_cache_current_owner[base + i] = 0u; d.contact_cache_old_keep[base + i] = 0u; d.contact_cache_match[base + i] = kInvalid; }
        const uint64_t mask = __ballot(valid);
        if (valid) {
            const uint32_t at = count + prefix_rank(mask, lane);
            e.pair[at] = d.ucontact_id_pair[base + i]; e.feature[at] = d.ucontact_id_feature[base + i];
            e.material[at] = d.contact_material[size_t{env} * S + i / 4u]; e.point[at] = i;
        }
        count += uint32_t(__popcll(mask));
    }
    const uint32_t current_count = count;
    for (uint32_t first = 0u; first < P; first += kWave) {   // cache entries, in point order
        const uint32_t j = first + lane;
        const bool valid = j < P && d.contact_cache_pair[base + j] != 0ull;
        const uint64_t mask = __ballot(valid);
        if (valid) {
            const uint32_t at = count + prefix_rank(mask, lane);
            e.pair[at] = d.contact_cache_pair[base + j]; e.feature[at] = d.contact_cache_feature[base + j];
            e.material[at] = d.contact_cache_material[base + j]; e.point[at] = j | kCacheFlag;
        }
        count += uint32_t(__popcll(mask));
    }
    __syncthreads();
    uint32_t owned = 0u, matched = 0u;
    for (uint32_t k = lane; k < count; k += kWave) {
        const uint64_t pair = e.pair[k], feature = e.feature[k], material = e.material[k];
        bool head = true;
        for (uint32_t earlier = 0u; earlier < k && head; ++earlier)
            head = !(e.pair[earlier] == pair && e.feature[earlier] == feature && e.material[earlier] == material);
        const uint32_t tagged = e.point[k];
        if ((tagged & kCacheFlag) == 0u) {
            const uint32_t i = tagged;
            uint32_t warm = kInvalid;
            if (head)
                for (uint32_t other = current_count; other < count; ++other) {
                    const uint32_t point = e.point[other] & ~kCacheFlag;
                    if (e.pair[other] == pair && e.feature[other] == feature && e.material[other] == material &&
                        d.contact_cache_age[base + point] < p.decay_steps && point < warm) warm = point;
                }
            d.contact_cache_match[base + i] = warm;
            if (warm != kInvalid) {
                const float* n = d.ucontact_normal + 3u * (base + i);
                const float* o = d.contact_cache_normal + 3u * (base + warm);
                if (n[0] * o[0] + n[1] * o[1] + n[2] * o[2] > 0.25f) ++matched;
            }
            if (head) { d.contact_cache_current_owner[base + i] = 1u; owned = max(owned, i + 1u); }
        } else if (head && p.decay_steps > 1u && d.contact_cache_age[base + (tagged & ~kCacheFlag)] < p.decay_steps - 1u) {
            d.contact_cache_old_keep[base + (tagged & ~kCacheFlag)] = 1u;
        }
    }
    owned = wave_max_u(owned);
    matched = wave_sum_u(matched);
    if (lane == 0u) {
        d.contact_cache_extent[2u * env + 1u] = owned;
        d.contact_warm_start_counts[2u * env] = current_count;
        d.contact_warm_start_counts[2u * env + 1u] = matched;
    }
    __syncthreads();   // this block's match writes are read back below
    // rows of matched points whose normal has kept its side start from the cached impulse, the tangential part carried
    // over in the world frame
    for (uint32_t i = lane; i < P; i += kWave) {
        const uint32_t match = d.contact_cache_match[base + i];
        if (match == kInvalid) continue;
        const V3 n{d.ucontact_normal[3u * (base + i)], d.ucontact_normal[3u * (base + i) + 1u], d.ucontact_normal[3u * (base + i) + 2u]};
        const V3 o{d.contact_cache_normal[3u * (base + match)], d.contact_cache_normal[3u * (base + match) + 1u],
                   d.contact_cache_normal[3u * (base + match) + 2u]};
        if (n.x * o.x + n.y * o.y + n.z * o.z <= 0.25f) continue;
        uint32_t rn, r1, r2;
        if (!row_offsets(d, env, S, i / 4u, i & 3u, &rn, &r1, &r2)) continue;
        const float* cached = d.contact_cache_lambda + 4u * (base + match);
        V3 ot1, ot2, t1, t2;
        contact_tangent_basis(o, &ot1, &ot2);
        contact_tangent_basis(n, &t1, &t2);
        const V3 old = add3(scale3(ot1, cached[1]), scale3(ot2, cached[2]));
        d.lambda[rn] = fmaxf(cached[0], 0.0f);
        d.lambda[r1] = dot3(old, t1);
        d.lambda[r2] = dot3(old, t2);
    }
}

// Phase 1: BuildRanks, CacheExtentKernel (contact_cache.cuh:340-365) and RebuildContactCacheKernel
// (assemble_rows.cu:1313-1391).  The retained old entries are copied to LDS before the cache is rewritten.
__global__ void __launch_bounds__(kWave) WarmStartCommitKernel(DataView d, ContactWarmStartParams p) {
    extern __shared__ uint64_t lds64[];
    const uint32_t env = blockIdx.x, lane = threadIdx.x, S = p.slot_count, P = S * 4u;
    const size_t base = size_t{env} * P;
    uint64_t* kept_pair = lds64, *kept_feature = lds64 + P, *kept_material = lds64 + 2u * P;
    float* kept_float = reinterpret_cast<float*>(lds64 + 3u * P);         // 7 per entry: impulse 4, normal 3
    uint32_t* kept_age = reinterpret_cast<uint32_t*>(kept_float + 7u * P);
    uint32_t* free_rank = kept_age + P;                                      // free points before each point
    uint32_t retained = 0u, unowned = 0u;
    for (uint32_t first = 0u; first < P; first += kWave) {
        const uint32_t i = first + lane;
        const bool keep = i < P && d.contact_cache_old_keep[base + i] != 0u;
        const bool is_free = i < P && d.contact_cache_current_owner[base + i] == 0u;
        const uint64_t keep_mask = __ballot(keep), free_mask = __ballot(is_free);
        if (i < P) free_rank[i] = unowned + prefix_rank(free_mask, lane);
        if (keep) {
            const uint32_t at = retained + prefix_rank(keep_mask, lane);
            kept_pair[at] = d.contact_cache_pair[base + i]; kept_feature[at] = d.contact_cache_feature[base + i];
            kept_material[at] = d.contact_cache_material[base + i];
#pragma unroll
            for (int k = 0; k < 4; ++k) kept_float[7u * at + k] = d.contact_cache_lambda[4u * (base + i) + k];
#pragma unroll
            for (int k = 0; k < 3; ++k) kept_float[7u * at + 4 + k] = d.contact_cache_normal[3u * (base + i) + k];
            kept_age[at] = d.contact_cache_age[base + i];
        }
        retained += uint32_t(__popcll(keep_mask));
        unowned += uint32_t(__popcll(free_mask));
    }
    const uint32_t extent_previous = d.contact_cache_extent[2u * env], extent_current = d.contact_cache_extent[2u * env + 1u];
    const uint32_t previous = extent_previous == 0u ? P : min(extent_previous - 1u, P);
    const uint32_t next = min(max(extent_current, P - unowned + retained), P);
    const uint32_t bound = min(max(previous, next), P);
    __syncthreads();
    if (lane == 0u) { d.contact_cache_extent[2u * env] = next + 1u; d.contact_cache_extent[2u * env + 1u] = max(previous, next); }
    for (uint32_t i = lane; i < bound; i += kWave) {
        uint32_t rn, r1, r2;
        if (d.contact_cache_current_owner[base + i] != 0u && row_offsets(d, env, S, i / 4u, i & 3u, &rn, &r1, &r2)) {
            const uint32_t stride = r1 - rn;
            d.contact_cache_pair[base + i] = d.ucontact_id_pair[base + i];
            d.contact_cache_feature[base + i] = d.ucontact_id_feature[base + i];
#pragma unroll
            for (uint32_t k = 0u; k < 4u; ++k) d.contact_cache_lambda[4u * (base + i) + k] = k < 3u ? d.lambda[rn + k * stride] : 0.0f;
#pragma unroll
            for (int k = 0; k < 3; ++k) d.contact_cache_normal[3u * (base + i) + k] = d.ucontact_normal[3u * (base + i) + k];
            d.contact_cache_material[base + i] = d.contact_material[size_t{env} * S + i / 4u];
            d.contact_cache_age[base + i] = 0u;
            continue;
        }
        const uint32_t rank = free_rank[i];
        if (rank < retained) {
            d.contact_cache_pair[base + i] = kept_pair[rank]; d.contact_cache_feature[base + i] = kept_feature[rank];
            d.contact_cache_material[base + i] = kept_material[rank];
#pragma unroll
            for (int k = 0; k < 4; ++k) d.contact_cache_lambda[4u * (base + i) + k] = kept_float[7u * rank + k];
#pragma unroll
            for (int k = 0; k < 3; ++k) d.contact_cache_normal[3u * (base + i) + k] = kept_float[7u * rank + 4 + k];
            d.contact_cache_age[base + i] = kept_age[rank] + 1u;
            continue;
        }
        d.contact_cache_pair[base + i] = 0ull; d.contact_cache_feature[base + i] = 0ull; d.contact_cache_material[base + i] = 0ull;
#pragma unroll
        for (int k = 0; k < 4; ++k) d.contact_cache_lambda[4u * (base + i) + k] = 0.0f;
#pragma unroll
        for (int k = 0; k < 3; ++k) d.contact_cache_normal[3u * (base + i) + k] = 0.0f;
        d.contact_cache_age[base + i] = 0u;
    }
}

}  // namespace

Status OpContactWarmStart(const ModelView&, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const ContactWarmStartParams*>(params);
    if (p == nullptr || p->phase > 1u) return Status::InvalidArgument;
    if (p->slot_count == 0u || p->env_count == 0u) return Status::Ok;
    const size_t points = size_t{p->slot_count} * 4u;
    if (p->phase == 0u) {
        const size_t lds = points * (6u * sizeof(uint64_t) + 2u * sizeof(uint32_t));
        if (lds > 150u * 1024u) return Status::InvalidArgument;
        hipLaunchKernelGGL(WarmStartPrepareKernel, dim3(p->env_count), dim3(kWave), lds, stream, d, *p);
    } else {
        const size_t lds = points * (3u * sizeof(uint64_t) + 7u * sizeof(float) + 2u * sizeof(uint32_t));
        if (lds > 150u * 1024u) return Status::InvalidArgument;
        hipLaunchKernelGGL(WarmStartCommitKernel, dim3(p->env_count), dim3(kWave), lds, stream, d, *p);
    }
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

namespace {
// ReadoutContactWrench (ops/readout.cu:59-220, 559-626): per contact slot the first manifold point and normal, the
// summed {normal, tangent, tangent} force, each point's world impulse, the two sides' owners and the contact's link;
// per link the world-frame wrench of every active row ending on it.  One wavefront per environment.  The reference
// sorts (link, row, side) keys to list a link's endpoints; here a lane per link walks the environment's rows in that
// same order - ascending row, side A before B - so the sums add in the same sequence.
__global__ void __launch_bounds__(kWave) ReadoutContactWrenchKernel(ModelView m, DataView d, ReadoutContactWrenchParams p) {
    const uint32_t env = blockIdx.x, lane = threadIdx.x;
    const uint32_t S = p.max_contacts_per_env, R = p.rows_per_env, nl = p.base_link_count;
    const float inv_dt = p.dt > 0.0f ? 1.0f / p.dt : 0.0f;
    const Row* rows = reinterpret_cast<const Row*>(d.urows);
    for (uint32_t s = lane; s < S; s += kWave) {
        const size_t slot = size_t{env} * S + s;
        const uint32_t points = d.ucontact_count[slot];
        for (uint32_t k = 0u; k < 3u; ++k) {   // LegacyContactGeometryKernel :59-77
            d.contact_point[slot * 3u + k] = points > 0u ? d.ucontact_point[slot * 12u + k] : 0.0f;
            d.contact_normal[slot * 3u + k] = points > 0u ? d.ucontact_normal[slot * 12u + k] : 0.0f;
        }
        const uint32_t first = d.ucontact_row_range[slot * 2u], pts = d.ucontact_row_range[slot * 2u + 1u];   // ContactForceKernel :80-123
        float fn = 0.0f, ft1 = 0.0f, ft2 = 0.0f;
        for (uint32_t i = 0u; i < pts; ++i) {
            fn += d.lambda[first + i]; ft1 += d.lambda[first + i + pts]; ft2 += d.lambda[first + i + 2u * pts];
        }
        for (uint32_t i = 0u; i < kPointsPerSlot; ++i) {   // ContactPointWorldImpulse, nk/contact/row_readout.hpp:38-48
            V3 impulse{0.0f, 0.0f, 0.0f};
            if (i < pts && (rows[first + i].flags & kRowActive) != 0u)
                for (uint32_t axis = 0u; axis < 3u; ++axis) {
                    const uint32_t index = first + i + axis * pts;
                    const float l = d.lambda[index];
                    impulse.x += rows[index].a.jlin.x * l; impulse.y += rows[index].a.jlin.y * l; impulse.z += rows[index].a.jlin.z * l;
                }
            float* out = d.ucontact_impulse + (slot * kPointsPerSlot + i) * 3u;
            out[0] = impulse.x; out[1] = impulse.y; out[2] = impulse.z;
        }
        d.contact_force[slot * 3u] = fn * inv_dt; d.contact_force[slot * 3u + 1u] = ft1 * inv_dt; d.contact_force[slot * 3u + 2u] = ft2 * inv_dt;
        const bool active = pts > 0u && (rows[first].flags & kRowActive) != 0u;
        const uint32_t kind_a = active ? rows[first].a.kind : uint32_t(kSideStatic), kind_b = active ? rows[first].b.kind : uint32_t(kSideStatic);
        d.contact_side_a_kind[slot] = kind_a; d.contact_side_b_kind[slot] = kind_b;
        d.contact_side_a_index[slot] = !active || kind_a == kSideStatic ? kInvalid : kind_a == kSideArtic ? d.row_cj_link[first] : rows[first].a.index;
        d.contact_side_b_index[slot] = !active || kind_b == kSideStatic ? kInvalid : kind_b == kSideArtic ? d.row_cj_link_b[first] : rows[first].b.index;
        uint32_t link = kInvalid;   // ContactLinkKernel :127-149
        for (uint32_t i = 0u; i < pts && link == kInvalid; ++i) link = d.row_cj_link[first + i];
        for (uint32_t i = 0u; i < pts && link == kInvalid; ++i) link = d.row_cj_link_b[first + i];
        d.contact_link[slot] = link;
    }
    // LinkContactWrenchKernel :154-220
    const uint32_t previous = d.contact_row_extent[2u * env], current = d.contact_row_extent[2u * env + 1u];
    const uint32_t bound = contact_row_bound(previous, current, p.contact_rows_per_env);
    for (uint32_t base = 0u; base < nl; base += kWave) {
        const uint32_t l = base + lane;
        const uint32_t link = env * nl + l;
        V3 origin{0.0f, 0.0f, 0.0f}, force{0.0f, 0.0f, 0.0f}, torque{0.0f, 0.0f, 0.0f};
        if (l < nl) origin = V3{d.link_pose[size_t{link} * 7u], d.link_pose[size_t{link} * 7u + 1u], d.link_pose[size_t{link} * 7u + 2u]};
        for (uint32_t r = 0u; r < bound; ++r) {
            const size_t rs = size_t{env} * R + r;
            if ((rows[rs].flags & kRowActive) == 0u) continue;
            const uint32_t ends[2] = {d.row_cj_link[rs], d.row_cj_link_b[rs]};
            const float scale = d.lambda[rs] * inv_dt;
            for (uint32_t side = 0u; side < 2u; ++side) {
                if (l >= nl || ends[side] != link) continue;
                const V3 dir = side == 0u ? rows[rs].a.jlin : rows[rs].b.jlin;
                const float* point = (side == 0u ? d.row_cj_point : d.row_cj_point_b) + rs * 3u;
                const V3 f{dir.x * scale, dir.y * scale, dir.z * scale};
                const V3 moment = cross3(sub3(V3{point[0], point[1], point[2]}, origin), f);
                force = V3{force.x + f.x, force.y + f.y, force.z + f.z};
                torque = V3{torque.x + moment.x, torque.y + moment.y, torque.z + moment.z};
            }
        }
        if (l < nl) {
            float* out = d.link_contact_wrench + size_t{link} * 6u;
            out[0] = force.x; out[1] = force.y; out[2] = force.z; out[3] = torque.x; out[4] = torque.y; out[5] = torque.z;
        }
    }
}
}  // namespace

Status OpReadoutContactWrench(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const ReadoutContactWrenchParams*>(params);
    if (p == nullptr) return Status::InvalidArgument;
    if (p->full_row_slot_count > p->max_contacts_per_env || p->contact_rows_per_env > p->rows_per_env) return Status::InvalidArgument;
    if (p->env_count == 0u || p->max_contacts_per_env == 0u) return Status::Ok;
    hipLaunchKernelGGL(ReadoutContactWrenchKernel, dim3(p->env_count), dim3(kWave), 0, stream, m, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

namespace {
// AccumulateStepKernel (ops/readout.cu:222-300), the outputs of a step of several substeps: status words are or-ed,
// joint limit impulses summed, the links' contact wrenches averaged as impulses and moments about the world origin
// over the whole step, and the applied link wrenches cleared after the last substep.  One thread per link.
__global__ void __launch_bounds__(256) AccumulateStepKernel(DataView d, AccumulateStepParams p) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t links = p.env_count * p.links_per_env;
    if (i < p.env_count) {
        const uint32_t status = d.env_status[i];
        const uint32_t combined = p.first != 0u ? status : d.step_env_status[i] | status;
        d.step_env_status[i] = combined;
        if (p.last != 0u) d.env_status[i] = combined;
    }
    if (i >= links) return;
    if ((p.flags & kAccumulateLinkWrench) != 0u) {
        float* wrench = d.link_contact_wrench + size_t{i} * 6u;
        const V3 impulse = scale3(V3{wrench[0], wrench[1], wrench[2]}, p.substep_dt);
        const V3 origin{d.link_pose[size_t{i} * 7u], d.link_pose[size_t{i} * 7u + 1u], d.link_pose[size_t{i} * 7u + 2u]};
        const V3 moment = add3(scale3(V3{wrench[3], wrench[4], wrench[5]}, p.substep_dt), cross3(origin, impulse));
        float* sum_impulse = d.step_link_impulse + size_t{i} * 3u, *sum_moment = d.step_link_moment + size_t{i} * 3u;
        V3 total_impulse = impulse, total_moment = moment;
        if (p.first == 0u) {
            total_impulse = add3(V3{sum_impulse[0], sum_impulse[1], sum_impulse[2]}, impulse);
            total_moment = add3(V3{sum_moment[0], sum_moment[1], sum_moment[2]}, moment);
        }
        sum_impulse[0] = total_impulse.x; sum_impulse[1] = total_impulse.y; sum_impulse[2] = total_impulse.z;
        sum_moment[0] = total_moment.x; sum_moment[1] = total_moment.y; sum_moment[2] = total_moment.z;
        if (p.last != 0u) {
            const V3 force = scale3(total_impulse, p.inv_outer_dt);
            const V3 torque = scale3(sub3(total_moment, cross3(origin, total_impulse)), p.inv_outer_dt);
            wrench[0] = force.x; wrench[1] = force.y; wrench[2] = force.z; wrench[3] = torque.x; wrench[4] = torque.y; wrench[5] = torque.z;
        }
    }
    if ((p.flags & kAccumulateJointLimit) != 0u) {
        for (uint32_t side = 0u; side < 2u; ++side) {
            const size_t slot = size_t{i} * 2u + side;
            const float impulse = d.joint_limit_impulse[slot];
            const float total = p.first != 0u ? impulse : d.step_joint_limit_impulse[slot] + impulse;
            d.step_joint_limit_impulse[slot] = total;
            if (p.last != 0u) d.joint_limit_impulse[slot] = total;
        }
    }
    if (p.last != 0u && (p.flags & kFinalizeLinkWrench) != 0u)
        for (uint32_t k = 0u; k < 6u; ++k) d.link_wrench[size_t{i} * 6u + k] = 0.0f;
}
}  // namespace

Status OpAccumulateStep(const ModelView&, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const AccumulateStepParams*>(params);
    if (p == nullptr || (p->flags & ~(kAccumulateOutputs | kAccumulateLinkWrench | kAccumulateJointLimit | kFinalizeLinkWrench)) != 0u ||
        (p->flags & kAccumulateOutputs) == 0u) return Status::InvalidArgument;
    const uint32_t count = p->env_count * (p->links_per_env > 0u ? p->links_per_env : 1u);
    if (count == 0u) return Status::Ok;
    hipLaunchKernelGGL(AccumulateStepKernel, dim3((count + 255u) / 256u), dim3(256), 0, stream, d, *p);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

namespace {
// PackQdotFlatMultiKernel (assemble_rows.cu:200-214) into step_qdot_flat
__global__ void __launch_bounds__(256) SnapshotStepVelocityKernel(ModelView m, DataView d, uint32_t env_count) {
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= env_count * m.max_dof) return;
    const uint32_t env = gid / m.max_dof, dof = gid - env * m.max_dof;
    float value = 0.0f;
    if (dof < m.dof && m.free_body != 0u) {   // a free body's six coordinates as its state holds them: linear, then angular velocity
        const size_t body = size_t{env} * m.bodies_per_env + m.link_body[0];
        value = dof < 3u ? d.body_linear_velocity[body * 3u + dof] : d.body_angular_velocity[body * 3u + dof - 3u];
    } else if (dof < m.dof) {
        const uint32_t link = m.dof_link[dof], component = m.dof_component[dof];
        value = component == kInvalid ? d.qdot[size_t{env} * m.links_per_env + link]
                                      : d.link_velocity[(size_t{env} * m.links_per_env + link) * 6u + component];
    }
    d.step_qdot_flat[gid] = value;
}
}  // namespace

// SnapshotStepVelocity (assemble_rows.cu:1457-1477): the generalized velocity the step starts from.  Only the
// compliant rows of the MuJoCo law read it (PrepareContactRowsKernel :1134-1140) and the damping a MuJoCo integrator
// applies after the solve, so a world with neither has nothing to record.
Status OpSnapshotStepVelocity(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const SnapshotStepVelocityParams*>(params);
    if (p == nullptr || p->env_count == 0u) return Status::Failed;
    if ((m.any_mujoco == 0u && m.integrator == 0u) || m.max_dof == 0u) return Status::Ok;
    if (p->max_dof != m.max_dof) return Status::InvalidArgument;
    const uint32_t total = p->env_count * m.max_dof;
    hipLaunchKernelGGL(SnapshotStepVelocityKernel, dim3((total + 255u) / 256u), dim3(256), 0, stream, m, d, p->env_count);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

void InitContactKernels() {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(AssembleRowsKernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    (void)hipGetLastError();
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(WarmStartPrepareKernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    (void)hipGetLastError();
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(WarmStartCommitKernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    (void)hipGetLastError();
}

}  // namespace nkh
