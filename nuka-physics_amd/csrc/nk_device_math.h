// Device-side small-vector, quaternion and 6-D spatial helpers for the gfx950 kernels.
// Operation order follows src/math/cuda_vec_ops.cuh and src/math/cuda_spatial_ops.cuh (left-to-right sums)
// so results stay within a few ulp of a serial evaluation of the same formulas.
#pragma once

#include <hip/hip_runtime.h>

#include <cfloat>
#include <cstdint>

namespace nkh {

struct V3 { float x, y, z; };
struct Q4 { float w, x, y, z; };
struct Xf { V3 p; Q4 r; };

__device__ __forceinline__ V3 mk3(float x, float y, float z) { return V3{x, y, z}; }
__device__ __forceinline__ V3 add3(V3 a, V3 b) { return V3{a.x + b.x, a.y + b.y, a.z + b.z}; }
__device__ __forceinline__ V3 sub3(V3 a, V3 b) { return V3{a.x - b.x, a.y - b.y, a.z - b.z}; }
__device__ __forceinline__ V3 scale3(V3 a, float s) { return V3{a.x * s, a.y * s, a.z * s}; }
__device__ __forceinline__ float dot3(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
__device__ __forceinline__ V3 cross3(V3 a, V3 b) {
    return V3{a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
// Full-precision reciprocal square root: v_rsq_f32 alone is 1 ulp-approximate, sqrt then divide is exact-rounded.
__device__ __forceinline__ float rsqrt_exact(float x) { return 1.0f / sqrtf(x); }

// Correctly rounded square root and quotient for operands in the normal range, without the range scaling, special-value
// fix-ups and second reciprocal that the general sqrtf and operator/ carry.  sqrt_rn_normal corrects v_sqrt_f32 (at
// most one ulp off) by the residuals of its two neighbours; make_recip / div_by are the Newton reciprocal and the two
// quotient corrections of the general division, so one reciprocal serves every quotient with the same divisor.  Both
// give the bits of sqrtf and a / b whenever |x|, |a|, |b| and the result lie between 2^-90 and 2^90 (compared on the
// device over 5e8 random operands each); outside that range they stay within an ulp.
__device__ __forceinline__ float sqrt_rn_normal(float x) {
    const float s = __builtin_amdgcn_sqrtf(x);
    const float down = __uint_as_float(__float_as_uint(s) - 1u), up = __uint_as_float(__float_as_uint(s) + 1u);
    const float below = fmaf(-down, s, x), above = fmaf(-up, s, x);
    float root = below <= 0.0f ? down : s;
    root = above > 0.0f ? up : root;
    return root;
}
struct Recip { float divisor, value; };
__device__ __forceinline__ Recip make_recip(float divisor) {
    float r = __builtin_amdgcn_rcpf(divisor);
    const float e = fmaf(-divisor, r, 1.0f);
    r = fmaf(e, r, r);
    return Recip{divisor, r};
}
__device__ __forceinline__ float div_by(float a, Recip d) {
    float q = a * d.value;
    float e = fmaf(-d.divisor, q, a);
    q = fmaf(e, d.value, q);
    e = fmaf(-d.divisor, q, a);
    return fmaf(e, d.value, q);
}

__device__ __forceinline__ Xf load_xf(const float* p) { return Xf{V3{p[0], p[1], p[2]}, Q4{p[3], p[4], p[5], p[6]}}; }
__device__ __forceinline__ void store_xf(float* p, Xf t) {
    p[0] = t.p.x; p[1] = t.p.y; p[2] = t.p.z; p[3] = t.r.w; p[4] = t.r.x; p[5] = t.r.y; p[6] = t.r.z;
}

// cuda_vec_ops.cuh:207-213
__device__ __forceinline__ Q4 qmul(Q4 a, Q4 b) {
    return Q4{a.w * b.w - a.x * b.x - a.y * b.y - a.z * b.z, a.w * b.x + a.x * b.w + a.y * b.z - a.z * b.y,
              a.w * b.y - a.x * b.z + a.y * b.w + a.z * b.x, a.w * b.z + a.x * b.y - a.y * b.x + a.z * b.w};
}
// cuda_vec_ops.cuh:254-261 (branch norm_sq <= eps)
__device__ __forceinline__ Q4 qnormalize_le(Q4 q, float eps) {
    const float n = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (n <= eps) return Q4{1.0f, 0.0f, 0.0f, 0.0f};
    const float inv = rsqrt_exact(n);
    return Q4{q.w * inv, q.x * inv, q.y * inv, q.z * inv};
}
// cuda_vec_ops.cuh:263-284 (strict branch)
__device__ __forceinline__ Q4 qnormalize_lt(Q4 q, float eps) {
    const float n = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (n < eps) return Q4{1.0f, 0.0f, 0.0f, 0.0f};
    const float inv = rsqrt_exact(n);
    return Q4{q.w * inv, q.x * inv, q.y * inv, q.z * inv};
}
__device__ __forceinline__ Q4 qunit_guard(Q4 q) {
    const float n = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
    if (n > 1.0e-12f) {
        const float inv = rsqrt_exact(n);
        q.w *= inv; q.x *= inv; q.y *= inv; q.z *= inv;
    }
    return q;
}
// cuda_vec_ops.cuh:297-312: v + w*(2 qv x v) + qv x (2 qv x v), component sums left to right
__device__ __forceinline__ V3 rotate_normalized(Q4 q, V3 v) {
    q = qunit_guard(q);
    const V3 qv{q.x, q.y, q.z};
    const V3 t = cross3(qv, v);
    const V3 t2{2.0f * t.x, 2.0f * t.y, 2.0f * t.z};
    const V3 wt{q.w * t2.x, q.w * t2.y, q.w * t2.z};
    const V3 qvt = cross3(qv, t2);
    return V3{v.x + wt.x + qvt.x, v.y + wt.y + qvt.y, v.z + wt.z + qvt.z};
}
// articulation.cu:220-233 / 709-721: v + (w t + qv x t), t = 2 (qv x v)
__device__ __forceinline__ V3 rotate_inverse(Q4 q, V3 v) {
    q = qunit_guard(q);
    const V3 qv{-q.x, -q.y, -q.z};
    const V3 t = scale3(cross3(qv, v), 2.0f);
    return add3(v, add3(scale3(t, q.w), cross3(qv, t)));
}
__device__ __forceinline__ V3 rotate_forward(Q4 q, V3 v) {
    q = qunit_guard(q);
    const V3 qv{q.x, q.y, q.z};
    const V3 t = scale3(cross3(qv, v), 2.0f);
    return add3(v, add3(scale3(t, q.w), cross3(qv, t)));
}
// prims_types.cuh:92-96 (no normalisation): (v + w t) + qv x t
__device__ __forceinline__ V3 rotate_raw(Q4 q, V3 v) {
    const V3 qv{q.x, q.y, q.z};
    const V3 t = scale3(cross3(qv, v), 2.0f);
    return add3(add3(v, scale3(t, q.w)), cross3(qv, t));
}
// articulation.cu:1136-1158 FK composition
__device__ __forceinline__ Xf compose_frame(Xf parent, Xf local) {
    const Q4 q = qunit_guard(parent.r);
    const V3 qv{q.x, q.y, q.z};
    const V3 t = scale3(cross3(qv, local.p), 2.0f);
    const V3 wt = scale3(t, q.w);
    const V3 qvt = cross3(qv, t);
    Xf out;
    out.p = add3(parent.p, add3(add3(local.p, wt), qvt));
    out.r = qnormalize_le(qmul(parent.r, local.r), 1.0e-12f);
    return out;
}
// collision/analytical_manifold.hpp:130-171 collidable pose composition (rotation product left unnormalised)
__device__ __forceinline__ Xf compose_collidable(Xf parent, Xf child) {
    const Q4 q = qunit_guard(parent.r);
    const V3 qv{q.x, q.y, q.z}, v = child.p;
    const V3 t{2.0f * (qv.y * v.z - qv.z * v.y), 2.0f * (qv.z * v.x - qv.x * v.z), 2.0f * (qv.x * v.y - qv.y * v.x)};
    const V3 qvt = cross3(qv, t);
    Xf out;
    out.p = add3(parent.p, V3{v.x + q.w * t.x + qvt.x, v.y + q.w * t.y + qvt.y, v.z + q.w * t.z + qvt.z});
    out.r = qmul(parent.r, child.r);
    return out;
}

// ---- 6-D spatial algebra on flat arrays, [angular; linear], 6x6 row-major ----
__device__ __forceinline__ void mat66_vec(const float* m, const float* v, float* out) {
#pragma unroll
    for (int r = 0; r < 6; ++r) {
        float value = 0.0f;
#pragma unroll
        for (int c = 0; c < 6; ++c) value += m[r * 6 + c] * v[c];
        out[r] = value;
    }
}
__device__ __forceinline__ void mat66t_vec(const float* m, const float* v, float* out) {
#pragma unroll
    for (int r = 0; r < 6; ++r) {
        float value = 0.0f;
#pragma unroll
        for (int c = 0; c < 6; ++c) value += m[c * 6 + r] * v[c];
        out[r] = value;
    }
}
__device__ __forceinline__ float dot6(const float* a, const float* b) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 6; ++i) s += a[i] * b[i];
    return s;
}
__device__ __forceinline__ void motion_cross(const float* l, const float* r, float* out) {
    const V3 lw{l[0], l[1], l[2]}, lv{l[3], l[4], l[5]}, rw{r[0], r[1], r[2]}, rv{r[3], r[4], r[5]};
    const V3 ang = cross3(lw, rw), lin = add3(cross3(lw, rv), cross3(lv, rw));
    out[0] = ang.x; out[1] = ang.y; out[2] = ang.z; out[3] = lin.x; out[4] = lin.y; out[5] = lin.z;
}
__device__ __forceinline__ void force_cross(const float* m, const float* f, float* out) {
    const V3 w{m[0], m[1], m[2]}, v{m[3], m[4], m[5]}, n{f[0], f[1], f[2]}, ff{f[3], f[4], f[5]};
    const V3 ang = add3(cross3(w, n), cross3(v, ff)), lin = cross3(w, ff);
    out[0] = ang.x; out[1] = ang.y; out[2] = ang.z; out[3] = lin.x; out[4] = lin.y; out[5] = lin.z;
}

__device__ __forceinline__ uint32_t joint_dof(uint8_t type) {
    return type <= 1u ? 1u : type == 3u ? 6u : type == 4u ? 3u : 0u;
}

// 64-lane wave helpers.  Reductions run inside each row of 16 lanes with DPP moves (lane^1, lane^2, mirror of 8,
// mirror of 16: every step pairs lanes that already hold equal partial results, so a commutative combine leaves all
// 16 lanes equal), then the four row results are read as scalars and combined as (r0 + r1) + (r2 + r3).  The result
// is uniform across the wave.
__device__ __forceinline__ float wave_bcast(float v, int lane) { return __shfl(v, lane, 64); }
template <int Ctrl>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), Ctrl, 0xF, 0xF, false));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;
__device__ __forceinline__ float row_value(float v, int row) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16 * row));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<kDppXor1>(v)); v = fmaxf(v, dpp_move<kDppXor2>(v));
    v = fmaxf(v, dpp_move<kDppHalfMirror>(v)); v = fmaxf(v, dpp_move<kDppMirror>(v));
    return fmaxf(fmaxf(row_value(v, 0), row_value(v, 1)), fmaxf(row_value(v, 2), row_value(v, 3)));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<kDppXor1>(v); v += dpp_move<kDppXor2>(v); v += dpp_move<kDppHalfMirror>(v); v += dpp_move<kDppMirror>(v);
    return (row_value(v, 0) + row_value(v, 1)) + (row_value(v, 2) + row_value(v, 3));
}
__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ uint32_t wave_max_u(uint32_t v) {
    // non-negative floats order like their bit patterns, and every caller passes such bits or small counts
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { const uint32_t other = __shfl_xor(v, o, 64); v = other > v ? other : v; }
    return v;
}
__device__ __forceinline__ uint32_t wave_or_u(uint32_t v) {   // uniform result
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v |= uint32_t(__shfl_xor(int(v), o, 64));
    return uint32_t(__builtin_amdgcn_readfirstlane(int(v)));
}
__device__ __forceinline__ uint32_t wave_sum_u(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += uint32_t(__shfl_xor(int(v), o, 64));
    return v;
}
// A lane's value of `v` for a lane index that is a compile-time constant at every call site: a scalar lane read.
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
// Lane predicates (lane == k, lane > j, ...) of fully unrolled loops are loop invariant; hoisted out of the enclosing
// loops they would occupy hundreds of scalar registers and spill.  Passing the lane index through this makes each
// use site compute its own predicate where it needs it.
__device__ __forceinline__ uint32_t local_lane(uint32_t lane) {
    asm volatile("" : "+v"(lane));
    return lane;
}
// The value itself, through a barrier the optimiser cannot look across: what is computed from it stays where it is
// written instead of being hoisted out of the enclosing loops.
__device__ __forceinline__ float opaque(float v) {
    asm volatile("" : "+v"(v));
    return v;
}
// The same for a value that does not change over a loop, tied to one that does (`with`): what is computed from the
// result cannot leave the loop, and since the statement has no side effect of its own it orders nothing - reads and
// arithmetic around it are scheduled freely, where the plain barrier above keeps every memory access on its side.
__device__ __forceinline__ float opaque_with(float v, float with) {
    asm("" : "+v"(v) : "v"(with));
    return v;
}
__device__ __forceinline__ uint32_t opaque_word(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}
__device__ __forceinline__ bool wave_all(bool p) { return __all(p); }
__device__ __forceinline__ bool wave_any(bool p) { return __any(p); }

}  // namespace nkh
