// UABD block-descent contact solve for gfx950.  One 64-lane wavefront owns one environment for the whole solve:
// every velocity sweep, the dual updates and the split-impulse position pass run in a single launch with the
// staged Jacobian rows and per-head state resident in LDS.  A lane is a block coordinate in the matrix phases and
// owns one matrix row IN REGISTERS: the kernel is compiled per padded width N (a multiple of 4, nv <= N <= 64), the
// mass row, the Newton Hessian row and its Cholesky factor row are fully unrolled register arrays, pivots and
// multipliers travel between lanes as scalar lane reads, and LDS only carries what must be read transposed (the
// factor columns of the backward substitution) or broadcast (Jacobian rows, small vectors, read as 16-byte words).
// The mass matrix is constant over a solve, so its factor is built once.  A lane is a head row in the per-head
// phases.  Sums that the reference carries as compensated two-float pairs are double accumulators here (a double
// multiply-add issues at the rate of a float one on this device); nothing is exchanged between environments.
// Two instantiations go beyond the plain block.  A reduced block (template argument K < N) eliminates, once per
// solve, the coordinates from K on that no contact of the world reaches, and sweeps K wide (described above
// mass_times).  A wide block (more than kTwoWaveWidth coordinates) of a world whose contact rows each act through one
// link keeps no Jacobian rows: every entry follows from the row's wrench and the coordinates' motion axes (described
// above link_motion and add_heads_through_links).
//
// Replaces src/phi/backend_cuda/ops/block_descent_tile.cuh (DescendTile :2941-3087 and everything it calls) and
// the helpers it takes from block_descent.cu (:735-820, 1593-1621, 1726-1753) and nk/solve/augmented_row.hpp.
// Blocks: one articulation per environment.  Rows on a single coordinate (joint limit, friction and drive rows) are
// "unit" rows (:799-833): they stage no Jacobian row and touch one diagonal entry and one force entry.
// Not built: free rigid 6x6 blocks, mimic couplings.
#pragma once

#include <utility>
#include "nk_device_math.h"
#include "backend.h"
#include "nk_ops.h"

namespace nkh {
namespace solver {
// This header compiles two ways.  Plainly, a block of up to kTwoWaveWidth coordinates runs two waves a SIMD with up to 256
// registers each.  With NKH_SOLVER_DENSE defined (ops_solver_d*.hip) everything below sits in namespace `dense` and a block
// of up to kThreeWaveWidth coordinates is compiled for three waves a SIMD: 168 registers, a few dozen values a lane in
// scratch memory, the same arithmetic.  A long environment runs a tenth slower that way and a full machine gets a tenth
// more done, so the launcher takes the dense kernels for batches that fill the machine several times over.
#ifdef NKH_SOLVER_DENSE
namespace dense {
#endif

constexpr int kWave = 64;
// Widths up to this run two waves per SIMD (at most 256 registers each); wider rows need the whole register file.
#ifndef NKH_TWO_WAVE_WIDTH
#define NKH_TWO_WAVE_WIDTH 36
#endif
constexpr int kTwoWaveWidth = NKH_TWO_WAVE_WIDTH;
// Widths up to this run three waves per SIMD in the dense build (none in the plain one).
#ifdef NKH_SOLVER_DENSE
constexpr int kThreeWaveWidth = 20;
#else
constexpr int kThreeWaveWidth = 0;
#endif
constexpr int WavesPerSimd(int width) { return width <= kThreeWaveWidth ? 3 : (width <= kTwoWaveWidth ? 2 : 1); }
// From this width on a block widens its mass rows to double where it uses them; below it the widened rows are kept over
// the solve (two registers an entry), which pays while they fit.  In the dense build's 168 registers they never do:
// kept, they are what spills (96 B a lane at 20 coordinates, none widened at use; 65536 quadrupeds 6.74 -> 6.48 ms).
#ifndef NKH_WIDEN_AT_USE
#ifdef NKH_SOLVER_DENSE
#define NKH_WIDEN_AT_USE 0
#else
#define NKH_WIDEN_AT_USE 24
#endif
#endif
constexpr int kWidenAtUse = NKH_WIDEN_AT_USE;
constexpr uint32_t kNewtonSteps = 16u;        // block_descent_dense.cuh:14
constexpr uint32_t kLineSearchSteps = 32u;    // block_descent_dense.cuh:15
constexpr float kLineTolerance = 1.0e-6f;     // block_descent_dense.cuh:17
constexpr float kRoundings = 8.0f;            // block_descent_dense.cuh:19
constexpr float kPenaltyConditionCap = 1.0e2f;   // block_descent.cu:71
// Unit heads a coordinate can list for itself (lower limit, upper limit, friction, drive, and room to spare); a block
// with more on one coordinate walks its unit heads serially instead.
constexpr uint32_t kUnitSlots = 6u;
// contributing heads from which a wide block takes the heads' curvature by way of the links (add_heads_through_links)
constexpr uint32_t kLinkHeads = 4u;
// words a head of Tile::wrench: 3 x 6 wrench components, the two words of its way to the root, one more for an odd stride
constexpr uint32_t kWrenchStride = 21u;

// Phase timers for development builds (-DNKH_SOLVER_PROFILE): cycles per phase and event counts per environment,
// written over the environment's solver_penalty words at the end of the solve.
#ifdef NKH_SOLVER_PROFILE
#define PROF_BEGIN(c, i) const long long prof_start_##i = clock64()
#define PROF_END(c, i) (c).prof[i] += clock64() - prof_start_##i
#define PROF_COUNT(c, i) (c).prof_count[i] += 1u
#else
#define PROF_BEGIN(c, i)
#define PROF_END(c, i)
#define PROF_COUNT(c, i)
#endif

// The reference sums its gradients, slopes and decrements as two-float compensated sums (TileSum, block_descent_tile.cuh
// :15-46).  Here the same sums run in double: a product of two floats is exact in double, the vector unit executes a
// double multiply-add at the rate of a float one, and one instruction replaces the nine of a compensated step.  The
// rounded result is at least as close to the exact sum as the two-float one.
struct TileSum { double value; };
__device__ __forceinline__ void tile_add(TileSum& s, float x) { s.value += double(x); }
__device__ __forceinline__ void tile_add_product(TileSum& s, float a, float b) { s.value = fma(double(a), double(b), s.value); }
template <int Ctrl>
__device__ __forceinline__ double dpp_move_d(double v) {
    const uint64_t bits = uint64_t(__double_as_longlong(v));
    const uint32_t low = uint32_t(__builtin_amdgcn_update_dpp(0, int(uint32_t(bits)), Ctrl, 0xF, 0xF, false));
    const uint32_t high = uint32_t(__builtin_amdgcn_update_dpp(0, int(uint32_t(bits >> 32u)), Ctrl, 0xF, 0xF, false));
    return __longlong_as_double((long long)((uint64_t(high) << 32u) | uint64_t(low)));
}
__device__ __forceinline__ double row_value_d(double v, int row) {
    const uint64_t bits = uint64_t(__double_as_longlong(v));
    const uint32_t low = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(bits)), 16 * row));
    const uint32_t high = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(bits >> 32u)), 16 * row));
    return __longlong_as_double((long long)((uint64_t(high) << 32u) | uint64_t(low)));
}
__device__ __forceinline__ double lane_value_d(double v, int lane) {   // `lane` a compile-time constant at every call site
    const uint64_t bits = uint64_t(__double_as_longlong(v));
    const uint32_t low = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(bits)), lane));
    const uint32_t high = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(bits >> 32u)), lane));
    return __longlong_as_double((long long)((uint64_t(high) << 32u) | uint64_t(low)));
}
// every lane of a row of sixteen ends with the row's sum
__device__ __forceinline__ double row_total_d(double v) {
    v += dpp_move_d<kDppXor1>(v); v += dpp_move_d<kDppXor2>(v); v += dpp_move_d<kDppHalfMirror>(v); v += dpp_move_d<kDppMirror>(v);
    return v;
}
// the sum over the wave: rows of 16 by DPP, then the four rows as scalars; uniform result
__device__ __forceinline__ float wave_total(TileSum s, bool first_row_only = false) {
    const double v = row_total_d(s.value);
    const double a = row_value_d(v, 0);
    // the copies of the first row's heads in lanes 16..63 are left out when only the first sixteen lanes carry terms
    if (first_row_only) return float(a);
    return float((a + row_value_d(v, 1)) + (row_value_d(v, 2) + row_value_d(v, 3)));
}
__device__ __forceinline__ float first_row_sum(float v) {
    v += dpp_move<kDppXor1>(v); v += dpp_move<kDppXor2>(v); v += dpp_move<kDppHalfMirror>(v); v += dpp_move<kDppMirror>(v);
    return row_value(v, 0);
}

struct Response { float dual_scale, residual_scale; };
// augmented_row.hpp:226-229
__device__ __forceinline__ Response scalar_response(float cap, float compliance) {
    const float product = cap * compliance;
    return product >= 1.0f ? Response{0.0f, 1.0f / compliance} : Response{1.0f - product, cap};
}
// augmented_row.hpp:232-247
__device__ __forceinline__ void scalar_impulse(float dual, float rho, float residual, float compliance, float lower, float upper,
                                               Response r, float* impulse, float* curvature) {
    *impulse = 0.0f; *curvature = 0.0f;
    if (rho <= 0.0f) return;
    if (dual != dual || rho != rho || residual != residual || compliance != compliance || lower != lower || upper != upper) {
        const float invalid = dual + rho + residual + compliance + lower + upper;
        *impulse = invalid; *curvature = invalid;
        return;
    }
    const float k = r.residual_scale;
    const float x = fmaf(k, residual, r.dual_scale * dual);
    *impulse = x < lower ? lower : (x > upper ? upper : x);
    *curvature = x != x ? x : (lower < upper && x >= lower && x <= upper ? k : 0.0f);
}
// augmented_row.hpp:302-318, in two parts: what depends on the dual, the penalty and the friction ratio only, and
// the rest, which takes the residual.  A line search evaluates the second part at every probe and the first once.
struct ConeAxis { float dd, d_low, p, p_low; };
__device__ __forceinline__ ConeAxis cone_axis(float dual, float rho, float mu) {
    // a friction ratio of exactly one (equal coefficients) divides to the dividend itself: skip the two divisions
    const bool unit = mu == 1.0f;
    const bool dual_zero = dual == 0.0f;
    const Recip by_mu = make_recip(mu);   // a ratio of zero gives values that every caller discards
    const float dual_quotient = unit ? dual + float(dual_zero) : div_by(dual + float(dual_zero), by_mu);
    const float dd = dual_zero ? dual : dual_quotient;
    const float low = fmaf(-dd, mu, dual);
    const bool low_zero = low == 0.0f;
    const float low_quotient = unit ? low + float(low_zero) : div_by(low + float(low_zero), by_mu);
    const float d_low = low_zero ? low : low_quotient;
    const float p = rho * mu;
    return ConeAxis{dd, d_low, p, fmaf(rho, mu, -p)};
}
__device__ __forceinline__ float cone_value(ConeAxis a, float residual) {
    const float t = a.p * residual;
    const float t_low = fmaf(a.p, residual, -t) + a.p_low * residual;
    const float sum = a.dd + t;
    const float t_part = sum - a.dd;
    const float sum_low = (a.dd - (sum - t_part)) + (t - t_part);
    return sum + (sum_low + a.d_low + t_low);
}
__device__ __forceinline__ float cone_argument(float dual, float rho, float mu, float residual) {
    return cone_value(cone_axis(dual, rho, mu), residual);
}
// augmented_row.hpp:321-348; curvature entries yy, zz, yz.  The friction ratios depend on the row only, so callers
// that evaluate one row many times compute them once (tangent_ratios) and pass them in.
struct TangentRatios { float mu_y, mu_z, scale; };
__device__ __forceinline__ TangentRatios tangent_ratios(float mu_first, float mu_second) {
    const float scale = fmaxf(mu_first, mu_second);
    return TangentRatios{mu_first <= 0.0f ? 0.0f : mu_first / scale, mu_second <= 0.0f ? 0.0f : mu_second / scale, scale};
}
__device__ __forceinline__ void tangent_impulse(V3 dual, float rho, float res_y, float res_z, float normal_impulse, TangentRatios t,
                                float* fy, float* fz, float* cyy, float* czz, float* cyz) {
    *fy = *fz = *cyy = *czz = *cyz = 0.0f;
    if (rho <= 0.0f) return;
    const float mu_y = t.mu_y, mu_z = t.mu_z;
    const float q_y = mu_y == 0.0f ? 0.0f : cone_argument(dual.y, rho, mu_y, res_y);
    const float q_z = mu_z == 0.0f ? 0.0f : cone_argument(dual.z, rho, mu_z, res_z);
    const float radius = (normal_impulse < 0.0f ? 0.0f : normal_impulse) * fmaxf(t.scale, 0.0f);
    if (q_y != q_y || q_z != q_z || radius != radius || rho != rho) {
        const float invalid = q_y + q_z + radius + rho;
        *fy = *fz = *cyy = *czz = *cyz = invalid;
        return;
    }
    if (radius == 0.0f) return;
    const float norm = hypotf(q_y, q_z);
    if (norm <= radius) {
        *fy = mu_y * q_y; *fz = mu_z * q_z; *cyy = rho * mu_y * mu_y; *czz = rho * mu_z * mu_z;
        return;
    }
    const float dy = q_y / norm, dz = q_z / norm;
    const float cs = rho * radius / norm;
    *fy = mu_y * radius * dy; *fz = mu_z * radius * dz;
    *cyy = cs * mu_y * mu_y * dz * dz; *czz = cs * mu_z * mu_z * dy * dy; *cyz = -cs * mu_y * mu_z * dy * dz;
}
__device__ __forceinline__ void tangent_impulse(V3 dual, float rho, float res_y, float res_z, float normal_impulse, float mu_first, float mu_second,
                                float* fy, float* fz, float* cyy, float* czz, float* cyz) {
    tangent_impulse(dual, rho, res_y, res_z, normal_impulse, tangent_ratios(mu_first, mu_second), fy, fz, cyy, czz, cyz);
}

// ComputeEllipticResponse (augmented_row.hpp:48-55): residual scale k and dual scale s of the three axes
struct EllipticResponse { float kx, ky, kz, sx, st; };
__device__ __forceinline__ EllipticResponse elliptic_response(float cap, float cn, float cy, float cz) {
    const double tangent = fmin(double(cy), double(cz));
    const double normal_scale = 1.0 / (1.0 + double(cap) * cn);
    const double tangent_scale = 1.0 / (1.0 + double(cap) * tangent);
    return EllipticResponse{float(cap * normal_scale), float(cap * tangent_scale * tangent / cy), float(cap * tangent_scale * tangent / cz),
                            float(normal_scale), float(tangent_scale)};
}
// EvaluateEllipticImpulse (augmented_row.hpp:58-80): the projection onto the friction cone in the metric that makes
// its cross section a circle; curvature xx yy zz xy xz yz
__device__ __forceinline__ void elliptic_impulse(V3 dual, float cap, float rx, float ry, float rz, float cn, float cy, float cz, float mu_first,
                                                 float* f, float* cv) {
    const EllipticResponse e = elliptic_response(cap, cn, cy, cz);
    const float xx = fmaf(e.kx, rx, e.sx * dual.x), xy = fmaf(e.ky, ry, e.st * dual.y), xz = fmaf(e.kz, rz, e.st * dual.z);
    const float root_x = sqrtf(e.kx), root_y = sqrtf(e.ky), root_z = sqrtf(e.kz);
    const float m = mu_first * root_x / root_y;
    const float p = xx / root_x, q1 = xy / root_y, q2 = xz / root_z;
    const float t = hypotf(q1, q2);
    f[0] = f[1] = f[2] = 0.0f;
    cv[0] = cv[1] = cv[2] = cv[3] = cv[4] = cv[5] = 0.0f;
    if (t <= m * p) { f[0] = xx; f[1] = xy; f[2] = xz; cv[0] = e.kx; cv[1] = e.ky; cv[2] = e.kz; return; }
    if (m * t + p <= 0.0f) return;
    const float a = 1.0f / (1.0f + m * m);
    const float projected = (p + m * t) * a;
    const float u1 = q1 / t, u2 = q2 / t;
    const float b = m * projected / t, along = m * m * a;
    f[0] = projected * root_x; f[1] = m * projected * u1 * root_y; f[2] = m * projected * u2 * root_z;
    cv[0] = e.kx * a; cv[1] = e.ky * (along * u1 * u1 + b * u2 * u2); cv[2] = e.kz * (along * u2 * u2 + b * u1 * u1);
    cv[3] = root_x * root_y * m * a * u1; cv[4] = root_x * root_z * m * a * u2; cv[5] = root_y * root_z * (along - b) * u1 * u2;
}

__device__ __forceinline__ uint32_t residual_bits(float value) { return __float_as_uint(value <= FLT_MAX ? fabsf(value) : FLT_MAX); }
__device__ __forceinline__ float along_axis(float impulse, float velocity) { return impulse > 0.0f ? velocity : impulse < 0.0f ? -velocity : 0.0f; }

// Per-head state in LDS, head-major with an odd stride so lane = head reads without bank conflicts.
enum HeadField : uint32_t {
    hSlot, hStride, hAxes, hOwned, hRho, hCompliance, hLower, hUpper, hMu1, hMu2, hNormalBound,
    hRes, hDual = hRes + 3, hMove = hDual + 3, hStep = hMove + 3, hBase = hStep + 3, hDualScale = hBase + 3, hResidualScale,
    hRelaxStep, hRelaxWeight = hRelaxStep + 3, hRelaxPoint, hF = hRelaxPoint + 3, hC = hF + 3, hNoise = hC + 6, hContrib = hNoise + 3, hColumnsLow, hColumnsHigh, hSourceA, hSourceB = hSourceA + 3, hSourceEnd = hSourceB + 3,
    hRow = hSourceEnd,   // first of the head's three staged Jacobian rows; kInvalid for a unit head
    hUnit,               // the one coordinate a unit head acts on; kInvalid for a staged head
    hUnitValue,          // its Jacobian entry there
    hFieldCount
};

// A contact head under the elliptic cone of the MuJoCo law (block_descent_tile.cuh:645, 778) carries 4 in hAxes: three
// axes, answered by elliptic_impulse.  Such a head has no relaxation state (its dual update takes the projection as it
// is), so the first two words of hRelaxStep hold what it needs instead: the compliances of its two tangent rows.
constexpr uint32_t kAxesElliptic = 4u;
constexpr uint32_t hTangentCompliance = hRelaxStep;
__device__ __forceinline__ bool block_axes(uint32_t axes) { return axes >= 3u; }

// A head on one axis uses the first component of every three-component field and none of the block-only fields;
// only block heads (three axes: contact points, which are listed first) use the rest.  The fields are therefore kept
// in two tables: "wide" fields have room for every head, "narrow" fields for the first `narrow` heads and one more
// word that every later head shares.  That word reads as zero and swallows what is written to it, which is always
// zero: a single-axis head keeps its second and third components, its relaxation state and its column masks at zero
// throughout.  A head's place in a narrow field is min(h, narrow), one operation whatever the number of fields read.
__host__ __device__ constexpr uint32_t clamped_span(uint32_t f, uint32_t first, uint32_t end) {   // fields of [first, end) below f
    return f <= first ? 0u : (f >= end ? end - first : f - first);
}
// the narrow fields are these ranges of field ids
__host__ __device__ constexpr uint32_t narrow_below(uint32_t f) {
    return clamped_span(f, hRes + 1, hRes + 3) + clamped_span(f, hDual + 1, hDual + 3) + clamped_span(f, hMove + 1, hMove + 3) +
           clamped_span(f, hStep + 1, hStep + 3) + clamped_span(f, hBase + 1, hBase + 3) + clamped_span(f, hRelaxStep, hF) +
           clamped_span(f, hF + 1, hF + 3) + clamped_span(f, hC + 1, hNoise) + clamped_span(f, hNoise + 1, hNoise + 3) +
           clamped_span(f, hColumnsLow, hColumnsHigh + 1);
}
__host__ __device__ constexpr bool narrow_field(uint32_t f) { return narrow_below(f + 1u) != narrow_below(f); }
constexpr uint32_t kNarrowFields = narrow_below(hFieldCount);
constexpr uint32_t kWideFields = hFieldCount - kNarrowFields;
static_assert(kNarrowFields <= 64u, "one lane clears the shared word of each narrow field");
// Both tables are head-major with an odd number of words a head: a field of head h sits at h * stride + its index, so
// every access is one base register (the head's) plus a constant offset, and lanes that read one field of consecutive
// heads fall on different banks.
constexpr uint32_t kWideStride = kWideFields | 1u, kNarrowStride = kNarrowFields | 1u;

struct Tile {
    uint32_t env, lane, n, ldj, heads, cap, narrow, iteration;
    uint32_t n_all;   // n, or past it the coordinates that follow the block's own (a reduced block, described above mass_times)
    float tolerance;
    float* mfac;     // FactorFloats(N) words: Cholesky factor of the mass matrix (rows; columns are read transposed); device memory for a wide block
    float* hfac;     // FactorFloats(N) words: Cholesky factor of the current Newton Hessian
    float* jac;      // 3 * staged capacity rows x ldj, ldj = N
    float* fields;   // cap x kWideStride, then (narrow + 1) x kNarrowStride
    float* vec;      // 4 x 64 scratch vectors, 16-byte aligned
    float mass_inverse;   // 1 / diagonal of the mass factor, lane = row
    mutable bool factor_current;     // no head's curvature has changed since hfac was factored: the Hessian is the same
    mutable uint32_t work;   // Newton steps and line probes of this solve, the next solve's scheduling key
    bool mass_valid;
    bool elliptic;   // some head is under the elliptic cone: every response goes through the general functions
    bool units;      // some head is a unit head
    bool unit_lists; // every coordinate's unit heads fit its list
    uint32_t* unit_list;      // kUnitSlots x 64: lane's unit heads in head order, slot-major
    uint32_t unit_count;      // lane's own count
    uint32_t staged_end;      // one past the last staged head
    uint32_t individual_end;  // one past the last head whose inertial response is computed for itself
    float momentum, residual;
    bool failed;
    // what add_heads_through_links needs (wide blocks only)
    bool from_links;          // the block keeps no contact rows: their entries follow from `wrench` and `axes` wherever a row is read
    float* wrench;            // cap x kWrenchStride: a head's three rows as wrenches about `pivot`, then its way to the root (two words)
    bool through_links;       // every staged head acts on the block through one link: the heads' curvature may go by way of the links
    float* axes;              // 64 x 12: a coordinate's motion axis about `pivot`, then the contact stiffness it carries times that axis
    uint32_t path_low, path_high;     // lane = coordinate: the coordinates on the way from its link to the root, itself included
    uint32_t under_low, under_high;   // the coordinates whose way to the root passes through lane's
    V3 pivot;                 // the point the axes and the heads' wrenches are taken about: the root link's origin
    const float* rows;        // the environment-major row records, row points and row links of device memory
    const float* row_point_a, *row_point_b;
    const uint32_t* row_link_a, *row_link_b;
    const uint64_t* link_paths;
    uint32_t first_link;      // index of the environment's first link
#ifdef NKH_SOLVER_PROFILE
    mutable long long prof[32];
    mutable uint32_t prof_count[4];
#endif
    // with a constant field, as at nearly every call, the place of the field folds to a constant
    __device__ __forceinline__ uint32_t at(uint32_t field, uint32_t h) const {
        const uint32_t below = narrow_below(field);
        if (!narrow_field(field)) return h * kWideStride + (field - below);
        return kWideStride * cap + min(h, narrow) * kNarrowStride + below;
    }
    __device__ __forceinline__ float& F(uint32_t field, uint32_t h) const { return fields[at(field, h)]; }
    __device__ __forceinline__ uint32_t& U(uint32_t field, uint32_t h) const { return reinterpret_cast<uint32_t*>(fields)[at(field, h)]; }
};

// TileResponse (block_descent_tile.cuh:678-681) with the Coulomb branch of EvaluateAugmentedResponse (block_descent.cu:1593-1621)
__device__ __forceinline__ void head_response(const Tile& c, uint32_t h, float mx, float my, float mz, float* f, float* cv) {
    const float rho = c.F(hRho, h);
    if (c.elliptic && c.U(hAxes, h) == kAxesElliptic) {   // block_descent.cu:1595-1601
        elliptic_impulse(V3{c.F(hDual, h), c.F(hDual + 1, h), c.F(hDual + 2, h)}, rho, c.F(hRes, h) - mx, c.F(hRes + 1, h) - my,
                         c.F(hRes + 2, h) - mz, c.F(hCompliance, h), c.F(hTangentCompliance, h), c.F(hTangentCompliance + 1, h),
                         c.F(hMu1, h), f, cv);
        return;
    }
    float ni, nc;
    scalar_impulse(c.F(hDual, h), rho, c.F(hRes, h) - mx, c.F(hCompliance, h), c.F(hLower, h), c.F(hUpper, h),
                   Response{c.F(hDualScale, h), c.F(hResidualScale, h)}, &ni, &nc);
    f[0] = ni; f[1] = f[2] = 0.0f;
    cv[0] = nc; cv[1] = cv[2] = cv[3] = cv[4] = cv[5] = 0.0f;
    if (!block_axes(c.U(hAxes, h))) return;
    tangent_impulse(V3{c.F(hDual, h), c.F(hDual + 1, h), c.F(hDual + 2, h)}, rho, c.F(hRes + 1, h) - my, c.F(hRes + 2, h) - mz,
                    c.F(hNormalBound, h), c.F(hMu1, h), c.F(hMu2, h), &f[1], &f[2], &cv[1], &cv[2], &cv[5]);
}

// A pivot's reciprocal square root by the hardware approximation (an ulp or so): the pivot's place in the factor is
// pivot * scale and its reciprocal is scale, two instructions on the chain every later pivot waits for where a
// correctly rounded root and quotient take about fifteen.  The factor differs from the correctly rounded one by a
// backward error of a few ulp in the matrix, which a Newton direction does not see.
__device__ __forceinline__ float pivot_scale(float pivot) { return __builtin_amdgcn_rsqf(pivot); }

// FactorTileBlock (:1622-1645) on register rows: lane i holds row i of the symmetric matrix; on return its entries
// k <= i are row i of the Cholesky factor.  Element (i, j) loses L_ik L_jk for k = 0, 1, ... in that order, as the
// reference's serial inner loop does; each product and subtraction is one fused multiply-add (the reference is
// built with its compiler's default contraction, so it fuses these too).  Uniform result: false on a bad pivot.
template <int N>
__device__ __forceinline__ bool factor_rows(uint32_t lane, float (&row)[N], float* inverse_out) {
    lane = local_lane(lane);
    bool valid = true;
    float inverse = 0.0f;
#pragma unroll
    for (int k = 0; k < N; ++k) {
        // the pivot's square root and reciprocal
        const float pivot = lane_value(row[k], k);
        valid = valid && pivot > 0.0f && pivot <= FLT_MAX;
        const float scale = pivot_scale(valid ? pivot : 1.0f);
        const float root = pivot * scale;
        row[k] = lane == uint32_t(k) ? root : row[k] * scale;
        if (lane == uint32_t(k)) inverse = scale;
        // lane reads in batches of eight ahead of their multiply-adds: a scalar read has to settle for two cycles
        // before an arithmetic instruction may use it, and the next reads fill that gap
#pragma unroll
        for (int j0 = k + 1; j0 < N; j0 += 8) {
            float l[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) l[t] = j0 + t < N ? lane_value(row[k], j0 + t) : 0.0f;
#pragma unroll
            for (int t = 0; t < 8; ++t)
                if (j0 + t < N) row[j0 + t] = fmaf(-row[k], l[t], row[j0 + t]);
        }
    }
    *inverse_out = inverse;
    return valid;
}

// Past 32 coordinates the reference's tile is "wide" (TileSpan > 1, :71-73) and factors H = U U^T from the last
// coordinate down, "so a tree's leaves go first" (FactorTileColumns :209-252); its substitutions run up the columns of
// U and then down its rows (SolveWideTileBlock :1866-1895).  Which end the elimination starts from decides whether a
// long chain's block can be factored in single precision at all, so the order is part of the path's arithmetic.
template <int N>
constexpr bool kLeavesFirst = N > 32;

// Where a factor is kept for its transposed reads.  Root first: rows of N + 1 words.  Leaves first: lane i's row of
// U holds the entries k >= i only, and the rows are packed - row i starts at i N - i (i - 1) / 2 and is N - i words
// long - which halves the storage; a column's words for consecutive lanes are consecutive.
__host__ __device__ constexpr uint32_t FactorFloats(uint32_t N) { return N > 32u ? (N * (N + 1u) / 2u + 3u) & ~3u : N * (N + 1u); }
template <int N>
__device__ __forceinline__ uint32_t factor_at(uint32_t i, uint32_t k) {   // leaves first: k >= i
    if constexpr (kLeavesFirst<N>) return i * uint32_t(N) - (i * (i - 1u)) / 2u + (k - i);
    else return i * uint32_t(N + 1) + k;
}

// FactorTileColumns on register rows: lane i holds row i of the symmetric matrix; on return its entries k >= i are
// row i of U.  Column k leaves exact zeros in the rows of other branches of the tree, and the update of a column by
// an exact zero changes nothing: such columns are skipped four at a time.
// With kStop > 0 the elimination ends after pivot kStop: rows and columns below it then hold the Schur complement of the
// eliminated coordinates, rows below it hold their coupling to them in the columns from kStop on.
template <int N, int kStop = 0>
__device__ __forceinline__ bool factor_rows_up(uint32_t lane, float (&row)[N], float* inverse_out) {
    lane = local_lane(lane);
    bool valid = true;
    float inverse = 0.0f;
#pragma unroll
    for (int k = N - 1; k >= kStop; --k) {
        const float pivot = lane_value(row[k], k);
        valid = valid && pivot > 0.0f && pivot <= FLT_MAX;
        const float scale = pivot_scale(valid ? pivot : 1.0f);
        const float root = pivot * scale;
        row[k] = lane == uint32_t(k) ? root : row[k] * scale;
        if (lane == uint32_t(k)) inverse = scale;
        const uint64_t reach = __ballot(lane < uint32_t(k) && row[k] != 0.0f);
#pragma unroll
        for (int q = (k - 1) / 4; q >= 0 && k >= 1; --q) {
            if (((reach >> (4 * q)) & 0xFull) == 0ull) continue;
            float u[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) u[t] = 4 * q + t <= k - 1 ? lane_value(row[k], 4 * q + t) : 0.0f;
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (4 * q + t <= k - 1) row[4 * q + t] = fmaf(-row[k], u[t], row[4 * q + t]);
        }
    }
    *inverse_out = inverse;
    return valid;
}

// SolveWideTileBlock: U w = g with lane's own row (entries right of the diagonal), then U^T d = w with the columns,
// read from the factor in LDS eight at a time.
template <int N>
__device__ __forceinline__ float substitute_up(uint32_t lane, const float (&row)[N], const float* factor, float inverse, float g) {
    lane = local_lane(lane);
    float r = g;
#pragma unroll
    for (int j = N - 1; j >= 0; --j) {
        const float y = lane_value(r * inverse, j);
        r = lane < uint32_t(j) ? fmaf(-row[j], y, r) : r;
    }
    r *= inverse;
    const uint32_t mine = lane < uint32_t(N) ? lane : 0u;
#pragma unroll
    for (int j0 = 0; j0 < N; j0 += 8) {
        float u[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)   // U[j][lane] for the lanes past j; the others read a word they do not use
            u[t] = j0 + t < N ? factor[mine >= uint32_t(j0 + t) ? factor_at<N>(uint32_t(j0 + t), mine) : 0u] : 0.0f;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if (j0 + t >= N) continue;
            const float x = lane_value(r * inverse, j0 + t);
            r = lane > uint32_t(j0 + t) && lane < uint32_t(N) ? fmaf(-u[t], x, r) : r;
        }
    }
    return r * inverse;
}

// SolveTileBlock (:1647-1666): forward with the factor's rows, backward with its columns (col[j] = L_j,lane).
template <int N>
__device__ __forceinline__ float substitute(uint32_t lane, const float (&row)[N], const float (&col)[N], float inverse, float g) {
    // Lane j's entry is final once the steps before it have run, so it is scaled by its reciprocal pivot where it is
    // read (the same product that would be stored back) and the lanes take it in one multiplication after the sweep.
    lane = local_lane(lane);
    float r = g;
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const float y = lane_value(r * inverse, j);
        r = lane > uint32_t(j) ? fmaf(-row[j], y, r) : r;
    }
    r *= inverse;
#pragma unroll
    for (int j = N - 1; j >= 0; --j) {
        const float x = lane_value(r * inverse, j);
        r = lane < uint32_t(j) ? fmaf(-col[j], x, r) : r;
    }
    return r * inverse;
}

template <int N>
__device__ __forceinline__ void store_rows(float* a, uint32_t lane, const float (&row)[N]) {
    lane = local_lane(lane);
    if (lane < uint32_t(N)) {
#pragma unroll
        for (int k = 0; k < N; ++k)
            if (!kLeavesFirst<N> || uint32_t(k) >= lane) a[factor_at<N>(lane, uint32_t(k))] = row[k];
    }
}
// (Every word is read whether or not the lane keeps it - a read under a condition compiles to a branch a word - from
// a place inside the factor: a lane past the rows reads the last row's, and a packed row's words left of its diagonal
// fall in the rows before it.)
template <int N>
__device__ __forceinline__ void load_rows(const float* a, uint32_t lane, float (&row)[N]) {
    lane = local_lane(lane);
    const uint32_t from = lane < uint32_t(N) ? lane : uint32_t(N - 1);
#pragma unroll
    for (int k = 0; k < N; ++k) {
        const bool kept = lane < uint32_t(N) && (!kLeavesFirst<N> || uint32_t(k) >= lane);
        if constexpr (N > kTwoWaveWidth) {   // such a block's mass factor is in device memory: only the words that are kept
            row[k] = kept ? a[factor_at<N>(lane, uint32_t(k))] : 0.0f;
        } else {
            const float word = a[factor_at<N>(from, uint32_t(k))];
            row[k] = kept ? word : 0.0f;
        }
    }
}
template <int N>
__device__ __forceinline__ void load_columns(const float* a, uint32_t lane, float (&col)[N]) {
    lane = local_lane(lane);
    const uint32_t from = lane < uint32_t(N) ? lane : uint32_t(N - 1);
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const float word = a[j * (N + 1) + from];
        col[j] = lane < uint32_t(N) ? word : 0.0f;
    }
}

// Cholesky of the Newton Hessian held in `hrow`, then d = H^-1 g.  The factor passes through LDS once, for the
// transposed read of the backward substitution.
template <int N>
__device__ __forceinline__ bool cholesky_solve(const Tile& c, float (&hrow)[N], float g, float* d_out) {
    const uint32_t row = local_lane(c.lane);
    float inverse = 0.0f;
    if (!c.factor_current) {   // otherwise the Hessian is the one factored last: its factor is still in hfac
        PROF_BEGIN(c, 14);
        const bool valid = kLeavesFirst<N> ? factor_rows_up<N>(c.lane, hrow, &inverse) : factor_rows<N>(c.lane, hrow, &inverse);
        PROF_END(c, 14);
        if (!valid) return false;
        PROF_BEGIN(c, 24);
        store_rows<N>(c.hfac, c.lane, hrow);
        __syncthreads();
        PROF_END(c, 24);
        c.factor_current = true;
    } else {
        PROF_COUNT(c, 3);
        // rows and the reciprocal diagonal come back from hfac (the factor's own reciprocal is 1 / its diagonal
        // entry, the same division)
        inverse = row < uint32_t(N) ? 1.0f / c.hfac[factor_at<N>(row, row)] : 0.0f;
        load_rows<N>(c.hfac, c.lane, hrow);
    }
    PROF_BEGIN(c, 15);
    if constexpr (kLeavesFirst<N>) {
        *d_out = substitute_up<N>(c.lane, hrow, c.hfac, inverse, c.lane < c.n ? g : 0.0f);
    } else {
        float col[N];
        load_columns<N>(c.hfac, c.lane, col);
        *d_out = substitute<N>(c.lane, hrow, col, inverse, c.lane < c.n ? g : 0.0f);
    }
    __syncthreads();
    PROF_END(c, 15);
    return true;
}

// SolveTileMass (:1898-1931).  The mass matrix does not change during a solve, so its factor (same arithmetic as the
// reference's per-call factorisation, hence the same numbers) is built once by factor_mass and reused here.
template <int N>
__device__ __forceinline__ bool factor_mass(Tile& c, const float (&mrow)[N]) {
    float row[N];
#pragma unroll
    for (int k = 0; k < N; ++k) row[k] = mrow[k];
    float inverse = 0.0f;
    const bool valid = kLeavesFirst<N> ? factor_rows_up<N>(c.lane, row, &inverse) : factor_rows<N>(c.lane, row, &inverse);
    c.mass_inverse = inverse;
    store_rows<N>(c.mfac, c.lane, row);
    __syncthreads();
    return valid;
}
template <int N>
__device__ __forceinline__ float solve_tile_mass(const Tile& c, float force) {
    float row[N];
    load_rows<N>(c.mfac, c.lane, row);
    if constexpr (kLeavesFirst<N>) return substitute_up<N>(c.lane, row, c.mfac, c.mass_inverse, c.lane < c.n ? force : 0.0f);
    float col[N];
    load_columns<N>(c.mfac, c.lane, col);
    return substitute<N>(c.lane, row, col, c.mass_inverse, c.lane < c.n ? force : 0.0f);
}

// The LDS byte address of a pointer into the block's shared memory.
__device__ __forceinline__ uint32_t lds_address(const float* p) {
    return uint32_t(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const float*)p));
}

// Four columns of a head's Hessian term, taken or left as a whole on a uniform mask, with the products and sums the
// plain loops of add_head form.  Three rows: h += a0 x0 + a1 x1 + a2 x2 as a product, two fused multiply-adds and a
// sum.  A single row: one fused multiply-add into h.  Written out because the compiled form of such a conditional
// update carries the whole row through the head loop twice and copies one set of registers into the other at every
// branch, about as many moves as the update has arithmetic.  Here the row's registers change in place, and the words
// come from LDS (`kFirst`, `kSecond`, `kThird` bytes past `row_address`) into twelve registers that the block takes for
// itself, v244-v255.  Only for widths that run two waves a SIMD: their kernels leave those registers free.  The waits
// count LDS reads only as far as those return in order; scalar loads in flight make them wait longer, never shorter.
#ifdef NKH_SOLVER_DENSE   // the same block on registers inside the dense build's 168: v152-v163
template <int kFirst, int kSecond, int kThird>
__device__ __forceinline__ void add_columns_if(uint32_t live, uint32_t single, uint32_t row_address, float a0, float a1, float a2, float& h0,
                                               float& h1, float& h2, float& h3) {
    asm volatile(
        "s_cmp_eq_u32 %[live], 0\n\t"
        "s_cbranch_scc1 .Lcolumns_done_%=\n\t"
        "s_cmp_eq_u32 %[single], 0\n\t"
        "s_cbranch_scc0 .Lcolumns_single_%=\n\t"
        "ds_read_b128 v[152:155], %[at] offset:%[first]\n\t"
        "ds_read_b128 v[156:159], %[at] offset:%[second]\n\t"
        "ds_read_b128 v[160:163], %[at] offset:%[third]\n\t"
        "s_waitcnt lgkmcnt(2)\n\t"
        "v_mul_f32 v152, %[a0], v152\n\t"
        "v_mul_f32 v153, %[a0], v153\n\t"
        "v_mul_f32 v154, %[a0], v154\n\t"
        "v_mul_f32 v155, %[a0], v155\n\t"
        "s_waitcnt lgkmcnt(1)\n\t"
        "v_fmac_f32 v152, %[a1], v156\n\t"
        "v_fmac_f32 v153, %[a1], v157\n\t"
        "v_fmac_f32 v154, %[a1], v158\n\t"
        "v_fmac_f32 v155, %[a1], v159\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        "v_fmac_f32 v152, %[a2], v160\n\t"
        "v_fmac_f32 v153, %[a2], v161\n\t"
        "v_fmac_f32 v154, %[a2], v162\n\t"
        "v_fmac_f32 v155, %[a2], v163\n\t"
        "v_add_f32 %[h0], %[h0], v152\n\t"
        "v_add_f32 %[h1], %[h1], v153\n\t"
        "v_add_f32 %[h2], %[h2], v154\n\t"
        "v_add_f32 %[h3], %[h3], v155\n\t"
        "s_branch .Lcolumns_done_%=\n"
        ".Lcolumns_single_%=:\n\t"
        "ds_read_b128 v[152:155], %[at] offset:%[first]\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        "v_fmac_f32 %[h0], %[a0], v152\n\t"
        "v_fmac_f32 %[h1], %[a0], v153\n\t"
        "v_fmac_f32 %[h2], %[a0], v154\n\t"
        "v_fmac_f32 %[h3], %[a0], v155\n"
        ".Lcolumns_done_%=:"
        : [h0] "+v"(h0), [h1] "+v"(h1), [h2] "+v"(h2), [h3] "+v"(h3)
        : [live] "s"(live), [single] "s"(single), [at] "v"(row_address), [a0] "v"(a0), [a1] "v"(a1), [a2] "v"(a2), [first] "n"(kFirst),
          [second] "n"(kSecond), [third] "n"(kThird)
        : "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "scc");
}
#else
template <int kFirst, int kSecond, int kThird>
__device__ __forceinline__ void add_columns_if(uint32_t live, uint32_t single, uint32_t row_address, float a0, float a1, float a2, float& h0,
                                               float& h1, float& h2, float& h3) {
    asm volatile(
        "s_cmp_eq_u32 %[live], 0\n\t"
        "s_cbranch_scc1 .Lcolumns_done_%=\n\t"
        "s_cmp_eq_u32 %[single], 0\n\t"
        "s_cbranch_scc0 .Lcolumns_single_%=\n\t"
        "ds_read_b128 v[244:247], %[at] offset:%[first]\n\t"
        "ds_read_b128 v[248:251], %[at] offset:%[second]\n\t"
        "ds_read_b128 v[252:255], %[at] offset:%[third]\n\t"
        "s_waitcnt lgkmcnt(2)\n\t"
        "v_mul_f32 v244, %[a0], v244\n\t"
        "v_mul_f32 v245, %[a0], v245\n\t"
        "v_mul_f32 v246, %[a0], v246\n\t"
        "v_mul_f32 v247, %[a0], v247\n\t"
        "s_waitcnt lgkmcnt(1)\n\t"
        "v_fmac_f32 v244, %[a1], v248\n\t"
        "v_fmac_f32 v245, %[a1], v249\n\t"
        "v_fmac_f32 v246, %[a1], v250\n\t"
        "v_fmac_f32 v247, %[a1], v251\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        "v_fmac_f32 v244, %[a2], v252\n\t"
        "v_fmac_f32 v245, %[a2], v253\n\t"
        "v_fmac_f32 v246, %[a2], v254\n\t"
        "v_fmac_f32 v247, %[a2], v255\n\t"
        "v_add_f32 %[h0], %[h0], v244\n\t"
        "v_add_f32 %[h1], %[h1], v245\n\t"
        "v_add_f32 %[h2], %[h2], v246\n\t"
        "v_add_f32 %[h3], %[h3], v247\n\t"
        "s_branch .Lcolumns_done_%=\n"
        ".Lcolumns_single_%=:\n\t"
        "ds_read_b128 v[244:247], %[at] offset:%[first]\n\t"
        "s_waitcnt lgkmcnt(0)\n\t"
        "v_fmac_f32 %[h0], %[a0], v244\n\t"
        "v_fmac_f32 %[h1], %[a0], v245\n\t"
        "v_fmac_f32 %[h2], %[a0], v246\n\t"
        "v_fmac_f32 %[h3], %[a0], v247\n"
        ".Lcolumns_done_%=:"
        : [h0] "+v"(h0), [h1] "+v"(h1), [h2] "+v"(h2), [h3] "+v"(h3)
        : [live] "s"(live), [single] "s"(single), [at] "v"(row_address), [a0] "v"(a0), [a1] "v"(a1), [a2] "v"(a2), [first] "n"(kFirst),
          [second] "n"(kSecond), [third] "n"(kThird)
        : "v244", "v245", "v246", "v247", "v248", "v249", "v250", "v251", "v252", "v253", "v254", "v255", "scc");
}
#endif
template <int N, int... Q>
__device__ __forceinline__ void add_column_groups(std::integer_sequence<int, Q...>, uint64_t columns, uint32_t single, uint32_t row_address,
                                                  float a0, float a1, float a2, float (&hrow)[N]) {
    // the mask and the flag are uniform; the lane read says so where they come out of LDS
    const uint32_t low = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(columns))));
    const uint32_t high = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(columns >> 32u))));
    const uint64_t uniform_columns = (uint64_t(high) << 32u) | uint64_t(low);
    single = uint32_t(__builtin_amdgcn_readfirstlane(int(single)));
    (add_columns_if<16 * Q, 16 * Q + 4 * N, 16 * Q + 8 * N>(uint32_t(uniform_columns >> (4 * Q)) & 0xFu, single, row_address, a0, a1, a2, hrow[4 * Q],
                                                            hrow[4 * Q + 1], hrow[4 * Q + 2], hrow[4 * Q + 3]), ...);
}

// One head's part of the block: g += J^T f and H += J^T C J for lane's row, skipping the column blocks the head's
// Jacobian rows leave at exact zero.  All head values are uniform.  Widths that run two waves a SIMD update the row
// through add_columns_if, wider ones through the plain loops.
template <int N>
__device__ __forceinline__ void add_head(const Tile& c, uint32_t h, bool coordinate, const float (&f)[3], const float (&cv)[6],
                                         const float (&noise)[3], uint32_t axes, uint64_t columns, float (&hrow)[N], TileSum& g,
                                         float& scale) {
    const float* j0r = c.jac + c.U(hRow, h) * uint32_t(N);
    // (the lane's words read whether or not it is a coordinate: a read under a condition compiles to a branch a word)
    const uint32_t column = c.lane < uint32_t(N) ? c.lane : uint32_t(N - 1);
    const float w0 = j0r[column];
    const float j0 = coordinate ? w0 : 0.0f;
    tile_add_product(g, j0, f[0]);
    scale += fabsf(j0) * noise[0];
    const float4* r0 = reinterpret_cast<const float4*>(j0r);
    if constexpr (N <= kTwoWaveWidth) {
        float a0 = j0 * cv[0], a1 = 0.0f, a2 = 0.0f;
        if (axes != 1u) {
            const float w1 = j0r[N + column], w2 = j0r[2 * N + column];
            const float j1 = coordinate ? w1 : 0.0f, j2 = coordinate ? w2 : 0.0f;
            const float cxx = cv[0], cyy = cv[1], czz = cv[2], cxy = cv[3], cxz = cv[4], cyz = cv[5];
            tile_add_product(g, j1, f[1]);
            tile_add_product(g, j2, f[2]);
            scale += fabsf(j1) * noise[1] + fabsf(j2) * noise[2];
            a0 = (j0 * cxx + j1 * cxy) + j2 * cxz;
            a1 = (j1 * cyy + j2 * cyz) + j0 * cxy;
            a2 = (j2 * czz + j1 * cyz) + j0 * cxz;
        }
        add_column_groups<N>(std::make_integer_sequence<int, N / 4>{}, columns, axes == 1u ? 1u : 0u, lds_address(j0r), a0, a1, a2, hrow);
        return;
    }
    if (axes == 1u) {
        const float a0 = j0 * cv[0];
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
            if (((columns >> (4 * q)) & 0xFull) == 0ull) continue;
            const float4 x0 = r0[q];
            hrow[4 * q] = fmaf(a0, x0.x, hrow[4 * q]); hrow[4 * q + 1] = fmaf(a0, x0.y, hrow[4 * q + 1]);
            hrow[4 * q + 2] = fmaf(a0, x0.z, hrow[4 * q + 2]); hrow[4 * q + 3] = fmaf(a0, x0.w, hrow[4 * q + 3]);
        }
        return;
    }
    const float* j1r = j0r + N, *j2r = j0r + 2 * N;
    const float j1 = coordinate ? j1r[c.lane] : 0.0f, j2 = coordinate ? j2r[c.lane] : 0.0f;
    const float cxx = cv[0], cyy = cv[1], czz = cv[2], cxy = cv[3], cxz = cv[4], cyz = cv[5];
    tile_add_product(g, j1, f[1]);
    tile_add_product(g, j2, f[2]);
    scale += fabsf(j1) * noise[1] + fabsf(j2) * noise[2];
    const float a0 = (j0 * cxx + j1 * cxy) + j2 * cxz;
    const float a1 = (j1 * cyy + j2 * cyz) + j0 * cxy;
    const float a2 = (j2 * czz + j1 * cyz) + j0 * cxz;
    const float4* r1 = reinterpret_cast<const float4*>(j1r);
    const float4* r2 = reinterpret_cast<const float4*>(j2r);
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
        if (((columns >> (4 * q)) & 0xFull) == 0ull) continue;
        const float4 x0 = r0[q], x1 = r1[q], x2 = r2[q];
        hrow[4 * q] += fmaf(a2, x2.x, fmaf(a1, x1.x, a0 * x0.x));
        hrow[4 * q + 1] += fmaf(a2, x2.y, fmaf(a1, x1.y, a0 * x0.y));
        hrow[4 * q + 2] += fmaf(a2, x2.z, fmaf(a1, x1.z, a0 * x0.z));
        hrow[4 * q + 3] += fmaf(a2, x2.w, fmaf(a1, x1.w, a0 * x0.w));
    }
}

// v[lane & 31] + v[32 + (lane & 31)] in every lane: the two halves of the wavefront swapped against each other
__device__ __forceinline__ float halves_sum(float v) {
    const auto pair = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(pair[0]) + __uint_as_float(pair[1]);
}
__device__ __forceinline__ double halves_sum(double v) {
    const uint64_t bits = uint64_t(__double_as_longlong(v));
    const auto low = __builtin_amdgcn_permlane32_swap(uint32_t(bits), uint32_t(bits), false, false);
    const auto high = __builtin_amdgcn_permlane32_swap(uint32_t(bits >> 32u), uint32_t(bits >> 32u), false, false);
    return __longlong_as_double((long long)((uint64_t(high[0]) << 32u) | uint64_t(low[0]))) +
           __longlong_as_double((long long)((uint64_t(high[1]) << 32u) | uint64_t(low[1])));
}

// Two heads in one pass, for blocks of at most 32 coordinates: lanes 0..31 add head `ha` to their rows, lanes 32..63
// add head `hb` (kInvalid: none) to rows of their own that start at zero, row = lane & 31 in both halves; the caller
// sums the halves afterwards (halves_sum).  A head's values come from its own lane (lane = head) through the lane
// permute, its Jacobian words from the head's own rows in LDS; a column group is taken when either head reaches it
// (the other then adds exact zeros).  The sums add in another order than head after head: the last place may differ.
template <int N>
__device__ __forceinline__ void add_head_pair(const Tile& c, uint32_t ha, uint32_t hb, const float (&mf)[3], const float (&mc)[6], const float (&mn)[3],
                                              uint32_t my_first, uint32_t my_low, uint32_t my_high, float (&hrow)[N], TileSum& g, float& scale) {
    static_assert(N <= 32, "both halves of the wavefront hold every row");
    const uint32_t row = c.lane & 31u;
    const bool none = c.lane >= 32u && hb == kInvalid;
    const int source = int(c.lane >= 32u ? (hb == kInvalid ? ha : hb) : ha);
    float f[3], cv[6], noise[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) { f[k] = __shfl(mf[k], source, kWave); noise[k] = __shfl(mn[k], source, kWave); }
#pragma unroll
    for (int k = 0; k < 6; ++k) cv[k] = __shfl(mc[k], source, kWave);
    const uint32_t first = uint32_t(__shfl(int(my_first), source, kWave));
    const float* j0r = c.jac + first * uint32_t(N);
    const bool live = !none && row < c.n;
    // (read whether or not the lane uses them: a read under a condition compiles to a branch a word)
    const uint32_t column = row < uint32_t(N) ? row : uint32_t(N - 1);
    const float w0 = j0r[column], w1 = j0r[N + column], w2 = j0r[2 * N + column];
    const float j0 = live ? w0 : 0.0f, j1 = live ? w1 : 0.0f, j2 = live ? w2 : 0.0f;
    tile_add_product(g, j0, f[0]);
    tile_add_product(g, j1, f[1]);
    tile_add_product(g, j2, f[2]);
    scale += (fabsf(j0) * noise[0] + fabsf(j1) * noise[1]) + fabsf(j2) * noise[2];
    const float cxx = cv[0], cyy = cv[1], czz = cv[2], cxy = cv[3], cxz = cv[4], cyz = cv[5];
    const float a0 = (j0 * cxx + j1 * cxy) + j2 * cxz;
    const float a1 = (j1 * cyy + j2 * cyz) + j0 * cxy;
    const float a2 = (j2 * czz + j1 * cyz) + j0 * cxz;
    uint64_t columns = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_high), int(ha)))) << 32u) |
                       uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_low), int(ha))));
    if (hb != kInvalid)
        columns |= (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_high), int(hb)))) << 32u) |
                   uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_low), int(hb))));
    if constexpr (N <= kTwoWaveWidth) {
        add_column_groups<N>(std::make_integer_sequence<int, N / 4>{}, columns, 0u, lds_address(j0r), a0, a1, a2, hrow);
    } else {
        const float4* r0 = reinterpret_cast<const float4*>(j0r);
        const float4* r1 = reinterpret_cast<const float4*>(j0r + N);
        const float4* r2 = reinterpret_cast<const float4*>(j0r + 2 * N);
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
            if (((columns >> (4 * q)) & 0xFull) == 0ull) continue;
            const float4 x0 = r0[q], x1 = r1[q], x2 = r2[q];
            hrow[4 * q] += fmaf(a2, x2.x, fmaf(a1, x1.x, a0 * x0.x));
            hrow[4 * q + 1] += fmaf(a2, x2.y, fmaf(a1, x1.y, a0 * x0.y));
            hrow[4 * q + 2] += fmaf(a2, x2.z, fmaf(a1, x1.z, a0 * x0.z));
            hrow[4 * q + 3] += fmaf(a2, x2.w, fmaf(a1, x1.w, a0 * x0.w));
        }
    }
}

// Heads a pass where three or four copies of the block's rows fit the wavefront (kGroups<N> of N lanes each): the
// lanes of group g add head `heads[g]` (kInvalid: none) to rows of their own, row = lane - g N; groups past the first
// start at zero and the caller adds the groups' rows together afterwards (groups_sum).  Otherwise as add_head_pair.
template <int N>
constexpr int kGroups = N <= 16 ? 4 : (N <= 20 ? 3 : 2);
template <int N>
__device__ __forceinline__ void add_head_group(const Tile& c, const uint32_t (&heads)[4], const float (&mf)[3], const float (&mc)[6],
                                               const float (&mn)[3], uint32_t my_first, uint32_t my_low, uint32_t my_high, float (&hrow)[N],
                                               TileSum& g, float& scale) {
    constexpr int G = kGroups<N>;
    static_assert(G >= 3 && G * N <= 64, "three or four copies of the rows fit the wavefront");
    const uint32_t group = c.lane / uint32_t(N), row = c.lane - group * uint32_t(N);
    uint32_t mine = kInvalid;
#pragma unroll
    for (int k = 0; k < G; ++k) mine = group == uint32_t(k) ? heads[k] : mine;
    const bool none = mine == kInvalid;   // also the lanes past the last group
    const int source = int(none ? heads[0] : mine);
    float f[3], cv[6], noise[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) { f[k] = __shfl(mf[k], source, kWave); noise[k] = __shfl(mn[k], source, kWave); }
#pragma unroll
    for (int k = 0; k < 6; ++k) cv[k] = __shfl(mc[k], source, kWave);
    const uint32_t first = uint32_t(__shfl(int(my_first), source, kWave));
    const float* j0r = c.jac + first * uint32_t(N);
    const bool live = !none && row < c.n;
    const uint32_t column = row < uint32_t(N) ? row : uint32_t(N - 1);
    const float w0 = j0r[column], w1 = j0r[N + column], w2 = j0r[2 * N + column];
    const float j0 = live ? w0 : 0.0f, j1 = live ? w1 : 0.0f, j2 = live ? w2 : 0.0f;
    tile_add_product(g, j0, f[0]);
    tile_add_product(g, j1, f[1]);
    tile_add_product(g, j2, f[2]);
    scale += (fabsf(j0) * noise[0] + fabsf(j1) * noise[1]) + fabsf(j2) * noise[2];
    const float cxx = cv[0], cyy = cv[1], czz = cv[2], cxy = cv[3], cxz = cv[4], cyz = cv[5];
    const float a0 = (j0 * cxx + j1 * cxy) + j2 * cxz;
    const float a1 = (j1 * cyy + j2 * cyz) + j0 * cxy;
    const float a2 = (j2 * czz + j1 * cyz) + j0 * cxz;
    uint64_t columns = 0ull;
#pragma unroll
    for (int k = 0; k < G; ++k) {
        if (heads[k] == kInvalid) continue;
        columns |= (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_high), int(heads[k])))) << 32u) |
                   uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_low), int(heads[k]))));
    }
    add_column_groups<N>(std::make_integer_sequence<int, N / 4>{}, columns, 0u, lds_address(j0r), a0, a1, a2, hrow);
}
// v[lane] + v[lane + N] + ... over the groups of add_head_group, in the lanes of the first group
template <int N>
__device__ __forceinline__ float groups_sum(uint32_t lane, float v) {
    float total = v;
#pragma unroll
    for (int k = 1; k < kGroups<N>; ++k) total += __shfl(v, int(lane) + k * N, kWave);
    return total;
}
template <int N>
__device__ __forceinline__ double groups_sum(uint32_t lane, double v) {
    const uint64_t bits = uint64_t(__double_as_longlong(v));
    double total = v;
#pragma unroll
    for (int k = 1; k < kGroups<N>; ++k) {
        const uint32_t low = uint32_t(__shfl(int(uint32_t(bits)), int(lane) + k * N, kWave));
        const uint32_t high = uint32_t(__shfl(int(uint32_t(bits >> 32u)), int(lane) + k * N, kWave));
        total += __longlong_as_double((long long)((uint64_t(high) << 32u) | uint64_t(low)));
    }
    return total;
}

// One head's line-search inputs in registers: nothing in them changes between the probes of one search, and neither
// do the parts of its response that do not depend on the probe (plain_line).
struct HeadLine {
    uint32_t head;
    bool owned, contact, bounded, cone, elliptic;
    float tangent_compliance[2], mu_first;
    float rho, compliance, lower, upper, bound;
    Response response;
    TangentRatios ratios;
    float dual[3], res[3], move[3], step[3];
    float dual_part, radius, rho_radius, radius_y, radius_z, inside_yy, inside_zz;
    ConeAxis y, z;
};
__device__ __forceinline__ HeadLine load_head_line(const Tile& c, uint32_t h) {
    HeadLine l{};
    l.head = h;
    l.owned = h < c.heads && c.U(hOwned, h) != 0u;
    if (!l.owned) return l;
    l.contact = block_axes(c.U(hAxes, h));
    l.elliptic = c.elliptic && c.U(hAxes, h) == kAxesElliptic;
    if (l.elliptic) { l.tangent_compliance[0] = c.F(hTangentCompliance, h); l.tangent_compliance[1] = c.F(hTangentCompliance + 1, h); l.mu_first = c.F(hMu1, h); }
    l.rho = c.F(hRho, h); l.compliance = c.F(hCompliance, h); l.lower = c.F(hLower, h); l.upper = c.F(hUpper, h);
    l.bound = c.F(hNormalBound, h);
    l.response = Response{c.F(hDualScale, h), c.F(hResidualScale, h)};
    l.ratios = tangent_ratios(c.F(hMu1, h), c.F(hMu2, h));
#pragma unroll
    for (int k = 0; k < 3; ++k) { l.dual[k] = c.F(hDual + k, h); l.res[k] = c.F(hRes + k, h); l.move[k] = c.F(hMove + k, h); l.step[k] = c.F(hStep + k, h); }
    l.bounded = l.lower < l.upper;
    l.dual_part = l.response.dual_scale * l.dual[0];
    if (l.contact) {
        l.radius = (l.bound < 0.0f ? 0.0f : l.bound) * fmaxf(l.ratios.scale, 0.0f);
        l.cone = l.radius != 0.0f;
        l.y = cone_axis(l.dual[1], l.rho, l.ratios.mu_y);
        l.z = cone_axis(l.dual[2], l.rho, l.ratios.mu_z);
        l.rho_radius = l.rho * l.radius;
        l.radius_y = l.ratios.mu_y * l.radius; l.radius_z = l.ratios.mu_z * l.radius;
        l.inside_yy = l.rho * l.ratios.mu_y * l.ratios.mu_y; l.inside_zz = l.rho * l.ratios.mu_z * l.ratios.mu_z;
    }
    return l;
}

// What the rounding of a head's residual and trial move does to its term of the slope: the impulse is curvature times
// (residual - move) plus a constant, so each of the two carries its own ulp into the impulse at the rate of the
// curvature - the noise the reference's block assembly allows its forces (AssembleTileBlock :1568-1572: impulse plus
// curvature times (|residual| + |move|)).  The reference's line search measures its slopes against the impulses alone
// (:2075-2083): where a stiff row nearly cancels its residual the slope then moves in steps many times the tolerance, no
// point of the line meets it, and the search halves its bracket down to one ulp, some twenty probes for nothing.
// Here the tolerance sees that noise; the accepted step differs from the reference's below the slope's own rounding.
__device__ __forceinline__ float line_noise(const float (&r)[6], float rx, float ry, float rz, float mx, float my, float mz, float sx, float sy, float sz) {
    return r[0] * (fabsf(rx) + fabsf(mx)) * fabsf(sx) + r[1] * (fabsf(ry) + fabsf(my)) * fabsf(sy) + r[2] * (fabsf(rz) + fabsf(mz)) * fabsf(sz);
}
__device__ __forceinline__ void add_line_terms(const float (&f)[3], const float (&r)[6], float sx, float sy, float sz, TileSum& row_slope,
                                               float& row_curvature, float& row_magnitude) {
    tile_add_product(row_slope, f[0], sx);
    tile_add_product(row_slope, f[1], sy);
    tile_add_product(row_slope, f[2], sz);
    row_magnitude += fabsf(f[0] * sx) + fabsf(f[1] * sy) + fabsf(f[2] * sz);
    row_curvature += r[0] * sx * sx + r[1] * sy * sy + r[2] * sz * sz + 2.0f * r[5] * sy * sz + 2.0f * r[3] * sx * sy +
                     2.0f * r[4] * sx * sz;
}
// TileLineDerivatives (:2048-2086); lane = head, heads beyond the first 64 go through `extra`
__device__ __forceinline__ void line_terms(const HeadLine& l, float alpha, TileSum& row_slope, float& row_curvature, float& row_magnitude) {
    const float sx = l.step[0], sy = l.step[1], sz = l.step[2];
    float f[3] = {0.0f, 0.0f, 0.0f}, r[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (l.elliptic) {
        elliptic_impulse(V3{l.dual[0], l.dual[1], l.dual[2]}, l.rho, l.res[0] - fmaf(alpha, sx, l.move[0]), l.res[1] - fmaf(alpha, sy, l.move[1]),
                         l.res[2] - fmaf(alpha, sz, l.move[2]), l.compliance, l.tangent_compliance[0], l.tangent_compliance[1], l.mu_first, f, r);
        add_line_terms(f, r, sx, sy, sz, row_slope, row_curvature, row_magnitude);
        row_magnitude += line_noise(r, l.res[0], l.res[1], l.res[2], fmaf(alpha, sx, l.move[0]), fmaf(alpha, sy, l.move[1]), fmaf(alpha, sz, l.move[2]), sx, sy, sz);
        return;
    }
    scalar_impulse(l.dual[0], l.rho, l.res[0] - fmaf(alpha, sx, l.move[0]), l.compliance, l.lower, l.upper, l.response, &f[0], &r[0]);
    if (l.contact)
        tangent_impulse(V3{l.dual[0], l.dual[1], l.dual[2]}, l.rho, l.res[1] - fmaf(alpha, sy, l.move[1]),
                        l.res[2] - fmaf(alpha, sz, l.move[2]), l.bound, l.ratios, &f[1], &f[2], &r[1], &r[2], &r[5]);
    add_line_terms(f, r, sx, sy, sz, row_slope, row_curvature, row_magnitude);
    row_magnitude += line_noise(r, l.res[0], l.res[1], l.res[2], fmaf(alpha, sx, l.move[0]), fmaf(alpha, sy, l.move[1]), fmaf(alpha, sz, l.move[2]), sx, sy, sz);
}
// A head's line-search constants as numbers only, so that the probes run without a branch: every selection the
// response makes on a constant of the head (a single-axis head has no tangent part, a friction ratio of zero takes no
// cone argument, a cone of radius zero gives no tangent impulse and no curvature) is made here once, by handing the
// probe constants on which the general formulas give those results exactly - zeros for what must come out as zero.
// A lane without an owned head gets zeros throughout and adds exact zeros to every sum.
// The cone argument dual / mu + rho mu residual (ConeArgument, augmented_row.hpp:302-318) is kept by the reference as
// compensated float pairs; here the same two constants are doubles (the sums of the reference's pairs) and the
// argument is one double multiply-add.  Everything but `move` and `step` is constant over a block descent.
struct PlainLine {
    float k, k_bounded, dual_part, lower, upper;
    float res[3], move[3], step[3];
    double cone_y, cone_z, gain_y, gain_z;
    float mu_y, mu_z, radius, rho_radius, radius_y, radius_z, inside_yy, inside_zz;
    uint32_t head;   // the head the constants belong to, kInvalid for none: `move` and `step` are then never read
};
__device__ __forceinline__ PlainLine plain_line(const HeadLine& l) {
    PlainLine p{};
    p.head = kInvalid;
    if (!l.owned || l.rho <= 0.0f) return p;   // no penalty: no impulse and no curvature (scalar_impulse, tangent_impulse)
    p.head = l.head;
    p.k = l.response.residual_scale; p.k_bounded = l.bounded ? p.k : 0.0f; p.dual_part = l.dual_part; p.lower = l.lower; p.upper = l.upper;
#pragma unroll
    for (int k = 0; k < 3; ++k) { p.res[k] = l.res[k]; p.move[k] = l.move[k]; p.step[k] = l.step[k]; }
    // a constant that is not a number makes the general response not a number; here it is handed on through the sum
    if (!(l.rho == l.rho && l.dual[0] == l.dual[0] && l.compliance == l.compliance && l.lower == l.lower && l.upper == l.upper)) p.dual_part = nanf("");
    if (!l.contact) return p;
    p.mu_y = l.ratios.mu_y; p.mu_z = l.ratios.mu_z;
    if (p.mu_y != 0.0f) { p.cone_y = double(l.y.dd) + double(l.y.d_low); p.gain_y = double(l.y.p) + double(l.y.p_low); }
    if (p.mu_z != 0.0f) { p.cone_z = double(l.z.dd) + double(l.z.d_low); p.gain_z = double(l.z.p) + double(l.z.p_low); }
    p.radius = l.radius; p.rho_radius = l.rho_radius; p.radius_y = l.radius_y; p.radius_z = l.radius_z;
    if (l.cone) { p.inside_yy = l.inside_yy; p.inside_zz = l.inside_zz; }
    return p;
}
// The response of a head from its constants: scalar_impulse and tangent_impulse operation for operation, both sides
// of the cone computed and one selected, the three quotients by the tangent norm sharing one reciprocal (the answers
// differ from the general functions' in the last place or two).  A residual
// that is not a number comes out as an impulse that is not a number, as in the general functions.  plain_line_terms
// is TileLineDerivatives (:2048-2086) on it, with at most one head a lane.
__device__ __forceinline__ void plain_response(const PlainLine& p, float mx, float my, float mz, float (&f)[3], float (&r)[6]) {
    const float x = fmaf(p.k, p.res[0] - mx, p.dual_part);
    f[0] = x < p.lower ? p.lower : (x > p.upper ? p.upper : x);
    r[0] = x >= p.lower && x <= p.upper ? p.k_bounded : 0.0f;
    const float q_y = float(fma(p.gain_y, double(p.res[1] - my), p.cone_y));
    const float q_z = float(fma(p.gain_z, double(p.res[2] - mz), p.cone_z));
    // the norm and its reciprocal by the hardware root and reciprocal (an ulp each): impulses lie far inside the range
    // where the squares neither overflow nor vanish
    const float norm = __builtin_amdgcn_sqrtf(fmaf(q_y, q_y, q_z * q_z));
    const bool inside = norm <= p.radius;
    const float by_norm = __builtin_amdgcn_rcpf(inside ? 1.0f : norm);
    const float dy = q_y * by_norm, dz = q_z * by_norm, cs = p.rho_radius * by_norm;
    f[1] = inside ? p.mu_y * q_y : p.radius_y * dy;
    f[2] = inside ? p.mu_z * q_z : p.radius_z * dz;
    r[1] = inside ? p.inside_yy : cs * p.mu_y * p.mu_y * dz * dz;
    r[2] = inside ? p.inside_zz : cs * p.mu_z * p.mu_z * dy * dy;
    r[3] = 0.0f; r[4] = 0.0f;
    r[5] = inside ? 0.0f : -cs * p.mu_y * p.mu_z * dy * dz;
}
// The constants of lane's own head for one block descent.  With at most sixteen heads the four rows of sixteen lanes
// hold copies of the heads (lane & 15), which the line search uses to evaluate several points of a line in one pass;
// the block assembly then takes the copies of the first row only.  `move` and `step` change with every Newton step
// and are read again where they are used.
// Widths whose register rows leave room keep the constants in registers over the whole block descent; the others
// (28 to 36, at two waves a SIMD) compute them again at each use, which costs less than the spills would.
template <int N>
constexpr bool kKeepLine = N <= 24 || N > kTwoWaveWidth;
__device__ __forceinline__ PlainLine own_line(const Tile& c) {
    return plain_line(load_head_line(c, c.heads <= 16u ? (c.lane & 15u) : c.lane));
}
__device__ __forceinline__ void refresh_moves(const Tile& c, PlainLine& p) {
    if (p.head == kInvalid) return;
#pragma unroll
    for (int k = 0; k < 3; ++k) p.move[k] = c.F(hMove + k, p.head);
}
__device__ __forceinline__ void refresh_steps(const Tile& c, PlainLine& p) {
    if (p.head == kInvalid) return;
#pragma unroll
    for (int k = 0; k < 3; ++k) { p.move[k] = c.F(hMove + k, p.head); p.step[k] = c.F(hStep + k, p.head); }
}
// A head's response at its current move with the rounding noise of each axis; false when nothing of it is non-zero.
__device__ __forceinline__ bool head_terms(const Tile& c, uint32_t h, float (&f)[3], float (&cv)[6], float (&noise)[3]) {
#pragma unroll
    for (int k = 0; k < 3; ++k) { f[k] = 0.0f; noise[k] = 0.0f; }
#pragma unroll
    for (int k = 0; k < 6; ++k) cv[k] = 0.0f;
    if (h >= c.heads || c.U(hOwned, h) == 0u) return false;
    head_response(c, h, c.F(hMove, h), c.F(hMove + 1, h), c.F(hMove + 2, h), f, cv);
#pragma unroll
    for (int k = 0; k < 3; ++k) noise[k] = fabsf(f[k]) + cv[k] * (fabsf(c.F(hRes + k, h)) + fabsf(c.F(hMove + k, h)));
    return f[0] != 0.0f || f[1] != 0.0f || f[2] != 0.0f || cv[0] != 0.0f || cv[1] != 0.0f || cv[2] != 0.0f || cv[5] != 0.0f ||
           cv[3] != 0.0f || cv[4] != 0.0f || noise[0] != 0.0f || noise[1] != 0.0f || noise[2] != 0.0f;
}

__device__ __forceinline__ float uniform_lane_value(float v, uint32_t lane) {   // `lane` is uniform, not a constant
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), int(lane)));
}

// The heads' part of the force only: g += J^T f for lane's coordinate, with the rounding scale of that sum.  A staged
// head has three rows in LDS whatever its axes (those it does not have hold zeros, as its response does), and the
// padded columns hold zeros: every head reads its three words without a condition, the next head's ahead of this
// one's arithmetic.  lane = head on the way in (mf, mn, my_first), lane = coordinate for the sums.
template <int N>
__device__ __forceinline__ void add_heads_force(const Tile& c, uint64_t heads, const float (&mf)[3], const float (&mn)[3], uint32_t my_first,
                                                TileSum& g, float& scale) {
    const uint32_t column = c.lane < uint32_t(N) ? c.lane : uint32_t(N - 1);
    auto rows_of = [&](uint32_t h, float (&j)[3]) {
        const float* at = c.jac + uint32_t(__builtin_amdgcn_readlane(int(my_first), int(h))) * uint32_t(N) + column;
        j[0] = at[0]; j[1] = at[N]; j[2] = at[2 * N];
    };
    float next[3] = {0.0f, 0.0f, 0.0f};
    if (heads != 0ull) rows_of(uint32_t(__builtin_ctzll(heads)), next);
    while (heads != 0ull) {
        const uint32_t h = uint32_t(__builtin_ctzll(heads));
        heads &= heads - 1ull;
        const float j[3] = {next[0], next[1], next[2]};
        if (heads != 0ull) rows_of(uint32_t(__builtin_ctzll(heads)), next);
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            tile_add_product(g, j[k], uniform_lane_value(mf[k], h));
            scale += fabsf(j[k]) * uniform_lane_value(mn[k], h);
        }
    }
}

// Blocks that keep no contact rows (Tile::from_links).  Entry j of a head's row is s_j . w where j lies on the head's
// way to the root, s_j the coordinate's motion axis (Tile::axes) and w the row's wrench (Tile::wrench); elsewhere zero.
// lane = head: the motion of the head's link, sum over the coordinates j on its way of s_j x_j, for a vector x in LDS.
template <int N>
__device__ __forceinline__ void link_motion(const Tile& c, uint64_t way, const float* x, float (&motion)[6]) {
    const float4* table = reinterpret_cast<const float4*>(c.axes);
    const float4* x4 = reinterpret_cast<const float4*>(x);
#pragma unroll
    for (int k = 0; k < 6; ++k) motion[k] = 0.0f;
    // a loop that stays a loop: unrolled, all of the table is fetched ahead of the first product, into registers the
    // block does not have
#pragma unroll 1
    for (uint32_t q = 0u; q < uint32_t(N / 4); ++q) {
        const float4 xq = x4[q];
        const float xs[4] = {xq.x, xq.y, xq.z, xq.w};
        const uint32_t four = uint32_t(way >> (4u * q)) & 0xFu;
#pragma unroll
        for (uint32_t t = 0u; t < 4u; ++t) {
            const float4 a = table[3u * (4u * q + t)], b = table[3u * (4u * q + t) + 1u];
            const float on = ((four >> t) & 1u) != 0u ? xs[t] : 0.0f;
            motion[0] = fmaf(a.x, on, motion[0]); motion[1] = fmaf(a.y, on, motion[1]); motion[2] = fmaf(a.z, on, motion[2]);
            motion[3] = fmaf(a.w, on, motion[3]); motion[4] = fmaf(b.x, on, motion[4]); motion[5] = fmaf(b.y, on, motion[5]);
        }
    }
}
// lane = head: row `axis` of head h times the vector whose link motion is `motion`
__device__ __forceinline__ float wrench_dot(const Tile& c, uint32_t h, uint32_t axis, const float (&motion)[6]) {
    const float* w = c.wrench + h * kWrenchStride + 6u * axis;
    return fmaf(w[5], motion[5], fmaf(w[4], motion[4], fmaf(w[3], motion[3], fmaf(w[2], motion[2], fmaf(w[1], motion[1], w[0] * motion[0])))));
}
__device__ __forceinline__ uint64_t way_of(const Tile& c, uint32_t h) {
    const uint32_t* w = reinterpret_cast<const uint32_t*>(c.wrench + h * kWrenchStride + 18u);
    return (uint64_t(w[1]) << 32u) | uint64_t(w[0]);
}
// lane = coordinate: sum over the heads `heads` (a uniform mask of the first 64) of J^T x, x one value an axis held by
// lane = head, in double: the heads' wrenches weighted by x summed over the heads whose way holds the coordinate, then
// taken against the coordinate's motion axis.  With `weights` (the magnitudes that go with x) also the rounding scale
// of that sum, an upper bound: sum |s_j| . sum |w| weights.
template <bool kScale>
__device__ __forceinline__ double rows_transposed_times(const Tile& c, uint64_t heads, const float (&x)[3], const float (&weights)[3], float* scale) {
    const uint32_t lane = c.lane;
    float sum[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f}, bound[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t way_low = 0u, way_high = 0u;
    if (lane < c.heads && ((heads >> lane) & 1ull) != 0ull) {
        const float* w = c.wrench + lane * kWrenchStride;
#pragma unroll
        for (int k = 0; k < 6; ++k) {
            sum[k] = (w[k] * x[0] + w[6 + k] * x[1]) + w[12 + k] * x[2];
            if constexpr (kScale) bound[k] = (fabsf(w[k]) * weights[0] + fabsf(w[6 + k]) * weights[1]) + fabsf(w[12 + k]) * weights[2];
        }
        const uint64_t way = way_of(c, lane);
        way_low = uint32_t(way); way_high = uint32_t(way >> 32u);
    }
    double carried[6] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
    float carried_bound[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (uint64_t rest = heads; rest != 0ull; rest &= rest - 1ull) {
        const int h = __builtin_ctzll(rest);
        const uint64_t way = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(way_high), h))) << 32u) |
                             uint64_t(uint32_t(__builtin_amdgcn_readlane(int(way_low), h)));
        const float through = ((way >> lane) & 1ull) != 0ull ? 1.0f : 0.0f;
#pragma unroll
        for (int k = 0; k < 6; ++k) {
            carried[k] = fma(double(through), double(uniform_lane_value(sum[k], uint32_t(h))), carried[k]);
            if constexpr (kScale) carried_bound[k] = fmaf(through, uniform_lane_value(bound[k], uint32_t(h)), carried_bound[k]);
        }
    }
    const float4* table = reinterpret_cast<const float4*>(c.axes);
    const float4 a = table[3u * lane], b = table[3u * lane + 1u];
    const float s[6] = {a.x, a.y, a.z, a.w, b.x, b.y};
    double total = 0.0;
#pragma unroll
    for (int k = 0; k < 6; ++k) total = fma(double(s[k]), carried[k], total);
    if constexpr (kScale) {
        float magnitude = 0.0f;
#pragma unroll
        for (int k = 0; k < 6; ++k) magnitude = fmaf(fabsf(s[k]), carried_bound[k], magnitude);
        *scale += magnitude;
    }
    return total;
}

// The heads' curvature sum_h J_h^T C_h J_h by way of the links, for blocks whose staged heads each act through one link.
// A row of such a head is a wrench w = [(p - o) x n; n] about a point o, met by every coordinate j on the way from the
// head's link to the root with its motion axis s_j = [a_j; (r_j - o) x a_j] (a sliding coordinate: [0; a_j]):
// J_j = s_j . w, the entry the row assembly wrote (assemble_rows.cu:122-169).  The head's term in H_ij is therefore
// s_i^T (W C W^T) s_j when both i and j lie on that way, else zero; and of two coordinates that share any head one lies
// on the other's way to the root.  With K_i the sum of W C W^T over the heads whose way to the root holds i - the
// contact stiffness coordinate i carries, as a composite inertia is the inertia it carries -
//     H_ij += (K_i s_i) . s_j   for j on i's way to the root,      (K_j s_j) . s_i   for i on j's,
// which takes 21 words a head and 12 a column where the plain sum over heads takes 3 N words a head.  The two forms
// of one entry multiply and add the same numbers in the same order: the rows stay each other's transposes to the bit.
// lane = head on the way in (mc: its curvature, `mine`: it contributes), lane = coordinate from the sums on.
template <int N>
__device__ __forceinline__ void add_heads_through_links(const Tile& c, bool mine, const float (&mc)[6], float (&hrow)[N]) {
    const uint32_t lane = c.lane;
    float k[21];
#pragma unroll
    for (int e = 0; e < 21; ++e) k[e] = 0.0f;
    uint32_t way_low = 0u, way_high = 0u;
    if (mine) {
        const uint32_t slot = c.U(hSlot, lane), stride = c.U(hStride, lane), axes = c.U(hAxes, lane);
        const bool second = c.U(hSourceA, lane) == kInvalid;   // the side that moves is the row's second
        const uint64_t way = c.from_links ? way_of(c, lane) : c.link_paths[(second ? c.row_link_b : c.row_link_a)[slot] - c.first_link];
        way_low = uint32_t(way); way_high = uint32_t(way >> 32u);
        float w[3][6];
#pragma unroll
        for (uint32_t a = 0u; a < 3u; ++a) {
            if (c.from_links) {
#pragma unroll
                for (int t = 0; t < 6; ++t) w[a][t] = c.wrench[lane * kWrenchStride + 6u * a + uint32_t(t)];
                continue;
            }
#pragma unroll
            for (int t = 0; t < 6; ++t) w[a][t] = 0.0f;
            if (a != 0u && axes == 1u) continue;
            const size_t rs = size_t{slot} + a * stride;
            const float* row = c.rows + rs * kRowWords + 12u;          // the first side's direction; the second side's is its negative,
            const float* at = (second ? c.row_point_b : c.row_point_a) + 3u * rs;   // and W C W^T does not see the sign
            const V3 n{row[0], row[1], row[2]};
            const V3 arm = sub3(V3{at[0], at[1], at[2]}, c.pivot);
            const V3 moment = cross3(arm, n);
            w[a][0] = moment.x; w[a][1] = moment.y; w[a][2] = moment.z; w[a][3] = n.x; w[a][4] = n.y; w[a][5] = n.z;
        }
        const float cxx = mc[0], cyy = mc[1], czz = mc[2], cxy = mc[3], cxz = mc[4], cyz = mc[5];
        float u[3][6];
#pragma unroll
        for (int t = 0; t < 6; ++t) {
            u[0][t] = (cxx * w[0][t] + cxy * w[1][t]) + cxz * w[2][t];
            u[1][t] = (cxy * w[0][t] + cyy * w[1][t]) + cyz * w[2][t];
            u[2][t] = (cxz * w[0][t] + cyz * w[1][t]) + czz * w[2][t];
        }
        int e = 0;
#pragma unroll
        for (int r = 0; r < 6; ++r) {
#pragma unroll
            for (int t = r; t < 6; ++t) k[e++] = (w[0][r] * u[0][t] + w[1][r] * u[1][t]) + w[2][r] * u[2][t];
        }
    }
    // lane = coordinate: the stiffness of every head whose way to the root passes through it
    float carried[21];
#pragma unroll
    for (int e = 0; e < 21; ++e) carried[e] = 0.0f;
    for (uint64_t rest = __ballot(mine); rest != 0ull; rest &= rest - 1ull) {
        const int h = __builtin_ctzll(rest);
        const uint64_t way = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(way_high), h))) << 32u) |
                             uint64_t(uint32_t(__builtin_amdgcn_readlane(int(way_low), h)));
        // one multiply-add an entry with a weight of one or zero: a conditional sum compiles to an add and two copies
        const float through = ((way >> lane) & 1ull) != 0ull ? 1.0f : 0.0f;
#pragma unroll
        for (int e = 0; e < 21; ++e) carried[e] = fmaf(through, uniform_lane_value(k[e], uint32_t(h)), carried[e]);
    }
    float4* table = reinterpret_cast<float4*>(c.axes);
    float s[6], y[6];
    {
        const float4 a = table[3u * lane], b = table[3u * lane + 1u];
        s[0] = a.x; s[1] = a.y; s[2] = a.z; s[3] = a.w; s[4] = b.x; s[5] = b.y;
        // y = K s, K symmetric with its upper triangle in `carried`, rows first
        auto entry = [&](int r, int t) { return r <= t ? carried[r * 6 - r * (r - 1) / 2 + (t - r)] : carried[t * 6 - t * (t - 1) / 2 + (r - t)]; };
#pragma unroll
        for (int r = 0; r < 6; ++r) {
            float sum = entry(r, 0) * s[0];
#pragma unroll
            for (int t = 1; t < 6; ++t) sum = fmaf(entry(r, t), s[t], sum);
            y[r] = sum;
        }
        table[3u * lane + 1u] = float4{b.x, b.y, y[0], y[1]};
        table[3u * lane + 2u] = float4{y[2], y[3], y[4], y[5]};
    }
    __syncthreads();
    // (through the barrier so that the sixty-four lane masks of each are made here, two instructions a column, instead of
    // ahead of the sweeps and kept in scalar registers the kernel does not have)
    const uint64_t path = (uint64_t(opaque_word(c.path_high)) << 32u) | uint64_t(opaque_word(c.path_low));
    const uint64_t under = (uint64_t(opaque_word(c.under_high)) << 32u) | uint64_t(opaque_word(c.under_low));
#pragma unroll
    for (int j = 0; j < N; ++j) {
        const float4 a = table[3 * j], b = table[3 * j + 1], d = table[3 * j + 2];
        // (K_i s_i) . s_j and (K_j s_j) . s_i, each the stiffness-times-axis of the coordinate further from the root first
        const float mine_first = fmaf(y[5], b.y, fmaf(y[4], b.x, fmaf(y[3], a.w, fmaf(y[2], a.z, fmaf(y[1], a.y, y[0] * a.x)))));
        const float other_first = fmaf(d.w, s[5], fmaf(d.z, s[4], fmaf(d.y, s[3], fmaf(d.x, s[2], fmaf(b.w, s[1], b.z * s[0])))));
        const bool on_my_way = ((path >> j) & 1ull) != 0ull, through_me = ((under >> j) & 1ull) != 0ull;
        hrow[j] += on_my_way ? mine_first : (through_me ? other_first : 0.0f);
    }
    __syncthreads();
}

// AssembleTileBlock (:1507-1618): lane i assembles row i of H = M + sum J^T C J in `hrow` and its force g_i.  The
// first 64 heads evaluate their response one per lane and hand it to the row lanes as scalar lane reads; heads beyond
// 64 pass theirs through the head fields.
// In a reduced block (kFollow) the mass row is the sum of two floats, `mrow` and `mlow`: the Schur complement as it comes
// out of the double-precision elimination.  The force takes both parts, so that the velocity the block converges to
// balances the momentum against the mass matrix itself; the Hessian takes the first.
template <int N, bool kFollow>
__device__ __forceinline__ bool assemble_block(const Tile& c, const float (&mrow)[N], const float (&mlow)[N], PlainLine& own, float u, float free_v,
                               float (&hrow)[N], float* force, float* inertia, bool* converged) {
    const uint32_t lane = c.lane;
    const bool coordinate = lane < c.n;
    // the difference of two floats, exact in double (the reference carries it as a float and its rounding error)
    double* dvec = reinterpret_cast<double*>(c.vec);
    float* uvec = c.vec + 128;
    dvec[lane] = double(u) - double(free_v); uvec[lane] = fabsf(u);
    PROF_BEGIN(c, 10);
    // lane's own head (the first 64 heads) from its constants, without a branch; a lane without an owned head gets zeros
    float mf[3], mc[6], mn[3];
    {
        if constexpr (kKeepLine<N>) refresh_moves(c, own);
        else own = own_line(c);
        plain_response(own, own.move[0], own.move[1], own.move[2], mf, mc);
#pragma unroll
        for (int k = 0; k < 3; ++k) mn[k] = fabsf(mf[k]) + mc[k] * (fabsf(own.res[k]) + fabsf(own.move[k]));
    }
    if (c.elliptic) head_terms(c, lane, mf, mc, mn);   // the cone's own response; the same values as above for every other head
    // (lanes from the heads' count on hold copies of the first sixteen heads when there are no more than that)
    const bool mine = lane < c.heads && (mf[0] != 0.0f || mf[1] != 0.0f || mf[2] != 0.0f || mc[0] != 0.0f || mc[1] != 0.0f || mc[2] != 0.0f || mc[5] != 0.0f ||
                      mc[3] != 0.0f || mc[4] != 0.0f || mn[0] != 0.0f || mn[1] != 0.0f || mn[2] != 0.0f);
    const uint32_t my_axes = lane < c.heads ? c.U(hAxes, lane) : 0u;
    const uint32_t my_low = lane < c.heads ? c.U(hColumnsLow, lane) : 0u, my_high = lane < c.heads ? c.U(hColumnsHigh, lane) : 0u;
    // The Hessian M + sum J^T C J changes only through the heads' curvatures: every head keeps the curvature of its
    // last assembly in its fields, and while none differs the factor of the last factorisation still stands.
    bool changed = false;
    for (uint32_t h = lane + kWave; h < c.heads; h += kWave) {
        float f[3], cv[6], noise[3];
        const bool contributes = head_terms(c, h, f, cv, noise);
#pragma unroll
        for (int k = 0; k < 3; ++k) { c.F(hF + k, h) = f[k]; c.F(hNoise + k, h) = noise[k]; }
#pragma unroll
        for (int k = 0; k < 6; ++k) { changed = changed || __float_as_uint(c.F(hC + k, h)) != __float_as_uint(cv[k]); c.F(hC + k, h) = cv[k]; }
        c.U(hContrib, h) = contributes ? 1u : 0u;
    }
    if (lane < c.heads) {
#pragma unroll
        for (int k = 0; k < 6; ++k) { changed = changed || __float_as_uint(c.F(hC + k, lane)) != __float_as_uint(mc[k]); c.F(hC + k, lane) = mc[k]; }
    }
    if (__any(changed)) c.factor_current = false;
    if (c.units && lane < c.heads && c.U(hUnit, lane) != kInvalid) {   // a coordinate reads its unit heads' responses from the fields
        c.F(hF, lane) = mf[0]; c.F(hNoise, lane) = mn[0];
        c.U(hContrib, lane) = mine ? 1u : 0u;
    }
    __syncthreads();
    PROF_END(c, 10);
    PROF_BEGIN(c, 11);
    // Padded columns (k >= n) hold exact zeros in the mass row, the vectors and the Jacobian rows: their terms add
    // nothing to any of the sums below.
    TileSum inertial{0.0};
    double inertial_scale = 0.0;
    const double2* d2 = reinterpret_cast<const double2*>(dvec);
#pragma unroll
    for (int q = 0; q < N / 2; ++q) {
        const double2 dv = d2[q];
        // (the mass rows do not change over the solve: left to itself the compiler widens them to double once, ahead of
        // the sweeps, and holds two registers an entry from there on - which pays while they fit, and a wide block
        // has no room for)
        const double m0 = double(N >= kWidenAtUse ? opaque_with(mrow[2 * q], u) : mrow[2 * q]);
        const double m1 = double(N >= kWidenAtUse ? opaque_with(mrow[2 * q + 1], u) : mrow[2 * q + 1]);
        hrow[2 * q] = mrow[2 * q]; hrow[2 * q + 1] = mrow[2 * q + 1];
        inertial.value = fma(m0, dv.x, inertial.value);
        inertial.value = fma(m1, dv.y, inertial.value);
        if constexpr (kFollow) {
            // (the low parts widened here, at every assembly: held widened over the solve beside the high parts they
            // take the block past its registers)
            inertial.value = fma(double(opaque_with(mlow[2 * q], u)), dv.x, inertial.value);
            inertial.value = fma(double(opaque_with(mlow[2 * q + 1], u)), dv.y, inertial.value);
        }
        inertial_scale = fma(fabs(m0), fabs(dv.x), inertial_scale);
        inertial_scale = fma(fabs(m1), fabs(dv.y), inertial_scale);
    }
    float scale = float(inertial_scale);
    TileSum g{-inertial.value};
    PROF_END(c, 11);
    PROF_BEGIN(c, 12);
    bool paired = false, grouped = false;
    if constexpr (N <= 32) {
        // two or more contributing heads (all of them staged, one a lane): two a pass, the second half of the
        // wavefront collecting its heads in rows of its own
        const uint64_t all = __ballot(mine);
        paired = !c.units && c.heads <= uint32_t(kWave) && (all & (all - 1ull)) != 0ull;
        if constexpr (N <= 20 && N <= kTwoWaveWidth) {
            // where three or four copies of the rows fit the wavefront, that many heads a pass - when it takes fewer
            // passes than two a pass would (adding the groups' rows together costs more than adding two halves)
            const int contributing = __popcll(all);
            if (paired && (contributing + kGroups<N> - 1) / kGroups<N> < (contributing + 1) / 2) {
                if (lane >= uint32_t(N)) {
#pragma unroll
                    for (int k = 0; k < N; ++k) hrow[k] = 0.0f;
                    g.value = 0.0; scale = 0.0f;
                }
                const uint32_t my_first = lane < c.heads ? c.U(hRow, lane) : 0u;
                for (uint64_t rest = all; rest != 0ull;) {
                    uint32_t taken[4] = {kInvalid, kInvalid, kInvalid, kInvalid};
#pragma unroll
                    for (int k = 0; k < kGroups<N>; ++k) {
                        if (rest == 0ull) break;
                        taken[k] = uint32_t(__builtin_ctzll(rest));
                        rest &= rest - 1ull;
                    }
                    add_head_group<N>(c, taken, mf, mc, mn, my_first, my_low, my_high, hrow, g, scale);
                }
#pragma unroll
                for (int k = 0; k < N; ++k) hrow[k] = groups_sum<N>(lane, hrow[k]);
                g.value = groups_sum<N>(lane, g.value); scale = groups_sum<N>(lane, scale);
                grouped = true;
            }
        }
        if (paired && !grouped) {
            if (lane >= 32u) {
#pragma unroll
                for (int k = 0; k < N; ++k) hrow[k] = 0.0f;
                g.value = 0.0; scale = 0.0f;
            }
            const uint32_t my_first = lane < c.heads ? c.U(hRow, lane) : 0u;
            for (uint64_t rest = all; rest != 0ull;) {
                const uint32_t ha = uint32_t(__builtin_ctzll(rest));
                rest &= rest - 1ull;
                const uint32_t hb = rest != 0ull ? uint32_t(__builtin_ctzll(rest)) : kInvalid;
                rest &= rest - 1ull;   // zero stays zero
                add_head_pair<N>(c, ha, hb, mf, mc, mn, my_first, my_low, my_high, hrow, g, scale);
            }
#pragma unroll
            for (int k = 0; k < N; ++k) hrow[k] = halves_sum(hrow[k]);
            g.value = halves_sum(g.value); scale = halves_sum(scale);
        }
    }
    if (paired) {
    } else if (N > kTwoWaveWidth && c.from_links) {
        if (__ballot(mine) != 0ull) {
            float weighted = 0.0f;
            g.value += rows_transposed_times<true>(c, __ballot(mine), mf, mn, &weighted);
            scale += weighted;
            add_heads_through_links<N>(c, mine, mc, hrow);
        }
    } else if (N > kTwoWaveWidth && c.through_links && __popcll(__ballot(mine)) >= int(kLinkHeads)) {
        // enough heads that their curvature is cheaper by way of the links; the force takes the staged rows as ever
        add_heads_force<N>(c, __ballot(mine), mf, mn, lane < c.heads ? c.U(hRow, lane) : 0u, g, scale);
        add_heads_through_links<N>(c, mine, mc, hrow);
    } else if (!c.units) {   // staged heads only: plain head order
        for (uint64_t rest = __ballot(mine); rest != 0ull; rest &= rest - 1ull) {
            const uint32_t h = uint32_t(__builtin_ctzll(rest));
            float f[3], cv[6], noise[3];
#pragma unroll
            for (int k = 0; k < 3; ++k) { f[k] = uniform_lane_value(mf[k], h); noise[k] = uniform_lane_value(mn[k], h); }
#pragma unroll
            for (int k = 0; k < 6; ++k) cv[k] = uniform_lane_value(mc[k], h);
            const uint32_t axes = uint32_t(__builtin_amdgcn_readlane(int(my_axes), int(h)));
            const uint64_t columns = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_high), int(h)))) << 32u) |
                                     uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_low), int(h))));
            add_head<N>(c, h, coordinate, f, cv, noise, axes, columns, hrow, g, scale);
        }
        for (uint32_t h = kWave; h < c.heads; ++h) {
            if (c.U(hContrib, h) == 0u) continue;
            const float f[3] = {c.F(hF, h), c.F(hF + 1, h), c.F(hF + 2, h)};
            const float cv[6] = {c.F(hC, h), c.F(hC + 1, h), c.F(hC + 2, h), c.F(hC + 3, h), c.F(hC + 4, h), c.F(hC + 5, h)};
            const float noise[3] = {c.F(hNoise, h), c.F(hNoise + 1, h), c.F(hNoise + 2, h)};
            const uint64_t columns = (uint64_t(__builtin_amdgcn_readfirstlane(c.U(hColumnsHigh, h))) << 32u) |
                                     uint64_t(__builtin_amdgcn_readfirstlane(c.U(hColumnsLow, h)));
            add_head<N>(c, h, coordinate, f, cv, noise, c.U(hAxes, h), columns, hrow, g, scale);
        }
    } else {
        // The heads add in the reference's order (:1533-1603): 32 at a time, and within each 32 the unit heads - a row on
        // one coordinate adds to that coordinate's diagonal and force only - before the staged ones.  Chunks past the
        // last staged head hold unit heads only and go in one pass.
        float diagonal = 0.0f;
        uint32_t next = 0u;
        const uint64_t contributing = __ballot(mine);
        const uint64_t unit_heads = __ballot(lane < c.heads && c.U(hUnit, lane) != kInvalid);
        auto add_unit = [&](uint32_t h) {
            const float v = c.F(hUnitValue, h);
            diagonal += v * c.F(hC, h) * v;
            tile_add_product(g, v, c.F(hF, h));
            scale += fabsf(v) * c.F(hNoise, h);
        };
        // unit heads below `below`: lane = coordinate walks its own short list, or, when some coordinate's list
        // overflowed, the wave walks every unit head in turn
        auto add_units = [&](uint32_t from, uint32_t below) {
            if (c.unit_lists) {
                while (next < c.unit_count) {
                    const uint32_t h = c.unit_list[next * uint32_t(kWave) + lane];
                    if (h >= below) break;
                    ++next;
                    if (c.U(hContrib, h) != 0u) add_unit(h);
                }
                return;
            }
            for (uint32_t h = from; h < below; ++h)
                if (c.U(hContrib, h) != 0u && c.U(hUnit, h) == lane) add_unit(h);
        };
        for (uint32_t chunk = 0u; chunk < c.staged_end; chunk += 32u) {
            const uint32_t end = min(chunk + 32u, c.heads);
            add_units(chunk, end);
            if (chunk < uint32_t(kWave)) {
                for (uint64_t rest = contributing & ~unit_heads & (0xFFFFFFFFull << chunk); rest != 0ull; rest &= rest - 1ull) {
                    const uint32_t h = uint32_t(__builtin_ctzll(rest));
                    float f[3], cv[6], noise[3];
#pragma unroll
                    for (int k = 0; k < 3; ++k) { f[k] = uniform_lane_value(mf[k], h); noise[k] = uniform_lane_value(mn[k], h); }
#pragma unroll
                    for (int k = 0; k < 6; ++k) cv[k] = uniform_lane_value(mc[k], h);
                    const uint32_t axes = uint32_t(__builtin_amdgcn_readlane(int(my_axes), int(h)));
                    const uint64_t columns = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_high), int(h)))) << 32u) |
                                             uint64_t(uint32_t(__builtin_amdgcn_readlane(int(my_low), int(h))));
                    add_head<N>(c, h, coordinate, f, cv, noise, axes, columns, hrow, g, scale);
                }
            } else {
                for (uint32_t h = chunk; h < end; ++h) {
                    if (c.U(hContrib, h) == 0u || c.U(hUnit, h) != kInvalid) continue;
                    const float f[3] = {c.F(hF, h), c.F(hF + 1, h), c.F(hF + 2, h)};
                    const float cv[6] = {c.F(hC, h), c.F(hC + 1, h), c.F(hC + 2, h), c.F(hC + 3, h), c.F(hC + 4, h), c.F(hC + 5, h)};
                    const float noise[3] = {c.F(hNoise, h), c.F(hNoise + 1, h), c.F(hNoise + 2, h)};
                    const uint64_t columns = (uint64_t(__builtin_amdgcn_readfirstlane(c.U(hColumnsHigh, h))) << 32u) |
                                             uint64_t(__builtin_amdgcn_readfirstlane(c.U(hColumnsLow, h)));
                    add_head<N>(c, h, coordinate, f, cv, noise, c.U(hAxes, h), columns, hrow, g, scale);
                }
            }
        }
        add_units((c.staged_end + 31u) & ~31u, c.heads);
        // the unit heads' curvature lands on the diagonal after every staged head (:1605-1606)
#pragma unroll
        for (int k = 0; k < N; ++k) hrow[k] += local_lane(lane) == uint32_t(k) ? diagonal : 0.0f;
    }
    PROF_END(c, 12);
    PROF_BEGIN(c, 13);
    *force = coordinate ? float(g.value) : 0.0f;
    *inertia = coordinate ? float(inertial.value) : 0.0f;
    bool finite = isfinite(*force);
    const float4* u4 = reinterpret_cast<const float4*>(uvec);
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
        const float4 uv = u4[q];
        const float uk[4] = {uv.x, uv.y, uv.z, uv.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float entry = hrow[4 * q + t];
            finite = finite && isfinite(entry);
            scale += fabsf(entry) * uk[t];
        }
    }
    *converged = __all(!coordinate || fabsf(*force) <= kRoundings * FLT_EPSILON * scale);
    const bool ok = __all(!coordinate || finite);
    __syncthreads();
    PROF_END(c, 13);
    return ok;
}

enum Failure : uint32_t { kFailNone = 0u, kFailEquation, kFailFactor, kFailDirection, kFailCandidate };

// A reduced block.  Where no contact of the world reaches the coordinates from K on (the arms of a humanoid that
// stands on its feet), those coordinates enter the block's objective through the mass matrix alone and the minimiser
// over them is linear in the others: u_U = free_U - P (u_T - free_T), P = M_UU^-1 M_UT.  Eliminating them once per
// solve leaves the same problem on the K coordinates T with the Schur complement M_TT - M_TU M_UU^-1 M_UT as its mass
// matrix: every Newton block, factorisation and substitution of the solve is K wide instead of N.  The lanes K..n-1
// ("followers") hold a row of -P where the block's lanes hold a mass row, so that the product every Newton step
// takes with the mass rows (mass_times) hands each follower its own move, and the tests the reference makes over all
// coordinates (step below rounding, largest step, mass-normalised residual) still see all of them.  The minimiser of
// each block is the one the full-width block has; the iterates on the way differ by rounding.
// mass_step_i = sum_k M_ik d_k in coordinate order (:2177-2187, 2228-2238).  In a reduced block the lanes past the
// block's coordinates hold a row of -P instead of a mass row, and get their own move -P d from the same products.
template <int N>
__device__ __forceinline__ float mass_times(const Tile& c, const float (&mrow)[N], float d) {
    float* dvec = c.vec + 192;
    dvec[c.lane] = d;
    __syncthreads();
    float out = 0.0f;
    const float4* d4 = reinterpret_cast<const float4*>(dvec);
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
        const float4 dv = d4[q];
        out += mrow[4 * q] * dv.x; out += mrow[4 * q + 1] * dv.y; out += mrow[4 * q + 2] * dv.z; out += mrow[4 * q + 3] * dv.w;
    }
    __syncthreads();
    return c.lane < c.n_all ? out : 0.0f;
}


// TileNewtonDirection (:1935-1992).  The reference re-assembles the block after the mass-normalised
// convergence test because its mass factor overwrites the Hessian storage; here the two live apart and the
// assembled row, force and inertia (which the second assembly would reproduce bit for bit) are simply kept.
template <int N, bool kFollow>
__device__ __forceinline__ Failure newton_direction(const Tile& c, const float (&mrow)[N], const float (&mlow)[N], PlainLine& line, float u, float free_v,
                                    float* force, float* inertia, float* d, bool* converged) {
    PROF_COUNT(c, 0);
    c.work += 16u;
    float hrow[N];
    PROF_BEGIN(c, 1);
    const bool assembled = assemble_block<N, kFollow>(c, mrow, mlow, line, u, free_v, hrow, force, inertia, converged);
    PROF_END(c, 1);
    if (!assembled) return kFailEquation;
    if (*converged && c.tolerance > 0.0f) {
        if (!c.mass_valid) return kFailFactor;
        PROF_BEGIN(c, 3);
        const float direction = solve_tile_mass<N>(c, *force);
        PROF_END(c, 3);
        *d = direction;
        bool small = c.lane >= c.n || fabsf(direction) < c.tolerance;
        if constexpr (kFollow) {
            const float follow = mass_times<N>(c, mrow, c.lane < c.n ? direction : 0.0f);
            if (c.lane >= c.n && c.lane < c.n_all) small = fabsf(follow) < c.tolerance;
        }
        *converged = __all(small);
        if (*converged) return kFailNone;
    }
    if (*converged) return kFailNone;
    PROF_BEGIN(c, 2);
    const bool factored = cholesky_solve<N>(c, hrow, *force, d);
    PROF_END(c, 2);
    if (!factored) return kFailFactor;
    return kFailNone;
}

// TileRowSteps (:2018-2044): step = J d per head axis by serial fused multiply-adds, lane = head.  The Jacobian row
// and the direction come in as 16-byte words; padded columns are zeros on both sides.
template <int N>
__device__ __forceinline__ float row_dot_fma(const float* jrow, const float* dvec) {
    const float4* j4 = reinterpret_cast<const float4*>(jrow);
    const float4* d4 = reinterpret_cast<const float4*>(dvec);
    float value = 0.0f;
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
        const float4 j = j4[q], d = d4[q];
        value = fmaf(j.x, d.x, value); value = fmaf(j.y, d.y, value); value = fmaf(j.z, d.z, value); value = fmaf(j.w, d.w, value);
    }
    return value;
}
template <int N>
__device__ __forceinline__ void row_steps(const Tile& c, float d) {
    float* dvec = c.vec;
    dvec[c.lane] = c.lane < c.n ? d : 0.0f;
    __syncthreads();
    for (uint32_t h = c.lane; h < c.heads; h += kWave) {
        if (c.U(hOwned, h) == 0u) continue;
        const uint32_t unit = c.U(hUnit, h);
        if (unit != kInvalid) {   // :2028-2032
            c.F(hStep, h) = c.F(hUnitValue, h) * dvec[unit]; c.F(hStep + 1, h) = 0.0f; c.F(hStep + 2, h) = 0.0f;
            continue;
        }
        const uint32_t axes = c.U(hAxes, h);
        if constexpr (N > kTwoWaveWidth) {
            if (c.from_links) {
                float motion[6];
                link_motion<N>(c, way_of(c, h), dvec, motion);
                c.F(hStep, h) = wrench_dot(c, h, 0u, motion);
                c.F(hStep + 1, h) = axes > 1u ? wrench_dot(c, h, 1u, motion) : 0.0f;
                c.F(hStep + 2, h) = axes > 2u ? wrench_dot(c, h, 2u, motion) : 0.0f;
                continue;
            }
        }
        const float* j = c.jac + c.U(hRow, h) * uint32_t(N);
        c.F(hStep, h) = row_dot_fma<N>(j, dvec);
        c.F(hStep + 1, h) = axes > 1u ? row_dot_fma<N>(j + N, dvec) : 0.0f;
        c.F(hStep + 2, h) = axes > 2u ? row_dot_fma<N>(j + 2 * N, dvec) : 0.0f;
    }
    __syncthreads();
}

__device__ __forceinline__ void plain_line_terms(const PlainLine& p, float alpha, TileSum& row_slope, float& row_curvature, float& row_magnitude) {
    const float sx = p.step[0], sy = p.step[1], sz = p.step[2];
    float f[3], r[6];
    const float mx = fmaf(alpha, sx, p.move[0]), my = fmaf(alpha, sy, p.move[1]), mz = fmaf(alpha, sz, p.move[2]);
    plain_response(p, mx, my, mz, f, r);
    tile_add_product(row_slope, f[0], sx);
    tile_add_product(row_slope, f[1], sy);
    tile_add_product(row_slope, f[2], sz);
    row_magnitude += fabsf(f[0] * sx) + fabsf(f[1] * sy) + fabsf(f[2] * sz) + line_noise(r, p.res[0], p.res[1], p.res[2], mx, my, mz, sx, sy, sz);
    row_curvature += r[0] * sx * sx + r[1] * sy * sy + r[2] * sz * sz + 2.0f * r[5] * sy * sz;
}
// The line search runs in one of three modes, the same for every probe of a solve: general (the block has more heads
// than lanes, or some head is under the elliptic cone), plain with the terms in the first sixteen lanes (narrow), plain
// over the whole wavefront.  The mode is a template argument so that the probes carry no branch on it.
enum LineMode : int { kLineGeneral = 0, kLineWide = 1, kLineNarrow = 2 };
template <LineMode kMode>
__device__ __forceinline__ void line_derivatives(const Tile& c, const HeadLine& mine, const PlainLine& plain, float alpha,
                                 float inertial_slope, float inertial_curvature, float* slope, float* curvature, float* magnitude) {
    PROF_COUNT(c, 1);
    c.work += 1u;
    TileSum row_slope{0.0};
    float row_curvature = 0.0f, row_magnitude = 0.0f;
    if constexpr (kMode == kLineGeneral) {
        if (mine.owned) line_terms(mine, alpha, row_slope, row_curvature, row_magnitude);
        for (uint32_t h = c.lane + kWave; h < c.heads; h += kWave) {
            const HeadLine extra = load_head_line(c, h);
            if (extra.owned) line_terms(extra, alpha, row_slope, row_curvature, row_magnitude);
        }
    } else {
        plain_line_terms(plain, alpha, row_slope, row_curvature, row_magnitude);
    }
    PROF_BEGIN(c, 25);
    TileSum total{-row_slope.value};
    if (c.lane == 0u) {
        tile_add_product(total, alpha, inertial_curvature);
        tile_add(total, inertial_slope);
    }
    if constexpr (kMode == kLineNarrow) {
        // with at most sixteen heads every term sits in the first row of lanes; (t + 0) + (0 + 0) is t, so the sums agree
        *slope = wave_total(total, true);
        *curvature = inertial_curvature + first_row_sum(row_curvature);
        *magnitude = fabsf(inertial_slope) + alpha * inertial_curvature + first_row_sum(row_magnitude);
    } else {
        // the general mode takes the first-row sums too when its heads fit the first sixteen lanes
        const bool narrow = c.heads <= 16u;
        *slope = wave_total(total, narrow);
        *curvature = inertial_curvature + (narrow ? first_row_sum(row_curvature) : wave_sum(row_curvature));
        *magnitude = fabsf(inertial_slope) + alpha * inertial_curvature + (narrow ? first_row_sum(row_magnitude) : wave_sum(row_magnitude));
    }
    PROF_END(c, 25);
}

// The search always evaluates the line at 0 and then at 1.  In the narrow mode the rows of sixteen lanes hold copies of
// the same heads (lane & 15) and the row sums stay within a row: the first row evaluates the line at 0 while the others
// evaluate it at 1, one pass for both points with the numbers either gives alone.  Each point's sums come out in its
// row's lanes.
struct LinePoint { float slope, curvature, magnitude; };
__device__ __forceinline__ void line_derivatives_pair(const Tile& c, const PlainLine& plain, float inertial_slope, float inertial_curvature,
                                                      LinePoint* at_zero, LinePoint* at_one) {
    PROF_COUNT(c, 1);
    const float alpha = c.lane < 16u ? 0.0f : 1.0f;
    TileSum row_slope{0.0};
    float row_curvature = 0.0f, row_magnitude = 0.0f;
    plain_line_terms(plain, alpha, row_slope, row_curvature, row_magnitude);
    TileSum total{-row_slope.value};
    if ((c.lane & 15u) == 0u) {
        tile_add_product(total, alpha, inertial_curvature);
        tile_add(total, inertial_slope);
    }
    const double slopes = row_total_d(total.value);
    float cv = row_curvature, mg = row_magnitude;
    cv += dpp_move<kDppXor1>(cv); cv += dpp_move<kDppXor2>(cv); cv += dpp_move<kDppHalfMirror>(cv); cv += dpp_move<kDppMirror>(cv);
    mg += dpp_move<kDppXor1>(mg); mg += dpp_move<kDppXor2>(mg); mg += dpp_move<kDppHalfMirror>(mg); mg += dpp_move<kDppMirror>(mg);
    at_zero->slope = float(row_value_d(slopes, 0));
    at_zero->curvature = inertial_curvature + row_value(cv, 0);
    at_zero->magnitude = fabsf(inertial_slope) + 0.0f * inertial_curvature + row_value(mg, 0);
    at_one->slope = float(row_value_d(slopes, 1));
    at_one->curvature = inertial_curvature + row_value(cv, 1);
    at_one->magnitude = fabsf(inertial_slope) + 1.0f * inertial_curvature + row_value(mg, 1);
}

// SearchTileLine (:2089-2125)
template <LineMode kMode, bool kKept>
__device__ __forceinline__ float search_line_in(const Tile& c, PlainLine& plain, float inertial_slope, float inertial_curvature) {
    constexpr bool kPaired = kMode == kLineNarrow;
    float slope = 0.0f, curvature = 0.0f, magnitude = 0.0f;
    HeadLine mine{};
    if constexpr (kMode == kLineGeneral) mine = load_head_line(c, c.lane);
    else if constexpr (kKept) refresh_steps(c, plain);
    else plain = own_line(c);
    float low = 0.0f, high = 0.0f, alpha = 1.0f;
    bool bounded = false;
    float initial;
    uint32_t step = 0u;
    // one turn of the search on the line's slope and curvature at alpha: true when the search ends, with its answer
    auto turn = [&](float* answer) {
        if (!isfinite(slope) || !isfinite(curvature)) {
            high = alpha; bounded = true; alpha = 0.5f * (low + high);
            return false;
        }
        if (fabsf(slope) <= fmaxf(kLineTolerance * -initial, kRoundings * FLT_EPSILON * magnitude)) { *answer = alpha; return true; }
        if (slope < 0.0f) low = alpha;
        else { high = alpha; bounded = true; }
        if (bounded && high - low <= FLT_EPSILON * high) { *answer = low; return true; }
        float next = alpha - slope * __builtin_amdgcn_rcpf(curvature);
        if (!(next > low && (!bounded || next < high))) next = bounded ? 0.5f * (low + high) : 2.0f * alpha;
        alpha = next;
        return false;
    };
    float answer = 0.0f;
    if constexpr (kPaired) {
        LinePoint at_zero, at_one;
        line_derivatives_pair(c, plain, inertial_slope, inertial_curvature, &at_zero, &at_one);
        c.work += 1u;
        initial = at_zero.slope;
        if (!(initial < 0.0f)) return 0.0f;
        slope = at_one.slope; curvature = at_one.curvature; magnitude = at_one.magnitude;
        c.work += 1u;
        if (turn(&answer)) return answer;
        step = 1u;
    } else {
        line_derivatives<kMode>(c, mine, plain, 0.0f, inertial_slope, inertial_curvature, &slope, &curvature, &magnitude);
        initial = slope;
        if (!(initial < 0.0f)) return 0.0f;
    }
    for (; step < kLineSearchSteps; ++step) {
        line_derivatives<kMode>(c, mine, plain, alpha, inertial_slope, inertial_curvature, &slope, &curvature, &magnitude);
        if (turn(&answer)) return answer;
    }
    return low;
}
template <bool kKept>
__device__ __forceinline__ float search_line(const Tile& c, PlainLine& line, float inertial_slope, float inertial_curvature) {
    if (c.heads > uint32_t(kWave) || c.elliptic) return search_line_in<kLineGeneral, kKept>(c, line, inertial_slope, inertial_curvature);
    if (c.heads <= 16u) return search_line_in<kLineNarrow, kKept>(c, line, inertial_slope, inertial_curvature);
    return search_line_in<kLineWide, kKept>(c, line, inertial_slope, inertial_curvature);
}

__device__ __forceinline__ void apply_moves(const Tile& c, float alpha) {
    for (uint32_t h = c.lane; h < c.heads; h += kWave) {
        if (c.U(hOwned, h) == 0u) continue;
#pragma unroll
        for (int k = 0; k < 3; ++k) c.F(hMove + k, h) = fmaf(alpha, c.F(hStep + k, h), c.F(hMove + k, h));
    }
    __syncthreads();
}

// DescendTileBlock (:2145-2301).  `u` is lane i's block coordinate; `has_free` is false in the position pass.
template <int N, bool kFollow>
__device__ __forceinline__ void descend_block(Tile& c, const float (&mrow)[N], const float (&mlow)[N], float* u_io, float free_in, bool has_free,
                                              DataView d) {
    const uint32_t lane = c.lane, n = c.n;
    const bool coordinate = lane < n;
    const bool follower = kFollow && lane >= n && lane < c.n_all;
    const bool moving = coordinate || follower;
    PROF_BEGIN(c, 26);
    for (uint32_t h = lane; h < c.heads; h += kWave) {   // StartTileBlock (:1386-1397)
        if (c.U(hOwned, h) == 0u) continue;
        c.F(hNormalBound, h) = c.F(hDual, h);
        c.F(hMove, h) = 0.0f; c.F(hMove + 1, h) = 0.0f; c.F(hMove + 2, h) = 0.0f;
    }
    __syncthreads();
    PlainLine line{};   // the heads' constants over this block descent
    if constexpr (kKeepLine<N>) line = own_line(c);
    float start = coordinate ? *u_io : 0.0f;
    const float free_v = moving && has_free ? free_in : 0.0f;
    if constexpr (kFollow) {   // the followers start where the block's coordinates put them
        const float follow = mass_times<N>(c, mrow, coordinate ? start - free_v : 0.0f);
        if (follower) start = free_v + follow;
    }
    float u = start;
    if (c.iteration == 0u && has_free) {   // first-sweep segment search (:2165-2209)
        float dd = coordinate ? free_v - u : 0.0f;
        const float mass_step = mass_times<N>(c, mrow, dd);
        if (follower) dd = mass_step;
        TileSum curvature{0.0};
        if (coordinate) tile_add_product(curvature, dd, mass_step);
        const float inertial_curvature = wave_total(curvature);
        if (inertial_curvature > 0.0f && isfinite(inertial_curvature)) {
            row_steps<N>(c, dd);
            const float alpha = search_line<kKeepLine<N>>(c, line, -inertial_curvature, inertial_curvature);
            if (alpha > 0.0f) {
                u = fmaf(alpha, dd, u);
                apply_moves(c, alpha);
            }
        }
    }
    PROF_END(c, 26);
    Failure failure = kFailNone;
    float primal = FLT_MAX;
    for (uint32_t step = 0u; step < kNewtonSteps; ++step) {
        float force = 0.0f, inertia = 0.0f, dd = 0.0f;
        bool converged = false;
        failure = newton_direction<N, kFollow>(c, mrow, mlow, line, u, free_v, &force, &inertia, &dd, &converged);
        if (converged) primal = 0.0f;
        if (failure != kFailNone || converged) break;
        if (!coordinate) dd = 0.0f;
        PROF_BEGIN(c, 8);
        const float mass_step = mass_times<N>(c, mrow, dd);
        if (follower) dd = mass_step;
        PROF_END(c, 8);
        PROF_BEGIN(c, 27);
        TileSum decrement{0.0}, slope{0.0}, curvature{0.0};
        if (coordinate) {
            tile_add_product(decrement, force, dd);
            tile_add_product(slope, inertia, dd);
            tile_add_product(curvature, dd, mass_step);
        }
        const float total_decrement = wave_total(decrement);
        const float inertial_slope = wave_total(slope);
        const float inertial_curvature = wave_total(curvature);
        if (!isfinite(total_decrement) || !isfinite(inertial_slope) || !isfinite(inertial_curvature)) { failure = kFailDirection; break; }
        if (!(total_decrement > 0.0f)) break;
        PROF_END(c, 27);
        PROF_BEGIN(c, 4);
        row_steps<N>(c, dd);
        PROF_END(c, 4);
        PROF_BEGIN(c, 5);
        const float alpha = search_line<kKeepLine<N>>(c, line, inertial_slope, inertial_curvature);
        PROF_END(c, 5);
        PROF_BEGIN(c, 28);
        const float after = fmaf(alpha, dd, u);
        const bool rounded = __all(!moving || after == u);
        if (!__all(!moving || isfinite(after))) { failure = kFailCandidate; break; }
        primal = 0.0f;
        if (moving && !rounded) primal = fmaxf(primal, fabsf(alpha * dd));
        if (!(alpha > 0.0f)) break;
        u = after;
        apply_moves(c, alpha);
        PROF_END(c, 28);
        if (rounded) break;
    }
    PROF_BEGIN(c, 29);
    for (uint32_t h = lane; h < c.heads; h += kWave) {   // EndTileBlock (:1400-1409)
        if (c.U(hOwned, h) == 0u) continue;
#pragma unroll
        for (int k = 0; k < 3; ++k) c.F(hRes + k, h) = c.F(hRes + k, h) - c.F(hMove + k, h);
    }
    __syncthreads();
    if (failure != kFailNone) {
        c.failed = true;
        if (lane == 0u) d.env_status[c.env] |= kEnvStatusSolverFailure;
    }
    float moved = failure == kFailNone ? 0.0f : FLT_MAX;
    if (moving) moved = fmaxf(moved, __uint_as_float(residual_bits(u - start)));
    c.momentum = fmaxf(c.momentum, wave_max(moved));
    if (failure != kFailNone) primal = FLT_MAX;
    c.residual = fmaxf(c.residual, wave_max(primal));   // one block per environment: no coupled heads
    if (moving) *u_io = u;
    PROF_END(c, 29);
}

// MeasureTilePrimal (:2378-2489): the mass-normalised momentum balance in double
template <int N, bool kFollow>
__device__ __forceinline__ void measure_primal(Tile& c, const float (&mrow)[N], const float (&mlow)[N], float* velocity_io, float free_v,
                               const float* lambda_env, uint32_t R, bool reconstruct, DataView d) {
    const uint32_t lane = c.lane, n = c.n;
    const bool coordinate = lane < n;
    const bool follower = kFollow && lane >= n && lane < c.n_all;
    // every coordinate's distance from its free velocity, exact in double, through LDS
    double* apart = reinterpret_cast<double*>(c.vec);
    const float here = coordinate ? *velocity_io : 0.0f;
    apart[lane] = coordinate ? double(here) - double(free_v) : 0.0;
    __syncthreads();
    double balance = 0.0;
    const double2* apart2 = reinterpret_cast<const double2*>(apart);
#pragma unroll
    for (int q = 0; q < N / 2; ++q) {
        // the mass row does not change over the solve: left to itself the compiler widens all of it to double once,
        // ahead of the sweeps, and holds two registers an entry from there on
        const double2 dv = apart2[q];   // padded terms are exact zeros
        balance = fma(-double(opaque_with(mrow[2 * q], here)), dv.x, balance);
        balance = fma(-double(opaque_with(mrow[2 * q + 1], here)), dv.y, balance);
        if constexpr (kFollow) {
            balance = fma(-double(opaque_with(mlow[2 * q], here)), dv.x, balance);
            balance = fma(-double(opaque_with(mlow[2 * q + 1], here)), dv.y, balance);
        }
    }
    // heads with an impulse add J^T lambda in head order (:2402-2436).  A unit head touches one coordinate: that
    // lane takes it from its own list when it comes up between the staged heads
    uint32_t next = 0u;
    auto add_units = [&](uint32_t from, uint32_t below) {
        if (!c.units) return;
        if (c.unit_lists) {
            while (next < c.unit_count) {
                const uint32_t h = c.unit_list[next * uint32_t(kWave) + lane];
                if (h >= below) break;
                ++next;
                if (c.U(hOwned, h) != 0u) balance += double(c.F(hUnitValue, h)) * lambda_env[c.U(hSlot, h) - c.env * R];
            }
            return;
        }
        for (uint32_t h = from; h < below; ++h)
            if (c.U(hOwned, h) != 0u && c.U(hUnit, h) == lane) balance += double(c.F(hUnitValue, h)) * lambda_env[c.U(hSlot, h) - c.env * R];
    };
    uint32_t done = 0u;
    bool rows_taken = false;
    if constexpr (N > kTwoWaveWidth) {
        if (c.from_links) {   // lane = head holds its impulse; the sum goes by way of the links
            float impulse[3] = {0.0f, 0.0f, 0.0f};
            if (lane < c.heads && c.U(hOwned, lane) != 0u) {
                const uint32_t local = c.U(hSlot, lane) - c.env * R, stride = c.U(hStride, lane), axes = c.U(hAxes, lane);
                impulse[0] = lambda_env[local];
                if (block_axes(axes)) { impulse[1] = lambda_env[local + stride]; impulse[2] = lambda_env[local + 2u * stride]; }
            }
            const double sum = rows_transposed_times<false>(c, __ballot(impulse[0] != 0.0f || impulse[1] != 0.0f || impulse[2] != 0.0f), impulse, impulse, nullptr);
            if (coordinate) balance += sum;
            rows_taken = true;
        }
    }
    for (uint32_t h = 0u; h < (rows_taken ? 0u : c.staged_end); ++h) {
        const uint32_t first = c.U(hRow, h);
        if (first == kInvalid || c.U(hOwned, h) == 0u) continue;
        add_units(done, h);
        done = h + 1u;
        const uint32_t local = c.U(hSlot, h) - c.env * R, stride = c.U(hStride, h), axes = c.U(hAxes, h);
        const float ix = lambda_env[local], iy = block_axes(axes) ? lambda_env[local + stride] : 0.0f,
                    iz = block_axes(axes) ? lambda_env[local + 2u * stride] : 0.0f;
        if (!(ix != 0.0f || iy != 0.0f || iz != 0.0f)) continue;
        if (!coordinate) continue;
        const float* j = c.jac + first * c.ldj;
        balance += double(j[lane]) * ix;
        if (block_axes(axes)) {
            balance += double(j[c.ldj + lane]) * iy;
            balance += double(j[2u * c.ldj + lane]) * iz;
        }
    }
    add_units(done, c.heads);
    __syncthreads();
    const float force = float(balance);
    const bool finite = __all(!coordinate || fabs(balance) <= double(FLT_MAX));
    Failure failure = finite ? kFailNone : kFailEquation;
    float direction = 0.0f;
    if (failure == kFailNone) {
        if (c.mass_valid) direction = solve_tile_mass<N>(c, force);
        else failure = kFailFactor;
    }
    float residual = failure == kFailNone ? 0.0f : FLT_MAX;
    if (failure != kFailNone && lane == 0u) d.env_status[c.env] |= kEnvStatusSolverFailure;
    if constexpr (kFollow) {   // the followers' part of M^-1 (balance, 0) is -P times the block's part
        const float follow = failure == kFailNone ? mass_times<N>(c, mrow, coordinate ? direction : 0.0f) : 0.0f;
        if (follower) direction = follow;
    }
    const bool moving = coordinate || follower;
    if (failure == kFailNone && moving) residual = fmaxf(residual, isfinite(direction) ? fabsf(direction) : FLT_MAX);
    residual = wave_max(residual);
    c.residual = fmaxf(c.residual, residual);
    if (reconstruct && failure == kFailNone) {
        if (!__all(!moving || isfinite(*velocity_io + direction))) { c.residual = FLT_MAX; return; }
        if (moving) *velocity_io += direction;
        c.momentum = fmaxf(c.momentum, residual);
    }
}

// InitializeTileResiduals (:890-930) on the staged rows: residual = fl(rhs dt) - J u, products summed in coordinate order
template <int N>
__device__ __forceinline__ void initialize_residuals(const Tile& c, float velocity, const float* urows, float dt) {
    float* dvec = c.vec;
    dvec[c.lane] = c.lane < c.n ? velocity : 0.0f;
    __syncthreads();
    const float4* d4 = reinterpret_cast<const float4*>(dvec);
    for (uint32_t h = c.lane; h < c.heads; h += kWave) {
        const uint32_t slot = c.U(hSlot, h), stride = c.U(hStride, h), axes = c.U(hAxes, h);
        const uint32_t unit = c.U(hUnit, h), first = c.U(hRow, h);
        if (unit != kInvalid || first == kInvalid) {   // one coordinate (or none): every other product is an exact zero
            const float along = unit != kInvalid ? c.F(hUnitValue, h) * dvec[unit] : 0.0f;
            c.F(hRes, h) = urows[size_t{slot} * kRowWords + 4u] * dt - (0.0f + along);
            c.F(hRes + 1, h) = 0.0f; c.F(hRes + 2, h) = 0.0f;
            continue;
        }
        if constexpr (N > kTwoWaveWidth) {
            if (c.from_links) {
                float motion[6];
                link_motion<N>(c, way_of(c, h), dvec, motion);
                for (uint32_t axis = 0u; axis < 3u; ++axis)
                    c.F(hRes + axis, h) = axis < axes ? urows[size_t{slot + axis * stride} * kRowWords + 4u] * dt - wrench_dot(c, h, axis, motion) : 0.0f;
                continue;
            }
        }
        for (uint32_t axis = 0u; axis < 3u; ++axis) {
            float residual = 0.0f;
            if (axis < axes) {
                const float rhs = urows[size_t{slot + axis * stride} * kRowWords + 4u];
                const float4* j4 = reinterpret_cast<const float4*>(c.jac + (first + axis) * uint32_t(N));
                float along = 0.0f;
#pragma unroll
                for (int q = 0; q < N / 4; ++q) {
                    const float4 j = j4[q], dv = d4[q];
                    along = along + j.x * dv.x; along = along + j.y * dv.y; along = along + j.z * dv.z; along = along + j.w * dv.w;
                }
                residual = rhs * dt - along;
            }
            c.F(hRes + axis, h) = residual;
        }
    }
    __syncthreads();
}

struct DualMomentum { float t, beta; };

// UpdateTileHeadDuals (:2493-2595); classes = {normal, tangent, joint}
__device__ __forceinline__ void update_duals(const Tile& c, float* lambda_env, uint32_t R, const float* urows, DualMomentum* momentum, bool velocity,
                             bool commit, float* classes) {
    uint32_t steps[3] = {0u, 0u, 0u};
    double restart = 0.0;
    for (uint32_t h = c.lane; h < c.heads; h += kWave) {
        const uint32_t slot = c.U(hSlot, h), local = slot - c.env * R, stride = c.U(hStride, h), axes = c.U(hAxes, h);
        const bool contact = block_axes(axes);
        const bool elliptic = c.elliptic && axes == kAxesElliptic;
        const float rho = c.F(hRho, h), compliance = c.F(hCompliance, h), lower = c.F(hLower, h), upper = c.F(hUpper, h);
        const float mu1 = c.F(hMu1, h), mu2 = c.F(hMu2, h);
        const Response response{c.F(hDualScale, h), c.F(hResidualScale, h)};
        const V3 residual{c.F(hRes, h), c.F(hRes + 1, h), c.F(hRes + 2, h)};
        const V3 base{c.F(hBase, h), c.F(hBase + 1, h), c.F(hBase + 2, h)};
        const V3 tdual = commit ? V3{c.F(hDual, h), c.F(hDual + 1, h), c.F(hDual + 2, h)} : base;
        float normal, ncurv;
        scalar_impulse(tdual.x, rho, residual.x, compliance, lower, upper, response, &normal, &ncurv);
        V3 dual{normal, 0.0f, 0.0f};
        V3 rstep{0, 0, 0}, rpoint{0, 0, 0};
        float rweight = 0.0f;
        float cone_y = 0.0f, cone_z = 0.0f;
        if (elliptic) {   // :2509-2510: the projection onto the elliptic cone as it is
            cone_y = c.F(hTangentCompliance, h); cone_z = c.F(hTangentCompliance + 1, h);
            float f[3], cv[6];
            elliptic_impulse(tdual, rho, residual.x, residual.y, residual.z, compliance, cone_y, cone_z, mu1, f, cv);
            dual = V3{f[0], f[1], f[2]};
        } else if (contact) {   // ProjectRowDual (block_descent.cu:799-804) with RelaxContactImpulse (augmented_row.hpp:128-138)
            float fy, fz, cyy, czz, cyz;
            tangent_impulse(tdual, rho, residual.y, residual.z, normal, mu1, mu2, &fy, &fz, &cyy, &czz, &cyz);
            const V3 next{normal, fy, fz};
            V3 last_step{0, 0, 0}, last_point{0, 0, 0};
            float last_weight = 0.0f;
            if (commit) {
                last_step = V3{c.F(hRelaxStep, h), c.F(hRelaxStep + 1, h), c.F(hRelaxStep + 2, h)};
                last_weight = c.F(hRelaxWeight, h);
                last_point = V3{c.F(hRelaxPoint, h), c.F(hRelaxPoint + 1, h), c.F(hRelaxPoint + 2, h)};
            }
            const V3 step{next.x - tdual.x, next.y - tdual.y, next.z - tdual.z};
            const V3 change{step.x - last_step.x, step.y - last_step.y, step.z - last_step.z};
            const V3 moved = sub3(tdual, last_point);
            const float square = change.x * change.x + change.y * change.y + change.z * change.z;
            const float along = -(moved.x * change.x + moved.y * change.y + moved.z * change.z);
            float weight = 1.0f;
            if (last_weight > 0.0f && along > 0.0f && square > 0.0f) weight = fminf(1.0f, along / square);
            rstep = step; rweight = weight; rpoint = tdual;
            dual = V3{tdual.x + weight * step.x, tdual.y + weight * step.y, tdual.z + weight * step.z};
        }
        // MultiplierSteps (block_descent.cu:761-770)
        float step_normal = response.residual_scale > 0.0f && response.dual_scale != 0.0f
            ? fabsf(dual.x - tdual.x) / response.residual_scale : 0.0f;
        float step_tangent = 0.0f;
        if (contact) {
            const float fs = fmaxf(mu1, mu2);
            const float m1 = mu1 <= 0.0f ? 0.0f : mu1 / fs, m2 = mu2 <= 0.0f ? 0.0f : mu2 / fs;
            const float first = m1 > 0.0f && rho > 0.0f ? (dual.y - tdual.y) / (rho * m1 * m1) : 0.0f;
            const float second = m2 > 0.0f && rho > 0.0f ? (dual.z - tdual.z) / (rho * m2 * m2) : 0.0f;
            step_tangent = hypotf(first, second);
        }
        if (!commit && response.residual_scale > 0.0f) step_normal = fabsf(dual.x - tdual.x) / response.residual_scale;
        EllipticResponse cone{};
        if (elliptic) {   // EllipticMultiplierStep (augmented_row.hpp:104-108; :2516-2519)
            cone = elliptic_response(rho, compliance, cone_y, cone_z);
            step_normal = fabsf(dual.x - tdual.x) / cone.kx;
            step_tangent = fmaxf(fabsf(dual.y - tdual.y) / cone.ky, fabsf(dual.z - tdual.z) / cone.kz);
        }
        const V3 physical = commit ? dual : tdual;
        if (!contact) {
            const bool normal_row = (__float_as_uint(urows[size_t{slot} * kRowWords]) & kRowContactNormal) != 0u;
            const float rate = -residual.x + compliance * physical.x;
            const float violation = physical.x > 0.0f ? fabsf(rate) : fmaxf(-rate, 0.0f);
            const float value = normal_row ? fmaxf(step_normal, violation) : step_normal;
            if (normal_row) steps[0] = max(steps[0], residual_bits(value));
            else steps[2] = max(steps[2], residual_bits(value));
        } else {
            if (commit) {
                if (!elliptic) {   // an elliptic head keeps its tangent compliances where the others keep this state
                    c.F(hRelaxStep, h) = rstep.x; c.F(hRelaxStep + 1, h) = rstep.y; c.F(hRelaxStep + 2, h) = rstep.z;
                    c.F(hRelaxWeight, h) = rweight;
                    c.F(hRelaxPoint, h) = rpoint.x; c.F(hRelaxPoint + 1, h) = rpoint.y; c.F(hRelaxPoint + 2, h) = rpoint.z;
                }
                lambda_env[local + stride] = dual.y;
                lambda_env[local + 2u * stride] = dual.z;
            }
            if (elliptic) {   // :2539-2542
                steps[0] = max(steps[0], residual_bits(step_normal));
                steps[1] = max(steps[1], residual_bits(step_tangent));
            } else {
                const V3 v{-residual.x + compliance * physical.x, -residual.y, -residual.z};
                steps[0] = max(steps[0], residual_bits(physical.x > 0.0f ? fabsf(v.x) : fmaxf(-v.x, 0.0f)));
                steps[1] = max(steps[1], residual_bits(fmaxf(step_tangent, fmaxf(along_axis(physical.y, v.y), along_axis(physical.z, v.z)))));
            }
        }
        if (!commit) continue;
        if (velocity) lambda_env[local] = dual.x;
        const bool extrapolate = contact || response.dual_scale != 0.0f;
        if (extrapolate) {   // MultiplierMetric (block_descent.cu:790-795) and MultiplierMomentumRestart (augmented_row.hpp:119-124)
            const float friction = fmaxf(mu1, mu2);
            const float first = contact && mu1 > 0.0f ? mu1 / friction : 0.0f;
            const float second = contact && mu2 > 0.0f ? mu2 / friction : 0.0f;
            V3 metric{response.residual_scale, rho * first * first, rho * second * second};
            if (elliptic) metric = V3{cone.kx, cone.ky, cone.kz};   // :2555-2557
            restart += (metric.x > 0.0f ? (double(tdual.x) - dual.x) * (double(dual.x) - base.x) / metric.x : 0.0) +
                       (metric.y > 0.0f ? (double(tdual.y) - dual.y) * (double(dual.y) - base.y) / metric.y : 0.0) +
                       (metric.z > 0.0f ? (double(tdual.z) - dual.z) * (double(dual.z) - base.z) / metric.z : 0.0);
        }
        if (momentum != nullptr) { c.F(hMove, h) = base.x; c.F(hMove + 1, h) = base.y; c.F(hMove + 2, h) = base.z; }
        c.F(hDual, h) = dual.x; c.F(hDual + 1, h) = dual.y; c.F(hDual + 2, h) = dual.z;
        c.F(hBase, h) = dual.x; c.F(hBase + 1, h) = dual.y; c.F(hBase + 2, h) = dual.z;
    }
    classes[0] = __uint_as_float(wave_max_u(steps[0]));
    classes[1] = __uint_as_float(wave_max_u(steps[1]));
    classes[2] = __uint_as_float(wave_max_u(steps[2]));
    restart = wave_sum_d(restart);
    if (momentum != nullptr) {
        // AdvanceDualMomentum (block_descent.cu:780-788) and ExtrapolateDual (:808-820)
        if (restart > 0.0) momentum->t = 1.0f;
        const float t = 0.5f * (1.0f + sqrtf(fmaf(4.0f * momentum->t, momentum->t, 1.0f)));
        momentum->beta = (momentum->t - 1.0f) / t;
        momentum->t = t;
        for (uint32_t h = c.lane; h < c.heads; h += kWave) {
            const bool contact = block_axes(c.U(hAxes, h));
            const bool extrapolate = contact || c.F(hDualScale, h) != 0.0f;
            const float beta = extrapolate ? momentum->beta : 0.0f;
            const V3 base{c.F(hMove, h), c.F(hMove + 1, h), c.F(hMove + 2, h)};
            const V3 next{c.F(hBase, h), c.F(hBase + 1, h), c.F(hBase + 2, h)};
            V3 out = next;
            if (beta != 0.0f) {
                V3 y{fmaf(beta, next.x - base.x, next.x), fmaf(beta, next.y - base.y, next.y), fmaf(beta, next.z - base.z, next.z)};
                y.x = fminf(fmaxf(y.x, c.F(hLower, h)), c.F(hUpper, h));
                if (!contact) out = V3{y.x, 0.0f, 0.0f};
                else {
                    const float mu1 = c.F(hMu1, h), mu2 = c.F(hMu2, h);
                    const float first = mu1 > 0.0f ? y.y / mu1 : 0.0f, second = mu2 > 0.0f ? y.z / mu2 : 0.0f;
                    const float slip = hypotf(first, second), radius = fmaxf(y.x, 0.0f);
                    const float scale = slip > radius ? radius / slip : 1.0f;
                    out = V3{y.x, mu1 > 0.0f ? y.y * scale : 0.0f, mu2 > 0.0f ? y.z * scale : 0.0f};
                }
            }
            c.F(hDual, h) = out.x; c.F(hDual + 1, h) = out.y; c.F(hDual + 2, h) = out.z;
        }
    }
    __syncthreads();
}

__host__ __device__ inline uint32_t PaddedWidth(uint32_t n) { return (n + 3u) & ~3u; }
// `n`: the width the solve works at - the block's coordinates, or the K of a reduced block
// The factor of the Newton Hessian, and at the widths that run two waves a SIMD the factor of the mass matrix beside
// it; wider blocks keep the mass factor, which a solve reads a few times a sweep, in device memory instead
// (DataView::solver_mass_factor), so that two of them fit a compute unit's LDS.
__host__ __device__ inline bool MassFactorInMemory(uint32_t n) { return PaddedWidth(n) > uint32_t(kTwoWaveWidth); }
__host__ __device__ inline uint32_t FactorRegionFloats(uint32_t n) {
    const uint32_t N = PaddedWidth(n);
    return (MassFactorInMemory(n) ? 1u : 2u) * FactorFloats(N);   // a multiple of 4
}
// what the set-up of a reduced block passes through LDS ahead of everything else: the eliminated coordinates' factor
// and their coupling to the others, transposed
__host__ __device__ inline uint32_t ReductionScratchFloats(uint32_t full, uint32_t reduced) {
    const uint32_t N = PaddedWidth(full);
    return reduced >= full ? 0u : 2u * (N - reduced) * N;   // doubles
}
// the coordinates' motion axes of a wide block (Tile::axes), twelve words a coordinate
__host__ __device__ inline uint32_t LinkAxisFloats(uint32_t n) { return PaddedWidth(n) > uint32_t(kTwoWaveWidth) ? 12u * uint32_t(kWave) : 0u; }
__host__ __device__ inline uint32_t HeadFieldFloats(uint32_t cap, uint32_t narrow) {
    return (kWideStride * cap + kNarrowStride * (narrow + 1u) + 3u) & ~3u;
}
// `cap` heads carry fields; `staged` of them (the contact heads) carry three Jacobian rows each.
// A block that keeps no contact rows (the world's contact rows each act through one link, ModelView::rows_from_links;
// a wide block of contact heads only) holds a wrench record a head in their place.
__host__ __device__ inline bool RowsFromLinks(uint32_t n, bool contacts_only, uint32_t world_flag) {
    return PaddedWidth(n) > uint32_t(kTwoWaveWidth) && contacts_only && world_flag != 0u;
}
__host__ __device__ inline uint32_t RowFloats(uint32_t N, uint32_t staged, bool from_links) {
    return from_links ? (kWrenchStride * staged + 3u) & ~3u : 3u * staged * N;
}
__host__ __device__ inline uint32_t SolverLdsFloats(uint32_t n, uint32_t cap, uint32_t staged, bool from_links = false) {
    const uint32_t N = PaddedWidth(n);
    // the per-coordinate unit lists exist only when some head beyond the staged ones can be listed; without joint rows
    // the block keeps the footprint that lets eight of them share a compute unit's LDS
    return FactorRegionFloats(n) + RowFloats(N, staged, from_links) + HeadFieldFloats(cap, staged) + 256u +
           (cap > staged ? kUnitSlots * uint32_t(kWave) : 0u) + LinkAxisFloats(n);
}
__host__ __device__ inline uint32_t ReducedSolverLdsFloats(uint32_t full, uint32_t reduced, uint32_t cap, uint32_t staged, bool from_links = false) {
    const uint32_t solve = SolverLdsFloats(reduced, cap, staged, from_links), scratch = ReductionScratchFloats(full, reduced);
    return solve > scratch ? solve : scratch;
}

// DescendTile (:2941-3087).  kContactsOnly is the instantiation for worlds without joint rows whose heads fit one a
// lane (cap <= 64, every head a staged contact head): the unit-head paths and the loops over heads beyond the first
// 64 are compiled out, which leaves the hot loop shorter and with fewer values to keep live.
// The set-up of a reduced block, in double.  Lane i < n comes with row i of the mass matrix at `mass` (md words a row).
// The coordinates N-1 .. K are eliminated leaves first (FactorTileColumns' order): the lanes below K are left with
// their rows of the Schur complement S = M_TT - M_TU M_UU^-1 M_UT and of U_TU = M_TU U_UU^-T, the followers with their
// rows of the factor M_UU = U_UU U_UU^T.  P = M_UU^-1 M_UT = U_UU^-T U_TU^T then follows by forward substitution over the
// followers in ascending order, its two operands passing through LDS to be read transposed.  On return a lane below K
// holds its row of S as the sum mrow + mlow of two floats, a follower its row of -P rounded to float in mrow.
// Double because these rows stand in for the mass matrix over the whole solve: a Schur complement eliminated in
// single precision moves the velocities the solve converges to by a few 1e-5 of the contact impulse's effect.
template <int N, int K>
__device__ __forceinline__ bool reduce_block(uint32_t lane, uint32_t n, const float* mass, uint32_t md, float* lds, float (&mrow)[K], float (&mlow)[K]) {
    constexpr int kFollowers = N - K;
    const bool row_lane = lane < n;
    double full[N];
    {
        float fetched[N];
        if (md % 4u == 0u && md >= uint32_t(N)) {
#pragma unroll
            for (int q = 0; q < N / 4; ++q) {
                const float4 m4 = reinterpret_cast<const float4*>(mass)[q];
                fetched[4 * q] = m4.x; fetched[4 * q + 1] = m4.y; fetched[4 * q + 2] = m4.z; fetched[4 * q + 3] = m4.w;
            }
        } else {
#pragma unroll
            for (int k = 0; k < N; ++k) fetched[k] = uint32_t(k) < n ? mass[k] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < N; ++k)   // rows and columns n..N-1 are those of the identity
            full[k] = row_lane && uint32_t(k) < n ? double(fetched[k]) : (lane == uint32_t(k) && lane < uint32_t(N) ? 1.0 : 0.0);
    }
    const uint32_t at = local_lane(lane);
    bool valid = true;
    double own_scale = 0.0;
#pragma unroll
    for (int k = N - 1; k >= K; --k) {
        const double pivot = lane_value_d(full[k], k);
        valid = valid && pivot > 0.0 && pivot <= double(FLT_MAX);
        // the reciprocal root: the single-precision approximation and two Newton steps
        const double safe = valid ? pivot : 1.0;
        double scale = double(__builtin_amdgcn_rsqf(float(safe)));
        scale = scale * fma(-0.5 * safe, scale * scale, 1.5);
        scale = scale * fma(-0.5 * safe, scale * scale, 1.5);
        full[k] = at == uint32_t(k) ? safe * scale : full[k] * scale;
        if (at == uint32_t(k)) own_scale = scale;
        const uint64_t reach = __ballot(at < uint32_t(k) && full[k] != 0.0);
#pragma unroll
        for (int q = (k - 1) / 4; q >= 0; --q) {
            if (((reach >> (4 * q)) & 0xFull) == 0ull) continue;
            double u[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) u[t] = 4 * q + t <= k - 1 ? lane_value_d(full[k], 4 * q + t) : 0.0;
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (4 * q + t <= k - 1) full[4 * q + t] = fma(-full[k], u[t], full[4 * q + t]);
        }
    }
    double* coupling = reinterpret_cast<double*>(lds);   // [follower][coordinate below K]: U_TU transposed
    double* corner = coupling + kFollowers * K;           // [follower i][follower k]: U_UU[i][k], zero below the diagonal
    if (lane < uint32_t(K)) {
#pragma unroll
        for (int k = K; k < N; ++k) coupling[(k - K) * K + int(lane)] = full[k];
    } else if (lane < uint32_t(N)) {
#pragma unroll
        for (int k = K; k < N; ++k) corner[(int(lane) - K) * kFollowers + (k - K)] = uint32_t(k) >= lane ? full[k] : 0.0;
    }
    __syncthreads();
    const uint32_t slot = lane >= uint32_t(K) && lane < uint32_t(N) ? lane - uint32_t(K) : 0u;
    double prow[K], column[kFollowers];
#pragma unroll
    for (int q = 0; q < K / 2; ++q) {
        const double2 v = reinterpret_cast<const double2*>(coupling + slot * uint32_t(K))[q];
        prow[2 * q] = v.x; prow[2 * q + 1] = v.y;
    }
#pragma unroll
    for (int i = 0; i < kFollowers; ++i) column[i] = corner[i * kFollowers + int(slot)];
    // Column by column (the columns do not meet in the substitution).  A column of the coupling that is zero in every
    // follower's row stays zero - a leg's coordinate and an arm's share no link - and is left out, on a uniform test.
#pragma unroll
    for (int c0 = 0; c0 < K; ++c0) {
        if (__ballot(lane >= uint32_t(K) && lane < uint32_t(N) && prow[c0] != 0.0) == 0ull) continue;
#pragma unroll
        for (int i = K; i < N; ++i) {
            const double y = lane_value_d(prow[c0] * own_scale, i);
            prow[c0] = at > uint32_t(i) ? fma(-column[i - K], y, prow[c0]) : prow[c0];
        }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const double entry = lane < uint32_t(K) ? full[k] : (lane < n ? -(prow[k] * own_scale) : 0.0);
        mrow[k] = float(entry);
        mlow[k] = lane < uint32_t(K) ? float(entry - double(mrow[k])) : 0.0f;
    }
    __syncthreads();
    return valid;
}

// K < N is a reduced block (described above mass_times): no contact of the world reaches the coordinates K..n-1, which are
// eliminated once in the set-up, and the sweeps run K wide.  K is a multiple of 4 with K <= n, contact heads only.
template <int N, bool kContactsOnly, int K = N>
__global__ void __launch_bounds__(kWave) __attribute__((amdgpu_waves_per_eu(WavesPerSimd(K), WavesPerSimd(K))))
BlockDescentTileKernel(ModelView m, DataView d, BlockDescentSolveParams p, uint32_t cap, uint32_t staged_cap, uint32_t points_lo,
                       uint32_t points_hi) {
    constexpr bool kReduced = K < N;
    constexpr int W = K;   // the width of the sweeps
    static_assert(K % 4 == 0 && K <= N && (!kReduced || kContactsOnly), "a reduced block holds contact heads only");
    extern __shared__ __align__(16) float lds[];
    const uint32_t env = d.tile_order[blockIdx.x], lane = threadIdx.x;
    // A world whose contact slots outnumber the contacts it usually has is solved by two launches of different LDS
    // capacity; each takes the environments whose contact points fall in its range and leaves the others at once.
    if (points_lo != 0u || points_hi != kInvalid) {
        const uint32_t points = d.contact_count[env];
        if (points < points_lo || points > points_hi) return;
    }
    const uint32_t R = p.rows_per_env, md = p.max_dof, n = m.dof, nl = m.links_per_env, S = p.contact_slots_per_env;
    Tile c;
    c.env = env; c.lane = lane; c.n = kReduced ? uint32_t(K) : n; c.n_all = n; c.ldj = uint32_t(W); c.cap = cap; c.narrow = staged_cap; c.heads = 0u; c.iteration = 0u;
    c.tolerance = p.velocity_tolerance; c.failed = false; c.momentum = 0.0f; c.residual = 0.0f;
    c.mass_inverse = 0.0f; c.mass_valid = false; c.work = 0u; c.units = false; c.elliptic = false;
    c.factor_current = false;
#ifdef NKH_SOLVER_PROFILE
    for (int i = 0; i < 32; ++i) c.prof[i] = 0;
    for (int i = 0; i < 4; ++i) c.prof_count[i] = 0u;
    const long long prof_wall_start = wall_clock64();
#endif
    PROF_BEGIN(c, 9);
    PROF_BEGIN(c, 0);
    if constexpr (W > kTwoWaveWidth) {
        c.mfac = d.solver_mass_factor + size_t{env} * FactorFloats(uint32_t(W));
        c.hfac = lds;
    } else {
        c.mfac = lds;
        c.hfac = c.mfac + FactorFloats(uint32_t(W));
    }
    c.from_links = RowsFromLinks(uint32_t(W), kContactsOnly, m.rows_from_links);
    c.jac = lds + FactorRegionFloats(uint32_t(W));
    c.wrench = c.jac;   // one or the other
    c.fields = c.jac + RowFloats(uint32_t(W), staged_cap, c.from_links);
    c.vec = c.fields + HeadFieldFloats(cap, staged_cap);
    // The block's mass rows: lane's row of M, or in a reduced block lane's row of the Schur complement (lanes below K)
    // and of -P (the followers).
    float mrow[W], mlow[W];
    bool reduction_valid = true;
    if constexpr (kReduced) {
        PROF_BEGIN(c, 30);
        reduction_valid = reduce_block<N, K>(lane, n, d.m + size_t{env} * md * md + size_t{lane < n ? lane : 0u} * md, md, lds, mrow, mlow);
        PROF_END(c, 30);
    } else {
#pragma unroll
        for (int k = 0; k < W; ++k) mlow[k] = 0.0f;   // never read
    }
    if (lane < kNarrowFields) c.fields[kWideStride * cap + staged_cap * kNarrowStride + lane] = 0.0f;   // what a narrow field reads beyond its heads
    c.unit_list = reinterpret_cast<uint32_t*>(c.vec + 256);
    c.unit_lists = true; c.unit_count = 0u; c.staged_end = 0u; c.individual_end = 0u;
    c.through_links = false;
    c.axes = c.vec + 256 + (cap > staged_cap ? kUnitSlots * uint32_t(kWave) : 0u);
    c.path_low = c.path_high = c.under_low = c.under_high = 0u;
    c.rows = d.urows; c.row_point_a = d.row_cj_point; c.row_point_b = d.row_cj_point_b; c.row_link_a = d.row_cj_link; c.row_link_b = d.row_cj_link_b;
    c.link_paths = m.link_dof_mask; c.first_link = env * nl;
    c.pivot = V3{0.0f, 0.0f, 0.0f};
    const bool coordinate = lane < n;
    const float* urows = d.urows;
    float* lambda_env = d.lambda + size_t{env} * R;
    const size_t lbase = size_t{env} * nl;
    // InitializeTile (:1327-1350): the free velocity and the constraint velocity carried from the previous solve
    uint32_t my_link = 0u, my_component = kInvalid;
    float free_v = 0.0f, velocity = 0.0f;
    if (coordinate) {
        my_link = m.dof_link[lane]; my_component = m.dof_component[lane];
        const float value = my_component == kInvalid ? d.qdot[lbase + my_link] : d.link_velocity[(lbase + my_link) * 6u + my_component];
        const float carried = d.solver_velocity[size_t{env} * md + lane] - d.solver_free[size_t{env} * md + lane];
        free_v = value;
        velocity = value + (isfinite(carried) ? carried : 0.0f);
    }
    PROF_BEGIN(c, 16);
    // ListTileHeads (:1250-1296): active rows that are not block tangents, in slot order
    // The reference scans the rows below the larger of the last two row extents (all of them when either is unknown,
    // as after a reset).  The rows between this step's extent and that bound were cleared by this step's row assembly
    // and hold no head, so the scan stops at this step's extent: the same heads from a fraction of the row records.
    const uint32_t current = d.contact_row_extent[2u * env + 1u];
    const uint32_t bound = current == 0u ? p.contact_rows_per_env : min(current - 1u, p.contact_rows_per_env);
    const uint32_t total = bound + (R - p.contact_rows_per_env);
    uint32_t heads = 0u;
    bool overflow = false;
    for (uint32_t base = 0u; base < total; base += kWave) {
        const uint32_t index = base + lane;
        const uint32_t slot = env * R + (index < bound ? index : p.contact_rows_per_env + (index - bound));
        bool head = false;
        if (index < total) {
            const uint32_t flags = __float_as_uint(urows[size_t{slot} * kRowWords]);
            head = (flags & kRowActive) != 0u && (flags & kRowBlockTangent) == 0u;
        }
        const uint64_t mask = __ballot(head);
        if (head) {
            const uint32_t at = heads + __popcll(mask & ((uint64_t{1} << lane) - 1u));
            if (at < cap) c.U(hSlot, at) = slot; else overflow = true;
        }
        heads += __popcll(mask);
    }
    if (__any(overflow)) {   // more heads than the staged LDS holds: fail loudly, solve the ones that fit
        heads = cap;
        if (lane == 0u) d.env_status[env] |= kEnvStatusSolverFailure;
    }
    if constexpr (kContactsOnly) __builtin_assume(heads <= uint32_t(kWave));
    c.heads = heads;
    __syncthreads();
    PROF_END(c, 16);
    PROF_BEGIN(c, 17);
    // stage Jacobian rows: the sum of the articulated sides' chain rows (TileBlock::Jacobian :555-573, CopyTileRows :836-869).
    // First every (head, axis) row finds its source rows, one per lane; then the copies run with their loads in flight
    // together instead of one row's latency after another.
    for (uint32_t r = lane; r < 3u * heads; r += kWave) {
        const uint32_t h = r / 3u, axis = r - 3u * h;
        const uint32_t slot = c.U(hSlot, h);
        const uint32_t flags = __float_as_uint(urows[size_t{slot} * kRowWords]);
        const uint32_t stride = __float_as_uint(urows[size_t{slot} * kRowWords + 2u]);
        const uint32_t axes = (flags & kRowBlockNormal) != 0u ? 3u : 1u;
        uint32_t source_a = kInvalid, source_b = kInvalid;
        if (axis < axes) {
            const uint32_t rs = slot + axis * stride;
            if (__float_as_uint(urows[size_t{rs} * kRowWords + 10u]) == kSideArtic) source_a = rs;
            if (__float_as_uint(urows[size_t{rs} * kRowWords + 18u]) == kSideArtic) source_b = rs;
        }
        c.U(hSourceA + axis, h) = source_a; c.U(hSourceB + axis, h) = source_b;
    }
    __syncthreads();
    PROF_BEGIN(c, 22);
    // FindTileRowSupport (:801-833), lane = head: a single-axis head whose Jacobian row has at most one entry is a unit
    // head and stages nothing; every other owned head stages three rows, placed in head order (PlaceTileRows).
    {
        // a single-axis head acting on one coordinate is a unit head; the rows carry that coordinate and its entry
        // from where they were emitted (row_unit, row_unit_value), which is what a scan of the head's Jacobian row
        // for its entries would find
        for (uint32_t base = 0u; base < heads; base += kWave) {
            const uint32_t h = base + lane;
            if (h >= heads) continue;
            const uint32_t source_a = c.U(hSourceA, h), source_b = c.U(hSourceB, h);
            const bool owned = source_a != kInvalid || source_b != kInvalid;
            // a block head has found the sources of its tangent rows on the sides that move
            const bool single_axis = c.U(hSourceA + 1u, h) == kInvalid && c.U(hSourceB + 1u, h) == kInvalid;
            const uint32_t slot = c.U(hSlot, h);
            uint32_t unit = kInvalid;
            float unit_value = 0.0f;
            if (owned && single_axis && d.row_unit[slot] != kInvalid) { unit = d.row_unit[slot]; unit_value = d.row_unit_value[slot]; }
            c.U(hUnit, h) = unit; c.F(hUnitValue, h) = unit_value; c.U(hRow, h) = owned && unit == kInvalid ? 0u : kInvalid;
            c.U(hColumnsLow, h) = 0u; c.U(hColumnsHigh, h) = 0u;
        }
        __syncthreads();
        PROF_END(c, 22);
        PROF_BEGIN(c, 23);
        // PlaceTileRows: the staged heads take their rows in head order
        uint32_t staged = 0u, staged_end = 0u, individual_end = 0u, my_units = 0u;
        bool overflow_rows = false, any_unit = false;
        for (uint32_t base = 0u; base < heads; base += kWave) {
            const uint32_t h = base + lane;
            const bool stage = h < heads && c.U(hRow, h) != kInvalid;
            const uint64_t mask = __ballot(stage);
            if (stage) {
                const uint32_t at = staged + uint32_t(__popcll(mask & ((uint64_t{1} << lane) - 1ull)));
                if (at < staged_cap) c.U(hRow, h) = 3u * at;
                else {   // no room: the head acts on nothing, and the solve is flagged
                    overflow_rows = true;
                    c.U(hRow, h) = kInvalid; c.U(hUnit, h) = 0u; c.F(hUnitValue, h) = 0.0f;
                }
            }
            staged += uint32_t(__popcll(mask));
            if (mask != 0ull) staged_end = base + uint32_t(64 - __builtin_clzll(mask));
            any_unit = any_unit || (h < heads && c.U(hUnit, h) != kInvalid);
            // heads that need a response of their own: staged ones, and unit heads whose entry is not +-1
            const uint64_t own = __ballot(h < heads && (c.U(hUnit, h) == kInvalid || fabsf(c.F(hUnitValue, h)) != 1.0f));
            if (own != 0ull) individual_end = base + uint32_t(64 - __builtin_clzll(own));
        }
        c.units = !kContactsOnly && __any(any_unit) && cap > staged_cap;   // the lists have room only when the world has joint heads
        c.staged_end = staged_end;
        c.individual_end = individual_end;
        if (__any(overflow_rows) && lane == 0u) d.env_status[env] |= kEnvStatusSolverFailure;
        __syncthreads();
        // every coordinate lists its own unit heads, in head order
        if (c.units) {
            for (uint32_t h = 0u; h < heads; ++h) {
                if (c.U(hUnit, h) != lane) continue;
                if (my_units < kUnitSlots) c.unit_list[my_units * uint32_t(kWave) + lane] = h;
                ++my_units;
            }
            c.unit_lists = !__any(my_units > kUnitSlots);
            c.unit_count = min(my_units, kUnitSlots);
        }
        PROF_END(c, 23);
    }
    __syncthreads();
    if constexpr (W > kTwoWaveWidth && kContactsOnly) {
        // The coordinates' motion axes about the root link's origin, for add_heads_through_links: a hinge or an angular
        // coordinate of a floating root turns about its axis through the joint's origin, a sliding one moves along it
        // (the columns the row assembly wrote, assemble_rows.cu:122-169, before the dot with a row's direction).
        const float* root = d.link_pose + lbase * 7u;
        c.pivot = V3{root[0], root[1], root[2]};
        float axis[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        uint64_t path = 0ull;
        bool plain = true;
        if (coordinate) {
            V3 along, at;
            bool turning;
            if (my_component == kInvalid) {
                const Xf pose = load_xf(d.link_pose + (lbase + my_link) * 7u);
                along = rotate_normalized(pose.r, V3{m.joint_axis[3u * my_link], m.joint_axis[3u * my_link + 1u], m.joint_axis[3u * my_link + 2u]});
                at = pose.p;
                turning = m.joint_type[my_link] != kPrismatic;
            } else {
                const Xf base = load_xf(d.base_pose + size_t{env} * 7u);
                const uint32_t k = my_component % 3u;
                along = rotate_normalized(base.r, V3{k == 0u ? 1.0f : 0.0f, k == 1u ? 1.0f : 0.0f, k == 2u ? 1.0f : 0.0f});
                at = base.p;
                turning = my_component < 3u;
                plain = my_component < 6u;
            }
            if (turning) {
                const V3 arm = cross3(sub3(at, c.pivot), along);
                axis[0] = along.x; axis[1] = along.y; axis[2] = along.z; axis[3] = arm.x; axis[4] = arm.y; axis[5] = arm.z;
            } else {
                axis[3] = along.x; axis[4] = along.y; axis[5] = along.z;
            }
            path = m.link_dof_mask[my_link];
        }
        float4* table = reinterpret_cast<float4*>(c.axes);
        table[3u * lane] = float4{axis[0], axis[1], axis[2], axis[3]};
        table[3u * lane + 1u] = float4{axis[4], axis[5], 0.0f, 0.0f};
        table[3u * lane + 2u] = float4{0.0f, 0.0f, 0.0f, 0.0f};
        c.path_low = uint32_t(path); c.path_high = uint32_t(path >> 32u);
        uint64_t under = 0ull;
        for (uint32_t i = 0u; i < n; ++i) {
            const uint64_t holders = __ballot(((path >> i) & 1ull) != 0ull);   // the coordinates whose way to the root holds i
            if (lane == i) under = holders;
        }
        c.under_low = uint32_t(under); c.under_high = uint32_t(under >> 32u);
        // every staged head with exactly one side that moves
        bool one_link = true;
        if (lane < heads) {
            const bool side_a = c.U(hSourceA, lane) != kInvalid, side_b = c.U(hSourceB, lane) != kInvalid;
            one_link = !(side_a && side_b) && (!(side_a || side_b) || c.U(hRow, lane) != kInvalid);
        }
        c.through_links = heads <= uint32_t(kWave) && !c.units && __all(plain && one_link);
        if (c.from_links) {
            // the world was cooked as one whose contact rows each act through one link: an environment that holds
            // anything else was given the wrong kernel
            if (!c.through_links && lane == 0u) d.env_status[env] |= kEnvStatusSolverFailure;
            // lane = head: its rows as wrenches about the pivot, [(p - o) x n; n] with n the direction of the side that
            // moves, and its way to the root
            if (lane < heads) {
                float* record = c.wrench + lane * kWrenchStride;
                const uint32_t slot = c.U(hSlot, lane);
                const float* row = urows + size_t{slot} * kRowWords;
                const uint32_t stride = __float_as_uint(row[2]);
                const uint32_t axes = (__float_as_uint(row[0]) & kRowBlockNormal) != 0u ? 3u : 1u;
                const bool side_a = c.U(hSourceA, lane) != kInvalid, side_b = c.U(hSourceB, lane) != kInvalid;
                const bool second = !side_a;
                uint64_t way = 0ull;
                if (side_a != side_b) way = m.link_dof_mask[(second ? d.row_cj_link_b : d.row_cj_link)[slot] - env * nl];
                for (uint32_t a = 0u; a < 3u; ++a) {
                    float w[6] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
                    if (a < axes && side_a != side_b) {
                        const size_t rs = size_t{slot} + a * stride;
                        const float* side = urows + rs * kRowWords + (second ? 20u : 12u);
                        const float* at = (second ? d.row_cj_point_b : d.row_cj_point) + 3u * rs;
                        const V3 n{side[0], side[1], side[2]};
                        const V3 moment = cross3(sub3(V3{at[0], at[1], at[2]}, c.pivot), n);
                        w[0] = moment.x; w[1] = moment.y; w[2] = moment.z; w[3] = n.x; w[4] = n.y; w[5] = n.z;
                    }
#pragma unroll
                    for (int t = 0; t < 6; ++t) record[6u * a + uint32_t(t)] = w[t];
                }
                reinterpret_cast<uint32_t*>(record)[18] = uint32_t(way);
                reinterpret_cast<uint32_t*>(record)[19] = uint32_t(way >> 32u);
                c.U(hColumnsLow, lane) = uint32_t(way); c.U(hColumnsHigh, lane) = uint32_t(way >> 32u);
            }
        }
        __syncthreads();
    }
    // CopyTileRows (:836-869): the staged heads' rows, their loads in flight together

    bool stray = false;   // a reduced block: an entry past the block's coordinates
    for (uint32_t h0 = 0u; h0 < (c.from_links ? 0u : c.staged_end); h0 += 4u) {   // four heads at a time: 24 reads in flight
        uint32_t first[4];
        float value[4][3];
#pragma unroll
        for (uint32_t t = 0u; t < 4u; ++t) {
            const uint32_t h = h0 + t;
            first[t] = h < c.staged_end ? c.U(hRow, h) : kInvalid;   // a unit head stages nothing and touches no column block
            const bool staged = first[t] != kInvalid;
#pragma unroll
            for (uint32_t axis = 0u; axis < 3u; ++axis) {
                const uint32_t source_a = staged ? c.U(hSourceA + axis, h) : kInvalid, source_b = staged ? c.U(hSourceB + axis, h) : kInvalid;
                const float from_a = coordinate && source_a != kInvalid ? d.chain_jacobian[size_t{source_a} * md + lane] : 0.0f;
                const float from_b = coordinate && source_b != kInvalid ? d.chain_jacobian_b[size_t{source_b} * md + lane] : 0.0f;
                value[t][axis] = (0.0f + from_a) + from_b;
            }
        }
#pragma unroll
        for (uint32_t t = 0u; t < 4u; ++t) {
            const uint32_t h = h0 + t;
            if (h >= c.staged_end) break;
            const bool staged = first[t] != kInvalid;
#pragma unroll
            for (uint32_t axis = 0u; axis < 3u; ++axis)
                if (staged && lane < c.ldj) c.jac[(first[t] + axis) * c.ldj + lane] = value[t][axis];   // padded columns hold zeros
            // the columns this head touches at all: a contact on one limb leaves most coordinates out, and the Hessian
            // update skips their exact-zero products four columns at a time
            uint64_t columns = __ballot(value[t][0] != 0.0f || value[t][1] != 0.0f || value[t][2] != 0.0f);
            if constexpr (kReduced) {
                stray = stray || (columns >> uint32_t(W)) != 0ull;
                columns &= (uint64_t{1} << uint32_t(W)) - 1ull;
            }
            if (lane == 0u) { c.U(hColumnsLow, h) = uint32_t(columns); c.U(hColumnsHigh, h) = uint32_t(columns >> 32u); }
        }
    }
    // a contact that reaches a coordinate the world's reduction left out: the launch was given the wrong width
    if (stray && lane == 0u) d.env_status[env] |= kEnvStatusSolverFailure;
    __syncthreads();
    PROF_END(c, 17);
    PROF_BEGIN(c, 18);
    // TileInertialResponse (:709-739): J M^-1 J^T of every head's first row through the stored LDL^T factor
    // (ForwardMass + MassDot, articulation_mass.cuh:414-431).  lane = DoF: the unit-lower factor row sits in
    // registers with zeros from the diagonal on, each y_j travels as a scalar lane read, so row i subtracts
    // L_ij y_j for j = 0, 1, ... exactly as the serial loop does; the ordered sum of y_i^2 / D_i follows the same way.
    {
        // Lane's own rows of the mass matrix and of its LDL^T factor (StageTileMass :2127-2142) straight into registers:
        // one row is md contiguous words, so every read of both rows is in flight at once, as 16-byte words where the
        // rows are long enough and aligned for that.
        const size_t tile = size_t{env} * md * md + size_t{coordinate ? lane : 0u} * md;
        const float* factor = d.m_factor + tile;
        const float* mass = d.m + tile;
        float lrow[N];
        if constexpr (kReduced) {   // the mass rows were taken, and reduced, at the start
            if (md % 4u == 0u && md >= uint32_t(N)) {
#pragma unroll
                for (int q = 0; q < N / 4; ++q) {
                    const float4 f4 = reinterpret_cast<const float4*>(factor)[q];
                    lrow[4 * q] = f4.x; lrow[4 * q + 1] = f4.y; lrow[4 * q + 2] = f4.z; lrow[4 * q + 3] = f4.w;
                }
            } else {
#pragma unroll
                for (int k = 0; k < N; ++k) lrow[k] = uint32_t(k) < n ? factor[k] : 0.0f;
            }
        } else {
            float fetched[N];
            if (md % 4u == 0u && md >= uint32_t(N)) {
#pragma unroll
                for (int q = 0; q < N / 4; ++q) {
                    const float4 f4 = reinterpret_cast<const float4*>(factor)[q], m4 = reinterpret_cast<const float4*>(mass)[q];
                    lrow[4 * q] = f4.x; lrow[4 * q + 1] = f4.y; lrow[4 * q + 2] = f4.z; lrow[4 * q + 3] = f4.w;
                    fetched[4 * q] = m4.x; fetched[4 * q + 1] = m4.y; fetched[4 * q + 2] = m4.z; fetched[4 * q + 3] = m4.w;
                }
            } else {
#pragma unroll
                for (int k = 0; k < N; ++k) {
                    lrow[k] = uint32_t(k) < n ? factor[k] : 0.0f;
                    fetched[k] = uint32_t(k) < n ? mass[k] : 0.0f;
                }
            }
#pragma unroll
            for (int k = 0; k < W; ++k)   // rows and columns n..N-1 of the mass matrix are those of the identity
                mrow[k] = coordinate && uint32_t(k) < n ? fetched[k] : (lane == uint32_t(k) && lane < uint32_t(N) ? 1.0f : 0.0f);
        }
        float pivot = 1.0f;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            if (coordinate && lane == uint32_t(k)) pivot = lrow[k];
            lrow[k] = coordinate && uint32_t(k) < lane ? lrow[k] : 0.0f;
        }
        // y = L^-1 a, then the ordered sum of y_i^2 / D_i
        auto response = [&](float a) -> float {
#pragma unroll
            for (int j = 0; j < N; ++j) a -= lrow[j] * lane_value(a, j);
            const float term = coordinate ? a * a / pivot : 0.0f;
            float total = 0.0f;
#pragma unroll
            for (int i = 0; i < N; ++i) total += lane_value(term, i);
            return total;
        };
        // Four heads at a time: their substitution chains are independent, and side by side each one's lane reads
        // settle under the others' arithmetic.  A head with one moving side, or with both sides on one owner (:752),
        // wants exactly the staged sum of its two sides' rows.  Unit heads with an entry of +-1 are left to the
        // per-coordinate pass below: y(-e) = -y(e), so every such head of one coordinate has the same response.
        const bool share_units = c.units && c.unit_lists;
        bool by_heads = false;
        if constexpr (W > kTwoWaveWidth && kContactsOnly) {
            if (c.from_links && c.through_links) {
                // Every head at once, lane = head: its first row sits in the lane's registers (the coordinates' axes against
                // the row's wrench), the factor's entries are the same for every lane, and the substitution and the ordered
                // sum run down the coordinates with the operations of the loop below, head beside head instead of
                // four heads a pass.
                by_heads = true;
                const float* factor_rows = d.m_factor + size_t{env} * md * md;
                const bool owned = lane < heads && (c.U(hSourceA, lane) != kInvalid || c.U(hSourceB, lane) != kInvalid);
                const uint64_t way = owned ? way_of(c, lane) : 0ull;
                float w[6];
#pragma unroll
                for (int t = 0; t < 6; ++t) w[t] = owned ? c.wrench[lane * kWrenchStride + uint32_t(t)] : 0.0f;
                const float4* table = reinterpret_cast<const float4*>(c.axes);
                float y[N];
                float total = 0.0f;
#pragma unroll
                for (int i = 0; i < N; ++i) {
                    if (uint32_t(i) >= n) { y[i] = 0.0f; continue; }
                    const float4 sa = table[3 * i], sb = table[3 * i + 1];
                    const float entry = fmaf(sb.y, w[5], fmaf(sb.x, w[4], fmaf(sa.w, w[3], fmaf(sa.z, w[2], fmaf(sa.y, w[1], sa.x * w[0])))));
                    float v = ((way >> i) & 1ull) != 0ull ? entry : 0.0f;
                    const float* factor_row = factor_rows + size_t(i) * md;
#pragma unroll
                    for (int j = 0; j < i; ++j) v -= factor_row[j] * y[j];
                    y[i] = v;
                    total += v * v / factor_row[i];
                }
                if (lane < heads) {
                    const bool second = c.U(hSourceA, lane) == kInvalid;
                    c.F(hStep, lane) = second ? 0.0f : total; c.F(hMove, lane) = second ? total : 0.0f;
                }
            }
        }
        for (uint32_t h0 = 0u; h0 < (by_heads ? 0u : share_units ? c.individual_end : heads); h0 += 4u) {
            float a[4], term[4], total[4];
            bool second[4], apart[4], skip[4];
#pragma unroll
            for (uint32_t t = 0u; t < 4u; ++t) {
                const uint32_t h = h0 + t;
                a[t] = 0.0f; second[t] = false; apart[t] = false; skip[t] = true;
                if (h >= heads) continue;
                const bool artic_a = c.U(hSourceA, h) != kInvalid, artic_b = c.U(hSourceB, h) != kInvalid;
                if (artic_a && artic_b) {
                    const float* row = urows + size_t{c.U(hSlot, h)} * kRowWords;
                    apart[t] = __float_as_uint(row[11]) != __float_as_uint(row[19]);
                }
                second[t] = artic_b && !artic_a;
                const uint32_t first = c.U(hRow, h), unit = c.U(hUnit, h);
                const float unit_value = c.F(hUnitValue, h);
                skip[t] = share_units && unit != kInvalid && fabsf(unit_value) == 1.0f && !apart[t];
                if (coordinate && (artic_a || artic_b) && !apart[t] && !skip[t]) {
                    if (W > kTwoWaveWidth && c.from_links) {   // the first row's entry: the coordinate's axis against the row's wrench
                        const float4* table = reinterpret_cast<const float4*>(c.axes);
                        const float4 sa = table[3u * lane], sb = table[3u * lane + 1u];
                        const float* w = c.wrench + h * kWrenchStride;
                        const float entry = fmaf(sb.y, w[5], fmaf(sb.x, w[4], fmaf(sa.w, w[3], fmaf(sa.z, w[2], fmaf(sa.y, w[1], sa.x * w[0])))));
                        a[t] = ((way_of(c, h) >> lane) & 1ull) != 0ull ? entry : 0.0f;
                    } else {
                        a[t] = first != kInvalid ? (lane < c.ldj ? c.jac[first * c.ldj + lane] : 0.0f) : (lane == unit ? unit_value : 0.0f);
                    }
                }
            }
            if (skip[0] && skip[1] && skip[2] && skip[3]) continue;
#pragma unroll
            for (int j = 0; j < N; ++j) {
#pragma unroll
                for (int t = 0; t < 4; ++t) a[t] -= lrow[j] * lane_value(a[t], j);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) { term[t] = coordinate ? a[t] * a[t] / pivot : 0.0f; total[t] = 0.0f; }
#pragma unroll
            for (int i = 0; i < N; ++i) {
#pragma unroll
                for (int t = 0; t < 4; ++t) total[t] += lane_value(term[t], i);
            }
#pragma unroll
            for (uint32_t t = 0u; t < 4u; ++t) {
                const uint32_t h = h0 + t;
                if (h >= heads || skip[t]) continue;
                float shares[2] = {second[t] ? 0.0f : total[t], second[t] ? total[t] : 0.0f};
                if (apart[t]) {   // two owners: one response each
                    shares[0] = response(coordinate ? d.chain_jacobian[size_t{c.U(hSourceA, h)} * md + lane] : 0.0f);
                    shares[1] = response(coordinate ? d.chain_jacobian_b[size_t{c.U(hSourceB, h)} * md + lane] : 0.0f);
                }
                if (lane == 0u) { c.F(hStep, h) = shares[0]; c.F(hMove, h) = shares[1]; }
            }
        }
        if (share_units) {   // (M^-1)_uu of every coordinate that has unit heads, four coordinates at a time
            float mine = 0.0f;
            for (uint64_t rest = __ballot(c.unit_count > 0u); rest != 0ull;) {
                uint32_t target[4];
                float a[4], term[4], total[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    target[t] = rest != 0ull ? uint32_t(__builtin_ctzll(rest)) : kInvalid;
                    rest &= rest - 1ull;   // zero stays zero
                    a[t] = lane == target[t] ? 1.0f : 0.0f;
                }
                // below the group's first coordinate every y_j is an exact zero: those steps subtract and add nothing
                const int first = int(target[0]);
#pragma unroll
                for (int j = 0; j < N; ++j) {
                    if (j < first) continue;
#pragma unroll
                    for (int t = 0; t < 4; ++t) a[t] -= lrow[j] * lane_value(a[t], j);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) { term[t] = coordinate ? a[t] * a[t] / pivot : 0.0f; total[t] = 0.0f; }
#pragma unroll
                for (int i = 0; i < N; ++i) {
                    if (i < first) continue;
#pragma unroll
                    for (int t = 0; t < 4; ++t) total[t] += lane_value(term[t], i);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) if (lane == target[t]) mine = total[t];
            }
            for (uint32_t k = 0u; k < c.unit_count; ++k) {   // lane = coordinate hands its response to its own unit heads
                const uint32_t h = c.unit_list[k * uint32_t(kWave) + lane];
                if (fabsf(c.F(hUnitValue, h)) != 1.0f) continue;
                const bool artic_a = c.U(hSourceA, h) != kInvalid, artic_b = c.U(hSourceB, h) != kInvalid;
                if (artic_a && artic_b) {   // both sides on one owner (two owners were answered above)
                    const float* row = urows + size_t{c.U(hSlot, h)} * kRowWords;
                    if (__float_as_uint(row[11]) != __float_as_uint(row[19])) continue;
                }
                const bool second = artic_b && !artic_a;
                c.F(hStep, h) = second ? 0.0f : mine; c.F(hMove, h) = second ? mine : 0.0f;
            }
        }
        __syncthreads();
    }
    PROF_END(c, 18);
    PROF_BEGIN(c, 19);
    // InitializeTileHead (:743-797), lane = head
    bool any_elliptic = false;
    for (uint32_t base = 0u; base < heads; base += kWave) {
        const uint32_t h = base + lane;
        if (h < heads) {
            const uint32_t slot = c.U(hSlot, h);
            const float* row = urows + size_t{slot} * kRowWords;
            const uint32_t flags = __float_as_uint(row[0]), stride = __float_as_uint(row[2]);
            const uint32_t axes = (flags & kRowBlockNormal) != 0u ? 3u : 1u;
            const uint32_t kind_a = __float_as_uint(row[10]), kind_b = __float_as_uint(row[18]);
            const float shares[2] = {c.F(hStep, h), c.F(hMove, h)};
            const bool valid = shares[0] >= 0.0f && isfinite(shares[0]) && shares[1] >= 0.0f && isfinite(shares[1]);
            float response = shares[0] + shares[1];
            const float coupling = shares[0] * shares[1], largest = fmaxf(shares[0], shares[1]);
            if (!(valid && isfinite(response))) response = nanf("");
            const float coupled = coupling > 0.0f ? (response + sqrtf(response * response + 12.0f * coupling)) / (6.0f * coupling) : FLT_MAX;
            const float capv = kPenaltyConditionCap / largest;
            float rho = response > 0.0f ? fminf(capv, coupled) : 0.0f;
            if (!(response == 0.0f || (response > 0.0f && rho > 0.0f && rho <= FLT_MAX))) {
                atomicOr(d.env_status + env, kEnvStatusSolverFailure);
                rho = nanf("");
            }
            d.solver_penalty[slot] = rho;
            const float compliance = row[5];
            const Response sr = scalar_response(rho, compliance);
            const uint32_t local = slot - env * R;
            // three axes of a MuJoCo-law contact: the elliptic cone, with the compliances of the two tangent rows (:778-780)
            const bool elliptic = !kContactsOnly && axes == 3u && (flags & kRowMuJoCo) != 0u;
            any_elliptic = any_elliptic || elliptic;
            c.U(hStride, h) = stride; c.U(hAxes, h) = elliptic ? kAxesElliptic : axes;
            c.U(hOwned, h) = (kind_a == kSideArtic || kind_b == kSideArtic) ? 1u : 0u;
            c.F(hRho, h) = rho; c.F(hCompliance, h) = compliance; c.F(hLower, h) = row[6]; c.F(hUpper, h) = row[7];
            c.F(hMu1, h) = row[8]; c.F(hMu2, h) = row[9]; c.F(hNormalBound, h) = 0.0f;
            c.F(hDualScale, h) = sr.dual_scale; c.F(hResidualScale, h) = sr.residual_scale;
            const float dx = lambda_env[local], dy = axes == 3u ? lambda_env[local + stride] : 0.0f,
                        dz = axes == 3u ? lambda_env[local + 2u * stride] : 0.0f;
            c.F(hDual, h) = dx; c.F(hDual + 1, h) = dy; c.F(hDual + 2, h) = dz;
            c.F(hBase, h) = dx; c.F(hBase + 1, h) = dy; c.F(hBase + 2, h) = dz;
#pragma unroll
            for (int k = 0; k < 3; ++k) { c.F(hRes + k, h) = 0.0f; c.F(hMove + k, h) = 0.0f; c.F(hStep + k, h) = 0.0f; c.F(hRelaxStep + k, h) = 0.0f; c.F(hRelaxPoint + k, h) = 0.0f; }
            c.F(hRelaxWeight, h) = 0.0f;
            if (elliptic) {
                c.F(hTangentCompliance, h) = urows[size_t{slot + stride} * kRowWords + 5u];
                c.F(hTangentCompliance + 1, h) = urows[size_t{slot + 2u * stride} * kRowWords + 5u];
            }
        }
    }
    c.elliptic = !kContactsOnly && __any(any_elliptic);
    __syncthreads();
    PROF_END(c, 19);
    PROF_BEGIN(c, 20);
    // the one factorisation of the mass matrix
    c.mass_valid = factor_mass<W>(c, mrow) && reduction_valid;
    PROF_END(c, 20);
    PROF_BEGIN(c, 21);
    initialize_residuals<W>(c, velocity, urows, p.dt);
    PROF_END(c, 21);
    PROF_END(c, 0);
    float residual4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t sweeps = 0u;
    DualMomentum momentum{1.0f, 0.0f};
    const float tol = c.tolerance;
    while (sweeps < p.iterations) {
        c.iteration = sweeps++;
        c.momentum = 0.0f; c.residual = 0.0f;
        PROF_COUNT(c, 2);
        descend_block<W, kReduced>(c, mrow, mlow, &velocity, free_v, true, d);
        float rowsr[3];
        PROF_BEGIN(c, 6);
        update_duals(c, lambda_env, R, urows, &momentum, true, true, rowsr);
        PROF_END(c, 6);
        PROF_BEGIN(c, 7);
        if (sweeps == p.iterations || fmaxf(fmaxf(rowsr[0], rowsr[1]), fmaxf(rowsr[2], c.residual)) < tol)
            measure_primal<W, kReduced>(c, mrow, mlow, &velocity, free_v, lambda_env, R, false, d);
        PROF_END(c, 7);
        if (fmaxf(fmaxf(rowsr[0], rowsr[1]), rowsr[2]) < tol && c.residual >= tol && c.residual < FLT_MAX) {
            measure_primal<W, kReduced>(c, mrow, mlow, &velocity, free_v, lambda_env, R, true, d);
            if (c.residual < FLT_MAX) {
                initialize_residuals<W>(c, velocity, urows, p.dt);
                update_duals(c, lambda_env, R, urows, nullptr, true, false, rowsr);
                c.residual = 0.0f;
                measure_primal<W, kReduced>(c, mrow, mlow, &velocity, free_v, lambda_env, R, false, d);
            }
        }
        residual4[0] = rowsr[0]; residual4[1] = rowsr[1]; residual4[2] = rowsr[2]; residual4[3] = c.residual;
        const float largest = fmaxf(fmaxf(rowsr[0], rowsr[1]), fmaxf(rowsr[2], c.residual));
        if (largest < tol || largest == FLT_MAX) break;
    }
    if (lane < 4u)
        d.solver_residual[size_t{env} * 4u + lane] =
            lane == 0u ? residual4[0] : lane == 1u ? residual4[1] : lane == 2u ? residual4[2] : residual4[3];
    if (lane == 0u) {
        d.vbd_velocity_sweep_count[env] = sweeps;
        // the scheduling key of the next solves: this solve's work, or what is left of an earlier, longer one - an
        // environment whose solves are long every other step or so keeps its early place in the launch order
        const uint32_t earlier = d.solver_cost[env];
        d.solver_cost[env] = max(c.work, earlier - earlier / 4u);
    }
#ifdef NKH_SOLVER_PROFILE
    PROF_END(c, 9);
    if (lane == 0u) {
        for (int i = 0; i < 10; ++i) d.solver_penalty[size_t{env} * R + i] = float(c.prof[i]);
        for (int i = 0; i < 4; ++i) d.solver_penalty[size_t{env} * R + 10 + i] = float(c.prof_count[i]);
        for (int i = 10; i < 26; ++i) d.solver_penalty[size_t{env} * R + 4 + i] = float(c.prof[i]);
        for (int i = 26; i < 32; ++i) if (uint32_t(7 + i) < R) d.solver_penalty[size_t{env} * R + 7 + i] = float(c.prof[i]);
        // launch slot and the wave's first and last moment on the constant 100 MHz clock, as raw words
        d.solver_penalty[size_t{env} * R + 30] = __uint_as_float(uint32_t(prof_wall_start));
        d.solver_penalty[size_t{env} * R + 31] = __uint_as_float(uint32_t(wall_clock64()));
        d.solver_penalty[size_t{env} * R + 32] = __uint_as_float(blockIdx.x);
    }
#endif
    // the block velocities persist for the next solve's carried start
    if (lane < md) {
        d.solver_velocity[size_t{env} * md + lane] = coordinate ? velocity : 0.0f;
        d.solver_free[size_t{env} * md + lane] = coordinate ? free_v : 0.0f;
    }
    // FinishTile (:2607-2650)
    const bool invalid = __any(coordinate && !(fabsf(velocity) <= FLT_MAX));
    if (!invalid) {
        if (lane < md) d.qdot_flat[size_t{env} * md + lane] = coordinate ? velocity : 0.0f;
        if (coordinate) {
            if (my_component == kInvalid) d.qdot[lbase + my_link] = velocity;
            else d.link_velocity[(lbase + my_link) * 6u + my_component] = velocity;
        }
    } else if (lane == 0u) d.env_status[env] |= kEnvStatusSolverFailure;
    // joint limit impulses (:2658-2668)
    if (p.base_link_count != 0u && p.joint_limit_rows_per_env >= 2u * p.base_link_count) {
        for (uint32_t l = lane; l < nl; l += kWave) {
            const size_t lower = size_t{env} * R + p.contact_rows_per_env + size_t{l} * 2u;
            d.joint_limit_impulse[2u * (lbase + l)] = (__float_as_uint(urows[lower * kRowWords]) & kRowActive) != 0u ? d.lambda[lower] : 0.0f;
            d.joint_limit_impulse[2u * (lbase + l) + 1u] = (__float_as_uint(urows[(lower + 1u) * kRowWords]) & kRowActive) != 0u ? d.lambda[lower + 1u] : 0.0f;
        }
    }
    // split-impulse position pass (:3059-3077; MarkTilePositions :2673-2708; PositionRowBias block_descent.cu:1734-1753)
    if (p.position_iterations != 0u) {
        float* qvec = c.vec + 128;
        qvec[lane] = coordinate ? velocity : 0.0f;   // the final generalized velocity, as qdot_flat
        __syncthreads();
        bool push = false;
        for (uint32_t h = lane; h < heads; h += kWave) {
            const uint32_t slot = c.U(hSlot, h);
            const float* row = urows + size_t{slot} * kRowWords;
            const uint32_t flags = __float_as_uint(row[0]);
            const float penetration = d.row_penetration[slot];
            const bool speculative = (flags & kRowSpeculative) != 0u;
            const float slop = speculative ? 0.0f : p.position_slop;
            const bool position = (flags & (kRowFriction | kRowVelocityOnly | kRowMuJoCo)) == 0u &&
                (speculative || penetration > slop || c.F(hDual, h) != 0.0f);
            float bias = 0.0f, rounding = 0.0f;
            if (position) {
                const float pen = fmaxf(penetration - slop, 0.0f);
                if (speculative) {
                    // the contact slot whose normal rows hold this row (MapRowContactsKernel, block_descent.cu:1756-1767)
                    const uint32_t group_first = __float_as_uint(row[1]), points = __float_as_uint(row[2]);
                    uint32_t contact = 0u;
                    for (uint32_t s = 0u; s < S; ++s)
                        if (d.ucontact_row_range[(size_t{env} * S + s) * 2u] == group_first &&
                            d.ucontact_row_range[(size_t{env} * S + s) * 2u + 1u] > 0u) contact = env * S + s;
                    const size_t point = size_t{contact} * 4u + (slot - group_first) % points;
                    const double depth = double(d.ucontact_depth[point]) - slop;
                    const double reserve = double(penetration) - d.ucontact_depth[point];
                    const double correction = p.position_beta * fmax(depth, 0.0) + reserve;
                    const double target = fmin(depth, 0.0) + correction;
                    double vel = 0.0;   // RowVelocity (block_descent.cu:1051-1082) per articulated side
                    const uint32_t kind_a = __float_as_uint(row[10]), kind_b = __float_as_uint(row[18]);
                    if (kind_a == kSideArtic) {
                        double value = 0.0;
                        for (uint32_t k = 0u; k < n; ++k) value += double(d.chain_jacobian[size_t{slot} * md + k]) * qvec[k];
                        vel += value;
                    }
                    if (kind_b == kSideArtic) {
                        double value = 0.0;
                        for (uint32_t k = 0u; k < n; ++k) value += double(d.chain_jacobian_b[size_t{slot} * md + k]) * qvec[k];
                        vel += value;
                    }
                    const double limit = fmin(correction / p.dt, double(p.position_max_velocity));
                    const double absorbed = target > 0.0 ? 0.0 : fmax(reserve, 0.0) / p.dt;
                    bias = float(fmin(target / p.dt - vel, limit));
                    rounding = float(absorbed);
                } else {
                    const float correction = p.position_beta * pen + fmaxf(pen - pen, 0.0f);
                    bias = fminf(correction / p.dt, p.position_max_velocity);
                }
            }
            if (!position) c.U(hOwned, h) = 0u;
            const Response sr = scalar_response(c.F(hRho, h), 0.0f);
            c.U(hAxes, h) = 1u;
            c.F(hCompliance, h) = 0.0f; c.F(hLower, h) = 0.0f; c.F(hUpper, h) = FLT_MAX;
            c.F(hDualScale, h) = sr.dual_scale; c.F(hResidualScale, h) = sr.residual_scale;
            c.F(hRes, h) = bias; c.F(hRes + 1, h) = 0.0f; c.F(hRes + 2, h) = 0.0f;
            c.F(hDual, h) = 0.0f; c.F(hDual + 1, h) = 0.0f; c.F(hDual + 2, h) = 0.0f;
            push = push || bias > rounding;
        }
        push = __any(push);
        __syncthreads();
        float pseudo = 0.0f;
        if (push) {
            const uint32_t positions = 1u;   // no head couples two moving blocks here, so one solve (:2716)
            for (uint32_t iteration = 0u; iteration < positions; ++iteration) {
                c.iteration = sweeps + iteration;
                descend_block<W, kReduced>(c, mrow, mlow, &pseudo, 0.0f, false, d);
            }
        }
        // FinishTilePositions (:2720-2744)
        if (coordinate) {
            if (my_component == kInvalid) d.qdot_pseudo[lbase + my_link] = pseudo;
            else d.link_velocity_pseudo[(lbase + my_link) * 6u + my_component] = pseudo;
        }
    }
}

#ifdef NKH_SOLVER_DENSE
}  // namespace dense
#endif
}  // namespace solver
}  // namespace nkh
