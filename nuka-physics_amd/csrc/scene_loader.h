// The robot-description loaders' result: the arrays behind a nuka_template_desc_t plus what else the file authors
// for the articulation-step path (names, initial state, drive parameters).  Host code only.
#pragma once

#include <array>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/nuka_hip.h"

namespace nkh {
namespace scene_file {

// Keep sphere and box geoms against planes only: other colliding geoms are dropped (and counted), and the robot's
// geoms share one negative collision group so that they meet the ground and not each other.
constexpr uint32_t kPlaneContactsOnly = 1u;
// URDF: the root link is welded to the world instead of floating.
constexpr uint32_t kFixedBase = 2u;
// A static ground plane z = 0 is added to the file's collidables (a URDF names none).
constexpr uint32_t kGroundPlane = 4u;
// MJCF: the geoms keep this library's native contact law (speculative velocity rows) instead of the MuJoCo law the
// reference's importer gives every MJCF shape (src/import/mjcf_importer.cpp:790).
constexpr uint32_t kNativeContactLaw = 8u;
// MJCF: the joints keep the native limit and friction rows and the native integrator (drive damping folded into the
// solve) instead of MuJoCo-sourced rows and the MuJoCo integrator of <option> (mjcf_importer.cpp:1193, 1720).
constexpr uint32_t kNativeJointLaw = 16u;

struct Scene {
    nuka_template_desc_t desc{};
    std::vector<std::string> link_names, joint_names;
    std::vector<uint8_t> joint_type, joint_limit_flags, joint_law;
    std::vector<uint32_t> parent_link, body_role, body_link, shape_kind, shape_contype, shape_conaffinity, shape_group, shape_profile,
        excluded_pairs;   // [pair][2] collidable rows that never pair
    std::vector<float> joint_axis, link_local_pose, link_inertial_frame, link_mass, link_diag_inertia, joint_damping, joint_armature,
        joint_stiffness, joint_spring_reference, joint_frictionloss, joint_limit_lower, joint_limit_upper, body_local, shape_params, profile_mu,
        profile_solref, profile_solimp, profile_margin, profile_solmix, joint_limit_margin, joint_limit_reference, joint_friction_reference;
    std::vector<uint32_t> profile_law, profile_condim;
    std::vector<int32_t> profile_priority;
    uint32_t contact_cone = 0u;      // <option cone>: 0 pyramidal (MuJoCo's default), 1 elliptic
    float contact_impratio = 1.0f;   // <option impratio>
    uint32_t integrator = 0u;        // 0 native; 1 MuJoCo's Euler; 2 implicit / implicitfast (<option integrator>)
    std::vector<float> initial_q, drive_stiffness, drive_damping, drive_force_limit, drive_joint_force_limit;
    std::array<float, 7> base_pose{0, 0, 0, 1, 0, 0, 0};
    bool floating_root = false;
    uint32_t actuator_count = 0u, dropped_geom_count = 0u, drive_mode = 1u;
    float timestep = 0.002f;
    float gravity[3] = {0.0f, 0.0f, -9.81f};
    void Bind();   // points `desc` at the arrays
};

// A well-formed file that uses what this path does not build (a ball joint, a mimic joint, an actuator kind).
struct Unsupported : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// Throws std::runtime_error with the reason when the file cannot be read, Unsupported when it uses what this path does
// not build.
std::unique_ptr<Scene> LoadMjcf(const std::string& path, uint32_t flags);
std::unique_ptr<Scene> LoadUrdf(const std::string& path, uint32_t flags);

}  // namespace scene_file
}  // namespace nkh
