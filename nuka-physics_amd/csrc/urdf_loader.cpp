// URDF template loader: reads a URDF robot description into the cook inputs of one environment
// (nuka_template_desc_t).  Counterpart, for the articulation-step path, of src/import/urdf_importer.cpp (LoadUrdf):
// links with their inertial and collision elements, revolute / continuous / prismatic / fixed joints with origin, axis,
// limits, dynamics and effort, and the robot-level nuka:exclude element.  Host code only.
//
// Not read: visuals and materials, meshes (a mesh collision is a shape this library has no manifold for), mimic,
// planar and floating joints (rejected), transmissions, gazebo extensions.
#include "scene_loader.h"

#include "scene_build.h"

namespace nkh {
namespace scene_file {
namespace {

// urdf_importer.cpp:45-56 ParseOrigin: xyz, and fixed-axis roll-pitch-yaw composed as Rz(yaw) Ry(pitch) Rx(roll)
void ParseOrigin(const Element* origin, V3* position, Quat* rotation) {
    *position = V3{};
    *rotation = Quat{};
    if (origin == nullptr) return;
    if (origin->Attribute("xyz")) *position = ParseV3(origin->Attribute("xyz"));
    if (origin->Attribute("rpy")) {
        const V3 angle = ParseV3(origin->Attribute("rpy"));
        *rotation = Normalized(Mul(Mul(AxisAngle(V3{0, 0, 1}, angle.z), AxisAngle(V3{0, 1, 0}, angle.y)), AxisAngle(V3{1, 0, 0}, angle.x)));
    }
}

struct UrdfLink {
    Link link;              // frame, joint and drive members are filled from the joint that carries it
    uint32_t parent = 0xFFFFFFFFu;   // index among the file's links
    bool carried = false;
};

}  // namespace

std::unique_ptr<Scene> LoadUrdf(const std::string& path, uint32_t flags) {
    const std::string text = ReadFile(path);
    std::unique_ptr<Element> robot = XmlReader(text).Document();
    if (robot->name != "robot") throw std::runtime_error("URDF: missing <robot> root element in " + path);

    std::vector<UrdfLink> links;
    std::map<std::string, uint32_t> link_index;
    // links (urdf_importer.cpp:380-470): a link without <inertial> is massless, as the format defines
    robot->Each("link", [&](const Element& e) {
        UrdfLink record;
        Link& link = record.link;
        link.name = e.Attribute("name") != nullptr ? e.Attribute("name") : "unnamed";
        if (const Element* inertial = e.First("inertial")) {
            if (const Element* mass = inertial->First("mass")) QueryFloat(*mass, "value", &link.mass);
            ParseOrigin(inertial->First("origin"), &link.inertial_position, &link.inertial_rotation);
            if (const Element* inertia = inertial->First("inertia")) {
                const char* keys[6] = {"ixx", "iyy", "izz", "ixy", "ixz", "iyz"};
                double full[6] = {0, 0, 0, 0, 0, 0};
                for (int k = 0; k < 6; ++k) { float v = 0.0f; QueryFloat(*inertia, keys[k], &v); full[k] = v; }
                Quat axes;
                Diagonalize(full, &link.inertia, &axes);
                link.inertial_rotation = Mul(link.inertial_rotation, axes);
            }
        }
        e.Each("collision", [&](const Element& collision) {
            const Element* geometry = collision.First("geometry");
            if (geometry == nullptr || geometry->children.empty()) return;
            const Element& shape = *geometry->children.front();
            Geom g;
            ParseOrigin(collision.First("origin"), &g.position, &g.rotation);
            if (shape.name == "box") {
                g.kind = kShapeBox;
                const V3 size = ParseV3(shape.Attribute("size"));
                g.params[0] = 0.5f * size.x; g.params[1] = 0.5f * size.y; g.params[2] = 0.5f * size.z;
            } else if (shape.name == "sphere") {
                g.kind = kShapeSphere;
                QueryFloat(shape, "radius", &g.params[0]);
            } else if (shape.name == "cylinder" || shape.name == "capsule") {
                g.kind = shape.name == "cylinder" ? kShapeCylinder : kShapeCapsule;
                float length = 1.0f;
                QueryFloat(shape, "radius", &g.params[0]);
                QueryFloat(shape, "length", &length);
                g.params[1] = 0.5f * length;
            } else {
                g.kind = kShapeUnknown;   // mesh
            }
            link.geoms.push_back(g);
        });
        if (!link_index.emplace(link.name, uint32_t(links.size())).second) throw std::runtime_error("URDF: link names must be unique");
        links.push_back(record);
    });
    if (links.empty()) throw std::runtime_error("URDF: no <link> in " + path);

    // joints (urdf_importer.cpp:563-640): the joint's origin is the child link's frame in the parent link's, its axis
    // is written in that frame and defaults to x
    SceneParts parts;
    std::map<std::string, bool> joint_names;
    uint32_t drive_mode = 1u;   // effort limits make torque motors
    robot->Each("joint", [&](const Element& e) {
        const std::string name = e.Attribute("name") != nullptr ? e.Attribute("name") : "";
        if (name.empty() || !joint_names.emplace(name, true).second) throw std::runtime_error("URDF: joint names must be unique and nonempty");
        const std::string type = e.Attribute("type") != nullptr ? e.Attribute("type") : "";
        auto link_of = [&](const char* tag) {
            const Element* element = e.First(tag);
            const char* link = element != nullptr ? element->Attribute("link") : nullptr;
            const auto found = link != nullptr ? link_index.find(link) : link_index.end();
            if (found == link_index.end()) throw std::runtime_error("URDF: joint '" + name + "' has no declared " + tag + " link");
            return found->second;
        };
        const uint32_t parent = link_of("parent"), child = link_of("child");
        UrdfLink& record = links[child];
        if (record.carried || parent == child) throw std::runtime_error("URDF: link '" + record.link.name + "' is the child of more than one joint");
        record.carried = true;
        record.parent = parent;
        Link& link = record.link;
        link.joint_name = name;
        if (type == "revolute" || type == "continuous") link.joint_type = 0u;
        else if (type == "prismatic") link.joint_type = 1u;
        else if (type == "fixed") link.joint_type = 2u;
        else throw Unsupported("URDF: joint '" + name + "' of type '" + type + "' is not supported on this path");
        ParseOrigin(e.First("origin"), &link.position, &link.rotation);
        link.axis = V3{1.0f, 0.0f, 0.0f};
        if (const Element* axis = e.First("axis")) if (axis->Attribute("xyz")) link.axis = ParseV3(axis->Attribute("xyz"));
        if (link.joint_type <= 1u) {
            if (!(Length(link.axis) > 0.0f)) throw std::runtime_error("URDF: joint '" + name + "' has a zero axis");
            link.axis = Unit(link.axis);
        }
        float effort = 0.0f;
        if (const Element* limit = e.First("limit")) {
            const bool lower = QueryFloat(*limit, "lower", &link.lower), upper = QueryFloat(*limit, "upper", &link.upper);
            link.limited = type != "continuous" && lower && upper;
            if (link.limited && link.lower > link.upper) throw std::runtime_error("URDF: joint '" + name + "' has its lower limit above the upper");
            QueryFloat(*limit, "effort", &effort);
        }
        if (const Element* dynamics = e.First("dynamics")) {
            QueryFloat(*dynamics, "damping", &link.damping);
            QueryFloat(*dynamics, "friction", &link.frictionloss);
        }
        if (link.damping < 0.0f || link.frictionloss < 0.0f || effort < 0.0f) throw std::runtime_error("URDF: joint '" + name + "' has a negative damping, friction or effort");
        if (e.First("mimic") != nullptr) throw Unsupported("URDF: mimic joint '" + name + "' is not supported on this path");
        if (effort > 0.0f && link.joint_type <= 1u) {   // a torque motor bounded by the effort (urdf_importer.cpp:631-638)
            link.drive_force_limit = effort;
            ++parts.actuator_count;
        }
    });

    // one root, parents before children in the order the file lists the links
    uint32_t root = 0xFFFFFFFFu;
    for (uint32_t l = 0u; l < links.size(); ++l)
        if (!links[l].carried) {
            if (root != 0xFFFFFFFFu) throw std::runtime_error("URDF: expected one root link in " + path);
            root = l;
        }
    if (root == 0xFFFFFFFFu) throw std::runtime_error("URDF: the joints form a loop in " + path);
    std::vector<uint32_t> order{root}, place(links.size(), 0xFFFFFFFFu);
    place[root] = 0u;
    for (size_t at = 0u; at < order.size(); ++at)
        for (uint32_t l = 0u; l < links.size(); ++l)
            if (links[l].carried && links[l].parent == order[at]) { place[l] = uint32_t(order.size()); order.push_back(l); }
    if (order.size() != links.size()) throw std::runtime_error("URDF: the joints form a loop in " + path);
    const bool fixed_base = (flags & kFixedBase) != 0u;
    for (uint32_t l : order) {
        Link link = links[l].link;
        if (l == root) {
            link.parent = 0xFFFFFFFFu;
            link.joint_type = fixed_base ? 2u : 3u;
            link.joint_name = link.name + "/base";
        } else {
            link.parent = place[links[l].parent];
            // a moving link the file gives no inertia would leave the mass matrix singular: it gets the inertia a
            // massless intermediate link of a several-joint MJCF body gets
            if (link.joint_type <= 1u && !(link.mass > 0.0f)) { link.mass = 1.0e-6f; link.inertia = {1.0e-9f, 1.0e-9f, 1.0e-9f}; }
        }
        parts.links.push_back(link);
    }
    parts.floating_root = !fixed_base;
    // nuka:exclude link1 link2 (urdf_importer.cpp:642-653): unknown or identical links are an error
    robot->Each("nuka:exclude", [&](const Element& e) {
        const char* first = e.Attribute("link1");
        const char* second = e.Attribute("link2");
        if (first == nullptr || second == nullptr || link_index.count(first) == 0u || link_index.count(second) == 0u || std::string(first) == second)
            throw std::runtime_error("URDF: nuka:exclude needs two distinct existing links");
        parts.excluded_bodies.emplace_back(first, second);
    });

    auto scene = std::make_unique<Scene>();
    scene->timestep = 1.0f / 240.0f;   // the format names none: the library's default step
    // a URDF carries no MuJoCo law: its shapes and joints keep the native rows (only the MJCF and USD importers of the
    // reference mark theirs MuJoCo-sourced)
    FlattenScene(parts, flags | kNativeContactLaw | kNativeJointLaw, drive_mode, scene.get());
    return scene;
}

}  // namespace scene_file
}  // namespace nkh
