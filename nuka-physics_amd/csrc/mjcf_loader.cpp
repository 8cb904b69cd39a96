// MJCF template loader: reads a MuJoCo XML robot description into the cook inputs of one environment
// (nuka_template_desc_t).  Counterpart, for the articulation-step path, of src/import/mjcf_importer.cpp (LoadMjcf)
// followed by the articulation part of the cook (src/runtime/articulation/articulation_state.cpp:345-435): the
// same body -> link rules, default classes, joint anchors, inertial sources and actuator mapping.  Host code only.
//
// Not read: meshes, height fields, materials, cameras, lights, sensors, sites, equalities, <contact> pairs, ball
// joints (rejected), tendons.  Geoms carry the MuJoCo contact law as in the reference's importer (every MJCF shape is
// MuJoCo-sourced, mjcf_importer.cpp:790): friction, solref, solimp, margin and gap go into contact profiles, and
// <option cone impratio> selects the cone.  Joints carry the MuJoCo law too (margin, solreflimit / solimplimit,
// solreffriction / solimpfriction: compliant limit and friction rows), and <option integrator> selects the damping
// pass after the solve.
#include "scene_loader.h"

#include "scene_build.h"

namespace nkh {
namespace scene_file {
namespace {

// ---- default classes (mjcf_importer.cpp:104-190, 309-430, 522-556) --------------------------------------------
enum class JointKind { Hinge, Slide, Free, Ball, Fixed };
JointKind JointKindOf(const char* type) {
    if (type == nullptr) return JointKind::Hinge;
    const std::string t(type);
    if (t == "hinge") return JointKind::Hinge;
    if (t == "slide") return JointKind::Slide;
    if (t == "free") return JointKind::Free;
    if (t == "ball") return JointKind::Ball;
    throw std::runtime_error("MJCF: unknown joint type '" + t + "'");
}
struct JointDefaults {
    JointKind type = JointKind::Hinge;
    V3 axis{0.0f, 0.0f, 1.0f};
    float lower = -3.14159f, upper = 3.14159f;
    bool has_range = false;
    int limited = -1;
    float damping = 0.0f, armature = 0.0f, frictionloss = 0.0f, actuator_force_limit = 0.0f, stiffness = 0.0f, spring_reference = 0.0f;
    float limit_margin = 0.0f;
    float limit_reference[7] = {0.02f, 1.0f, 0.9f, 0.95f, 0.001f, 0.5f, 2.0f};      // solreflimit, solimplimit
    float friction_reference[7] = {0.02f, 1.0f, 0.9f, 0.95f, 0.001f, 0.5f, 2.0f};   // solreffriction, solimpfriction
};
struct Frame {
    V3 position;
    std::string orientation_tag, orientation_value, fromto;
};
struct GeomDefaults : Frame {
    bool has_type = false;        std::string type;
    bool has_size = false;        float size[3] = {0.5f, 0.5f, 0.5f};
    bool has_contype = false;     uint32_t contype = 1u;
    bool has_conaffinity = false; uint32_t conaffinity = 1u;
    bool has_group = false;       int32_t group = 0;
    float friction[3] = {1.0f, 0.005f, 0.0001f};
    float solref[2] = {0.02f, 1.0f};
    float solimp[5] = {0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
    float margin = 0.0f, gap = 0.0f, solmix = 1.0f;
    long priority = 0, condim = 3;
    float density = 1000.0f, mass = -1.0f;
};
struct GeneralDefaults {
    float gear = 1.0f, force_limit = 0.0f, gain = 1.0f;
    float bias[3] = {0.0f, 0.0f, 0.0f};
    bool affine = false;
};
struct DefaultClass { JointDefaults joint; GeomDefaults geom; GeneralDefaults general; };

void ParseActuatorForceRange(const Element& e, float* limit) {
    if (const char* range = e.Attribute("actuatorfrcrange")) {
        float bounds[2] = {0.0f, 0.0f};
        ParseFloats(range, bounds, 2);
        *limit = std::max(std::fabs(bounds[0]), std::fabs(bounds[1]));
    }
    if (const char* limited = e.Attribute("actuatorfrclimited"); limited != nullptr && std::string(limited) == "false") *limit = 0.0f;
}
void ApplyJointAttributes(const Element& e, JointDefaults* j) {
    if (e.Attribute("type")) j->type = JointKindOf(e.Attribute("type"));
    if (e.Attribute("axis")) j->axis = ParseV3(e.Attribute("axis"));
    if (e.Attribute("range")) {
        float bounds[2] = {j->lower, j->upper};
        ParseFloats(e.Attribute("range"), bounds, 2);
        j->lower = bounds[0]; j->upper = bounds[1];
        j->has_range = true;
    }
    j->limited = ParseLimited(e.Attribute("limited"), j->limited);
    QueryFloat(e, "damping", &j->damping);
    QueryFloat(e, "armature", &j->armature);
    QueryFloat(e, "frictionloss", &j->frictionloss);
    QueryFloat(e, "margin", &j->limit_margin);   // mjcf_importer.cpp:334-338, 1209-1213
    ParseFloats(e.Attribute("solreflimit"), j->limit_reference, 2);
    ParseFloats(e.Attribute("solimplimit"), j->limit_reference + 2, 5);
    ParseFloats(e.Attribute("solreffriction"), j->friction_reference, 2);
    ParseFloats(e.Attribute("solimpfriction"), j->friction_reference + 2, 5);
    ParseActuatorForceRange(e, &j->actuator_force_limit);
    QueryFloat(e, "stiffness", &j->stiffness);
    QueryFloat(e, "springref", &j->spring_reference);
}
void ApplyFrame(const Element& e, Frame* frame) {
    if (e.Attribute("pos")) frame->position = ParseV3(e.Attribute("pos"));
    uint32_t rotations = 0u;
    for (const char* tag : {"quat", "axisangle", "euler", "xyaxes", "zaxis"})
        if (const char* value = e.Attribute(tag)) { frame->orientation_tag = tag; frame->orientation_value = value; ++rotations; }
    if (rotations > 1u) throw std::runtime_error("MJCF: multiple orientation attributes");
    if (e.Attribute("fromto")) frame->fromto = e.Attribute("fromto");
}
void ApplyGeomAttributes(const Element& e, GeomDefaults* g) {
    ApplyFrame(e, g);
    if (e.Attribute("size")) {
        if (ParseFloats(e.Attribute("size"), g->size, 3) == 0) throw std::runtime_error("MJCF: invalid geom size");
        g->has_size = true;
    }
    if (e.Attribute("type")) { g->type = e.Attribute("type"); g->has_type = true; }
    long value = 0;
    if (QueryInt(e, "contype", &value)) { g->contype = uint32_t(value); g->has_contype = true; }
    if (QueryInt(e, "conaffinity", &value)) { g->conaffinity = uint32_t(value); g->has_conaffinity = true; }
    if (QueryInt(e, "group", &value)) { g->group = int32_t(value); g->has_group = true; }
    ParseFloats(e.Attribute("friction"), g->friction, 3);
    ParseFloats(e.Attribute("solref"), g->solref, 2);
    ParseFloats(e.Attribute("solimp"), g->solimp, 5);
    QueryFloat(e, "margin", &g->margin);
    QueryFloat(e, "gap", &g->gap);
    QueryFloat(e, "solmix", &g->solmix);
    QueryInt(e, "priority", &g->priority);
    QueryInt(e, "condim", &g->condim);
    QueryFloat(e, "density", &g->density);
    QueryFloat(e, "mass", &g->mass);
}
void ApplyGeneralAttributes(const Element& e, GeneralDefaults* g) {
    QueryFloat(e, "gear", &g->gear);
    if (e.Attribute("forcerange")) { float bounds[2] = {g->force_limit, g->force_limit}; ParseFloats(e.Attribute("forcerange"), bounds, 2); g->force_limit = bounds[1]; }
    ParseFloats(e.Attribute("gainprm"), &g->gain, 1);
    ParseFloats(e.Attribute("biasprm"), g->bias, 3);
    if (const char* bias = e.Attribute("biastype")) g->affine = std::string(bias) == "affine";
}

struct Context {
    DefaultClass root;
    std::map<std::string, DefaultClass> classes;
    float angle_scale = 0.017453292519943295f;   // compiler angle="degree" is MuJoCo's default
    std::string euler_sequence = "xyz";
    int inertia_from_geom = -1;
    int inertia_groups[2] = {0, 5};
    uint32_t flags = 0u;
    const DefaultClass& Class(const char* name) const {
        if (name == nullptr) return root;
        const auto found = classes.find(name);
        return found == classes.end() ? root : found->second;
    }
};
void ParseDefaultElement(const Element& e, const DefaultClass& inherited, Context* context) {
    DefaultClass current = inherited;
    if (const Element* joint = e.First("joint")) ApplyJointAttributes(*joint, &current.joint);
    if (const Element* general = e.First("general")) ApplyGeneralAttributes(*general, &current.general);
    if (const Element* geom = e.First("geom")) ApplyGeomAttributes(*geom, &current.geom);
    if (const char* name = e.Attribute("class")) context->classes[name] = current;
    else context->root = current;
    e.Each("default", [&](const Element& child) { ParseDefaultElement(child, current, context); });
}

Quat FrameOrientation(const Frame& frame, const Context& context) {   // mjcf_importer.cpp:452-489
    if (frame.orientation_tag.empty()) return Quat{};
    float v[6] = {};
    const int required = frame.orientation_tag == "xyaxes" ? 6 : frame.orientation_tag == "euler" || frame.orientation_tag == "zaxis" ? 3 : 4;
    if (ParseFloats(frame.orientation_value.c_str(), v, required) != required) throw std::runtime_error("MJCF: incomplete orientation");
    for (float value : v) if (!std::isfinite(value)) throw std::runtime_error("MJCF: invalid orientation");
    if (frame.orientation_tag == "quat") return Normalized(Quat{v[0], v[1], v[2], v[3]});
    if (frame.orientation_tag == "axisangle") return AxisAngle(Unit({v[0], v[1], v[2]}), v[3] * context.angle_scale);
    if (frame.orientation_tag == "zaxis") return ZRotation({v[0], v[1], v[2]});
    if (frame.orientation_tag == "xyaxes") {
        const V3 x = Unit({v[0], v[1], v[2]});
        const V3 raw_y{v[3], v[4], v[5]};
        const V3 y = Unit(raw_y - x * Dot(raw_y, x));
        const V3 z = Cross(x, y);
        const double matrix[3][3] = {{x.x, y.x, z.x}, {x.y, y.y, z.y}, {x.z, y.z, z.z}};
        return FromMatrix(matrix);
    }
    if (context.euler_sequence.size() != 3u) throw std::runtime_error("MJCF: invalid eulerseq");
    Quat q{};
    for (uint32_t axis = 0u; axis < 3u; ++axis) {
        const char code = context.euler_sequence[axis];
        V3 vector{};
        if (code == 'x' || code == 'X') vector.x = 1.0f;
        else if (code == 'y' || code == 'Y') vector.y = 1.0f;
        else if (code == 'z' || code == 'Z') vector.z = 1.0f;
        else throw std::runtime_error("MJCF: invalid eulerseq axis");
        const Quat rotation = AxisAngle(vector, v[axis] * context.angle_scale);
        q = code >= 'a' && code <= 'z' ? Mul(q, rotation) : Mul(rotation, q);
    }
    return Normalized(q);
}

// ---- the scene being built -------------------------------------------------------------------------------------
uint32_t GeomKind(const char* type) {
    if (type == nullptr) return kShapeSphere;   // MJCF's default geom is a sphere
    const std::string t(type);
    if (t == "sphere") return kShapeSphere;
    if (t == "capsule") return kShapeCapsule;
    if (t == "box") return kShapeBox;
    if (t == "plane") return kShapePlane;
    if (t == "cylinder") return kShapeCylinder;
    return kShapeUnknown;   // ellipsoid, mesh, sdf, hfield
}

// Mass properties of a primitive about its own centre (import/geom_inertia.cpp:62-97) summed into its body (:99-125).
void AddGeomMass(const Geom& g, float density, float mass, BodyMass* body) {
    const double kPi = 3.14159265358979323846;
    double volume = 0.0, d[3] = {0.0, 0.0, 0.0};
    const double r = g.params[0], h = g.params[1];
    if (g.kind == kShapeSphere) { volume = 4.0 / 3.0 * kPi * r * r * r; d[0] = d[1] = d[2] = 0.4 * volume * r * r; }
    else if (g.kind == kShapeCapsule) {
        const double tube = 2.0 * kPi * r * r * h, caps = 4.0 / 3.0 * kPi * r * r * r;
        volume = tube + caps;
        d[0] = d[1] = tube * (r * r / 4.0 + h * h / 3.0) + caps * (0.4 * r * r + h * h + 0.75 * h * r);
        d[2] = (tube / 2.0 + caps * 0.4) * r * r;
    } else if (g.kind == kShapeCylinder) {
        volume = 2.0 * kPi * r * r * h;
        d[0] = d[1] = volume * (r * r / 4.0 + h * h / 3.0);
        d[2] = volume * r * r / 2.0;
    } else if (g.kind == kShapeBox) {
        const double ex = g.params[0], ey = g.params[1], ez = g.params[2];
        volume = 8.0 * ex * ey * ez;
        d[0] = volume * (ey * ey + ez * ez) / 3.0; d[1] = volume * (ex * ex + ez * ez) / 3.0; d[2] = volume * (ex * ex + ey * ey) / 3.0;
    }
    if (volume <= 0.0) return;
    const double rho = mass < 0.0f ? density : mass / volume;
    const double m = rho * volume;
    const V3 x = Rotate(g.rotation, {1, 0, 0}), y = Rotate(g.rotation, {0, 1, 0}), z = Rotate(g.rotation, {0, 0, 1});
    const double rot[3][3] = {{x.x, y.x, z.x}, {x.y, y.y, z.y}, {x.z, y.z, z.z}};
    const double c[3] = {g.position.x, g.position.y, g.position.z};
    const double cc = c[0] * c[0] + c[1] * c[1] + c[2] * c[2];
    for (int i = 0; i < 3; ++i) {
        body->first[i] += m * c[i];
        for (int j = 0; j < 3; ++j) {
            double turned = 0.0;
            for (int k = 0; k < 3; ++k) turned += rot[i][k] * d[k] * rot[j][k];
            body->inertia[i][j] += rho * turned + m * ((i == j ? cc : 0.0) - c[i] * c[j]);
        }
    }
    body->mass += m;
}
void SetBodyMass(const BodyMass& sum, Link* link) {   // geom_inertia.cpp:127-143
    link->mass = float(sum.mass);
    link->inertia = {};
    link->inertial_position = {};
    link->inertial_rotation = {};
    if (sum.mass <= 0.0) return;
    const double c[3] = {sum.first[0] / sum.mass, sum.first[1] / sum.mass, sum.first[2] / sum.mass};
    const double cc = c[0] * c[0] + c[1] * c[1] + c[2] * c[2];
    double i[3][3];
    for (int a = 0; a < 3; ++a)
        for (int b = 0; b < 3; ++b) i[a][b] = sum.inertia[a][b] - sum.mass * ((a == b ? cc : 0.0) - c[a] * c[b]);
    const double full[6] = {double(float(i[0][0])), double(float(i[1][1])), double(float(i[2][2])), double(float(i[0][1])), double(float(i[0][2])), double(float(i[1][2]))};
    Diagonalize(full, &link->inertia, &link->inertial_rotation);
    link->inertial_position = {float(c[0]), float(c[1]), float(c[2])};
}

struct Builder : SceneParts {
    Context context;
    std::map<std::string, uint32_t> joint_links;   // joint name -> the link it moves

    // ParseGeoms (mjcf_importer.cpp:779-1036), collision attributes and mass only
    void ParseGeoms(const Element& body, const char* child_class, V3 shift, std::vector<Geom>* out, BodyMass* mass) {
        body.Each("geom", [&](const Element& e) {
            const char* geom_class = e.Attribute("class");
            const GeomDefaults& gd = context.Class(geom_class != nullptr ? geom_class : child_class).geom;
            Geom g;
            g.kind = GeomKind(e.Attribute("type") != nullptr ? e.Attribute("type") : gd.has_type ? gd.type.c_str() : nullptr);
            Frame frame = gd;
            ApplyFrame(e, &frame);
            g.position = frame.position;
            g.rotation = FrameOrientation(frame, context);
            float size[3] = {gd.size[0], gd.size[1], gd.size[2]};
            const char* size_attr = e.Attribute("size");
            if (size_attr != nullptr && ParseFloats(size_attr, size, 3) == 0) throw std::runtime_error("MJCF: invalid geom size");
            if (size_attr != nullptr || gd.has_size) {
                if (g.kind == kShapeBox || g.kind == kShapePlane) { g.params[0] = size[0]; g.params[1] = size[1]; g.params[2] = size[2]; }
                else if (g.kind == kShapeSphere) g.params[0] = size[0];
                else if (g.kind == kShapeCapsule || g.kind == kShapeCylinder) { g.params[0] = size[0]; if (size[1] > 0.0f) g.params[1] = size[1]; }
            }
            if (!frame.fromto.empty()) {
                float points[6];
                const bool axial = g.kind == kShapeCapsule || g.kind == kShapeCylinder;
                if (ParseFloats(frame.fromto.c_str(), points, 6) != 6 || (!axial && g.kind != kShapeBox)) throw std::runtime_error("MJCF: invalid geom fromto");
                const V3 a{points[0], points[1], points[2]}, b{points[3], points[4], points[5]};
                g.position = (a + b) * 0.5f;
                g.rotation = ZRotation(b - a);
                const float half_length = Length(b - a) * 0.5f;
                if (axial) g.params[1] = half_length; else g.params[2] = half_length;
            }
            g.position = g.position + shift;
            if (gd.has_contype) g.contype = gd.contype;
            if (gd.has_conaffinity) g.conaffinity = gd.conaffinity;
            if (gd.has_group) g.group = gd.group;
            long value = 0;
            if (QueryInt(e, "contype", &value)) g.contype = uint32_t(value);
            if (QueryInt(e, "conaffinity", &value)) g.conaffinity = uint32_t(value);
            if (QueryInt(e, "group", &value)) g.group = int32_t(value);
            float friction[3] = {gd.friction[0], gd.friction[1], gd.friction[2]};
            ParseFloats(e.Attribute("friction"), friction, 3);
            g.friction = friction[0];
            g.friction_authored = g.friction != 1.0f;
            g.solref[0] = gd.solref[0]; g.solref[1] = gd.solref[1];
            for (int k = 0; k < 5; ++k) g.solimp[k] = gd.solimp[k];
            g.margin = gd.margin; g.gap = gd.gap;
            ParseFloats(e.Attribute("solref"), g.solref, 2);
            ParseFloats(e.Attribute("solimp"), g.solimp, 5);
            QueryFloat(e, "margin", &g.margin);
            QueryFloat(e, "gap", &g.gap);
            long priority = gd.priority, condim = gd.condim;
            g.solmix = gd.solmix;
            QueryFloat(e, "solmix", &g.solmix);
            QueryInt(e, "priority", &priority);
            QueryInt(e, "condim", &condim);
            g.priority = int32_t(priority);
            // the contact dimensions the path has rows for (scene/cook/cook_to_model.cpp:188-196 and nk/model/model.cpp:66
            // refuse every other value; torsional and rolling friction, condim 4 and 6, get no rows in assemble_rows.cu)
            if (condim != 1 && condim != 3) throw Unsupported("MJCF: geom condim " + std::to_string(condim) + " is not supported on this path (1 or 3)");
            g.condim = uint32_t(condim);
            if (!(g.margin >= 0.0f) || !(g.gap >= 0.0f)) throw std::runtime_error("MJCF: geom margin and gap must not be negative");
            float density = gd.density, geom_mass = gd.mass;
            QueryFloat(e, "density", &density);
            QueryFloat(e, "mass", &geom_mass);
            if (mass != nullptr && g.group >= context.inertia_groups[0] && g.group <= context.inertia_groups[1]) AddGeomMass(g, density, geom_mass, mass);
            out->push_back(g);
        });
    }

    // ParseBody (mjcf_importer.cpp:1038-1295)
    void ParseBody(const Element& e, uint32_t parent, const char* inherited_class) {
        const std::string body_name = e.Attribute("name") != nullptr ? e.Attribute("name") : "unnamed";
        const char* child_class = e.Attribute("childclass") != nullptr ? e.Attribute("childclass") : inherited_class;
        const bool root = parent == 0xFFFFFFFFu;
        const Element* free_joint = e.First("freejoint");
        // the joints that move this body, in order; a free joint may also be written <joint type="free"/>
        struct Hinge { const Element* element; V3 anchor; };
        std::vector<Hinge> chain;
        V3 anchor;
        bool free_by_type = false;
        e.Each("joint", [&](const Element& joint) {
            const char* joint_class = joint.Attribute("class");
            const JointKind kind = joint.Attribute("type") != nullptr ? JointKindOf(joint.Attribute("type"))
                                                                      : context.Class(joint_class != nullptr ? joint_class : child_class).joint.type;
            if (kind == JointKind::Free) { free_by_type = true; return; }
            if (kind == JointKind::Fixed) return;
            if (kind == JointKind::Ball) throw Unsupported("MJCF: ball joint on body '" + body_name + "' is not supported on this path");
            if (kind != JointKind::Slide && joint.Attribute("pos") != nullptr) anchor = ParseV3(joint.Attribute("pos"));
            chain.push_back({&joint, anchor});
        });
        const bool is_free = free_joint != nullptr || free_by_type;
        if (is_free && (!root || !chain.empty())) throw std::runtime_error("MJCF: a free joint must be the only joint of the only body under <worldbody>");
        if (root) {
            // articulations root at static bodies, so a root hinge or slide turns against a static anchor
            if (!chain.empty()) {
                Link anchor_link;
                anchor_link.name = body_name + "_anchor";
                links.push_back(anchor_link);
                parent = uint32_t(links.size() - 1u);
            }
        }
        Link rec;
        rec.name = body_name;
        rec.parent = parent;
        Frame frame;
        ApplyFrame(e, &frame);
        rec.position = frame.position;
        rec.rotation = FrameOrientation(frame, context);
        if (parent != 0xFFFFFFFFu) rec.position = rec.position + links[parent].anchor_shift;
        // every joint but the last moves a massless link on its own anchor, and the body hangs off the last one
        std::vector<uint32_t> joint_link(chain.size(), 0u);
        V3 previous;
        uint32_t walk_parent = parent;
        for (size_t k = 0u; k + 1u < chain.size(); ++k) {
            Link link;
            const char* jname = chain[k].element->Attribute("name");
            link.name = body_name + "/" + (jname != nullptr ? std::string(jname) : "joint" + std::to_string(k));
            link.parent = walk_parent;
            link.position = k == 0u ? rec.position + Rotate(rec.rotation, chain[k].anchor) : chain[k].anchor - previous;
            link.rotation = k == 0u ? rec.rotation : Quat{};
            link.mass = 1.0e-6f;
            link.inertia = {1.0e-9f, 1.0e-9f, 1.0e-9f};
            link.intermediate = true;
            links.push_back(link);
            joint_link[k] = uint32_t(links.size() - 1u);
            walk_parent = joint_link[k];
            previous = chain[k].anchor;
        }
        if (chain.size() > 1u) {
            rec.parent = walk_parent;
            rec.position = anchor - previous;
            rec.rotation = Quat{};
        } else {
            rec.position = rec.position + Rotate(rec.rotation, anchor);
        }
        const Element* inertial = e.First("inertial");
        if (inertial != nullptr) {
            QueryFloat(*inertial, "mass", &rec.mass);
            if (inertial->Attribute("pos")) rec.inertial_position = ParseV3(inertial->Attribute("pos"));
            if (inertial->Attribute("quat")) { float q[4] = {1, 0, 0, 0}; ParseFloats(inertial->Attribute("quat"), q, 4); rec.inertial_rotation = Quat{q[0], q[1], q[2], q[3]}; }
            if (inertial->Attribute("diaginertia")) rec.inertia = ParseV3(inertial->Attribute("diaginertia"));
            else if (inertial->Attribute("fullinertia")) {
                float v[6] = {1.0f, 1.0f, 1.0f, 0.0f, 0.0f, 0.0f};
                const int n = ParseFloats(inertial->Attribute("fullinertia"), v, 6);
                if (n >= 6) {
                    const double full[6] = {v[0], v[1], v[2], v[3], v[4], v[5]};
                    Diagonalize(full, &rec.inertia, &rec.inertial_rotation);
                } else if (n >= 3) rec.inertia = {v[0], v[1], v[2]};
            }
        }
        rec.inertial_position = rec.inertial_position - anchor;
        rec.anchor_shift = V3{} - anchor;
        const bool is_static = root && chain.empty() && !is_free;
        const bool from_geoms = !is_static && (context.inertia_from_geom == 1 || (context.inertia_from_geom == -1 && inertial == nullptr));
        BodyMass mass;
        ParseGeoms(e, child_class, rec.anchor_shift, &rec.geoms, from_geoms ? &mass : nullptr);
        if (from_geoms) SetBodyMass(mass, &rec);
        if (is_free) {
            rec.joint_type = 3u;
            rec.joint_name = free_joint != nullptr && free_joint->Attribute("name") != nullptr ? free_joint->Attribute("name") : body_name + "/free";
            floating_root = true;
            base_position = rec.position;
            base_rotation = rec.rotation;
            rec.position = {};
            rec.rotation = {};
        }
        links.push_back(rec);
        const uint32_t body_link = uint32_t(links.size() - 1u);
        if (!chain.empty()) joint_link.back() = body_link;
        if (is_free) joint_links[links[body_link].joint_name] = body_link;
        // the joints' own records (mjcf_importer.cpp:1167-1237)
        for (size_t k = 0u; k < chain.size(); ++k) {
            const Element& joint = *chain[k].element;
            const char* joint_class = joint.Attribute("class");
            JointDefaults j = context.Class(joint_class != nullptr ? joint_class : child_class).joint;
            ApplyJointAttributes(joint, &j);
            Link& link = links[joint_link[k]];
            link.joint_name = joint.Attribute("name") != nullptr ? joint.Attribute("name") : "unnamed_joint";
            link.joint_type = j.type == JointKind::Slide ? 1u : 0u;
            link.axis = j.axis;
            link.damping = j.damping; link.armature = j.armature; link.frictionloss = j.frictionloss;
            link.limit_margin = j.limit_margin;
            for (int i = 0; i < 7; ++i) { link.limit_reference[i] = j.limit_reference[i]; link.friction_reference[i] = j.friction_reference[i]; }
            link.stiffness = j.stiffness; link.spring_reference = j.spring_reference;
            link.actuator_force_limit = j.actuator_force_limit;
            link.lower = j.lower; link.upper = j.upper;
            link.limited = j.has_range && j.limited != 0;
            QueryFloat(joint, "nuka:initial_position", &link.initial_position);
            joint_links[link.joint_name] = joint_link[k];
        }
        e.Each("body", [&](const Element& child) { ParseBody(child, body_link, child_class); });
    }

    // JointInertiaAtRest (mjcf_importer.cpp:1381-1409): the inertia a joint sees with every joint at zero
    float JointInertiaAtRest(uint32_t joint_link) const {
        std::vector<V3> position(links.size());
        std::vector<Quat> rotation(links.size());
        for (size_t b = 0u; b < links.size(); ++b) {
            const Link& link = links[b];
            if (link.parent == 0xFFFFFFFFu) {
                position[b] = link.joint_type == 3u ? base_position : link.position;
                rotation[b] = link.joint_type == 3u ? base_rotation : link.rotation;
            } else {
                position[b] = position[link.parent] + Rotate(rotation[link.parent], link.position);
                rotation[b] = Mul(rotation[link.parent], link.rotation);
            }
        }
        const Link& joint = links[joint_link];
        const V3 anchor = position[joint_link];
        const V3 axis = Rotate(rotation[joint_link], joint.axis * (1.0f / Length(joint.axis)));
        float inertia = joint.armature;
        for (size_t b = 0u; b < links.size(); ++b) {
            uint32_t walk = uint32_t(b);
            while (walk != 0xFFFFFFFFu && walk != joint_link) walk = links[walk].parent;
            if (walk == 0xFFFFFFFFu) continue;
            const Link& body = links[b];
            if (joint.joint_type == 1u) { inertia += body.mass; continue; }
            const Quat frame_rotation = Mul(rotation[b], body.inertial_rotation);
            const V3 frame_position = position[b] + Rotate(rotation[b], body.inertial_position);
            const V3 local = Rotate(Quat{frame_rotation.w, -frame_rotation.x, -frame_rotation.y, -frame_rotation.z}, axis);
            const V3 arm = Cross(frame_position - anchor, axis);
            inertia += body.inertia.x * local.x * local.x + body.inertia.y * local.y * local.y + body.inertia.z * local.z * local.z + body.mass * Dot(arm, arm);
        }
        return inertia;
    }

    // ParseActuators (mjcf_importer.cpp:1411-1488) folded onto the driven link's drive parameters
    void ParseActuators(const Element& mujoco, uint32_t* drive_mode) {
        int kinds[3] = {0, 0, 0};   // position, velocity, motor
        std::vector<const Element*> actuators;
        mujoco.Each("actuator", [&](const Element& section) { for (const auto& a : section.children) actuators.push_back(a.get()); });
        if (actuators.empty()) return;
        for (const Element* actuator : actuators) {
            const std::string tag = actuator->name;
            const std::string name = actuator->Attribute("name") != nullptr ? actuator->Attribute("name") : "actuator";
            const GeneralDefaults& defaults = context.Class(actuator->Attribute("class")).general;
            float force_limit = defaults.force_limit, gear = defaults.gear, gain = defaults.gain;
            float bias[3] = {defaults.bias[0], defaults.bias[1], defaults.bias[2]};
            bool affine = defaults.affine;
            QueryFloat(*actuator, "gear", &gear);
            if (tag == "position") {
                float kp = 1.0f, kv = 0.0f;
                QueryFloat(*actuator, "kp", &kp); QueryFloat(*actuator, "kv", &kv);
                gain = kp; bias[0] = 0.0f; bias[1] = -kp; bias[2] = -kv;
                QueryFloat(*actuator, "dampratio", &bias[2]);
                affine = true;
            } else if (tag == "velocity") {
                float kv = 1.0f;
                QueryFloat(*actuator, "kv", &kv);
                gain = kv; bias[0] = 0.0f; bias[1] = 0.0f; bias[2] = -kv;
                affine = true;
            } else if (tag == "motor") { gain = 1.0f; affine = false; }
            else if (tag == "general") {
                ParseFloats(actuator->Attribute("gainprm"), &gain, 1);
                ParseFloats(actuator->Attribute("biasprm"), bias, 3);
                if (const char* type = actuator->Attribute("biastype")) affine = std::string(type) == "affine";
            } else throw Unsupported("MJCF: actuator '" + name + "' of type '" + tag + "' is not supported on this path");
            const char* joint_name = actuator->Attribute("joint");
            const auto found = joint_name != nullptr ? joint_links.find(joint_name) : joint_links.end();
            if (found == joint_links.end()) throw std::runtime_error("MJCF: actuator '" + name + "' needs a known joint transmission");
            Link& link = links[found->second];
            if (link.joint_type > 1u) throw std::runtime_error("MJCF: actuator '" + name + "' must drive a hinge or slide joint");
            // a positive velocity bias on a position servo is MuJoCo's damping ratio over the reflected inertia
            if (affine && gain > 0.0f && gain == -bias[1] && bias[2] > 0.0f)
                bias[2] = -bias[2] * 2.0f * std::sqrt(gain * JointInertiaAtRest(found->second) / (gear * gear));
            if (!affine || (bias[1] == 0.0f && bias[2] == 0.0f)) { ++kinds[2]; }   // motor: torque = gear gain u
            else if (bias[1] != 0.0f) {
                if (bias[1] > 0.0f || bias[0] != 0.0f) throw std::runtime_error("MJCF: actuator '" + name + "' bias is not a position servo");
                link.drive_stiffness = -gear * gear * bias[1];
                link.drive_damping = -gear * gear * bias[2];
                ++kinds[0];
            } else {
                if (bias[2] > 0.0f || bias[0] != 0.0f) throw std::runtime_error("MJCF: actuator '" + name + "' bias is not a velocity servo");
                link.drive_stiffness = -gear * gear * bias[2];   // a velocity drive's gain rides in the stiffness field
                link.drive_damping = link.drive_stiffness;
                ++kinds[1];
            }
            if (actuator->Attribute("forcerange") != nullptr) { float bounds[2] = {force_limit, force_limit}; ParseFloats(actuator->Attribute("forcerange"), bounds, 2); force_limit = bounds[1]; }
            link.drive_force_limit = force_limit;
            ++actuator_count;
        }
        // one control mode per world (nuka.h:72-74): the kind most of the file's actuators have
        *drive_mode = kinds[0] >= kinds[1] && kinds[0] >= kinds[2] && kinds[0] > 0 ? 0u : kinds[1] > kinds[2] ? 2u : 1u;
    }
};

}  // namespace

std::unique_ptr<Scene> LoadMjcf(const std::string& path, uint32_t flags) {
    const std::string text = ReadFile(path);
    std::unique_ptr<Element> mujoco = XmlReader(text).Document();
    if (mujoco->name != "mujoco") throw std::runtime_error("MJCF: missing <mujoco> root element in " + path);
    ResolveIncludes(*mujoco, Directory(path), 0);
    if (mujoco->First("worldbody") == nullptr) throw std::runtime_error("MJCF: missing <worldbody> element in " + path);

    Builder b;
    b.context.flags = flags;
    auto scene = std::make_unique<Scene>();
    scene->timestep = 0.002f;   // MuJoCo's default
    scene->integrator = 1u;     // Euler, MuJoCo's default: joint damping implicit after the solve (pipeline.cpp:264-265)
    scene->gravity[0] = 0.0f; scene->gravity[1] = 0.0f; scene->gravity[2] = -9.81f;
    if (const Element* option = mujoco->First("option")) {
        QueryFloat(*option, "timestep", &scene->timestep);
        ParseFloats(option->Attribute("gravity"), scene->gravity, 3);
        if (const char* cone = option->Attribute("cone")) {   // mjcf_importer.cpp:1724-1728
            if (std::string(cone) == "elliptic") scene->contact_cone = 1u;
            else if (std::string(cone) == "pyramidal") scene->contact_cone = 0u;
            else throw std::runtime_error("MJCF: invalid option cone");
        }
        QueryFloat(*option, "impratio", &scene->contact_impratio);
        if (const char* integrator = option->Attribute("integrator")) {
            const std::string name(integrator);
            if (name == "Euler") scene->integrator = 1u;
            else if (name == "implicit" || name == "implicitfast") scene->integrator = 2u;
            else if (name == "RK4") throw Unsupported("MJCF: the RK4 integrator is not built on this path");
            else throw std::runtime_error("MJCF: invalid option integrator");
        }
    }
    if (const Element* compiler = mujoco->First("compiler")) {
        if (const char* angle = compiler->Attribute("angle")) {
            if (std::string(angle) == "radian") b.context.angle_scale = 1.0f;
            else if (std::string(angle) != "degree") throw std::runtime_error("MJCF: invalid compiler angle");
        }
        if (const char* sequence = compiler->Attribute("eulerseq")) b.context.euler_sequence = sequence;
        if (const char* from_geom = compiler->Attribute("inertiafromgeom")) {
            const std::string mode(from_geom);
            if (mode != "auto" && mode != "true" && mode != "false") throw std::runtime_error("MJCF: invalid compiler inertiafromgeom");
            b.context.inertia_from_geom = mode == "auto" ? -1 : mode == "true" ? 1 : 0;
        }
        float groups[2] = {0.0f, 5.0f};
        ParseFloats(compiler->Attribute("inertiagrouprange"), groups, 2);
        b.context.inertia_groups[0] = int(groups[0]); b.context.inertia_groups[1] = int(groups[1]);
    }
    mujoco->Each("default", [&](const Element& e) { ParseDefaultElement(e, b.context.root, &b.context); });
    // Several bodies straight under <worldbody> (a robot beside a table, say) hang off one static link that stands for
    // the world; a single one is the articulation's root itself.  A floating body has to be that single root.
    uint32_t top_level_bodies = 0u;
    mujoco->Each("worldbody", [&](const Element& worldbody) { worldbody.Each("body", [&](const Element&) { ++top_level_bodies; }); });
    uint32_t top_parent = 0xFFFFFFFFu;
    if (top_level_bodies > 1u) {
        Link world;
        world.name = "world";
        b.links.push_back(world);
        top_parent = 0u;
    }
    // geoms placed straight in <worldbody> are static collidables; included files bring worldbody sections of their own
    mujoco->Each("worldbody", [&](const Element& worldbody) {
        b.ParseGeoms(worldbody, nullptr, V3{}, &b.world_geoms, nullptr);
        worldbody.Each("body", [&](const Element& e) { b.ParseBody(e, top_parent, nullptr); });
    });
    if (b.links.empty()) throw std::runtime_error("MJCF: no body under <worldbody> in " + path);
    mujoco->Each("contact", [&](const Element& contact) {
        contact.Each("exclude", [&](const Element& e) {
            if (e.Attribute("body1") == nullptr || e.Attribute("body2") == nullptr) throw std::runtime_error("MJCF: <exclude> needs body1 and body2");
            b.excluded_bodies.emplace_back(e.Attribute("body1"), e.Attribute("body2"));
        });
    });
    uint32_t drive_mode = 1u;
    b.ParseActuators(*mujoco, &drive_mode);
    if ((flags & kNativeJointLaw) != 0u) scene->integrator = 0u;
    FlattenScene(b, flags, drive_mode, scene.get());
    return scene;
}

// ---- flatten into the template arrays ---------------------------------------------------------------------------
void FlattenScene(const SceneParts& b, uint32_t flags, uint32_t drive_mode, Scene* scene) {
    Scene& s = *scene;
    uint32_t dropped_geoms = 0u;
    const uint32_t nl = uint32_t(b.links.size());
    s.floating_root = b.floating_root;
    s.actuator_count = b.actuator_count;
    s.base_pose = {b.base_position.x, b.base_position.y, b.base_position.z, b.base_rotation.w, b.base_rotation.x, b.base_rotation.y, b.base_rotation.z};
    bool any_friction_profile = false;
    for (uint32_t l = 0u; l < nl; ++l) {
        const Link& k = b.links[l];
        s.link_names.push_back(k.name);
        s.joint_names.push_back(k.joint_name);
        s.joint_type.push_back(k.joint_type);
        s.parent_link.push_back(k.parent);
        for (float v : {k.axis.x, k.axis.y, k.axis.z}) s.joint_axis.push_back(v);
        for (float v : {k.position.x, k.position.y, k.position.z, k.rotation.w, k.rotation.x, k.rotation.y, k.rotation.z}) s.link_local_pose.push_back(v);
        for (float v : {k.inertial_position.x, k.inertial_position.y, k.inertial_position.z, k.inertial_rotation.w, k.inertial_rotation.x,
                        k.inertial_rotation.y, k.inertial_rotation.z}) s.link_inertial_frame.push_back(v);
        s.link_mass.push_back(k.mass);
        for (float v : {k.inertia.x, k.inertia.y, k.inertia.z}) s.link_diag_inertia.push_back(v);
        s.joint_damping.push_back(k.damping); s.joint_armature.push_back(k.armature);
        s.joint_stiffness.push_back(k.stiffness); s.joint_spring_reference.push_back(k.spring_reference);
        s.joint_frictionloss.push_back(k.frictionloss);
        s.joint_law.push_back((flags & kNativeJointLaw) != 0u ? 0u : 1u);
        s.joint_limit_margin.push_back(k.limit_margin);
        for (float v : k.limit_reference) s.joint_limit_reference.push_back(v);
        for (float v : k.friction_reference) s.joint_friction_reference.push_back(v);
        s.joint_limit_lower.push_back(k.limited ? k.lower : 0.0f); s.joint_limit_upper.push_back(k.limited ? k.upper : 0.0f);
        s.joint_limit_flags.push_back(k.limited ? 3u : 0u);
        s.initial_q.push_back(k.initial_position);
        s.drive_stiffness.push_back(k.drive_stiffness); s.drive_damping.push_back(k.drive_damping);
        s.drive_force_limit.push_back(k.drive_force_limit);
        s.drive_joint_force_limit.push_back(k.actuator_force_limit);
    }
    // collidable rows: the static geoms, then per link its own body row (with its first geom) and its further geoms
    const bool plane_only = (flags & kPlaneContactsOnly) != 0u;
    auto supported = [](const Geom& g) {
        return g.kind == kShapeSphere || g.kind == kShapeCapsule || g.kind == kShapeBox || g.kind == kShapePlane || g.kind == kShapeCylinder;
    };
    auto collides = [](const Geom& g) { return g.contype != 0u || g.conaffinity != 0u; };
    // Every geom's contact terms are one profile, shared by the geoms that agree on all of them.  Under the native law
    // only an authored friction needs one (the other terms are not read).
    const bool native_law = (flags & kNativeContactLaw) != 0u;
    auto profile_of = [&](const Geom& g) -> uint32_t {
        if (native_law && !g.friction_authored) return 0xFFFFFFFFu;
        const uint32_t law = native_law ? 0u : 1u;
        for (size_t i = 0u; i < s.profile_law.size(); ++i) {
            bool same = s.profile_mu[2u * i] == g.friction && s.profile_law[i] == law && s.profile_solref[2u * i] == g.solref[0] &&
                        s.profile_solref[2u * i + 1u] == g.solref[1] && s.profile_margin[2u * i] == g.margin && s.profile_margin[2u * i + 1u] == g.gap;
            for (size_t k = 0u; k < 5u; ++k) same = same && s.profile_solimp[5u * i + k] == g.solimp[k];
            same = same && s.profile_priority[i] == g.priority && s.profile_solmix[i] == g.solmix && s.profile_condim[i] == g.condim;
            if (same) return uint32_t(i);
        }
        s.profile_mu.push_back(g.friction); s.profile_mu.push_back(g.friction);
        s.profile_law.push_back(law);
        s.profile_solref.push_back(g.solref[0]); s.profile_solref.push_back(g.solref[1]);
        for (float v : g.solimp) s.profile_solimp.push_back(v);
        s.profile_margin.push_back(g.margin); s.profile_margin.push_back(g.gap);
        s.profile_priority.push_back(g.priority); s.profile_solmix.push_back(g.solmix); s.profile_condim.push_back(g.condim);
        any_friction_profile = true;
        return uint32_t(s.profile_law.size() - 1u);
    };
    auto add_row = [&](uint32_t role, uint32_t link, const Geom* g, int32_t group_override) {
        s.body_role.push_back(role); s.body_link.push_back(link);
        const Geom none{};
        const Geom& geom = g != nullptr ? *g : none;
        for (float v : {geom.position.x, geom.position.y, geom.position.z, geom.rotation.w, geom.rotation.x, geom.rotation.y, geom.rotation.z}) s.body_local.push_back(v);
        s.shape_kind.push_back(g != nullptr ? geom.kind : 0xFFFFFFFFu);
        for (float v : geom.params) s.shape_params.push_back(v);
        s.shape_contype.push_back(g != nullptr ? geom.contype : 0u);
        s.shape_conaffinity.push_back(g != nullptr ? geom.conaffinity : 0u);
        s.shape_group.push_back(uint32_t(g != nullptr ? (group_override != 0 ? group_override : geom.group) : 0));
        s.shape_profile.push_back(g != nullptr ? profile_of(geom) : 0xFFFFFFFFu);
    };
    auto keep = [&](const Geom& g) {
        if (!collides(g)) return false;   // visual geometry has no collidable row
        if (supported(g)) return true;
        if (!plane_only) return true;     // kept: the cook refuses the shape kind it has no manifold for
        ++dropped_geoms;
        return false;
    };
    if ((flags & kGroundPlane) != 0u) {
        Geom ground;
        ground.kind = kShapePlane;
        add_row(0u, 0xFFFFFFFFu, &ground, 0);
    }
    for (const Geom& g : b.world_geoms) if (keep(g)) add_row(0u, 0xFFFFFFFFu, &g, 0);
    std::vector<std::vector<uint32_t>> link_rows(nl);
    for (uint32_t l = 0u; l < nl; ++l) {
        std::vector<const Geom*> kept;
        for (const Geom& g : b.links[l].geoms) if (keep(g)) kept.push_back(&g);
        // with plane contacts only, the robot's geoms share one negative group: they meet the ground, not each other
        const int32_t group = plane_only ? -1 : 0;
        link_rows[l].push_back(uint32_t(s.body_role.size()));
        add_row(1u, l, kept.empty() ? nullptr : kept[0], group);
        for (size_t i = 1u; i < kept.size(); ++i) { link_rows[l].push_back(uint32_t(s.body_role.size())); add_row(2u, l, kept[i], group); }
    }
    // Excluded pairs (src/scene/cooker.cpp:470-538): bodies welded together by fixed joints form a cluster; no two
    // bodies of a cluster collide, nor a cluster with the cluster of its parent body, nor the bodies an <exclude>
    // names.  The massless links that carry the earlier joints of a several-joint body stand for no body of the file:
    // the parent of such a body is the body above them.
    {
        auto weld = [&](uint32_t link) {
            while (b.links[link].parent != 0xFFFFFFFFu && (b.links[link].joint_type == 2u || b.links[link].intermediate)) link = b.links[link].parent;
            return link;
        };
        std::vector<std::vector<uint32_t>> clusters(nl);
        for (uint32_t l = 0u; l < nl; ++l) clusters[weld(l)].push_back(l);
        auto exclude_links = [&](uint32_t la, uint32_t lb) {
            if (la == lb) return;   // the rows of one link are excluded by the cook
            for (uint32_t ra : link_rows[la]) for (uint32_t rb : link_rows[lb]) {
                if (s.shape_kind[ra] == 0xFFFFFFFFu || s.shape_kind[rb] == 0xFFFFFFFFu) continue;   // a row without a shape meets nothing
                s.excluded_pairs.push_back(ra); s.excluded_pairs.push_back(rb);
            }
        };
        for (uint32_t root = 0u; root < nl; ++root) {
            const auto& members = clusters[root];
            for (size_t i = 0u; i < members.size(); ++i) for (size_t k = i + 1u; k < members.size(); ++k) exclude_links(members[i], members[k]);
            if (members.empty() || b.links[root].parent == 0xFFFFFFFFu) continue;
            for (uint32_t other : clusters[weld(b.links[root].parent)]) for (uint32_t member : members) exclude_links(member, other);
        }
        for (const auto& names : b.excluded_bodies) {
            uint32_t found[2] = {0xFFFFFFFFu, 0xFFFFFFFFu};
            for (uint32_t l = 0u; l < nl; ++l) for (int k = 0; k < 2; ++k) if (!b.links[l].intermediate && b.links[l].name == (k == 0 ? names.first : names.second)) found[k] = l;
            if (found[0] == 0xFFFFFFFFu || found[1] == 0xFFFFFFFFu) continue;   // an unknown body name is skipped, as the reference's importer does
            exclude_links(found[0], found[1]);
        }
    }
    (void)any_friction_profile;
    s.dropped_geom_count = dropped_geoms;
    s.drive_mode = drive_mode;
    s.Bind();
}

void Scene::Bind() {
    desc = {};
    desc.struct_size = sizeof(desc);
    desc.link_count = uint32_t(joint_type.size());
    desc.body_count = uint32_t(body_role.size());
    desc.profile_count = uint32_t(profile_mu.size() / 2u);
    desc.joint_type = joint_type.data(); desc.parent_link = parent_link.data(); desc.joint_axis = joint_axis.data();
    desc.link_local_pose = link_local_pose.data(); desc.link_inertial_frame = link_inertial_frame.data();
    desc.link_mass = link_mass.data(); desc.link_diag_inertia = link_diag_inertia.data();
    desc.joint_damping = joint_damping.data(); desc.joint_armature = joint_armature.data();
    desc.joint_stiffness = joint_stiffness.data(); desc.joint_spring_reference = joint_spring_reference.data();
    desc.body_role = body_role.data(); desc.body_link = body_link.data(); desc.body_local = body_local.data();
    desc.shape_kind = shape_kind.data(); desc.shape_params = shape_params.data(); desc.shape_contype = shape_contype.data();
    desc.shape_conaffinity = shape_conaffinity.data(); desc.shape_group = shape_group.data(); desc.shape_profile = shape_profile.data();
    desc.profile_mu = profile_mu.data();
    desc.joint_limit_lower = joint_limit_lower.data(); desc.joint_limit_upper = joint_limit_upper.data();
    desc.joint_limit_flags = joint_limit_flags.data(); desc.joint_frictionloss = joint_frictionloss.data();
    desc.drive_mode = drive_mode;
    desc.drive_rows = 1u;   // the reference always cooks one drive row per link (src/nk/pipeline/world.cpp:61)
    desc.excluded_pairs = excluded_pairs.data();
    desc.excluded_pair_count = uint32_t(excluded_pairs.size() / 2u);
    if (!profile_law.empty()) {   // a loader that authors no law leaves every profile native
        desc.profile_law = profile_law.data(); desc.profile_solref = profile_solref.data();
        desc.profile_solimp = profile_solimp.data(); desc.profile_margin = profile_margin.data();
        desc.profile_priority = profile_priority.data(); desc.profile_solmix = profile_solmix.data(); desc.profile_condim = profile_condim.data();
    }
    desc.contact_cone = contact_cone;
    desc.contact_impratio = contact_impratio;
    if (!joint_law.empty()) {
        desc.joint_law = joint_law.data(); desc.joint_limit_margin = joint_limit_margin.data();
        desc.joint_limit_reference = joint_limit_reference.data(); desc.joint_friction_reference = joint_friction_reference.data();
    }
    desc.integrator = integrator;
    // A lone body on a free joint is no articulation in the reference: CookArticulations passes over a root that no joint
    // hangs a child on (src/runtime/articulation/articulation_cooker.cpp:148-151), and the body stays a free rigid body of
    // the rigid-body ops.  It has no joint for a joint law or the joints' integrator to act on.
    if (desc.link_count == 1u && floating_root) {
        desc.free_body = 1u;
        desc.drive_rows = 0u;
        desc.integrator = 0u;
        desc.joint_law = nullptr;
    }
}

}  // namespace scene_file
}  // namespace nkh
