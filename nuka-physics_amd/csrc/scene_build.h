// Shared pieces of the robot-description loaders (MJCF, URDF): a small XML reader, the vector and quaternion helpers,
// the link and geom records a file is read into, and the flattening of those records into the template arrays with
// the cook-time pair exclusions.  Internal to the loaders; host code only.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "scene_loader.h"

namespace nkh {
namespace scene_file {

// ---- a small XML reader: elements, attributes, comments, declarations ---------------------------------------
struct Element {
    std::string name;
    std::vector<std::pair<std::string, std::string>> attributes;
    std::vector<std::unique_ptr<Element>> children;
    const char* Attribute(const char* key) const {
        for (const auto& a : attributes) if (a.first == key) return a.second.c_str();
        return nullptr;
    }
    const Element* First(const char* tag) const {
        for (const auto& c : children) if (c->name == tag) return c.get();
        return nullptr;
    }
    template <class F> void Each(const char* tag, F&& f) const {
        for (const auto& c : children) if (c->name == tag) f(*c);
    }
};

class XmlReader {
public:
    explicit XmlReader(const std::string& text) : s_(text) {}
    std::unique_ptr<Element> Document() {
        std::unique_ptr<Element> root;
        for (;;) {
            SkipMisc();
            if (at_ >= s_.size()) break;
            if (s_[at_] != '<') Fail("text outside the root element");
            if (root) Fail("more than one root element");
            root = ReadElement();
        }
        if (!root) Fail("no root element");
        return root;
    }

private:
    [[noreturn]] void Fail(const std::string& what) const {
        size_t line = 1u;
        for (size_t i = 0u; i < at_ && i < s_.size(); ++i) if (s_[i] == '\n') ++line;
        throw std::runtime_error("XML: " + what + " (line " + std::to_string(line) + ")");
    }
    bool StartsWith(const char* token) const { return s_.compare(at_, std::strlen(token), token) == 0; }
    void SkipSpace() { while (at_ < s_.size() && std::isspace(static_cast<unsigned char>(s_[at_]))) ++at_; }
    void SkipPast(const char* token) {
        const size_t found = s_.find(token, at_);
        if (found == std::string::npos) Fail(std::string("unterminated construct, expected ") + token);
        at_ = found + std::strlen(token);
    }
    void SkipMisc() {   // whitespace, comments, processing instructions, doctype
        for (;;) {
            SkipSpace();
            if (StartsWith("<!--")) SkipPast("-->");
            else if (StartsWith("<?")) SkipPast("?>");
            else if (StartsWith("<!")) SkipPast(">");
            else return;
        }
    }
    static bool NameChar(char c) { return std::isalnum(static_cast<unsigned char>(c)) || c == '_' || c == '-' || c == ':' || c == '.'; }
    std::string ReadName() {
        const size_t start = at_;
        while (at_ < s_.size() && NameChar(s_[at_])) ++at_;
        if (at_ == start) Fail("expected a name");
        return s_.substr(start, at_ - start);
    }
    static std::string Decode(const std::string& raw) {
        std::string out;
        for (size_t i = 0u; i < raw.size(); ++i) {
            if (raw[i] != '&') { out += raw[i]; continue; }
            static const std::pair<const char*, char> kEntities[] = {{"&lt;", '<'}, {"&gt;", '>'}, {"&amp;", '&'}, {"&quot;", '"'}, {"&apos;", '\''}};
            bool matched = false;
            for (const auto& e : kEntities)
                if (raw.compare(i, std::strlen(e.first), e.first) == 0) { out += e.second; i += std::strlen(e.first) - 1u; matched = true; break; }
            if (!matched) out += raw[i];
        }
        return out;
    }
    std::unique_ptr<Element> ReadElement() {
        ++at_;   // '<'
        auto element = std::make_unique<Element>();
        element->name = ReadName();
        for (;;) {
            SkipSpace();
            if (at_ >= s_.size()) Fail("unterminated tag");
            if (StartsWith("/>")) { at_ += 2u; return element; }
            if (s_[at_] == '>') { ++at_; break; }
            const std::string key = ReadName();
            SkipSpace();
            if (at_ >= s_.size() || s_[at_] != '=') Fail("expected '=' after attribute " + key);
            ++at_;
            SkipSpace();
            if (at_ >= s_.size() || (s_[at_] != '"' && s_[at_] != '\'')) Fail("expected a quoted value for " + key);
            const char quote = s_[at_++];
            const size_t end = s_.find(quote, at_);
            if (end == std::string::npos) Fail("unterminated attribute value");
            element->attributes.emplace_back(key, Decode(s_.substr(at_, end - at_)));
            at_ = end + 1u;
        }
        for (;;) {   // content: child elements; character data is ignored (MJCF carries none)
            const size_t open = s_.find('<', at_);
            if (open == std::string::npos) Fail("missing closing tag of " + element->name);
            at_ = open;
            if (StartsWith("<!--")) { SkipPast("-->"); continue; }
            if (StartsWith("<?")) { SkipPast("?>"); continue; }
            if (StartsWith("<![CDATA[")) { SkipPast("]]>"); continue; }
            if (StartsWith("</")) {
                at_ += 2u;
                if (ReadName() != element->name) Fail("mismatched closing tag of " + element->name);
                SkipSpace();
                if (at_ >= s_.size() || s_[at_] != '>') Fail("malformed closing tag");
                ++at_;
                return element;
            }
            element->children.push_back(ReadElement());
        }
    }
    const std::string& s_;
    size_t at_ = 0u;
};

inline std::string ReadFile(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) throw std::runtime_error("MJCF: failed to load file: " + path);
    std::ostringstream buffer;
    buffer << in.rdbuf();
    return buffer.str();
}

inline std::string Directory(const std::string& path) {
    const size_t slash = path.find_last_of('/');
    return slash == std::string::npos ? std::string(".") : path.substr(0u, slash);
}

// <include file="..."/> splices the included file's top-level sections in place.
inline void ResolveIncludes(Element& element, const std::string& directory, int depth) {
    if (depth > 16) throw std::runtime_error("MJCF: include nesting too deep");
    std::vector<std::unique_ptr<Element>> out;
    for (auto& child : element.children) {
        if (child->name != "include") {
            ResolveIncludes(*child, directory, depth);
            out.push_back(std::move(child));
            continue;
        }
        const char* file = child->Attribute("file");
        if (file == nullptr) throw std::runtime_error("MJCF: include without file");
        const std::string path = file[0] == '/' ? std::string(file) : directory + "/" + file;
        const std::string text = ReadFile(path);
        auto included = XmlReader(text).Document();
        ResolveIncludes(*included, Directory(path), depth + 1);
        for (auto& grandchild : included->children) out.push_back(std::move(grandchild));
    }
    element.children = std::move(out);
}

// ---- small math ------------------------------------------------------------------------------------------------
struct V3 { float x = 0.0f, y = 0.0f, z = 0.0f; };
struct Quat { float w = 1.0f, x = 0.0f, y = 0.0f, z = 0.0f; };
inline V3 operator+(V3 a, V3 b) { return {a.x + b.x, a.y + b.y, a.z + b.z}; }
inline V3 operator-(V3 a, V3 b) { return {a.x - b.x, a.y - b.y, a.z - b.z}; }
inline V3 operator*(V3 a, float s) { return {a.x * s, a.y * s, a.z * s}; }
inline float Dot(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
inline V3 Cross(V3 a, V3 b) { return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x}; }
inline float Length(V3 a) { return std::sqrt(Dot(a, a)); }
inline Quat Mul(Quat a, Quat b) {
    return {a.w * b.w - a.x * b.x - a.y * b.y - a.z * b.z, a.w * b.x + a.x * b.w + a.y * b.z - a.z * b.y,
            a.w * b.y - a.x * b.z + a.y * b.w + a.z * b.x, a.w * b.z + a.x * b.y - a.y * b.x + a.z * b.w};
}
inline Quat Normalized(Quat q) {
    const float n = std::sqrt(q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z);
    if (!(n > 0.0f)) throw std::runtime_error("MJCF: zero quaternion");
    return {q.w / n, q.x / n, q.y / n, q.z / n};
}
inline V3 Rotate(Quat q, V3 v) {
    const V3 u{q.x, q.y, q.z};
    const V3 t = Cross(u, v) * 2.0f;
    return v + t * q.w + Cross(u, t);
}
inline Quat AxisAngle(V3 axis, float angle) {
    const float h = 0.5f * angle, s = std::sin(h);
    return {std::cos(h), axis.x * s, axis.y * s, axis.z * s};
}
inline V3 Unit(V3 v) {
    const float length = Length(v);
    if (!(length > 0.0f) || !std::isfinite(length)) throw std::runtime_error("MJCF: invalid orientation axis");
    return v * (1.0f / length);
}
inline Quat ZRotation(V3 direction) {   // the shortest rotation taking +z onto `direction` (mjcf_importer.cpp:446-450)
    const V3 z = Unit(direction);
    return z.z <= -1.0f ? Quat{0.0f, 1.0f, 0.0f, 0.0f} : Normalized(Quat{1.0f + z.z, -z.y, z.x, 0.0f});
}
inline Quat FromMatrix(const double m[3][3]) {
    const double trace = m[0][0] + m[1][1] + m[2][2];
    double w, x, y, z;
    if (trace > 0.0) { const double s = std::sqrt(trace + 1.0) * 2.0; w = 0.25 * s; x = (m[2][1] - m[1][2]) / s; y = (m[0][2] - m[2][0]) / s; z = (m[1][0] - m[0][1]) / s; }
    else if (m[0][0] > m[1][1] && m[0][0] > m[2][2]) { const double s = std::sqrt(1.0 + m[0][0] - m[1][1] - m[2][2]) * 2.0; w = (m[2][1] - m[1][2]) / s; x = 0.25 * s; y = (m[0][1] + m[1][0]) / s; z = (m[0][2] + m[2][0]) / s; }
    else if (m[1][1] > m[2][2]) { const double s = std::sqrt(1.0 + m[1][1] - m[0][0] - m[2][2]) * 2.0; w = (m[0][2] - m[2][0]) / s; x = (m[0][1] + m[1][0]) / s; y = 0.25 * s; z = (m[1][2] + m[2][1]) / s; }
    else { const double s = std::sqrt(1.0 + m[2][2] - m[0][0] - m[1][1]) * 2.0; w = (m[1][0] - m[0][1]) / s; x = (m[0][2] + m[2][0]) / s; y = (m[1][2] + m[2][1]) / s; z = 0.25 * s; }
    return Normalized(Quat{float(w), float(x), float(y), float(z)});
}

// Principal moments and the rotation onto them by cyclic Jacobi sweeps (import/principal_inertia.hpp); full =
// {xx, yy, zz, xy, xz, yz}.
inline void Diagonalize(const double full[6], V3* principal, Quat* rotation) {
    double a[3][3] = {{full[0], full[3], full[4]}, {full[3], full[1], full[5]}, {full[4], full[5], full[2]}};
    double v[3][3] = {{1, 0, 0}, {0, 1, 0}, {0, 0, 1}};
    for (int sweep = 0; sweep < 64; ++sweep) {
        const double off = std::fabs(a[0][1]) + std::fabs(a[0][2]) + std::fabs(a[1][2]);
        if (off < 1e-15 * (std::fabs(a[0][0]) + std::fabs(a[1][1]) + std::fabs(a[2][2]) + 1e-300)) break;
        for (int p = 0; p < 3; ++p)
            for (int q = p + 1; q < 3; ++q) {
                if (a[p][q] == 0.0) continue;
                const double theta = (a[q][q] - a[p][p]) / (2.0 * a[p][q]);
                const double t = (theta >= 0.0 ? 1.0 : -1.0) / (std::fabs(theta) + std::sqrt(theta * theta + 1.0));
                const double c = 1.0 / std::sqrt(t * t + 1.0), s = t * c;
                for (int k = 0; k < 3; ++k) { const double kp = a[k][p], kq = a[k][q]; a[k][p] = c * kp - s * kq; a[k][q] = s * kp + c * kq; }
                for (int k = 0; k < 3; ++k) { const double pk = a[p][k], qk = a[q][k]; a[p][k] = c * pk - s * qk; a[q][k] = s * pk + c * qk; }
                for (int k = 0; k < 3; ++k) { const double kp = v[k][p], kq = v[k][q]; v[k][p] = c * kp - s * kq; v[k][q] = s * kp + c * kq; }
            }
    }
    // a right-handed frame: flip the third axis when the eigenvector matrix is a reflection
    const double det = v[0][0] * (v[1][1] * v[2][2] - v[1][2] * v[2][1]) - v[0][1] * (v[1][0] * v[2][2] - v[1][2] * v[2][0]) +
                       v[0][2] * (v[1][0] * v[2][1] - v[1][1] * v[2][0]);
    if (det < 0.0) for (int k = 0; k < 3; ++k) v[k][2] = -v[k][2];
    *principal = {float(a[0][0]), float(a[1][1]), float(a[2][2])};
    *rotation = FromMatrix(v);
}

inline int ParseFloats(const char* text, float* out, int count) {   // entries the text does not provide keep their value
    if (text == nullptr || count <= 0) return 0;
    std::istringstream ss(text);
    int n = 0;
    for (; n < count; ++n) {
        float value;
        if (!(ss >> value)) break;
        out[n] = value;
    }
    return n;
}
inline V3 ParseV3(const char* text) { float v[3] = {0, 0, 0}; ParseFloats(text, v, 3); return {v[0], v[1], v[2]}; }
inline bool QueryFloat(const Element& e, const char* key, float* out) {
    const char* text = e.Attribute(key);
    if (text == nullptr) return false;
    char* end = nullptr;
    const float value = std::strtof(text, &end);
    if (end == text) return false;
    *out = value;
    return true;
}
inline bool QueryInt(const Element& e, const char* key, long* out) {
    const char* text = e.Attribute(key);
    if (text == nullptr) return false;
    char* end = nullptr;
    const long value = std::strtol(text, &end, 10);
    if (end == text) return false;
    *out = value;
    return true;
}
inline int ParseLimited(const char* text, int fallback) {   // -1 auto, 0 false, 1 true
    if (text == nullptr) return fallback;
    const std::string value(text);
    if (value == "true" || value == "1") return 1;
    if (value == "false" || value == "0") return 0;
    return -1;
}

struct BodyMass { double mass = 0.0, first[3] = {}, inertia[3][3] = {}; };
struct Geom {
    uint32_t kind = 0u;   // collision/shape_kind.hpp:9-18; 0xFFFFFFFF for a shape this library does not know
    float params[4] = {0, 0, 0, 0};
    V3 position;
    Quat rotation;
    uint32_t contype = 1u, conaffinity = 1u;
    int32_t group = 0;
    float friction = 1.0f;
    bool friction_authored = false;
    // the MuJoCo contact law's terms of the geom (src/import/mjcf_importer.cpp:162-165, 1009-1015)
    float solref[2] = {0.02f, 1.0f};
    float solimp[5] = {0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
    float margin = 0.0f, gap = 0.0f, solmix = 1.0f;
    int32_t priority = 0;
    uint32_t condim = 3u;
};
struct Link {
    std::string name, joint_name;
    uint32_t parent = 0xFFFFFFFFu;
    uint8_t joint_type = 2u;   // phi/articulation_contract.hpp:8-16
    V3 axis{0.0f, 0.0f, 1.0f};
    V3 position;   // parent link frame to this link frame at q = 0
    Quat rotation;
    float mass = 0.0f;
    V3 inertia, inertial_position;
    Quat inertial_rotation;
    float damping = 0.0f, armature = 0.0f, frictionloss = 0.0f, stiffness = 0.0f, spring_reference = 0.0f;
    float lower = 0.0f, upper = 0.0f;
    bool limited = false;
    // a MuJoCo-sourced joint's limit margin and the solref[2], solimp[5] of its limit and dry-friction rows
    float limit_margin = 0.0f;
    float limit_reference[7] = {0.02f, 1.0f, 0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
    float friction_reference[7] = {0.02f, 1.0f, 0.9f, 0.95f, 0.001f, 0.5f, 2.0f};
    float initial_position = 0.0f;
    float actuator_force_limit = 0.0f;
    V3 anchor_shift;   // what the body authors in its own frame moves by this: minus its joint anchor
    std::vector<Geom> geoms;
    float drive_stiffness = 0.0f, drive_damping = 0.0f, drive_force_limit = 0.0f;
    bool intermediate = false;   // a massless link that carries one of several joints of a body
};

constexpr uint32_t kShapeSphere = 0u, kShapeCapsule = 1u, kShapeBox = 2u, kShapePlane = 3u, kShapeCylinder = 7u, kShapeUnknown = 0xFFFFFFFEu;
// What a description file is read into before it is flattened.
struct SceneParts {
    std::vector<Link> links;         // parents before children
    std::vector<Geom> world_geoms;   // static collidables, world frame
    std::vector<std::pair<std::string, std::string>> excluded_bodies;   // body (link) names that never collide
    bool floating_root = false;
    V3 base_position;
    Quat base_rotation;
    uint32_t actuator_count = 0u;
};

// Fills the template arrays of `scene` from the links and geoms, with the excluded pairs of the reference's cook-time
// policy, and binds its descriptor.
void FlattenScene(const SceneParts& parts, uint32_t flags, uint32_t drive_mode, Scene* scene);

}  // namespace scene_file
}  // namespace nkh
