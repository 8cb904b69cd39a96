"""Independent float64 rigid-tree model used to pin the oracle's dynamics: rotation matrices and finite
differences of world poses only - no spatial algebra, no recursion shared with the oracle.

Generalised velocity: the root's body-frame twist [omega; v] for a floating root, then one rate per joint."""
import numpy as np


def rot(q):
    w, x, y, z = np.asarray(q, np.float64) / np.linalg.norm(q)
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def axis_angle(axis, angle):
    a = np.asarray(axis, np.float64)
    a = a / np.linalg.norm(a)
    K = np.array([[0, -a[2], a[1]], [a[2], 0, -a[0]], [-a[1], a[0], 0]])
    return np.eye(3) + np.sin(angle) * K + (1 - np.cos(angle)) * K @ K


def expm_so3(w):
    w = np.asarray(w, np.float64)
    angle = np.linalg.norm(w)
    return np.eye(3) if angle < 1e-300 else axis_angle(w / angle, angle)


class Model:
    REVOLUTE, PRISMATIC, FIXED, FLOATING = 0, 1, 3, 4

    def __init__(self, template, abi):
        self.links = template.links
        self.nl = len(self.links)
        self.REVOLUTE, self.PRISMATIC = abi.JOINT_REVOLUTE, abi.JOINT_PRISMATIC
        self.FIXED, self.FLOATING = abi.JOINT_FIXED, abi.JOINT_FLOATING
        self.invalid = abi.INVALID
        self.floating = self.links[0]["joint_type"] == self.FLOATING
        self.scalar_links = [i for i, l in enumerate(self.links) if l["joint_type"] in (self.REVOLUTE, self.PRISMATIC)]
        self.dof = (6 if self.floating else 0) + len(self.scalar_links)

    def fk(self, q, base_R=None, base_p=None):
        """World rotation and origin of every link."""
        R, p = [None] * self.nl, [None] * self.nl
        for i, l in enumerate(self.links):   # parents precede children in every template used here
            local = np.asarray(l["local"], np.float64)
            lp, lR = local[:3] + np.asarray(l["parent_offset"], np.float64), rot(local[3:])
            if l["joint_type"] == self.REVOLUTE:
                lR = lR @ axis_angle(l["axis"], q[i])
            elif l["joint_type"] == self.PRISMATIC:
                a = np.asarray(l["axis"], np.float64)
                lp = lp + lR @ (a / np.linalg.norm(a) * q[i])
            if l["parent"] == self.invalid:
                R[i], p[i] = (base_R, base_p) if l["joint_type"] == self.FLOATING else (lR, lp)
            else:
                R[i], p[i] = R[l["parent"]] @ lR, p[l["parent"]] + R[l["parent"]] @ lp
        return R, p

    def displaced(self, q, base_R, base_p, velocity, h):
        """Configuration reached by following the generalised velocity for time h."""
        q2 = np.array(q, np.float64)
        velocity = np.asarray(velocity, np.float64)
        at = 0
        if self.floating:
            base_p = base_p + base_R @ velocity[3:6] * h
            base_R = base_R @ expm_so3(velocity[0:3] * h)
            at = 6
        for k, link in enumerate(self.scalar_links):
            q2[link] += velocity[at + k] * h
        return q2, base_R, base_p

    def link_motion(self, q, base_R, base_p, velocity, h=1e-6):
        """World angular velocity and world COM velocity of every link, by central differences of the poses."""
        qa, Ra, pa = self.displaced(q, base_R, base_p, velocity, +h)
        qb, Rb, pb = self.displaced(q, base_R, base_p, velocity, -h)
        R1, p1 = self.fk(qa, Ra, pa)
        R0, p0 = self.fk(qb, Rb, pb)
        out = []
        for i, l in enumerate(self.links):
            com = np.asarray(l["inertial"][:3], np.float64)
            W = (R1[i] @ R0[i].T - R0[i] @ R1[i].T) / (4 * h)
            omega = np.array([W[2, 1], W[0, 2], W[1, 0]])
            vc = ((p1[i] + R1[i] @ com) - (p0[i] + R0[i] @ com)) / (2 * h)
            out.append((omega, vc))
        return out

    def world_inertia(self, R, i):
        l = self.links[i]
        Ri = R[i] @ rot(l["inertial"][3:])
        return Ri @ np.diag(np.asarray(l["diag"], np.float64)) @ Ri.T

    def mass_matrix(self, q, base_R=None, base_p=None):
        """M[i][j] = sum over links of m v_i . v_j + w_i^T I w_j for the unit generalised velocities, plus armature."""
        R, _ = self.fk(q, base_R, base_p)
        n = self.dof
        motions = [self.link_motion(q, base_R, base_p, np.eye(n)[j]) for j in range(n)]
        M = np.zeros((n, n))
        for i in range(self.nl):
            Iw, m = self.world_inertia(R, i), self.links[i]["mass"]
            W = np.array([motions[j][i][0] for j in range(n)])
            V = np.array([motions[j][i][1] for j in range(n)])
            M += m * V @ V.T + W @ Iw @ W.T
        at = 6 if self.floating else 0
        for k, link in enumerate(self.scalar_links):
            M[at + k, at + k] += self.links[link]["armature"]
        return M

    def kinetic_energy(self, q, base_R, base_p, velocity):
        R, _ = self.fk(q, base_R, base_p)
        total = 0.0
        for i, (omega, vc) in enumerate(self.link_motion(q, base_R, base_p, velocity)):
            total += 0.5 * self.links[i]["mass"] * vc @ vc + 0.5 * omega @ self.world_inertia(R, i) @ omega
        return total

    def potential(self, q, base_R, base_p, gravity):
        R, p = self.fk(q, base_R, base_p)
        return -sum(l["mass"] * np.asarray(gravity, np.float64) @ (p[i] + R[i] @ np.asarray(l["inertial"][:3], np.float64))
                    for i, l in enumerate(self.links))

    def momentum(self, q, base_R, base_p, velocity):
        """World linear momentum and angular momentum about the world origin."""
        R, p = self.fk(q, base_R, base_p)
        P, L = np.zeros(3), np.zeros(3)
        for i, (omega, vc) in enumerate(self.link_motion(q, base_R, base_p, velocity)):
            m = self.links[i]["mass"]
            c = p[i] + R[i] @ np.asarray(self.links[i]["inertial"][:3], np.float64)
            P += m * vc
            L += np.cross(c, m * vc) + self.world_inertia(R, i) @ omega
        return P, L

    def lagrange_bias(self, q, qdot, gravity, h=1e-5):
        """Fixed-base Euler-Lagrange bias c_i = sum_jk (dM_ij/dq_k - 0.5 dM_jk/dq_i) qd_j qd_k + dV/dq_i, with
        derivatives by central differences of the float64 mass matrix and potential."""
        assert not self.floating
        n = self.dof
        dM = np.zeros((n, n, n))
        dV = np.zeros(n)
        for k, link in enumerate(self.scalar_links):
            qa, qb = np.array(q, np.float64), np.array(q, np.float64)
            qa[link] += h
            qb[link] -= h
            dM[:, :, k] = (self.mass_matrix(qa) - self.mass_matrix(qb)) / (2 * h)
            dV[k] = (self.potential(qa, None, None, gravity) - self.potential(qb, None, None, gravity)) / (2 * h)
        v = np.array([qdot[l] for l in self.scalar_links], np.float64)
        return np.einsum("ijk,j,k->i", dM, v, v) - 0.5 * np.einsum("jki,j,k->i", dM, v, v) + dV
