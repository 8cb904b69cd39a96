"""Templates of a free rigid body for the tests: a box (the body's own collidable row) over an optional static plane."""
import numpy as np

from conftest import nk

abi = nk.abi


def box_template(half=(0.2, 0.2, 0.1), mass=1.0, diag=(0.01, 0.01, 0.01), com=(0.0, 0.0, 0.0), mu=0.7, plane=True):
    t = abi.Template()
    t.free_body = True
    t.add_link(abi.JOINT_FLOATING, None, mass=mass, diag_inertia=diag, com=com)
    profile = t.add_profile(mu)
    if plane:
        t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, kind=abi.SHAPE_BOX, params=(half[0], half[1], half[2], 0.0), contype=1, conaffinity=2,
               profile=profile)
    t.max_contacts_per_env = 1 if plane else 0
    return t


def rotation_matrix(q):
    """Rotation matrix of a quaternion w x y z, in float64."""
    w, x, y, z = np.asarray(q, np.float64) / np.linalg.norm(q)
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def body_field(template, values):
    """A per-body field of a free-body world from the free body's values [E][k]: the body's own row (the last one of
    box_template) holds them, the other rows zeros."""
    values = np.asarray(values, np.float32)
    nb = len(template.bodies)
    out = np.zeros((values.shape[0], nb) + values.shape[1:], np.float32)
    out[:, nb - 1] = values
    return out


def of_body(template, field, E):
    """The free body's values of a per-body field as downloaded."""
    nb = len(template.bodies)
    return np.asarray(field).reshape(E, nb, -1)[:, nb - 1]
