// A collidable row's world pose from its link's (sync_body_pose.cu:23-83): link-owned rows only, static rows keep their
// cooked pose.  Shared by SyncLinkBodyPose and by the kernel that runs the ops after the solve as one launch.
#pragma once

#include "nk_device_math.h"
#include "nk_types.h"

namespace nkh {

// `link_pose` holds the environment's link poses (its slice of the field, or a copy in LDS)
__device__ __forceinline__ void sync_body_pose(const ModelView& m, const DataView& d, uint32_t env, uint32_t b, const float* link_pose) {
    const size_t gid = size_t{env} * m.bodies_per_env + b;
    const uint32_t own = m.body_to_link[b], proxy = m.body_collidable_link[b];
    if (own != kInvalid) {
        if (m.link_body[own] != b) return;
        Xf world = load_xf(link_pose + own * 7u);
        if (m.link_geom_kind[own] != 0u) world = compose_collidable(world, load_xf(m.link_geom_local + 7u * own));
        store_xf(d.body_pose + gid * 7u, world);
    } else if (proxy != kInvalid && proxy < m.links_per_env) {
        store_xf(d.body_pose + gid * 7u,
                 compose_collidable(load_xf(link_pose + proxy * 7u),
                                    load_xf(m.body_collidable_local + 7u * b)));
    }
}

}  // namespace nkh
