// Host side shared by every multi-tensor entry point: device resolution, plan lookup and the
// launch geometry of a plan's segments.
#pragma once

#include "gm_plan.hpp"
#include "gm_rules.hpp"

#include <mutex>

namespace gm {

// Launch shape when the caller has not fixed it (gm_set_tuning, gm_set_workgroup_lanes), measured on
// MI355X over lists of 25M, 125M and 1B parameters.  Rules with five streams (SGD-momentum, AdaGrad,
// plain RMSProp: 3 reads + 2 writes): 8-byte lanes in 128-lane workgroups, 81-83 % of peak, against
// 76-82 % in 256-lane workgroups and 71-77 % with 4-byte lanes.  Seven streams and more (Adam, NAdam,
// AdaDelta, the mixed-precision step): 4-byte lanes in 256-lane workgroups, 81-82 %, against 79-80 %
// in 128-lane workgroups and 76-79 % with 8-byte lanes.
int auto_vec(int streams);
int auto_block(int streams);

StepParams zero_params();

struct Launch {
    Context *ctx;
    MultiTensorPlan *plan;
};

// Resolves the device, takes the context lock, finds the plan.  Returns the
// entry point's code on failure (hip_error_code for HIP trouble) or 0; when 0
// and out.plan->num_chunks == 0 there is nothing to launch.
int prepare(uintptr_t device, const PlanRequest &req, int hip_error_code, Launch &out,
            std::unique_lock<std::mutex> &lock);

// One launch per segment.  Grid size: every chunk of a segment gets the same number of slices; the
// slices past the end of a short chunk exit at once.
struct SegmentLaunch {
    const Chunk *chunks;
    uint32_t grid, shift;
};

// Fills out[0 .. count) for the plan's non-empty segments; false (nothing may be launched) when a
// segment needs more workgroups than a launch can address.
bool launch_geometry(const MultiTensorPlan &plan, int vec, int block, SegmentLaunch out[2], int &count);

}  // namespace gm
