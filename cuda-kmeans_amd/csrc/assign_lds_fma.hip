/*
 * Low-dimensional assignment on the vector ALUs (centroids in LDS, points in registers, fp32 FMA).
 * Placeholder: the variant reports every shape as unsupported until the kernel lands.
 */
#include "kmx_internal.h"

namespace kmx {

bool lds_fma_supports(const AssignArgs&, const DeviceInfo&) { return false; }

int launch_assign_lds_fma(const AssignArgs& a, kmx_exec_params*, Workspace*, const DeviceInfo&)
{
	return fail(KMX_ERR_UNSUPPORTED, "assign (LDS/FMA): dim %u, k %u not supported", a.dim, a.k);
}

} // namespace kmx
