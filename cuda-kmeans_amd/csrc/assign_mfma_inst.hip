/*
 * One instantiation of the MFMA assignment kernel family: per-half row width KMX_DPH (given on the command line).
 */
#include "assign_mfma_impl.h"

#ifndef KMX_DPH
#error "compile with -DKMX_DPH=<per-half dimension count>"
#endif

#define KMX_CAT2(a, b) a##b
#define KMX_CAT(a, b) KMX_CAT2(a, b)

namespace kmx {

int KMX_CAT(launch_mfma_, KMX_DPH)(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	return launch_mfma_dph<KMX_DPH>(a, exec, ws, dev, kp, kd);
}

} // namespace kmx
