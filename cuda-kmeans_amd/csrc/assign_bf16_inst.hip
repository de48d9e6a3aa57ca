/*
 * One instantiation of the split-bf16 MFMA assignment kernel family: KMX_KB blocks of 16 dimensions per row
 * (given on the command line).
 */
#include "assign_bf16_impl.h"

#ifndef KMX_KB
#error "compile with -DKMX_KB=<blocks of 16 dimensions per row>"
#endif

#define KMX_CAT2(a, b) a##b
#define KMX_CAT(a, b) KMX_CAT2(a, b)

namespace kmx {

int KMX_CAT(launch_bf16_, KMX_KB)(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	return launch_bf16_kb<KMX_KB>(a, exec, ws, dev, kp, kd);
}

int KMX_CAT(launch_screen_bf16_, KMX_KB)(const float* rows, const Workspace* ws, const uint32_t* row_queue, const uint32_t* row_count,
                                         uint32_t* pairs, uint32_t* item_pairs, unsigned long long* keys, uint32_t dim, uint32_t k, uint32_t kp,
                                         const DeviceInfo& dev, uint32_t* waves)
{
	return launch_screen_bf16_kb<KMX_KB>(rows, ws, row_queue, row_count, pairs, item_pairs, keys, dim, k, kp, dev, waves);
}

} // namespace kmx
