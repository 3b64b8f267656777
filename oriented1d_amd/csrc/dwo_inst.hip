// One translation unit per (element type, plane extent): compile with
//   -DDWO_INST_T=<float|bf16_t|f16_t> -DDWO_INST_K=<K> -DDWO_INST_H=<H> -DDWO_INST_W=<W>
#include "dwo_static.h"
#include "dwo_nhwc_plane.h"
#include "dwo_regplane.h"

namespace dwo {
template int launch_plane_conv<DWO_INST_T, DWO_INST_K, DWO_INST_H, DWO_INST_W>(
    int, const void *, const float *, const float *, const void *, void *, int, int, hipStream_t);
template int launch_plane_wgrad<DWO_INST_T, DWO_INST_K, DWO_INST_H, DWO_INST_W>(
    const void *, const void *, const void *, float *, float *, float *, unsigned *, int, int, int *,
    hipStream_t);
template int launch_nhwc_plane_conv<DWO_INST_T, DWO_INST_K, DWO_INST_H, DWO_INST_W>(
    int, const void *, const float *, const float *, const void *, void *, int, int, hipStream_t);
template int launch_nhwc_plane_wgrad<DWO_INST_T, DWO_INST_K, DWO_INST_H, DWO_INST_W>(
    const void *, const void *, const void *, float *, float *, float *, unsigned *, int, int, int *,
    hipStream_t);
}  // namespace dwo
