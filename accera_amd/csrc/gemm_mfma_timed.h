// Timed instantiations of the 256x256 MFMA kernels for one input type, for the probes library
// (libaccera_mi355x_probes.so): a translation unit defines ACC950_IN and ACC950_TIMED_FN and includes this.
#include "gemm_mfma16w4.h"
#include "probe_timed.h"

namespace acc950 {

// Timed build of the kernel the automatic choice takes for large aligned problems with row-major B:
// the four-wave kernel when K has at least four K tiles, else the 256x256 ping-pong kernel on the
// 16x16 MFMA shapes.  Same code plus four clock stamps per workgroup.
hipError_t ACC950_TIMED_FN(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    constexpr int K4 = 4 * 64 / InTraits<ACC950_IN>::ES;
    if (a.K >= K4 && (a.M / 256) * (a.N / 256) > kComputeUnits) // more than one round of tiles: the multi-tile form
        return launch_mfma16w4<Mfma16W4Config<ACC950_IN, false, true, 256, true>>(a, stream, geom, dry_run);
    if (a.K >= K4) return launch_mfma16w4<Mfma16W4Config<ACC950_IN, false, true>>(a, stream, geom, dry_run);
    return launch_mfma16<Mfma16Config<ACC950_IN, 256, 256, 2, 4, true, false, 64, 4, false, true>>(a, stream, geom, dry_run);
}


} // namespace acc950
