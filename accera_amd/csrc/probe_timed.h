// Launchers of the timed kernel builds (probe_timed_*.hip), used by the phase probe (probes.hip).
#pragma once
#include "common.h"

namespace acc950 {

hipError_t launch_mfma_timed_f16(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run);
hipError_t launch_mfma_timed_bf16(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run);
hipError_t launch_mfma_timed_i8(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run);

} // namespace acc950
