// The linear scan with tiles of 16 columns a wave.
#include "recurrence_scan.inc"

int cisr_scan_launch_c16(const ScanArgs& p, int segments, bool vec, hipStream_t stream) {
    return launch_scan_cols<16>(p, segments, vec, stream);
}
