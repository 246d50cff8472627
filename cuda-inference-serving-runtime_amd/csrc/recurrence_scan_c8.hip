// The linear scan with tiles of 8 columns a wave.
#include "recurrence_scan.inc"

int cisr_scan_launch_c8(const ScanArgs& p, int segments, bool vec, hipStream_t stream) {
    return launch_scan_cols<8>(p, segments, vec, stream);
}
