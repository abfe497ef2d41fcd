// What the batch-normalisation entry points decide on the host before they
// launch: the family of kernels, the vector width, the grid and the index maps
// of every tensor.  A caller can ask for these decisions without anything being
// launched (LaunchLog): the launch audit walks them on the CPU, and the
// two-launch entry points use the same switch to validate their second launch
// before they issue the first.
#pragma once

#include <vector>

#include "h2x_bn_maps.hpp"

namespace h2x
{
namespace bn
{

enum Kernel : int
{
    kKernelSums = 0,
    kKernelApply = 1,
    kKernelBackprop1 = 2,
    kKernelBackprop2 = 3,
    kKernelFinish = 4,      // adds the partial sums of a reduction
    kKernelStatistics = 5,  // sums -> mean / variance / running statistics
    kKernelFill = 6,        // zeroes per-channel outputs (empty tensors)
    kKernelClearing = 7     // normalise / input gradient over the real tensor, halo of the output zeroed
};

enum Family : int
{
    kFamilyDense = 0,   // segments addressed as they lie: aligned vectors or single elements
    kFamilyStrided = 1, // index splitting: haloed rows, folded samples, unaligned dense segments
    kFamilyShort = 2    // segments of at most 256 elements: windows of whole channels
};

constexpr int kMaxLaunchTensors = 3;

// One kernel launch as the host planned it.
struct LaunchRecord
{
    int kernel = 0;
    int family = 0;
    int vec = 1;            // elements per access
    int tail = 0;           // ShortTail (short family)
    bool fused = false;     // the kernel finishes the preceding reduction itself
    bool folded = false;    // samples folded into the rows of one long segment
    bool rewrite = true;    // elements two vectors share may be stored by both
    unsigned int grid_x = 0, grid_y = 1;
    int num_sums = 0;       // reductions: sums per channel (2 or 4)
    int groups_max = 0;     // reductions: partial sums the workspace holds per channel and sum
    bool partials = false;  // reductions: results go to the workspace, a finishing step follows
    int num_samples = 0, num_channels = 0; // as the kernel sees them (after folding)
    size_t spatial = 0;     // elements of a segment as the kernel counts them (rows padded)
    size_t chunk = 0;
    int chunks_per_seg = 0;
    unsigned int num_units = 0;
    int num_tensors = 0;    // tensors addressed through maps: inputs first, the output last
    bool last_is_output = false;
    TensorMap map[kMaxLaunchTensors];     // dense and strided families
    ShortTensor tensor[kMaxLaunchTensors]; // short family
    ShortGeometry geometry;                // short family
    RealBox box;                           // halo-clearing kernel: real extents and interior
    size_t real = 0;                       // halo-clearing kernel: cells of a real segment
};

struct LaunchLog
{
    std::vector<LaunchRecord> records;
};

// While a log is installed on the calling thread, the entry points of
// h2x_bn.hip plan as usual and append their launches to it instead of issuing
// them; no GPU call is made.  Returns the log that was installed before.
LaunchLog* install_launch_log(LaunchLog* log);

} // namespace bn
} // namespace h2x
