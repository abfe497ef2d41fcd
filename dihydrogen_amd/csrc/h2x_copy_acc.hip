// Accumulating instantiations of the box copy kernel: unpack and tensor-to-
// tensor transfer with SUM / MAX / MIN on float and double elements
// (legacy/include/distconv/tensor/halo_packing_cuda.hpp:36-58).
#include "h2x_copy_kernel.hpp"

namespace h2x
{
namespace copy
{
namespace
{

template <typename T, int VEC, typename Op>
int launch_op(const LaunchShape& s, const BoxBatch& batch)
{
    if (s.mode == kUnpack)
        return s.sparse ? run_box_copy<T, VEC, Op, true, kUnpack, false>(s.grid, s.stream, batch, Op())
                        : run_box_copy<T, VEC, Op, false, kUnpack, false>(s.grid, s.stream, batch, Op());
    if (s.mode == kTransfer)
        return s.sparse ? run_box_copy<T, VEC, Op, true, kTransfer, false>(s.grid, s.stream, batch, Op())
                        : run_box_copy<T, VEC, Op, false, kTransfer, false>(s.grid, s.stream, batch, Op());
    return H2X_ERR_UNSUPPORTED;
}

template <typename T, int VEC>
int launch_vec(const LaunchShape& s, const BoxBatch& batch)
{
    switch (s.op)
    {
    case H2X_HALO_SUM: return launch_op<T, VEC, OpSum>(s, batch);
    case H2X_HALO_MAX: return launch_op<T, VEC, OpMax>(s, batch);
    case H2X_HALO_MIN: return launch_op<T, VEC, OpMin>(s, batch);
    default: return H2X_ERR_UNSUPPORTED;
    }
}

} // namespace

int launch_accumulate(const LaunchShape& s, h2x_dtype dtype, const BoxBatch& batch)
{
    if (dtype == H2X_F32 && s.elem_size == 4)
    {
        switch (s.vec)
        {
        case 4: return launch_vec<float, 4>(s, batch);
        case 2: return launch_vec<float, 2>(s, batch);
        case 1: return launch_vec<float, 1>(s, batch);
        }
    }
    else if (dtype == H2X_F64 && s.elem_size == 8)
    {
        switch (s.vec)
        {
        case 2: return launch_vec<double, 2>(s, batch);
        case 1: return launch_vec<double, 1>(s, batch);
        }
    }
    return H2X_ERR_UNSUPPORTED;
}

} // namespace copy
} // namespace h2x
