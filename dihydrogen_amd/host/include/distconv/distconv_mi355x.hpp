// Umbrella header of the MI355X hot path behind the DistConv layer API:
//   distconv::BatchNormalization<BackendMI355X, T>, distconv::Softmax<BackendMI355X>,
//   distconv::tensor::HaloExchange / HaloExchangeVirtual,
//   distconv::tensor::TensorMPICUDAShuffler / TensorShufflerVirtual,
//   distconv::tensor::Transform / ReduceSum / TransformReduceSum,
// and the tensor model they are written against.  Link with libh2x.so.
#pragma once

#include "distconv/algorithms_mi355x.hpp"
#include "distconv/base_mi355x.hpp"
#include "distconv/halo_shuffle_mi355x.hpp"
#include "distconv/layers_mi355x.hpp"
#include "distconv/tensor_mi355x.hpp"

#include <fstream>
#include <string>
#include <vector>

namespace distconv
{

// legacy/include/distconv/distconv.hpp:634-671 -- debugging aid: the local part
// of a tensor in <file_path>_<rank>.txt (one value a line) or .out (raw bytes).
// The whole local allocation is written, halo cells included, in memory order:
// what the reference's copyout hands over (for a tensor without halos that is
// its local elements, the case the reference sizes its buffer for).  Blocking.
template <typename DataType>
inline int dump_local_tensor(tensor::Tensor<DataType, tensor::LocaleVirtual, tensor::CUDAAllocator>& t,
                             std::string file_path, bool binary = false)
{
    file_path += "_" + std::to_string(t.get_locale().get_rank()) + (binary ? ".out" : ".txt");
    std::vector<DataType> h(t.get_local_real_size());
    if (!h.empty())
        DISTCONV_CHECK_HIP(hipMemcpy(h.data(), t.get_buffer(), h.size() * sizeof(DataType),
                                     hipMemcpyDeviceToHost));
    std::ofstream out;
    if (!binary)
    {
        out.open(file_path, std::ios::out | std::ios::trunc);
        for (const DataType& v : h)
            out << v << std::endl;
    }
    else
    {
        out.open(file_path, std::ios::out | std::ios::trunc | std::ios::binary);
        out.write(reinterpret_cast<const char*>(h.data()), h.size() * sizeof(DataType));
    }
    return out.good() ? 0 : -1;
}

} // namespace distconv
