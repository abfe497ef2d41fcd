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
