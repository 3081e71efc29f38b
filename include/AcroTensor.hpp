// Umbrella header of the library (same include name as the reference's AcroTensor.hpp:6-9).
#ifndef ACRO_HIP_ACROTENSOR_HPP
#define ACRO_HIP_ACROTENSOR_HPP

#include "Error.hpp"
#include "HipRuntime.hpp"
#include "IndexMapping.hpp"
#include "IndexVector.hpp"
#include "SliceTensor.hpp"
#include "Tensor.hpp"
#include "TensorEngine.hpp"

#endif
