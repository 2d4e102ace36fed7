// The public device API of OriginDL (include/origin/cuda/cuda.h:25-105 in the reference: is_available, device_count,
// current_device, set_device, device_info, synchronize) answered by the gfx950 backend.
//
// The reference's header implements these inline over the CUDA runtime (under WITH_CUDA) or as "not available" stubs. A
// build against this backend force-includes this file first (-include): it claims the reference header's include guard,
// so the applications' and tests' `#include "origin/cuda/cuda.h"` then contributes nothing, and the same names resolve
// to the functions below. The device keeps its reference label: DeviceType::kCUDA / "cuda:N".
#ifndef __ORIGIN_DL_CUDA_H__
#define __ORIGIN_DL_CUDA_H__

#include <iostream>
#include <stdexcept>
#include <string>

#include "odl_hip.h"

namespace origin
{
namespace cuda
{
inline void throw_last(const char *what)
{
    throw std::runtime_error(std::string(what) + ": " + odl_hip_last_error());
}

inline int device_count()
{
    int n = 0;
    return odl_hip_device_count(&n) == ODL_OK ? n : 0;
}

inline bool is_available()
{
    return device_count() > 0;
}

inline int current_device()
{
    int d = 0;
    if (odl_hip_get_device(&d) != ODL_OK)
        throw_last("current_device");
    return d;
}

inline void set_device(int device_id)
{
    if (odl_hip_set_device(device_id) != ODL_OK)
        throw_last("set_device");
}

inline void device_info()
{
    const int n = device_count();
    std::cout << "Devices: " << n << std::endl;
    for (int i = 0; i < n; ++i)
    {
        char text[256] = {0};
        if (odl_hip_device_info(i, text, sizeof(text)) == ODL_OK)
            std::cout << "  cuda:" << i << "  " << text << std::endl;
    }
}

inline void synchronize()
{
    if (odl_hip_synchronize() != ODL_OK)
        throw_last("synchronize");
}
}  // namespace cuda
}  // namespace origin

#endif  // __ORIGIN_DL_CUDA_H__
