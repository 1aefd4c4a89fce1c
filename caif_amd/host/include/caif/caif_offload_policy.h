// Where a frozen weight lives between uses (include/caif/caif_offload_policy.h of the reference).
#pragma once

#include <cstdint>

namespace instance
{

class CAIF_OffloadPolicy
{
  public:
    enum class CAIF_OffloadPolicy_e:uint8_t{GpuResident_e,HostPinned_e};
};

}//end instance namespace
