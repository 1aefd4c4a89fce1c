// Dtype-erased interface of a frozen linear (include/caif/caif_device_frozen_linear_base.h:45-80):
// what loaders, the factory's callers and the offload scheduler use after a dynamic_cast.
#pragma once

#include <cstddef>
#include <cstdint>

#include "caif_cuda_stream.h"
#include "caif_device_tensor.h"
#include "caif_offload_policy.h"
#include "caif_ops.h"

namespace instance
{

class CAIF_DeviceFrozenLinearBase
{
  public:
    virtual ~CAIF_DeviceFrozenLinearBase()=default;
    virtual void LoadFromTensor(CAIF_DeviceTensor &&weight)=0;
    virtual void LoadScalesFromHost(const void *data,size_t num_bytes)=0;
    virtual void ClearFP32Cache()=0;
    virtual bool NeedsScales()const=0;
    virtual CAIF_Ops::QuantScheme_e Int8Scheme()const=0;
    virtual bool CacheFP32()const=0;
    virtual uint32_t InputDim()const=0;
    virtual uint32_t OutputDim()const=0;
    virtual void SetOffloadPolicy(const CAIF_OffloadPolicy::CAIF_OffloadPolicy_e p){(void)p;}
    virtual CAIF_OffloadPolicy::CAIF_OffloadPolicy_e OffloadPolicy()const
    {
      return CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::GpuResident_e;
    }
    virtual void Prefetch(CAIF_CudaStream &stream){(void)stream;}
    virtual void Evict(){}
    virtual bool IsPrefetched()const{return true;}
};

}//end instance namespace
