// Runtime (storage dtype, compute dtype) -> template cell.  Signature of
// CAIF_DeviceFrozenLinearFactory::Create (src/caif_device_frozen_linear_factory.cpp:46-54); callers
// dynamic_cast the result to CAIF_DeviceFrozenLinearBase* to load weights and scales
// (tests/test_device_frozen_linear.cpp:237-238).  All fifteen cells of the reference's grid are built; the nine
// float-storage ones run on the fp32 matrix-core kernel (they are not on the quantised fast paths).
#pragma once

#include <memory>

#include "caif_device_frozen_linear.h"

namespace instance
{

class CAIF_DeviceFrozenLinearFactory
{
  public:
    typedef CAIF_DataType::CAIF_DataType_e Dtype_e;

    static std::unique_ptr<CAIF_DeviceLayer> Create(uint32_t input_dim,uint32_t output_dim,Dtype_e storage_dtype,
                                                    CAIF_CudaStream &stream,
                                                    uint32_t group_size=g_caif_quant_default_group_size,
                                                    bool cache_fp32=true,Dtype_e compute_dtype=Dtype_e::Float32,
                                                    CAIF_Ops::QuantScheme_e int8_scheme=CAIF_Ops::QuantScheme_e::PerTensor_e)
    {
      try
      {
        if(storage_dtype==Dtype_e::Int8)
        {
          return ByCompute<int8_t>(input_dim,output_dim,stream,group_size,cache_fp32,compute_dtype,int8_scheme);
        }
        if(storage_dtype==Dtype_e::Int4)
        {
          return ByCompute<caif_int4_packed_t>(input_dim,output_dim,stream,group_size,cache_fp32,compute_dtype,int8_scheme);
        }
        if(storage_dtype==Dtype_e::Float32)
        {
          return ByCompute<float>(input_dim,output_dim,stream,group_size,cache_fp32,compute_dtype,int8_scheme);
        }
        if(storage_dtype==Dtype_e::Float16)
        {
          return ByCompute<caif_fp16_t>(input_dim,output_dim,stream,group_size,cache_fp32,compute_dtype,int8_scheme);
        }
        if(storage_dtype==Dtype_e::BFloat16)
        {
          return ByCompute<caif_bf16_t>(input_dim,output_dim,stream,group_size,cache_fp32,compute_dtype,int8_scheme);
        }
        THROW_CAIFE("FrozenLinearFactory: unsupported storage dtype");
      }
      CAIF_CATCH_BLOCK()
    }

  private:
    template<typename StorageT>
    static std::unique_ptr<CAIF_DeviceLayer> ByCompute(uint32_t in,uint32_t out,CAIF_CudaStream &stream,uint32_t group,
                                                       bool cache,Dtype_e compute,CAIF_Ops::QuantScheme_e scheme)
    {
      if(compute==Dtype_e::Float32)
      {
        return std::make_unique<CAIF_DeviceFrozenLinear<float,StorageT>>(in,out,stream,group,cache,scheme);
      }
      if(compute==Dtype_e::Float16)
      {
        return std::make_unique<CAIF_DeviceFrozenLinear<caif_fp16_t,StorageT>>(in,out,stream,group,cache,scheme);
      }
      if(compute==Dtype_e::BFloat16)
      {
        return std::make_unique<CAIF_DeviceFrozenLinear<caif_bf16_t,StorageT>>(in,out,stream,group,cache,scheme);
      }
      THROW_CAIFE("FrozenLinearFactory: unsupported compute dtype");
    }
};

}//end instance namespace
