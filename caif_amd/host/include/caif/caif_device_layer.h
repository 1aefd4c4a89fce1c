// Layer base classes.  Mirrors include/caif/caif_device_layer.h:83-106 (non-virtual
// Forward/Backward wrappers over ForwardImpl/BackwardImpl) and caif_device_layer_typed.h
// (compile-time ComputeT / StorageT), reduced to what the frozen layers use.
#pragma once

#include <string>
#include <vector>

#include "caif_cuda_stream.h"
#include "caif_data_type.h"
#include "caif_device_tensor.h"
#include "caif_run_context.h"

namespace instance
{

class CAIF_DeviceLayer
{
  public:
    explicit CAIF_DeviceLayer(CAIF_CudaStream &stream):_stream(&stream){}
    virtual ~CAIF_DeviceLayer()=default;
    CAIF_DeviceLayer(CAIF_DeviceLayer &&)=default;
    CAIF_DeviceLayer &operator=(CAIF_DeviceLayer &&)=default;

    CAIF_DeviceTensor Forward(const CAIF_DeviceTensor &input,CAIF_RunContext &ctx){return ForwardImpl(input,ctx);}
    CAIF_DeviceTensor Backward(const CAIF_DeviceTensor &grad_output,CAIF_RunContext &ctx){return BackwardImpl(grad_output,ctx);}

    virtual CAIF_DeviceTensor ForwardImpl(const CAIF_DeviceTensor &input,CAIF_RunContext &ctx)=0;
    virtual CAIF_DeviceTensor BackwardImpl(const CAIF_DeviceTensor &grad_output,CAIF_RunContext &ctx)=0;
    virtual void ZeroGradients()=0;
    virtual size_t ParameterTensorCount()const=0;
    virtual CAIF_DeviceTensor &ParameterTensor(size_t index)=0;
    virtual CAIF_DeviceTensor &GradientTensor(size_t index)=0;
    virtual size_t TotalParameterCount()const=0;
    virtual std::string Description()const=0;
    virtual std::vector<std::string> ParameterNames(const std::string &prefix="")const=0;
    virtual size_t FrozenTensorCount()const{return 0;}
    virtual CAIF_DeviceTensor FrozenTensorFP32(size_t index)const
    {
      (void)index;
      THROW_CAIFE("layer has no frozen tensors");
    }
    virtual std::vector<std::string> FrozenTensorNames(const std::string &prefix="")const
    {
      (void)prefix;
      return {};
    }

    bool HasStream()const{return _stream!=nullptr;}
    CAIF_CudaStream &Stream()const{return *_stream;}

  private:
    CAIF_CudaStream *_stream;
};

template<typename ComputeT,typename StorageT>
class CAIF_DeviceLayerTyped:public CAIF_DeviceLayer
{
  public:
    using CAIF_DeviceLayer::CAIF_DeviceLayer;
    static constexpr CAIF_DataType::CAIF_DataType_e ComputeDtype(){return CAIF_DtypeOf<ComputeT>::value;}
    static constexpr CAIF_DataType::CAIF_DataType_e StorageDtype(){return CAIF_DtypeOf<StorageT>::value;}
};

}//end instance namespace
