// CAIF_DeviceFrozenLinear<ComputeT,StorageT>: a linear layer whose weight is frozen and stored
// quantised (int8 or packed int4), with zero trainable parameters.
//
// Same public surface and error behaviour as the reference's class
// (include/caif/caif_device_frozen_linear.h:73-260, src/caif_device_frozen_linear.cpp), different
// inside: the reference materialises the whole weight in the compute dtype (dequantise kernel +
// cast, optionally cached) and calls a vendor GEMM; here Forward/Backward are each ONE fused
// dequant-GEMM launch through the C ABI (caifx_qlinear_forward / _backward_input), so no dense
// copy of the weight exists and `cache_fp32` is only a remembered hint.
//   * weight layout: [OutputDim, InputDim] row-major codes, exactly as the reference keeps it;
//   * int8 scales: 1 (PerTensor_e) or OutputDim (PerChannel_e) fp32 values, applied with the
//     reference's indexing scale[(n*K + k) % OutputDim] (src/caif_device_frozen_linear.cpp:356-361);
//   * int4 scales: fp16, one per `group_size` consecutive flat elements;
//   * output of Forward and Backward is always fp32 (:442, :580);
//   * Backward needs a preceding Forward with training=true (:543-546); the reference checks a
//     cached copy of the input that it never reads, this class keeps the flag and no copy.
// Float storage cells (fp32/fp16/bf16 weights) of the reference's 5x3 grid are outside this build.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "caif_device_frozen_linear_base.h"
#include "caif_device_layer.h"
#include "caif_offload_policy.h"
#include "caif_ops.h"

namespace instance
{

constexpr uint32_t g_caif_quant_default_group_size=128;   // include/caif/caif_constants.h:257

template<typename ComputeT=float,typename StorageT=int8_t>
class CAIF_DeviceFrozenLinear:public CAIF_DeviceLayerTyped<ComputeT,StorageT>,
                              public CAIF_DeviceFrozenLinearBase
{
  static_assert(std::is_same<StorageT,int8_t>::value||std::is_same<StorageT,caif_int4_packed_t>::value||
                std::is_same<StorageT,float>::value||std::is_same<StorageT,caif_fp16_t>::value||
                std::is_same<StorageT,caif_bf16_t>::value,
                "CAIF_DeviceFrozenLinear: storage is int8, packed int4 or one of the three float types");

  public:
    typedef CAIF_DeviceLayerTyped<ComputeT,StorageT> Base_t;
    typedef CAIF_DataType::CAIF_DataType_e Dtype_e;
    using Base_t::Stream;
    using Base_t::HasStream;

    CAIF_DeviceFrozenLinear(uint32_t input_dim,uint32_t output_dim,CAIF_CudaStream &stream,
                            uint32_t group_size=g_caif_quant_default_group_size,bool cache_fp32=true,
                            CAIF_Ops::QuantScheme_e int8_scheme=CAIF_Ops::QuantScheme_e::PerTensor_e)
      :Base_t(stream),_input_dim(input_dim),_output_dim(output_dim),_int8_scheme(int8_scheme),
       _group_size(group_size),_cache_fp32(cache_fp32),_trained_forward(false),
       _offload_policy(CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::GpuResident_e),_host_weight(nullptr),
       _host_bytes(0),_is_prefetched(false)
    {
      try
      {
        if(input_dim==0||output_dim==0)
        {
          THROW_CAIFE("FrozenLinear: input_dim and output_dim must be > 0");
        }
      }
      CAIF_CATCH_BLOCK()
    }
    ~CAIF_DeviceFrozenLinear()override{FreeHostWeight();}
    CAIF_DeviceFrozenLinear(CAIF_DeviceFrozenLinear &&)=delete;
    CAIF_DeviceFrozenLinear &operator=(CAIF_DeviceFrozenLinear &&)=delete;

    // --- CAIF_DeviceLayer interface ---
    CAIF_DeviceTensor ForwardImpl(const CAIF_DeviceTensor &input,CAIF_RunContext &ctx)override
    {
      try
      {
        CheckReady("FrozenLinear::ForwardImpl","forward");
        const auto &shape=input.Shape();
        if(shape.size()<2){THROW_CAIFE("FrozenLinear::Forward: input must be at least 2D");}
        if(shape.back()!=InputDim()){THROW_CAIFE("FrozenLinear::Forward: last dim must match input_dim");}
        uint32_t n=1;
        for(size_t i=0;i+1<shape.size();++i)
        {
          n*=shape[i];
        }
        if(ctx.Training()==true)
        {
          _trained_forward=true;
        }
        CAIF_DeviceTensor out=CAIF_DeviceTensor::Uninitialized({n,OutputDim()},Stream());
        CAIF_DeviceTensor ws=Workspace(n,CAIF_DataType(input.Dtype()).CaifxCode(),false);
        CAIF_Ops::Check(caifx_qlinear_forward(n,OutputDim(),InputDim(),input.DeviceDataRaw(),
                                              CAIF_DataType(input.Dtype()).CaifxCode(),
                                              CAIF_DataType(Base_t::ComputeDtype()).CaifxCode(),
                                              _weight.DeviceDataRaw(),WeightKind(),ScalesPtr(),ScalePeriod(),
                                              static_cast<int>(_group_size),out.DeviceDataRaw(),CAIFX_F32,
                                              ws.DeviceDataRaw(),ws.SizeBytes(),Stream().Handle()),
                        "FrozenLinear: dequant-GEMM forward failed");
        if(shape.size()>2)
        {
          std::vector<uint32_t> out_shape(shape.begin(),shape.end()-1);
          out_shape.push_back(OutputDim());
          out.Reshape(out_shape);
        }
        return out;
      }
      CAIF_CATCH_BLOCK()
    }

    CAIF_DeviceTensor BackwardImpl(const CAIF_DeviceTensor &grad_output,CAIF_RunContext &ctx)override
    {
      try
      {
        (void)ctx;
        if(HasStream()==false){THROW_CAIFE("FrozenLinear: stream is null");}
        if(OffloadPolicy()==CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e&&IsPrefetched()==false)
        {
          THROW_CAIFE("FrozenLinear::BackwardImpl: HostPinned policy but layer is not prefetched."
                      " The block-level scheduler must call Prefetch(stream) before backward.");
        }
        if(_trained_forward==false){THROW_CAIFE("FrozenLinear::Backward: must call Forward with training=true first");}
        if(_weight.IsEmpty()==true){THROW_CAIFE("FrozenLinear: weight not loaded");}
        RequireScales();
        const auto &shape=grad_output.Shape();
        if(shape.empty()==true||shape.back()!=OutputDim())
        {
          THROW_CAIFE("FrozenLinear::Backward: last dim must match output_dim");
        }
        uint32_t n=1;
        for(size_t i=0;i+1<shape.size();++i)
        {
          n*=shape[i];
        }
        CAIF_DeviceTensor dx=CAIF_DeviceTensor::Uninitialized({n,InputDim()},Stream());
        CAIF_DeviceTensor ws=Workspace(n,CAIF_DataType(grad_output.Dtype()).CaifxCode(),true);
        CAIF_Ops::Check(caifx_qlinear_backward_input(n,OutputDim(),InputDim(),grad_output.DeviceDataRaw(),
                                                     CAIF_DataType(grad_output.Dtype()).CaifxCode(),
                                                     CAIF_DataType(Base_t::ComputeDtype()).CaifxCode(),
                                                     _weight.DeviceDataRaw(),WeightKind(),ScalesPtr(),ScalePeriod(),
                                                     static_cast<int>(_group_size),dx.DeviceDataRaw(),CAIFX_F32,
                                                     ws.DeviceDataRaw(),ws.SizeBytes(),Stream().Handle()),
                        "FrozenLinear: dequant-GEMM backward failed");
        if(shape.size()>2)
        {
          std::vector<uint32_t> in_shape(shape.begin(),shape.end()-1);
          in_shape.push_back(InputDim());
          dx.Reshape(in_shape);
        }
        return dx;
      }
      CAIF_CATCH_BLOCK()
    }

    void ZeroGradients()override{}
    size_t ParameterTensorCount()const override{return 0;}
    CAIF_DeviceTensor &ParameterTensor(size_t index)override
    {
      (void)index;
      THROW_CAIFE("FrozenLinear: no trainable parameters");
    }
    CAIF_DeviceTensor &GradientTensor(size_t index)override
    {
      (void)index;
      THROW_CAIFE("FrozenLinear: no trainable parameters");
    }
    size_t TotalParameterCount()const override{return 0;}
    std::string Description()const override
    {
      return std::string("FrozenLinear(")+std::to_string(InputDim())+","+std::to_string(OutputDim())+","+
             CAIF_DataType(Base_t::StorageDtype()).Name()+")";
    }
    std::vector<std::string> ParameterNames(const std::string &prefix="")const override
    {
      (void)prefix;
      return {};
    }
    size_t FrozenTensorCount()const override{return 1;}
    // The stored weight dequantised to fp32 [OutputDim, InputDim] (checkpoint export path,
    // src/caif_device_frozen_linear.cpp:760-826).
    CAIF_DeviceTensor FrozenTensorFP32(size_t index)const override
    {
      try
      {
        if(index!=0){THROW_CAIFE("FrozenLinear: frozen tensor index out of range");}
        if(_weight.IsEmpty()==true){THROW_CAIFE("FrozenLinear: weight not loaded");}
        if(IsFloatStorage()==true)
        {
          // float storage: the weight itself, widened (src/caif_device_frozen_linear.cpp:780-790); nothing else is
          // allocated on this path
          CAIF_DeviceTensor wide=_weight.To(Dtype_e::Float32);
          wide.Reshape({OutputDim(),InputDim()});
          return wide;
        }
        const int64_t total=static_cast<int64_t>(InputDim())*OutputDim();
        CAIF_DeviceTensor fp32=CAIF_DeviceTensor::Uninitialized({OutputDim(),InputDim()},Stream());
        hipStream_t s=Stream().Handle();
        int st;
        if(IsInt4()==true)
        {
          if(_scales.IsEmpty()==true){THROW_CAIFE("FrozenLinear: scales not loaded");}
          st=caifx_dequantize_int4(_weight.DeviceDataRaw(),_scales.DeviceDataRaw(),fp32.DevicePtr<float>(),total,
                                   static_cast<int>(_group_size),s);
        }
        else if(_scales.IsEmpty()==true)
        {
          st=caifx_convert_int8_to_fp32(_weight.DeviceDataRaw(),fp32.DevicePtr<float>(),total,s);
        }
        else if(_int8_scheme==CAIF_Ops::QuantScheme_e::PerTensor_e)
        {
          st=caifx_dequantize_int8_per_tensor(_weight.DeviceDataRaw(),fp32.DevicePtr<float>(),_scales.DeviceDataRaw(),total,s);
        }
        else
        {
          st=caifx_dequantize_int8_per_channel(_weight.DeviceDataRaw(),fp32.DevicePtr<float>(),_scales.DeviceDataRaw(),
                                               static_cast<int>(InputDim()),static_cast<int>(OutputDim()),s);
        }
        CAIF_Ops::Check(st,"FrozenLinear::FrozenTensorFP32");
        return fp32;
      }
      CAIF_CATCH_BLOCK()
    }
    std::vector<std::string> FrozenTensorNames(const std::string &prefix="")const override{return {prefix+"weight"};}

    // --- CAIF_DeviceFrozenLinearBase interface ---
    void LoadFromTensor(CAIF_DeviceTensor &&weight)override
    {
      try
      {
        _weight=std::move(weight);
        if(_offload_policy==CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e)
        {
          MigrateWeightToHost();
        }
        else
        {
          _is_prefetched=true;
        }
      }
      CAIF_CATCH_BLOCK()
    }
    void LoadScalesFromHost(const void *data,size_t num_bytes)override
    {
      try
      {
        if(IsInt4()==true)
        {
          const size_t total=static_cast<size_t>(InputDim())*OutputDim();
          const uint32_t num_groups=static_cast<uint32_t>((total+_group_size-1)/_group_size);
          _scales=CAIF_DeviceTensor::Zeros({num_groups},Stream(),Dtype_e::Float16);
        }
        else if(_int8_scheme==CAIF_Ops::QuantScheme_e::PerTensor_e)
        {
          _scales=CAIF_DeviceTensor::Zeros({1u},Stream(),Dtype_e::Float32);
        }
        else
        {
          _scales=CAIF_DeviceTensor::Zeros({OutputDim()},Stream(),Dtype_e::Float32);
        }
        _scales.CopyFromHostRaw(data,num_bytes);
      }
      CAIF_CATCH_BLOCK()
    }
    // Device-to-device variant (not in the reference, whose callers bounce scales through the
    // host): adopts an already device-resident scales tensor of the right length.
    void LoadScalesFromTensor(CAIF_DeviceTensor &&scales)
    {
      try
      {
        const size_t total=static_cast<size_t>(InputDim())*OutputDim();
        size_t want=1;
        if(IsInt4()==true){want=(total+_group_size-1)/_group_size;}
        else if(_int8_scheme==CAIF_Ops::QuantScheme_e::PerChannel_e){want=OutputDim();}
        const Dtype_e dt=IsInt4()?Dtype_e::Float16:Dtype_e::Float32;
        if(scales.TotalElements()!=want||scales.Dtype()!=dt)
        {
          THROW_CAIFE("FrozenLinear::LoadScalesFromTensor: scales length or dtype does not match the layer");
        }
        _scales=std::move(scales);
      }
      CAIF_CATCH_BLOCK()
    }
    // On-disk form of the quantised storage (not in the reference, which exports frozen weights as
    // fp32 only, src/caif_device_frozen_linear.cpp:760-826): "<prefix>weight" = the codes as they sit
    // in memory (I8 [OutputDim,InputDim], or I4 of the same shape packed two codes per byte, low
    // nibble = even flat index) and "<prefix>scales" (F32 [1] or [OutputDim]; F16 [groups]), plus
    // the three facts a reader needs to interpret them.  The pointers stay owned by the layer.
    void ExportQuantized(const std::string &prefix,
                         std::vector<std::pair<std::string,const CAIF_DeviceTensor*>> &tensors,
                         std::map<std::string,std::string> &metadata)const
    {
      try
      {
        if(_weight.IsEmpty()==true||(IsFloatStorage()==false&&_scales.IsEmpty()==true))
        {
          THROW_CAIFE("FrozenLinear::ExportQuantized: weight and scales must be loaded (and resident on the device)");
        }
        tensors.emplace_back(prefix+"weight",&_weight);
        if(IsFloatStorage()==false)
        {
          tensors.emplace_back(prefix+"scales",&_scales);
        }
        metadata[prefix+"storage"]=CAIF_DataType(Base_t::StorageDtype()).Name();
        metadata[prefix+"group_size"]=std::to_string(_group_size);
        metadata[prefix+"int8_scheme"]=SchemeName(_int8_scheme);
      }
      CAIF_CATCH_BLOCK()
    }
    // Takes "<prefix>weight" and "<prefix>scales" out of `tensors` (e.g. what
    // CAIF_SafeTensorsFormat::Load returned) after checking them against this layer: storage type,
    // shape, group size, int8 scheme, scales length.  Nothing passes through host memory here.
    void ImportQuantized(const std::string &prefix,std::map<std::string,CAIF_DeviceTensor> &tensors,
                         const std::map<std::string,std::string> &metadata)
    {
      try
      {
        auto w=tensors.find(prefix+"weight");
        auto s=tensors.find(prefix+"scales");
        if(w==tensors.end()||(s==tensors.end()&&IsFloatStorage()==false))
        {
          THROW_CAIFE("FrozenLinear::ImportQuantized: missing tensor "+prefix+(w==tensors.end()?"weight":"scales"));
        }
        auto meta=[&](const char *key)
        {
          const auto it=metadata.find(prefix+key);
          if(it==metadata.end())
          {
            THROW_CAIFE("FrozenLinear::ImportQuantized: missing metadata "+prefix+key);
          }
          return it->second;
        };
        if(meta("storage")!=CAIF_DataType(Base_t::StorageDtype()).Name()||w->second.Dtype()!=Base_t::StorageDtype())
        {
          THROW_CAIFE("FrozenLinear::ImportQuantized: storage type does not match the layer");
        }
        if(IsInt4()==true&&meta("group_size")!=std::to_string(_group_size))
        {
          THROW_CAIFE("FrozenLinear::ImportQuantized: group size does not match the layer");
        }
        if(IsInt4()==false&&IsFloatStorage()==false&&meta("int8_scheme")!=SchemeName(_int8_scheme))
        {
          THROW_CAIFE("FrozenLinear::ImportQuantized: int8 scheme does not match the layer");
        }
        if(w->second.Shape()!=std::vector<uint32_t>{OutputDim(),InputDim()})
        {
          THROW_CAIFE("FrozenLinear::ImportQuantized: weight shape must be [output_dim, input_dim]");
        }
        if(IsFloatStorage()==false)
        {
          LoadScalesFromTensor(std::move(s->second));
        }
        LoadFromTensor(std::move(w->second));
        tensors.erase(prefix+"weight");
        tensors.erase(prefix+"scales");
      }
      CAIF_CATCH_BLOCK()
    }
    void ClearFP32Cache()override{}
    bool NeedsScales()const override{return IsFloatStorage()==false;}
    CAIF_Ops::QuantScheme_e Int8Scheme()const override{return _int8_scheme;}
    bool CacheFP32()const override{return _cache_fp32;}
    uint32_t InputDim()const override{return _input_dim;}
    uint32_t OutputDim()const override{return _output_dim;}
    uint32_t GroupSize()const{return _group_size;}

    // Raw views for callers that batch several layers into one grouped launch.
    const void *WeightData()const{return _weight.DeviceDataRaw();}
    const void *ScalesData()const{return _scales.IsEmpty()?nullptr:_scales.DeviceDataRaw();}
    int WeightKind()const
    {
      if(std::is_same<StorageT,float>::value){return CAIFX_W_F32;}
      if(std::is_same<StorageT,caif_fp16_t>::value){return CAIFX_W_F16;}
      if(std::is_same<StorageT,caif_bf16_t>::value){return CAIFX_W_BF16;}
      return IsInt4()?CAIFX_W_INT4_GROUP:CAIFX_W_INT8;
    }
    int64_t ScalePeriod()const
    {
      return (IsInt4()==false&&IsFloatStorage()==false&&_int8_scheme==CAIF_Ops::QuantScheme_e::PerChannel_e)?static_cast<int64_t>(OutputDim()):1;
    }

    // --- CPU offload surface (src/caif_device_frozen_linear.cpp:145-232) ---
    void SetOffloadPolicy(const CAIF_OffloadPolicy::CAIF_OffloadPolicy_e p)override
    {
      try
      {
        if(_offload_policy==p)
        {
          return;
        }
        if(p==CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e)
        {
          _offload_policy=p;
          if(_weight.IsAllocated()==true)
          {
            MigrateWeightToHost();
          }
          return;
        }
        if(_host_weight!=nullptr&&_weight.IsAllocated()==false)
        {
          Upload(Stream());
          Stream().Synchronize();
        }
        FreeHostWeight();
        _is_prefetched=true;
        _offload_policy=p;
      }
      CAIF_CATCH_BLOCK()
    }
    CAIF_OffloadPolicy::CAIF_OffloadPolicy_e OffloadPolicy()const override{return _offload_policy;}
    void Prefetch(CAIF_CudaStream &stream)override
    {
      try
      {
        if(_offload_policy!=CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e||_is_prefetched==true)
        {
          return;
        }
        if(_host_weight==nullptr){THROW_CAIFE("FrozenLinear::Prefetch: HostPinned policy but no host weight");}
        Upload(stream);
        _is_prefetched=true;
      }
      CAIF_CATCH_BLOCK()
    }
    void Evict()override
    {
      if(_offload_policy!=CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e)
      {
        return;
      }
      _weight=CAIF_DeviceTensor();
      _is_prefetched=false;
    }
    bool IsPrefetched()const override{return _is_prefetched;}

  private:
    static constexpr bool IsInt4(){return std::is_same<StorageT,caif_int4_packed_t>::value;}
    static constexpr bool IsFloatStorage()
    {
      return std::is_same<StorageT,float>::value||std::is_same<StorageT,caif_fp16_t>::value||
             std::is_same<StorageT,caif_bf16_t>::value;
    }
    static const char *SchemeName(CAIF_Ops::QuantScheme_e s)
    {
      return s==CAIF_Ops::QuantScheme_e::PerChannel_e?"per_channel":"per_tensor";
    }
    const void *ScalesPtr()const{return (IsFloatStorage()||_scales.IsEmpty())?nullptr:_scales.DeviceDataRaw();}
    void RequireScales()const
    {
      if(IsInt4()==true&&_scales.IsEmpty()==true){THROW_CAIFE("FrozenLinear: scales not loaded");}
    }
    void CheckReady(const char *where,const char *pass)const
    {
      if(HasStream()==false){THROW_CAIFE("FrozenLinear: stream is null");}
      if(OffloadPolicy()==CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e&&IsPrefetched()==false)
      {
        THROW_CAIFE(std::string(where)+": HostPinned policy but layer is not prefetched."
                    " The block-level scheduler must call Prefetch(stream) before "+pass+".");
      }
      if(_weight.IsEmpty()==true){THROW_CAIFE("FrozenLinear: weight not loaded");}
      RequireScales();
    }
    CAIF_DeviceTensor Workspace(uint32_t n,int x_code,bool backward)const
    {
      const size_t bytes=caifx_qlinear_workspace_bytes(n,OutputDim(),InputDim(),x_code,
                                                       CAIF_DataType(Base_t::ComputeDtype()).CaifxCode(),WeightKind(),
                                                       backward?1:0);
      if(bytes==0)
      {
        return CAIF_DeviceTensor();
      }
      return CAIF_DeviceTensor::Uninitialized({static_cast<uint32_t>(bytes)},Stream(),Dtype_e::UInt8);
    }
    void MigrateWeightToHost()
    {
      if(_weight.IsAllocated()==false)
      {
        _is_prefetched=false;
        return;
      }
      FreeHostWeight();
      _host_bytes=_weight.SizeBytes();
      _host_shape=_weight.Shape();
      _host_dtype=_weight.Dtype();
      if(hipHostMalloc(&_host_weight,_host_bytes,hipHostMallocDefault)!=hipSuccess)
      {
        THROW_CAIFE("FrozenLinear: pinned host allocation failed");
      }
      _weight.CopyToHostRaw(_host_weight);
      _weight=CAIF_DeviceTensor();
      _is_prefetched=false;
    }
    void Upload(CAIF_CudaStream &stream)
    {
      _weight=CAIF_DeviceTensor::Uninitialized(_host_shape,stream,_host_dtype);
      if(hipMemcpyAsync(_weight.DeviceDataRaw(),_host_weight,_host_bytes,hipMemcpyHostToDevice,stream.Handle())!=hipSuccess)
      {
        THROW_CAIFE("FrozenLinear::Prefetch: upload failed");
      }
    }
    void FreeHostWeight()
    {
      if(_host_weight!=nullptr)
      {
        (void)hipHostFree(_host_weight);
        _host_weight=nullptr;
      }
    }

    uint32_t _input_dim;
    uint32_t _output_dim;
    CAIF_Ops::QuantScheme_e _int8_scheme;
    uint32_t _group_size;
    CAIF_DeviceTensor _weight;
    CAIF_DeviceTensor _scales;
    bool _cache_fp32;
    bool _trained_forward;
    CAIF_OffloadPolicy::CAIF_OffloadPolicy_e _offload_policy;
    void *_host_weight;
    size_t _host_bytes;
    std::vector<uint32_t> _host_shape;
    Dtype_e _host_dtype=Dtype_e::Int8;
    bool _is_prefetched;
};

}//end instance namespace
