// CAIF_DeviceMoEFrozenExpert<ComputeT,StorageT>: a frozen (gated) FFN expert over three frozen
// linears, and CAIF_DeviceMoEFrozenExpertBank, the same arithmetic for ALL experts of a layer in
// a handful of grouped launches.
//
// The expert follows src/caif_device_moe_frozen_expert.cpp:92-332 step for step, including where
// a tensor is rounded to StorageT: every frozen linear returns fp32 and is cast to StorageT
// (:117-126,:131-141,:171-176); hidden = SiLU(gate_out) * up_out with both element-wise ops
// rounding to StorageT (:148-153); backward as :252-316.  ForwardInto writes into a caller-owned
// [tokens, InputDim] slice of StorageT (include/caif/caif_device_moe_expert_base.h:75-86).
//
// The bank replaces the per-expert host loop of CAIF_DeviceMoELayer
// (src/caif_device_moe_layer.cpp:534-557 forward, :754-778 backward): it takes the token-sorted
// packed buffer and the int32 expert_offsets[E+1] that MoEDispatchGPU / MoEBuildDispatchMap
// produce and runs gate, up and down for every expert as one grouped dequant-GEMM each, with the
// casts to StorageT folded into the GEMM stores.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "caif_device_frozen_linear.h"
#include "caif_device_layer.h"
#include "caif_ops.h"

namespace instance
{

class CAIF_DeviceMoEFrozenExpertConfig
{
  public:
    CAIF_DeviceMoEFrozenExpertConfig(uint32_t input_dim,uint32_t hidden_dim,bool use_gated)
      :_input_dim(input_dim),_hidden_dim(hidden_dim),_use_gated(use_gated){}
    uint32_t InputDim()const{return _input_dim;}
    uint32_t HiddenDim()const{return _hidden_dim;}
    bool UseGated()const{return _use_gated;}

  private:
    uint32_t _input_dim;
    uint32_t _hidden_dim;
    bool _use_gated;
};

template<typename ComputeT,typename StorageT>
class CAIF_DeviceMoEFrozenExpert:public CAIF_DeviceLayerTyped<ComputeT,StorageT>
{
  public:
    typedef CAIF_DeviceLayerTyped<ComputeT,StorageT> Base_t;
    typedef CAIF_DataType::CAIF_DataType_e Dtype_e;
    using Base_t::Stream;
    using Base_t::StorageDtype;

    struct FrozenSubLayers_t
    {
      std::unique_ptr<CAIF_DeviceFrozenLinearBase> gate;
      std::unique_ptr<CAIF_DeviceFrozenLinearBase> up;
      std::unique_ptr<CAIF_DeviceFrozenLinearBase> down;
    };

    CAIF_DeviceMoEFrozenExpert(const CAIF_DeviceMoEFrozenExpertConfig &config,FrozenSubLayers_t sub_layers,
                               CAIF_CudaStream &stream)
      :Base_t(stream),_config(config),_sub(std::move(sub_layers))
    {
      try
      {
        if(config.InputDim()==0){THROW_CAIFE("MoEFrozenExpert: input_dim must be > 0");}
        if(config.HiddenDim()==0){THROW_CAIFE("MoEFrozenExpert: hidden_dim must be > 0");}
        if(_sub.up==nullptr){THROW_CAIFE("MoEFrozenExpert: up sub-layer required");}
        if(_sub.down==nullptr){THROW_CAIFE("MoEFrozenExpert: down sub-layer required");}
        if(config.UseGated()==true&&_sub.gate==nullptr){THROW_CAIFE("MoEFrozenExpert: gated config requires gate sub-layer");}
      }
      CAIF_CATCH_BLOCK()
    }

    const CAIF_DeviceMoEFrozenExpertConfig &Config()const{return _config;}
    const FrozenSubLayers_t &SubLayers()const{return _sub;}

    CAIF_DeviceTensor ForwardImpl(const CAIF_DeviceTensor &input,CAIF_RunContext &ctx)override
    {
      try
      {
        const auto &shape=input.Shape();
        if(shape.size()!=2||shape[1]!=_config.InputDim()){THROW_CAIFE("MoEFrozenExpert::Forward: expected [N, input_dim]");}
        const uint32_t tokens=shape[0];
        const Dtype_e sd=StorageDtype();
        CAIF_DeviceTensor up_out=AsStorage(Layer(_sub.up)->Forward(input,ctx));
        CAIF_DeviceTensor hidden=CAIF_DeviceTensor::Uninitialized({tokens,_config.HiddenDim()},Stream(),sd);
        if(_config.UseGated()==true)
        {
          CAIF_DeviceTensor gate_out=AsStorage(Layer(_sub.gate)->Forward(input,ctx));
          CAIF_DeviceTensor gate_act=CAIF_DeviceTensor::Uninitialized({tokens,_config.HiddenDim()},Stream(),sd);
          CAIF_Ops::SiLU(gate_out,gate_act);
          CAIF_Ops::Multiply(gate_act,up_out,hidden);
          if(ctx.Training()==true)
          {
            _cached_gate_out=std::move(gate_out);
          }
        }
        else
        {
          CAIF_Ops::SiLU(up_out,hidden);
        }
        if(ctx.Training()==true)
        {
          _cached_up_out=std::move(up_out);
          _trained_tokens=tokens;
          _trained=true;
        }
        return AsStorage(Layer(_sub.down)->Forward(hidden,ctx));
      }
      CAIF_CATCH_BLOCK()
    }

    void ForwardInto(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output,CAIF_RunContext &ctx)
    {
      try
      {
        const auto &os=output.Shape();
        if(os.size()!=2||os[0]!=input.Shape()[0]||os[1]!=_config.InputDim())
        {
          THROW_CAIFE("MoEFrozenExpert::ForwardInto: output shape must be [N, input_dim]");
        }
        if(output.Dtype()!=StorageDtype()){THROW_CAIFE("MoEFrozenExpert::ForwardInto: output dtype must match StorageDtype()");}
        CAIF_DeviceTensor produced=ForwardImpl(input,ctx);
        if(hipMemcpyAsync(output.DeviceDataRaw(),produced.DeviceDataRaw(),output.SizeBytes(),hipMemcpyDeviceToDevice,
                          Stream().Handle())!=hipSuccess)
        {
          THROW_CAIFE("MoEFrozenExpert::ForwardInto: copy failed");
        }
      }
      CAIF_CATCH_BLOCK()
    }

    CAIF_DeviceTensor BackwardImpl(const CAIF_DeviceTensor &grad_output,CAIF_RunContext &ctx)override
    {
      try
      {
        if(_trained==false){THROW_CAIFE("MoEFrozenExpert::Backward: must call Forward(training=true) first");}
        const uint32_t tokens=_trained_tokens;
        const Dtype_e sd=StorageDtype();
        const std::vector<uint32_t> hshape={tokens,_config.HiddenDim()};
        CAIF_DeviceTensor grad_hidden=AsStorage(Layer(_sub.down)->Backward(grad_output,ctx));
        if(_config.UseGated()==false)
        {
          CAIF_DeviceTensor grad_up=CAIF_DeviceTensor::Uninitialized(hshape,Stream(),sd);
          CAIF_Ops::SiLUBackward(_cached_up_out,grad_hidden,grad_up);
          return AsStorage(Layer(_sub.up)->Backward(grad_up,ctx));
        }
        // grad_up = grad_hidden * silu(gate_out); grad_gate = SiLUBackward(gate_out, grad_hidden * up_out):
        // the reference's four launches in one, same bits
        CAIF_DeviceTensor grad_up=CAIF_DeviceTensor::Uninitialized(hshape,Stream(),sd);
        CAIF_DeviceTensor grad_gate=CAIF_DeviceTensor::Uninitialized(hshape,Stream(),sd);
        CAIF_Ops::SwiGLUBackward(_cached_gate_out,_cached_up_out,grad_hidden,grad_gate,grad_up);
        CAIF_DeviceTensor gi_up=AsStorage(Layer(_sub.up)->Backward(grad_up,ctx));
        CAIF_DeviceTensor gi_gate=AsStorage(Layer(_sub.gate)->Backward(grad_gate,ctx));
        CAIF_DeviceTensor grad_input=CAIF_DeviceTensor::Uninitialized({tokens,_config.InputDim()},Stream(),sd);
        CAIF_Ops::Add(gi_up,gi_gate,grad_input);
        return grad_input;
      }
      CAIF_CATCH_BLOCK()
    }

    void ZeroGradients()override{}
    size_t ParameterTensorCount()const override{return 0;}
    CAIF_DeviceTensor &ParameterTensor(size_t)override{THROW_CAIFE("MoEFrozenExpert: no trainable parameters");}
    CAIF_DeviceTensor &GradientTensor(size_t)override{THROW_CAIFE("MoEFrozenExpert: no trainable parameters / gradients");}
    size_t TotalParameterCount()const override{return 0;}
    std::string Description()const override
    {
      return std::string("CAIF_DeviceMoEFrozenExpert(input_dim=")+std::to_string(_config.InputDim())+",hidden_dim="+
             std::to_string(_config.HiddenDim())+",use_gated="+(_config.UseGated()?"true":"false")+",frozen=true)";
    }
    std::vector<std::string> ParameterNames(const std::string &)const override{return {};}

  private:
    static CAIF_DeviceLayer *Layer(const std::unique_ptr<CAIF_DeviceFrozenLinearBase> &p)
    {
      CAIF_DeviceLayer *l=dynamic_cast<CAIF_DeviceLayer*>(p.get());
      if(l==nullptr){THROW_CAIFE("MoEFrozenExpert: sub-layer is not a CAIF_DeviceLayer");}
      return l;
    }
    CAIF_DeviceTensor AsStorage(CAIF_DeviceTensor t)const
    {
      if(t.Dtype()==StorageDtype())
      {
        return t;
      }
      return t.To(StorageDtype());
    }

    CAIF_DeviceMoEFrozenExpertConfig _config;
    FrozenSubLayers_t _sub;
    CAIF_DeviceTensor _cached_gate_out;
    CAIF_DeviceTensor _cached_up_out;
    uint32_t _trained_tokens=0;
    bool _trained=false;
};

// All frozen experts of one MoE layer, run as grouped launches over the token-sorted buffer.
// Sub-layers are borrowed from the experts (same weights, nothing is copied); they must all be
// frozen linears of one ComputeT with the same storage kind, scheme and group size.
template<typename ComputeT,typename StorageT>
class CAIF_DeviceMoEFrozenExpertBank
{
  public:
    typedef CAIF_DataType::CAIF_DataType_e Dtype_e;
    typedef CAIF_DeviceMoEFrozenExpert<ComputeT,StorageT> Expert_t;

    CAIF_DeviceMoEFrozenExpertBank(const std::vector<Expert_t*> &experts,CAIF_CudaStream &stream):_stream(&stream)
    {
      try
      {
        if(experts.empty()==true){THROW_CAIFE("MoEFrozenExpertBank: no experts");}
        _input_dim=experts[0]->Config().InputDim();
        _hidden_dim=experts[0]->Config().HiddenDim();
        _num_experts=static_cast<int>(experts.size());
        for(int which=0;which<3;++which)
        {
          for(Expert_t *e:experts)
          {
            if(e->Config().UseGated()==false){THROW_CAIFE("MoEFrozenExpertBank: experts must be gated");}
            const auto &sub=e->SubLayers();
            _subs[which].push_back(which==0?sub.gate.get():(which==1?sub.up.get():sub.down.get()));
          }
        }
        Refresh();
      }
      CAIF_CATCH_BLOCK()
    }

    // x: packed [total_rows, InputDim] of StorageT; offsets: device int32 [E+1].  Returns the expert
    // outputs [total_rows, InputDim] of StorageT; keeps gate_out / up_out when training.
    CAIF_DeviceTensor Forward(const CAIF_DeviceTensor &x,const CAIF_DeviceTensor &offsets,bool training)
    {
      try
      {
        Refresh();
        const uint32_t rows=x.Shape()[0];
        const Dtype_e sd=CAIF_DtypeOf<StorageT>::value;
        CAIF_DeviceTensor up_out=CAIF_DeviceTensor::Zeros({rows,_hidden_dim},*_stream,sd);
        CAIF_DeviceTensor gate_out=CAIF_DeviceTensor::Zeros({rows,_hidden_dim},*_stream,sd);
        Grouped(false,1,x,offsets,up_out,_hidden_dim,_input_dim);
        Grouped(false,0,x,offsets,gate_out,_hidden_dim,_input_dim);
        CAIF_DeviceTensor hidden=CAIF_DeviceTensor::Uninitialized({rows,_hidden_dim},*_stream,sd);
        CAIF_Ops::Check(caifx_silu_multiply(gate_out.DeviceDataRaw(),up_out.DeviceDataRaw(),hidden.DeviceDataRaw(),
                                            static_cast<int64_t>(rows)*_hidden_dim,CAIF_DataType(sd).CaifxCode(),
                                            _stream->Handle()),"MoEFrozenExpertBank: silu*up");
        CAIF_DeviceTensor out=CAIF_DeviceTensor::Zeros({rows,_input_dim},*_stream,sd);
        Grouped(false,2,hidden,offsets,out,_input_dim,_hidden_dim);
        if(training==true)
        {
          _gate_out=std::move(gate_out);
          _up_out=std::move(up_out);
        }
        return out;
      }
      CAIF_CATCH_BLOCK()
    }

    CAIF_DeviceTensor Backward(const CAIF_DeviceTensor &grad_out,const CAIF_DeviceTensor &offsets)
    {
      try
      {
        if(_gate_out.IsEmpty()==true){THROW_CAIFE("MoEFrozenExpertBank::Backward: must call Forward(training=true) first");}
        Refresh();
        const uint32_t rows=grad_out.Shape()[0];
        const Dtype_e sd=CAIF_DtypeOf<StorageT>::value;
        const std::vector<uint32_t> hs={rows,_hidden_dim};
        CAIF_DeviceTensor grad_hidden=CAIF_DeviceTensor::Zeros(hs,*_stream,sd);
        Grouped(true,2,grad_out,offsets,grad_hidden,_input_dim,_hidden_dim);
        // the four element-wise launches of the gated backward in one, and gi_up + gi_gate folded into the second
        // input-gradient GEMM's store: same bits as the reference's sequence
        CAIF_DeviceTensor grad_up=CAIF_DeviceTensor::Uninitialized(hs,*_stream,sd);
        CAIF_DeviceTensor grad_gate=CAIF_DeviceTensor::Uninitialized(hs,*_stream,sd);
        CAIF_Ops::SwiGLUBackward(_gate_out,_up_out,grad_hidden,grad_gate,grad_up);
        CAIF_DeviceTensor gi_up=CAIF_DeviceTensor::Zeros({rows,_input_dim},*_stream,sd);
        Grouped(true,1,grad_up,offsets,gi_up,_hidden_dim,_input_dim);
        CAIF_DeviceTensor grad_in=CAIF_DeviceTensor::Zeros({rows,_input_dim},*_stream,sd);
        if(Grouped(true,0,grad_gate,offsets,grad_in,_hidden_dim,_input_dim,&gi_up)==false)
        {
          // shapes the matrix-core kernel does not take: plain call, then the Add
          CAIF_DeviceTensor gi_gate=CAIF_DeviceTensor::Zeros({rows,_input_dim},*_stream,sd);
          Grouped(true,0,grad_gate,offsets,gi_gate,_hidden_dim,_input_dim);
          CAIF_Ops::Add(gi_up,gi_gate,grad_in);
        }
        return grad_in;
      }
      CAIF_CATCH_BLOCK()
    }

  private:
    struct Kind_t{int kind=-1;int64_t period=1;int group=0;uint32_t in=0;uint32_t out=0;};

    // The grouped launches read the experts' weights through device arrays of device addresses.  A sub-layer
    // under the HostPinned offload policy frees its device copy in Evict() and gets a new one, at a new address,
    // in Prefetch() (src/caif_device_frozen_linear.cpp:145-232), so the addresses are gathered again before every
    // pass and uploaded when any of them has moved; an expert that is not resident throws like the layer's own
    // Forward does (:391-396).
    void Refresh()
    {
      for(int which=0;which<3;++which)
      {
        std::vector<const void*> w,s;
        for(const CAIF_DeviceFrozenLinearBase *b:_subs[which])
        {
          Describe(b,which,w,s);
        }
        if(w!=_host_wq[which])
        {
          Upload(w,_wq_ptrs[which]);
          _host_wq[which]=w;
        }
        if(s!=_host_scales[which])
        {
          Upload(s,_scale_ptrs[which]);
          _host_scales[which]=s;
        }
      }
    }

    void Describe(const CAIF_DeviceFrozenLinearBase *b,int which,std::vector<const void*> &w,std::vector<const void*> &s)
    {
      const void *wq=nullptr;
      const void *sc=nullptr;
      Kind_t k;
      if(const auto *l8=dynamic_cast<const CAIF_DeviceFrozenLinear<ComputeT,int8_t>*>(b))
      {
        wq=l8->WeightData();sc=l8->ScalesData();
        k.kind=l8->WeightKind();k.period=l8->ScalePeriod();k.group=static_cast<int>(l8->GroupSize());
        k.in=l8->InputDim();k.out=l8->OutputDim();
      }
      else if(const auto *l4=dynamic_cast<const CAIF_DeviceFrozenLinear<ComputeT,caif_int4_packed_t>*>(b))
      {
        wq=l4->WeightData();sc=l4->ScalesData();
        k.kind=l4->WeightKind();k.period=l4->ScalePeriod();k.group=static_cast<int>(l4->GroupSize());
        k.in=l4->InputDim();k.out=l4->OutputDim();
      }
      else
      {
        THROW_CAIFE("MoEFrozenExpertBank: sub-layer must be an int8 or int4 frozen linear of the bank's ComputeT");
      }
      if(b->OffloadPolicy()==CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e&&b->IsPrefetched()==false)
      {
        THROW_CAIFE("MoEFrozenExpertBank: an expert's weight is not on the device (HostPinned policy)."
                    " The block-level scheduler must call Prefetch(stream) before the bank runs.");
      }
      if(wq==nullptr){THROW_CAIFE("MoEFrozenExpertBank: sub-layer weight not loaded");}
      if(w.empty()==true)
      {
        _kinds[which]=k;
      }
      else if(_kinds[which].kind!=k.kind||_kinds[which].period!=k.period||_kinds[which].group!=k.group||
              _kinds[which].in!=k.in||_kinds[which].out!=k.out||(sc==nullptr)!=(s[0]==nullptr))
      {
        THROW_CAIFE("MoEFrozenExpertBank: experts must share storage kind, scheme, group size and dims");
      }
      w.push_back(wq);
      s.push_back(sc);
    }
    void Upload(const std::vector<const void*> &host,CAIF_DeviceTensor &dev)
    {
      if(host[0]==nullptr)
      {
        return;     // int8 without scales: the grouped call takes a null scales array
      }
      dev=CAIF_DeviceTensor::Uninitialized({static_cast<uint32_t>(host.size()*sizeof(void*))},*_stream,Dtype_e::UInt8);
      dev.CopyFromHostRaw(host.data(),host.size()*sizeof(void*));
    }
    // which: 0 gate, 1 up, 2 down.  N/K are the frozen linear's OutputDim/InputDim.
    // addend (backward only): out = T(T(in * W_e) + addend) in the store; returns false when that form is not
    // available for the shape (nothing has been launched then)
    bool Grouped(bool backward,int which,const CAIF_DeviceTensor &in,const CAIF_DeviceTensor &offsets,CAIF_DeviceTensor &out,
                 uint32_t N,uint32_t K,const CAIF_DeviceTensor *addend=nullptr)
    {
      const Kind_t &k=_kinds[which];
      const int code=CAIF_DataType(CAIF_DtypeOf<StorageT>::value).CaifxCode();
      const int cc=CAIF_DataType(CAIF_DtypeOf<ComputeT>::value).CaifxCode();
      const void *const *wp=static_cast<const void *const *>(_wq_ptrs[which].DeviceDataRaw());
      const void *const *sp=_scale_ptrs[which].IsEmpty()?nullptr:static_cast<const void *const *>(_scale_ptrs[which].DeviceDataRaw());
      const int64_t rows=in.Shape()[0];
      const int32_t *off=static_cast<const int32_t*>(offsets.DeviceDataRaw());
      int st;
      if(backward==true&&addend!=nullptr)
      {
        st=caifx_qlinear_grouped_backward_input_add(_num_experts,off,rows,N,K,in.DeviceDataRaw(),code,cc,wp,k.kind,sp,k.period,
                                                    k.group,out.DeviceDataRaw(),code,addend->DeviceDataRaw(),nullptr,0,
                                                    _stream->Handle());
        if(st==CAIFX_ERR_UNSUPPORTED)
        {
          return false;
        }
      }
      else if(backward==true)
      {
        st=caifx_qlinear_grouped_backward_input(_num_experts,off,rows,N,K,in.DeviceDataRaw(),code,cc,wp,k.kind,sp,k.period,
                                                k.group,out.DeviceDataRaw(),code,nullptr,0,_stream->Handle());
      }
      else
      {
        st=caifx_qlinear_grouped_forward(_num_experts,off,rows,N,K,in.DeviceDataRaw(),code,cc,wp,k.kind,sp,k.period,k.group,
                                         out.DeviceDataRaw(),code,nullptr,0,_stream->Handle());
      }
      CAIF_Ops::Check(st,"MoEFrozenExpertBank: grouped dequant-GEMM");
      return true;
    }

    CAIF_CudaStream *_stream;
    uint32_t _input_dim=0;
    uint32_t _hidden_dim=0;
    int _num_experts=0;
    Kind_t _kinds[3];
    std::vector<const CAIF_DeviceFrozenLinearBase*> _subs[3];      // borrowed: gate, up, down of every expert
    std::vector<const void*> _host_wq[3];                          // what _wq_ptrs / _scale_ptrs hold right now
    std::vector<const void*> _host_scales[3];
    CAIF_DeviceTensor _wq_ptrs[3];
    CAIF_DeviceTensor _scale_ptrs[3];
    CAIF_DeviceTensor _gate_out;
    CAIF_DeviceTensor _up_out;
};

}//end instance namespace
