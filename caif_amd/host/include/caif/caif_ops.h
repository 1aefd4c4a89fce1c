// CAIF_Ops: the quantise / dequantise entry points and the element-wise ops the frozen experts
// use, with the reference's signatures (include/caif/caif_ops.h:365-446) and validation order
// (src/caif_ops.cpp:504-680 dispatch, src/caif_ops_device.cpp:1517-1743 checks).  Each validated
// call lands in one C-ABI launcher of caifx.h; a non-zero status becomes a CAIF_Exception.
#pragma once

#include <cstdint>
#include <string>

#include "caif_device_tensor.h"
#include "caif_run_context.h"
#include "caifx.h"

namespace instance
{

class CAIF_Ops
{
  public:
    typedef CAIF_DataType::CAIF_DataType_e Dtype_e;
    enum class QuantScheme_e:uint8_t{PerTensor_e,PerChannel_e};

    static void QuantizeInt8(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output,CAIF_DeviceTensor &scales,
                             QuantScheme_e scheme,CAIF_RunContext &ctx)
    {
      try
      {
        (void)ctx;
        RequireDevice(input,"QuantizeInt8");
        if(input.Dtype()!=Dtype_e::Float32){THROW_CAIFE("QuantizeInt8: input must be fp32");}
        if(output.Dtype()!=Dtype_e::Int8){THROW_CAIFE("QuantizeInt8: output must be Int8");}
        if(scales.Dtype()!=Dtype_e::Float32){THROW_CAIFE("QuantizeInt8: scales must be fp32");}
        if(input.Shape()!=output.Shape()){THROW_CAIFE("QuantizeInt8: input/output shape mismatch");}
        hipStream_t stream=output.StreamHandle();
        const int64_t n=static_cast<int64_t>(input.TotalElements());
        if(scheme==QuantScheme_e::PerTensor_e)
        {
          if(scales.TotalElements()!=1){THROW_CAIFE("QuantizeInt8 PerTensor: scales must have 1 element");}
          Check(caifx_quantize_int8_per_tensor(input.DevicePtr<float>(),output.DeviceDataRaw(),scales.DeviceDataRaw(),n,
                                               stream),"QuantizeInt8");
          return;
        }
        if(input.Shape().size()!=2){THROW_CAIFE("QuantizeInt8 PerChannel: input must be 2D");}
        const int rows=static_cast<int>(input.Shape()[0]);
        const int cols=static_cast<int>(input.Shape()[1]);
        if(scales.TotalElements()!=static_cast<size_t>(cols))
        {
          THROW_CAIFE("QuantizeInt8 PerChannel: scales length must equal cols");
        }
        Check(caifx_quantize_int8_per_channel(input.DevicePtr<float>(),output.DeviceDataRaw(),scales.DeviceDataRaw(),
                                              rows,cols,stream),"QuantizeInt8");
      }
      CAIF_CATCH_BLOCK()
    }

    static void DequantizeInt8(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output,const CAIF_DeviceTensor &scales,
                               QuantScheme_e scheme,CAIF_RunContext &ctx)
    {
      try
      {
        (void)ctx;
        RequireDevice(input,"DequantizeInt8");
        if(input.Dtype()!=Dtype_e::Int8){THROW_CAIFE("DequantizeInt8: input must be Int8");}
        if(output.Dtype()!=Dtype_e::Float32){THROW_CAIFE("DequantizeInt8: output must be fp32");}
        if(scales.Dtype()!=Dtype_e::Float32){THROW_CAIFE("DequantizeInt8: scales must be fp32");}
        if(input.Shape()!=output.Shape()){THROW_CAIFE("DequantizeInt8: input/output shape mismatch");}
        hipStream_t stream=output.StreamHandle();
        const int64_t n=static_cast<int64_t>(input.TotalElements());
        if(scheme==QuantScheme_e::PerTensor_e)
        {
          if(scales.TotalElements()!=1){THROW_CAIFE("DequantizeInt8 PerTensor: scales must have 1 element");}
          Check(caifx_dequantize_int8_per_tensor(input.DeviceDataRaw(),output.DevicePtr<float>(),scales.DeviceDataRaw(),n,
                                                 stream),"DequantizeInt8");
          return;
        }
        if(input.Shape().size()!=2){THROW_CAIFE("DequantizeInt8 PerChannel: input must be 2D");}
        const int rows=static_cast<int>(input.Shape()[0]);
        const int cols=static_cast<int>(input.Shape()[1]);
        if(scales.TotalElements()!=static_cast<size_t>(cols))
        {
          THROW_CAIFE("DequantizeInt8 PerChannel: scales length must equal cols");
        }
        Check(caifx_dequantize_int8_per_channel(input.DeviceDataRaw(),output.DevicePtr<float>(),scales.DeviceDataRaw(),
                                                rows,cols,stream),"DequantizeInt8");
      }
      CAIF_CATCH_BLOCK()
    }

    static void QuantizeInt4PerGroup(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output,CAIF_DeviceTensor &scales,
                                     uint32_t group_size,CAIF_RunContext &ctx)
    {
      try
      {
        (void)ctx;
        RequireDevice(input,"QuantizeInt4PerGroup");
        if(input.Dtype()!=Dtype_e::Float32){THROW_CAIFE("QuantizeInt4PerGroup: input must be fp32");}
        if(output.Dtype()!=Dtype_e::Int4){THROW_CAIFE("QuantizeInt4PerGroup: output must be Int4");}
        if(scales.Dtype()!=Dtype_e::Float16){THROW_CAIFE("QuantizeInt4PerGroup: scales must be fp16");}
        if(group_size==0){THROW_CAIFE("QuantizeInt4PerGroup: group_size must be > 0");}
        const int64_t n=static_cast<int64_t>(input.TotalElements());
        const size_t num_groups=(static_cast<size_t>(n)+group_size-1)/group_size;
        if(scales.TotalElements()!=num_groups){THROW_CAIFE("QuantizeInt4PerGroup: scales length must equal num_groups");}
        Check(caifx_quantize_to_int4(input.DevicePtr<float>(),output.DeviceDataRaw(),scales.DeviceDataRaw(),n,
                                     static_cast<int>(group_size),output.StreamHandle()),"QuantizeInt4PerGroup");
      }
      CAIF_CATCH_BLOCK()
    }

    static void DequantizeInt4PerGroup(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output,
                                       const CAIF_DeviceTensor &scales,uint32_t group_size,CAIF_RunContext &ctx)
    {
      try
      {
        (void)ctx;
        RequireDevice(input,"DequantizeInt4PerGroup");
        if(input.Dtype()!=Dtype_e::Int4){THROW_CAIFE("DequantizeInt4PerGroup: input must be Int4");}
        if(output.Dtype()!=Dtype_e::Float32){THROW_CAIFE("DequantizeInt4PerGroup: output must be fp32");}
        if(scales.Dtype()!=Dtype_e::Float16){THROW_CAIFE("DequantizeInt4PerGroup: scales must be fp16");}
        if(group_size==0){THROW_CAIFE("DequantizeInt4PerGroup: group_size must be > 0");}
        const int64_t n=static_cast<int64_t>(output.TotalElements());
        const size_t num_groups=(static_cast<size_t>(n)+group_size-1)/group_size;
        if(scales.TotalElements()!=num_groups){THROW_CAIFE("DequantizeInt4PerGroup: scales length must equal num_groups");}
        Check(caifx_dequantize_int4(input.DeviceDataRaw(),scales.DeviceDataRaw(),output.DevicePtr<float>(),n,
                                    static_cast<int>(group_size),output.StreamHandle()),"DequantizeInt4PerGroup");
      }
      CAIF_CATCH_BLOCK()
    }

    // QAT fake quantisation: quantise then dequantise, scratch discarded (include/caif/caif_ops.h:430-446).
    static void FakeQuantInt8(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output,QuantScheme_e scheme,
                              CAIF_RunContext &ctx)
    {
      try
      {
        const CAIF_CudaStream view=CAIF_CudaStream::Wrap(output.StreamHandle());
        CAIF_DeviceTensor q=CAIF_DeviceTensor::Uninitialized(input.Shape(),view,Dtype_e::Int8);
        uint32_t ns=1;
        if(scheme==QuantScheme_e::PerChannel_e)
        {
          if(input.Shape().size()!=2){THROW_CAIFE("FakeQuantInt8 PerChannel: input must be 2D");}
          ns=input.Shape()[1];
        }
        CAIF_DeviceTensor s=CAIF_DeviceTensor::Uninitialized({ns},view,Dtype_e::Float32);
        QuantizeInt8(input,q,s,scheme,ctx);
        DequantizeInt8(q,output,s,scheme,ctx);
      }
      CAIF_CATCH_BLOCK()
    }
    static void FakeQuantInt4PerGroup(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output,uint32_t group_size,
                                      CAIF_RunContext &ctx)
    {
      try
      {
        if(group_size==0){THROW_CAIFE("FakeQuantInt4PerGroup: group_size must be > 0");}
        const CAIF_CudaStream view=CAIF_CudaStream::Wrap(output.StreamHandle());
        const uint32_t n=static_cast<uint32_t>(input.TotalElements());
        CAIF_DeviceTensor q=CAIF_DeviceTensor::Uninitialized({n},view,Dtype_e::Int4);
        CAIF_DeviceTensor s=CAIF_DeviceTensor::Uninitialized({(n+group_size-1)/group_size},view,Dtype_e::Float16);
        QuantizeInt4PerGroup(input,q,s,group_size,ctx);
        DequantizeInt4PerGroup(q,output,s,group_size,ctx);
      }
      CAIF_CATCH_BLOCK()
    }

    // Element-wise ops between the expert GEMMs; operands share dtype and element count.
    static void SiLU(const CAIF_DeviceTensor &input,CAIF_DeviceTensor &output)
    {
      try
      {
        SameKind(input,output,"SiLU");
        Check(caifx_silu(input.DeviceDataRaw(),output.DeviceDataRaw(),static_cast<int64_t>(input.TotalElements()),
                         CAIF_DataType(input.Dtype()).CaifxCode(),output.StreamHandle()),"SiLU");
      }
      CAIF_CATCH_BLOCK()
    }
    static void SiLUBackward(const CAIF_DeviceTensor &input,const CAIF_DeviceTensor &grad_output,
                             CAIF_DeviceTensor &grad_input)
    {
      try
      {
        SameKind(input,grad_output,"SiLUBackward");
        SameKind(input,grad_input,"SiLUBackward");
        Check(caifx_silu_backward(input.DeviceDataRaw(),grad_output.DeviceDataRaw(),grad_input.DeviceDataRaw(),
                                  static_cast<int64_t>(input.TotalElements()),CAIF_DataType(input.Dtype()).CaifxCode(),
                                  grad_input.StreamHandle()),"SiLUBackward");
      }
      CAIF_CATCH_BLOCK()
    }
    static void Multiply(const CAIF_DeviceTensor &a,const CAIF_DeviceTensor &b,CAIF_DeviceTensor &output)
    {
      try
      {
        SameKind(a,b,"Multiply");
        SameKind(a,output,"Multiply");
        Check(caifx_multiply(a.DeviceDataRaw(),b.DeviceDataRaw(),output.DeviceDataRaw(),
                             static_cast<int64_t>(a.TotalElements()),CAIF_DataType(a.Dtype()).CaifxCode(),
                             output.StreamHandle()),"Multiply");
      }
      CAIF_CATCH_BLOCK()
    }
    static void Add(const CAIF_DeviceTensor &a,const CAIF_DeviceTensor &b,CAIF_DeviceTensor &output)
    {
      try
      {
        SameKind(a,b,"Add");
        SameKind(a,output,"Add");
        Check(caifx_add(a.DeviceDataRaw(),b.DeviceDataRaw(),output.DeviceDataRaw(),static_cast<int64_t>(a.TotalElements()),
                        CAIF_DataType(a.Dtype()).CaifxCode(),output.StreamHandle()),"Add");
      }
      CAIF_CATCH_BLOCK()
    }

    // Map a C-ABI status to the reference's error convention.
    static void Check(int status,const char *what)
    {
      if(status!=CAIFX_OK)
      {
        THROW_CAIFE(std::string(what)+": "+caifx_status_string(status));
      }
    }

  private:
    static void RequireDevice(const CAIF_DeviceTensor &t,const char *op)
    {
      if(t.Location()==CAIF_DeviceTensor::Location_e::Host_e)
      {
        THROW_CAIFE(std::string(op)+": host backend not supported");
      }
    }
    static void SameKind(const CAIF_DeviceTensor &a,const CAIF_DeviceTensor &b,const char *op)
    {
      if(a.Dtype()!=b.Dtype()||a.TotalElements()!=b.TotalElements())
      {
        THROW_CAIFE(std::string(op)+": operands must share dtype and element count");
      }
    }
};

}//end instance namespace
