// CAIF_Ops: the quantise / dequantise entry points and the element-wise ops the frozen experts
// use, with the reference's signatures (include/caif/caif_ops.h:365-446) and validation order
// (src/caif_ops.cpp:504-680 dispatch, src/caif_ops_device.cpp:1517-1743 checks).  Each validated
// call lands in one C-ABI launcher of caifx.h; a non-zero status becomes a CAIF_Exception.
#pragma once

#include <algorithm>
#include <cstdint>
#include <string>
#include <vector>

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
    // SiLU, Multiply, Multiply, SiLUBackward of the gated expert's backward pass in one launch; the bits equal
    // the four-op chain (every intermediate is rounded where those ops round)
    static void SwiGLUBackward(const CAIF_DeviceTensor &gate,const CAIF_DeviceTensor &up,const CAIF_DeviceTensor &grad_hidden,
                               CAIF_DeviceTensor &grad_gate,CAIF_DeviceTensor &grad_up)
    {
      try
      {
        SameKind(gate,up,"SwiGLUBackward");
        SameKind(gate,grad_hidden,"SwiGLUBackward");
        SameKind(gate,grad_gate,"SwiGLUBackward");
        SameKind(gate,grad_up,"SwiGLUBackward");
        Check(caifx_swiglu_backward(gate.DeviceDataRaw(),up.DeviceDataRaw(),grad_hidden.DeviceDataRaw(),
                                    grad_gate.DeviceDataRaw(),grad_up.DeviceDataRaw(),
                                    static_cast<int64_t>(gate.TotalElements()),CAIF_DataType(gate.Dtype()).CaifxCode(),
                                    grad_gate.StreamHandle()),"SwiGLUBackward");
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

    // ---- MoE token routing (include/caif/caif_ops.h:1234-1326 of the reference) ----------------------
    // expert_indices and dispatch_map hold int32 [num_tokens, top_k], expert_offsets int32 [num_experts+1].

    // Returns the number of assigned rows like the reference (src/caif_ops_device.cpp:4876-4960), which makes
    // this call synchronise the stream for one 4-byte copy; map and offsets themselves never leave the device.
    static uint32_t MoEBuildDispatchMap(const CAIF_DeviceTensor &expert_indices,uint32_t num_experts,uint32_t top_k,
                                        uint32_t capacity_per_expert,CAIF_DeviceTensor &dispatch_map,
                                        CAIF_DeviceTensor &expert_offsets)
    {
      try
      {
        RequireDevice(expert_indices,"MoEBuildDispatchMap");
        if(expert_indices.Shape().size()!=2)
        {
          THROW_CAIFE("MoEBuildDispatchMap: expert_indices must be 2D [num_tokens x top_k]");
        }
        if(!FourByte(expert_indices)||!FourByte(dispatch_map)||!FourByte(expert_offsets))
        {
          THROW_CAIFE("MoEBuildDispatchMap: indices, map and offsets must hold 32-bit integers");
        }
        const uint32_t num_tokens=expert_indices.Shape()[0];
        if(expert_indices.Shape()[1]!=top_k||dispatch_map.TotalElements()!=expert_indices.TotalElements()||
           expert_offsets.TotalElements()!=static_cast<size_t>(num_experts)+1)
        {
          THROW_CAIFE("MoEBuildDispatchMap: shape mismatch");
        }
        const size_t ws_bytes=std::max<size_t>(caifx_moe_dispatch_map_workspace_bytes(num_tokens,static_cast<int>(top_k),
                                                                                      static_cast<int>(num_experts)),
                                               static_cast<size_t>(num_experts)*4);
        CAIF_DeviceTensor ws=CAIF_DeviceTensor::Uninitialized({static_cast<uint32_t>(ws_bytes)},
                                                              CAIF_CudaStream::Wrap(expert_offsets.StreamHandle()),
                                                              Dtype_e::UInt8);
        Check(caifx_moe_build_dispatch_map(static_cast<const int32_t*>(expert_indices.DeviceDataRaw()),num_tokens,
                                           static_cast<int>(top_k),static_cast<int>(num_experts),
                                           static_cast<int>(capacity_per_expert),
                                           static_cast<int32_t*>(dispatch_map.DeviceDataRaw()),
                                           static_cast<int32_t*>(expert_offsets.DeviceDataRaw()),ws.DeviceDataRaw(),ws_bytes,
                                           expert_offsets.StreamHandle()),"MoEBuildDispatchMap");
        std::vector<int32_t> offsets(static_cast<size_t>(num_experts)+1);
        expert_offsets.CopyToHostRaw(offsets.data());
        return static_cast<uint32_t>(offsets[num_experts]);
      }
      CAIF_CATCH_BLOCK()
    }
    static void MoEDispatchGPU(const CAIF_DeviceTensor &input,const CAIF_DeviceTensor &expert_indices,
                               const CAIF_DeviceTensor &dispatch_map,const CAIF_DeviceTensor &expert_offsets,uint32_t top_k,
                               CAIF_DeviceTensor &expert_buffer)
    {
      try
      {
        RouteShapes(input,expert_indices,dispatch_map,expert_offsets,top_k,expert_buffer,"MoEDispatchGPU");
        Check(caifx_moe_dispatch(input.DeviceDataRaw(),Idx(expert_indices),Idx(dispatch_map),Idx(expert_offsets),
                                 expert_buffer.DeviceDataRaw(),input.Shape()[0],input.Shape()[1],static_cast<int>(top_k),
                                 Experts(expert_offsets),CAIF_DataType(input.Dtype()).CaifxCode(),expert_buffer.StreamHandle()),
              "MoEDispatchGPU");
      }
      CAIF_CATCH_BLOCK()
    }
    static void MoECombineGPU(const CAIF_DeviceTensor &expert_buffer,const CAIF_DeviceTensor &expert_indices,
                              const CAIF_DeviceTensor &expert_weights,const CAIF_DeviceTensor &dispatch_map,
                              const CAIF_DeviceTensor &expert_offsets,uint32_t top_k,CAIF_DeviceTensor &output)
    {
      try
      {
        RouteShapes(output,expert_indices,dispatch_map,expert_offsets,top_k,expert_buffer,"MoECombineGPU");
        RouteWeights(expert_weights,expert_indices,output,"MoECombineGPU");
        Check(caifx_moe_combine(expert_buffer.DeviceDataRaw(),Idx(expert_indices),expert_weights.DeviceDataRaw(),
                                Idx(dispatch_map),Idx(expert_offsets),output.DeviceDataRaw(),output.Shape()[0],
                                output.Shape()[1],static_cast<int>(top_k),Experts(expert_offsets),
                                CAIF_DataType(output.Dtype()).CaifxCode(),output.StreamHandle()),"MoECombineGPU");
      }
      CAIF_CATCH_BLOCK()
    }
    static void MoECombineBackwardGPU(const CAIF_DeviceTensor &grad_output,const CAIF_DeviceTensor &expert_buffer,
                                      const CAIF_DeviceTensor &expert_indices,const CAIF_DeviceTensor &expert_weights,
                                      const CAIF_DeviceTensor &dispatch_map,const CAIF_DeviceTensor &expert_offsets,
                                      uint32_t top_k,CAIF_DeviceTensor &grad_expert_buffer,CAIF_DeviceTensor &grad_weights)
    {
      try
      {
        RouteShapes(grad_output,expert_indices,dispatch_map,expert_offsets,top_k,grad_expert_buffer,"MoECombineBackwardGPU");
        RouteWeights(expert_weights,expert_indices,grad_output,"MoECombineBackwardGPU");
        RouteWeights(grad_weights,expert_indices,grad_output,"MoECombineBackwardGPU");
        SameKind(expert_buffer,grad_expert_buffer,"MoECombineBackwardGPU");
        const int code=CAIF_DataType(grad_output.Dtype()).CaifxCode();
        Check(caifx_moe_combine_backward_grad_expert(grad_output.DeviceDataRaw(),Idx(expert_indices),
                                                     expert_weights.DeviceDataRaw(),Idx(dispatch_map),Idx(expert_offsets),
                                                     grad_expert_buffer.DeviceDataRaw(),grad_output.Shape()[0],
                                                     grad_output.Shape()[1],static_cast<int>(top_k),Experts(expert_offsets),
                                                     code,grad_expert_buffer.StreamHandle()),"MoECombineBackwardGPU");
        Check(caifx_moe_combine_backward_grad_weights(grad_output.DeviceDataRaw(),expert_buffer.DeviceDataRaw(),
                                                      Idx(expert_indices),Idx(dispatch_map),Idx(expert_offsets),
                                                      grad_weights.DeviceDataRaw(),grad_output.Shape()[0],
                                                      grad_output.Shape()[1],static_cast<int>(top_k),Experts(expert_offsets),
                                                      code,grad_weights.StreamHandle()),"MoECombineBackwardGPU");
      }
      CAIF_CATCH_BLOCK()
    }
    static void MoEDispatchBackwardGPU(const CAIF_DeviceTensor &grad_expert_buffer,const CAIF_DeviceTensor &expert_indices,
                                       const CAIF_DeviceTensor &dispatch_map,const CAIF_DeviceTensor &expert_offsets,
                                       uint32_t top_k,CAIF_DeviceTensor &grad_input)
    {
      try
      {
        RouteShapes(grad_input,expert_indices,dispatch_map,expert_offsets,top_k,grad_expert_buffer,"MoEDispatchBackwardGPU");
        Check(caifx_moe_dispatch_backward(grad_expert_buffer.DeviceDataRaw(),Idx(expert_indices),Idx(dispatch_map),
                                          Idx(expert_offsets),grad_input.DeviceDataRaw(),grad_input.Shape()[0],
                                          grad_input.Shape()[1],static_cast<int>(top_k),Experts(expert_offsets),
                                          CAIF_DataType(grad_input.Dtype()).CaifxCode(),grad_input.StreamHandle()),
              "MoEDispatchBackwardGPU");
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
    // The reference keeps these int32 arrays in tensors of its default dtype (Float32): only the
    // element size is part of the contract (tests/test_device_moe.cpp:1574-1583).
    static bool FourByte(const CAIF_DeviceTensor &t){return t.Dtype()==Dtype_e::Int32||t.Dtype()==Dtype_e::Float32;}
    static const int32_t *Idx(const CAIF_DeviceTensor &t){return static_cast<const int32_t*>(t.DeviceDataRaw());}
    static int Experts(const CAIF_DeviceTensor &offsets){return static_cast<int>(offsets.TotalElements())-1;}
    // tokens [T, dim] and buffer [rows, dim] of one float dtype; indices / map Int32 [T, top_k]; offsets Int32
    static void RouteShapes(const CAIF_DeviceTensor &tokens,const CAIF_DeviceTensor &indices,const CAIF_DeviceTensor &map,
                            const CAIF_DeviceTensor &offsets,uint32_t top_k,const CAIF_DeviceTensor &buffer,const char *op)
    {
      RequireDevice(tokens,op);
      RequireDevice(buffer,op);
      if(tokens.Shape().size()!=2||buffer.Shape().size()!=2||indices.Shape().size()!=2)
      {
        THROW_CAIFE(std::string(op)+": tokens, buffer and indices must be 2D");
      }
      if(!FourByte(indices)||!FourByte(map)||!FourByte(offsets))
      {
        THROW_CAIFE(std::string(op)+": indices, map and offsets must hold 32-bit integers");
      }
      if(tokens.Dtype()!=buffer.Dtype()||tokens.Shape()[1]!=buffer.Shape()[1]||indices.Shape()[0]!=tokens.Shape()[0]||
         indices.Shape()[1]!=top_k||map.TotalElements()!=indices.TotalElements()||offsets.TotalElements()<2)
      {
        THROW_CAIFE(std::string(op)+": shape or dtype mismatch");
      }
    }
    static void RouteWeights(const CAIF_DeviceTensor &weights,const CAIF_DeviceTensor &indices,const CAIF_DeviceTensor &like,
                             const char *op)
    {
      if(weights.Dtype()!=like.Dtype()||weights.TotalElements()!=indices.TotalElements())
      {
        THROW_CAIFE(std::string(op)+": routing weights must be [num_tokens x top_k] of the token dtype");
      }
    }
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
