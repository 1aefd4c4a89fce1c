// Move-only tensor over HIP memory: the subset of the reference's CAIF_DeviceTensor
// (include/caif/caif_device_tensor.h:57-498, src/caif_device_tensor.cpp) that the frozen
// quantized-linear path touches.  Device allocations are stream ordered (hipMallocAsync /
// hipFreeAsync on the tensor's stream, as the reference does with cudaMallocAsync :176,:214);
// WrapView is non-owning (:284-293); To() between float dtypes and int8 runs the cast kernels of
// the C ABI (:604-706).  Host_e tensors exist so that ops can refuse them the way the reference
// does ("host backend not supported", src/caif_ops.cpp:514-517).
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "caif_cuda_stream.h"
#include "caif_data_type.h"
#include "caif_exception.h"
#include "caifx.h"

namespace instance
{

class CAIF_DeviceTensor
{
  public:
    typedef CAIF_DataType::CAIF_DataType_e Dtype_e;
    enum class Location_e:uint8_t{Device_e,Host_e};

    CAIF_DeviceTensor():_data(nullptr),_bytes(0),_dtype(Dtype_e::Float32),_stream(nullptr),_owned(false),
                        _location(Location_e::Device_e){}
    ~CAIF_DeviceTensor(){Release();}
    CAIF_DeviceTensor(const CAIF_DeviceTensor &)=delete;
    CAIF_DeviceTensor &operator=(const CAIF_DeviceTensor &)=delete;
    CAIF_DeviceTensor(CAIF_DeviceTensor &&o)noexcept{MoveFrom(o);}
    CAIF_DeviceTensor &operator=(CAIF_DeviceTensor &&o)noexcept
    {
      if(this!=&o)
      {
        Release();
        MoveFrom(o);
      }
      return *this;
    }

    static CAIF_DeviceTensor Uninitialized(const std::vector<uint32_t> &shape,const CAIF_CudaStream &stream,
                                           Dtype_e dtype=Dtype_e::Float32)
    {
      CAIF_DeviceTensor t;
      t._shape=shape;
      t._dtype=dtype;
      t._stream=stream.Handle();
      t._bytes=CAIF_DataType(dtype).StorageSizeBytes(t.TotalElements());
      if(t._bytes>0)
      {
        if(hipMallocAsync(&t._data,t._bytes,t._stream)!=hipSuccess)
        {
          THROW_CAIFE("CAIF_DeviceTensor: device allocation failed");
        }
        t._owned=true;
      }
      return t;
    }
    static CAIF_DeviceTensor Zeros(const std::vector<uint32_t> &shape,const CAIF_CudaStream &stream,
                                   Dtype_e dtype=Dtype_e::Float32)
    {
      CAIF_DeviceTensor t=Uninitialized(shape,stream,dtype);
      if(t._bytes>0&&hipMemsetAsync(t._data,0,t._bytes,t._stream)!=hipSuccess)
      {
        THROW_CAIFE("CAIF_DeviceTensor: memset failed");
      }
      return t;
    }
    static CAIF_DeviceTensor WrapView(void *data,const std::vector<uint32_t> &shape,const CAIF_CudaStream &stream,
                                      Dtype_e dtype=Dtype_e::Float32)
    {
      CAIF_DeviceTensor t;
      t._shape=shape;
      t._dtype=dtype;
      t._stream=stream.Handle();
      t._bytes=CAIF_DataType(dtype).StorageSizeBytes(t.TotalElements());
      t._data=data;
      t._owned=false;
      return t;
    }
    // Host-resident tensor (malloc).  Only what the "host backend" refusals need.
    static CAIF_DeviceTensor HostZeros(const std::vector<uint32_t> &shape,Dtype_e dtype=Dtype_e::Float32)
    {
      CAIF_DeviceTensor t;
      t._shape=shape;
      t._dtype=dtype;
      t._location=Location_e::Host_e;
      t._bytes=CAIF_DataType(dtype).StorageSizeBytes(t.TotalElements());
      t._data=t._bytes>0?std::calloc(1,t._bytes):nullptr;
      t._owned=true;
      return t;
    }

    const std::vector<uint32_t> &Shape()const{return _shape;}
    Dtype_e Dtype()const{return _dtype;}
    Location_e Location()const{return _location;}
    hipStream_t StreamHandle()const{return _stream;}
    size_t TotalElements()const
    {
      if(_shape.empty()==true)
      {
        return 0;
      }
      size_t n=1;
      for(uint32_t d:_shape)
      {
        n*=d;
      }
      return n;
    }
    size_t SizeBytes()const{return _bytes;}
    bool IsEmpty()const{return _data==nullptr||TotalElements()==0;}
    bool IsAllocated()const{return _data!=nullptr;}
    void *DeviceDataRaw(){return _data;}
    const void *DeviceDataRaw()const{return _data;}
    template<typename T> T *DevicePtr(){return static_cast<T*>(_data);}
    template<typename T> const T *DevicePtr()const{return static_cast<const T*>(_data);}

    void Reshape(const std::vector<uint32_t> &shape)
    {
      size_t n=shape.empty()?0:1;
      for(uint32_t d:shape)
      {
        n*=d;
      }
      if(n!=TotalElements())
      {
        THROW_CAIFE("CAIF_DeviceTensor::Reshape: element count mismatch");
      }
      _shape=shape;
    }

    // Byte-count-checked raw copies (src/caif_device_tensor.cpp:456-459).  Synchronous with
    // respect to the host, ordered after prior work on the tensor's stream.
    void CopyFromHostRaw(const void *src,size_t num_bytes)
    {
      if(num_bytes!=_bytes)
      {
        THROW_CAIFE("CAIF_DeviceTensor::CopyFromHostRaw: byte count does not match tensor size");
      }
      if(_bytes==0)
      {
        return;
      }
      if(_location==Location_e::Host_e)
      {
        std::memcpy(_data,src,num_bytes);
        return;
      }
      if(hipMemcpyAsync(_data,src,num_bytes,hipMemcpyHostToDevice,_stream)!=hipSuccess||
         hipStreamSynchronize(_stream)!=hipSuccess)
      {
        THROW_CAIFE("CAIF_DeviceTensor::CopyFromHostRaw: copy failed");
      }
    }
    void CopyToHostRaw(void *dst)const
    {
      if(_bytes==0)
      {
        return;
      }
      if(_location==Location_e::Host_e)
      {
        std::memcpy(dst,_data,_bytes);
        return;
      }
      if(hipMemcpyAsync(dst,_data,_bytes,hipMemcpyDeviceToHost,_stream)!=hipSuccess||
         hipStreamSynchronize(_stream)!=hipSuccess)
      {
        THROW_CAIFE("CAIF_DeviceTensor::CopyToHostRaw: copy failed");
      }
    }

    CAIF_DeviceTensor Clone()const
    {
      if(_location==Location_e::Host_e)
      {
        CAIF_DeviceTensor t=HostZeros(_shape,_dtype);
        if(_bytes>0)
        {
          std::memcpy(t._data,_data,_bytes);
        }
        return t;
      }
      CAIF_DeviceTensor t=Uninitialized(_shape,CAIF_CudaStream::Wrap(_stream),_dtype);
      if(_bytes>0&&hipMemcpyAsync(t._data,_data,_bytes,hipMemcpyDeviceToDevice,_stream)!=hipSuccess)
      {
        THROW_CAIFE("CAIF_DeviceTensor::Clone: copy failed");
      }
      return t;
    }

    // Cast to another dtype (same dtype = Clone, :612-615).  fp16 <-> bf16 go through fp32 (:665-678).
    CAIF_DeviceTensor To(Dtype_e target)const
    {
      try
      {
        if(target==_dtype)
        {
          return Clone();
        }
        if(_location==Location_e::Host_e)
        {
          THROW_CAIFE("CAIF_DeviceTensor::To: host backend not supported");
        }
        const CAIF_CudaStream view=CAIF_CudaStream::Wrap(_stream);
        const int64_t n=static_cast<int64_t>(TotalElements());
        if(_dtype!=Dtype_e::Float32&&target!=Dtype_e::Float32)
        {
          CAIF_DeviceTensor mid=To(Dtype_e::Float32);
          return mid.To(target);
        }
        CAIF_DeviceTensor out=Uninitialized(_shape,view,target);
        int st=CAIFX_ERR_UNSUPPORTED;
        if(_dtype==Dtype_e::Float32)
        {
          const float *src=static_cast<const float*>(_data);
          if(target==Dtype_e::Float16){st=caifx_convert_fp32_to_fp16(src,out._data,n,_stream);}
          else if(target==Dtype_e::BFloat16){st=caifx_convert_fp32_to_bf16(src,out._data,n,_stream);}
          else if(target==Dtype_e::Int8){st=caifx_convert_fp32_to_int8(src,out._data,n,_stream);}
        }
        else
        {
          float *dst=static_cast<float*>(out._data);
          if(_dtype==Dtype_e::Float16){st=caifx_convert_fp16_to_fp32(_data,dst,n,_stream);}
          else if(_dtype==Dtype_e::BFloat16){st=caifx_convert_bf16_to_fp32(_data,dst,n,_stream);}
          else if(_dtype==Dtype_e::Int8){st=caifx_convert_int8_to_fp32(_data,dst,n,_stream);}
        }
        if(st!=CAIFX_OK)
        {
          THROW_CAIFE(std::string("CAIF_DeviceTensor::To: unsupported conversion (")+caifx_status_string(st)+")");
        }
        return out;
      }
      CAIF_CATCH_BLOCK()
    }

  private:
    void Release()
    {
      if(_owned==true&&_data!=nullptr)
      {
        if(_location==Location_e::Host_e)
        {
          std::free(_data);
        }
        else
        {
          (void)hipFreeAsync(_data,_stream);
        }
      }
      _data=nullptr;
      _owned=false;
      _bytes=0;
    }
    void MoveFrom(CAIF_DeviceTensor &o)
    {
      _data=o._data;
      _bytes=o._bytes;
      _shape=std::move(o._shape);
      _dtype=o._dtype;
      _stream=o._stream;
      _owned=o._owned;
      _location=o._location;
      o._data=nullptr;
      o._bytes=0;
      o._owned=false;
      o._shape.clear();
    }

    void *_data;
    size_t _bytes;
    std::vector<uint32_t> _shape;
    Dtype_e _dtype;
    hipStream_t _stream;
    bool _owned;
    Location_e _location;
};

}//end instance namespace
