// RAII HIP stream.  Keeps the reference's class name (include/caif/caif_cuda_stream.h) so host
// code that takes a CAIF_CudaStream& compiles unchanged; the handle is a hipStream_t.
#pragma once

#include <hip/hip_runtime_api.h>

#include "caif_exception.h"

namespace instance
{

class CAIF_CudaStream
{
  public:
    CAIF_CudaStream():_handle(nullptr),_owned(false)
    {
      if(hipStreamCreateWithFlags(&_handle,hipStreamNonBlocking)!=hipSuccess)
      {
        THROW_CAIFE("CAIF_CudaStream: hipStreamCreate failed");
      }
      _owned=true;
    }
    // Non-owning view of an existing stream (nullptr = the default stream); touches no device.
    static CAIF_CudaStream Wrap(hipStream_t s){return CAIF_CudaStream(s,false);}
    ~CAIF_CudaStream(){Release();}
    CAIF_CudaStream(const CAIF_CudaStream &)=delete;
    CAIF_CudaStream &operator=(const CAIF_CudaStream &)=delete;
    CAIF_CudaStream(CAIF_CudaStream &&o)noexcept:_handle(o._handle),_owned(o._owned){o._handle=nullptr;o._owned=false;}
    CAIF_CudaStream &operator=(CAIF_CudaStream &&o)noexcept
    {
      if(this!=&o)
      {
        Release();
        _handle=o._handle;
        _owned=o._owned;
        o._handle=nullptr;
        o._owned=false;
      }
      return *this;
    }
    hipStream_t Handle()const{return _handle;}
    void Synchronize()const
    {
      if(hipStreamSynchronize(_handle)!=hipSuccess)
      {
        THROW_CAIFE("CAIF_CudaStream: synchronize failed");
      }
    }

  private:
    CAIF_CudaStream(hipStream_t s,bool owned):_handle(s),_owned(owned){}
    void Release()
    {
      if(_owned==true&&_handle!=nullptr)
      {
        (void)hipStreamDestroy(_handle);
      }
      _handle=nullptr;
      _owned=false;
    }
    hipStream_t _handle;
    bool _owned;
};

}//end instance namespace
