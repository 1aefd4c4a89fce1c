// Per-pass state handed to every layer call.  The frozen path reads only Training() and Stream()
// (src/caif_device_frozen_linear.cpp:437; include/caif/caif_run_context.h:104-111: non-copyable).
#pragma once

#include "caif_cuda_stream.h"

namespace instance
{

class CAIF_RunContext
{
  public:
    CAIF_RunContext(CAIF_CudaStream &stream,bool training):_stream(&stream),_training(training){}
    CAIF_RunContext(const CAIF_RunContext &)=delete;
    CAIF_RunContext &operator=(const CAIF_RunContext &)=delete;
    bool Training()const{return _training;}
    void SetTraining(bool t){_training=t;}
    CAIF_CudaStream &Stream(){return *_stream;}

  private:
    CAIF_CudaStream *_stream;
    bool _training;
};

}//end instance namespace
