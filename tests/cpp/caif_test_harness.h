// Minimal test harness in the style of the reference's tests/caif_test_harness.h:36-42 (Report,
// counters, FloatEqual, exit code) plus helpers to move small tensors between host and device.
#pragma once

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <string>
#include <vector>

#include "caif/caif_device_tensor.h"

namespace caif_test
{

inline int &Passed(){static int n=0;return n;}
inline int &Failed(){static int n=0;return n;}
inline void Report(const std::string &name,bool ok)
{
  std::printf("[%s] %s\n",ok?"PASS":"FAIL",name.c_str());
  std::fflush(stdout);
  if(ok){++Passed();}else{++Failed();}
}
inline bool FloatEqual(float a,float b,float tol){return std::fabs(a-b)<=tol;}
inline int FinalExitCode()
{
  std::printf("passed %d, failed %d\n",Passed(),Failed());
  return Failed()==0?0:1;
}
// true when fn throws a CAIF_Exception whose text contains `needle`
inline bool Throws(const std::function<void()> &fn,const std::string &needle="")
{
  try
  {
    fn();
  }
  catch(const instance::CAIF_Exception &e)
  {
    return needle.empty()||std::string(e.what()).find(needle)!=std::string::npos;
  }
  return false;
}

inline bool HasGpu()
{
  int n=0;
  return hipGetDeviceCount(&n)==hipSuccess&&n>0;
}

using instance::CAIF_DeviceTensor;
using instance::CAIF_CudaStream;
typedef instance::CAIF_DataType::CAIF_DataType_e Dtype_e;

inline CAIF_DeviceTensor Upload(const std::vector<float> &v,const std::vector<uint32_t> &shape,CAIF_CudaStream &s)
{
  CAIF_DeviceTensor t=CAIF_DeviceTensor::Uninitialized(shape,s,Dtype_e::Float32);
  t.CopyFromHostRaw(v.data(),v.size()*sizeof(float));
  return t;
}
inline std::vector<float> Download(const CAIF_DeviceTensor &t)
{
  if(t.Dtype()!=Dtype_e::Float32)
  {
    CAIF_DeviceTensor f=t.To(Dtype_e::Float32);
    return Download(f);
  }
  std::vector<float> v(t.TotalElements());
  t.CopyToHostRaw(v.data());
  return v;
}
inline std::vector<float> Uniform(size_t n,float lo,float hi,uint32_t seed)
{
  std::mt19937 gen(seed);
  std::uniform_real_distribution<float> d(lo,hi);
  std::vector<float> v(n);
  for(float &x:v){x=d(gen);}
  return v;
}
inline float MaxAbs(const std::vector<float> &v)
{
  float m=0.0f;
  for(float x:v){m=std::fmax(m,std::fabs(x));}
  return m;
}
inline bool AllFinite(const std::vector<float> &v)
{
  for(float x:v){if(std::isfinite(x)==false){return false;}}
  return true;
}
// max |a-b| / max |b|  (tests/test_device_frozen_linear.cpp:154-175)
inline float RelToMax(const std::vector<float> &a,const std::vector<float> &b)
{
  float e=0.0f;
  for(size_t i=0;i<a.size();++i){e=std::fmax(e,std::fabs(a[i]-b[i]));}
  const float m=MaxAbs(b);
  return m>0.0f?e/m:e;
}

}//end caif_test namespace
