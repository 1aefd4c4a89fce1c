// Quantise / dequantise ops through the CAIF_Ops surface: the checks of the reference's
// tests/test_quantize_ops.cpp (round-trip bounds :161-300, zero input :232-267, error contracts
// :302-402, fake-quant :404-481) against this build's host layer.
#include "caif/caif_ops.h"
#include "caif_test_harness.h"

using namespace instance;
using namespace caif_test;
typedef CAIF_Ops::QuantScheme_e Scheme;

static void GpuTests()
{
  CAIF_CudaStream stream;
  CAIF_RunContext ctx(stream,false);
  {
    const size_t n=1024;
    std::vector<float> x=Uniform(n,-2.5f,2.5f,11);
    CAIF_DeviceTensor in=Upload(x,{(uint32_t)n},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({(uint32_t)n},stream,Dtype_e::Int8);
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({1u},stream,Dtype_e::Float32);
    CAIF_DeviceTensor out=CAIF_DeviceTensor::Zeros({(uint32_t)n},stream,Dtype_e::Float32);
    CAIF_Ops::QuantizeInt8(in,q,s,Scheme::PerTensor_e,ctx);
    CAIF_Ops::DequantizeInt8(q,out,s,Scheme::PerTensor_e,ctx);
    std::vector<float> y=Download(out);
    float err=0.0f;
    for(size_t i=0;i<n;++i){err=std::fmax(err,std::fabs(x[i]-y[i]));}
    Report("Int8 per-tensor round trip within max/127",err<=MaxAbs(x)/127.0f+1e-6f);
    Report("Int8 per-tensor scale is max/127",FloatEqual(Download(s)[0],MaxAbs(x)/127.0f,0.0f));
  }
  {
    const uint32_t rows=32,cols=64;
    std::vector<float> x(rows*cols);
    std::mt19937 gen(22);
    for(uint32_t r=0;r<rows;++r)
    {
      for(uint32_t c=0;c<cols;++c)
      {
        std::uniform_real_distribution<float> d(-(0.1f+0.05f*c),0.1f+0.05f*c);
        x[r*cols+c]=d(gen);
      }
    }
    CAIF_DeviceTensor in=Upload(x,{rows,cols},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({rows,cols},stream,Dtype_e::Int8);
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({cols},stream,Dtype_e::Float32);
    CAIF_DeviceTensor out=CAIF_DeviceTensor::Zeros({rows,cols},stream,Dtype_e::Float32);
    CAIF_Ops::QuantizeInt8(in,q,s,Scheme::PerChannel_e,ctx);
    CAIF_Ops::DequantizeInt8(q,out,s,Scheme::PerChannel_e,ctx);
    std::vector<float> y=Download(out),sc=Download(s);
    bool ok=true;
    for(uint32_t i=0;i<rows*cols;++i){ok=ok&&std::fabs(x[i]-y[i])<=sc[i%cols]*0.5f*1.000001f;}
    Report("Int8 per-channel round trip within half a step of its column",ok);
  }
  {
    std::vector<float> z(256,0.0f);
    CAIF_DeviceTensor in=Upload(z,{16u,16u},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({16u,16u},stream,Dtype_e::Int8);
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({1u},stream,Dtype_e::Float32);
    CAIF_DeviceTensor out=CAIF_DeviceTensor::Zeros({16u,16u},stream,Dtype_e::Float32);
    CAIF_Ops::QuantizeInt8(in,q,s,Scheme::PerTensor_e,ctx);
    CAIF_Ops::DequantizeInt8(q,out,s,Scheme::PerTensor_e,ctx);
    Report("zero input: scale 1.0 and exact zeros",Download(s)[0]==1.0f&&MaxAbs(Download(out))==0.0f);
  }
  {
    const uint32_t n=512,g=128;
    std::vector<float> x=Uniform(n,-1.0f,1.0f,33);
    CAIF_DeviceTensor in=Upload(x,{n},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({n},stream,Dtype_e::Int4);
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({n/g},stream,Dtype_e::Float16);
    CAIF_DeviceTensor out=CAIF_DeviceTensor::Zeros({n},stream,Dtype_e::Float32);
    CAIF_Ops::QuantizeInt4PerGroup(in,q,s,g,ctx);
    CAIF_Ops::DequantizeInt4PerGroup(q,out,s,g,ctx);
    std::vector<float> y=Download(out);
    float err=0.0f;
    for(uint32_t i=0;i<n;++i){err=std::fmax(err,std::fabs(x[i]-y[i]));}
    Report("Int4 per-group round trip within max/7",err<=MaxAbs(x)/7.0f+1e-3f);
    Report("Int4 storage is half a byte per element",q.SizeBytes()==n/2);
    CAIF_DeviceTensor fq=CAIF_DeviceTensor::Zeros({n},stream,Dtype_e::Float32);
    CAIF_Ops::FakeQuantInt4PerGroup(in,fq,g,ctx);
    Report("FakeQuantInt4 equals quantise+dequantise",Download(fq)==y);
    CAIF_DeviceTensor fq8=CAIF_DeviceTensor::Zeros({n},stream,Dtype_e::Float32);
    CAIF_Ops::FakeQuantInt8(in,fq8,Scheme::PerTensor_e,ctx);
    float e8=0.0f;
    std::vector<float> y8=Download(fq8);
    for(uint32_t i=0;i<n;++i){e8=std::fmax(e8,std::fabs(x[i]-y8[i]));}
    Report("FakeQuantInt8 within max/127",e8<=MaxAbs(x)/127.0f+1e-6f);
  }
  {
    CAIF_DeviceTensor in=CAIF_DeviceTensor::Zeros({4u,8u},stream,Dtype_e::Float32);
    CAIF_DeviceTensor q8=CAIF_DeviceTensor::Zeros({4u,8u},stream,Dtype_e::Int8);
    CAIF_DeviceTensor wrong=CAIF_DeviceTensor::Zeros({4u,8u},stream,Dtype_e::Float32);
    CAIF_DeviceTensor s1=CAIF_DeviceTensor::Zeros({1u},stream,Dtype_e::Float32);
    CAIF_DeviceTensor s8=CAIF_DeviceTensor::Zeros({8u},stream,Dtype_e::Float32);
    CAIF_DeviceTensor s3=CAIF_DeviceTensor::Zeros({3u},stream,Dtype_e::Float32);
    Report("wrong output dtype throws",Throws([&]{CAIF_Ops::QuantizeInt8(in,wrong,s1,Scheme::PerTensor_e,ctx);},"output must be Int8"));
    Report("per-tensor scales length throws",Throws([&]{CAIF_Ops::QuantizeInt8(in,q8,s8,Scheme::PerTensor_e,ctx);},"1 element"));
    Report("per-channel scales length throws",Throws([&]{CAIF_Ops::QuantizeInt8(in,q8,s3,Scheme::PerChannel_e,ctx);},"equal cols"));
    CAIF_DeviceTensor in1=CAIF_DeviceTensor::Zeros({32u},stream,Dtype_e::Float32);
    CAIF_DeviceTensor q1=CAIF_DeviceTensor::Zeros({32u},stream,Dtype_e::Int8);
    Report("per-channel on 1-D throws",Throws([&]{CAIF_Ops::QuantizeInt8(in1,q1,s8,Scheme::PerChannel_e,ctx);},"must be 2D"));
    CAIF_DeviceTensor q4=CAIF_DeviceTensor::Zeros({32u},stream,Dtype_e::Int4);
    CAIF_DeviceTensor sh=CAIF_DeviceTensor::Zeros({2u},stream,Dtype_e::Float16);
    Report("int4 scales length mismatch throws",Throws([&]{CAIF_Ops::QuantizeInt4PerGroup(in1,q4,sh,8,ctx);},"num_groups"));
    Report("int4 group_size 0 throws",Throws([&]{CAIF_Ops::QuantizeInt4PerGroup(in1,q4,sh,0,ctx);},"group_size must be > 0"));
    Report("int4 wrong scales dtype throws",Throws([&]{CAIF_Ops::QuantizeInt4PerGroup(in1,q4,s1,16,ctx);},"scales must be fp16"));
    CAIF_DeviceTensor host_in=CAIF_DeviceTensor::HostZeros({32u});
    Report("host tensors are refused",Throws([&]{CAIF_Ops::QuantizeInt8(host_in,q1,s1,Scheme::PerTensor_e,ctx);},"host backend not supported"));
  }
  stream.Synchronize();
}

int main(int argc,char **argv)
{
  const bool cpu_only=(argc>1&&std::string(argv[1])=="--cpu")||HasGpu()==false;
  Report("Int4 StorageSizeBytes rounds up",CAIF_DataType(Dtype_e::Int4).StorageSizeBytes(5)==3&&
                                           CAIF_DataType(Dtype_e::Float16).StorageSizeBytes(5)==10);
  Report("dtype names",CAIF_DataType(Dtype_e::Int4).Name()=="int4"&&CAIF_DataType(Dtype_e::BFloat16).Name()=="bf16");
  if(cpu_only==false)
  {
    try{GpuTests();}
    catch(const std::exception &e){std::printf("unexpected exception: %s\n",e.what());Report("no unexpected exception",false);}
  }
  else
  {
    std::printf("[SKIP] device tests (no GPU)\n");
  }
  return FinalExitCode();
}
