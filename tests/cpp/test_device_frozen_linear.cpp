// CAIF_DeviceFrozenLinear through the reference's layer API: accuracy bars, layout pin, state and
// error contracts of tests/test_device_frozen_linear.cpp (shape K=16, N=8, M=2 :43-46; tolerances
// :1103-1206,:1303; layout :996-1072; backward :416-468), plus the offload hooks.
#include "caif/caif_device_frozen_linear_factory.h"
#include "caif_test_harness.h"

using namespace instance;
using namespace caif_test;
typedef CAIF_Ops::QuantScheme_e Scheme;

static const uint32_t K=16,N=8,M=2;

// y[m][n] = sum_k x[m][k] w[n][k]   (w is [out,in] row-major: the HuggingFace layout the layer expects)
static std::vector<float> RefForward(const std::vector<float> &x,const std::vector<float> &w,uint32_t m,uint32_t n,uint32_t k)
{
  std::vector<float> y(m*n,0.0f);
  for(uint32_t i=0;i<m;++i)for(uint32_t j=0;j<n;++j){double a=0;for(uint32_t t=0;t<k;++t){a+=(double)x[i*k+t]*w[j*k+t];}y[i*n+j]=(float)a;}
  return y;
}
static std::vector<float> RefBackward(const std::vector<float> &g,const std::vector<float> &w,uint32_t m,uint32_t n,uint32_t k)
{
  std::vector<float> d(m*k,0.0f);
  for(uint32_t i=0;i<m;++i)for(uint32_t t=0;t<k;++t){double a=0;for(uint32_t j=0;j<n;++j){a+=(double)g[i*n+j]*w[j*k+t];}d[i*k+t]=(float)a;}
  return d;
}

// Build a loaded layer the way the reference's callers do: quantise on the device through CAIF_Ops,
// move the codes in, bounce the scales through the host.
static std::unique_ptr<CAIF_DeviceLayer> MakeLayer(const std::vector<float> &w,Dtype_e storage,Dtype_e compute,Scheme scheme,
                                                   uint32_t group,CAIF_CudaStream &stream,CAIF_RunContext &ctx)
{
  std::unique_ptr<CAIF_DeviceLayer> layer=CAIF_DeviceFrozenLinearFactory::Create(K,N,storage,stream,group,true,compute,scheme);
  CAIF_DeviceFrozenLinearBase *base=dynamic_cast<CAIF_DeviceFrozenLinearBase*>(layer.get());
  if(storage==Dtype_e::Int4)
  {
    CAIF_DeviceTensor in=Upload(w,{N*K},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({N*K},stream,Dtype_e::Int4);
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({(N*K+group-1)/group},stream,Dtype_e::Float16);
    CAIF_Ops::QuantizeInt4PerGroup(in,q,s,group,ctx);
    std::vector<uint16_t> sh(s.TotalElements());
    s.CopyToHostRaw(sh.data());
    base->LoadFromTensor(std::move(q));
    base->LoadScalesFromHost(sh.data(),sh.size()*sizeof(uint16_t));
  }
  else
  {
    // callers label the [out,in] buffer as [in,out] for the quantiser (cols = OutputDim)
    CAIF_DeviceTensor in=Upload(w,{K,N},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({K,N},stream,Dtype_e::Int8);
    const uint32_t ns=scheme==Scheme::PerTensor_e?1u:N;
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({ns},stream,Dtype_e::Float32);
    CAIF_Ops::QuantizeInt8(in,q,s,scheme,ctx);
    std::vector<float> sh=Download(s);
    base->LoadFromTensor(std::move(q));
    base->LoadScalesFromHost(sh.data(),sh.size()*sizeof(float));
  }
  return layer;
}

static void GpuTests()
{
  CAIF_CudaStream stream;
  CAIF_RunContext infer(stream,false),train(stream,true);
  const std::vector<float> w=Uniform(N*K,-0.5f,0.5f,71);
  const std::vector<float> x=Uniform(M*K,-1.0f,1.0f,201);
  const std::vector<float> g=Uniform(M*N,-1.0f,1.0f,303);
  const std::vector<float> ref=RefForward(x,w,M,N,K);

  struct Cell{const char *name;Dtype_e storage;Scheme scheme;float tol[3];};
  const Cell cells[]={{"INT8 per-tensor",Dtype_e::Int8,Scheme::PerTensor_e,{2e-2f,2e-2f,3e-2f}},
                      {"INT8 per-channel",Dtype_e::Int8,Scheme::PerChannel_e,{3e-2f,3e-2f,4e-2f}},
                      {"INT4 per-group",Dtype_e::Int4,Scheme::PerTensor_e,{1.5e-1f,1.5e-1f,1.5e-1f}}};
  const Dtype_e computes[3]={Dtype_e::Float32,Dtype_e::Float16,Dtype_e::BFloat16};
  for(const Cell &c:cells)
  {
    for(int ci=0;ci<3;++ci)
    {
      auto layer=MakeLayer(w,c.storage,computes[ci],c.scheme,16,stream,infer);
      CAIF_DeviceTensor in=Upload(x,{M,K},stream);
      CAIF_DeviceTensor out=layer->Forward(in,infer);
      const std::vector<float> y=Download(out);
      const std::string tag=std::string(c.name)+" / "+CAIF_DataType(computes[ci]).Name();
      Report(tag+": forward close to dense fp32",out.Dtype()==Dtype_e::Float32&&out.Shape()==std::vector<uint32_t>({M,N})&&
                                                 RelToMax(y,ref)<=c.tol[ci]);
      // parity against the layer's own dequantised weight (isolates the GEMM from quantisation noise)
      const std::vector<float> wd=Download(layer->FrozenTensorFP32(0));
      const float gemm_tol=computes[ci]==Dtype_e::Float32?1e-4f:2e-2f;
      Report(tag+": forward matches dequantised-weight GEMM",RelToMax(y,RefForward(x,wd,M,N,K))<=gemm_tol);
      Report(tag+": backward before a training forward throws",
             Throws([&]{CAIF_DeviceTensor go=Upload(g,{M,N},stream);layer->Backward(go,train);},"training=true first"));
      layer->Forward(in,train);
      CAIF_DeviceTensor go=Upload(g,{M,N},stream);
      CAIF_DeviceTensor dx=layer->Backward(go,train);
      Report(tag+": dX matches dequantised-weight GEMM",dx.Dtype()==Dtype_e::Float32&&dx.Shape()==std::vector<uint32_t>({M,K})&&
                                                         RelToMax(Download(dx),RefBackward(g,wd,M,N,K))<=gemm_tol);
    }
  }
  {
    // Float storage: the nine remaining cells of the grid.  The weight is loaded as stored ([output_dim, input_dim],
    // the layout tests/test_device_frozen_linear.cpp:996-1072 pins against a dense layer), no scales.
    const Dtype_e storages[3]={Dtype_e::Float32,Dtype_e::Float16,Dtype_e::BFloat16};
    for(int si=0;si<3;++si)
    {
      for(int ci=0;ci<3;++ci)
      {
        auto layer=CAIF_DeviceFrozenLinearFactory::Create(K,N,storages[si],stream,16,true,computes[ci]);
        CAIF_DeviceFrozenLinearBase *base=dynamic_cast<CAIF_DeviceFrozenLinearBase*>(layer.get());
        CAIF_DeviceTensor wt=Upload(w,{N,K},stream);
        base->LoadFromTensor(storages[si]==Dtype_e::Float32?std::move(wt):wt.To(storages[si]));
        const std::string tag=std::string("float storage ")+CAIF_DataType(storages[si]).Name()+" / "+CAIF_DataType(computes[ci]).Name();
        Report(tag+": needs no scales",base->NeedsScales()==false);
        CAIF_DeviceTensor in=Upload(x,{M,K},stream);
        CAIF_DeviceTensor out=layer->Forward(in,infer);
        const bool exact=storages[si]==Dtype_e::Float32&&computes[ci]==Dtype_e::Float32;
        const float tol=exact?1e-5f:2e-2f;
        Report(tag+": forward matches the dense product",out.Dtype()==Dtype_e::Float32&&out.Shape()==std::vector<uint32_t>({M,N})&&
                                                         RelToMax(Download(out),ref)<=tol);
        const std::vector<float> wd=Download(layer->FrozenTensorFP32(0));
        Report(tag+": frozen tensor is the stored weight widened",RelToMax(wd,w)<=(storages[si]==Dtype_e::Float32?0.0f:1e-2f));
        layer->Forward(in,train);
        CAIF_DeviceTensor go=Upload(g,{M,N},stream);
        CAIF_DeviceTensor dx=layer->Backward(go,train);
        Report(tag+": dX matches the dense product",dx.Shape()==std::vector<uint32_t>({M,K})&&
                                                     RelToMax(Download(dx),RefBackward(g,wd,M,N,K))<=tol);
      }
    }
  }
  {
    // 3-D input is flattened over the leading dims and reshaped back
    auto layer=MakeLayer(w,Dtype_e::Int8,Dtype_e::Float32,Scheme::PerChannel_e,16,stream,infer);
    std::vector<float> x3=Uniform(2*3*K,-1.0f,1.0f,202);
    CAIF_DeviceTensor in=Upload(x3,{2u,3u,K},stream);
    CAIF_DeviceTensor out=layer->Forward(in,infer);
    Report("N-D input keeps leading dims",out.Shape()==std::vector<uint32_t>({2u,3u,N}));
    CAIF_DeviceTensor bad=Upload(Uniform(2*(K+1),-1,1,5),{2u,K+1},stream);
    Report("last dim mismatch throws",Throws([&]{layer->Forward(bad,infer);},"last dim must match input_dim"));
    CAIF_DeviceTensor one_d=Upload(Uniform(K,-1,1,6),{K},stream);
    Report("1-D input throws",Throws([&]{layer->Forward(one_d,infer);},"at least 2D"));
    Report("description names the dims and dtype",layer->Description()=="FrozenLinear(16,8,int8)");
    Report("no trainable parameters",layer->ParameterTensorCount()==0&&layer->TotalParameterCount()==0&&
                                     layer->ParameterNames("p.").empty()&&Throws([&]{layer->ParameterTensor(0);},"no trainable parameters")&&
                                     Throws([&]{layer->GradientTensor(0);},"no trainable parameters"));
    Report("one frozen tensor named <prefix>weight",layer->FrozenTensorCount()==1&&layer->FrozenTensorNames("ffn.up.")[0]=="ffn.up.weight");
    Report("frozen tensor index out of range throws",Throws([&]{layer->FrozenTensorFP32(1);},"out of range"));
  }
  {
    auto layer=CAIF_DeviceFrozenLinearFactory::Create(K,N,Dtype_e::Int4,stream,16,true,Dtype_e::BFloat16);
    CAIF_DeviceTensor in=Upload(x,{M,K},stream);
    Report("forward before load throws",Throws([&]{layer->Forward(in,infer);},"weight not loaded"));
    CAIF_DeviceFrozenLinearBase *base=dynamic_cast<CAIF_DeviceFrozenLinearBase*>(layer.get());
    Report("base interface reachable by dynamic_cast",base!=nullptr&&base->InputDim()==K&&base->OutputDim()==N&&
                                                      base->NeedsScales()==true&&base->CacheFP32()==true);
    base->LoadFromTensor(CAIF_DeviceTensor::Zeros({N*K},stream,Dtype_e::Int4));
    Report("int4 forward without scales throws",Throws([&]{layer->Forward(in,infer);},"scales not loaded"));
    std::vector<uint16_t> few(3,0);
    Report("scale byte count mismatch throws",Throws([&]{base->LoadScalesFromHost(few.data(),few.size()*2);},"byte count"));
  }
  {
    // offload hooks: HostPinned keeps the codes in pinned host memory between Prefetch and Evict
    auto layer=MakeLayer(w,Dtype_e::Int8,Dtype_e::BFloat16,Scheme::PerChannel_e,16,stream,infer);
    CAIF_DeviceFrozenLinearBase *base=dynamic_cast<CAIF_DeviceFrozenLinearBase*>(layer.get());
    CAIF_DeviceTensor in=Upload(x,{M,K},stream);
    const std::vector<float> before=Download(layer->Forward(in,infer));
    base->SetOffloadPolicy(CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::HostPinned_e);
    Report("HostPinned without prefetch throws",base->IsPrefetched()==false&&Throws([&]{layer->Forward(in,infer);},"not prefetched"));
    base->Prefetch(stream);
    Report("prefetched forward is unchanged",Download(layer->Forward(in,infer))==before);
    base->Evict();
    Report("evicted layer throws again",Throws([&]{layer->Forward(in,infer);},"not prefetched"));
    base->SetOffloadPolicy(CAIF_OffloadPolicy::CAIF_OffloadPolicy_e::GpuResident_e);
    Report("back to GpuResident works",Download(layer->Forward(in,infer))==before);
  }
  stream.Synchronize();
}

int main(int argc,char **argv)
{
  const bool cpu_only=(argc>1&&std::string(argv[1])=="--cpu")||HasGpu()==false;
  {
    CAIF_CudaStream null_stream=CAIF_CudaStream::Wrap(nullptr);
    Report("zero dims throw",Throws([&]{CAIF_DeviceFrozenLinear<float,int8_t> l(0,8,null_stream);},"must be > 0"));
    Report("float storage cells are built",CAIF_DeviceFrozenLinearFactory::Create(K,N,Dtype_e::Float32,null_stream)->Description()=="FrozenLinear(16,8,fp32)");
    CAIF_DeviceFrozenLinear<caif_bf16_t,caif_int4_packed_t> l(K,N,null_stream);
    Report("defaults: group 128, cache hint true, per-tensor scheme",l.GroupSize()==128&&l.CacheFP32()==true&&
                                                                    l.Int8Scheme()==Scheme::PerTensor_e&&
                                                                    l.Description()=="FrozenLinear(16,8,int4)");
  }
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
