// CAIF_DeviceMoEFrozenExpert and the grouped expert bank: the reference's checks
// (tests/test_device_moe_frozen_expert.cpp:186-453: finite forward/backward, zero parameters,
// ForwardInto == ForwardImpl within 1e-3; dims from tests/caif_test_constants.h:39-68) plus
// bank == per-expert loop over a routed batch.
#include "caif/caif_device_frozen_linear_factory.h"
#include "caif/caif_device_moe_frozen_expert.h"
#include "caif_test_harness.h"

using namespace instance;
using namespace caif_test;
typedef CAIF_Ops::QuantScheme_e Scheme;
typedef CAIF_DeviceMoEFrozenExpert<caif_bf16_t,caif_bf16_t> Expert;

static std::unique_ptr<CAIF_DeviceFrozenLinearBase> Linear(uint32_t in,uint32_t out,uint32_t seed,CAIF_CudaStream &stream,
                                                          CAIF_RunContext &ctx)
{
  auto *l=new CAIF_DeviceFrozenLinear<caif_bf16_t,int8_t>(in,out,stream,128,true,Scheme::PerChannel_e);
  std::unique_ptr<CAIF_DeviceFrozenLinearBase> owner(l);
  CAIF_DeviceTensor w=Upload(Uniform(in*out,-0.05f,0.05f,seed),{in,out},stream);
  CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({in,out},stream,Dtype_e::Int8);
  CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({out},stream,Dtype_e::Float32);
  CAIF_Ops::QuantizeInt8(w,q,s,Scheme::PerChannel_e,ctx);
  l->LoadFromTensor(std::move(q));
  l->LoadScalesFromTensor(std::move(s));
  return owner;
}

static std::unique_ptr<Expert> MakeExpert(uint32_t dim,uint32_t hidden,uint32_t seed,CAIF_CudaStream &stream,CAIF_RunContext &ctx)
{
  Expert::FrozenSubLayers_t sub;
  sub.gate=Linear(dim,hidden,seed,stream,ctx);
  sub.up=Linear(dim,hidden,seed+1,stream,ctx);
  sub.down=Linear(hidden,dim,seed+2,stream,ctx);
  return std::make_unique<Expert>(CAIF_DeviceMoEFrozenExpertConfig(dim,hidden,true),std::move(sub),stream);
}

static void GpuTests()
{
  CAIF_CudaStream stream;
  CAIF_RunContext infer(stream,false),train(stream,true);
  const uint32_t dim=16,hidden=32,batch=2;
  {
    auto expert=MakeExpert(dim,hidden,100,stream,infer);
    CAIF_DeviceTensor x=Upload(Uniform(batch*dim,-1,1,7),{batch,dim},stream).To(Dtype_e::BFloat16);
    CAIF_DeviceTensor y=expert->Forward(x,train);
    Report("forward: [batch, input_dim] of StorageT, finite, non-zero",y.Dtype()==Dtype_e::BFloat16&&
           y.Shape()==std::vector<uint32_t>({batch,dim})&&AllFinite(Download(y))&&MaxAbs(Download(y))>0.0f);
    CAIF_DeviceTensor g=Upload(Uniform(batch*dim,-1,1,8),{batch,dim},stream).To(Dtype_e::BFloat16);
    CAIF_DeviceTensor dx=expert->Backward(g,train);
    Report("backward: [batch, input_dim], finite, non-zero",dx.Shape()==std::vector<uint32_t>({batch,dim})&&
           AllFinite(Download(dx))&&MaxAbs(Download(dx))>0.0f);
    Report("zero trainable parameters",expert->ParameterTensorCount()==0&&expert->TotalParameterCount()==0&&
           Throws([&]{expert->ParameterTensor(0);},"no trainable parameters"));
    Report("description",expert->Description()=="CAIF_DeviceMoEFrozenExpert(input_dim=16,hidden_dim=32,use_gated=true,frozen=true)");
    CAIF_DeviceTensor into=CAIF_DeviceTensor::Zeros({batch,dim},stream,Dtype_e::BFloat16);
    expert->ForwardInto(x,into,infer);
    Report("ForwardInto equals ForwardImpl",RelToMax(Download(into),Download(expert->Forward(x,infer)))<=1e-3f);
    CAIF_DeviceTensor wrong=CAIF_DeviceTensor::Zeros({batch,dim},stream,Dtype_e::Float32);
    Report("ForwardInto with the wrong dtype throws",Throws([&]{expert->ForwardInto(x,wrong,infer);},"StorageDtype"));
    CAIF_DeviceTensor bad=Upload(Uniform(batch*(dim+1),-1,1,9),{batch,dim+1},stream).To(Dtype_e::BFloat16);
    Report("wrong input width throws",Throws([&]{expert->Forward(bad,infer);},"expected [N, input_dim]"));
    auto fresh=MakeExpert(dim,hidden,200,stream,infer);
    Report("backward before a training forward throws",Throws([&]{fresh->Backward(g,train);},"training=true"));
  }
  {
    // bank over 4 experts vs the per-expert loop, on segments of 5, 0, 130 and 3 rows
    const uint32_t D=64,H=128,E=4;
    std::vector<std::unique_ptr<Expert>> experts;
    std::vector<Expert*> raw;
    for(uint32_t e=0;e<E;++e){experts.push_back(MakeExpert(D,H,300+10*e,stream,infer));raw.push_back(experts.back().get());}
    const std::vector<int32_t> offsets={0,5,5,135,138};
    const uint32_t rows=138;
    CAIF_DeviceTensor off=CAIF_DeviceTensor::Uninitialized({E+1},stream,Dtype_e::Int32);
    off.CopyFromHostRaw(offsets.data(),offsets.size()*sizeof(int32_t));
    const std::vector<float> xh=Uniform(rows*D,-1,1,11),gh=Uniform(rows*D,-0.01f,0.01f,12);
    CAIF_DeviceTensor x=Upload(xh,{rows,D},stream).To(Dtype_e::BFloat16);
    CAIF_DeviceTensor g=Upload(gh,{rows,D},stream).To(Dtype_e::BFloat16);
    CAIF_DeviceMoEFrozenExpertBank<caif_bf16_t,caif_bf16_t> bank(raw,stream);
    const std::vector<float> yb=Download(bank.Forward(x,off,true));
    const std::vector<float> db=Download(bank.Backward(g,off));
    std::vector<float> yl(rows*D,0.0f),dl(rows*D,0.0f);
    const std::vector<float> xr=Download(x),gr=Download(g);
    for(uint32_t e=0;e<E;++e)
    {
      const uint32_t lo=offsets[e],cnt=offsets[e+1]-offsets[e];
      if(cnt==0){continue;}
      std::vector<float> xs(xr.begin()+lo*D,xr.begin()+(lo+cnt)*D),gs(gr.begin()+lo*D,gr.begin()+(lo+cnt)*D);
      CAIF_DeviceTensor xe=Upload(xs,{cnt,D},stream).To(Dtype_e::BFloat16);
      CAIF_DeviceTensor ge=Upload(gs,{cnt,D},stream).To(Dtype_e::BFloat16);
      const std::vector<float> ye=Download(experts[e]->Forward(xe,train));
      const std::vector<float> de=Download(experts[e]->Backward(ge,train));
      std::copy(ye.begin(),ye.end(),yl.begin()+lo*D);
      std::copy(de.begin(),de.end(),dl.begin()+lo*D);
    }
    Report("bank forward equals the per-expert loop",RelToMax(yb,yl)<=1e-2f);
    Report("bank backward equals the per-expert loop",RelToMax(db,dl)<=1e-2f);

    // Offloaded experts (src/caif_device_frozen_linear.cpp:145-232): SetOffloadPolicy(HostPinned) and Evict()
    // free a weight's device copy and Prefetch() uploads it to a new allocation.  The bank must refuse to run
    // while an expert is away and must follow the weight to its new address afterwards.
    typedef CAIF_OffloadPolicy::CAIF_OffloadPolicy_e Policy;
    CAIF_DeviceFrozenLinearBase *moved=experts[2]->SubLayers().up.get();
    moved->SetOffloadPolicy(Policy::HostPinned_e);
    Report("bank forward with an evicted expert throws",Throws([&]{bank.Forward(x,off,false);},"Prefetch"));
    // occupy the freed block so that the upload lands somewhere else
    CAIF_DeviceTensor squatter=CAIF_DeviceTensor::Zeros({D,H},stream,Dtype_e::Int8);
    moved->Prefetch(stream);
    Report("bank forward after Prefetch equals the first result",Download(bank.Forward(x,off,true))==yb);
    moved->Evict();
    Report("bank backward with an evicted expert throws",Throws([&]{bank.Backward(g,off);},"Prefetch"));
    moved->Prefetch(stream);
    Report("bank backward after Prefetch equals the first result",Download(bank.Backward(g,off))==db);
    moved->SetOffloadPolicy(Policy::GpuResident_e);
    Report("bank forward after returning to GpuResident equals the first result",Download(bank.Forward(x,off,false))==yb);
  }
  stream.Synchronize();
}

int main(int argc,char **argv)
{
  const bool cpu_only=(argc>1&&std::string(argv[1])=="--cpu")||HasGpu()==false;
  {
    CAIF_CudaStream null_stream=CAIF_CudaStream::Wrap(nullptr);
    Expert::FrozenSubLayers_t none;
    Report("missing up sub-layer throws",Throws([&]{Expert e(CAIF_DeviceMoEFrozenExpertConfig(16,32,true),std::move(none),null_stream);},"up sub-layer required"));
    Expert::FrozenSubLayers_t no_gate;
    no_gate.up=std::make_unique<CAIF_DeviceFrozenLinear<caif_bf16_t,int8_t>>(16,32,null_stream);
    no_gate.down=std::make_unique<CAIF_DeviceFrozenLinear<caif_bf16_t,int8_t>>(32,16,null_stream);
    Report("gated config without gate throws",Throws([&]{Expert e(CAIF_DeviceMoEFrozenExpertConfig(16,32,true),std::move(no_gate),null_stream);},"requires gate"));
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
