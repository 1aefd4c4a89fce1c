// CAIF_Ops::MoEBuildDispatchMap / MoEDispatchGPU / MoECombineGPU and their backward passes: the reference's
// smoke checks (tests/test_device_moe.cpp:1574-1650: total_assigned in range, buffer and output non-zero)
// plus the definitions themselves on a small routed batch: arrival-order positions, row copies, weighted
// sums, capacity drops, the error contract.
#include "caif/caif_ops.h"
#include "caif_test_harness.h"

using namespace instance;
using namespace caif_test;

static CAIF_DeviceTensor UploadI32(const std::vector<int32_t> &v,const std::vector<uint32_t> &shape,CAIF_CudaStream &s,
                                   Dtype_e tag=Dtype_e::Int32)
{
  CAIF_DeviceTensor t=CAIF_DeviceTensor::Uninitialized(shape,s,tag);
  t.CopyFromHostRaw(v.data(),v.size()*sizeof(int32_t));
  return t;
}
static std::vector<int32_t> DownloadI32(const CAIF_DeviceTensor &t)
{
  std::vector<int32_t> v(t.TotalElements());
  t.CopyToHostRaw(v.data());
  return v;
}

static void GpuTests()
{
  CAIF_CudaStream stream;
  const uint32_t tokens=50,top_k=3,experts=7,dim=24;
  std::mt19937 gen(5);
  std::vector<int32_t> idx(tokens*top_k);
  for(int32_t &e:idx){e=static_cast<int32_t>(gen()%experts);}
  idx[4]=-1;                                   // an invalid expert id routes nothing

  for(uint32_t capacity:{0u,9u})
  {
    // the reference keeps the int32 arrays in Float32-tagged tensors; both tags are accepted
    CAIF_DeviceTensor indices=UploadI32(idx,{tokens,top_k},stream,capacity==0?Dtype_e::Float32:Dtype_e::Int32);
    CAIF_DeviceTensor map=CAIF_DeviceTensor::Uninitialized({tokens,top_k},stream,indices.Dtype());
    CAIF_DeviceTensor offsets=CAIF_DeviceTensor::Uninitialized({experts+1},stream,indices.Dtype());
    const uint32_t total=CAIF_Ops::MoEBuildDispatchMap(indices,experts,top_k,capacity,map,offsets);
    const std::vector<int32_t> m=DownloadI32(map),off=DownloadI32(offsets);
    // definition: position = number of earlier assignments to the same expert, dropped at the capacity
    bool ok=off[0]==0&&static_cast<uint32_t>(off[experts])==total&&total>0&&total<=tokens*top_k;
    std::vector<int32_t> seen(experts,0);
    for(size_t a=0;a<idx.size();++a)
    {
      int32_t want=-1;
      if(idx[a]>=0)
      {
        const int32_t kept=off[idx[a]+1]-off[idx[a]];
        if(seen[idx[a]]<kept){want=seen[idx[a]];}
        ++seen[idx[a]];
      }
      ok=ok&&m[a]==want;
    }
    for(uint32_t e=0;e<experts;++e)
    {
      const int32_t expect=capacity>0?std::min<int32_t>(seen[e],static_cast<int32_t>(capacity)):seen[e];
      ok=ok&&off[e+1]-off[e]==expect;
    }
    Report(capacity==0?"dispatch map: arrival-order positions, offsets, total":"dispatch map with a capacity limit",ok);

    CAIF_DeviceTensor x=Upload(Uniform(tokens*dim,-1,1,11),{tokens,dim},stream);
    CAIF_DeviceTensor buffer=CAIF_DeviceTensor::Zeros({total,dim},stream,Dtype_e::Float32);
    CAIF_Ops::MoEDispatchGPU(x,indices,map,offsets,top_k,buffer);
    const std::vector<float> xh=Download(x),bh=Download(buffer);
    ok=true;
    for(size_t a=0;a<idx.size();++a)
    {
      if(m[a]<0){continue;}
      const size_t row=static_cast<size_t>(off[idx[a]]+m[a]);
      ok=ok&&std::memcmp(&bh[row*dim],&xh[(a/top_k)*dim],dim*sizeof(float))==0;
    }
    Report("dispatch copies every kept token row to its slot",ok&&MaxAbs(bh)>0.0f);

    std::vector<float> wh=Uniform(tokens*top_k,0.1f,1.0f,12);
    CAIF_DeviceTensor w=Upload(wh,{tokens,top_k},stream);
    CAIF_DeviceTensor out=CAIF_DeviceTensor::Zeros({tokens,dim},stream,Dtype_e::Float32);
    CAIF_Ops::MoECombineGPU(buffer,indices,w,map,offsets,top_k,out);
    const std::vector<float> oh=Download(out);
    ok=true;
    for(uint32_t t=0;t<tokens;++t)
    {
      for(uint32_t d=0;d<dim;++d)
      {
        float sum=0.0f;
        for(uint32_t k=0;k<top_k;++k)
        {
          if(m[t*top_k+k]>=0){sum=std::fmaf(wh[t*top_k+k],xh[t*dim+d],sum);}
        }
        ok=ok&&oh[t*dim+d]==sum;
      }
    }
    Report("combine: fp32 weighted sum over the kept assignments in order",ok&&MaxAbs(oh)>0.0f);

    CAIF_DeviceTensor g=Upload(Uniform(tokens*dim,-1,1,13),{tokens,dim},stream);
    CAIF_DeviceTensor gbuf=CAIF_DeviceTensor::Zeros({total,dim},stream,Dtype_e::Float32);
    CAIF_DeviceTensor gw=CAIF_DeviceTensor::Zeros({tokens,top_k},stream,Dtype_e::Float32);
    CAIF_Ops::MoECombineBackwardGPU(g,buffer,indices,w,map,offsets,top_k,gbuf,gw);
    CAIF_DeviceTensor gin=CAIF_DeviceTensor::Zeros({tokens,dim},stream,Dtype_e::Float32);
    CAIF_Ops::MoEDispatchBackwardGPU(gbuf,indices,map,offsets,top_k,gin);
    const std::vector<float> gh=Download(g),gih=Download(gin),gwh=Download(gw);
    ok=true;
    bool okw=true;
    for(uint32_t t=0;t<tokens;++t)
    {
      for(uint32_t d=0;d<dim;++d)
      {
        float sum=0.0f;
        for(uint32_t k=0;k<top_k;++k)
        {
          if(m[t*top_k+k]>=0){sum+=wh[t*top_k+k]*gh[t*dim+d];}
        }
        ok=ok&&gih[t*dim+d]==sum;
      }
      for(uint32_t k=0;k<top_k;++k)
      {
        double dot=0.0;
        if(m[t*top_k+k]>=0)
        {
          for(uint32_t d=0;d<dim;++d){dot+=static_cast<double>(gh[t*dim+d])*xh[t*dim+d];}
        }
        okw=okw&&std::fabs(gwh[t*top_k+k]-dot)<=1e-5*(1.0+std::fabs(dot));
      }
    }
    Report("backward: grad_expert_buffer then dispatch backward equals the weighted gradient sum",ok);
    Report("backward: grad_weights is the row dot product, zero for dropped assignments",okw);
  }

  CAIF_DeviceTensor indices=UploadI32(idx,{tokens,top_k},stream);
  CAIF_DeviceTensor map=CAIF_DeviceTensor::Uninitialized({tokens,top_k},stream,Dtype_e::Int32);
  CAIF_DeviceTensor offsets=CAIF_DeviceTensor::Uninitialized({experts+1},stream,Dtype_e::Int32);
  CAIF_DeviceTensor flat=UploadI32(idx,{tokens*top_k},stream);
  Report("1-D indices throw",Throws([&]{CAIF_Ops::MoEBuildDispatchMap(flat,experts,top_k,0,map,offsets);},"must be 2D"));
  CAIF_DeviceTensor short_offsets=CAIF_DeviceTensor::Uninitialized({experts},stream,Dtype_e::Int32);
  Report("offsets of the wrong length throw",Throws([&]{CAIF_Ops::MoEBuildDispatchMap(indices,experts,top_k,0,map,short_offsets);},
                                                    "shape mismatch"));
  CAIF_Ops::MoEBuildDispatchMap(indices,experts,top_k,0,map,offsets);
  CAIF_DeviceTensor x=Upload(Uniform(tokens*dim,-1,1,11),{tokens,dim},stream);
  CAIF_DeviceTensor narrow=CAIF_DeviceTensor::Zeros({tokens*top_k,dim-1},stream,Dtype_e::Float32);
  Report("buffer of another width throws",Throws([&]{CAIF_Ops::MoEDispatchGPU(x,indices,map,offsets,top_k,narrow);},"mismatch"));
  CAIF_DeviceTensor half=CAIF_DeviceTensor::Zeros({tokens*top_k,dim},stream,Dtype_e::Float16);
  Report("buffer of another dtype throws",Throws([&]{CAIF_Ops::MoEDispatchGPU(x,indices,map,offsets,top_k,half);},"mismatch"));
}

int main(int argc,char **argv)
{
  const bool cpu_only=argc>1&&std::string(argv[1])=="--cpu";
  CAIF_DeviceTensor host=CAIF_DeviceTensor::HostZeros({4,2},Dtype_e::Int32);
  CAIF_DeviceTensor hmap=CAIF_DeviceTensor::HostZeros({4,2},Dtype_e::Int32);
  CAIF_DeviceTensor hoff=CAIF_DeviceTensor::HostZeros({3},Dtype_e::Int32);
  Report("host tensors are rejected",Throws([&]{CAIF_Ops::MoEBuildDispatchMap(host,2,2,0,hmap,hoff);},"host backend not supported"));
  if(!cpu_only&&HasGpu()){GpuTests();}
  return FinalExitCode();
}
