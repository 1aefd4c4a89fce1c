// Quantised storage on disk: CAIF_SafeTensorsFormat (names, limits and error texts of the reference's
// src/caif_safetensors_format.cpp:269-520) and CAIF_DeviceFrozenLinear::ExportQuantized / ImportQuantized.
//   --cpu            host-level checks only (writer, header reader, parser, error contracts)
//   --write <path>   write a fixed file of standard dtypes for another SafeTensors reader to check
//   --write-quantized <path>   write the I8 / I4 / F16 / F32 sample of the host checks (header layout check)
//   --read <path>    print every tensor of a file (name|dtype|shape|hex bytes) and its metadata
//   (no argument)    everything, including save -> load -> forward on the GPU
#include <algorithm>
#include <cstdio>
#include <fstream>

#include "caif/caif_device_frozen_linear_factory.h"
#include "caif/caif_safetensors_format.h"
#include "caif_test_harness.h"

using namespace instance;
using namespace caif_test;
typedef CAIF_Ops::QuantScheme_e Scheme;
typedef CAIF_SafeTensorsFormat Fmt;

static std::string TmpPath(const std::string &name)
{
  const char *dir=std::getenv("TMPDIR");
  return std::string(dir!=nullptr?dir:"/tmp")+"/caif_st_"+std::to_string(static_cast<long>(getpid()))+"_"+name;
}
static void WriteRaw(const std::string &path,const std::string &bytes)
{
  std::ofstream out(path,std::ios::binary);
  out.write(bytes.data(),static_cast<std::streamsize>(bytes.size()));
}
static std::string ReadRaw(const std::string &path)
{
  std::ifstream in(path,std::ios::binary);
  return std::string((std::istreambuf_iterator<char>(in)),std::istreambuf_iterator<char>());
}
// a file with the given header text (length prefix added) and `data_bytes` bytes of payload
static void WriteWithHeader(const std::string &path,const std::string &json,size_t data_bytes)
{
  std::string f(8,'\0');
  for(int i=0;i<8;++i)
  {
    f[i]=static_cast<char>((static_cast<uint64_t>(json.size())>>(8*i))&0xFF);
  }
  WriteRaw(path,f+json+std::string(data_bytes,'\x5a'));
}

// the fixed content of --write: name, dtype, shape, bytes = (17*i + seed) mod 251
struct Fixed{const char *name;Dtype_e dtype;std::vector<uint32_t> shape;int seed;};
static std::vector<Fixed> FixedTensors()
{
  return {{"layer.0.weight",Dtype_e::Int8,{3u,4u},1},{"bytes",Dtype_e::UInt8,{5u},2},{"half",Dtype_e::Float16,{2u,2u},3},
          {"single",Dtype_e::Float32,{3u},4},{"brain",Dtype_e::BFloat16,{4u},5},{"ints",Dtype_e::Int32,{2u},6}};
}
static std::vector<char> FixedBytes(const Fixed &f)
{
  size_t n=1;
  for(uint32_t d:f.shape){n*=d;}
  std::vector<char> b(CAIF_DataType(f.dtype).StorageSizeBytes(n));
  for(size_t i=0;i<b.size();++i)
  {
    // keep float patterns finite: the top byte of every element stays small
    const size_t es=CAIF_DataType(f.dtype).ElementSizeBytes();
    const int v=static_cast<int>((17*i+f.seed)%251);
    b[i]=static_cast<char>((CAIF_DataType(f.dtype).IsFloat()==true&&i%es==es-1)?(v&0x3F):v);
  }
  return b;
}

static int WriteFixed(const std::string &path)
{
  std::vector<std::vector<char>> keep;
  std::vector<Fmt::HostTensor_t> tensors;
  for(const Fixed &f:FixedTensors())
  {
    keep.push_back(FixedBytes(f));
    tensors.push_back({f.name,f.dtype,f.shape,keep.back().data(),keep.back().size()});
  }
  Fmt::WriteHost(path,tensors,{{"format","pt"},{"note","quote \" backslash \\ tab \t"}});
  return 0;
}

static int DumpFile(const std::string &path)
{
  uint64_t data_start=0;
  const std::string json=Fmt::ReadHeader(path,data_start);
  for(const auto &kv:Fmt::ParseTensorInfos(json))
  {
    std::printf("%s|%s|",kv.first.c_str(),kv.second.dtype.c_str());
    for(size_t i=0;i<kv.second.shape.size();++i){std::printf(i>0?",%u":"%u",kv.second.shape[i]);}
    std::printf("|");
    for(const char c:Fmt::ReadTensorBytes(path,data_start,kv.second)){std::printf("%02x",static_cast<unsigned char>(c));}
    std::printf("\n");
  }
  for(const auto &kv:Fmt::ParseMetadata(json))
  {
    std::printf("meta|%s|%s\n",kv.first.c_str(),kv.second.c_str());
  }
  return 0;
}

// I8 codes, 15 packed I4 codes (the odd tail's high nibble is 0), F16 and F32 scales, a name that needs escaping
static const std::vector<int8_t> g_codes8={-127,-1,0,1,2,3,4,5,6,7,8,127};
static const std::vector<uint8_t> g_codes4={0x21,0x43,0x65,0x87,0xA9,0xCB,0xED,0x0F};
static const std::vector<uint16_t> g_s16={0x3C00,0x2E66};
static const std::vector<float> g_s32={0.015625f};
static const std::string g_odd_name="blk \"q\"\\w\n";
static std::vector<Fmt::HostTensor_t> QuantizedSample()
{
  return {{"ffn.weight",Dtype_e::Int8,{3u,4u},g_codes8.data(),12},{g_odd_name,Dtype_e::Int4,{3u,5u},g_codes4.data(),8},
          {"ffn.scales",Dtype_e::Float16,{2u},g_s16.data(),4},{"t.scales",Dtype_e::Float32,{1u},g_s32.data(),4}};
}
static const std::map<std::string,std::string> g_sample_meta={{"ffn.group_size","128"},{"ffn.int8_scheme","per_channel"}};

static void HostTests()
{
  const std::string path=TmpPath("host.safetensors");
  const std::vector<uint8_t> &codes4=g_codes4;
  const std::string &odd_name=g_odd_name;
  const std::vector<Fmt::HostTensor_t> tensors=QuantizedSample();
  const std::map<std::string,std::string> &meta=g_sample_meta;
  Fmt::WriteHost(path,tensors,meta);

  uint64_t data_start=0;
  const std::string json=Fmt::ReadHeader(path,data_start);
  const std::string raw=ReadRaw(path);
  Report("header length is a multiple of 8 and the payload follows it",json.size()%8==0&&data_start==8+json.size()&&
                                                                     raw.size()==data_start+12+8+4+4);
  const auto infos=Fmt::ParseTensorInfos(json);
  bool ok=infos.size()==4&&infos.count(odd_name)==1;
  if(ok==true)
  {
    const Fmt::SafeTensorInfo_t &w=infos.at("ffn.weight");
    const Fmt::SafeTensorInfo_t &q=infos.at(odd_name);
    ok=w.dtype=="I8"&&w.shape==std::vector<uint32_t>({3u,4u})&&w.data_offset_start==0&&w.data_offset_end==12&&
       q.dtype=="I4"&&q.shape==std::vector<uint32_t>({3u,5u})&&q.data_offset_start==12&&q.data_offset_end==20&&
       infos.at("ffn.scales").dtype=="F16"&&infos.at("ffn.scales").data_offset_start==20&&
       infos.at("t.scales").dtype=="F32"&&infos.at("t.scales").data_offset_end==28;
  }
  Report("entries: dtype tags, shapes, back-to-back offsets, I4 takes ceil(n/2) bytes, escaped name survives",ok);
  Report("metadata round trip",Fmt::ParseMetadata(json)==meta);
  bool same=true;
  for(const Fmt::HostTensor_t &t:tensors)
  {
    const std::vector<char> b=Fmt::ReadTensorBytes(path,data_start,infos.at(t.name));
    same=same&&b.size()==t.bytes&&std::memcmp(b.data(),t.data,t.bytes)==0;
  }
  Report("tensor bytes round trip",same);

  // reader tolerance: whitespace, member order, unknown members, \u escapes, non-string metadata values
  const std::string loose=" {\n \"__metadata__\" : {\"k\":\"v\\u00e9\\ud83d\\ude00\",\"n\":3,\"o\":{\"x\":[1,2]}},\n"
                          "  \"a\\u0041\":{\"data_offsets\":[ 0 , 6 ],\"extra\":[{\"y\":null},true],\"shape\":[3],\"dtype\":\"F16\"} } ";
  const auto linfo=Fmt::ParseTensorInfos(loose);
  const auto lmeta=Fmt::ParseMetadata(loose);
  Report("parser: whitespace, any member order, unknown members, unicode escapes",
         linfo.size()==1&&linfo.count("aA")==1&&linfo.at("aA").dtype=="F16"&&linfo.at("aA").data_offset_end==6&&
         lmeta.size()==1&&lmeta.at("k")=="v\xC3\xA9\xF0\x9F\x98\x80");
  Report("empty header object is a file with no tensors",Fmt::ParseTensorInfos("{}").empty()&&Fmt::ParseMetadata("{}").empty());

  // error contracts
  Report("missing file throws",Throws([&]{uint64_t d;Fmt::ReadHeader(path+".absent",d);},"cannot open file"));
  const std::string bad=TmpPath("bad.safetensors");
  WriteRaw(bad,"abcd");
  Report("file shorter than the length prefix throws",Throws([&]{uint64_t d;Fmt::ReadHeader(bad,d);},"file too small"));
  WriteWithHeader(bad,"{}",0);
  {
    std::string f=ReadRaw(bad);
    f[0]=static_cast<char>(200);      // claims a 200-byte header in a 10-byte file
    WriteRaw(bad,f);
  }
  Report("header length beyond the file throws",Throws([&]{uint64_t d;Fmt::ReadHeader(bad,d);},"invalid header size"));
  {
    std::string f=ReadRaw(bad);
    f[0]=0;
    f[4]=1;                            // 2^32 bytes
    WriteRaw(bad,f);
  }
  Report("header length above the limit throws",Throws([&]{uint64_t d;Fmt::ReadHeader(bad,d);},"header too large"));
  const std::string entry="{\"t\":{\"dtype\":\"F32\",\"shape\":[4],\"data_offsets\":[0,16]}}";
  WriteWithHeader(bad,entry,8);
  Report("tensor data past the end of the file throws",Throws([&]
         {uint64_t d;const auto i=Fmt::ParseTensorInfos(Fmt::ReadHeader(bad,d));Fmt::ReadTensorBytes(bad,d,i.at("t"));},"extends past end of file"));
  Report("offsets that disagree with dtype and shape throw",Throws([&]
         {Fmt::SafeTensorInfo_t i{"F32",{4u},0,12};Fmt::ReadTensorBytes(path,data_start,i);},"data size mismatch")&&
         Throws([&]{Fmt::SafeTensorInfo_t i{"I4",{3u,5u},0,15};Fmt::ReadTensorBytes(path,data_start,i);},"data size mismatch"));
  Report("start after end throws",Throws([&]{Fmt::SafeTensorInfo_t i{"I8",{2u},8,6};Fmt::ReadTensorBytes(path,data_start,i);},
                                         "data_offset_start exceeds data_offset_end"));
  Report("unknown dtype tag throws",Throws([&]{Fmt::SafeTensorInfo_t i{"F8_E4M3",{2u},0,2};Fmt::ReadTensorBytes(path,data_start,i);},
                                           "unrecognised name"));
  Report("malformed headers throw",Throws([&]{Fmt::ParseTensorInfos("{\"t\":{\"dtype\":\"F32\",\"shape\":[4]}}");},"lacks dtype, shape or data_offsets")&&
                                   Throws([&]{Fmt::ParseTensorInfos("{\"t\":{\"dtype\":\"F32\",\"shape\":[-4],\"data_offsets\":[0,16]}}");},"non-negative integer")&&
                                   Throws([&]{Fmt::ParseTensorInfos("{\"t\":{\"dtype\":\"F32\",\"shape\":[4],\"data_offsets\":[0]}}");},"two entries")&&
                                   Throws([&]{Fmt::ParseTensorInfos("{\"t\":{\"dtype\":\"F32\"");},"malformed header")&&
                                   Throws([&]{Fmt::ParseTensorInfos("{} x");},"after the closing brace")&&
                                   Throws([&]{Fmt::ParseTensorInfos(entry.substr(0,entry.size()-1)+",\"t\":{\"dtype\":\"F32\",\"shape\":[4],\"data_offsets\":[0,16]}}");},"duplicate"));
  Report("writer refuses a byte count that does not match dtype and shape",Throws([&]
         {std::vector<Fmt::HostTensor_t> t={{"w",Dtype_e::Int4,{3u,5u},codes4.data(),7}};Fmt::WriteHost(bad,t);},"data size mismatch"));
  Report("writer refuses an unwritable path",Throws([&]{Fmt::WriteHost("/nonexistent-dir/x.safetensors",tensors);},"cannot open file for writing"));
  std::remove(path.c_str());
  std::remove(bad.c_str());
}

static const uint32_t K=256,N=24,M=5;

static std::unique_ptr<CAIF_DeviceLayer> Quantised(const std::vector<float> &w,Dtype_e storage,Scheme scheme,uint32_t group,
                                                   CAIF_CudaStream &stream,CAIF_RunContext &ctx)
{
  std::unique_ptr<CAIF_DeviceLayer> layer=CAIF_DeviceFrozenLinearFactory::Create(K,N,storage,stream,group,true,Dtype_e::BFloat16,scheme);
  CAIF_DeviceFrozenLinearBase *base=dynamic_cast<CAIF_DeviceFrozenLinearBase*>(layer.get());
  if(storage==Dtype_e::Int4)
  {
    CAIF_DeviceTensor in=Upload(w,{N*K},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({N,K},stream,Dtype_e::Int4);
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({(N*K+group-1)/group},stream,Dtype_e::Float16);
    CAIF_Ops::QuantizeInt4PerGroup(in,q,s,group,ctx);
    std::vector<uint16_t> sh(s.TotalElements());
    s.CopyToHostRaw(sh.data());
    base->LoadFromTensor(std::move(q));
    base->LoadScalesFromHost(sh.data(),sh.size()*sizeof(uint16_t));
  }
  else
  {
    CAIF_DeviceTensor in=Upload(w,{K,N},stream);
    CAIF_DeviceTensor q=CAIF_DeviceTensor::Zeros({K,N},stream,Dtype_e::Int8);
    CAIF_DeviceTensor s=CAIF_DeviceTensor::Zeros({scheme==Scheme::PerTensor_e?1u:N},stream,Dtype_e::Float32);
    CAIF_Ops::QuantizeInt8(in,q,s,scheme,ctx);
    std::vector<float> sh=Download(s);
    q.Reshape({N,K});                 // the layer reads the buffer as [out,in]
    base->LoadFromTensor(std::move(q));
    base->LoadScalesFromHost(sh.data(),sh.size()*sizeof(float));
  }
  return layer;
}

template<typename StorageT>
static CAIF_DeviceFrozenLinear<caif_bf16_t,StorageT> *Typed(const std::unique_ptr<CAIF_DeviceLayer> &layer)
{
  auto *typed=dynamic_cast<CAIF_DeviceFrozenLinear<caif_bf16_t,StorageT>*>(layer.get());
  if(typed==nullptr){THROW_CAIFE("test: layer is not the bf16-compute cell of this storage type");}
  return typed;
}

template<typename StorageT>
static void RoundTrip(const char *name,Dtype_e storage,Scheme scheme,uint32_t group,CAIF_CudaStream &stream,CAIF_RunContext &ctx)
{
  const std::vector<float> w=Uniform(N*K,-0.5f,0.5f,71);
  const std::vector<float> x=Uniform(M*K,-1.0f,1.0f,201);
  auto src=Quantised(w,storage,scheme,group,stream,ctx);
  CAIF_DeviceTensor in=Upload(x,{M,K},stream);
  const std::vector<float> want=Download(src->Forward(in,ctx));

  const std::string path=TmpPath(std::string(name)+".safetensors");
  std::vector<std::pair<std::string,const CAIF_DeviceTensor*>> tensors;
  std::map<std::string,std::string> meta;
  Typed<StorageT>(src)->ExportQuantized("blk.0.up.",tensors,meta);
  CAIF_SafeTensorsFormat fmt;
  fmt.Save(path,tensors,meta);

  const auto infos=fmt.TensorInfos(path);
  const bool int4=storage==Dtype_e::Int4;
  const uint64_t wbytes=int4?N*K/2:N*K;
  Report(std::string(name)+": file holds the codes in their storage type and the scales",
         infos.size()==2&&infos.at("blk.0.up.weight").dtype==(int4?"I4":"I8")&&
         infos.at("blk.0.up.weight").shape==std::vector<uint32_t>({N,K})&&
         infos.at("blk.0.up.weight").data_offset_end-infos.at("blk.0.up.weight").data_offset_start==wbytes&&
         infos.at("blk.0.up.scales").dtype==(int4?"F16":"F32")&&
         fmt.Metadata(path).at("blk.0.up.storage")==(int4?"int4":"int8"));

  auto loaded=fmt.Load(path,stream);
  const auto file_meta=fmt.Metadata(path);
  auto dst=CAIF_DeviceFrozenLinearFactory::Create(K,N,storage,stream,group,true,Dtype_e::BFloat16,scheme);
  Typed<StorageT>(dst)->ImportQuantized("blk.0.up.",loaded,file_meta);
  Report(std::string(name)+": save -> load -> forward is bit-identical",loaded.empty()==true&&Download(dst->Forward(in,ctx))==want);

  // a layer configured differently refuses the same file
  auto again=fmt.Load(path,stream);
  if(int4==true)
  {
    auto other=CAIF_DeviceFrozenLinearFactory::Create(K,N,storage,stream,group*2,true,Dtype_e::BFloat16,scheme);
    Report(std::string(name)+": other group size is refused",Throws([&]{Typed<StorageT>(other)->ImportQuantized("blk.0.up.",again,file_meta);},"group size"));
  }
  else
  {
    const Scheme flipped=scheme==Scheme::PerTensor_e?Scheme::PerChannel_e:Scheme::PerTensor_e;
    auto other=CAIF_DeviceFrozenLinearFactory::Create(K,N,storage,stream,group,true,Dtype_e::BFloat16,flipped);
    Report(std::string(name)+": other int8 scheme is refused",Throws([&]{Typed<StorageT>(other)->ImportQuantized("blk.0.up.",again,file_meta);},"int8 scheme"));
  }
  auto wrong_shape=CAIF_DeviceFrozenLinearFactory::Create(N,K,storage,stream,group,true,Dtype_e::BFloat16,scheme);
  Report(std::string(name)+": other dims are refused",Throws([&]{Typed<StorageT>(wrong_shape)->ImportQuantized("blk.0.up.",again,file_meta);},"weight shape"));
  Report(std::string(name)+": a missing tensor or metadata key is named",
         Throws([&]{Typed<StorageT>(dst)->ImportQuantized("blk.1.up.",again,file_meta);},"missing tensor blk.1.up.weight")&&
         Throws([&]{Typed<StorageT>(dst)->ImportQuantized("blk.0.up.",again,{});},"missing metadata blk.0.up.storage"));
  std::remove(path.c_str());
}

static void GpuTests()
{
  CAIF_CudaStream stream;
  CAIF_RunContext infer(stream,false);
  RoundTrip<int8_t>("int8 per-tensor",Dtype_e::Int8,Scheme::PerTensor_e,128,stream,infer);
  RoundTrip<int8_t>("int8 per-channel",Dtype_e::Int8,Scheme::PerChannel_e,128,stream,infer);
  RoundTrip<caif_int4_packed_t>("int4 group 64",Dtype_e::Int4,Scheme::PerTensor_e,64,stream,infer);
  {
    // storage type is checked against the file, not only against the metadata
    auto src=Quantised(Uniform(N*K,-0.5f,0.5f,3),Dtype_e::Int8,Scheme::PerTensor_e,128,stream,infer);
    std::vector<std::pair<std::string,const CAIF_DeviceTensor*>> tensors;
    std::map<std::string,std::string> meta;
    Typed<int8_t>(src)->ExportQuantized("",tensors,meta);
    const std::string path=TmpPath("mix.safetensors");
    CAIF_SafeTensorsFormat().Save(path,tensors,meta);
    auto loaded=CAIF_SafeTensorsFormat().Load(path,stream);
    auto int4_layer=CAIF_DeviceFrozenLinearFactory::Create(K,N,Dtype_e::Int4,stream,128,true,Dtype_e::BFloat16);
    Report("int8 file into an int4 layer is refused",Throws([&]{Typed<caif_int4_packed_t>(int4_layer)->ImportQuantized("",loaded,meta);},"storage type"));
    auto empty=CAIF_DeviceFrozenLinearFactory::Create(K,N,Dtype_e::Int8,stream,128,true,Dtype_e::BFloat16);
    Report("export before load throws",Throws([&]{Typed<int8_t>(empty)->ExportQuantized("",tensors,meta);},"must be loaded"));
    std::remove(path.c_str());
  }
  stream.Synchronize();
}

int main(int argc,char **argv)
{
  const std::string mode=argc>1?argv[1]:"";
  try
  {
    if(mode=="--write"&&argc>2){return WriteFixed(argv[2]);}
    if(mode=="--write-quantized"&&argc>2){Fmt::WriteHost(argv[2],QuantizedSample(),g_sample_meta);return 0;}
    if(mode=="--read"&&argc>2){return DumpFile(argv[2]);}
  }
  catch(const std::exception &e)
  {
    std::printf("error: %s\n",e.what());
    return 2;
  }
  const bool cpu_only=mode=="--cpu"||HasGpu()==false;
  try{HostTests();}
  catch(const std::exception &e){std::printf("unexpected exception: %s\n",e.what());Report("no unexpected exception",false);}
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
