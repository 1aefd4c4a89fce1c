// SafeTensors files for tensors of the frozen quantized-linear path, quantised storage included.
//
// Same public names and error texts as the reference's CAIF_SafeTensorsFormat
// (include/caif/caif_safetensors_format.h:37-120, src/caif_safetensors_format.cpp:40-520): an
// 8-byte little-endian header length, a JSON header (padded with spaces to a multiple of 8), then
// the tensors' raw bytes back to back in header order; dtype tags "F32","F16","BF16","I8","I4",
// "U8","I32" (include/caif/caif_serialization_constants.h:210-223), "I4" being the reference's own
// tag for packed int4 whose byte count is ceil(elements/2) (include/caif/caif_data_type.h:80-87);
// the limits of include/caif/caif_constants.h:493-495.  The reference can tag I8/I4 but only ever
// exports frozen weights as fp32 (src/caif_device_frozen_linear.cpp:760-826); here the codes and
// their scales go to disk as they sit in memory (CAIF_DeviceFrozenLinear::ExportQuantized).
//
// Unlike the reference, the file logic is separated from device memory: WriteHost / ReadHeader /
// ParseTensorInfos / ReadTensorBytes work on host buffers (and are tested without a GPU against
// the `safetensors` Python package), Save / Load add the copies to and from CAIF_DeviceTensor.
#pragma once

#include <cstdint>
#include <cstdio>
#include <fstream>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "caif_cuda_stream.h"
#include "caif_data_type.h"
#include "caif_device_tensor.h"
#include "caif_exception.h"

namespace instance
{

constexpr uint64_t g_caif_safetensors_max_file_size=2ULL<<40;
constexpr size_t g_caif_safetensors_max_tensors=4096;
constexpr size_t g_caif_safetensors_max_header_size=100*1024*1024;

class CAIF_SafeTensorsFormat
{
  public:
    typedef CAIF_DataType::CAIF_DataType_e Dtype_e;

    struct SafeTensorInfo_t
    {
      std::string dtype;
      std::vector<uint32_t> shape;
      uint64_t data_offset_start;
      uint64_t data_offset_end;
    };
    // one tensor of the writer, in host memory
    struct HostTensor_t
    {
      std::string name;
      Dtype_e dtype;
      std::vector<uint32_t> shape;
      const void *data;
      size_t bytes;
    };

    static const char *DtypeToSafeTensorsName(Dtype_e dt)
    {
      switch(dt)
      {
        case Dtype_e::Float32:return "F32";
        case Dtype_e::Float16:return "F16";
        case Dtype_e::BFloat16:return "BF16";
        case Dtype_e::Int8:return "I8";
        case Dtype_e::Int4:return "I4";
        case Dtype_e::UInt8:return "U8";
        case Dtype_e::Int32:return "I32";
      }
      THROW_CAIFE("CAIF_SafeTensorsFormat::DtypeToSafeTensorsName: unsupported dtype");
    }
    static Dtype_e DtypeFromSafeTensorsName(const std::string &name)
    {
      static const Dtype_e all[]={Dtype_e::Float32,Dtype_e::Float16,Dtype_e::BFloat16,Dtype_e::Int8,Dtype_e::Int4,
                                  Dtype_e::UInt8,Dtype_e::Int32};
      for(Dtype_e dt:all)
      {
        if(name==DtypeToSafeTensorsName(dt))
        {
          return dt;
        }
      }
      THROW_CAIFE("CAIF_SafeTensorsFormat::DtypeFromSafeTensorsName: unrecognised name");
    }

    static std::string EscapeJsonString(const std::string &s)
    {
      std::string out;
      out.reserve(s.size()+8);
      for(const char c:s)
      {
        switch(c)
        {
          case '"':out+="\\\"";break;
          case '\\':out+="\\\\";break;
          case '\n':out+="\\n";break;
          case '\r':out+="\\r";break;
          case '\t':out+="\\t";break;
          default:out+=c;
        }
      }
      return out;
    }

    // Header text for `tensors` in this order; data_offsets receives start,end per tensor.  Tensors
    // are packed without gaps: the format's own validator rejects a file whose tensor i does not
    // start where tensor i-1 ends (src/caif_safetensors_format.cpp:161-168).
    static std::string BuildJsonHeader(const std::vector<HostTensor_t> &tensors,
                                       const std::map<std::string,std::string> &metadata,
                                       std::vector<uint64_t> &data_offsets)
    {
      std::string json="{";
      uint64_t offset=0;
      bool first=true;
      data_offsets.clear();
      for(const HostTensor_t &t:tensors)
      {
        size_t elements=1;
        for(const uint32_t d:t.shape)
        {
          elements*=d;
        }
        if(CAIF_DataType(t.dtype).StorageSizeBytes(elements)!=t.bytes)
        {
          THROW_CAIFE("SafeTensors: data size mismatch");
        }
        const uint64_t end=offset+t.bytes;
        data_offsets.push_back(offset);
        data_offsets.push_back(end);
        json+=first?"\"":",\"";
        first=false;
        json+=EscapeJsonString(t.name)+"\":{\"dtype\":\""+DtypeToSafeTensorsName(t.dtype)+"\",\"shape\":[";
        for(size_t i=0;i<t.shape.size();++i)
        {
          json+=(i>0?",":"")+std::to_string(t.shape[i]);
        }
        json+="],\"data_offsets\":["+std::to_string(offset)+","+std::to_string(end)+"]}";
        offset=end;
      }
      if(metadata.empty()==false)
      {
        json+=first?"\"__metadata__\":{":",\"__metadata__\":{";
        bool first_meta=true;
        for(const auto &kv:metadata)
        {
          json+=first_meta?"\"":",\"";
          first_meta=false;
          json+=EscapeJsonString(kv.first)+"\":\""+EscapeJsonString(kv.second)+"\"";
        }
        json+="}";
      }
      json+="}";
      return json;
    }

    static void WriteHost(const std::string &path,const std::vector<HostTensor_t> &tensors,
                          const std::map<std::string,std::string> &metadata=std::map<std::string,std::string>())
    {
      try
      {
        if(tensors.size()>g_caif_safetensors_max_tensors)
        {
          THROW_CAIFE("SafeTensors: too many tensors");
        }
        std::vector<uint64_t> offsets;
        std::string header=BuildJsonHeader(tensors,metadata,offsets);
        header.append((8-header.size()%8)%8,' ');
        if(header.size()>g_caif_safetensors_max_header_size)
        {
          THROW_CAIFE("SafeTensors: header too large");
        }
        std::ofstream out(path,std::ios::binary);
        if(out.is_open()==false)
        {
          THROW_CAIFE("SafeTensors: cannot open file for writing: "+path);
        }
        unsigned char len[8];
        const uint64_t n=header.size();
        for(int i=0;i<8;++i)
        {
          len[i]=static_cast<unsigned char>(n>>(8*i));
        }
        out.write(reinterpret_cast<const char*>(len),8);
        out.write(header.data(),static_cast<std::streamsize>(header.size()));
        for(const HostTensor_t &t:tensors)
        {
          out.write(static_cast<const char*>(t.data),static_cast<std::streamsize>(t.bytes));
        }
        out.close();
        if(out.fail()==true)
        {
          THROW_CAIFE("SafeTensors: write failed: "+path);
        }
      }
      CAIF_CATCH_BLOCK()
    }

    // The JSON header of a file; data_start = offset of the first tensor byte.
    static std::string ReadHeader(const std::string &path,uint64_t &data_start)
    {
      std::ifstream in(path,std::ios::binary|std::ios::ate);
      if(in.is_open()==false)
      {
        THROW_CAIFE("SafeTensors: cannot open file: "+path);
      }
      const std::streamoff size=in.tellg();
      in.seekg(0,std::ios::beg);
      if(size<8)
      {
        THROW_CAIFE("SafeTensors: file too small");
      }
      if(static_cast<uint64_t>(size)>g_caif_safetensors_max_file_size)
      {
        THROW_CAIFE("SafeTensors: file too large");
      }
      unsigned char len[8];
      in.read(reinterpret_cast<char*>(len),8);
      uint64_t header_size=0;
      for(int i=0;i<8;++i)
      {
        header_size|=static_cast<uint64_t>(len[i])<<(8*i);
      }
      if(header_size>g_caif_safetensors_max_header_size)
      {
        THROW_CAIFE("SafeTensors: header too large");
      }
      if(8+header_size>static_cast<uint64_t>(size))
      {
        THROW_CAIFE("SafeTensors: invalid header size");
      }
      std::string json(static_cast<size_t>(header_size),'\0');
      in.read(&json[0],static_cast<std::streamsize>(header_size));
      if(in.gcount()!=static_cast<std::streamsize>(header_size))
      {
        THROW_CAIFE("SafeTensors: short read loading header");
      }
      data_start=8+header_size;
      return json;
    }

    static std::map<std::string,SafeTensorInfo_t> ParseTensorInfos(const std::string &json)
    {
      std::map<std::string,SafeTensorInfo_t> infos;
      std::map<std::string,std::string> metadata;
      Parser(json).Run(infos,metadata);
      return infos;
    }
    static std::map<std::string,std::string> ParseMetadata(const std::string &json)
    {
      std::map<std::string,SafeTensorInfo_t> infos;
      std::map<std::string,std::string> metadata;
      Parser(json).Run(infos,metadata);
      return metadata;
    }

    // Raw bytes of one tensor, after checking its header entry against its dtype and shape and
    // against the file (src/caif_safetensors_format.cpp:297-361).
    static std::vector<char> ReadTensorBytes(const std::string &path,uint64_t data_start,const SafeTensorInfo_t &info)
    {
      const Dtype_e dtype=DtypeFromSafeTensorsName(info.dtype);
      size_t elements=1;
      for(const uint32_t d:info.shape)
      {
        elements*=d;
      }
      const size_t expected=CAIF_DataType(dtype).StorageSizeBytes(elements);
      if(info.data_offset_start>info.data_offset_end)
      {
        THROW_CAIFE("SafeTensors: data_offset_start exceeds data_offset_end");
      }
      if(info.data_offset_end-info.data_offset_start!=static_cast<uint64_t>(expected))
      {
        THROW_CAIFE("SafeTensors: data size mismatch");
      }
      std::ifstream in(path,std::ios::binary|std::ios::ate);
      if(in.is_open()==false)
      {
        THROW_CAIFE("SafeTensors: cannot open file: "+path);
      }
      const std::streamoff end=in.tellg();
      if(end<0)
      {
        THROW_CAIFE("SafeTensors: cannot determine file size");
      }
      const uint64_t file_size=static_cast<uint64_t>(end);
      if(data_start>file_size||info.data_offset_end>file_size-data_start)
      {
        THROW_CAIFE("SafeTensors: tensor data extends past end of file");
      }
      std::vector<char> bytes(expected);
      in.seekg(static_cast<std::streamoff>(data_start+info.data_offset_start));
      in.read(bytes.data(),static_cast<std::streamsize>(expected));
      if(in.gcount()!=static_cast<std::streamsize>(expected))
      {
        THROW_CAIFE("SafeTensors: short read loading tensor data");
      }
      return bytes;
    }

    // --- device tensors ---
    void Save(const std::string &path,const std::vector<std::pair<std::string,const CAIF_DeviceTensor*>> &tensors,
              const std::map<std::string,std::string> &metadata=std::map<std::string,std::string>())const
    {
      try
      {
        std::vector<std::vector<char>> staged;
        std::vector<HostTensor_t> host;
        staged.reserve(tensors.size());
        for(const auto &entry:tensors)
        {
          const CAIF_DeviceTensor *t=entry.second;
          if(t==nullptr)
          {
            continue;
          }
          staged.emplace_back(t->SizeBytes());
          t->CopyToHostRaw(staged.back().data());
          host.push_back(HostTensor_t{entry.first,t->Dtype(),t->Shape(),staged.back().data(),t->SizeBytes()});
        }
        WriteHost(path,host,metadata);
      }
      CAIF_CATCH_BLOCK()
    }
    std::map<std::string,CAIF_DeviceTensor> Load(const std::string &path,CAIF_CudaStream &stream)const
    {
      try
      {
        uint64_t data_start=0;
        const std::string json=ReadHeader(path,data_start);
        const std::map<std::string,SafeTensorInfo_t> infos=ParseTensorInfos(json);
        if(infos.size()>g_caif_safetensors_max_tensors)
        {
          THROW_CAIFE("SafeTensors: too many tensors");
        }
        std::map<std::string,CAIF_DeviceTensor> result;
        for(const auto &kv:infos)
        {
          const std::vector<char> bytes=ReadTensorBytes(path,data_start,kv.second);
          CAIF_DeviceTensor t=CAIF_DeviceTensor::Uninitialized(kv.second.shape,stream,
                                                               DtypeFromSafeTensorsName(kv.second.dtype));
          t.CopyFromHostRaw(bytes.data(),bytes.size());
          result.emplace(kv.first,std::move(t));
        }
        return result;
      }
      CAIF_CATCH_BLOCK()
    }
    std::map<std::string,SafeTensorInfo_t> TensorInfos(const std::string &path)const
    {
      try
      {
        uint64_t data_start=0;
        return ParseTensorInfos(ReadHeader(path,data_start));
      }
      CAIF_CATCH_BLOCK()
    }
    std::map<std::string,std::string> Metadata(const std::string &path)const
    {
      try
      {
        uint64_t data_start=0;
        return ParseMetadata(ReadHeader(path,data_start));
      }
      CAIF_CATCH_BLOCK()
    }

  private:
    // Recursive-descent reader for the header: one object whose members are tensor entries
    // ({"dtype":string,"shape":[ints],"data_offsets":[start,end]}, unknown members skipped) or
    // "__metadata__" (an object of strings; other value types there are skipped).
    class Parser
    {
      public:
        explicit Parser(const std::string &text):_s(text),_i(0){}
        void Run(std::map<std::string,SafeTensorInfo_t> &infos,std::map<std::string,std::string> &metadata)
        {
          Expect('{');
          if(Peek()!='}')
          {
            do
            {
              const std::string key=String();
              Expect(':');
              if(key=="__metadata__")
              {
                Metadata(metadata);
              }
              else
              {
                if(infos.count(key)!=0)
                {
                  THROW_CAIFE("SafeTensors: malformed header: duplicate tensor name");
                }
                infos.emplace(key,Tensor());
              }
            }
            while(Accept(','));
          }
          Expect('}');
          SkipSpace();
          if(_i!=_s.size())
          {
            THROW_CAIFE("SafeTensors: malformed header: text after the closing brace");
          }
        }

      private:
        void SkipSpace()
        {
          while(_i<_s.size()&&(_s[_i]==' '||_s[_i]=='\n'||_s[_i]=='\r'||_s[_i]=='\t'))
          {
            ++_i;
          }
        }
        char Peek()
        {
          SkipSpace();
          if(_i>=_s.size())
          {
            THROW_CAIFE("SafeTensors: malformed header: unexpected end");
          }
          return _s[_i];
        }
        bool Accept(char c)
        {
          if(Peek()==c)
          {
            ++_i;
            return true;
          }
          return false;
        }
        void Expect(char c)
        {
          if(Accept(c)==false)
          {
            THROW_CAIFE(std::string("SafeTensors: malformed header: expected '")+c+"'");
          }
        }
        static void AppendUtf8(std::string &out,uint32_t cp)
        {
          if(cp<0x80){out+=static_cast<char>(cp);}
          else if(cp<0x800)
          {
            out+=static_cast<char>(0xC0|(cp>>6));
            out+=static_cast<char>(0x80|(cp&0x3F));
          }
          else if(cp<0x10000)
          {
            out+=static_cast<char>(0xE0|(cp>>12));
            out+=static_cast<char>(0x80|((cp>>6)&0x3F));
            out+=static_cast<char>(0x80|(cp&0x3F));
          }
          else
          {
            out+=static_cast<char>(0xF0|(cp>>18));
            out+=static_cast<char>(0x80|((cp>>12)&0x3F));
            out+=static_cast<char>(0x80|((cp>>6)&0x3F));
            out+=static_cast<char>(0x80|(cp&0x3F));
          }
        }
        uint32_t Hex4()
        {
          if(_i+4>_s.size())
          {
            THROW_CAIFE("SafeTensors: malformed header: short \\u escape");
          }
          uint32_t v=0;
          for(int k=0;k<4;++k)
          {
            const char c=_s[_i++];
            v<<=4;
            if(c>='0'&&c<='9'){v|=static_cast<uint32_t>(c-'0');}
            else if(c>='a'&&c<='f'){v|=static_cast<uint32_t>(c-'a'+10);}
            else if(c>='A'&&c<='F'){v|=static_cast<uint32_t>(c-'A'+10);}
            else{THROW_CAIFE("SafeTensors: malformed header: bad \\u escape");}
          }
          return v;
        }
        std::string String()
        {
          Expect('"');
          std::string out;
          while(true)
          {
            if(_i>=_s.size())
            {
              THROW_CAIFE("SafeTensors: malformed header: unterminated string");
            }
            const char c=_s[_i++];
            if(c=='"')
            {
              return out;
            }
            if(c!='\\')
            {
              out+=c;
              continue;
            }
            if(_i>=_s.size())
            {
              THROW_CAIFE("SafeTensors: malformed header: unterminated escape");
            }
            const char e=_s[_i++];
            switch(e)
            {
              case '"':out+='"';break;
              case '\\':out+='\\';break;
              case '/':out+='/';break;
              case 'b':out+='\b';break;
              case 'f':out+='\f';break;
              case 'n':out+='\n';break;
              case 'r':out+='\r';break;
              case 't':out+='\t';break;
              case 'u':
              {
                uint32_t cp=Hex4();
                if(cp>=0xD800&&cp<0xDC00&&_i+1<_s.size()&&_s[_i]=='\\'&&_s[_i+1]=='u')
                {
                  _i+=2;
                  const uint32_t lo=Hex4();
                  cp=0x10000+((cp-0xD800)<<10)+(lo-0xDC00);
                }
                AppendUtf8(out,cp);
                break;
              }
              default:THROW_CAIFE("SafeTensors: malformed header: unknown escape");
            }
          }
        }
        uint64_t Unsigned()
        {
          SkipSpace();
          if(_i>=_s.size()||_s[_i]<'0'||_s[_i]>'9')
          {
            THROW_CAIFE("SafeTensors: malformed header: expected a non-negative integer");
          }
          uint64_t v=0;
          while(_i<_s.size()&&_s[_i]>='0'&&_s[_i]<='9')
          {
            const uint64_t digit=static_cast<uint64_t>(_s[_i]-'0');
            if(v>(UINT64_MAX-digit)/10)
            {
              THROW_CAIFE("SafeTensors: malformed header: integer out of range");
            }
            v=v*10+digit;
            ++_i;
          }
          return v;
        }
        std::vector<uint64_t> UnsignedArray()
        {
          std::vector<uint64_t> v;
          Expect('[');
          if(Peek()!=']')
          {
            do
            {
              v.push_back(Unsigned());
            }
            while(Accept(','));
          }
          Expect(']');
          return v;
        }
        // any JSON value, ignored
        void SkipValue()
        {
          const char c=Peek();
          if(c=='"')
          {
            (void)String();
          }
          else if(c=='{'||c=='[')
          {
            const char close=(c=='{')?'}':']';
            ++_i;
            if(Peek()!=close)
            {
              do
              {
                if(c=='{')
                {
                  (void)String();
                  Expect(':');
                }
                SkipValue();
              }
              while(Accept(','));
            }
            Expect(close);
          }
          else
          {
            const size_t start=_i;
            while(_i<_s.size()&&_s[_i]!=','&&_s[_i]!='}'&&_s[_i]!=']'&&_s[_i]!=' '&&_s[_i]!='\n'&&_s[_i]!='\r'&&
                  _s[_i]!='\t')
            {
              ++_i;
            }
            if(_i==start)
            {
              THROW_CAIFE("SafeTensors: malformed header: expected a value");
            }
          }
        }
        SafeTensorInfo_t Tensor()
        {
          SafeTensorInfo_t info{std::string(),std::vector<uint32_t>(),0,0};
          bool have_dtype=false;
          bool have_shape=false;
          bool have_offsets=false;
          Expect('{');
          if(Peek()!='}')
          {
            do
            {
              const std::string key=String();
              Expect(':');
              if(key=="dtype")
              {
                info.dtype=String();
                have_dtype=true;
              }
              else if(key=="shape")
              {
                for(const uint64_t d:UnsignedArray())
                {
                  if(d>UINT32_MAX)
                  {
                    THROW_CAIFE("SafeTensors: malformed header: dimension out of range");
                  }
                  info.shape.push_back(static_cast<uint32_t>(d));
                }
                have_shape=true;
              }
              else if(key=="data_offsets")
              {
                const std::vector<uint64_t> o=UnsignedArray();
                if(o.size()!=2)
                {
                  THROW_CAIFE("SafeTensors: malformed header: data_offsets needs two entries");
                }
                info.data_offset_start=o[0];
                info.data_offset_end=o[1];
                have_offsets=true;
              }
              else
              {
                SkipValue();
              }
            }
            while(Accept(','));
          }
          Expect('}');
          if(have_dtype==false||have_shape==false||have_offsets==false)
          {
            THROW_CAIFE("SafeTensors: malformed header: tensor entry lacks dtype, shape or data_offsets");
          }
          return info;
        }
        void Metadata(std::map<std::string,std::string> &metadata)
        {
          Expect('{');
          if(Peek()!='}')
          {
            do
            {
              const std::string key=String();
              Expect(':');
              if(Peek()=='"')
              {
                metadata[key]=String();
              }
              else
              {
                SkipValue();
              }
            }
            while(Accept(','));
          }
          Expect('}');
        }

        const std::string &_s;
        size_t _i;
    };
};

}//end instance namespace
