// Tensor element types.  Mirrors include/caif/caif_data_type.h of the reference for the members
// the frozen quantized-linear path touches (names, element sizes, Int4 storage size :80-87).
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>

#include "caif_exception.h"
#include "caifx.h"

namespace instance
{

// Storage tag of a packed-int4 frozen weight (two codes per byte); never dereferenced.
struct caif_int4_packed_t{uint8_t byte;};
typedef _Float16 caif_fp16_t;     // the reference's __half
typedef __bf16 caif_bf16_t;       // the reference's __nv_bfloat16

class CAIF_DataType
{
  public:
    enum class CAIF_DataType_e:uint8_t{Float32,Float16,BFloat16,Int8,Int4,UInt8,Int32};

    explicit CAIF_DataType(CAIF_DataType_e v):_value(v){}
    CAIF_DataType_e Value()const{return _value;}

    size_t ElementSizeBytes()const
    {
      switch(_value)
      {
        case CAIF_DataType_e::Float32:return 4;
        case CAIF_DataType_e::Int32:return 4;
        case CAIF_DataType_e::Float16:return 2;
        case CAIF_DataType_e::BFloat16:return 2;
        default:return 1;
      }
    }
    // Bytes that hold n elements: two int4 codes share a byte.
    size_t StorageSizeBytes(size_t n)const
    {
      if(_value==CAIF_DataType_e::Int4)
      {
        return (n+1)/2;
      }
      return n*ElementSizeBytes();
    }
    std::string Name()const
    {
      switch(_value)
      {
        case CAIF_DataType_e::Float32:return "fp32";
        case CAIF_DataType_e::Float16:return "fp16";
        case CAIF_DataType_e::BFloat16:return "bf16";
        case CAIF_DataType_e::Int8:return "int8";
        case CAIF_DataType_e::Int4:return "int4";
        case CAIF_DataType_e::UInt8:return "uint8";
        default:return "int32";
      }
    }
    bool IsFloat()const
    {
      return _value==CAIF_DataType_e::Float32||_value==CAIF_DataType_e::Float16||
             _value==CAIF_DataType_e::BFloat16;
    }
    // caifx_dtype code of a float type
    int CaifxCode()const
    {
      switch(_value)
      {
        case CAIF_DataType_e::Float32:return CAIFX_F32;
        case CAIF_DataType_e::Float16:return CAIFX_F16;
        case CAIF_DataType_e::BFloat16:return CAIFX_BF16;
        default:THROW_CAIFE("CAIF_DataType: not a floating-point type");
      }
    }

  private:
    CAIF_DataType_e _value;
};

// compile-time map C++ type -> dtype enum
template<typename T> struct CAIF_DtypeOf;
template<> struct CAIF_DtypeOf<float>{static constexpr CAIF_DataType::CAIF_DataType_e value=CAIF_DataType::CAIF_DataType_e::Float32;};
template<> struct CAIF_DtypeOf<caif_fp16_t>{static constexpr CAIF_DataType::CAIF_DataType_e value=CAIF_DataType::CAIF_DataType_e::Float16;};
template<> struct CAIF_DtypeOf<caif_bf16_t>{static constexpr CAIF_DataType::CAIF_DataType_e value=CAIF_DataType::CAIF_DataType_e::BFloat16;};
template<> struct CAIF_DtypeOf<int8_t>{static constexpr CAIF_DataType::CAIF_DataType_e value=CAIF_DataType::CAIF_DataType_e::Int8;};
template<> struct CAIF_DtypeOf<caif_int4_packed_t>{static constexpr CAIF_DataType::CAIF_DataType_e value=CAIF_DataType::CAIF_DataType_e::Int4;};

}//end instance namespace
