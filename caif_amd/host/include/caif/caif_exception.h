// Exception type and throw/catch macros of the host layer.
// Mirrors include/caif/caif_exception.h:23-62 of the reference: THROW_CAIFE(desc) raises a
// CAIF_Exception carrying line/file/function/description; CAIF_CATCH_BLOCK() appends a trace
// frame and rethrows (the reference also logs through ISE_Out, which this build leaves out).
#pragma once

#include <exception>
#include <string>

namespace instance
{

class CAIF_Exception:public std::exception
{
  public:
    CAIF_Exception(int line,const char *file,const char *func,const std::string &desc):_desc(desc)
    {
      AddTrace(line,file,func);
    }
    const char *what()const noexcept override{return _what.c_str();}
    const std::string &Description()const{return _desc;}
    void AddTrace(int line,const char *file,const char *func)
    {
      _trace+=std::string("\n  at ")+func+" ("+file+":"+std::to_string(line)+")";
      _what=_desc+_trace;
    }

  private:
    std::string _desc;
    std::string _trace;
    std::string _what;
};

}//end instance namespace

#define THROW_CAIFE(desc) throw instance::CAIF_Exception(__LINE__,__FILE__,__func__,(desc))

#define CAIF_CATCH_BLOCK() \
  catch(instance::CAIF_Exception &caif_e_) \
  { \
    caif_e_.AddTrace(__LINE__,__FILE__,__func__); \
    throw; \
  } \
  catch(const std::exception &std_e_) \
  { \
    throw instance::CAIF_Exception(__LINE__,__FILE__,__func__,std_e_.what()); \
  }
