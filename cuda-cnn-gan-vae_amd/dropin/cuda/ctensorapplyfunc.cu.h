// Drop-in for the reference's cuda/ctensorapplyfunc.cu.h (class at :60-...): the scalar functions (host side, same
// float/double promotions as cpu/ctensorapplyfunc.h:111-255) and the twelve tensor functions, one C-ABI call each.
#ifndef C_TENSOR_APPLY_FUNC_CU_H
#define C_TENSOR_APPLY_FUNC_CU_H

#include <math.h>

#include "ctensor.cu.h"
#include "ctensormath.cu.h"

template<class type_t>
class CTensorApplyFunc
{
 private:
  static void Apply(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,int func)
  {
   static_assert(std::is_same<type_t,float>::value,"the MI355X tensor path computes in fp32 only");
   if (&cTensor_Output!=&cTensor_Input && mi355::FusedFunction(func>=MT_F_DIFFERENTIAL?func-MT_F_DIFFERENTIAL:func)==true)
   {
    // A function layer's Forward, or the first call of its SetOutputError: deferred, since it may be the end of a
    // batch-norm layer's forward sequence or the beginning of its backward sequence (mi355::COpQueue).
    mt_tensor i=cTensor_Input.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
    if (func>=MT_F_DIFFERENTIAL) mi355::Queue().Submit(mi355::MakeDifferential(o,i,func-MT_F_DIFFERENTIAL));
                            else mi355::Queue().Submit(mi355::MakeFunction(o,i,func));
    cTensor_Output.SetDeviceOnChange();
    return;
   }
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_apply_func(&o,&i,func));
   cTensor_Output.SetDeviceOnChange();
  }
  static type_t Clamp30(type_t v)
  {
   if (v>30) v=static_cast<type_t>(29.99999);
   if (v<-30) v=static_cast<type_t>(-29.99999);
   return(v);
  }
 public:
  static type_t tanh(type_t v) {return(::tanh(v));}
  static type_t ch(type_t v) {return(cosh(v));}
  static type_t sech(type_t v) {return(1/ch(v));}

  static type_t Sigmoid(type_t v) {v=Clamp30(v);return(static_cast<type_t>(1.0/(1.0+exp(-v))));}
  static type_t ReLU(type_t v) {return(v>0?v:0);}
  static type_t GeLU(type_t v)
  {
   const type_t PI=static_cast<type_t>(3.141592654);
   type_t ft=static_cast<type_t>(sqrt(2/PI)*(v+0.044715*v*v*v));
   ft=tanh(ft);
   return(static_cast<type_t>(0.5*v*(1+ft)));
  }
  static type_t LeakyReLU(type_t v) {return(v>0?v:static_cast<type_t>(0.1*v));}
  static type_t Linear(type_t v) {return(v);}
  static type_t Tangence(type_t v) {return(tanh(Clamp30(v)));}

  static type_t dSigmoid(type_t v) {type_t s=Sigmoid(v);return(static_cast<type_t>((1.0-s)*s));}
  static type_t dReLU(type_t v) {return(v>=0?1:0);}
  static type_t dGeLU(type_t v)
  {
   const type_t PI=static_cast<type_t>(3.141592654);
   type_t ft=static_cast<type_t>(sqrt(2/PI)*(v+0.044715*v*v*v));
   type_t fa=static_cast<type_t>(sqrt(2/PI)*(1+3*0.044715*v*v));
   return(static_cast<type_t>(0.5*((1+tanh(ft))+0.5*v*sech(ft)*sech(ft))*fa));
  }
  static type_t dLeakyReLU(type_t v) {return(v>=0?1:static_cast<type_t>(0.1));}
  static type_t dLinear(type_t) {return(1);}
  static type_t dTangence(type_t v) {type_t t=Tangence(v);return(1-t*t);}

  static void ApplySigmoid(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_SIGMOID);}
  static void ApplyReLU(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_RELU);}
  static void ApplyGeLU(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_GELU);}
  static void ApplyLeakyReLU(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_LEAKY_RELU);}
  static void ApplyLinear(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_LINEAR);}
  static void ApplyTangence(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_TANGENCE);}

  static void ApplyDifferentialSigmoid(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_DIFFERENTIAL+MT_F_SIGMOID);}
  static void ApplyDifferentialReLU(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_DIFFERENTIAL+MT_F_RELU);}
  static void ApplyDifferentialGeLU(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_DIFFERENTIAL+MT_F_GELU);}
  static void ApplyDifferentialLeakyReLU(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_DIFFERENTIAL+MT_F_LEAKY_RELU);}
  static void ApplyDifferentialLinear(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_DIFFERENTIAL+MT_F_LINEAR);}
  static void ApplyDifferentialTangence(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input) {Apply(cTensor_Output,cTensor_Input,MT_F_DIFFERENTIAL+MT_F_TANGENCE);}
};

#endif
