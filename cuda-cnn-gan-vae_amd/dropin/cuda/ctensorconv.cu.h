// Drop-in for the reference's cuda/ctensorconv.cu.h (class at :48-69): the four static functions with the reference's
// signatures, each one C-ABI call.
#ifndef C_TENSOR_CONV_CU_H
#define C_TENSOR_CONV_CU_H

#include "ctensor.cu.h"
#include "ctensormath.cu.h"

template<class type_t>
class CTensorConv
{
 private:
  static void OnlyFloat(void) {static_assert(std::is_same<type_t,float>::value,"the MI355X tensor path computes in fp32 only");}
 public:
  static void ForwardConvolution(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Image,const CTensor<type_t> &cTensor_Kernel,int32_t kernel_x,int32_t kernel_y,int32_t kernel_z,uint32_t kernel_amount,const CTensor<type_t> &cTensor_Bias,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Image.Device(true),k=cTensor_Kernel.Device(true),b=cTensor_Bias.Device(true),o=cTensor_Output.Device(false);
   mi355::Check(mt_forward_convolution(&o,&i,&k,kernel_x,kernel_y,kernel_z,kernel_amount,&b,stride_x,stride_y,padding_x,padding_y));
   cTensor_Output.SetDeviceOnChange();
  }
  static void BackwardConvolution(CTensor<type_t> &cTensor_OutputDelta,const CTensor<type_t> &cTensor_Delta,const CTensor<type_t> &cTensor_Kernel,int32_t kernel_x,int32_t kernel_y,int32_t kernel_z,uint32_t kernel_amount,const CTensor<type_t> &cTensor_Bias,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   mt_tensor d=cTensor_Delta.Device(true),k=cTensor_Kernel.Device(true),b=cTensor_Bias.Device(true),o=cTensor_OutputDelta.Device(false);
   mi355::Check(mt_backward_convolution(&o,&d,&k,kernel_x,kernel_y,kernel_z,kernel_amount,&b,stride_x,stride_y,padding_x,padding_y));
   cTensor_OutputDelta.SetDeviceOnChange();
  }
  static void CreateDeltaWeightAndBias(CTensor<type_t> &cTensor_dKernel,int32_t dkernel_x,int32_t dkernel_y,int32_t dkernel_z,uint32_t dkernel_amount,CTensor<type_t> &cTensor_dBias,const CTensor<type_t> &cTensor_Image,CTensor<type_t> &cTensor_Delta,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   // both gradients accumulate: bring their device copies up to date first
   mt_tensor dk=cTensor_dKernel.Device(true),db=cTensor_dBias.Device(true),i=cTensor_Image.Device(true),d=cTensor_Delta.Device(true);
   mi355::Check(mt_create_delta_weight_and_bias(&dk,dkernel_x,dkernel_y,dkernel_z,dkernel_amount,&db,&i,&d,stride_x,stride_y,padding_x,padding_y));
   cTensor_dKernel.SetDeviceOnChange();
   cTensor_dBias.SetDeviceOnChange();
  }
  static void CreateBackDeltaWeightAndBias(CTensor<type_t> &cTensor_dKernel,int32_t dkernel_x,int32_t dkernel_y,int32_t dkernel_z,uint32_t dkernel_amount,CTensor<type_t> &cTensor_dBias,CTensor<type_t> &cTensor_Image,const CTensor<type_t> &cTensor_Delta,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   mt_tensor dk=cTensor_dKernel.Device(true),db=cTensor_dBias.Device(true),i=cTensor_Image.Device(true),d=cTensor_Delta.Device(true);
   mi355::Check(mt_create_back_delta_weight_and_bias(&dk,dkernel_x,dkernel_y,dkernel_z,dkernel_amount,&db,&i,&d,stride_x,stride_y,padding_x,padding_y));
   cTensor_dKernel.SetDeviceOnChange();
   cTensor_dBias.SetDeviceOnChange();
  }
};

#endif
