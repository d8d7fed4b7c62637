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
  // Whether CreateDeltaWeightAndBias may keep the per-sample gradients uncomputed (mi355::CDeferredGradient): both
  // tensors were zeroed and not touched since, one slice per sample of the batch, the bias gradient [B,Kamt,1,1], and
  // enough gradients for the bookkeeping to matter (the record shares the operands' device blocks: holding them costs
  // nothing unless somebody overwrites an operand before the sums are taken, and then only a new block).
  static bool Deferrable(const CTensor<type_t> &dkernel,const CTensor<type_t> &dbias,const CTensor<type_t> &image,const CTensor<type_t> &delta)
  {
   if (mi355::DeferGradients()==false) return(false);
   if (dkernel.Lazy!=CTensor<type_t>::LAZY_ZERO || dbias.Lazy!=CTensor<type_t>::LAZY_ZERO || &dkernel==&dbias) return(false);
   const uint32_t batch=dkernel.GetSizeW();
   if (batch<2 || dbias.GetSizeW()!=batch || image.GetSizeW()!=batch || delta.GetSizeW()!=batch) return(false);
   if (dbias.GetSizeY()!=1 || dbias.GetSizeX()!=1) return(false);
   // (... or enough pixels: a layer with few filters on large images, whose per-sample gradients are small but each of
   // them is a sum over a whole image -- summed over the batch directly, that work spreads over the chip)
   return(dkernel.Count()>=(static_cast<size_t>(1)<<16) || delta.Count()>=(static_cast<size_t>(1)<<20));
  }
 public:
  static void ForwardConvolution(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Image,const CTensor<type_t> &cTensor_Kernel,int32_t kernel_x,int32_t kernel_y,int32_t kernel_z,uint32_t kernel_amount,const CTensor<type_t> &cTensor_Bias,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   if (cTensor_Image.Lazy==CTensor<type_t>::LAZY_UPSAMPLING && &cTensor_Output!=&cTensor_Image && kernel_x==3 && kernel_y==3 && stride_x==1 && stride_y==1 && padding_x==1 && padding_y==1)
   {
    // the image was never written: the convolution of the up-sampled image from its source (mi355::CDeferredUpSampling)
    const std::shared_ptr<mi355::CDeferredUpSampling> up=cTensor_Image.DeferredUpSampling;///<(kept alive over the call)
    const mt_tensor &source=up->SourceTensor;
    if (up->Factor_X==2 && up->Factor_Y==2 && cTensor_Image.GetSizeW()==source.w && cTensor_Image.GetSizeZ()==source.z &&
        cTensor_Image.GetSizeY()==2*source.y && cTensor_Image.GetSizeX()==2*source.x && source.z==static_cast<uint32_t>(kernel_z))
    {
     mt_tensor k=cTensor_Kernel.DeviceRead(),b=cTensor_Bias.DeviceRead(),o=cTensor_Output.Device(false);
     mi355::Check(mt_upsampling_convolution_func(&o,&source,2,2,&k,kernel_x,kernel_y,kernel_z,kernel_amount,&b,stride_x,stride_y,padding_x,padding_y,MT_F_NONE));
     cTensor_Output.SetDeviceOnChange();
     return;
    }
   }
   mt_tensor i=cTensor_Image.DeviceRead(),k=cTensor_Kernel.DeviceRead(),b=cTensor_Bias.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_forward_convolution(&o,&i,&k,kernel_x,kernel_y,kernel_z,kernel_amount,&b,stride_x,stride_y,padding_x,padding_y));
   cTensor_Output.SetDeviceOnChange();
  }
  static void BackwardConvolution(CTensor<type_t> &cTensor_OutputDelta,const CTensor<type_t> &cTensor_Delta,const CTensor<type_t> &cTensor_Kernel,int32_t kernel_x,int32_t kernel_y,int32_t kernel_z,uint32_t kernel_amount,const CTensor<type_t> &cTensor_Bias,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   const bool zeros=cTensor_Bias.HoldsZeros(),unwritten=(cTensor_Bias.Lazy==CTensor<type_t>::LAZY_ZERO);
   mt_tensor d=cTensor_Delta.DeviceRead(),k=cTensor_Kernel.DeviceRead(),b,o=cTensor_OutputDelta.Device(false);
   // Zeros come from one address for every call (mi355::ZeroBlock).  A tensor whose zeros were never written stays
   // unwritten; one that was filled is still brought up to date like any operand, so that the calls that wait in the
   // queue keep their order.
   if (unwritten==true) b=cTensor_Bias.Descriptor();
   else b=cTensor_Bias.DeviceRead();
   if (zeros==true) b.p=mi355::ZeroBlock(static_cast<size_t>(b.w)*b.z*b.y*b.x);
   mi355::Check(mt_backward_convolution(&o,&d,&k,kernel_x,kernel_y,kernel_z,kernel_amount,&b,stride_x,stride_y,padding_x,padding_y));
   cTensor_OutputDelta.SetDeviceOnChange();
  }
  static void CreateDeltaWeightAndBias(CTensor<type_t> &cTensor_dKernel,int32_t dkernel_x,int32_t dkernel_y,int32_t dkernel_z,uint32_t dkernel_amount,CTensor<type_t> &cTensor_dBias,const CTensor<type_t> &cTensor_Image,CTensor<type_t> &cTensor_Delta,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   if (Deferrable(cTensor_dKernel,cTensor_dBias,cTensor_Image,cTensor_Delta)==true)
   {
    // Two zeroed per-sample tensors: nothing is computed yet.  The record keeps the operands as they are (it shares their
    // blocks; a tensor that is written later takes a new one); AddSumW of the per-sample tensors computes their sums over
    // the batch, anybody else who reads them gets them computed then (mi355::CDeferredGradient).
    std::shared_ptr<mi355::CDeferredGradient> record(new mi355::CDeferredGradient);
    mt_tensor i=cTensor_Image.DeviceRead(),d=cTensor_Delta.DeviceRead();
    record->Kernel_X=dkernel_x;record->Kernel_Y=dkernel_y;record->Kernel_Z=dkernel_z;record->Kernel_Amount=dkernel_amount;
    record->Stride_X=stride_x;record->Stride_Y=stride_y;record->Padding_X=padding_x;record->Padding_Y=padding_y;
    const CTensor<type_t> *batch[2]={&cTensor_dKernel,&cTensor_dBias};
    uint32_t *size[2]={record->KernelSize,record->BiasSize};
    for(int n=0;n<2;n++)
    {
     size[n][0]=batch[n]->GetSizeW();size[n][1]=batch[n]->GetSizeZ();size[n][2]=batch[n]->GetSizeY();size[n][3]=batch[n]->GetSizeX();
    }
    record->Image=cTensor_Image.DeviceItem;
    record->Delta=cTensor_Delta.DeviceItem;
    record->ImageTensor=i;
    record->DeltaTensor=d;
    cTensor_dKernel.Lazy=CTensor<type_t>::LAZY_GRADIENT_KERNEL;cTensor_dKernel.Deferred=record;
    cTensor_dBias.Lazy=CTensor<type_t>::LAZY_GRADIENT_BIAS;cTensor_dBias.Deferred=record;
    return;
   }
   // both gradients accumulate: bring their device copies up to date first
   mt_tensor dk=cTensor_dKernel.Device(true),db=cTensor_dBias.Device(true),i=cTensor_Image.DeviceRead(),d=cTensor_Delta.DeviceRead();
   mi355::Check(mt_create_delta_weight_and_bias(&dk,dkernel_x,dkernel_y,dkernel_z,dkernel_amount,&db,&i,&d,stride_x,stride_y,padding_x,padding_y));
   cTensor_dKernel.SetDeviceOnChange();
   cTensor_dBias.SetDeviceOnChange();
  }
  static void CreateBackDeltaWeightAndBias(CTensor<type_t> &cTensor_dKernel,int32_t dkernel_x,int32_t dkernel_y,int32_t dkernel_z,uint32_t dkernel_amount,CTensor<type_t> &cTensor_dBias,CTensor<type_t> &cTensor_Image,const CTensor<type_t> &cTensor_Delta,int32_t stride_x,int32_t stride_y,int32_t padding_x,int32_t padding_y)
  {
   OnlyFloat();
   mt_tensor dk=cTensor_dKernel.Device(true),db=cTensor_dBias.Device(true),i=cTensor_Image.DeviceRead(),d=cTensor_Delta.DeviceRead();
   mi355::Check(mt_create_back_delta_weight_and_bias(&dk,dkernel_x,dkernel_y,dkernel_z,dkernel_amount,&db,&i,&d,stride_x,stride_y,padding_x,padding_y));
   cTensor_dKernel.SetDeviceOnChange();
   cTensor_dBias.SetDeviceOnChange();
  }
};

#endif
