// Drop-in for the reference's cuda/ctensormath.cu.h (class at :52-138): every static function keeps the reference's
// name, argument order and defaults and forwards to one C-ABI call.  Inputs are brought up to date on the device
// first and the output is marked device-side, as the reference does (:845-870).  The elementwise calls that the layers
// string into long sequences (Fill, Add, Sub, AddSumW, Pow2, SQRT, Inv, TensorItemProduction, Mul by a value, Adam) go
// through mi355::COpQueue, which runs a whole known sequence as its one kernel and everything else as written.
#ifndef C_TENSOR_MATH_CU_H
#define C_TENSOR_MATH_CU_H

#include <stdlib.h>
#include <type_traits>

#include "ctensor.cu.h"

template<class type_t>
class CTensorMath
{
 public:
  struct SPos
  {
   uint32_t X;
   uint32_t Y;
  };
 private:
  static void OnlyFloat(void) {static_assert(std::is_same<type_t,float>::value,"the MI355X tensor path computes in fp32 only");}
  static mt_pos_tensor Position(const CTensor<SPos> &cTensor,bool upload)
  {
   mt_tensor t=(upload==true)?cTensor.DeviceRead():cTensor.Device(false);
   mt_pos_tensor p;
   p.p=reinterpret_cast<mt_spos*>(t.p);
   p.w=t.w;p.z=t.z;p.y=t.y;p.x=t.x;
   return(p);
  }
 public:
  static void Fill(CTensor<type_t> &cTensor_Output,type_t value=0)
  {
   OnlyFloat();
   cTensor_Output.DropLazy();   // whatever the tensor was said to hold is overwritten
   if (value==0 && cTensor_Output.GetSizeW()>1 && mi355::DeferGradients()==true)
   {
    // zeros for a tensor with a batch axis: written when somebody asks for them (mi355::CDeferredGradient)
    cTensor_Output.SetLazyZero();
    return;
   }
   mi355::Queue().Submit(mi355::MakeFill(cTensor_Output.DeviceQueued(false),value));
   cTensor_Output.SetDeviceOnChange();
   if (value==0) cTensor_Output.SetKnownZero();
  }
  static void Inv(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeUnary(mi355::OP_INV,o,i));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Div(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right,type_t left_scale=1,type_t right_scale=1)
  {
   OnlyFloat();
   mt_tensor l=cTensor_Left.DeviceRead(),r=cTensor_Right.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_div(&o,&l,&r,left_scale,right_scale));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Add(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right,type_t left_scale=1,type_t right_scale=1)
  {
   OnlyFloat();
   mt_tensor l=cTensor_Left.DeviceQueuedRead(),r=cTensor_Right.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeBinary(mi355::OP_ADD,o,l,r,left_scale,right_scale));
   cTensor_Output.SetDeviceOnChange();
  }
  // The batch-norm layer of the reference calls Add(out,left,right,EMA_K,1,0-EMA_K) (netlayer/cnetlayerbatchnormalization.cu.h:655-658,
  // a typo for 1.0-EMA_K that matches no overload of the reference): this overload gives it the intended right scale 1-EMA_K.
  static void Add(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right,type_t left_scale,int right_scale_a,type_t right_scale_b)
  {
   Add(cTensor_Output,cTensor_Left,cTensor_Right,left_scale,static_cast<type_t>(right_scale_a+right_scale_b));
  }
  static void AddSumW(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right,type_t left_scale=1,type_t right_scale=1)
  {
   OnlyFloat();
   if (&cTensor_Right!=&cTensor_Output && &cTensor_Right!=&cTensor_Left &&
       (cTensor_Right.Lazy==CTensor<type_t>::LAZY_GRADIENT_KERNEL || cTensor_Right.Lazy==CTensor<type_t>::LAZY_GRADIENT_BIAS))
   {
    // per-sample gradients that were not computed: their sum over the batch is, from the operands the record keeps
    const std::shared_ptr<mi355::CDeferredGradient> record=cTensor_Right.Deferred;
    const bool kernel=(cTensor_Right.Lazy==CTensor<type_t>::LAZY_GRADIENT_KERNEL);
    if (kernel==true && record->KernelReady==false && &cTensor_Left==&cTensor_Output && left_scale==1 && right_scale==1 && cTensor_Output.GetSizeW()==1 &&
        cTensor_Output.GetSizeZ()==cTensor_Right.GetSizeZ() && cTensor_Output.GetSizeY()==cTensor_Right.GetSizeY() && cTensor_Output.GetSizeX()==cTensor_Right.GetSizeX())
    {
     // the layer's own call, AddSumW(dKernel,dKernel,per-sample tensor): the sums are added straight onto dKernel
     mt_tensor o=cTensor_Output.Device(true);
     record->Compute(&o);
     cTensor_Output.SetDeviceOnChange();
     return;
    }
    if ((kernel==true && record->KernelReady==false) || (kernel==false && record->BiasReady==false)) record->Compute(NULL);
    mt_tensor r=record->Sum(kernel);
    mt_tensor l=cTensor_Left.DeviceRead(),o=cTensor_Output.Device(false);
    mi355::Check(mt_add_sum_w(&o,&l,&r,left_scale,right_scale));
    cTensor_Output.SetDeviceOnChange();
    return;
   }
   if (&cTensor_Right!=&cTensor_Output && cTensor_Right.Lazy==CTensor<type_t>::LAZY_PRODUCT && &cTensor_Left==&cTensor_Output && left_scale==1 && right_scale==1 &&
       cTensor_Output.GetSizeW()==1 && cTensor_Output.GetSizeZ()==1)
   {
    // the linear layer's own call, AddSumW(dW,dW,per-sample products): dW += columns^T x rows, one product over the batch
    const std::shared_ptr<mi355::CDeferredProduct> record=cTensor_Right.DeferredProduct;
    mt_tensor columns=record->LeftTensor,rows=record->RightTensor;
    const uint32_t batch=columns.w,m=columns.y,n=rows.x;
    if (cTensor_Output.GetSizeY()==m && cTensor_Output.GetSizeX()==n)
    {
     columns.w=1;columns.y=batch;columns.x=m;   // [B,1,M,1] read as the matrix [B][M]
     rows.w=1;rows.y=batch;rows.x=n;            // [B,1,1,N] read as the matrix [B][N]
     mi355::CDeviceBuffer sum;
     sum.resize(static_cast<size_t>(m)*n*sizeof(float));
     mt_tensor s;
     s.p=static_cast<float*>(sum.get());
     s.w=1;s.z=1;s.y=m;s.x=n;
     mi355::Check(mt_transponse_mul(&s,&columns,&rows));
     mt_tensor o=cTensor_Output.Device(true);
     mi355::Check(mt_add(&o,&o,&s,1,1));
     cTensor_Output.SetDeviceOnChange();
     return;
    }
   }
   mt_tensor l=cTensor_Left.DeviceQueuedRead(),r=cTensor_Right.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeBinary(mi355::OP_ADD_SUM_W,o,l,r,left_scale,right_scale));
   cTensor_Output.SetDeviceOnChange();
  }
  static void AddValue(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,type_t tensor_scale,type_t value)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_add_value(&o,&i,tensor_scale,value));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Sub(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right,type_t left_scale=1,type_t right_scale=1)
  {
   OnlyFloat();
   mt_tensor l=cTensor_Left.DeviceQueuedRead(),r=cTensor_Right.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeBinary(mi355::OP_SUB,o,l,r,left_scale,right_scale));
   cTensor_Output.SetDeviceOnChange();
  }
  static void SubValue(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,type_t tensor_scale,type_t value)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_sub_value(&o,&i,tensor_scale,value));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Set(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,type_t scale=1,type_t add_value=0)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_set(&o,&i,scale,add_value));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Pow2(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,type_t scale=1)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeUnary(mi355::OP_POW2,o,i,scale));
   cTensor_Output.SetDeviceOnChange();
  }
  static void SQRT(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,type_t scale,type_t add_sqrt_value)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeUnary(mi355::OP_SQRT,o,i,scale,add_sqrt_value));
   cTensor_Output.SetDeviceOnChange();
  }
  static void AddBias(CTensor<type_t> &cTensor_Working,const CTensor<type_t> &cTensor_Bias)
  {
   OnlyFloat();
   mt_tensor b=cTensor_Bias.DeviceRead(),o=cTensor_Working.Device(true);
   mi355::Check(mt_add_bias(&o,&b));
   cTensor_Working.SetDeviceOnChange();
  }
  static void SummXY(CTensor<type_t> &cTensor_Output,CTensor<type_t> &cTensor_Input)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(true);
   mi355::Check(mt_summ_xy(&o,&i));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Mul(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right,bool tensor_core=false)
  {
   OnlyFloat();
   (void)tensor_core;  // the reference's fp16 tensor-core switch; this path is always fp32 on the matrix cores
   if (mi355::DeferGradients()==true && &cTensor_Output!=&cTensor_Left && &cTensor_Output!=&cTensor_Right && cTensor_Left.GetSizeX()==1 && cTensor_Right.GetSizeY()==1 &&
       cTensor_Left.GetSizeW()>=2 && cTensor_Right.GetSizeW()==cTensor_Left.GetSizeW() && cTensor_Output.GetSizeW()==cTensor_Left.GetSizeW() &&
       cTensor_Left.GetSizeZ()==1 && cTensor_Right.GetSizeZ()==1 && cTensor_Output.GetSizeZ()==1 &&
       cTensor_Output.GetSizeY()==cTensor_Left.GetSizeY() && cTensor_Output.GetSizeX()==cTensor_Right.GetSizeX() && cTensor_Output.Count()>=(static_cast<size_t>(1)<<16))
   {
    // per-sample outer products: computed when somebody reads them; their sum over the batch never needs them (mi355::CDeferredProduct)
    mt_tensor l=cTensor_Left.DeviceRead(),r=cTensor_Right.DeviceRead();
    cTensor_Output.SetLazyProduct(cTensor_Left.DeviceItem,l,cTensor_Right.DeviceItem,r);
    return;
   }
   mt_tensor l=cTensor_Left.DeviceRead(),r=cTensor_Right.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_mul(&o,&l,&r));
   cTensor_Output.SetDeviceOnChange();
  }
  static void TransponseMul(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right,bool tensor_core=false)
  {
   OnlyFloat();
   (void)tensor_core;
   mt_tensor l=cTensor_Left.DeviceRead(),r=cTensor_Right.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_transponse_mul(&o,&l,&r));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Mul(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Left,const type_t &value_right)
  {
   OnlyFloat();
   mt_tensor l=cTensor_Left.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeUnary(mi355::OP_MUL_VALUE,o,l,value_right));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Mul(CTensor<type_t> &cTensor_Output,const type_t &value_left,const CTensor<type_t> &cTensor_Right)
  {
   Mul(cTensor_Output,cTensor_Right,value_left);
  }
  static void Transponse(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_transponse(&o,&i));
   cTensor_Output.SetDeviceOnChange();
  }
  static void TensorItemProduction(CTensor<type_t> &cTensor_Output,CTensor<type_t> &cTensor_Left,CTensor<type_t> &cTensor_Right)
  {
   OnlyFloat();
   mt_tensor l=cTensor_Left.DeviceQueuedRead(),r=cTensor_Right.DeviceQueuedRead(),o=cTensor_Output.DeviceQueued(false);
   mi355::Queue().Submit(mi355::MakeBinary(mi355::OP_ITEM_PRODUCTION,o,l,r));
   cTensor_Output.SetDeviceOnChange();
  }
  static CTensor<type_t> Transpose(const CTensor<type_t> &cTensor_Input)
  {
   CTensor<type_t> cTensor(cTensor_Input.Size_W,cTensor_Input.Size_Z,cTensor_Input.Size_X,cTensor_Input.Size_Y);
   Transponse(cTensor,cTensor_Input);
   return(cTensor);
  }
  static void UpSampling(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,uint32_t upsampling_x,uint32_t upsampling_y)
  {
   OnlyFloat();
   if (mi355::DeferGradients()==true && upsampling_x==2 && upsampling_y==2 && &cTensor_Output!=&cTensor_Input &&
       cTensor_Output.GetSizeW()==cTensor_Input.GetSizeW() && cTensor_Output.GetSizeZ()==cTensor_Input.GetSizeZ() &&
       cTensor_Output.GetSizeY()==2*cTensor_Input.GetSizeY() && cTensor_Output.GetSizeX()==2*cTensor_Input.GetSizeX())
   {
    // written when somebody asks for it; a 3x3 convolution that follows never does (mi355::CDeferredUpSampling)
    mt_tensor source=cTensor_Input.DeviceRead();
    cTensor_Output.SetLazyUpSampling(cTensor_Input.DeviceItem,source,upsampling_x,upsampling_y);
    return;
   }
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_upsampling(&o,&i,upsampling_x,upsampling_y));
   cTensor_Output.SetDeviceOnChange();
  }
  static void DownSampling(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,uint32_t downsampling_x,uint32_t downsampling_y)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_downsampling(&o,&i,downsampling_x,downsampling_y));
   cTensor_Output.SetDeviceOnChange();
  }
  static void MaxPooling(CTensor<type_t> &cTensor_Output,const CTensor<SPos> &cTensor_Position,const CTensor<type_t> &cTensor_Input,uint32_t pooling_x,uint32_t pooling_y)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mt_pos_tensor p=Position(cTensor_Position,false);
   mi355::Check(mt_max_pooling(&o,&p,&i,pooling_x,pooling_y));
   cTensor_Output.SetDeviceOnChange();
   cTensor_Position.SetDeviceOnChange();
  }
  static void MaxPoolingBackward(CTensor<type_t> &cTensor_Output,const CTensor<SPos> &cTensor_Position,const CTensor<type_t> &cTensor_Input,uint32_t pooling_x,uint32_t pooling_y)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false);
   mt_pos_tensor p=Position(cTensor_Position,true);
   mi355::Check(mt_max_pooling_backward(&o,&p,&i,pooling_x,pooling_y));
   cTensor_Output.SetDeviceOnChange();
  }
  static void Clip(CTensor<type_t> &cTensor,type_t min_value,type_t max_value)
  {
   OnlyFloat();
   mt_tensor o=cTensor.Device(true);
   mi355::Check(mt_clip(&o,min_value,max_value));
   cTensor.SetDeviceOnChange();
  }
  static void Signum(CTensor<type_t> &cTensor)
  {
   OnlyFloat();
   mt_tensor o=cTensor.Device(true);
   mi355::Check(mt_signum(&o));
   cTensor.SetDeviceOnChange();
  }
  // the functions below exist in the GPU class only (cuda/ctensormath.cu.h:92-93, 128-134)
  static void ConcatecationZ(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_InputA,const CTensor<type_t> &cTensor_InputB)
  {
   OnlyFloat();
   mt_tensor a=cTensor_InputA.DeviceRead(),b=cTensor_InputB.DeviceRead(),o=cTensor_Output.Device(false);
   mi355::Check(mt_concatecation_z(&o,&a,&b));
   cTensor_Output.SetDeviceOnChange();
  }
  static void SplitZ(CTensor<type_t> &cTensor_OutputA,CTensor<type_t> &cTensor_OutputB,const CTensor<type_t> &cTensor_Input)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),a=cTensor_OutputA.Device(false),b=cTensor_OutputB.Device(false);
   mi355::Check(mt_split_z(&a,&b,&i));
   cTensor_OutputA.SetDeviceOnChange();
   cTensor_OutputB.SetDeviceOnChange();
  }
  static void SetTimeStep(CTensor<type_t> &cTensor_Output,const CTensor<type_t> &cTensor_Input,const CTensor<uint32_t> &cTensor_TimeStep)
  {
   OnlyFloat();
   mt_tensor i=cTensor_Input.DeviceRead(),o=cTensor_Output.Device(false),t=cTensor_TimeStep.DeviceRead();
   mt_u32_tensor ts;
   ts.p=reinterpret_cast<uint32_t*>(t.p);
   ts.w=t.w;ts.z=t.z;ts.y=t.y;ts.x=t.x;
   mi355::Check(mt_set_time_step(&o,&i,&ts));
   cTensor_Output.SetDeviceOnChange();
  }
  // the reference seeds its generator with rand() at each call (cuda/ctensormath.cu.h:3117, 3169, 3257); so does this
  static void CreateDropOutMatrix(CTensor<type_t> &cTensor_Output,type_t drop_out)
  {
   OnlyFloat();
   mt_tensor o=cTensor_Output.Device(false);
   mi355::Check(mt_create_drop_out_matrix(&o,drop_out,static_cast<uint64_t>(rand())));
   cTensor_Output.SetDeviceOnChange();
  }
  static void SetNormalNoise(CTensor<type_t> &cTensor_Output)
  {
   OnlyFloat();
   mt_tensor o=cTensor_Output.Device(false);
   mi355::Check(mt_set_normal_noise(&o,static_cast<uint64_t>(rand())));
   cTensor_Output.SetDeviceOnChange();
  }
  static void GetNoiseImageAndNoise(CTensor<type_t> &cTensor_NoisyImage,CTensor<type_t> &cTensor_Noise,const CTensor<type_t> &cTensor_Image,const CTensor<type_t> &cTensor_SqrtAlphaBar,const CTensor<type_t> &cTensor_SqrtOneMinusAlphaBar)
  {
   OnlyFloat();
   mt_tensor im=cTensor_Image.DeviceRead(),sa=cTensor_SqrtAlphaBar.DeviceRead(),sb=cTensor_SqrtOneMinusAlphaBar.DeviceRead();
   mt_tensor ni=cTensor_NoisyImage.Device(false),no=cTensor_Noise.Device(false);
   mi355::Check(mt_get_noise_image_and_noise(&ni,&no,&im,&sa,&sb,static_cast<uint64_t>(rand())));
   cTensor_Noise.SetDeviceOnChange();
   cTensor_NoisyImage.SetDeviceOnChange();
  }
  static void Adam(CTensor<type_t> &cTensor_Weight,CTensor<type_t> &cTensor_dWeight,CTensor<type_t> &cTensor_M,CTensor<type_t> &cTensor_V,uint32_t batch_size,double speed,double beta1,double beta2,double epsilon,double iteration)
  {
   OnlyFloat();
   mt_tensor w=cTensor_Weight.DeviceQueued(true),dw=cTensor_dWeight.DeviceQueuedRead(),m=cTensor_M.DeviceQueued(true),v=cTensor_V.DeviceQueued(true);
   mi355::Queue().Submit(mi355::MakeAdam(w,dw,m,v,batch_size,speed,beta1,beta2,epsilon,iteration));
   cTensor_Weight.SetDeviceOnChange();
   cTensor_M.SetDeviceOnChange();
   cTensor_V.SetDeviceOnChange();
  }
};

template<class type_t>
CTensor<type_t> operator+(const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right)
{
 CTensor<type_t> cTensor(cTensor_Right.Size_W,cTensor_Left.Size_Z,cTensor_Left.Size_Y,cTensor_Left.Size_X);
 CTensorMath<type_t>::Add(cTensor,cTensor_Left,cTensor_Right);
 return(cTensor);
}
template<class type_t>
CTensor<type_t> operator-(const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right)
{
 CTensor<type_t> cTensor(cTensor_Right.Size_W,cTensor_Left.Size_Z,cTensor_Left.Size_Y,cTensor_Left.Size_X);
 CTensorMath<type_t>::Sub(cTensor,cTensor_Left,cTensor_Right);
 return(cTensor);
}
template<class type_t>
CTensor<type_t> operator*(const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right)
{
 CTensor<type_t> cTensor(cTensor_Right.Size_W,cTensor_Left.Size_Z,cTensor_Left.Size_Y,cTensor_Right.Size_X);
 CTensorMath<type_t>::Mul(cTensor,cTensor_Left,cTensor_Right);
 return(cTensor);
}
template<class type_t>
CTensor<type_t> operator*(const CTensor<type_t> &cTensor_Left,const type_t &value_right)
{
 CTensor<type_t> cTensor(cTensor_Left.Size_W,cTensor_Left.Size_Z,cTensor_Left.Size_Y,cTensor_Left.Size_X);
 CTensorMath<type_t>::Mul(cTensor,cTensor_Left,value_right);
 return(cTensor);
}
template<class type_t>
CTensor<type_t> operator*(const type_t &value_left,const CTensor<type_t> &cTensor_Right)
{
 CTensor<type_t> cTensor(cTensor_Right.Size_W,cTensor_Right.Size_Z,cTensor_Right.Size_Y,cTensor_Right.Size_X);
 CTensorMath<type_t>::Mul(cTensor,value_left,cTensor_Right);
 return(cTensor);
}

#endif
