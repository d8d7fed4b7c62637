// Drop-in for the reference's cuda/ctensor.cu.h (class at :69-168): a dense [W,Z,Y,X] tensor with a host copy and a
// device copy kept coherent lazily (HostOnChange / DeviceOnChange, :664-704).  Device memory goes through the C ABI of
// libmi355tensor.so (mt_malloc / mt_copy_*), which replaces CCUDADeviceVector (cuda/ccudadevicevector.cu.h).
// Failures are thrown as `const char *`, as the reference does.
#ifndef C_TENSOR_CU_H
#define C_TENSOR_CU_H

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../common/idatastream.h"
#include "../system/system.h"
#include "mi355_tensor.h"
#include "copqueue.cu.h"

namespace mi355
{
 // `floats` zeros on the device, made once per size and kept until the process ends.  CTensorConv::BackwardConvolution
 // hands them to the library in place of a bias tensor that is known to hold zeros: the convolution layer zeroes a fresh
 // copy of its bias on every backward pass (netlayer/cnetlayerconvolution.cu.h:494-497), and the library keeps its
 // re-ordered weights per (kernel, bias) pair -- with one address for all those zeros the pair stays the same from step
 // to step, with a new temporary per step it never does.
 inline float* ZeroBlock(size_t floats)
 {
  static std::map<size_t,float*> blocks;
  std::map<size_t,float*>::iterator found=blocks.find(floats);
  if (found!=blocks.end()) return(found->second);
  void *ptr=NULL;
  Check(mt_malloc(&ptr,floats*sizeof(float)));
  mt_tensor t;
  t.p=static_cast<float*>(ptr);
  t.w=1;t.z=1;t.y=1;t.x=static_cast<uint32_t>(floats);
  Check(mt_fill(&t,0));
  blocks[floats]=t.p;
  return(t.p);
 }

 // Device buffer with value semantics (copying a CCUDADeviceVector copies the device data, cuda/ccudadevicevector.cu.h:159-170)
 // whose copies share one block until one of them is written: the layers hand whole activations on with operator= on
 // every step (cTensor_Delta=error in every SetOutputError, netlayer/cnetlayerconvolution.cu.h:571; the batch-norm layer's
 // running statistics, netlayer/cnetlayerbatchnormalization.cu.h:617-618), and the copy is almost always replaced as a whole
 // before anybody changes one side.  Whoever is about to write calls Own() first: a block of its own, with the present
 // contents only if the write keeps part of them.  The block goes back to the library when its last owner lets go.
 class CDeviceBuffer
 {
   struct SBlock
   {
    void *Ptr;
    size_t Bytes;
    SBlock(void):Ptr(NULL),Bytes(0) {}
    ~SBlock()
    {
     if (Ptr==NULL) return;
     try {Queue().Access(Ptr,Bytes,false,true);} catch(const char*) {}///<deferred calls that name the block run (or are forgotten) before it goes
     mt_free(Ptr);
    }
   };
   std::shared_ptr<SBlock> Block;
   static std::shared_ptr<SBlock> Make(size_t bytes)
   {
    std::shared_ptr<SBlock> block(new SBlock);
    Check(mt_malloc(&block->Ptr,bytes));
    block->Bytes=bytes;
    return(block);
   }
  public:
   CDeviceBuffer(void) {}
   CDeviceBuffer(const CDeviceBuffer &other):Block(other.Block) {}
   CDeviceBuffer& operator=(const CDeviceBuffer &other) {Block=other.Block;return(*this);}
   void clear(void) {Block.reset();}
   // a block of `bytes` bytes that nobody else holds; the contents are undefined
   void resize(size_t bytes)
   {
    if (bytes==size() && (bytes==0 || Block.use_count()==1)) return;
    Block.reset();
    if (bytes!=0) Block=Make(bytes);
   }
   void assign(const void *device_source,size_t bytes)
   {
    resize(bytes);
    if (bytes==0) return;
    Queue().Access(device_source,bytes,true,false);
    Queue().Access(Block->Ptr,bytes,false,true);
    Check(mt_copy_d2d(Block->Ptr,device_source,bytes));
   }
   // before a write: the block becomes this object's alone; `keep` carries the present contents over
   void Own(bool keep)
   {
    if (!Block || Block.use_count()==1) return;
    std::shared_ptr<SBlock> mine=Make(Block->Bytes);
    if (keep==true)
    {
     Queue().Access(Block->Ptr,Block->Bytes,true,false);
     Check(mt_copy_d2d(mine->Ptr,Block->Ptr,Block->Bytes));
    }
    Block.swap(mine);
   }
   bool Shared(void) const {return(Block && Block.use_count()>1);}
   void swap(CDeviceBuffer &other) {Block.swap(other.Block);}
   void* get(void) const {return(Block?Block->Ptr:NULL);}
   size_t size(void) const {return(Block?Block->Bytes:0);}
 };

 // Per-sample weight gradients of a convolution layer that were asked for and not computed.  The reference's layer
 // (netlayer/cnetlayerconvolution.cu.h:501-508) fills a [B,1,Kamt,C*Ky*Kx] tensor with zeros, has
 // CreateDeltaWeightAndBias add every sample's gradient into its slice and then sums the slices with AddSumW: at
 // 512 kernels of 256x4x4 and a batch of 128 that tensor is 1 GiB, written twice and read twice per step, to obtain
 // 8 MiB.  The drop-in classes defer the three steps: Fill(0) of a batch tensor only marks it, CreateDeltaWeightAndBias
 // on two marked tensors computes the sums over the batch directly (mt_convolution_backward_weights_sum) and keeps
 // copies of its two operands, AddSumW of such a tensor adds the sum.  Whoever reads the per-sample gradients in any
 // other way gets them: they are then computed from the kept operands (CTensor::Materialise).
 struct CDeferredGradient
 {
  CDeviceBuffer Image;///<the operands as they were when the gradients were asked for (their blocks, shared)
  CDeviceBuffer Delta;
  mt_tensor ImageTensor;
  mt_tensor DeltaTensor;
  int32_t Kernel_X,Kernel_Y,Kernel_Z,Stride_X,Stride_Y,Padding_X,Padding_Y;
  uint32_t Kernel_Amount;
  uint32_t KernelSize[4];///<sizes of the two per-sample tensors when the gradients were asked for
  uint32_t BiasSize[4];
  CDeviceBuffer KernelSum;///<[1,Z,Y,X] of the kernel tensor: the sum over the batch, once somebody needs it on its own
  CDeviceBuffer BiasSum;
  bool KernelReady;
  bool BiasReady;
  CDeferredGradient(void):KernelReady(false),BiasReady(false) {}
  mt_tensor Sum(bool kernel)
  {
   const uint32_t *size=kernel?KernelSize:BiasSize;
   CDeviceBuffer &buffer=kernel?KernelSum:BiasSum;
   buffer.resize(static_cast<size_t>(size[1])*size[2]*size[3]*sizeof(float));
   mt_tensor t;
   t.p=static_cast<float*>(buffer.get());
   t.w=1;t.z=size[1];t.y=size[2];t.x=size[3];
   return(t);
  }
  // The sums over the batch from the kept operands.  `onto`: the kernel gradients are added straight onto this tensor
  // (the layer's AddSumW(dKernel,dKernel,per-sample tensor)); without it they go to KernelSum.  The bias sums always go
  // to BiasSum (a few hundred values).
  void Compute(const mt_tensor *onto)
  {
   mt_tensor bias=Sum(false),kernel;
   Check(mt_fill(&bias,0));
   if (onto!=NULL) kernel=*onto;
   else
   {
    kernel=Sum(true);
    Check(mt_fill(&kernel,0));
   }
   // the summed kernel gradient is addressed as [1,1,Kamt,C*Ky*Kx] whatever Z x Y split the layer gave its tensor
   kernel.y*=kernel.z;kernel.z=1;
   Check(mt_convolution_backward_weights_sum(&kernel,Kernel_X,Kernel_Y,Kernel_Z,Kernel_Amount,&bias,&ImageTensor,&DeltaTensor,Stride_X,Stride_Y,Padding_X,Padding_Y));
   BiasReady=true;
   if (onto==NULL) KernelReady=true;
  }
 };
 // An up-sampled tensor that was not written yet (CTensorMath::UpSampling by 2 x 2): the source as it was (its block,
 // shared) and the factors.  The generator of the reference's GAN model follows every up-sampling layer by a 3x3
 // convolution (cuda/netmodel/cmodel_gan.cu.h:153-170); CTensorConv::ForwardConvolution on such a tensor computes the
 // convolution of the up-sampled image from the source itself (mt_upsampling_convolution_func: four 2x2 convolutions,
 // 4/9 of the multiplications, the image of four times the size neither written nor read).  Whoever reads the tensor
 // in any other way gets it written first (CTensor::Materialise), e.g. the layer's weight gradient in training.
 struct CDeferredUpSampling
 {
  CDeviceBuffer Source;
  mt_tensor SourceTensor;
  uint32_t Factor_X;
  uint32_t Factor_Y;
 };
 // Per-sample outer products that were not computed (CTensorMath::Mul of a column [B,1,M,1] by a row [B,1,1,N]): the
 // linear layer forms its weight gradient that way and sums it over the batch at once (netlayer/cnetlayerlinear.cu.h:
 // 436-444), B x M x N values written and read back for an M x N result.  AddSumW of such a tensor onto the layer's
 // gradient is one product over the batch instead, columns^T x rows; any other reader gets the products computed.
 struct CDeferredProduct
 {
  CDeviceBuffer Left;
  CDeviceBuffer Right;
  mt_tensor LeftTensor;
  mt_tensor RightTensor;
 };
 // switch for the deferral (on by default): with `false` every call runs when it is made
 inline bool& DeferGradients(void)
 {
  static bool on=true;
  return(on);
 }
}

template<class type_t> class CTensorMath;
template<class type_t> class CTensorConv;
template<class type_t> class CTensorApplyFunc;
template<class type_t> class CTensor;

template<class type_t> CTensor<type_t> operator+(const CTensor<type_t>& cTensor_Left,const CTensor<type_t>& cTensor_Right);
template<class type_t> CTensor<type_t> operator-(const CTensor<type_t>& cTensor_Left,const CTensor<type_t>& cTensor_Right);
template<class type_t> CTensor<type_t> operator*(const CTensor<type_t>& cTensor_Left,const CTensor<type_t>& cTensor_Right);
template<class type_t> CTensor<type_t> operator*(const CTensor<type_t>& cTensor_Left,const type_t& value_right);
template<class type_t> CTensor<type_t> operator*(const type_t& value_left,const CTensor<type_t>& cTensor_Right);

template<class type_t>
class CTensor
{
 template<class new_type_t> friend class CTensorMath;
 template<class new_type_t> friend class CTensorConv;
 template<class new_type_t> friend class CTensorApplyFunc;
 template<class new_type_t> friend class CTensorTest;
 private:
  mutable uint32_t Size_X;
  mutable uint32_t Size_Y;
  mutable uint32_t Size_Z;
  mutable uint32_t Size_W;
  mutable uint32_t BasedSize_X;
  mutable uint32_t BasedSize_Y;
  mutable uint32_t BasedSize_Z;
  mutable uint32_t BasedSize_W;
  mutable std::vector<type_t> Item;
  mutable mi355::CDeviceBuffer DeviceItem;
  mutable bool HostOnChange;
  mutable bool DeviceOnChange;
  // What the device copy holds when it was not written yet (mi355::CDeferredGradient): while Lazy is not LAZY_NONE the
  // device copy is the current one (DeviceOnChange) and every access goes through Materialise() first.
  enum {LAZY_NONE=0,LAZY_ZERO,LAZY_GRADIENT_KERNEL,LAZY_GRADIENT_BIAS,LAZY_UPSAMPLING,LAZY_PRODUCT};
  mutable uint8_t Lazy;
  mutable std::shared_ptr<mi355::CDeferredGradient> Deferred;
  mutable std::shared_ptr<mi355::CDeferredUpSampling> DeferredUpSampling;
  mutable std::shared_ptr<mi355::CDeferredProduct> DeferredProduct;
  // The last write was a fill with zeros (set by the fills, cleared by everything that hands out the tensor for writing
  // and by every change of either copy): see mi355::ZeroBlock.
  mutable bool KnownZero;
 public:
  CTensor(uint32_t size_w=1,uint32_t size_z=1,uint32_t size_y=1,uint32_t size_x=1)
  {
   Lazy=LAZY_NONE;
   KnownZero=false;
   Size_X=size_x;Size_Y=size_y;Size_Z=size_z;Size_W=size_w;
   BasedSize_X=Size_X;BasedSize_Y=Size_Y;BasedSize_Z=Size_Z;BasedSize_W=Size_W;
   Item.resize(Count());
   DeviceItem.resize(Count()*sizeof(type_t));
   HostOnChange=false;
   DeviceOnChange=false;
  }
  CTensor(const CTensor<type_t> &cTensor)
  {
   Lazy=LAZY_NONE;
   KnownZero=false;
   CopyValues(cTensor);
   Size_X=cTensor.Size_X;Size_Y=cTensor.Size_Y;Size_Z=cTensor.Size_Z;Size_W=cTensor.Size_W;
   BasedSize_X=Size_X;BasedSize_Y=Size_Y;BasedSize_Z=Size_Z;BasedSize_W=Size_W;
  }
  ~CTensor() {}
 public:
  uint32_t GetSizeX(void) const {return(Size_X);}
  uint32_t GetSizeY(void) const {return(Size_Y);}
  uint32_t GetSizeZ(void) const {return(Size_Z);}
  uint32_t GetSizeW(void) const {return(Size_W);}
  type_t GetElement(uint32_t w,uint32_t z,uint32_t y,uint32_t x) const
  {
   if (x>=Size_X || y>=Size_Y || z>=Size_Z || w>=Size_W) throw("CTensor::GetElement: index outside the tensor");
   CopyFromDevice();
   return(Item[Index(w,z,y,x)]);
  }
  void SetElement(uint32_t w,uint32_t z,uint32_t y,uint32_t x,type_t value)
  {
   if (x>=Size_X || y>=Size_Y || z>=Size_Z || w>=Size_W) throw("CTensor::SetElement: index outside the tensor");
   CopyFromDevice();
   Item[Index(w,z,y,x)]=value;
   SetHostOnChange();
  }
  type_t* GetColumnPtr(uint32_t w,uint32_t z,uint32_t y)
  {
   if (y>=Size_Y || z>=Size_Z || w>=Size_W) throw("CTensor::GetColumnPtr: row outside the tensor");
   CopyFromDevice();
   SetHostOnChange();
   return(&Item[Index(w,z,y,0)]);
  }
  const type_t* GetColumnPtr(uint32_t w,uint32_t z,uint32_t y) const
  {
   if (y>=Size_Y || z>=Size_Z || w>=Size_W) throw("CTensor::GetColumnPtr: row outside the tensor");
   CopyFromDevice();
   SetHostOnChange();
   return(&Item[Index(w,z,y,0)]);
  }
  void Unitary(void)
  {
   size_t n=0;
   for(uint32_t w=0;w<Size_W;w++)
    for(uint32_t z=0;z<Size_Z;z++)
     for(uint32_t y=0;y<Size_Y;y++)
      for(uint32_t x=0;x<Size_X;x++,n++) Item[n]=(x==y)?1:0;
   SetHostOnChange();
  }
  void Zero(void) {Fill(0);}
  void Fill(type_t value)
  {
   for(size_t n=0;n<Item.size();n++) Item[n]=value;
   SetHostOnChange();
   KnownZero=(value==0);
  }
  void Move(CTensor<type_t> &cTensor)
  {
   if (this==&cTensor) return;
   cTensor.Materialise();
   DropLazy();
   Item=std::move(cTensor.Item);
   DeviceItem.swap(cTensor.DeviceItem);
   Size_X=cTensor.Size_X;Size_Y=cTensor.Size_Y;Size_Z=cTensor.Size_Z;Size_W=cTensor.Size_W;
   BasedSize_X=cTensor.BasedSize_X;BasedSize_Y=cTensor.BasedSize_Y;BasedSize_Z=cTensor.BasedSize_Z;BasedSize_W=cTensor.BasedSize_W;
   HostOnChange=cTensor.HostOnChange;
   DeviceOnChange=cTensor.DeviceOnChange;
   KnownZero=cTensor.KnownZero;
   cTensor.Size_X=0;cTensor.Size_Y=0;cTensor.Size_Z=0;cTensor.Size_W=0;
   cTensor.BasedSize_X=0;cTensor.BasedSize_Y=0;cTensor.BasedSize_Z=0;cTensor.BasedSize_W=0;
   cTensor.Item.clear();
   cTensor.HostOnChange=false;
   cTensor.DeviceOnChange=false;
  }
  void CopyItem(CTensor<type_t> &cTensor)
  {
   if (Count()!=cTensor.Count()) throw("CTensor::CopyItem: element counts differ");
   cTensor.CopyFromDevice();
   Item=cTensor.Item;
   SetHostOnChange();
  }
  void CopyItemToHost(type_t *item_array,uint32_t size)
  {
   if (Item.size()<size) throw("CTensor::CopyItemToHost: array larger than the tensor");
   CopyFromDevice();
   memcpy(&Item[0],item_array,size*sizeof(type_t));
   SetHostOnChange();
  }
  void CopyItemToDevice(type_t *item_array,uint32_t size)
  {
   if (Item.size()<size) throw("CTensor::CopyItemToDevice: array larger than the tensor");
   Materialise();
   CopyToDevice();
   DeviceItem.Own(true);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),true,true);
   mi355::Check(mt_copy_h2d(DeviceItem.get(),item_array,size*sizeof(type_t)));
   SetDeviceOnChange();
  }
  void CopyItemLayerWToHost(uint32_t w,type_t *item_array,uint32_t size)
  {
   size_t offset=static_cast<size_t>(w)*Size_X*Size_Y*Size_Z;
   if (Item.size()<size+offset) throw("CTensor::CopyItemLayerWToHost: array larger than the tensor");
   CopyFromDevice();
   memcpy(&Item[offset],item_array,size*sizeof(type_t));
   SetHostOnChange();
  }
  void CopyItemLayerWToDevice(uint32_t w,type_t *item_array,uint32_t size)
  {
   size_t offset=static_cast<size_t>(w)*Size_X*Size_Y*Size_Z;
   if (Item.size()<size+offset) throw("CTensor::CopyItemLayerWToDevice: array larger than the tensor");
   Materialise();
   CopyToDevice();
   DeviceItem.Own(true);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),true,true);
   mi355::Check(mt_copy_h2d(static_cast<type_t*>(DeviceItem.get())+offset,item_array,size*sizeof(type_t)));
   SetDeviceOnChange();
  }
  CTensor<type_t>& operator=(const CTensor<type_t> &cTensor)
  {
   if (this!=&cTensor)
   {
    CopyValues(cTensor);
    Size_X=cTensor.Size_X;Size_Y=cTensor.Size_Y;Size_Z=cTensor.Size_Z;Size_W=cTensor.Size_W;
    BasedSize_X=cTensor.BasedSize_X;BasedSize_Y=cTensor.BasedSize_Y;BasedSize_Z=cTensor.BasedSize_Z;BasedSize_W=cTensor.BasedSize_W;
   }
   return(*this);
  }

  friend CTensor<type_t> operator+<type_t>(const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right);
  friend CTensor<type_t> operator-<type_t>(const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right);
  friend CTensor<type_t> operator*<type_t>(const CTensor<type_t> &cTensor_Left,const CTensor<type_t> &cTensor_Right);
  friend CTensor<type_t> operator*<type_t>(const CTensor<type_t> &cTensor_Left,const type_t &value_right);
  friend CTensor<type_t> operator*<type_t>(const type_t &value_left,const CTensor<type_t> &cTensor_Right);

  // on-disk form: W,Z,Y,X as uint32 then every element as a double (reference :525-571)
  bool Save(IDataStream *iDataStream_Ptr)
  {
   CopyFromDevice();
   iDataStream_Ptr->SaveUInt32(Size_W);
   iDataStream_Ptr->SaveUInt32(Size_Z);
   iDataStream_Ptr->SaveUInt32(Size_Y);
   iDataStream_Ptr->SaveUInt32(Size_X);
   for(size_t n=0;n<Count();n++) iDataStream_Ptr->SaveDouble(static_cast<double>(Item[n]));
   return(true);
  }
  bool Load(IDataStream *iDataStream_Ptr,bool check_size=false)
  {
   if (check_size==true)
   {
    if (Size_W!=iDataStream_Ptr->LoadUInt32()) throw("CTensor::Load: stored W differs");
    if (Size_Z!=iDataStream_Ptr->LoadUInt32()) throw("CTensor::Load: stored Z differs");
    if (Size_Y!=iDataStream_Ptr->LoadUInt32()) throw("CTensor::Load: stored Y differs");
    if (Size_X!=iDataStream_Ptr->LoadUInt32()) throw("CTensor::Load: stored X differs");
   }
   else
   {
    Size_W=iDataStream_Ptr->LoadUInt32();
    Size_Z=iDataStream_Ptr->LoadUInt32();
    Size_Y=iDataStream_Ptr->LoadUInt32();
    Size_X=iDataStream_Ptr->LoadUInt32();
   }
   DropLazy();
   Item.assign(Count(),type_t());
   DeviceItem.resize(Item.size()*sizeof(type_t));
   for(size_t n=0;n<Count();n++) Item[n]=static_cast<type_t>(iDataStream_Ptr->LoadDouble());
   SetHostOnChange();
   return(true);
  }

  void ExchangeSizeXY(void) const {uint32_t tmp=Size_X;Size_X=Size_Y;Size_Y=tmp;}
  void ReinterpretSize(uint32_t size_w,uint32_t size_z,uint32_t size_y,uint32_t size_x) const
  {
   if (Count()!=static_cast<size_t>(size_x)*size_y*size_z*size_w)
   {
    char str[256];
    snprintf(str,sizeof(str),"%ux%ux%ux%u->%ux%ux%ux%u",Size_W,Size_Z,Size_Y,Size_X,size_w,size_z,size_y,size_x);
    SYSTEM::PutMessageToConsole(str);
    throw("CTensor::ReinterpretSize: the element count must not change");
   }
   Size_X=size_x;Size_Y=size_y;Size_Z=size_z;Size_W=size_w;
  }
  void RestoreSize(void) const {Size_X=BasedSize_X;Size_Y=BasedSize_Y;Size_Z=BasedSize_Z;Size_W=BasedSize_W;}

  void Normalize(void)
  {
   CopyFromDevice();
   for(uint32_t w=0;w<Size_W;w++)
    for(uint32_t z=0;z<Size_Z;z++)
    {
     type_t norma=GetNorma(w,z);
     if (norma<0.0000000001) continue;
     for(uint32_t y=0;y<Size_Y;y++)
      for(uint32_t x=0;x<Size_X;x++) Item[Index(w,z,y,x)]/=norma;
    }
   SetHostOnChange();
  }
  type_t GetNorma(uint32_t w,uint32_t z) const
  {
   CopyFromDevice();
   type_t norma=0;
   for(uint32_t y=0;y<Size_Y;y++)
    for(uint32_t x=0;x<Size_X;x++)
    {
     type_t v=Item[Index(w,z,y,x)];
     norma+=v*v;
    }
   return(sqrt(norma));
  }

  void CopyToDevice(bool force=false) const
  {
   if (HostOnChange==false && force==false) return;
   DropLazy();
   DeviceItem.Own(false);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),false,true);
   if (!Item.empty()) mi355::Check(mt_copy_h2d(DeviceItem.get(),&Item[0],Item.size()*sizeof(type_t)));
   HostOnChange=false;
   DeviceOnChange=false;
  }
  void CopyFromDevice(bool force=false) const
  {
   Materialise();
   if (DeviceOnChange==false && force==false) return;
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),true,false);
   if (!Item.empty()) mi355::Check(mt_copy_d2h(&Item[0],DeviceItem.get(),Item.size()*sizeof(type_t)));
   HostOnChange=false;
   DeviceOnChange=false;
  }
  void SetDeviceOnChange(void) const {DeviceOnChange=true;HostOnChange=false;KnownZero=false;}
  void SetHostOnChange(void) const {DropLazy();DeviceOnChange=false;HostOnChange=true;KnownZero=false;}
  void SetKnownZero(void) const {KnownZero=true;}///<CTensorMath::Fill, after its write was noted
  bool HoldsZeros(void) const {return(Lazy==LAZY_ZERO || (Lazy==LAZY_NONE && KnownZero==true));}
  // Writes what the device copy was only said to hold: zeros, or the per-sample gradients computed from the operands
  // that were kept (CreateDeltaWeightAndBias of the reference adds into the zeroed tensor, netlayer/
  // cnetlayerconvolution.cu.h:503-506; a sample's bias gradient is the sum of its delta over the pixels).
  void Materialise(void) const
  {
   if (Lazy==LAZY_NONE) return;
   DeviceItem.Own(false);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),false,true);
   const uint8_t kind=Lazy;
   std::shared_ptr<mi355::CDeferredGradient> record;
   record.swap(Deferred);
   std::shared_ptr<mi355::CDeferredUpSampling> up;
   up.swap(DeferredUpSampling);
   std::shared_ptr<mi355::CDeferredProduct> product;
   product.swap(DeferredProduct);
   Lazy=LAZY_NONE;
   KnownZero=(kind==LAZY_ZERO);
   mt_tensor own;
   own.p=static_cast<float*>(DeviceItem.get());
   own.w=Size_W;own.z=Size_Z;own.y=Size_Y;own.x=Size_X;
   if (kind==LAZY_PRODUCT)
   {
    own.w=product->LeftTensor.w;own.z=product->LeftTensor.z;own.y=product->LeftTensor.y;own.x=product->RightTensor.x;
    mi355::Check(mt_mul(&own,&product->LeftTensor,&product->RightTensor));
    return;
   }
   if (kind==LAZY_UPSAMPLING)
   {
    // (the sizes of the source as it was: the tensor may have been reinterpreted since)
    own.w=up->SourceTensor.w;own.z=up->SourceTensor.z;own.y=up->SourceTensor.y*up->Factor_Y;own.x=up->SourceTensor.x*up->Factor_X;
    mi355::Check(mt_upsampling(&own,&up->SourceTensor,up->Factor_X,up->Factor_Y));
    return;
   }
   if (kind==LAZY_ZERO)
   {
    mi355::Check(mt_fill(&own,0));
    return;
   }
   const uint32_t *size=(kind==LAZY_GRADIENT_KERNEL)?record->KernelSize:record->BiasSize;
   own.w=size[0];own.z=size[1];own.y=size[2];own.x=size[3];
   if (kind==LAZY_GRADIENT_BIAS)
   {
    mi355::Check(mt_summ_xy(&own,&record->DeltaTensor));
    return;
   }
   mi355::CDeviceBuffer bias;
   bias.resize(static_cast<size_t>(record->BiasSize[0])*record->BiasSize[1]*sizeof(float));
   mt_tensor db;
   db.p=static_cast<float*>(bias.get());
   db.w=record->BiasSize[0];db.z=record->BiasSize[1];db.y=1;db.x=1;
   mi355::Check(mt_fill(&own,0));
   mi355::Check(mt_fill(&db,0));
   mi355::Check(mt_create_delta_weight_and_bias(&own,record->Kernel_X,record->Kernel_Y,record->Kernel_Z,record->Kernel_Amount,&db,&record->ImageTensor,&record->DeltaTensor,
                                                record->Stride_X,record->Stride_Y,record->Padding_X,record->Padding_Y));
  }

  void Print(const std::string &name,bool print_value=true) const
  {
   char str[255];
   CopyFromDevice();
   snprintf(str,sizeof(str),"***** %s *****",name.c_str());
   SYSTEM::PutMessageToConsole(str);
   snprintf(str,sizeof(str),"W:%u Z:%u Y:%u X:%u",Size_W,Size_Z,Size_Y,Size_X);
   SYSTEM::PutMessageToConsole(str);
   if (print_value==false) return;
   for(uint32_t w=0;w<Size_W;w++)
    for(uint32_t z=0;z<Size_Z;z++)
     for(uint32_t y=0;y<Size_Y;y++)
     {
      std::string line;
      for(uint32_t x=0;x<Size_X;x++)
      {
       snprintf(str,sizeof(str),"%f ",static_cast<double>(Item[Index(w,z,y,x)]));
       line+=str;
      }
      SYSTEM::PutMessageToConsole(line);
     }
  }
  void PrintToFile(const std::string &file_name,const std::string &name,bool print_value=true) const
  {
   CopyFromDevice();
   FILE *file=fopen(file_name.c_str(),"wb");
   if (file==NULL) return;
   fprintf(file,"***** %s *****\r\nW:%u Z:%u Y:%u X:%u\r\n",name.c_str(),Size_W,Size_Z,Size_Y,Size_X);
   if (print_value==true)
   {
    for(uint32_t w=0;w<Size_W;w++)
     for(uint32_t z=0;z<Size_Z;z++)
      for(uint32_t y=0;y<Size_Y;y++)
      {
       for(uint32_t x=0;x<Size_X;x++) fprintf(file,"%f ",static_cast<double>(Item[Index(w,z,y,x)]));
       fprintf(file,"\r\n");
      }
   }
   fclose(file);
  }
  // absolute tolerance 1e-5, as the reference (:787)
  bool Compare(const CTensor<type_t> &cTensor_Control,const std::string &name="",bool print_value=true) const
  {
   CopyFromDevice();
   cTensor_Control.CopyFromDevice();
   if (print_value==true && !name.empty()) SYSTEM::PutMessageToConsole(name);
   bool ret=true;
   for(uint32_t w=0;w<Size_W;w++)
    for(uint32_t z=0;z<Size_Z;z++)
     for(uint32_t y=0;y<Size_Y;y++)
      for(uint32_t x=0;x<Size_X;x++)
      {
       double e1=static_cast<double>(GetElement(w,z,y,x));
       double e2=static_cast<double>(cTensor_Control.GetElement(w,z,y,x));
       if (fabs(e1-e2)>0.00001) ret=false;
      }
   return(ret);
  }
 private:
  // Values and coherence state of another tensor.  Only the side that is current is copied: the layers hand their
  // errors on with operator= on every step (netlayer/cnetlayerconvolution.cu.h:571), and a host copy that the device
  // copy has overtaken would cost a memcpy of the whole activation for values nobody may read.
  void CopyValues(const CTensor<type_t> &cTensor)
  {
   cTensor.Materialise();
   DropLazy();
   if (cTensor.DeviceOnChange==true)
   {
    Item.resize(cTensor.Item.size());
    DeviceItem=cTensor.DeviceItem;
   }
   else if (cTensor.HostOnChange==true)
   {
    Item=cTensor.Item;
    DeviceItem.resize(cTensor.DeviceItem.size());
   }
   else
   {
    Item=cTensor.Item;
    DeviceItem=cTensor.DeviceItem;
   }
   HostOnChange=cTensor.HostOnChange;
   DeviceOnChange=cTensor.DeviceOnChange;
   KnownZero=cTensor.KnownZero;
  }
  void DropLazy(void) const {Lazy=LAZY_NONE;Deferred.reset();DeferredUpSampling.reset();DeferredProduct.reset();}
  // the device copy is said to hold the per-sample products left x right; nothing is launched (CTensorMath::Mul)
  void SetLazyProduct(const mi355::CDeviceBuffer &left,const mt_tensor &left_tensor,const mi355::CDeviceBuffer &right,const mt_tensor &right_tensor) const
  {
   DeviceItem.Own(false);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),false,true);
   DropLazy();
   std::shared_ptr<mi355::CDeferredProduct> record(new mi355::CDeferredProduct);
   record->Left=left;record->LeftTensor=left_tensor;
   record->Right=right;record->RightTensor=right_tensor;
   DeferredProduct=record;
   Lazy=LAZY_PRODUCT;
   DeviceOnChange=true;
   HostOnChange=false;
   KnownZero=false;
  }
  // the device copy is said to hold `source` up-sampled by the factors; nothing is launched (CTensorMath::UpSampling)
  void SetLazyUpSampling(const mi355::CDeviceBuffer &source,const mt_tensor &source_tensor,uint32_t factor_x,uint32_t factor_y) const
  {
   DeviceItem.Own(false);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),false,true);
   DropLazy();
   std::shared_ptr<mi355::CDeferredUpSampling> record(new mi355::CDeferredUpSampling);
   record->Source=source;
   record->SourceTensor=source_tensor;
   record->Factor_X=factor_x;record->Factor_Y=factor_y;
   DeferredUpSampling=record;
   Lazy=LAZY_UPSAMPLING;
   DeviceOnChange=true;
   HostOnChange=false;
   KnownZero=false;
  }
  // the device copy is said to hold zeros; nothing is launched (CTensorMath::Fill)
  void SetLazyZero(void) const
  {
   DeviceItem.Own(false);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),false,true);///<as far as deferred calls are concerned the tensor is overwritten now
   DropLazy();
   Lazy=LAZY_ZERO;
   DeviceOnChange=true;
   HostOnChange=false;
  }
  size_t Count(void) const {return(static_cast<size_t>(Size_X)*Size_Y*Size_Z*Size_W);}
  size_t Index(uint32_t w,uint32_t z,uint32_t y,uint32_t x) const {return(x+static_cast<size_t>(Size_X)*(y+static_cast<size_t>(Size_Y)*(z+static_cast<size_t>(Size_Z)*w)));}
  // Descriptors of the device copy for the C ABI.  Read: the tensor is an input (brought up to date first).  Device(true):
  // the call reads and writes it (an accumulator, an in-place operation); Device(false): the call overwrites all of it.
  // A tensor that is about to be written stops sharing its block with its copies (CDeviceBuffer::Own).  Deferred calls
  // (mi355::COpQueue) that involve the tensor run first; the *Queued forms are for calls that are deferred themselves,
  // whose order the queue keeps.
  mt_tensor Descriptor(void) const
  {
   mt_tensor t;
   t.p=static_cast<float*>(DeviceItem.get());
   t.w=Size_W;t.z=Size_Z;t.y=Size_Y;t.x=Size_X;
   return(t);
  }
  mt_tensor DeviceQueuedRead(void) const
  {
   Materialise();
   CopyToDevice();
   return(Descriptor());
  }
  mt_tensor DeviceQueued(bool upload) const
  {
   Materialise();
   if (upload==true) CopyToDevice();
   DeviceItem.Own(upload);
   KnownZero=false;
   return(Descriptor());
  }
  mt_tensor DeviceRead(void) const
  {
   Materialise();
   CopyToDevice();
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),true,false);
   return(Descriptor());
  }
  mt_tensor Device(bool upload) const
  {
   Materialise();
   if (upload==true) CopyToDevice();
   DeviceItem.Own(upload);
   mi355::Queue().Access(DeviceItem.get(),DeviceItem.size(),upload,true);
   KnownZero=false;
   return(Descriptor());
  }
};

#endif
