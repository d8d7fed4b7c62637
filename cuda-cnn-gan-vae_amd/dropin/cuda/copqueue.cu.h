// Deferred tensor operations of the drop-in classes.  No counterpart in the reference, whose CTensorMath runs every call
// when it is made.
//
// The reference's layers are written as long sequences of small tensor operations: the batch-norm layer's forward pass
// in training mode is 13 calls (netlayer/cnetlayerbatchnormalization.cu.h:301-371), its backward pass 12 or 15
// (:578-604), with the two calls of a function layer's SetOutputError in front of it when one follows the batch norm
// (netlayer/cnetlayerfunction.cu.h:347-358), and every layer clears its gradients and runs Adam tensor by tensor
// (netlayer/cnetlayerconvolution.cu.h:522-539).  The library has one kernel for each of these sequences
// (mt_batchnorm_forward_train_from, mt_batchnorm_forward_infer_func, mt_batchnorm_backward_keep,
// mt_batchnorm_backward_func_keep, mt_fill_many, mt_adam_many).  So the elementwise calls of CTensorMath are not run at once: they are appended to a queue, and
//   * while the queue is the beginning of one of the known sequences (same operations, same tensors in the same roles,
//     same scalars), it waits;
//   * when it is a whole sequence, the sequence's one kernel runs instead;
//   * consecutive Fill calls (one value) and consecutive Adam calls (one set of hyper-parameters) collect, across
//     layers, into one launch each;
//   * anything else -- an operation that fits no sequence, any other call of the tensor classes that touches a tensor of
//     the queue, any host access to one -- runs the queue call by call, exactly as written, first (calls and accesses
//     that touch none of the queue's tensors pass it: neither side depends on the other).
// A sequence's kernel does not write the sequence's scratch tensors that nobody can have read yet (sqrt(var + eps) and
// gamma * xhat of the forward pass; xhat * sum of the backward pass).  Their defining calls stay "pending": they run the
// moment somebody reads such a tensor or is about to change one of their inputs, and are forgotten when the tensor is
// overwritten without having been read (which is what the layer does on its next pass).  Every tensor therefore holds,
// whenever it is looked at, what the call-by-call path would have left in it, within fp32 rounding of the fused kernels.
// mi355::FuseSequences() = false switches all of this off.
#ifndef C_OP_QUEUE_CU_H
#define C_OP_QUEUE_CU_H

#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <vector>

#include "mi355_tensor.h"

namespace mi355
{
 inline void Check(int rc)
 {
  if (rc!=MT_OK) throw static_cast<const char*>(mt_last_error());
 }
 // switch for the deferral of elementwise sequences (on by default)
 inline bool& FuseSequences(void)
 {
  static bool on=true;
  return(on);
 }

 enum {OP_FILL=0,OP_ADD_SUM_W,OP_ADD,OP_SUB,OP_POW2,OP_SQRT,OP_INV,OP_ITEM_PRODUCTION,OP_MUL_VALUE,OP_ADAM,OP_DIFFERENTIAL,OP_FUNCTION};

 // one call of CTensorMath as it was made: T[0] is the output (Adam: the weights), the inputs follow
 struct SOp
 {
  int Kind;
  mt_tensor T[4];
  uint8_t Count;///<tensors in use
  uint8_t Reads;///<bit i: T[i] is read
  uint8_t Writes;///<bit i: all of T[i] is written
  float A;
  float B;
  int Func;///<OP_FUNCTION: the function applied; OP_DIFFERENTIAL: the function whose derivative is applied (MT_F_*)
  uint32_t BatchSize;
  double Speed,Beta1,Beta2,Epsilon,Iteration;
  uint8_t Own;///<1: writes a batch-norm layer's own output that a fused forward pass left pending (COpQueue::RunForward)
 };

 inline SOp MakeOp(int kind,uint8_t count,uint8_t reads,uint8_t writes,float a=0,float b=0)
 {
  SOp op;
  op.Kind=kind;op.Count=count;op.Reads=reads;op.Writes=writes;op.A=a;op.B=b;op.Func=MT_F_NONE;
  op.BatchSize=0;op.Speed=0;op.Beta1=0;op.Beta2=0;op.Epsilon=0;op.Iteration=0;op.Own=0;
  for(int n=0;n<4;n++) {op.T[n].p=NULL;op.T[n].w=0;op.T[n].z=0;op.T[n].y=0;op.T[n].x=0;}
  return(op);
 }
 inline SOp MakeFill(const mt_tensor &o,float value)
 {
  SOp op=MakeOp(OP_FILL,1,0,1,value);
  op.T[0]=o;
  return(op);
 }
 inline SOp MakeUnary(int kind,const mt_tensor &o,const mt_tensor &i,float a=0,float b=0)
 {
  SOp op=MakeOp(kind,2,2,1,a,b);
  op.T[0]=o;op.T[1]=i;
  return(op);
 }
 inline SOp MakeDifferential(const mt_tensor &o,const mt_tensor &i,int func)///<o = f'(i), CTensorApplyFunc::ApplyDifferential...
 {
  SOp op=MakeOp(OP_DIFFERENTIAL,2,2,1);
  op.T[0]=o;op.T[1]=i;op.Func=func;
  return(op);
 }
 inline SOp MakeFunction(const mt_tensor &o,const mt_tensor &i,int func)///<o = f(i), CTensorApplyFunc::Apply...
 {
  SOp op=MakeOp(OP_FUNCTION,2,2,1);
  op.T[0]=o;op.T[1]=i;op.Func=func;
  return(op);
 }
 inline SOp MakeBinary(int kind,const mt_tensor &o,const mt_tensor &l,const mt_tensor &r,float a=0,float b=0)
 {
  SOp op=MakeOp(kind,3,6,1,a,b);
  op.T[0]=o;op.T[1]=l;op.T[2]=r;
  return(op);
 }
 inline SOp MakeAdam(const mt_tensor &w,const mt_tensor &dw,const mt_tensor &m,const mt_tensor &v,uint32_t batch_size,double speed,double beta1,double beta2,double epsilon,double iteration)
 {
  SOp op=MakeOp(OP_ADAM,4,15,13);
  op.T[0]=w;op.T[1]=dw;op.T[2]=m;op.T[3]=v;
  op.BatchSize=batch_size;op.Speed=speed;op.Beta1=beta1;op.Beta2=beta2;op.Epsilon=epsilon;op.Iteration=iteration;
  return(op);
 }

 inline size_t Bytes(const mt_tensor &t) {return(static_cast<size_t>(t.w)*t.z*t.y*t.x*sizeof(float));}
 inline bool Same(const mt_tensor &a,const mt_tensor &b) {return(a.p==b.p && a.w==b.w && a.z==b.z && a.y==b.y && a.x==b.x);}
 inline bool SameSample(const mt_tensor &a,const mt_tensor &b) {return(a.z==b.z && a.y==b.y && a.x==b.x);}
 inline bool Overlap(const void *p,size_t bytes,const mt_tensor &t)
 {
  const char *a=static_cast<const char*>(p);
  const char *b=reinterpret_cast<const char*>(t.p);
  return(bytes!=0 && Bytes(t)!=0 && a<b+Bytes(t) && b<a+bytes);
 }
 inline bool Overlap(const mt_tensor &a,const mt_tensor &b) {return(Overlap(a.p,Bytes(a),b));}
 inline bool Covers(const void *p,size_t bytes,const mt_tensor &t)///<[p,p+bytes) holds all of t
 {
  const char *a=static_cast<const char*>(p);
  const char *b=reinterpret_cast<const char*>(t.p);
  return(a<=b && b+Bytes(t)<=a+bytes);
 }
 // the functions (and derivatives) that the batch-norm kernels apply themselves
 inline bool FusedFunction(int func) {return(func==MT_F_RELU || func==MT_F_LEAKY_RELU || func==MT_F_LINEAR);}
 inline bool Near(float a,double b) {return(fabs(static_cast<double>(a)-b)<=1e-6*(fabs(b)>1?fabs(b):1));}

 // the call as the reference's layer wrote it
 inline void RunLiteral(const SOp &op)
 {
  switch(op.Kind)
  {
   case OP_FILL:Check(mt_fill(&op.T[0],op.A));break;
   case OP_ADD_SUM_W:Check(mt_add_sum_w(&op.T[0],&op.T[1],&op.T[2],op.A,op.B));break;
   case OP_ADD:Check(mt_add(&op.T[0],&op.T[1],&op.T[2],op.A,op.B));break;
   case OP_SUB:Check(mt_sub(&op.T[0],&op.T[1],&op.T[2],op.A,op.B));break;
   case OP_POW2:Check(mt_pow2(&op.T[0],&op.T[1],op.A));break;
   case OP_SQRT:Check(mt_sqrt(&op.T[0],&op.T[1],op.A,op.B));break;
   case OP_INV:Check(mt_inv(&op.T[0],&op.T[1]));break;
   case OP_ITEM_PRODUCTION:Check(mt_tensor_item_production(&op.T[0],&op.T[1],&op.T[2]));break;
   case OP_MUL_VALUE:Check(mt_mul_value(&op.T[0],&op.T[1],op.A));break;
   case OP_FUNCTION:Check(mt_apply_func(&op.T[0],&op.T[1],op.Func));break;
   case OP_DIFFERENTIAL:Check(mt_apply_func(&op.T[0],&op.T[1],MT_F_DIFFERENTIAL+op.Func));break;
   case OP_ADAM:Check(mt_adam(&op.T[0],&op.T[1],&op.T[2],&op.T[3],op.BatchSize,op.Speed,op.Beta1,op.Beta2,op.Epsilon,op.Iteration));break;
   default:throw("mi355::RunLiteral: unknown operation");
  }
 }

 // ---- the known sequences ---------------------------------------------------------------------------------------------
 // A matcher walks the queue from `first` and returns 0 (not this sequence), 1 (its beginning), 2 (all of it) or 3 (all
 // of it, and the next call may still belong to it: the function layer's Forward behind a batch-norm layer's,
 // netlayer/cnetlayerfunction.cu.h:202-212).
 struct SBatchNormForward///<netlayer/cnetlayerbatchnormalization.cu.h:301-371, training mode
 {
  mt_tensor Mean,X,NewMean,XHat,Var,Scratch,NewVar,SqrtVar,IVar,Gamma,Beta,H;
  mt_tensor OldMean,OldVar;///<what the running statistics are blended from: the same tensors, unless they shared their block with a copy
  float Momentum,Epsilon;
  bool HasFunction;
  int Func;
  mt_tensor F;///<the function layer's output, when its call follows
  enum {LENGTH=13};
 };
 struct SBatchNormInference///<the same lines in inference mode (:326-371)
 {
  mt_tensor X,Mean,XHat,Var,SqrtVar,IVar,Scratch,Gamma,Beta,H;
  float Epsilon;
  bool HasFunction;
  int Func;
  mt_tensor F;
  enum {LENGTH=6};
 };
 struct SBatchNormBackward///<:578-604
 {
  mt_tensor SumA,SumB,DXHat,Delta,Gamma,Scratch,XHat,DGamma,DBeta,Prev,IVar;
  bool Gradients;
  size_t Length;
 };
 inline bool Distinct(const mt_tensor *const *list,size_t count)
 {
  for(size_t a=0;a<count;a++)
   for(size_t b=a+1;b<count;b++)
    if (Overlap(*list[a],*list[b])==true) return(false);
  return(true);
 }
 inline bool OneSampleOf(const mt_tensor &t,const mt_tensor &batch) {return(t.w==1 && SameSample(t,batch)==true);}

 inline int MatchBatchNormForward(const std::vector<SOp> &q,size_t first,SBatchNormForward &m)
 {
  const size_t n=q.size()-first;
  if (n>SBatchNormForward::LENGTH+1) return(0);
  m.HasFunction=false;m.Func=MT_F_NONE;
  for(size_t i=0;i<n;i++)
  {
   const SOp &o=q[first+i];
   switch(i)
   {
    case 0:if (o.Kind!=OP_FILL || o.A!=0 || o.T[0].w!=1) return(0);
           m.Mean=o.T[0];break;
    case 1:if (o.Kind!=OP_ADD_SUM_W || !Same(o.T[0],m.Mean) || !Same(o.T[1],m.Mean) || o.A!=1 || o.T[2].w==0 || !Near(o.B,1.0/o.T[2].w) || !SameSample(o.T[2],m.Mean)) return(0);
           m.X=o.T[2];break;
    case 2:if (o.Kind!=OP_ADD || !OneSampleOf(o.T[1],m.X) || !Same(o.T[2],m.Mean) || !OneSampleOf(o.T[0],m.X) || !Near(o.B,1.0-static_cast<double>(o.A))) return(0);
           m.NewMean=o.T[0];m.OldMean=o.T[1];m.Momentum=o.A;break;
    case 3:if (o.Kind!=OP_SUB || !Same(o.T[1],m.X) || !Same(o.T[2],m.Mean) || o.A!=1 || o.B!=1 || o.T[0].w!=m.X.w || !SameSample(o.T[0],m.X)) return(0);
           m.XHat=o.T[0];break;
    case 4:if (o.Kind!=OP_FILL || o.A!=0 || !OneSampleOf(o.T[0],m.X)) return(0);
           m.Var=o.T[0];break;
    case 5:if (o.Kind!=OP_POW2 || !Same(o.T[1],m.XHat) || o.A!=1 || o.T[0].w!=m.X.w || !SameSample(o.T[0],m.X)) return(0);
           m.Scratch=o.T[0];break;
    case 6:if (o.Kind!=OP_ADD_SUM_W || !Same(o.T[0],m.Var) || !Same(o.T[1],m.Var) || !Same(o.T[2],m.Scratch) || o.A!=1 || !Near(o.B,1.0/m.X.w)) return(0);
           break;
    case 7:if (o.Kind!=OP_ADD || !OneSampleOf(o.T[1],m.X) || !Same(o.T[2],m.Var) || !OneSampleOf(o.T[0],m.X) || o.A!=m.Momentum || !Near(o.B,1.0-static_cast<double>(o.A))) return(0);
           m.NewVar=o.T[0];m.OldVar=o.T[1];break;
    case 8:if (o.Kind!=OP_SQRT || !Same(o.T[1],m.Var) || o.A!=1 || !OneSampleOf(o.T[0],m.X)) return(0);
           m.SqrtVar=o.T[0];m.Epsilon=o.B;break;
    case 9:if (o.Kind!=OP_INV || !Same(o.T[1],m.SqrtVar) || !OneSampleOf(o.T[0],m.X)) return(0);
           m.IVar=o.T[0];break;
    case 10:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[0],m.XHat) || !Same(o.T[1],m.XHat) || !Same(o.T[2],m.IVar)) return(0);
            break;
    case 11:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[0],m.Scratch) || !Same(o.T[2],m.XHat) || !OneSampleOf(o.T[1],m.X)) return(0);
            m.Gamma=o.T[1];break;
    case 12:if (o.Kind!=OP_ADD || !Same(o.T[1],m.Scratch) || !OneSampleOf(o.T[2],m.X) || o.A!=1 || o.B!=1 || o.T[0].w!=m.X.w || !SameSample(o.T[0],m.X)) return(0);
            m.Beta=o.T[2];m.H=o.T[0];break;
    case 13:if (o.Kind!=OP_FUNCTION || FusedFunction(o.Func)==false || !Same(o.T[1],m.H) || o.T[0].w!=m.X.w || !SameSample(o.T[0],m.X)) return(0);
            m.F=o.T[0];m.Func=o.Func;m.HasFunction=true;break;
   }
  }
  if (n<SBatchNormForward::LENGTH) return(1);
  const mt_tensor *all[13]={&m.Mean,&m.X,&m.NewMean,&m.XHat,&m.Var,&m.Scratch,&m.NewVar,&m.SqrtVar,&m.IVar,&m.Gamma,&m.Beta,&m.H,&m.F};
  if (Distinct(all,m.HasFunction==true?13:12)==false) return(0);
  if (m.HasFunction==true && (Overlap(m.F,m.OldMean)==true || Overlap(m.F,m.OldVar)==true)) return(0);
  // a running statistic blended from another block (its tensor shared the old one with a copy) must not be one of the outputs
  for(int n=0;n<12;n++)
  {
   if (Same(m.OldMean,m.NewMean)==false && Overlap(m.OldMean,*all[n])==true && all[n]!=&m.NewMean) return(0);
   if (Same(m.OldVar,m.NewVar)==false && Overlap(m.OldVar,*all[n])==true && all[n]!=&m.NewVar) return(0);
  }
  if ((Same(m.OldMean,m.NewMean)==false && Overlap(m.OldMean,m.NewMean)==true) || (Same(m.OldVar,m.NewVar)==false && Overlap(m.OldVar,m.NewVar)==true)) return(0);
  return(m.HasFunction==true?2:3);
 }

 inline int MatchBatchNormInference(const std::vector<SOp> &q,size_t first,SBatchNormInference &m)
 {
  const size_t n=q.size()-first;
  if (n>SBatchNormInference::LENGTH+1) return(0);
  m.HasFunction=false;m.Func=MT_F_NONE;
  for(size_t i=0;i<n;i++)
  {
   const SOp &o=q[first+i];
   switch(i)
   {
    case 0:if (o.Kind!=OP_SUB || o.A!=1 || o.B!=1 || o.T[1].w==0 || o.T[0].w!=o.T[1].w || !SameSample(o.T[0],o.T[1]) || !OneSampleOf(o.T[2],o.T[1])) return(0);
           m.XHat=o.T[0];m.X=o.T[1];m.Mean=o.T[2];break;
    case 1:if (o.Kind!=OP_SQRT || o.A!=1 || !OneSampleOf(o.T[0],m.X) || !OneSampleOf(o.T[1],m.X)) return(0);
           m.SqrtVar=o.T[0];m.Var=o.T[1];m.Epsilon=o.B;break;
    case 2:if (o.Kind!=OP_INV || !Same(o.T[1],m.SqrtVar) || !OneSampleOf(o.T[0],m.X)) return(0);
           m.IVar=o.T[0];break;
    case 3:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[0],m.XHat) || !Same(o.T[1],m.XHat) || !Same(o.T[2],m.IVar)) return(0);
           break;
    case 4:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[2],m.XHat) || !OneSampleOf(o.T[1],m.X) || o.T[0].w!=m.X.w || !SameSample(o.T[0],m.X)) return(0);
           m.Scratch=o.T[0];m.Gamma=o.T[1];break;
    case 5:if (o.Kind!=OP_ADD || !Same(o.T[1],m.Scratch) || !OneSampleOf(o.T[2],m.X) || o.A!=1 || o.B!=1 || o.T[0].w!=m.X.w || !SameSample(o.T[0],m.X)) return(0);
           m.Beta=o.T[2];m.H=o.T[0];break;
    case 6:if (o.Kind!=OP_FUNCTION || FusedFunction(o.Func)==false || !Same(o.T[1],m.H) || o.T[0].w!=m.X.w || !SameSample(o.T[0],m.X)) return(0);
           m.F=o.T[0];m.Func=o.Func;m.HasFunction=true;break;
   }
  }
  if (n<SBatchNormInference::LENGTH) return(1);
  const mt_tensor *all[11]={&m.X,&m.Mean,&m.XHat,&m.Var,&m.SqrtVar,&m.IVar,&m.Scratch,&m.Gamma,&m.Beta,&m.H,&m.F};
  if (Distinct(all,m.HasFunction==true?11:10)==false) return(0);
  return(m.HasFunction==true?2:3);
 }

 inline int MatchBatchNormBackward(const std::vector<SOp> &q,size_t first,SBatchNormBackward &m)
 {
  const size_t n=q.size()-first;
  if (n>15) return(0);
  m.Gradients=false;
  m.Length=12;
  for(size_t i=0;i<n;i++)
  {
   const SOp &o=q[first+i];
   size_t step=i;
   if (i>=6)
   {
    // with create_delta_weight three more calls follow the two sums (:586-592); the seventh call tells which form this is
    if (i==6) m.Gradients=(o.Kind==OP_ITEM_PRODUCTION);
    if (m.Gradients==true) m.Length=15;
    else step=i+3;
   }
   switch(step)
   {
    case 0:if (o.Kind!=OP_FILL || o.A!=0 || o.T[0].w!=1) return(0);
           m.SumA=o.T[0];break;
    case 1:if (o.Kind!=OP_FILL || o.A!=0 || o.T[0].w!=1 || !SameSample(o.T[0],m.SumA)) return(0);
           m.SumB=o.T[0];break;
    case 2:if (o.Kind!=OP_ITEM_PRODUCTION || o.T[1].w==0 || o.T[0].w!=o.T[1].w || !SameSample(o.T[0],o.T[1]) || !SameSample(o.T[1],m.SumA) || !OneSampleOf(o.T[2],o.T[1])) return(0);
           m.DXHat=o.T[0];m.Delta=o.T[1];m.Gamma=o.T[2];break;
    case 3:if (o.Kind!=OP_ADD_SUM_W || !Same(o.T[0],m.SumA) || !Same(o.T[1],m.SumA) || !Same(o.T[2],m.DXHat) || o.A!=1 || o.B!=1) return(0);
           break;
    case 4:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[1],m.DXHat) || o.T[0].w!=m.Delta.w || !SameSample(o.T[0],m.Delta) || o.T[2].w!=m.Delta.w || !SameSample(o.T[2],m.Delta)) return(0);
           m.Scratch=o.T[0];m.XHat=o.T[2];break;
    case 5:if (o.Kind!=OP_ADD_SUM_W || !Same(o.T[0],m.SumB) || !Same(o.T[1],m.SumB) || !Same(o.T[2],m.Scratch) || o.A!=1 || o.B!=1) return(0);
           break;
    case 6:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[0],m.Scratch) || !Same(o.T[1],m.Delta) || !Same(o.T[2],m.XHat)) return(0);
           break;
    case 7:if (o.Kind!=OP_ADD_SUM_W || !Same(o.T[0],o.T[1]) || !Same(o.T[2],m.Scratch) || !OneSampleOf(o.T[0],m.Delta) || o.A!=1 || o.B!=1) return(0);
           m.DGamma=o.T[0];break;
    case 8:if (o.Kind!=OP_ADD_SUM_W || !Same(o.T[0],o.T[1]) || !Same(o.T[2],m.Delta) || !OneSampleOf(o.T[0],m.Delta) || o.A!=1 || o.B!=1) return(0);
           m.DBeta=o.T[0];break;
    case 9:if (o.Kind!=OP_MUL_VALUE || !Same(o.T[1],m.DXHat) || o.A!=static_cast<float>(m.Delta.w) || o.T[0].w!=m.Delta.w || !SameSample(o.T[0],m.Delta)) return(0);
           m.Prev=o.T[0];break;
    case 10:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[0],m.Scratch) || !Same(o.T[1],m.XHat) || !Same(o.T[2],m.SumB)) return(0);
            break;
    case 11:if (o.Kind!=OP_SUB || !Same(o.T[0],m.Prev) || !Same(o.T[1],m.Prev) || !Same(o.T[2],m.Scratch) || o.A!=1 || o.B!=1) return(0);
            break;
    case 12:if (o.Kind!=OP_SUB || !Same(o.T[0],m.Prev) || !Same(o.T[1],m.Prev) || !Same(o.T[2],m.SumA) || o.A!=1 || o.B!=1) return(0);
            break;
    case 13:if (o.Kind!=OP_ITEM_PRODUCTION || !Same(o.T[0],m.Prev) || !Same(o.T[1],m.Prev) || !OneSampleOf(o.T[2],m.Delta)) return(0);
            m.IVar=o.T[2];break;
    case 14:if (o.Kind!=OP_MUL_VALUE || !Same(o.T[0],m.Prev) || !Same(o.T[1],m.Prev) || !Near(o.A,1.0/m.Delta.w)) return(0);
            break;
   }
  }
  if (n>m.Length) return(0);
  if (n<=6 || n<m.Length) return(1);
  const mt_tensor *all[11]={&m.SumA,&m.SumB,&m.DXHat,&m.Delta,&m.Gamma,&m.Scratch,&m.XHat,&m.Prev,&m.IVar,&m.DGamma,&m.DBeta};
  return(Distinct(all,m.Gradients==true?11:9)==true?2:0);
 }

 // The two calls of CNetLayerFunction::SetOutputError (netlayer/cnetlayerfunction.cu.h:347-358) followed by the batch-norm
 // layer's backward pass on the tensor they produce:  Front = f'(Output of the batch norm);  Front = Error * Front;  then
 // the sequence above with Delta = Front (the batch-norm layer's copy of it shares its block).
 struct SFunctionBackward
 {
  mt_tensor Front,Output,Error;
  int Func;
  SBatchNormBackward Norm;
 };
 inline int MatchFunctionBackward(const std::vector<SOp> &q,size_t first,SFunctionBackward &m)
 {
  const size_t n=q.size()-first;
  if (n>17) return(0);
  const SOp &d=q[first];
  if (d.Kind!=OP_DIFFERENTIAL || FusedFunction(d.Func)==false || d.T[0].w==0 || d.T[0].w!=d.T[1].w || !SameSample(d.T[0],d.T[1]) || Overlap(d.T[0],d.T[1])) return(0);
  m.Front=d.T[0];m.Output=d.T[1];m.Func=d.Func;
  if (n==1) return(1);
  const SOp &p=q[first+1];
  if (p.Kind!=OP_ITEM_PRODUCTION || !Same(p.T[0],m.Front) || !Same(p.T[2],m.Front) || p.T[1].w!=m.Front.w || !SameSample(p.T[1],m.Front) || Overlap(p.T[1],m.Front) || Overlap(p.T[1],m.Output)) return(0);
  m.Error=p.T[1];
  if (n==2) return(1);
  const int inner=MatchBatchNormBackward(q,first+2,m.Norm);
  if (inner==0) return(0);
  if (n>=5 && Same(m.Norm.Delta,m.Front)==false) return(0);///<(the third call of the inner sequence names its Delta)
  if (inner==1) return(1);
  const mt_tensor *mine[2]={&m.Error,&m.Output};
  const mt_tensor *theirs[10]={&m.Norm.SumA,&m.Norm.SumB,&m.Norm.DXHat,&m.Norm.Gamma,&m.Norm.Scratch,&m.Norm.XHat,&m.Norm.Prev,&m.Norm.IVar,&m.Norm.DGamma,&m.Norm.DBeta};
  for(int a=0;a<2;a++)
   for(int b=0;b<(m.Norm.Gradients==true?10:8);b++)
    if (Overlap(*mine[a],*theirs[b])==true) return(0);
  return(2);
 }

 // Fill calls with one value, or Adam calls with one set of hyper-parameters: neighbours in the queue run as one launch
 inline bool SameRun(const SOp &h,const SOp &o)
 {
  if (h.Kind!=OP_FILL && h.Kind!=OP_ADAM) return(false);
  if (o.Kind!=h.Kind) return(false);
  if (h.Kind==OP_FILL && o.A!=h.A) return(false);
  if (h.Kind==OP_ADAM && (o.BatchSize!=h.BatchSize || o.Speed!=h.Speed || o.Beta1!=h.Beta1 || o.Beta2!=h.Beta2 || o.Epsilon!=h.Epsilon || o.Iteration!=h.Iteration)) return(false);
  return(true);
 }

 // whether the first `count` calls of the queue are one such run
 inline bool IsRun(const std::vector<SOp> &q,size_t count)
 {
  if (count==0) return(true);
  if (q[0].Kind!=OP_FILL && q[0].Kind!=OP_ADAM) return(false);
  for(size_t i=1;i<count;i++)
   if (SameRun(q[0],q[i])==false) return(false);
  return(true);
 }

 class COpQueue
 {
  private:
   std::vector<SOp> Queue;///<calls made and not yet run, in order
   std::vector<SOp> Pending;///<defining calls of scratch tensors that a sequence's kernel did not write, in order
   // What a forward pass in training mode established: Output = Gamma * XHat + Beta, element by element, for as long as
   // none of the four tensors is written.  The backward pass behind a function layer needs Beta, which its own calls
   // never name, to take the function's derivative at Gamma * XHat + Beta instead of reading Output.
   struct SNormFact {mt_tensor Output,Gamma,Beta,XHat;};
   std::vector<SNormFact> Facts;
   std::vector<const void*> OwnOutputsRead;///<batch-norm outputs that were left pending once and had to be written after all
  public:
   // counters, for tests and measurements
   size_t ForwardFused,InferenceFused,BackwardFused,FunctionBackwardFused,FillRuns,AdamRuns,RunCalls,LiteralCalls,PendingRun,PendingDropped,OwnOutputsPending;
   COpQueue(void):ForwardFused(0),InferenceFused(0),BackwardFused(0),FunctionBackwardFused(0),FillRuns(0),AdamRuns(0),RunCalls(0),LiteralCalls(0),PendingRun(0),PendingDropped(0),OwnOutputsPending(0) {}

   // a call of CTensorMath; operands are up to date on the device, the output is marked device-side by the caller
   void Submit(const SOp &op)
   {
    if (FuseSequences()==false)
    {
     Flush();
     Settle(&op,1);
     RunLiteral(op);
     return;
    }
    Queue.push_back(op);
    for(;;)
    {
     if (Scan(false)!=0) return;
     if (IsRun(Queue,Queue.size())==true) return;
     if (Queue.size()==1) {RunQueue();return;}
     // the last call fits nothing the queue was waiting for: the calls before it run (as the sequence they are, if they
     // are a whole one; else as written), it starts anew
     const SOp last=Queue.back();
     Queue.pop_back();
     RunQueue();
     Queue.push_back(last);
    }
   }
   // everything queued runs now, call by call (a collected run as its one launch)
   void Flush(void)
   {
    if (Queue.empty()==false) RunQueue();
   }
   // Somebody outside the queue is about to read and/or write device memory [p,p+bytes): a call of the tensor classes
   // that is not deferred, a copy to or from the host, a buffer that is freed.  `write` means all of it is overwritten
   // (or goes away); with `read` as well the old contents are used first.
   void Access(const void *p,size_t bytes,bool read,bool write)
   {
    if (p==NULL || bytes==0) return;
    if (Queue.empty()==false)
    {
     bool touches=false;///<calls on other tensors pass: they depend on nothing the queue holds, and nothing in it on them
     for(size_t i=0;i<Queue.size() && touches==false;i++)
      for(uint8_t t=0;t<Queue[i].Count;t++)
       if (Overlap(p,bytes,Queue[i].T[t])==true) touches=true;
     if (touches==true) RunQueue();
    }
    if (Pending.empty()==false) SettleRange(p,bytes,read,write);
    if (write==true && Facts.empty()==false)
    {
     mt_tensor range=Range(p,bytes);
     Forget(&range,1);
    }
   }
   bool Idle(void) const {return(Queue.empty() && Pending.empty());}
   size_t ForwardPassesOnRecord(void) const {return(Facts.size());}
   size_t QueuedCalls(void) const {return(Queue.size());}
   size_t PendingCalls(void) const {return(Pending.size());}
  private:
   // Looks for a known sequence in the queue, which may begin with a run that is still collecting.  Returns 2 when a
   // whole sequence was found and has run (with everything in front of it), 1 when the queue is the beginning of one (or a
   // whole one that the next call may extend) and waits, 0 when it is neither.  `final`: nothing more will be added --
   // beginnings do not count, a whole sequence that could have been extended runs as it is.
   int Scan(bool final)
   {
    for(size_t first=0;first<Queue.size();first++)
    {
     if (IsRun(Queue,first)==false) break;
     SBatchNormForward f;
     SBatchNormInference i;
     SBatchNormBackward b;
     SFunctionBackward fb;
     const int mf=MatchBatchNormForward(Queue,first,f),mi=MatchBatchNormInference(Queue,first,i),mb=MatchBatchNormBackward(Queue,first,b);
     const int mfb=MatchFunctionBackward(Queue,first,fb);
     const bool forward=(mf==2 || (final==true && mf==3)),inference=(mi==2 || (final==true && mi==3));
     if (forward==true || inference==true || mb==2 || mfb==2)
     {
      std::vector<SOp> sequence(Queue.begin()+first,Queue.end());
      Queue.resize(first);
      if (Queue.empty()==false) RunQueue();
      if (forward==true) RunForward(sequence,f);
      else if (inference==true) RunInference(sequence,i);
      else if (mb==2) RunBackward(sequence,b);
      else RunFunctionBackward(sequence,fb);
      return(2);
     }
     if (final==false && (mf==1 || mi==1 || mb==1 || mfb==1 || mf==3 || mi==3)) return(1);
    }
    return(0);
   }
   void RunQueue(void)
   {
    if (Scan(true)==2) return;
    std::vector<SOp> q;
    q.swap(Queue);
    size_t first=0;
    while(first<q.size())
    {
     size_t end=first+1;
     while(end<q.size() && SameRun(q[first],q[end])==true) end++;
     const size_t count=end-first;
     if (count>=2)   // a run of fills or of Adam updates (other calls may stand in front of it and behind it)
     {
      Settle(&q[first],count);
      RunCalls+=count;
      std::vector<const mt_tensor*> a(count),b(count),c(count),d(count);
      for(size_t i=0;i<count;i++) {a[i]=&q[first+i].T[0];b[i]=&q[first+i].T[1];c[i]=&q[first+i].T[2];d[i]=&q[first+i].T[3];}
      if (q[first].Kind==OP_FILL)
      {
       FillRuns++;
       Check(mt_fill_many(static_cast<uint32_t>(count),&a[0],q[first].A));
      }
      else
      {
       AdamRuns++;
       Check(mt_adam_many(static_cast<uint32_t>(count),&a[0],&b[0],&c[0],&d[0],q[first].BatchSize,q[first].Speed,q[first].Beta1,q[first].Beta2,q[first].Epsilon,q[first].Iteration));
      }
     }
     else
     {
      Settle(&q[first],1);
      LiteralCalls++;
      RunLiteral(q[first]);
     }
     first=end;
    }
   }
   void RunForward(const std::vector<SOp> &sequence,const SBatchNormForward &m)
   {
    Settle(&sequence[0],sequence.size());
    ForwardFused++;
    // With the function layer's call behind it the kernel writes that layer's output.  The batch-norm layer's own output
    // is one more store of the whole activation that a forward pass on its own never reads (the next layer takes the
    // function's output, the next pass overwrites it): it stays pending as H = Gamma * XHat, H = H + Beta -- the layer's
    // own two calls with H in place of the scratch tensor, which the backward pass reuses.  In a training loop the
    // optimiser changes Gamma and Beta, and the pending calls have to run first: two launches instead of one store.  So
    // an output whose pending calls ever ran is written by the kernel from then on (OwnOutputsRead).
    const bool written=(m.HasFunction==false || WasRead(m.H.p)==true);
    if (m.HasFunction==true) Check(mt_batchnorm_forward_train_from(&m.F,&m.X,&m.Gamma,&m.Beta,&m.XHat,&m.IVar,&m.Mean,&m.Var,&m.NewMean,&m.NewVar,&m.OldMean,&m.OldVar,m.Momentum,m.Epsilon,m.Func,written==true?&m.H:NULL));
    else Check(mt_batchnorm_forward_train_from(&m.H,&m.X,&m.Gamma,&m.Beta,&m.XHat,&m.IVar,&m.Mean,&m.Var,&m.NewMean,&m.NewVar,&m.OldMean,&m.OldVar,m.Momentum,m.Epsilon,MT_F_NONE,NULL));
    Pending.push_back(sequence[8]);///<SqrtVar = sqrt(Var + epsilon)
    Pending.push_back(sequence[11]);///<Scratch = Gamma * XHat
    if (written==false)
    {
     SOp product=sequence[11],sum=sequence[12];
     product.T[0]=m.H;product.Own=1;
     sum.T[1]=m.H;sum.Own=1;
     Pending.push_back(product);
     Pending.push_back(sum);
     OwnOutputsPending++;
    }
    SNormFact fact;
    fact.Output=m.H;fact.Gamma=m.Gamma;fact.Beta=m.Beta;fact.XHat=m.XHat;
    Facts.push_back(fact);
   }
   void RunInference(const std::vector<SOp> &sequence,const SBatchNormInference &m)
   {
    Settle(&sequence[0],sequence.size());
    InferenceFused++;
    if (m.HasFunction==true)
    {
     // the function layer's output from the kernel; the batch-norm layer's own output stays pending with the scratch tensors
     Check(mt_batchnorm_forward_infer_func(&m.F,&m.X,&m.Gamma,&m.Beta,&m.Mean,&m.Var,m.Epsilon,m.Func));
     for(size_t i=0;i<6;i++) Pending.push_back(sequence[i]);
     return;
    }
    Check(mt_batchnorm_forward_infer_func(&m.H,&m.X,&m.Gamma,&m.Beta,&m.Mean,&m.Var,m.Epsilon,MT_F_NONE));
    for(size_t i=0;i<5;i++) Pending.push_back(sequence[i]);///<everything but the output itself
   }
   void RunBackward(const std::vector<SOp> &sequence,const SBatchNormBackward &m)
   {
    Settle(&sequence[0],sequence.size());
    BackwardFused++;
    Check(mt_batchnorm_backward_keep(&m.Prev,m.Gradients==true?&m.DGamma:NULL,m.Gradients==true?&m.DBeta:NULL,&m.Delta,&m.Gamma,&m.XHat,&m.IVar,&m.DXHat,&m.SumA,&m.SumB));
    Pending.push_back(sequence[m.Gradients==true?10:7]);///<Scratch = XHat * SumB
   }

   // The function layer's two calls and the batch-norm layer's backward pass as one kernel, when the forward pass that
   // produced the function layer's input is on record (Beta); else the two calls as written and the backward pass as its
   // own kernel.
   void RunFunctionBackward(const std::vector<SOp> &sequence,const SFunctionBackward &m)
   {
    const SNormFact *fact=NULL;
    for(size_t i=0;i<Facts.size();i++)
     if (Same(Facts[i].Output,m.Output)==true && Same(Facts[i].Gamma,m.Norm.Gamma)==true && Same(Facts[i].XHat,m.Norm.XHat)==true) fact=&Facts[i];
    if (fact==NULL)
    {
     for(size_t i=0;i<2;i++)
     {
      Settle(&sequence[i],1);
      LiteralCalls++;
      RunLiteral(sequence[i]);
     }
     const std::vector<SOp> rest(sequence.begin()+2,sequence.end());
     RunBackward(rest,m.Norm);
     return;
    }
    const mt_tensor beta=fact->Beta;///<(Settle below may drop the record)
    Settle(&sequence[0],sequence.size(),&m.Output);///<(the kernel does not read the function's input: it has Gamma, XHat and Beta)
    FunctionBackwardFused++;
    const SBatchNormBackward &b=m.Norm;
    Check(mt_batchnorm_backward_func_keep(&b.Prev,b.Gradients==true?&b.DGamma:NULL,b.Gradients==true?&b.DBeta:NULL,&m.Error,&b.Gamma,&beta,&b.XHat,&b.IVar,m.Func,&b.DXHat,&b.SumA,&b.SumB,&m.Front));
    Pending.push_back(sequence[2+(b.Gradients==true?10:7)]);///<Scratch = XHat * SumB
   }

   // ---- pending calls ------------------------------------------------------------------------------------------------
   // Runs pending call `j` after every earlier pending call that shares a tensor with it (program order among related calls).
   void RunPending(size_t j,std::vector<uint8_t> &state)///<state: 0 waiting, 1 done or dropped
   {
    if (state[j]!=0) return;
    for(size_t i=0;i<j;i++)
    {
     if (state[i]!=0) continue;
     bool related=false;
     for(uint8_t a=0;a<Pending[i].Count && related==false;a++)
      for(uint8_t b=0;b<Pending[j].Count;b++)
       if (Overlap(Pending[i].T[a],Pending[j].T[b])==true) {related=true;break;}
     if (related==true) RunPending(i,state);
    }
    state[j]=1;
    PendingRun++;
    if (Pending[j].Own!=0 && WasRead(Pending[j].T[0].p)==false && OwnOutputsRead.size()<1024) OwnOutputsRead.push_back(Pending[j].T[0].p);
    RunLiteral(Pending[j]);
   }
   bool WasRead(const void *p) const
   {
    for(size_t i=0;i<OwnOutputsRead.size();i++)
     if (OwnOutputsRead[i]==p) return(true);
    return(false);
   }
   // Before `count` calls run as one unit (a sequence's kernel, a run, one literal call): pending calls whose output the
   // unit overwrites without anybody having read it are forgotten; those whose output the unit reads, or whose inputs
   // it changes, run first.
   // `unread`: a tensor that the unit's calls name as an input but the kernel that stands for them does not touch.
   void Settle(const SOp *unit,size_t count,const mt_tensor *unread=NULL)
   {
    if (Facts.empty()==false)
    {
     std::vector<mt_tensor> written;
     for(size_t i=0;i<count;i++)
      for(uint8_t t=0;t<unit[i].Count;t++)
       if ((unit[i].Writes&(1u<<t))!=0) written.push_back(unit[i].T[t]);
     if (written.empty()==false) Forget(&written[0],written.size());
    }
    if (Pending.empty()==true) return;
    // what the unit reads from outside itself, and what it overwrites
    std::vector<mt_tensor> reads,writes;
    for(size_t i=0;i<count;i++)
    {
     const SOp &o=unit[i];
     for(uint8_t t=0;t<o.Count;t++)
     {
      if ((o.Reads&(1u<<t))==0) continue;
      if (unread!=NULL && Same(o.T[t],*unread)==true) continue;
      bool inside=false;
      for(size_t w=0;w<writes.size();w++)
       if (Covers(writes[w].p,Bytes(writes[w]),o.T[t])==true) inside=true;
      if (inside==false) reads.push_back(o.T[t]);
     }
     for(uint8_t t=0;t<o.Count;t++)
      if ((o.Writes&(1u<<t))!=0) writes.push_back(o.T[t]);
    }
    SettleSets(reads,writes);
   }
   // a forward pass on record is forgotten when any of its four tensors is written
   void Forget(const mt_tensor *written,size_t count)
   {
    std::vector<SNormFact> left;
    for(size_t f=0;f<Facts.size();f++)
    {
     bool touched=false;
     for(size_t w=0;w<count && touched==false;w++)
      touched=Overlap(written[w],Facts[f].Output) || Overlap(written[w],Facts[f].Gamma) || Overlap(written[w],Facts[f].Beta) || Overlap(written[w],Facts[f].XHat);
     if (touched==false) left.push_back(Facts[f]);
    }
    Facts.swap(left);
   }
   static mt_tensor Range(const void *p,size_t bytes)
   {
    mt_tensor range;
    range.p=static_cast<float*>(const_cast<void*>(p));
    range.w=1;range.z=1;range.y=1;range.x=static_cast<uint32_t>(bytes/sizeof(float));
    if (static_cast<size_t>(range.x)*sizeof(float)!=bytes) {range.y=static_cast<uint32_t>((bytes/sizeof(float)+0xffffu)>>16);range.x=1u<<16;}///<(a buffer of 16 GiB or more, or one that is no whole number of floats: a range that covers it)
    return(range);
   }
   void SettleRange(const void *p,size_t bytes,bool read,bool write)
   {
    const mt_tensor range=Range(p,bytes);
    std::vector<mt_tensor> reads,writes;
    if (read==true) reads.push_back(range);
    if (write==true) writes.push_back(range);
    SettleSets(reads,writes);
   }
   void SettleSets(const std::vector<mt_tensor> &reads,const std::vector<mt_tensor> &writes)
   {
    const size_t n=Pending.size();
    std::vector<uint8_t> state(n,0);
    std::vector<uint8_t> dead(n,0);
    // from the last pending call to the first: forgotten when its output is overwritten whole, read by nobody outside
    // and by no later pending call that stays
    for(size_t k=n;k>0;k--)
    {
     const size_t j=k-1;
     const mt_tensor &out=Pending[j].T[0];
     bool overwritten=false,wanted=false;
     for(size_t w=0;w<writes.size();w++)
      if (Covers(writes[w].p,Bytes(writes[w]),out)==true) overwritten=true;
     for(size_t r=0;r<reads.size();r++)
      if (Overlap(reads[r],out)==true) wanted=true;
     for(size_t l=j+1;l<n && wanted==false;l++)
     {
      if (dead[l]!=0) continue;
      for(uint8_t t=0;t<Pending[l].Count;t++)
       if ((Pending[l].Reads&(1u<<t))!=0 && Overlap(Pending[l].T[t],out)==true) wanted=true;
     }
     if (overwritten==true && wanted==false) dead[j]=1;
    }
    for(size_t j=0;j<n;j++)
     if (dead[j]!=0) {state[j]=1;PendingDropped++;}
    // the others run when the unit reads their output, or writes into their output or one of their inputs
    for(size_t j=0;j<n;j++)
    {
     if (state[j]!=0) continue;
     bool now=false;
     for(size_t r=0;r<reads.size() && now==false;r++)
      if (Overlap(reads[r],Pending[j].T[0])==true) now=true;
     for(size_t w=0;w<writes.size() && now==false;w++)
      for(uint8_t t=0;t<Pending[j].Count;t++)
       if (Overlap(writes[w],Pending[j].T[t])==true) {now=true;break;}
     if (now==true) RunPending(j,state);
    }
    std::vector<SOp> left;
    for(size_t j=0;j<n;j++)
     if (state[j]==0) left.push_back(Pending[j]);
    Pending.swap(left);
   }
 };

 inline COpQueue& Queue(void)
 {
  static COpQueue *queue=new COpQueue;///<never destroyed: tensors with static lifetime may outlive any static object
  return(*queue);
 }
}

#endif
