// Self-test of the drop-in C++ classes: the checks of the reference's CTensorTest::Test()
// (cuda/ctensortest.cu.h:725-928 and the five convolution tests at :77-652) written against the same public API,
// plus the lazy host/device coherence and the error convention.  Every tensor op below runs on the GPU through
// libmi355tensor.so.  Prints one line per check; exit code 0 when all pass.
#include <math.h>
#include <stdio.h>
#include <string.h>
#include <string>

#include "cuda/tensor.cu.h"
#include "cuda/ctimestamp.cu.h"

namespace SYSTEM
{
 void PutMessage(const std::string &message) {printf("%s\n",message.c_str());}
 void PutMessageToConsole(const std::string &message) {printf("%s\n",message.c_str());}
}

typedef float type_t;
static const uint32_t BATCH=10;
static int failures=0;

static void Report(const char *name,bool ok)
{
 printf("%-64s %s\n",name,ok?"PASS":"FAIL");
 if (!ok) failures++;
}

static bool AllEqual(const CTensor<type_t> &t,const type_t *expected)
{
 for(uint32_t w=0;w<t.GetSizeW();w++)
 {
  uint32_t n=0;
  for(uint32_t z=0;z<t.GetSizeZ();z++)
   for(uint32_t y=0;y<t.GetSizeY();y++)
    for(uint32_t x=0;x<t.GetSizeX();x++,n++)
     if (t.GetElement(w,z,y,x)!=expected[n]) return(false);
 }
 return(true);
}

// fills every batch layer with the same [Z,Y,X] data
static void FillLayers(CTensor<type_t> &t,const type_t *data)
{
 for(uint32_t w=0;w<t.GetSizeW();w++)
 {
  uint32_t n=0;
  for(uint32_t z=0;z<t.GetSizeZ();z++)
   for(uint32_t y=0;y<t.GetSizeY();y++)
    for(uint32_t x=0;x<t.GetSizeX();x++,n++) t.SetElement(w,z,y,x,data[n]);
 }
}

static void MatrixChecks(void)
{
 const type_t m[4]={1,2,3,4};
 CTensor<type_t> a(BATCH,1,2,2),b(BATCH,1,2,2),c(BATCH,1,2,2),a_one(1,1,2,2),b_one(1,1,2,2);
 FillLayers(a,m);FillLayers(b,m);FillLayers(a_one,m);FillLayers(b_one,m);
 Report("element set/get",AllEqual(a,m));
 const type_t twice[4]={2,4,6,8};
 c=a*static_cast<type_t>(2.0);
 Report("tensor * scalar",AllEqual(c,twice));
 c=static_cast<type_t>(2.0)*a;
 Report("scalar * tensor",AllEqual(c,twice));
 const type_t prod[4]={7,10,15,22};
 c=a*b;
 Report("Mul, equal batch",AllEqual(c,prod) && c.GetSizeW()==BATCH);
 c=a_one*b;
 Report("Mul, left operand broadcast over W",AllEqual(c,prod) && c.GetSizeW()==BATCH);
 CTensorMath<type_t>::Mul(c,a,b_one);
 Report("Mul, right operand broadcast over W",AllEqual(c,prod));
 const type_t zero[4]={0,0,0,0};
 c=a-b;
 Report("Sub",AllEqual(c,zero));
 c=a+b;
 Report("Add",AllEqual(c,twice));
 const type_t tr[4]={1,3,2,4};
 c=CTensorMath<type_t>::Transpose(a);
 Report("Transpose",AllEqual(c,tr));
 const type_t sq[4]={1,4,9,16};
 CTensor<type_t> e(BATCH,1,2,2);
 CTensorMath<type_t>::TensorItemProduction(e,a,b);
 Report("TensorItemProduction",AllEqual(e,sq));
}

static void ForwardConvolutionCheck(void)
{
 type_t kernel_a[12],kernel_b[12],image[27];
 for(int n=0;n<12;n++) {kernel_a[n]=n+1;kernel_b[n]=12-n;}
 for(int n=0;n<27;n++) image[n]=n+1;
 CTensor<type_t> kernel(1,1,2,12),bias(1,2,1,1),img(BATCH,3,3,3),out(BATCH,2,2,2);
 for(uint32_t n=0;n<12;n++) {kernel.SetElement(0,0,0,n,kernel_a[n]);kernel.SetElement(0,0,1,n,kernel_b[n]);}
 CTensorMath<type_t>::Fill(bias,0);
 FillLayers(img,image);
 CTensorConv<type_t>::ForwardConvolution(out,img,kernel,2,2,3,2,bias,1,1,0,0);
 const type_t expected[8]={1245,1323,1479,1557,627,705,861,939};
 Report("ForwardConvolution 2x2x3, stride 1",AllEqual(out,expected));
}

static void DeltaWeightChecks(void)
{
 type_t image[49],delta[16];
 for(int n=0;n<49;n++) image[n]=n+1;
 for(int n=0;n<16;n++) delta[n]=n+1;
 CTensor<type_t> img(BATCH,1,7,7),dl(BATCH,1,4,4),dk(BATCH,1,1,25),db(BATCH,1,1,1);
 FillLayers(img,image);FillLayers(dl,delta);
 CTensorMath<type_t>::Fill(db,0);
 CTensorMath<type_t>::Fill(dk,0);
 CTensorConv<type_t>::CreateDeltaWeightAndBias(dk,5,5,1,1,db,img,dl,2,2,2,2);
 const type_t expected[25]={2031,2130,2746,1968,2058, 2724,2823,3628,2598,2688, 3448,3556,4560,3256,3352, 1860,1923,2428,1698,1752, 2301,2364,2974,2076,2130};
 bool ok=true;
 for(uint32_t w=0;w<BATCH;w++)
 {
  for(uint32_t n=0;n<25;n++) ok=ok && dk.GetElement(w,0,0,n)==expected[n];
  ok=ok && db.GetElement(w,0,0,0)==136;
 }
 Report("CreateDeltaWeightAndBias 5x5, stride 2, padding 2",ok);

 const type_t image2[16]={4,5,8,7, 1,8,8,8, 3,6,6,4, 6,5,7,8};
 const type_t dout[4]={2,1,4,4};
 CTensor<type_t> img2(BATCH,1,4,4),d2(BATCH,1,2,2),dk2(BATCH,1,1,9),db2(BATCH,1,1,1);
 FillLayers(img2,image2);FillLayers(d2,dout);
 CTensorMath<type_t>::Fill(dk2,0);
 CTensorMath<type_t>::Fill(db2,0);
 CTensorConv<type_t>::CreateDeltaWeightAndBias(dk2,3,3,1,1,db2,img2,d2,1,1,0,0);
 const type_t expected2[9]={49,82,87,46,72,64,56,66,76};
 ok=true;
 for(uint32_t w=0;w<BATCH;w++)
  for(uint32_t n=0;n<9;n++) ok=ok && dk2.GetElement(w,0,0,n)==expected2[n];
 Report("CreateDeltaWeightAndBias 3x3, stride 1",ok);
}

static void BackwardConvolutionCheck(void)
{
 type_t delta[16];
 for(int n=0;n<16;n++) delta[n]=n+1;
 CTensor<type_t> kernel(1,1,1,25),bias(1,1,1,1),dl(BATCH,1,4,4),out(BATCH,1,7,7);
 for(uint32_t n=0;n<25;n++) kernel.SetElement(0,0,0,n,n+1);
 bias.Zero();
 FillLayers(dl,delta);
 CTensorConv<type_t>::BackwardConvolution(out,dl,kernel,5,5,1,1,bias,2,2,2,2);
 const type_t expected[49]={56,70,124,102,172,134,156, 126,140,244,192,322,244,266, 233,266,450,344,567,422,467, 318,348,556,400,634,452,490,
                            521,578,918,656,1035,734,803, 510,556,868,608,946,660,714, 740,786,1228,858,1336,930,984};
 CTensor<type_t> control(BATCH,1,7,7);
 FillLayers(control,expected);
 Report("BackwardConvolution 5x5, stride 2, padding 2",out.Compare(control,"",false));
}

// A bias that is known to hold zeros reaches the library as one shared block of zeros (mi355::ZeroBlock) and is not read:
// the result is that of a tensor whose zeros were written element by element, and every later write to the tensor ends it.
static void ZeroBiasCheck(void)
{
 type_t delta[16];
 for(int n=0;n<16;n++) delta[n]=n+1;
 CTensor<type_t> kernel(1,1,2,3*16),trained(1,2,1,1),dl(BATCH,2,4,4),out(BATCH,3,8,8),control(BATCH,3,8,8);
 for(uint32_t f=0;f<2;f++)
  for(uint32_t n=0;n<48;n++) kernel.SetElement(0,0,f,n,static_cast<type_t>((n*7+f*5)%11)-5);
 trained.SetElement(0,0,0,0,0.5f);trained.SetElement(0,1,0,0,-0.25f);
 for(uint32_t w=0;w<BATCH;w++)
  for(uint32_t f=0;f<2;f++)
   for(uint32_t n=0;n<16;n++) dl.SetElement(w,f,n/4,n%4,delta[n]*(f+1)+w);
 CTensor<type_t> written(1,2,1,1);
 written.SetElement(0,0,0,0,0);written.SetElement(0,1,0,0,0);   // zeros that the class does not know to be zeros
 CTensorConv<type_t>::BackwardConvolution(control,dl,kernel,4,4,3,2,written,2,2,1,1);
 CTensor<type_t> zeroed=trained;                                   // the layer's own sequence: a copy of the bias, filled with 0
 CTensorMath<type_t>::Fill(zeroed,0);
 CTensorConv<type_t>::BackwardConvolution(out,dl,kernel,4,4,3,2,zeroed,2,2,1,1);
 bool ok=out.Compare(control,"",false) && zeroed.GetElement(0,1,0,0)==0 && trained.GetElement(0,1,0,0)==-0.25f;
 Report("BackwardConvolution with a bias filled with zeros",ok);
 // writes end it: an element set on the host, a device operation into the tensor, a copy of other values
 zeroed.SetElement(0,0,0,0,0.5f);zeroed.SetElement(0,1,0,0,-0.25f);
 CTensorConv<type_t>::BackwardConvolution(out,dl,kernel,4,4,3,2,zeroed,2,2,1,1);
 CTensorConv<type_t>::BackwardConvolution(control,dl,kernel,4,4,3,2,trained,2,2,1,1);
 ok=out.Compare(control,"",false) && out.GetElement(0,0,3,3)!=0;
 CTensorMath<type_t>::Fill(zeroed,0);
 CTensorMath<type_t>::Add(zeroed,zeroed,trained);
 CTensorConv<type_t>::BackwardConvolution(out,dl,kernel,4,4,3,2,zeroed,2,2,1,1);
 ok=ok && out.Compare(control,"",false);
 CTensorMath<type_t>::Fill(zeroed,0);
 zeroed=trained;
 CTensorConv<type_t>::BackwardConvolution(out,dl,kernel,4,4,3,2,zeroed,2,2,1,1);
 ok=ok && out.Compare(control,"",false);
 CTensor<type_t> copy_of_zeros;
 CTensorMath<type_t>::Fill(zeroed,0);
 copy_of_zeros=zeroed;                                               // a copy of zeros holds zeros
 CTensorConv<type_t>::BackwardConvolution(out,dl,kernel,4,4,3,2,copy_of_zeros,2,2,1,1);
 CTensorConv<type_t>::BackwardConvolution(control,dl,kernel,4,4,3,2,written,2,2,1,1);
 ok=ok && out.Compare(control,"",false);
 Report("a write to the bias ends it",ok);
}

static void SummXYCheck(void)
{
 bool ok=true;
 for(uint32_t size=1;size<512;size+=32)
 {
  CTensor<type_t> in(8,16,size,size),out(8,16,1,1);
  in.Fill(1);
  CTensorMath<type_t>::SummXY(out,in);
  for(uint32_t w=0;w<8;w++)
   for(uint32_t z=0;z<16;z++) ok=ok && static_cast<uint32_t>(out.GetElement(w,z,0,0))==size*size;
 }
 Report("SummXY of all-ones, sizes 1..481",ok);
}

static void CoherenceAndErrors(void)
{
 CTensor<type_t> a(2,1,2,3),b(2,1,2,3),c(2,1,2,3);
 a.Fill(3);b.Fill(4);
 CTensorMath<type_t>::Add(c,a,b);             // device result
 bool ok=c.GetElement(1,0,1,2)==7;               // lazy download
 c.SetElement(1,0,1,2,100);                      // host change
 CTensorMath<type_t>::Mul(c,c,static_cast<type_t>(2));  // must upload before computing in place
 ok=ok && c.GetElement(1,0,1,2)==200 && c.GetElement(0,0,0,0)==14;
 CTensor<type_t> d=c;                            // deep copy, device data included
 CTensorMath<type_t>::Fill(c,0);
 ok=ok && d.GetElement(1,0,1,2)==200 && c.GetElement(1,0,1,2)==0;
 c.ReinterpretSize(1,1,4,3);
 ok=ok && c.GetSizeY()==4;
 c.RestoreSize();
 ok=ok && c.GetSizeW()==2 && c.GetSizeY()==2;
 Report("host/device coherence, copies, reinterpretation",ok);

 bool thrown=false;
 try
 {
  CTensor<type_t> wrong(2,1,3,3);
  CTensorMath<type_t>::Add(wrong,a,b);
 }
 catch(const char *message) {thrown=(message!=NULL && strlen(message)>0);}
 Report("shape mismatch throws const char*",thrown);
 thrown=false;
 try {a.GetElement(0,0,5,0);} catch(const char*) {thrown=true;}
 Report("out-of-range element access throws",thrown);

 CTensor<CTensorMath<type_t>::SPos> pos(1,1,2,2);
 CTensor<type_t> in(1,1,4,4),pooled(1,1,2,2),back(1,1,4,4);
 for(uint32_t y=0;y<4;y++) for(uint32_t x=0;x<4;x++) in.SetElement(0,0,y,x,static_cast<type_t>((x*7+y*3)%5));
 CTensorMath<type_t>::MaxPooling(pooled,pos,in,2,2);
 CTensorMath<type_t>::SPos p=pos.GetElement(0,0,1,1);
 ok=pooled.GetElement(0,0,1,1)==in.GetElement(0,0,p.Y,p.X) && p.X>=2 && p.Y>=2;
 CTensorMath<type_t>::MaxPoolingBackward(back,pos,pooled,2,2);
 ok=ok && back.GetElement(0,0,p.Y,p.X)==pooled.GetElement(0,0,1,1);
 Report("MaxPooling positions and backward",ok);
}

// the functions that only the GPU class of the reference declares (cuda/ctensormath.cu.h:92-93, 128-134)
static void GpuClassOnlyChecks(void)
{
 CTensor<type_t> a(2,2,2,2),b(2,1,2,2),cat(2,3,2,2),sa(2,2,2,2),sb(2,1,2,2);
 for(uint32_t n=0;n<16;n++) a.SetElement(n/8,(n/4)%2,(n/2)%2,n%2,static_cast<type_t>(n));
 for(uint32_t n=0;n<8;n++) b.SetElement(n/4,0,(n/2)%2,n%2,static_cast<type_t>(100+n));
 CTensorMath<type_t>::ConcatecationZ(cat,a,b);
 bool ok=cat.GetElement(1,1,1,0)==a.GetElement(1,1,1,0) && cat.GetElement(1,2,0,1)==b.GetElement(1,0,0,1);
 CTensorMath<type_t>::SplitZ(sa,sb,cat);
 ok=ok && sa.Compare(a,"",false) && sb.Compare(b,"",false);
 Report("ConcatecationZ / SplitZ round trip",ok);

 CTensor<uint32_t> step(2,1,1,1);
 step.SetElement(0,0,0,0,0);
 step.SetElement(1,0,0,0,3);
 CTensor<type_t> x(2,1,2,2),y(2,1,2,2);
 x.Fill(1);
 CTensorMath<type_t>::SetTimeStep(y,x,step);
 ok=y.GetElement(0,0,0,0)==1 && y.GetElement(0,0,0,1)==2;          // t=0: +sin 0 at even positions, +cos 0 at odd ones
 ok=ok && fabs(y.GetElement(1,0,0,0)-(1+sin(3.0)))<1e-5;
 Report("SetTimeStep",ok);

 CTensor<type_t> mask(4,4,16,16),noise(4,4,16,16),noisy(4,4,16,16),image(4,4,16,16),alpha(4,1,1,1),beta(4,1,1,1);
 CTensorMath<type_t>::CreateDropOutMatrix(mask,static_cast<type_t>(0.5));
 uint32_t kept=0;
 ok=true;
 for(uint32_t n=0;n<4096;n++)
 {
  type_t v=mask.GetElement(n/1024,(n/256)%4,(n/16)%16,n%16);
  if (v!=0) {kept++;ok=ok && v==2;}
 }
 Report("CreateDropOutMatrix keeps about half, scaled by 1/(1-p)",ok && kept>1850 && kept<2250);
 image.Fill(2);alpha.Fill(static_cast<type_t>(0.5));beta.Fill(static_cast<type_t>(0.25));
 CTensorMath<type_t>::GetNoiseImageAndNoise(noisy,noise,image,alpha,beta);
 double sum=0,sum2=0;
 ok=true;
 for(uint32_t n=0;n<4096;n++)
 {
  type_t e=noise.GetElement(n/1024,(n/256)%4,(n/16)%16,n%16),v=noisy.GetElement(n/1024,(n/256)%4,(n/16)%16,n%16);
  sum+=e;sum2+=e*e;
  ok=ok && fabs(v-(1+0.25*e))<1e-6;
 }
 Report("GetNoiseImageAndNoise: standard normal noise, blended image",ok && fabs(sum/4096)<0.08 && fabs(sum2/4096-1)<0.12);
 CTensorMath<type_t>::SetNormalNoise(noise);
 sum=0;
 for(uint32_t n=0;n<4096;n++) sum+=noise.GetElement(n/1024,(n/256)%4,(n/16)%16,n%16);
 Report("SetNormalNoise",fabs(sum/4096)<0.08);
}

// The weight-gradient sequence of the reference's convolution layer (netlayer/cnetlayerconvolution.cu.h:501-508) at a
// size where the drop-in classes defer the per-sample gradients (mi355::CDeferredGradient), against the same calls
// with the deferral switched off.
static type_t Pattern(uint32_t n,type_t scale) {return(static_cast<type_t>(static_cast<int>((n*2654435761u)>>20)%2001-1000)*scale/1000);}
static void FillPattern(CTensor<type_t> &t,uint32_t seed,type_t scale)
{
 uint32_t n=seed;
 for(uint32_t w=0;w<t.GetSizeW();w++)
  for(uint32_t z=0;z<t.GetSizeZ();z++)
   for(uint32_t y=0;y<t.GetSizeY();y++)
    for(uint32_t x=0;x<t.GetSizeX();x++,n++) t.SetElement(w,z,y,x,Pattern(n,scale));
}
static double MaxDifference(const CTensor<type_t> &a,const CTensor<type_t> &b,double &largest)
{
 double diff=0;
 largest=0;
 for(uint32_t w=0;w<a.GetSizeW();w++)
  for(uint32_t z=0;z<a.GetSizeZ();z++)
   for(uint32_t y=0;y<a.GetSizeY();y++)
    for(uint32_t x=0;x<a.GetSizeX();x++)
    {
     double va=a.GetElement(w,z,y,x),vb=b.GetElement(w,z,y,x);
     if (fabs(va-vb)>diff) diff=fabs(va-vb);
     if (fabs(vb)>largest) largest=fabs(vb);
    }
 return(diff);
}
static void DeferredGradientChecks(void)
{
 const uint32_t batch=8,amount=128,depth=64,size=4;
 CTensor<type_t> image(batch,depth,8,8),delta(batch,amount,4,4);
 FillPattern(image,1,1.0f);
 FillPattern(delta,77,0.5f);
 // [0]: every call runs when it is made; [1]: deferred
 CTensor<type_t> dkernel[2],dbias[2],dkernel_batch[2],dbias_batch[2];
 for(int n=0;n<2;n++)
 {
  mi355::DeferGradients()=(n==1);
  dkernel[n]=CTensor<type_t>(1,1,amount,depth*size*size);
  dbias[n]=CTensor<type_t>(1,amount,1,1);
  dkernel_batch[n]=CTensor<type_t>(batch,1,amount,depth*size*size);
  dbias_batch[n]=CTensor<type_t>(batch,amount,1,1);
  FillPattern(dkernel[n],5,0.25f);   // the sums accumulate onto what the layer holds
  FillPattern(dbias[n],9,0.25f);
  CTensorMath<type_t>::Fill(dkernel_batch[n],0);
  CTensorMath<type_t>::Fill(dbias_batch[n],0);
  CTensorConv<type_t>::CreateDeltaWeightAndBias(dkernel_batch[n],size,size,depth,amount,dbias_batch[n],image,delta,2,2,1,1);
  CTensorMath<type_t>::AddSumW(dkernel[n],dkernel[n],dkernel_batch[n]);
  CTensorMath<type_t>::AddSumW(dbias[n],dbias[n],dbias_batch[n],0.5f,2.0f);
 }
 double largest=0;
 double diff=MaxDifference(dkernel[1],dkernel[0],largest);
 bool ok=diff<=2e-5*largest && largest>1;
 diff=MaxDifference(dbias[1],dbias[0],largest);
 ok=ok && diff<=2e-5*largest && largest>1;
 Report("deferred per-sample gradients: the sums over the batch",ok);
 // the operands change (the next step's forward pass), then somebody reads the per-sample gradients after all
 CTensorMath<type_t>::Fill(image,3);
 CTensorMath<type_t>::Fill(delta,-2);
 CTensor<type_t> copy=dkernel_batch[1];   // a copy is a reader
 diff=MaxDifference(copy,dkernel_batch[0],largest);
 ok=diff<=2e-5*largest && largest>0.1;
 diff=MaxDifference(dkernel_batch[1],dkernel_batch[0],largest);
 ok=ok && diff<=2e-5*largest;
 diff=MaxDifference(dbias_batch[1],dbias_batch[0],largest);
 ok=ok && diff<=2e-5*largest && largest>0.1;
 Report("deferred per-sample gradients: read later, operands changed",ok);
 // a zeroed tensor that nothing was added to is zeros; zeroed and then written by the host, it is what was written
 CTensor<type_t> zero(batch,2,3,3),other(batch,2,3,3);
 FillPattern(zero,3,1.0f);
 CTensorMath<type_t>::Fill(zero,0);
 ok=(zero.GetElement(batch-1,1,2,2)==0 && zero.GetElement(0,0,0,0)==0);
 CTensorMath<type_t>::Fill(zero,0);
 zero.SetElement(1,1,1,1,7);
 ok=ok && zero.GetElement(1,1,1,1)==7 && zero.GetElement(1,1,1,0)==0;
 FillPattern(other,4,1.0f);
 CTensorMath<type_t>::Fill(zero,0);
 CTensorMath<type_t>::Add(zero,zero,other);
 diff=MaxDifference(zero,other,largest);
 ok=ok && diff==0;
 // gradients added onto a tensor that is not zero take the plain path
 FillPattern(dkernel_batch[1],11,0.5f);
 dkernel_batch[0]=dkernel_batch[1];
 CTensorMath<type_t>::Fill(dbias_batch[0],0);
 CTensorMath<type_t>::Fill(dbias_batch[1],0);
 FillPattern(image,1,1.0f);
 FillPattern(delta,77,0.5f);
 mi355::DeferGradients()=false;
 CTensorConv<type_t>::CreateDeltaWeightAndBias(dkernel_batch[0],size,size,depth,amount,dbias_batch[0],image,delta,2,2,1,1);
 mi355::DeferGradients()=true;
 CTensorConv<type_t>::CreateDeltaWeightAndBias(dkernel_batch[1],size,size,depth,amount,dbias_batch[1],image,delta,2,2,1,1);
 diff=MaxDifference(dkernel_batch[1],dkernel_batch[0],largest);
 ok=ok && diff==0 && largest>0.5;
 Report("deferred zero fill: reads, host writes, accumulation onto data",ok);
}

// The call sequences of the reference's batch-norm layer (netlayer/cnetlayerbatchnormalization.cu.h:301-371 forward in
// training and in inference mode, :578-604 backward) and the per-layer Fill / Adam loops, written out as the layer
// writes them, with the deferral of mi355::COpQueue on and off: every tensor a reader could look at afterwards --
// outputs, statistics and the scratch tensors -- must hold the same values, and the counters must show that the
// sequences ran as one kernel each.
struct SBatchNormTensors
{
 CTensor<type_t> X,H,XHat,TmpAH,TmpA,TmpB,TmpC,IVar,Gamma,Beta,Mean,Variable,NewMean,NewVariable,Delta,DXHat,Prev,DGamma,DBeta;
 CTensor<type_t> Error,FunctionDelta,F;///<what a function layer behind the batch norm is handed, its own delta tensor, its output
 SBatchNormTensors(uint32_t w,uint32_t z,uint32_t y,uint32_t x)
  :X(w,z,y,x),H(w,z,y,x),XHat(w,z,y,x),TmpAH(w,z,y,x),TmpA(1,z,y,x),TmpB(1,z,y,x),TmpC(1,z,y,x),IVar(1,z,y,x),Gamma(1,z,y,x),Beta(1,z,y,x),Mean(1,z,y,x),
   Variable(1,z,y,x),NewMean(1,z,y,x),NewVariable(1,z,y,x),Delta(w,z,y,x),DXHat(w,z,y,x),Prev(w,z,y,x),DGamma(1,z,y,x),DBeta(1,z,y,x),Error(w,z,y,x),FunctionDelta(w,z,y,x),F(w,z,y,x)
 {
  FillPattern(X,1,2.0f);FillPattern(Gamma,2,0.5f);FillPattern(Beta,3,0.5f);FillPattern(NewMean,4,0.3f);FillPattern(NewVariable,5,0.3f);
  FillPattern(Error,11,1.0f);
  FillPattern(Delta,6,1.0f);FillPattern(DGamma,7,0.2f);FillPattern(DBeta,8,0.2f);FillPattern(Mean,9,0.3f);FillPattern(Variable,10,0.3f);
  for(uint32_t n=0;n<z*y*x;n++) Gamma.SetElement(0,n/(y*x),(n/x)%y,n%x,Gamma.GetElement(0,n/(y*x),(n/x)%y,n%x)+1.5f);
  for(uint32_t n=0;n<z*y*x;n++) Variable.SetElement(0,n/(y*x),(n/x)%y,n%x,static_cast<type_t>(fabs(Variable.GetElement(0,n/(y*x),(n/x)%y,n%x))+0.2));
 }
 void ForwardTraining(int read_at=-1)///<read_at >= 0: somebody reads a tensor after that many calls
 {
  const type_t N=static_cast<type_t>(X.GetSizeW()),Momentum=0.9f,EPSILON=0.000001f;
  CTensor<type_t> &VAR=TmpB;
  int call=0;
  #define STEP(code) {code;if (call++==read_at) XHat.GetElement(0,0,0,0);}
  STEP(CTensorMath<type_t>::Fill(TmpA,0))
  STEP(CTensorMath<type_t>::AddSumW(TmpA,TmpA,X,1,1.0/N))
  STEP(CTensorMath<type_t>::Add(NewMean,NewMean,TmpA,Momentum,1.0-Momentum))
  STEP(CTensorMath<type_t>::Sub(XHat,X,TmpA,1.0,1.0))
  STEP(CTensorMath<type_t>::Fill(VAR,0))
  STEP(CTensorMath<type_t>::Pow2(TmpAH,XHat,1))
  STEP(CTensorMath<type_t>::AddSumW(VAR,VAR,TmpAH,1,1.0/N))
  STEP(CTensorMath<type_t>::Add(NewVariable,NewVariable,VAR,Momentum,1.0-Momentum))
  STEP(CTensorMath<type_t>::SQRT(TmpC,VAR,1,EPSILON))
  STEP(CTensorMath<type_t>::Inv(IVar,TmpC))
  STEP(CTensorMath<type_t>::TensorItemProduction(XHat,XHat,IVar))
  STEP(CTensorMath<type_t>::TensorItemProduction(TmpAH,Gamma,XHat))
  STEP(CTensorMath<type_t>::Add(H,TmpAH,Beta))
 }
 void ForwardInference(void)
 {
  const type_t EPSILON=0.000001f;
  CTensor<type_t> &VAR=TmpB;
  VAR=Variable;
  CTensorMath<type_t>::Sub(XHat,X,Mean,1.0,1.0);
  CTensorMath<type_t>::SQRT(TmpC,VAR,1,EPSILON);
  CTensorMath<type_t>::Inv(IVar,TmpC);
  CTensorMath<type_t>::TensorItemProduction(XHat,XHat,IVar);
  CTensorMath<type_t>::TensorItemProduction(TmpAH,Gamma,XHat);
  CTensorMath<type_t>::Add(H,TmpAH,Beta);
 }
 // a function layer behind the batch norm: its Forward (netlayer/cnetlayerfunction.cu.h:202-212)
 void Function(bool leaky)
 {
  if (leaky==true) CTensorApplyFunc<type_t>::ApplyLeakyReLU(F,H);
              else CTensorApplyFunc<type_t>::ApplyReLU(F,H);
 }
 // a function layer behind the batch norm: its SetOutputError (netlayer/cnetlayerfunction.cu.h:347-358), the batch-norm
 // layer's (a copy of the tensor, :677-680), then the backward pass
 void FunctionBackward(bool leaky,bool create_delta_weight,int read_at=-1)
 {
  if (leaky==true) CTensorApplyFunc<type_t>::ApplyDifferentialLeakyReLU(FunctionDelta,H);
              else CTensorApplyFunc<type_t>::ApplyDifferentialReLU(FunctionDelta,H);
  if (read_at==100) H.GetElement(0,0,0,0);
  CTensorMath<type_t>::TensorItemProduction(FunctionDelta,Error,FunctionDelta);
  if (read_at==101) FunctionDelta.GetElement(0,0,0,0);
  Delta=FunctionDelta;
  Backward(create_delta_weight,read_at);
 }
 void Backward(bool create_delta_weight,int read_at=-1)
 {
  const type_t N=static_cast<type_t>(X.GetSizeW());
  int call=0;
  STEP(CTensorMath<type_t>::Fill(TmpB,0))
  STEP(CTensorMath<type_t>::Fill(TmpC,0))
  STEP(CTensorMath<type_t>::TensorItemProduction(DXHat,Delta,Gamma))
  STEP(CTensorMath<type_t>::AddSumW(TmpB,TmpB,DXHat))
  STEP(CTensorMath<type_t>::TensorItemProduction(TmpAH,DXHat,XHat))
  STEP(CTensorMath<type_t>::AddSumW(TmpC,TmpC,TmpAH))
  if (create_delta_weight==true)
  {
   STEP(CTensorMath<type_t>::TensorItemProduction(TmpAH,Delta,XHat))
   STEP(CTensorMath<type_t>::AddSumW(DGamma,DGamma,TmpAH))
   STEP(CTensorMath<type_t>::AddSumW(DBeta,DBeta,Delta))
  }
  STEP(CTensorMath<type_t>::Mul(Prev,DXHat,N))
  STEP(CTensorMath<type_t>::TensorItemProduction(TmpAH,XHat,TmpC))
  STEP(CTensorMath<type_t>::Sub(Prev,Prev,TmpAH))
  STEP(CTensorMath<type_t>::Sub(Prev,Prev,TmpB))
  STEP(CTensorMath<type_t>::TensorItemProduction(Prev,Prev,IVar))
  STEP(CTensorMath<type_t>::Mul(Prev,Prev,static_cast<type_t>(1.0/N)))
  #undef STEP
 }
 // every tensor against the same tensor of a run without deferral; differences are measured against the largest value
 bool Agrees(const SBatchNormTensors &eager,double tolerance) const
 {
  const CTensor<type_t> *mine[20]={&H,&XHat,&TmpAH,&TmpA,&TmpB,&TmpC,&IVar,&NewMean,&NewVariable,&DXHat,&Prev,&DGamma,&DBeta,&Gamma,&Beta,&X,&Error,&FunctionDelta,&Delta,&F};
  const CTensor<type_t> *theirs[20]={&eager.H,&eager.XHat,&eager.TmpAH,&eager.TmpA,&eager.TmpB,&eager.TmpC,&eager.IVar,&eager.NewMean,&eager.NewVariable,
                                     &eager.DXHat,&eager.Prev,&eager.DGamma,&eager.DBeta,&eager.Gamma,&eager.Beta,&eager.X,&eager.Error,&eager.FunctionDelta,&eager.Delta,&eager.F};
  bool ok=true;
  for(int n=0;n<20;n++)
  {
   double largest=0;
   const double diff=MaxDifference(*mine[n],*theirs[n],largest);
   if (diff>tolerance*(largest>1e-3?largest:1e-3))
   {
    printf("  tensor %d differs by %g (largest value %g)\n",n,diff,largest);
    ok=false;
   }
  }
  return(ok);
 }
};

// UpSampling by 2 x 2 writes nothing; a 3x3 convolution (stride 1, padding 1) of the tensor is computed from the source,
// every other reader gets the up-sampled values, and the source may change in between.
static void DeferredUpSamplingChecks(void)
{
 CTensor<type_t> source(BATCH,16,5,6),kernel(1,1,8,16*9),bias(1,8,1,1),wide(1,1,8,16*25);
 CTensor<type_t> up(BATCH,16,10,12),up_now(BATCH,16,10,12),out(BATCH,8,10,12),control(BATCH,8,10,12),out5(BATCH,8,10,12),control5(BATCH,8,10,12);
 FillPattern(source,3,1.0f);FillPattern(kernel,5,0.1f);FillPattern(bias,7,0.5f);FillPattern(wide,9,0.05f);
 mi355::DeferGradients()=false;   // the two calls one after the other
 CTensorMath<type_t>::UpSampling(up_now,source,2,2);
 CTensorConv<type_t>::ForwardConvolution(control,up_now,kernel,3,3,16,8,bias,1,1,1,1);
 CTensorConv<type_t>::ForwardConvolution(control5,up_now,wide,5,5,16,8,bias,1,1,2,2);
 mi355::DeferGradients()=true;
 CTensorMath<type_t>::UpSampling(up,source,2,2);
 CTensor<type_t> kept=source;
 CTensorMath<type_t>::Fill(source,7);   // the source changes after the call: the tensor stands for the values it had
 CTensorConv<type_t>::ForwardConvolution(out,up,kernel,3,3,16,8,bias,1,1,1,1);
 double largest=0;
 bool ok=MaxDifference(out,control,largest)<=2e-5*largest && largest>0.1;
 // (coefficient sums: not the same roundings as the two calls, so not the same bits either -- the fused call ran)
 bool fused=false;
 for(uint32_t x=0;x<12 && fused==false;x++) fused=(out.GetElement(1,3,4,x)!=control.GetElement(1,3,4,x));
 Report("3x3 convolution of an up-sampled tensor that was never written",ok && fused);
 // a reader of the tensor itself: the up-sampled values of the source as it was
 ok=up.GetElement(1,3,7,9)==kept.GetElement(1,3,3,4) && up.GetElement(0,15,9,11)==kept.GetElement(0,15,4,5) && up.GetElement(1,0,0,1)==kept.GetElement(1,0,0,0);
 CTensorConv<type_t>::ForwardConvolution(out,up,kernel,3,3,16,8,bias,1,1,1,1);   // written now: the convolution as it always was
 ok=ok && MaxDifference(out,control,largest)==0;
 Report("a reader of the up-sampled tensor gets it written",ok);
 // another geometry writes the tensor first
 CTensorMath<type_t>::UpSampling(up,kept,2,2);
 CTensorConv<type_t>::ForwardConvolution(out5,up,wide,5,5,16,8,bias,1,1,2,2);
 ok=MaxDifference(out5,control5,largest)==0;
 // a copy and a later write to the tensor end the deferral
 CTensorMath<type_t>::UpSampling(up,kept,2,2);
 CTensor<type_t> copy=up;
 ok=ok && MaxDifference(copy,up_now,largest)==0;
 CTensorMath<type_t>::UpSampling(up,kept,2,2);
 CTensorMath<type_t>::Add(up,up_now,up_now,1.0f,1.0f);
 ok=ok && up.GetElement(1,3,7,9)==2*kept.GetElement(1,3,3,4);
 // other factors are written at once
 CTensor<type_t> up3(BATCH,16,15,18);
 CTensorMath<type_t>::UpSampling(up3,kept,3,3);
 ok=ok && up3.GetElement(1,3,11,13)==kept.GetElement(1,3,3,4);
 Report("other kernels, copies, writes and factors",ok);
}

// The linear layer's weight gradient: per-sample outer products, then their sum over the batch (netlayer/cnetlayerlinear.cu.h:
// 436-444).  The products are not computed; their sum is one product over the batch.
static void DeferredProductChecks(void)
{
 const uint32_t batch=8,m=64,n=160;
 CTensor<type_t> delta(batch,1,m,1),input(batch,1,1,n),products(batch,1,m,n),control_products(batch,1,m,n),dw(1,1,m,n),control_dw(1,1,m,n);
 FillPattern(delta,31,1.0f);FillPattern(input,37,1.0f);FillPattern(dw,41,0.5f);
 control_dw=dw;
 mi355::DeferGradients()=false;   // every call when it is made
 CTensorMath<type_t>::Mul(control_products,delta,input);
 CTensorMath<type_t>::AddSumW(control_dw,control_dw,control_products);
 mi355::DeferGradients()=true;
 CTensorMath<type_t>::Mul(products,delta,input);
 CTensor<type_t> kept=delta;
 CTensorMath<type_t>::Fill(delta,3);   // an operand changes after the call: the products are those of the values it had
 CTensorMath<type_t>::AddSumW(dw,dw,products);
 double largest=0;
 bool ok=MaxDifference(dw,control_dw,largest)<=1e-5*largest && largest>1;
 Report("sum over the batch of per-sample outer products that were never computed",ok);
 ok=MaxDifference(products,control_products,largest)==0;   // a reader: the products themselves, bit for bit
 // other shapes and small products run at once; a scaled sum takes the products
 CTensor<type_t> small(batch,1,4,8),column(batch,1,4,1),row(batch,1,1,8),sum(1,1,4,8),control_sum(1,1,4,8);
 FillPattern(column,43,1.0f);FillPattern(row,47,1.0f);
 CTensorMath<type_t>::Mul(small,column,row);
 CTensorMath<type_t>::Fill(sum,0);
 CTensorMath<type_t>::AddSumW(sum,sum,small);
 for(uint32_t y=0;y<4;y++)
  for(uint32_t x=0;x<8;x++)
  {
   double expected=0;
   for(uint32_t w=0;w<batch;w++) expected+=static_cast<double>(column.GetElement(w,0,y,0))*row.GetElement(w,0,0,x);
   ok=ok && fabs(sum.GetElement(0,0,y,x)-expected)<=1e-5*(1+fabs(expected));
  }
 CTensorMath<type_t>::Mul(products,kept,input);
 CTensorMath<type_t>::AddSumW(dw,control_dw,products,0.5f,2.0f);   // not the layer's call: out = 0.5 control_dw + 2 sum
 CTensorMath<type_t>::AddSumW(control_dw,control_dw,control_products,0.5f,2.0f);
 ok=ok && MaxDifference(dw,control_dw,largest)<=1e-5*largest;
 Report("readers of the products, small products, scaled sums",ok);
}

static void FusedSequenceChecks(void)
{
 mi355::COpQueue &queue=mi355::Queue();
 const uint32_t shapes[3][4]={{16,3,6,8},{5,2,3,3},{64,8,16,16}};
 for(int s=0;s<3;s++)
 {
  const uint32_t *d=shapes[s];
  char name[128];
  // training: forward, backward with and without the parameter gradients, a second forward (the layer's next step)
  mi355::FuseSequences()=false;
  SBatchNormTensors eager(d[0],d[1],d[2],d[3]);
  eager.ForwardTraining();eager.Backward(true);eager.Backward(false);eager.ForwardTraining();eager.Backward(true);
  mi355::FuseSequences()=true;
  SBatchNormTensors fused(d[0],d[1],d[2],d[3]);
  const size_t forward=queue.ForwardFused,backward=queue.BackwardFused,literal=queue.LiteralCalls;
  fused.ForwardTraining();fused.Backward(true);fused.Backward(false);fused.ForwardTraining();fused.Backward(true);
  bool ok=queue.ForwardFused==forward+2 && queue.BackwardFused==backward+3 && queue.LiteralCalls==literal;
  ok=fused.Agrees(eager,2e-5) && ok;   // (the statistics of the one-pass kernel against sums over the batch: fp32 rounding)
  snprintf(name,sizeof(name),"batch-norm sequences as one kernel each, batch %u x %ux%ux%u",d[0],d[1],d[2],d[3]);
  Report(name,ok);
  // a reader in the middle of a sequence gets what the calls so far have left; the rest then runs as written
  bool all=true;
  for(int read_at=0;read_at<13;read_at+=3)
  {
   mi355::FuseSequences()=false;
   SBatchNormTensors a(d[0],d[1],d[2],d[3]);
   a.ForwardTraining(read_at);a.Backward(true,read_at);
   mi355::FuseSequences()=true;
   SBatchNormTensors b(d[0],d[1],d[2],d[3]);
   b.ForwardTraining(read_at);b.Backward(true,read_at);
   all=b.Agrees(a,2e-5) && all;
  }
  snprintf(name,sizeof(name),"a sequence interrupted by a reader, batch %u",d[0]);
  Report(name,all);
  // a function layer behind the batch norm: its two calls and the backward pass as one kernel while the forward pass is
  // on record; as two calls and one kernel after somebody has written gamma; as written when a reader comes between
  mi355::FuseSequences()=false;
  SBatchNormTensors ef(d[0],d[1],d[2],d[3]);
  ef.ForwardTraining();ef.FunctionBackward(true,true);ef.ForwardTraining();ef.FunctionBackward(false,false);
  mi355::FuseSequences()=true;
  SBatchNormTensors ff(d[0],d[1],d[2],d[3]);
  const size_t function=queue.FunctionBackwardFused,plain=queue.BackwardFused,calls=queue.LiteralCalls;
  ff.ForwardTraining();ff.FunctionBackward(true,true);ff.ForwardTraining();ff.FunctionBackward(false,false);
  ok=queue.FunctionBackwardFused==function+2 && queue.BackwardFused==plain && queue.LiteralCalls==calls;
  ok=ff.Agrees(ef,2e-5) && ok;
  mi355::FuseSequences()=false;
  SBatchNormTensors eg(d[0],d[1],d[2],d[3]);
  eg.ForwardTraining();CTensorMath<type_t>::Mul(eg.Gamma,eg.Gamma,static_cast<type_t>(1));eg.FunctionBackward(true,true);
  mi355::FuseSequences()=true;
  SBatchNormTensors fg(d[0],d[1],d[2],d[3]);
  const size_t function2=queue.FunctionBackwardFused,plain2=queue.BackwardFused;
  fg.ForwardTraining();CTensorMath<type_t>::Mul(fg.Gamma,fg.Gamma,static_cast<type_t>(1));fg.FunctionBackward(true,true);
  ok=queue.FunctionBackwardFused==function2 && queue.BackwardFused==plain2+1 && ok;
  ok=fg.Agrees(eg,2e-5) && ok;
  for(int read_at=100;read_at<=101;read_at++)
  {
   mi355::FuseSequences()=false;
   SBatchNormTensors a(d[0],d[1],d[2],d[3]);
   a.ForwardTraining();a.FunctionBackward(true,true,read_at);
   mi355::FuseSequences()=true;
   SBatchNormTensors b(d[0],d[1],d[2],d[3]);
   b.ForwardTraining();b.FunctionBackward(true,true,read_at);
   ok=b.Agrees(a,2e-5) && ok;
  }
  for(int read_at=1;read_at<15;read_at+=4)
  {
   mi355::FuseSequences()=false;
   SBatchNormTensors a(d[0],d[1],d[2],d[3]);
   a.ForwardTraining();a.FunctionBackward(false,true,read_at);
   mi355::FuseSequences()=true;
   SBatchNormTensors b(d[0],d[1],d[2],d[3]);
   b.ForwardTraining();b.FunctionBackward(false,true,read_at);
   ok=b.Agrees(a,2e-5) && ok;
  }
  snprintf(name,sizeof(name),"function layer and batch-norm layer backward as one kernel, batch %u",d[0]);
  Report(name,ok);
  // the function layer's Forward behind the batch-norm layer's: one kernel leaves both outputs (training mode), or the
  // function layer's with the batch-norm layer's own pending (inference mode); a whole training step through both layers
  mi355::FuseSequences()=false;
  SBatchNormTensors eh(d[0],d[1],d[2],d[3]);
  eh.ForwardTraining();eh.Function(true);eh.FunctionBackward(true,true);eh.ForwardInference();eh.Function(false);eh.ForwardInference();eh.Function(false);
  mi355::FuseSequences()=true;
  SBatchNormTensors fh(d[0],d[1],d[2],d[3]);
  const size_t forward2=queue.ForwardFused,inference2=queue.InferenceFused,function3=queue.FunctionBackwardFused,calls2=queue.LiteralCalls;
  fh.ForwardTraining();fh.Function(true);fh.FunctionBackward(true,true);fh.ForwardInference();fh.Function(false);fh.ForwardInference();fh.Function(false);
  queue.Flush();
  ok=queue.ForwardFused==forward2+1 && queue.InferenceFused==inference2+2 && queue.FunctionBackwardFused==function3+1 && queue.LiteralCalls==calls2;
  ok=fh.Agrees(eh,2e-5) && ok;
  // ... and when a reader looks at the batch-norm layer's output between the two layers
  mi355::FuseSequences()=false;
  SBatchNormTensors ej(d[0],d[1],d[2],d[3]);
  ej.ForwardTraining();ej.H.GetElement(0,0,0,0);ej.Function(false);ej.ForwardInference();ej.H.GetElement(0,0,0,0);ej.Function(true);
  mi355::FuseSequences()=true;
  SBatchNormTensors fj(d[0],d[1],d[2],d[3]);
  fj.ForwardTraining();fj.H.GetElement(0,0,0,0);fj.Function(false);fj.ForwardInference();fj.H.GetElement(0,0,0,0);fj.Function(true);
  ok=fj.Agrees(ej,2e-5) && ok;
  snprintf(name,sizeof(name),"function layer forward behind the batch-norm layer's as one kernel, batch %u",d[0]);
  Report(name,ok);
  // Forward passes on their own: the batch-norm layer's own output is not written (pending, then dropped by the next
  // pass); a reader gets it from its two calls, and from then on the kernel writes it.
  {
   mi355::FuseSequences()=false;
   SBatchNormTensors ek(d[0],d[1],d[2],d[3]);
   ek.ForwardTraining();ek.Function(true);
   mi355::FuseSequences()=true;
   SBatchNormTensors fk(d[0],d[1],d[2],d[3]);
   const size_t kept=queue.OwnOutputsPending,ran=queue.PendingRun;
   for(int pass=0;pass<3;pass++) {fk.ForwardTraining();fk.Function(true);}
   queue.Flush();
   ok=queue.OwnOutputsPending==kept+3 && queue.PendingRun==ran;
   double largest=0;
   ok=ok && MaxDifference(fk.F,ek.F,largest)<=2e-5*largest;
   ok=ok && MaxDifference(fk.H,ek.H,largest)<=2e-5*largest && queue.PendingRun>ran;   // the reader: the two calls run now
   const size_t kept2=queue.OwnOutputsPending;
   fk.ForwardTraining();fk.Function(true);
   queue.Flush();
   ok=ok && queue.OwnOutputsPending==kept2 && MaxDifference(fk.H,ek.H,largest)<=2e-5*largest && MaxDifference(fk.F,ek.F,largest)<=2e-5*largest;
   // the optimiser's write to Gamma reaches a pending output before the new values do
   SBatchNormTensors fl(d[0],d[1],d[2],d[3]);
   fl.ForwardTraining();fl.Function(true);
   queue.Flush();
   CTensorMath<type_t>::Mul(fl.Gamma,fl.Gamma,static_cast<type_t>(3));
   ok=ok && MaxDifference(fl.H,ek.H,largest)<=2e-5*largest;
   snprintf(name,sizeof(name),"the batch-norm layer's own output behind a fused forward pass, batch %u",d[0]);
   Report(name,ok);
  }
  // inference mode, twice (the scratch tensors of the first pass are overwritten unread by the second)
  mi355::FuseSequences()=false;
  SBatchNormTensors ei(d[0],d[1],d[2],d[3]);
  ei.ForwardInference();ei.ForwardInference();
  mi355::FuseSequences()=true;
  SBatchNormTensors fi(d[0],d[1],d[2],d[3]);
  const size_t inference=queue.InferenceFused,dropped=queue.PendingDropped;
  fi.ForwardInference();fi.ForwardInference();
  queue.Flush();   // (a whole forward sequence waits for the function layer's call that may follow)
  ok=queue.InferenceFused==inference+2 && queue.PendingDropped>dropped;
  ok=fi.Agrees(ei,2e-5) && ok;
  snprintf(name,sizeof(name),"batch-norm inference sequence as one kernel, batch %u",d[0]);
  Report(name,ok);
 }
 // the per-layer loops: gradients cleared and Adam run tensor by tensor collect into one launch each, whatever the
 // layers do to other tensors in between; a reader of one of the tensors gets the call-by-call result
 const int count=6;
 CTensor<type_t> w[2][count],dw[2][count],m[2][count],v[2][count],unrelated(4,4,4,4),copy(4,4,4,4);
 FillPattern(unrelated,1,1.0f);
 size_t runs[2]={0,0};
 for(int mode=0;mode<2;mode++)
 {
  mi355::FuseSequences()=(mode==1);
  for(int n=0;n<count;n++)
  {
   w[mode][n]=CTensor<type_t>(1,1,8+n,16);dw[mode][n]=w[mode][n];m[mode][n]=w[mode][n];v[mode][n]=w[mode][n];
   FillPattern(w[mode][n],10+n,1.0f);FillPattern(dw[mode][n],20+n,1.0f);
  }
  const size_t fill_runs=queue.FillRuns,adam_runs=queue.AdamRuns;
  for(int n=0;n<count;n++)
  {
   CTensorMath<type_t>::Fill(m[mode][n],0);
   CTensorMath<type_t>::Fill(v[mode][n],0);
   copy=unrelated;   // what a layer does between its calls (the batch-norm layer copies its running statistics)
  }
  for(int step=1;step<=2;step++)
   for(int n=0;n<count;n++)
   {
    CTensorMath<type_t>::Adam(w[mode][n],dw[mode][n],m[mode][n],v[mode][n],8,0.01,0.9,0.999,1e-8,step);
    copy=unrelated;
   }
  queue.Flush();
  runs[mode]=(queue.FillRuns-fill_runs)+(queue.AdamRuns-adam_runs);
 }
 bool ok=(runs[0]==0);
 double largest=0;
 for(int n=0;n<count;n++) ok=ok && MaxDifference(w[1][n],w[0][n],largest)==0 && MaxDifference(m[1][n],m[0][n],largest)==0 && MaxDifference(v[1][n],v[0][n],largest)==0;
 ok=ok && runs[1]==3 && copy.GetElement(3,3,3,3)==unrelated.GetElement(3,3,3,3);   // one Fill launch, one Adam launch per step
 Report("Fill and Adam loops over the layers' tensors as one launch each",ok);
 mi355::FuseSequences()=true;
}

// Copies share their device block until one side is written (mi355::CDeviceBuffer): every way of writing one side must
// leave the other as it was.
static void SharedBlockChecks(void)
{
 CTensor<type_t> a(4,2,8,8),b(4,2,8,8),ones(4,2,8,8),bias(1,2,1,1);
 FillPattern(a,1,1.0f);
 CTensorMath<type_t>::Fill(ones,1);
 bias.SetElement(0,0,0,0,10);bias.SetElement(0,1,0,0,20);
 CTensorMath<type_t>::Add(a,a,ones,1,0);        // a lives on the device now
 CTensor<type_t> original=a;
 original.GetElement(0,0,0,0);                   // ... and `original` on the host as well: a reference that no later write can reach
 double largest=0;
 bool ok=true;
 // overwritten as a whole
 b=a;
 CTensorMath<type_t>::Fill(a,5);
 ok=ok && MaxDifference(b,original,largest)==0 && a.GetElement(3,1,7,7)==5;
 // written in place by a deferred call, and by a call that is not deferred
 a=b;
 CTensorMath<type_t>::Add(a,a,ones,1,1);
 ok=ok && MaxDifference(b,original,largest)==0 && a.GetElement(0,0,0,1)==original.GetElement(0,0,0,1)+1;
 a=b;
 CTensorMath<type_t>::AddBias(a,bias);
 ok=ok && MaxDifference(b,original,largest)==0 && a.GetElement(2,1,3,3)==original.GetElement(2,1,3,3)+20;
 // the copy is written, the source stays
 a=b;
 CTensorMath<type_t>::Mul(b,b,static_cast<type_t>(2));
 ok=ok && MaxDifference(a,original,largest)==0 && b.GetElement(1,0,2,2)==2*original.GetElement(1,0,2,2);
 // written from the host, partly and as a whole
 b=a;
 type_t row[8]={9,9,9,9,9,9,9,9};
 b.CopyItemToDevice(row,8);
 ok=ok && MaxDifference(a,original,largest)==0 && b.GetElement(0,0,0,7)==9 && b.GetElement(0,0,1,0)==original.GetElement(0,0,1,0);
 b=a;
 b.SetElement(0,0,0,0,-3);
 CTensorMath<type_t>::Add(b,b,ones,1,0);
 ok=ok && MaxDifference(a,original,largest)==0 && b.GetElement(0,0,0,0)==-3 && b.GetElement(3,1,7,7)==original.GetElement(3,1,7,7);
 // a chain of copies, the middle one updated by Adam (reads and writes weights and both moments)
 CTensor<type_t> w1=original,w2,w3,m(4,2,8,8),v(4,2,8,8);
 w2=w1;w3=w2;
 CTensor<type_t> m_copy=m;
 CTensorMath<type_t>::Fill(m,0);CTensorMath<type_t>::Fill(v,0);
 CTensorMath<type_t>::Adam(w2,ones,m,v,4,0.01,0.9,0.999,1e-8,1);
 ok=ok && MaxDifference(w1,original,largest)==0 && MaxDifference(w3,original,largest)==0 && MaxDifference(w2,original,largest)>0;
 Report("copies share a device block until one side is written",ok);
}

// the scope timer the reference's models wrap around their training phases (cuda/ctimestamp.cu.h)
static void TimerCheck(void)
{
 CTensor<type_t> a(8,4,64,64),b(8,4,64,64),c(8,4,64,64);
 a.Fill(1);b.Fill(2);
 CCUDATimeSpent spent;
 spent.Start();
 for(int n=0;n<20;n++) CTensorMath<type_t>::Add(c,a,b);
 float ms=spent.Stop();
 {
  CTimeStamp stamp("Add x20: ",true);   // prints through SYSTEM::PutMessageToConsole when it goes out of scope
  for(int n=0;n<20;n++) CTensorMath<type_t>::Add(c,a,b);
 }
 Report("CCUDATimeSpent / CTimeStamp measure queued work",ms>0 && ms<1000 && c.GetElement(7,3,63,63)==3);
}

int main(void)
{
 try
 {
  mi355::Check(mt_init(0));
  MatrixChecks();
  ForwardConvolutionCheck();
  DeltaWeightChecks();
  BackwardConvolutionCheck();
  ZeroBiasCheck();
  DeferredGradientChecks();
  DeferredUpSamplingChecks();
  DeferredProductChecks();
  FusedSequenceChecks();
  SharedBlockChecks();
  SummXYCheck();
  CoherenceAndErrors();
  GpuClassOnlyChecks();
  TimerCheck();
 }
 catch(const char *message)
 {
  printf("exception: %s\n",message);
  return(2);
 }
 printf("%s\n",failures==0?"ALL PASS":"SOME FAILED");
 return(failures==0?0:1);
}
