// TEST INFRASTRUCTURE ONLY.
//
// Runs the reference's OWN layer classes (netlayer/cnetlayer*.cu.h, compiled from /root/reference where they lie)
// on seeded inputs and writes every layer output, back-propagated error and updated weight to a file.
// The same source is built twice by oracle/Makefile, only where /root/reference exists, into oracle/_ref/:
//   layers_cpu    -DUSE_CPU: the layers on the reference's CPU tensor classes (cpu/tensor.h)
//   layers_mi355  the layers on the drop-in tensor classes (cuda-cnn-gan-vae_amd/dropin) -> libmi355tensor.so
// A GPU test runs both and compares the files: the unchanged layers produce the same numbers on the HIP path.
// Weights enter through Load() from an in-memory stream (Reset() uses an unseeded RNG, and Load() is the only way
// to give the transposed-convolution layer a correctly shaped kernel).
//
// Chain A: input [B,3,16,16] -> Convolution 8 x 4x4 s2 p1 -> LeakyReLU -> Linear 24 -> Sigmoid
// Chain B: input [B,8,4,4]   -> BackConvolution 4x4 s2 p1 to 3 channels -> Tangence
// Chain C: input [B,4,5,5]   -> BatchNormalization (training) -> ReLU            (layers_mi355 only: the reference's
//          batch-norm layer does not compile on its own CPU classes, netlayer/cnetlayerbatchnormalization.cu.h:655)
// Chain D: input [B,4,4,4]   -> UpSampling 2x2 -> AveragePooling 4x4, forward and backward
// Chain U: input [B,16,6,8]  -> UpSampling 2x2 -> Convolution 8 x 3x3 s1 p1 -> LeakyReLU, two training steps (a layer pair of the
//          reference's GAN generator, cuda/netmodel/cmodel_gan.cu.h:153-170: the drop-in classes compute the convolution from
//          the input of the up-sampling layer and write the up-sampled image only for the weight gradient)
// Chain E: inputs [B,2,4,4] and [B,3,4,4] -> Concatenator -> TimeEmbedding       (layers_mi355 only: ConcatecationZ and
//          SetTimeStep exist in the reference's GPU tensor class only)
// Chain F: input [B,4,8,8]   -> Linear function -> MaxPooling 2x2, forward and backward           (layers_mi355 only: the layer names the
//          position type CTensorMath<type_t>::SPos, which the CPU class does not nest)
// Chain H: the layers that work element by element on the host through GetElement/SetElement: SoftMax; Splitter with two
//          consumers; DropOut and VAECoderOutput (both draw from std::random_device: the test recovers mask and noise
//          from the outputs and checks the rest against them); MaxDePooling
// "deferred" as the second argument (layers_mi355 only): chain K, two training steps of the DCGAN-64 discriminator at batch
//          16 with and without the drop-in classes' deferral of the per-sample weight gradients
// "time" as the second argument (layers_mi355 only): the DCGAN-64 generator's forward pass at batch 256, the
//          discriminator's training step at batch 128 and the forward pass of the reference's own GAN generator (192x256
//          images, batch 32) on the reference's layer classes, timed with the drop-in CTimeStamp; a fifth argument "literal"
//          repeats the last chain with every call run when it is made, "train" adds that generator's whole training step
// Each chain: TrainingStart, Forward, SetOutputError, TrainingBackward, TrainingUpdateWeight (gradient descent), Save.
// SYSTEM::PutMessage* come from the reference's own system/system.cpp, compiled beside this file.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <memory>
#include <string>
#include <vector>

#ifdef USE_CPU
#include "common/idatastream.h"
#include "system/system.h"
#include "cuda/tensor.cu.h"   // with USE_CPU this is the reference's cpu/tensor.h
#else
#include "cuda/tensor.cu.h"   // the drop-in, found first on the include path
#include "cuda/ctimestamp.cu.h"
#endif

#include "netlayer/cnetlayerconvolutioninput.cu.h"
#include "netlayer/cnetlayerconvolution.cu.h"
#include "netlayer/cnetlayerbackconvolution.cu.h"
#include "netlayer/cnetlayerlinear.cu.h"
#include "netlayer/cnetlayerfunction.cu.h"
#include "netlayer/cnetlayerupsampling.cu.h"
#include "netlayer/cnetlayeraveragepooling.cu.h"
#ifndef USE_CPU
#include "netlayer/cnetlayerbatchnormalization.cu.h"
#include "netlayer/cnetlayerconcatenator.cu.h"
#include "netlayer/cnetlayertimeembedding.cu.h"
#include "netlayer/cnetlayermaxpooling.cu.h"
#endif
#include "netlayer/cnetlayermaxdepooling.cu.h"
#include "netlayer/cnetlayerdropout.cu.h"
#include "netlayer/cnetlayersplitter.cu.h"
#include "netlayer/cnetlayervaecoderoutput.cu.h"
#include "netlayer/cnetlayersoftmax.cu.h"
// every member function of each, also those no chain calls
template class CNetLayerMaxDePooling<float>;
template class CNetLayerDropOut<float>;
template class CNetLayerSplitter<float>;
template class CNetLayerVAECoderOutput<float>;
template class CNetLayerSoftMax<float>;

// the reference's IDataStream declares a file factory that nothing here calls
#ifdef USE_CPU
IDataStream* IDataStream::CreateNewDataStreamFile(std::string,bool) {return(NULL);}
#endif

typedef float type_t;

// bytes in memory, typed access in host byte order like the reference's file stream
class CMemoryStream:public IDataStream
{
  std::vector<uint8_t> Data;
  size_t Pos;
  template<class T> T Get(void) {T v;memcpy(&v,&Data[Pos],sizeof(T));Pos+=sizeof(T);return(v);}
  template<class T> void Put(T v) {const uint8_t *p=reinterpret_cast<const uint8_t*>(&v);Data.insert(Data.end(),p,p+sizeof(T));}
 public:
  CMemoryStream(void):Pos(0) {}
  void Rewind(void) {Pos=0;}
  const std::vector<uint8_t>& Bytes(void) const {return(Data);}
  bool ReadFile(const char *name)
  {
   FILE *file=fopen(name,"rb");
   if (file==NULL) return(false);
   uint8_t buffer[4096];
   size_t n;
   while((n=fread(buffer,1,sizeof(buffer),file))>0) Data.insert(Data.end(),buffer,buffer+n);
   fclose(file);
   Pos=0;
   return(true);
  }
  int8_t LoadInt8(void) {return(Get<int8_t>());}
  int16_t LoadInt16(void) {return(Get<int16_t>());}
  int32_t LoadInt32(void) {return(Get<int32_t>());}
  uint8_t LoadUInt8(void) {return(Get<uint8_t>());}
  uint16_t LoadUInt16(void) {return(Get<uint16_t>());}
  uint32_t LoadUInt32(void) {return(Get<uint32_t>());}
  float LoadFloat(void) {return(Get<float>());}
  double LoadDouble(void) {return(Get<double>());}
  void SaveFloat(float value) {Put(value);}
  void SaveDouble(double value) {Put(value);}
  void SaveInt8(int8_t value) {Put(value);}
  void SaveInt16(int16_t value) {Put(value);}
  void SaveInt32(int32_t value) {Put(value);}
  void SaveUInt8(int8_t value) {Put(value);}
  void SaveUInt16(int16_t value) {Put(value);}
  void SaveUInt32(int32_t value) {Put(value);}
  bool IsFail(void) const {return(false);}
  // a tensor as CTensor::Save writes it: four sizes, then doubles
  void PutTensor(uint32_t w,uint32_t z,uint32_t y,uint32_t x,const std::vector<double> &v)
  {
   Put<uint32_t>(w);Put<uint32_t>(z);Put<uint32_t>(y);Put<uint32_t>(x);
   for(size_t n=0;n<v.size();n++) Put<double>(v[n]);
  }
};

// small deterministic generator (the same stream of numbers in both builds)
static uint64_t rng_state=0x9E3779B97F4A7C15ull;
static double Uniform(void)
{
 rng_state=rng_state*6364136223846793005ull+1442695040888963407ull;
 return(static_cast<double>((rng_state>>11)&0xFFFFFFFFFFFFFull)/4503599627370496.0*2.0-1.0);
}
static std::vector<double> Values(size_t n,double scale)
{
 std::vector<double> v(n);
 for(size_t i=0;i<n;i++) v[i]=static_cast<double>(static_cast<float>(Uniform()*scale));  // exactly representable in fp32
 return(v);
}
static void FillTensor(CTensor<type_t> &t,double scale)
{
 for(uint32_t w=0;w<t.GetSizeW();w++)
  for(uint32_t z=0;z<t.GetSizeZ();z++)
   for(uint32_t y=0;y<t.GetSizeY();y++)
    for(uint32_t x=0;x<t.GetSizeX();x++) t.SetElement(w,z,y,x,static_cast<type_t>(Uniform()*scale));
}

static FILE *out_file=NULL;
static void Dump(const char *name,const CTensor<type_t> &t)
{
 char label[32];
 memset(label,0,sizeof(label));
 strncpy(label,name,sizeof(label)-1);
 uint32_t dims[4]={t.GetSizeW(),t.GetSizeZ(),t.GetSizeY(),t.GetSizeX()};
 fwrite(label,1,sizeof(label),out_file);
 fwrite(dims,sizeof(uint32_t),4,out_file);
 for(uint32_t w=0;w<dims[0];w++)
  for(uint32_t z=0;z<dims[1];z++)
   for(uint32_t y=0;y<dims[2];y++)
    for(uint32_t x=0;x<dims[3];x++)
    {
     float v=t.GetElement(w,z,y,x);
     fwrite(&v,sizeof(float),1,out_file);
    }
}
// the saved form of a layer (what Save() wrote), as one row of doubles converted to float
static void DumpStream(const char *name,CMemoryStream &stream,size_t skip_bytes,uint32_t tensors)
{
 stream.Rewind();
 for(size_t n=0;n<skip_bytes;n++) stream.LoadUInt8();
 for(uint32_t i=0;i<tensors;i++)
 {
  uint32_t w=stream.LoadUInt32(),z=stream.LoadUInt32(),y=stream.LoadUInt32(),x=stream.LoadUInt32();
  CTensor<type_t> t(w,z,y,x);
  for(uint32_t a=0;a<w;a++) for(uint32_t b=0;b<z;b++) for(uint32_t c=0;c<y;c++) for(uint32_t d=0;d<x;d++) t.SetElement(a,b,c,d,static_cast<type_t>(stream.LoadDouble()));
  char label[32];
  snprintf(label,sizeof(label),"%s.%u",name,i);
  Dump(label,t);
 }
}

// the bytes of a stream as they would be in a checkpoint file, four per dump slot (the reader takes the bit patterns)
static void DumpRaw(const char *name,CMemoryStream &stream)
{
 const std::vector<uint8_t> &bytes=stream.Bytes();
 char label[32];
 memset(label,0,sizeof(label));
 strncpy(label,name,sizeof(label)-1);
 uint32_t dims[4]={1,1,1,static_cast<uint32_t>(bytes.size()/4)};
 fwrite(label,1,sizeof(label),out_file);
 fwrite(dims,sizeof(uint32_t),4,out_file);
 fwrite(&bytes[0],1,dims[3]*4,out_file);
}

static const uint32_t BATCH=6;

static void ChainA(void)
{
 CNetLayerConvolutionInput<type_t> input(3,16,16,BATCH);
 CNetLayerConvolution<type_t> conv(8,4,2,2,1,1,&input,BATCH);
 CNetLayerFunction<type_t> f1(NNeuron::NEURON_FUNCTION_LEAKY_RELU,&conv,BATCH);
 CNetLayerLinear<type_t> lin(24,&f1,BATCH);
 CNetLayerFunction<type_t> f2(NNeuron::NEURON_FUNCTION_SIGMOID,&lin,BATCH);

 CMemoryStream conv_w;
 conv_w.SaveUInt32(8);conv_w.SaveInt32(4);conv_w.SaveInt32(4);conv_w.SaveInt32(3);conv_w.SaveInt32(2);conv_w.SaveInt32(2);conv_w.SaveInt32(1);conv_w.SaveInt32(1);
 conv_w.PutTensor(1,1,8,3*16,Values(8*48,0.2));
 conv_w.PutTensor(1,8,1,1,Values(8,0.1));
 conv.Load(&conv_w);
 CMemoryStream lin_w;
 lin_w.PutTensor(1,1,24,8*8*8,Values(24*512,0.08));
 lin_w.PutTensor(1,1,24,1,Values(24,0.1));
 lin.Load(&lin_w);

 CTensor<type_t> image(BATCH,3,16,16);
 FillTensor(image,1.0);
 input.SetOutput(image);
 INetLayer<type_t> *layers[5]={&input,&conv,&f1,&lin,&f2};
 DumpStream("A.conv_loaded",conv_w,8*sizeof(int32_t),2);
 DumpStream("A.linear_loaded",lin_w,0,2);
 CMemoryStream ema_off;   // averaged weights of a network that never enabled them
 for(int n=0;n<5;n++) layers[n]->SaveEMAWeight(&ema_off);
 DumpRaw("A.ema_off_stream",ema_off);
 for(int n=0;n<5;n++) layers[n]->EnableEMA(true);   // the averages start as copies of the loaded weights
 for(int n=0;n<5;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
 for(int n=0;n<5;n++) layers[n]->Forward();
 Dump("A.conv",conv.GetOutputTensor());
 Dump("A.leaky",f1.GetOutputTensor());
 Dump("A.linear",lin.GetOutputTensor());
 Dump("A.sigmoid",f2.GetOutputTensor());

 CTensor<type_t> error(BATCH,1,24,1);
 FillTensor(error,0.5);
 f2.SetOutputError(error);
 for(int n=4;n>=1;n--) layers[n]->TrainingBackward(true);
 Dump("A.delta_linear",lin.GetDeltaTensor());
 Dump("A.delta_leaky",f1.GetDeltaTensor());
 Dump("A.delta_conv",conv.GetDeltaTensor());
 for(int n=1;n<5;n++) layers[n]->TrainingUpdateWeight(0.05,1);
 CMemoryStream conv_saved,lin_saved;
 conv.Save(&conv_saved);
 lin.Save(&lin_saved);
 DumpStream("A.conv_updated",conv_saved,8*sizeof(int32_t),2);
 DumpStream("A.linear_updated",lin_saved,0,2);
 DumpRaw("A.conv_stream",conv_saved);
 DumpRaw("A.linear_stream",lin_saved);
 CMemoryStream net_saved;   // the whole chain, layer after layer, as CModelMain::SaveNetLayers writes a network
 for(int n=0;n<5;n++) layers[n]->Save(&net_saved);
 DumpRaw("A.net_stream",net_saved);
 CMemoryStream ema_saved;   // the averaged weights after one update, layer after layer, as CModelMain::SaveNetLayersEMAWeight writes them
 for(int n=0;n<5;n++) layers[n]->SaveEMAWeight(&ema_saved);
 DumpRaw("A.ema_stream",ema_saved);
 {
  CMemoryStream conv_ema,lin_ema;
  conv.SaveEMAWeight(&conv_ema);
  lin.SaveEMAWeight(&lin_ema);
  DumpStream("A.conv_ema",conv_ema,8*sizeof(int32_t),2);
  DumpStream("A.linear_ema",lin_ema,0,2);
 }
 // forward with the averaged weights
 for(int n=0;n<5;n++) layers[n]->SetUseEMA(true);
 for(int n=0;n<5;n++) layers[n]->Forward();
 Dump("A.sigmoid_ema",f2.GetOutputTensor());
 for(int n=0;n<5;n++) layers[n]->SetUseEMA(false);
 // known Adam moments into the convolution layer (this chain steps by plain gradient descent, its own moments are zero)
 CMemoryStream moments;
 const std::vector<double> mk=Values(8*48,0.3),vk=Values(8*48,0.2),mb=Values(8,0.3),vb=Values(8,0.2);
 moments.PutTensor(1,1,8,3*16,mk);moments.PutTensor(1,1,8,3*16,vk);moments.PutTensor(1,8,1,1,mb);moments.PutTensor(1,8,1,1,vb);
 conv.LoadTrainingParam(&moments);
 {
  CTensor<type_t> t(1,1,8,48),u(1,8,1,1);
  for(uint32_t n=0;n<8*48;n++) t.SetElement(0,0,n/48,n%48,static_cast<type_t>(mk[n]));
  Dump("A.mk",t);
  for(uint32_t n=0;n<8*48;n++) t.SetElement(0,0,n/48,n%48,static_cast<type_t>(vk[n]));
  Dump("A.vk",t);
  for(uint32_t n=0;n<8;n++) u.SetElement(0,n,0,0,static_cast<type_t>(mb[n]));
  Dump("A.mb",u);
  for(uint32_t n=0;n<8;n++) u.SetElement(0,n,0,0,static_cast<type_t>(vb[n]));
  Dump("A.vb",u);
 }
 CMemoryStream train_saved;   // the training state as CModelMain::SaveNetLayersTrainingParam writes it: iteration, then every layer
 train_saved.SaveUInt32(7);
 for(int n=0;n<5;n++) layers[n]->SaveTrainingParam(&train_saved);
 DumpRaw("A.train_stream",train_saved);
}

static void ChainB(void)
{
 CNetLayerConvolutionInput<type_t> input(8,4,4,BATCH);
 CNetLayerBackConvolution<type_t> tconv(4,3,2,2,1,1,&input,BATCH);
 CNetLayerFunction<type_t> f(NNeuron::NEURON_FUNCTION_TANGENCE,&tconv,BATCH);

 CMemoryStream w;
 w.SaveUInt32(8);w.SaveInt32(4);w.SaveInt32(4);w.SaveInt32(3);w.SaveInt32(2);w.SaveInt32(2);w.SaveInt32(1);w.SaveInt32(1);
 w.PutTensor(1,1,8,3*16,Values(8*48,0.3));   // row = input channel, column = output channel * 16 + tap
 w.PutTensor(1,8,1,1,std::vector<double>(8,0.0));
 tconv.Load(&w);

 CTensor<type_t> x(BATCH,8,4,4);
 FillTensor(x,1.0);
 input.SetOutput(x);
 INetLayer<type_t> *layers[3]={&input,&tconv,&f};
 for(int n=0;n<3;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
 for(int n=0;n<3;n++) layers[n]->Forward();
 Dump("B.tconv",tconv.GetOutputTensor());
 Dump("B.tanh",f.GetOutputTensor());
 CTensor<type_t> error(BATCH,3,8,8);
 FillTensor(error,0.5);
 f.SetOutputError(error);
 for(int n=2;n>=1;n--) layers[n]->TrainingBackward(true);
 Dump("B.delta_tconv",tconv.GetDeltaTensor());
 for(int n=1;n<3;n++) layers[n]->TrainingUpdateWeight(0.05,1);
 CMemoryStream saved;
 tconv.Save(&saved);
 DumpStream("B.tconv_updated",saved,8*sizeof(int32_t),2);
 DumpRaw("B.tconv_stream",saved);
}

// Chain D: resampling layers, forward and backward (no weights)
static void ChainD(void)
{
 CNetLayerConvolutionInput<type_t> input(4,4,4,BATCH);
 CNetLayerUpSampling<type_t> up(2,2,&input,BATCH);
 CNetLayerAveragePooling<type_t> avg(4,4,&up,BATCH);
 CTensor<type_t> image(BATCH,4,4,4);
 FillTensor(image,1.0);
 input.SetOutput(image);
 INetLayer<type_t> *layers[3]={&input,&up,&avg};
 for(int n=0;n<3;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
 for(int n=0;n<3;n++) layers[n]->Forward();
 Dump("D.input",image);
 Dump("D.upsampling",up.GetOutputTensor());
 Dump("D.average",avg.GetOutputTensor());
 CTensor<type_t> error(BATCH,4,2,2);
 FillTensor(error,0.5);
 avg.SetOutputError(error);
 for(int n=2;n>=1;n--) layers[n]->TrainingBackward(true);
 Dump("D.delta_average",avg.GetDeltaTensor());
 Dump("D.delta_upsampling",up.GetDeltaTensor());
 CMemoryStream net_saved;
 for(int n=0;n<3;n++) layers[n]->Save(&net_saved);
 DumpRaw("D.net_stream",net_saved);
}

static void ChainU(void)
{
 CNetLayerConvolutionInput<type_t> input(16,6,8,BATCH);
 CNetLayerUpSampling<type_t> up(2,2,&input,BATCH);
 CNetLayerConvolution<type_t> conv(8,3,1,1,1,1,&up,BATCH);
 CNetLayerFunction<type_t> f(NNeuron::NEURON_FUNCTION_LEAKY_RELU,&conv,BATCH);
 CMemoryStream conv_w;
 conv_w.SaveUInt32(8);conv_w.SaveInt32(3);conv_w.SaveInt32(3);conv_w.SaveInt32(16);conv_w.SaveInt32(1);conv_w.SaveInt32(1);conv_w.SaveInt32(1);conv_w.SaveInt32(1);
 conv_w.PutTensor(1,1,8,16*9,Values(8*144,0.15));
 conv_w.PutTensor(1,8,1,1,Values(8,0.1));
 conv.Load(&conv_w);
 CTensor<type_t> image(BATCH,16,6,8),error(BATCH,8,12,16);
 INetLayer<type_t> *layers[4]={&input,&up,&conv,&f};
 for(int n=0;n<4;n++) layers[n]->TrainingStart();
 for(int step=0;step<2;step++)
 {
  FillTensor(image,1.0+step);
  input.SetOutput(image);
  for(int n=0;n<4;n++) layers[n]->TrainingResetDeltaWeight();
  for(int n=0;n<4;n++) layers[n]->Forward();
  const std::string tag=std::string("U.")+(step==0?"first.":"second.");
  Dump((tag+"conv").c_str(),conv.GetOutputTensor());
  Dump((tag+"leaky").c_str(),f.GetOutputTensor());
  FillTensor(error,0.5);
  f.SetOutputError(error);
  for(int n=3;n>=1;n--) layers[n]->TrainingBackward(true);
  Dump((tag+"delta_conv").c_str(),conv.GetDeltaTensor());
  Dump((tag+"delta_upsampling").c_str(),up.GetDeltaTensor());
  for(int n=1;n<4;n++) layers[n]->TrainingUpdateWeight(0.05,step+1);
  CMemoryStream saved;
  conv.Save(&saved);
  DumpStream((tag+"conv_updated").c_str(),saved,8*sizeof(int32_t),2);
 }
 Dump("U.upsampling",up.GetOutputTensor());   // read at last: whoever asks for the up-sampled image gets it
}


// Chain H: layers that work on the host, element by element
static void ChainH(void)
{
 // soft-max over all elements of a sample, forward and the full Jacobian backward
 {
  CNetLayerConvolutionInput<type_t> input(2,3,4,BATCH);
  CNetLayerFunction<type_t> pass(NNeuron::NEURON_FUNCTION_LINEAR,&input,BATCH);
  CNetLayerSoftMax<type_t> soft(&pass,BATCH);
  CTensor<type_t> x(BATCH,2,3,4);
  FillTensor(x,2.0);
  input.SetOutput(x);
  INetLayer<type_t> *layers[3]={&input,&pass,&soft};
  for(int n=0;n<3;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
  for(int n=0;n<3;n++) layers[n]->Forward();
  Dump("H.soft_input",x);
  Dump("H.softmax",soft.GetOutputTensor());
  CTensor<type_t> error(BATCH,2,3,4);
  FillTensor(error,0.5);
  Dump("H.soft_error",error);
  soft.SetOutputError(error);
  soft.TrainingBackward(true);
  Dump("H.soft_delta",pass.GetDeltaTensor());
 }
 // splitter with two consumers: the output is the input, the errors of both consumers add up
 {
  CNetLayerConvolutionInput<type_t> input(3,4,4,BATCH);
  CNetLayerFunction<type_t> pass(NNeuron::NEURON_FUNCTION_LINEAR,&input,BATCH);
  CNetLayerSplitter<type_t> split(2,&pass,BATCH);
  CNetLayerFunction<type_t> branch_a(NNeuron::NEURON_FUNCTION_LINEAR,&split,BATCH),branch_b(NNeuron::NEURON_FUNCTION_TANGENCE,&split,BATCH);
  CTensor<type_t> x(BATCH,3,4,4);
  FillTensor(x,1.0);
  input.SetOutput(x);
  INetLayer<type_t> *layers[5]={&input,&pass,&split,&branch_a,&branch_b};
  for(int n=0;n<5;n++) layers[n]->Forward();   // the splitter's training tensors are copies of its output
  for(int n=0;n<5;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
  for(int n=0;n<5;n++) layers[n]->Forward();
  Dump("H.split_input",x);
  Dump("H.split_output",split.GetOutputTensor());
  Dump("H.split_tanh",branch_b.GetOutputTensor());
  CTensor<type_t> error_a(BATCH,3,4,4),error_b(BATCH,3,4,4);
  FillTensor(error_a,0.5);
  FillTensor(error_b,0.5);
  Dump("H.split_error_a",error_a);
  Dump("H.split_error_b",error_b);
  branch_a.SetOutputError(error_a);
  branch_b.SetOutputError(error_b);
  branch_a.TrainingBackward(true);
  branch_b.TrainingBackward(true);
  Dump("H.split_delta",split.GetDeltaTensor());
  split.TrainingBackward(true);
  Dump("H.split_prev_delta",pass.GetDeltaTensor());
 }
 // drop-out: the mask comes from std::random_device
 {
  CNetLayerConvolutionInput<type_t> input(4,8,8,BATCH);
  CNetLayerFunction<type_t> pass(NNeuron::NEURON_FUNCTION_LINEAR,&input,BATCH);
  CNetLayerDropOut<type_t> drop(0.25,&pass,BATCH);
  CTensor<type_t> x(BATCH,4,8,8);
  FillTensor(x,1.0);
  input.SetOutput(x);
  INetLayer<type_t> *layers[3]={&input,&pass,&drop};
  for(int n=0;n<3;n++) layers[n]->Forward();
  Dump("H.drop_inference",drop.GetOutputTensor());   // not training: the layer hands its input through
  for(int n=0;n<3;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
  for(int n=0;n<3;n++) layers[n]->Forward();
  Dump("H.drop_input",x);
  Dump("H.drop_output",drop.GetOutputTensor());
  CTensor<type_t> error(BATCH,4,8,8);
  FillTensor(error,0.5);
  Dump("H.drop_error",error);
  drop.SetOutputError(error);
  drop.TrainingBackward(true);
  Dump("H.drop_prev_delta",pass.GetDeltaTensor());
  CMemoryStream saved;
  drop.Save(&saved);
  DumpRaw("H.drop_stream",saved);
 }
 // output of a VAE coder: mu + exp(logvar/2)*noise, the noise from std::random_device; Kullback-Leibler terms in the error
 {
  CNetLayerConvolutionInput<type_t> input_mu(1,16,1,BATCH),input_logvar(1,16,1,BATCH);
  CNetLayerFunction<type_t> mu(NNeuron::NEURON_FUNCTION_LINEAR,&input_mu,BATCH),logvar(NNeuron::NEURON_FUNCTION_LINEAR,&input_logvar,BATCH);
  CNetLayerVAECoderOutput<type_t> coder(0.125f,&mu,&logvar,BATCH);
  CTensor<type_t> m(BATCH,1,16,1),l(BATCH,1,16,1);
  FillTensor(m,1.0);
  FillTensor(l,12.0);   // beyond the clamp at +-10 in places
  input_mu.SetOutput(m);
  input_logvar.SetOutput(l);
  INetLayer<type_t> *layers[5]={&input_mu,&input_logvar,&mu,&logvar,&coder};
  for(int n=0;n<5;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
  for(int n=0;n<5;n++) layers[n]->Forward();
  Dump("H.vae_mu",m);
  Dump("H.vae_logvar",l);
  Dump("H.vae_output",coder.GetOutputTensor());
  CTensor<type_t> error(BATCH,1,16,1);
  FillTensor(error,0.5);
  Dump("H.vae_error",error);
  coder.SetOutputError(error);   // the Kullback-Leibler weight is 0 until iteration 6
  Dump("H.vae_delta_mu0",mu.GetDeltaTensor());
  Dump("H.vae_delta_logvar0",logvar.GetDeltaTensor());
  coder.TrainingUpdateWeight(0.05,6);
  coder.SetOutputError(error);
  Dump("H.vae_delta_mu",mu.GetDeltaTensor());
  Dump("H.vae_delta_logvar",logvar.GetDeltaTensor());
 }
 // max de-pooling: every input element fills its block; backward through the layer
 {
  CNetLayerConvolutionInput<type_t> input(3,4,4,BATCH);
  CNetLayerFunction<type_t> pass(NNeuron::NEURON_FUNCTION_LINEAR,&input,BATCH);
  CNetLayerMaxDePooling<type_t> depool(2,3,&pass,BATCH);
  CTensor<type_t> x(BATCH,3,4,4);
  FillTensor(x,1.0);
  input.SetOutput(x);
  INetLayer<type_t> *layers[3]={&input,&pass,&depool};
  for(int n=0;n<3;n++) layers[n]->Forward();
  for(int n=0;n<3;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
  for(int n=0;n<3;n++) layers[n]->Forward();
  Dump("H.depool_input",x);
  Dump("H.depool_output",depool.GetOutputTensor());
  CTensor<type_t> error(BATCH,3,8,12);
  FillTensor(error,0.5);
  Dump("H.depool_error",error);
  depool.SetOutputError(error);
  depool.TrainingBackward(true);
  Dump("H.depool_prev_delta",pass.GetDeltaTensor());
  CMemoryStream saved;
  depool.Save(&saved);
  DumpRaw("H.depool_stream",saved);
 }
}

#ifndef USE_CPU
// Chain E: layers whose tensor functions exist in the GPU class only: two inputs -> Concatenator -> TimeEmbedding
static void ChainE(void)
{
 CNetLayerConvolutionInput<type_t> input_a(2,4,4,BATCH),input_b(3,4,4,BATCH);
 CNetLayerConcatenator<type_t> cat(&input_a,&input_b,BATCH);
 CNetLayerTimeEmbedding<type_t> time(&cat,BATCH);
 CTensor<type_t> a(BATCH,2,4,4),b(BATCH,3,4,4);
 FillTensor(a,1.0);
 FillTensor(b,1.0);
 input_a.SetOutput(a);
 input_b.SetOutput(b);
 INetLayer<type_t> *layers[4]={&input_a,&input_b,&cat,&time};
 for(int n=0;n<4;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
 CTensor<type_t> steps(BATCH,1,1,1);
 for(uint32_t w=0;w<BATCH;w++) {time.SetTimeStep(w,w*7);steps.SetElement(w,0,0,0,static_cast<type_t>(w*7));}
 for(int n=0;n<4;n++) layers[n]->Forward();
 Dump("E.a",a);
 Dump("E.b",b);
 Dump("E.steps",steps);
 Dump("E.concatenated",cat.GetOutputTensor());
 Dump("E.time",time.GetOutputTensor());
}

// Chain F: the max-pooling layer keeps a CTensor<CTensorMath<type_t>::SPos>, a type only the GPU class nests
static void ChainF(void)
{
 CNetLayerConvolutionInput<type_t> input(4,8,8,BATCH);
 CNetLayerFunction<type_t> pass(NNeuron::NEURON_FUNCTION_LINEAR,&input,BATCH);   // keeps the error it is handed (derivative 1)
 CNetLayerMaxPooling<type_t> pool(2,2,&pass,BATCH);
 CTensor<type_t> image(BATCH,4,8,8);
 FillTensor(image,1.0);
 input.SetOutput(image);
 INetLayer<type_t> *layers[3]={&input,&pass,&pool};
 for(int n=0;n<3;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
 for(int n=0;n<3;n++) layers[n]->Forward();
 Dump("F.input",image);
 Dump("F.maxpool",pool.GetOutputTensor());
 CTensor<type_t> error(BATCH,4,4,4);
 FillTensor(error,0.5);
 Dump("F.error",error);
 pool.SetOutputError(error);
 pool.TrainingBackward(true);
 Dump("F.prev_error",pass.GetDeltaTensor());
}


// Timing of the unchanged layer classes on the drop-in tensors at the sizes of the two networks the library is tuned
// for; CTimeStamp (the reference's own scope timer, here the drop-in's) prints each figure through SYSTEM::PutMessageToConsole
// and CCUDATimeSpent returns it.  One JSON line per chain on stdout.
static void LoadConvolutionWeights(INetLayer<type_t> &layer,uint32_t rows,uint32_t amount_field,int32_t size,int32_t depth_field,uint32_t columns,uint32_t biases,double scale,int32_t padding=1)
{
 CMemoryStream w;
 w.SaveUInt32(amount_field);w.SaveInt32(size);w.SaveInt32(size);w.SaveInt32(depth_field);w.SaveInt32(2);w.SaveInt32(2);w.SaveInt32(padding);w.SaveInt32(padding);
 w.PutTensor(1,1,rows,columns,Values(static_cast<size_t>(rows)*columns,scale));
 w.PutTensor(1,biases,1,1,std::vector<double>(biases,0.0));
 layer.Load(&w);
}

static long long driver_allocations_in_the_timed_steps=0;   // blocks asked of the driver during the last TimeSteps' timed pass
static double TimeSteps(const char *name,std::vector<INetLayer<type_t>*> &net,CTensor<type_t> *error,uint32_t warmup,uint32_t steps)
{
 double ms=0;
 int64_t before=0,after=0;
 for(uint32_t pass=0;pass<2;pass++)
 {
  const uint32_t count=(pass==0)?warmup:steps;
  mt_get_info("driver_allocations",&before);
  CCUDATimeSpent timer;
  timer.Start();
  {
   CTimeStamp stamp(std::string(name)+(pass==0?" (warm-up): ":": "),true);
   for(uint32_t step=0;step<count;step++)
   {
    for(size_t n=0;n<net.size();n++) net[n]->Forward();
    if (error==NULL) continue;
    for(size_t n=0;n<net.size();n++) net[n]->TrainingResetDeltaWeight();
    net[net.size()-1]->SetOutputError(*error);
    for(size_t n=net.size()-1;n>=1;n--) net[n]->TrainingBackward(true);
    for(size_t n=1;n<net.size();n++) net[n]->TrainingUpdateWeight(0.0002,step+1);
   }
  }
  ms=timer.Stop();
  mt_get_info("driver_allocations",&after);
 }
 driver_allocations_in_the_timed_steps=after-before;
 return(ms/steps);
}

// DCGAN-64 generator, forward pass in training mode (batch statistics), batch 256
static void TimeGenerator(uint32_t batch,uint32_t warmup,uint32_t steps)
{
 static const uint32_t channels[5]={512,256,128,64,3};
 std::vector<std::shared_ptr<INetLayer<type_t> > > owner;
 std::vector<INetLayer<type_t>*> net;
#define PUSH(LAYER) {owner.push_back(std::shared_ptr<INetLayer<type_t> >(LAYER));net.push_back(owner.back().get());}
 PUSH(new CNetLayerLinear<type_t>(100,NULL,batch));
 PUSH(new CNetLayerLinear<type_t>(channels[0]*16,net.back(),batch));
 {
  CMemoryStream w;
  w.PutTensor(1,1,channels[0]*16,100,Values(channels[0]*16*100,0.02));
  w.PutTensor(1,1,channels[0]*16,1,std::vector<double>(channels[0]*16,0.0));
  net.back()->Load(&w);
 }
 for(uint32_t i=0;i<4;i++)
 {
  PUSH(new CNetLayerBatchNormalization<type_t>(0.9f,net.back(),batch));
  net.back()->Reset();
  PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_RELU,net.back(),batch));
  // the first transposed convolution takes the vector as [512,4,4]: it remembers the shape it was constructed on and
  // reinterprets its input to it in every Forward (netlayer/cnetlayerbackconvolution.cu.h:305-315)
  if (i==0) net.back()->GetOutputTensor().ReinterpretSize(batch,channels[0],4,4);
  INetLayer<type_t> *function=net.back();
  PUSH(new CNetLayerBackConvolution<type_t>(4,channels[i+1],2,2,1,1,net.back(),batch));
  if (i==0) function->GetOutputTensor().ReinterpretSize(batch,1,channels[0]*16,1);
  LoadConvolutionWeights(*net.back(),channels[i],channels[i],4,channels[i+1],channels[i+1]*16,channels[i],0.02);
 }
 PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_TANGENCE,net.back(),batch));
 CTensor<type_t> latent(batch,1,100,1);
 FillTensor(latent,1.0);
 net[0]->SetOutput(latent);
 for(size_t n=0;n<net.size();n++) net[n]->TrainingStart();
 double ms=TimeSteps("generator forward",net,NULL,warmup,steps);
 CTensor<type_t> &image=net.back()->GetOutputTensor();
 double sum=0;
 for(uint32_t x=0;x<64;x++) sum+=fabs(image.GetElement(batch-1,2,63,x));
 printf("{\"chain\": \"dcgan64_generator_forward\", \"batch\": %u, \"steps\": %u, \"ms_per_step\": %.4f, \"output\": [%u,%u,%u,%u], \"last_row_abs_sum\": %.6f, \"driver_allocations_in_the_timed_steps\": %lld}\n",
        batch,steps,ms,image.GetSizeW(),image.GetSizeZ(),image.GetSizeY(),image.GetSizeX(),sum,driver_allocations_in_the_timed_steps);
}

// The generator of the reference's GAN model (cuda/netmodel/cmodel_gan.cu.h:136-225), forward pass in training mode, batch 32:
// Linear 1024 -> 512x3x4, leaky ReLU, six times (UpSampling 2x2, Convolution 3x3, BatchNormalization, leaky ReLU) through
// 512, 256, 128, 64, 32, 16 channels, Convolution 3x3 to 3 channels, Tangence: 192x256 images
static void TimeGanGenerator(uint32_t batch,uint32_t warmup,uint32_t steps,bool train=false)
{
 static const uint32_t channels[8]={512,512,256,128,64,32,16,3};
 rng_state=0x243F6A8885A308D3ull;   // the same weights and latent vectors on every call (the chain may run twice)
 std::vector<std::shared_ptr<INetLayer<type_t> > > owner;
 std::vector<INetLayer<type_t>*> net;
 PUSH(new CNetLayerLinear<type_t>(1024,NULL,batch));
 PUSH(new CNetLayerLinear<type_t>(channels[0]*12,net.back(),batch));
 {
  CMemoryStream w;
  w.PutTensor(1,1,channels[0]*12,1024,Values(static_cast<size_t>(channels[0])*12*1024,0.025));
  w.PutTensor(1,1,channels[0]*12,1,std::vector<double>(channels[0]*12,0.1));
  net.back()->Load(&w);
 }
 PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));
 // the first up-sampling layer takes the vector as [512,3,4]: it remembers the shape it was constructed on and reinterprets
 // its input to it in every Forward (netlayer/cnetlayerupsampling.cu.h:243-252)
 INetLayer<type_t> *function=net.back();
 function->GetOutputTensor().ReinterpretSize(batch,channels[0],3,4);
 for(uint32_t i=0;i<7;i++)
 {
  if (i<6) PUSH(new CNetLayerUpSampling<type_t>(2,2,net.back(),batch));
  if (i==0) function->GetOutputTensor().ReinterpretSize(batch,1,channels[0]*12,1);
  PUSH(new CNetLayerConvolution<type_t>(channels[i+1],3,1,1,1,1,net.back(),batch));
  {
   const uint32_t columns=channels[i]*9;
   CMemoryStream w;
   w.SaveUInt32(channels[i+1]);w.SaveInt32(3);w.SaveInt32(3);w.SaveInt32(channels[i]);w.SaveInt32(1);w.SaveInt32(1);w.SaveInt32(1);w.SaveInt32(1);
   w.PutTensor(1,1,channels[i+1],columns,Values(static_cast<size_t>(channels[i+1])*columns,sqrt(6.0/columns)));
   w.PutTensor(1,channels[i+1],1,1,Values(channels[i+1],0.05));
   net.back()->Load(&w);
  }
  if (i<6)
  {
   PUSH(new CNetLayerBatchNormalization<type_t>(0.9f,net.back(),batch));
   net.back()->Reset();
   PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));
  }
 }
 PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_TANGENCE,net.back(),batch));
 CTensor<type_t> latent(batch,1,1024,1);
 FillTensor(latent,1.0);
 net[0]->SetOutput(latent);
 for(size_t n=0;n<net.size();n++)
 {
  if (train==true) net[n]->TrainingModeAdam(0.5,0.9);   // as the model trains it (cuda/netmodel/cmodel_basicgan.cu.h:852)
  net[n]->TrainingStart();
 }
 CTensor<type_t> error(batch,3,192,256);
 if (train==true) FillTensor(error,0.01);
 double ms=TimeSteps(train==true?"GAN generator step":"GAN generator forward",net,train==true?&error:NULL,warmup,steps);
 CTensor<type_t> &image=net.back()->GetOutputTensor();
 double sum=0;
 for(uint32_t x=0;x<256;x++) sum+=fabs(image.GetElement(batch-1,2,191,x));
 if (train==true)
 {
  printf("{\"chain\": \"gan_generator_step\", \"batch\": %u, \"steps\": %u, \"ms_per_step\": %.4f, \"output\": [%u,%u,%u,%u], \"last_row_abs_sum\": %.6f, \"driver_allocations_in_the_timed_steps\": %lld}\n",
         batch,steps,ms,image.GetSizeW(),image.GetSizeZ(),image.GetSizeY(),image.GetSizeX(),sum,driver_allocations_in_the_timed_steps);
  return;
 }
 printf("{\"chain\": \"gan_generator_forward\", \"batch\": %u, \"steps\": %u, \"ms_per_step\": %.4f, \"output\": [%u,%u,%u,%u], \"last_row_abs_sum\": %.6f, \"driver_allocations_in_the_timed_steps\": %lld}\n",
        batch,steps,ms,image.GetSizeW(),image.GetSizeZ(),image.GetSizeY(),image.GetSizeX(),sum,driver_allocations_in_the_timed_steps);
}

// DCGAN-64 discriminator, whole training step (forward, backward with weight gradients, Adam), batch 128
// the discriminator's layers with seeded weights, in training mode (Adam or plain gradient descent)
static void BuildDiscriminator(uint32_t batch,std::vector<std::shared_ptr<INetLayer<type_t> > > &owner,std::vector<INetLayer<type_t>*> &net,bool adam=true)
{
 static const uint32_t channels[5]={3,64,128,256,512};
 PUSH(new CNetLayerConvolutionInput<type_t>(3,64,64,batch));
 for(uint32_t i=0;i<4;i++)
 {
  PUSH(new CNetLayerConvolution<type_t>(channels[i+1],4,2,2,1,1,net.back(),batch));
  LoadConvolutionWeights(*net.back(),channels[i+1],channels[i+1],4,channels[i],channels[i]*16,channels[i+1],0.02);
  PUSH(new CNetLayerBatchNormalization<type_t>(0.9f,net.back(),batch));
  net.back()->Reset();
  PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));
 }
 PUSH(new CNetLayerLinear<type_t>(1,net.back(),batch));
 {
  CMemoryStream w;
  w.PutTensor(1,1,1,512*16,Values(512*16,0.02));
  w.PutTensor(1,1,1,1,std::vector<double>(1,0.0));
  net.back()->Load(&w);
 }
 PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_SIGMOID,net.back(),batch));
#undef PUSH
 for(size_t n=0;n<net.size();n++)
 {
  if (adam==true) net[n]->TrainingModeAdam();
  net[n]->TrainingStart();
 }
}

static void TimeDiscriminator(uint32_t batch,uint32_t warmup,uint32_t steps)
{
 std::vector<std::shared_ptr<INetLayer<type_t> > > owner;
 std::vector<INetLayer<type_t>*> net;
 BuildDiscriminator(batch,owner,net);
 CTensor<type_t> image(batch,3,64,64),error(batch,1,1,1);
 FillTensor(image,1.0);
 FillTensor(error,0.5);
 net[0]->SetOutput(image);
 double ms=TimeSteps("discriminator step",net,&error,warmup,steps);
 CTensor<type_t> &out=net.back()->GetOutputTensor();
 printf("{\"chain\": \"dcgan64_discriminator_step\", \"batch\": %u, \"steps\": %u, \"ms_per_step\": %.4f, \"output\": [%u,%u,%u,%u], \"first\": %.6f, \"driver_allocations_in_the_timed_steps\": %lld}\n",
        batch,steps,ms,out.GetSizeW(),out.GetSizeZ(),out.GetSizeY(),out.GetSizeX(),out.GetElement(0,0,0,0),driver_allocations_in_the_timed_steps);
}

// The discriminator of the reference's GAN model (cuda/netmodel/cmodel_gan.cu.h:236-287), whole training step in Adam mode, batch 32:
// Convolution 5x5 stride 2 padding 2 to 16 filters, leaky ReLU, five times (Convolution 5x5 stride 2 padding 2, BatchNormalization,
// leaky ReLU) through 32, 64, 128, 256, 512 filters, Linear to one output; 192x256 images
static void TimeGanDiscriminator(uint32_t batch,uint32_t warmup,uint32_t steps)
{
 static const uint32_t channels[7]={3,16,32,64,128,256,512};
 rng_state=0x13198A2E03707344ull;
 std::vector<std::shared_ptr<INetLayer<type_t> > > owner;
 std::vector<INetLayer<type_t>*> net;
#define PUSH(LAYER) {owner.push_back(std::shared_ptr<INetLayer<type_t> >(LAYER));net.push_back(owner.back().get());}
 PUSH(new CNetLayerConvolutionInput<type_t>(3,192,256,batch));
 for(uint32_t i=0;i<6;i++)
 {
  PUSH(new CNetLayerConvolution<type_t>(channels[i+1],5,2,2,2,2,net.back(),batch));
  LoadConvolutionWeights(*net.back(),channels[i+1],channels[i+1],5,channels[i],channels[i]*25,channels[i+1],sqrt(2.0/(channels[i]*25)),2);
  if (i>0)
  {
   PUSH(new CNetLayerBatchNormalization<type_t>(0.9f,net.back(),batch));
   net.back()->Reset();
  }
  PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));
 }
 PUSH(new CNetLayerLinear<type_t>(1,net.back(),batch));
 {
  CMemoryStream w;
  w.PutTensor(1,1,1,512*12,Values(512*12,0.02));
  w.PutTensor(1,1,1,1,std::vector<double>(1,0.0));
  net.back()->Load(&w);
 }
#undef PUSH
 for(size_t n=0;n<net.size();n++)
 {
  net[n]->TrainingModeAdam(0.5,0.9);
  net[n]->TrainingStart();
 }
 CTensor<type_t> image(batch,3,192,256),error(batch,1,1,1);
 FillTensor(image,1.0);
 FillTensor(error,0.5);
 net[0]->SetOutput(image);
 double ms=TimeSteps("GAN discriminator step",net,&error,warmup,steps);
 CTensor<type_t> &out=net.back()->GetOutputTensor();
 printf("{\"chain\": \"gan_discriminator_step\", \"batch\": %u, \"steps\": %u, \"ms_per_step\": %.4f, \"output\": [%u,%u,%u,%u], \"first\": %.6f, \"driver_allocations_in_the_timed_steps\": %lld}\n",
        batch,steps,ms,out.GetSizeW(),out.GetSizeZ(),out.GetSizeY(),out.GetSizeX(),out.GetElement(0,0,0,0),driver_allocations_in_the_timed_steps);
}

// a convolution layer's weights as the layer saves them: uniform in +-scale (scale 0: sqrt(6 / columns)), small biases
static void LoadConvolution(INetLayer<type_t> &layer,uint32_t amount,int32_t size,uint32_t depth,int32_t stride,int32_t padding,double scale=0)
{
 const uint32_t columns=depth*size*size;
 CMemoryStream w;
 w.SaveUInt32(amount);w.SaveInt32(size);w.SaveInt32(size);w.SaveInt32(depth);w.SaveInt32(stride);w.SaveInt32(stride);w.SaveInt32(padding);w.SaveInt32(padding);
 w.PutTensor(1,1,amount,columns,Values(static_cast<size_t>(amount)*columns,scale>0?scale:sqrt(6.0/columns)));
 w.PutTensor(1,amount,1,1,Values(amount,0.05));
 layer.Load(&w);
}

// The reference's VAE model (cuda/netmodel/cmodel_vae.cu.h:130-230), whole training step in Adam mode, batch 32, 256x256 images.
// Coder: three times (Convolution 5x5 stride 2 padding 2, BatchNormalization, leaky ReLU) to 32, 64, 128 filters, Splitter, two
// Convolutions 5x5 stride 2 to one filter (mu, log variance: 16x16), VAECoderOutput.  Decoder: seven Convolutions 3x3 (128, 128, 128,
// 64, 64, 32 filters with BatchNormalization and leaky ReLU, UpSampling 2x2 in front of the third to the sixth; then 3 filters and
// leaky ReLU): 256x256 images.
static void TimeVae(uint32_t batch,uint32_t warmup,uint32_t steps)
{
 rng_state=0xA4093822299F31D0ull;
 std::vector<std::shared_ptr<INetLayer<type_t> > > owner;
 std::vector<INetLayer<type_t>*> net;
#define PUSH(LAYER) {owner.push_back(std::shared_ptr<INetLayer<type_t> >(LAYER));net.push_back(owner.back().get());}
 PUSH(new CNetLayerConvolutionInput<type_t>(3,256,256,batch));
 static const uint32_t coder[4]={3,32,64,128};
 for(uint32_t i=0;i<3;i++)
 {
  PUSH(new CNetLayerConvolution<type_t>(coder[i+1],5,2,2,2,2,net.back(),batch));
  LoadConvolution(*net.back(),coder[i+1],5,coder[i],2,2);
  PUSH(new CNetLayerBatchNormalization<type_t>(0.9f,net.back(),batch));
  net.back()->Reset();
  PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));
 }
 PUSH(new CNetLayerSplitter<type_t>(2,net.back(),batch));
 INetLayer<type_t> *splitter=net.back();
 PUSH(new CNetLayerConvolution<type_t>(1,5,2,2,2,2,splitter,batch));
 LoadConvolution(*net.back(),1,5,128,2,2);
 INetLayer<type_t> *mu=net.back();
 PUSH(new CNetLayerConvolution<type_t>(1,5,2,2,2,2,splitter,batch));
 LoadConvolution(*net.back(),1,5,128,2,2,0.01);
 INetLayer<type_t> *logvar=net.back();
 PUSH(new CNetLayerVAECoderOutput<type_t>(0.001f,mu,logvar,batch));
 static const uint32_t decoder[8]={1,128,128,128,64,64,32,3};
 for(uint32_t i=0;i<7;i++)
 {
  if (i>=2 && i<=5) PUSH(new CNetLayerUpSampling<type_t>(2,2,net.back(),batch));
  PUSH(new CNetLayerConvolution<type_t>(decoder[i+1],3,1,1,1,1,net.back(),batch));
  LoadConvolution(*net.back(),decoder[i+1],3,decoder[i],1,1);
  if (i<6)
  {
   PUSH(new CNetLayerBatchNormalization<type_t>(0.9f,net.back(),batch));
   net.back()->Reset();
  }
  PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));
 }
#undef PUSH
 for(size_t n=0;n<net.size();n++)
 {
  net[n]->TrainingModeAdam(0.9,0.999);   // as the model trains it (cuda/netmodel/cmodel_basicvae.cu.h:487-492)
  net[n]->TrainingStart();
 }
 CTensor<type_t> image(batch,3,256,256),error(batch,3,256,256);
 FillTensor(image,1.0);
 FillTensor(error,0.01);
 net[0]->SetOutput(image);
 double ms=TimeSteps("VAE step",net,&error,warmup,steps);
 CTensor<type_t> &out=net.back()->GetOutputTensor();
 double sum=0;
 for(uint32_t x=0;x<256;x++) sum+=fabs(out.GetElement(batch-1,2,255,x));
 printf("{\"chain\": \"vae_step\", \"batch\": %u, \"steps\": %u, \"ms_per_step\": %.4f, \"output\": [%u,%u,%u,%u], \"last_row_abs_sum\": %.6f, \"driver_allocations_in_the_timed_steps\": %lld}\n",
        batch,steps,ms,out.GetSizeW(),out.GetSizeZ(),out.GetSizeY(),out.GetSizeX(),sum,driver_allocations_in_the_timed_steps);
}

// The reference's diffusion model (cuda/netmodel/cmodel_diffusion.cu.h:106-230), whole training step in Adam mode, batch 32, 192x256 images:
// a U-net.  Down: five blocks (Convolution 3x3, TimeEmbedding, leaky ReLU, Splitter, Convolution 3x3 stride 2) with 16, 32, 64, 128, 256
// filters; bottom: three times (Convolution 3x3 to 512 filters, TimeEmbedding, leaky ReLU) at 6x8; up: five blocks (UpSampling 2x2,
// Concatenator with the splitter of the same size, Convolution 3x3, TimeEmbedding, leaky ReLU) with 256, 128, 64, 32, 16 filters; then
// Convolution 3x3 to 16 filters, leaky ReLU, Convolution 3x3 to the image.  The time steps are set before every step, sample by sample
// and layer by layer, as the model does (cuda/netmodel/cmodel_basicdiffusion.cu.h:303).
static void TimeDiffusion(uint32_t batch,uint32_t warmup,uint32_t steps)
{
 rng_state=0x082EFA98EC4E6C89ull;
 std::vector<std::shared_ptr<INetLayer<type_t> > > owner;
 std::vector<INetLayer<type_t>*> net;
#define PUSH(LAYER) {owner.push_back(std::shared_ptr<INetLayer<type_t> >(LAYER));net.push_back(owner.back().get());}
#define BLOCK(FILTERS,DEPTH) {PUSH(new CNetLayerConvolution<type_t>(FILTERS,3,1,1,1,1,net.back(),batch));LoadConvolution(*net.back(),FILTERS,3,DEPTH,1,1);\
                              PUSH(new CNetLayerTimeEmbedding<type_t>(net.back(),batch));\
                              PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));}
 PUSH(new CNetLayerConvolutionInput<type_t>(3,192,256,batch));
 static const uint32_t down[6]={3,16,32,64,128,256};
 INetLayer<type_t> *split[5];
 for(uint32_t i=0;i<5;i++)
 {
  BLOCK(down[i+1],down[i]);
  PUSH(new CNetLayerSplitter<type_t>(2,net.back(),batch));
  split[i]=net.back();
  PUSH(new CNetLayerConvolution<type_t>(down[i+1],3,2,2,1,1,net.back(),batch));
  LoadConvolution(*net.back(),down[i+1],3,down[i+1],2,1);
 }
 BLOCK(512,256);
 BLOCK(512,512);
 BLOCK(512,512);
 uint32_t depth=512;
 for(int i=4;i>=0;i--)
 {
  PUSH(new CNetLayerUpSampling<type_t>(2,2,net.back(),batch));
  PUSH(new CNetLayerConcatenator<type_t>(net.back(),split[i],batch));
  BLOCK(down[i+1],depth+down[i+1]);
  depth=down[i+1];
 }
 PUSH(new CNetLayerConvolution<type_t>(16,3,1,1,1,1,net.back(),batch));
 LoadConvolution(*net.back(),16,3,16,1,1);
 PUSH(new CNetLayerFunction<type_t>(NNeuron::NEURON_FUNCTION_LEAKY_RELU,net.back(),batch));
 PUSH(new CNetLayerConvolution<type_t>(3,3,1,1,1,1,net.back(),batch));
 LoadConvolution(*net.back(),3,3,16,1,1);
#undef BLOCK
#undef PUSH
 for(size_t n=0;n<net.size();n++)
 {
  net[n]->TrainingModeAdam(0.9,0.999);   // as the model trains it (cuda/netmodel/cmodel_basicdiffusion.cu.h:598)
  net[n]->TrainingStart();
 }
 CTensor<type_t> image(batch,3,192,256),error(batch,3,192,256);
 FillTensor(image,1.0);
 FillTensor(error,0.01);
 net[0]->SetOutput(image);
 double ms=0;
 int64_t before=0,after=0;
 for(uint32_t pass=0;pass<2;pass++)
 {
  const uint32_t count=(pass==0)?warmup:steps;
  mt_get_info("driver_allocations",&before);
  CCUDATimeSpent timer;
  timer.Start();
  for(uint32_t step=0;step<count;step++)
  {
   for(uint32_t b=0;b<batch;b++)
    for(size_t n=0;n<net.size();n++) net[n]->SetTimeStep(b,(b*37+step*11)%1000);
   for(size_t n=0;n<net.size();n++) net[n]->Forward();
   for(size_t n=0;n<net.size();n++) net[n]->TrainingResetDeltaWeight();
   net[net.size()-1]->SetOutputError(error);
   for(size_t n=net.size()-1;n>=1;n--) net[n]->TrainingBackward(true);
   for(size_t n=1;n<net.size();n++) net[n]->TrainingUpdateWeight(0.0002,step+1);
  }
  ms=timer.Stop();
  mt_get_info("driver_allocations",&after);
 }
 CTensor<type_t> &out=net.back()->GetOutputTensor();
 double sum=0;
 for(uint32_t x=0;x<256;x++) sum+=fabs(out.GetElement(batch-1,2,191,x));
 printf("{\"chain\": \"diffusion_step\", \"batch\": %u, \"steps\": %u, \"ms_per_step\": %.4f, \"output\": [%u,%u,%u,%u], \"last_row_abs_sum\": %.6f, \"driver_allocations_in_the_timed_steps\": %lld}\n",
        batch,steps,ms/steps,out.GetSizeW(),out.GetSizeZ(),out.GetSizeY(),out.GetSizeX(),sum,static_cast<long long>(after-before));
}

// Chain K: two training steps (gradient descent) of the discriminator at batch 16, once with the per-sample weight gradients deferred by the
// drop-in classes (mi355::CDeferredGradient; the last two convolution layers qualify) and once with every call run when
// it is made: same seeds, the updated convolution weights of both runs go to the dump
static void ChainK(void)
{
 const uint32_t batch=16;
 for(int deferred=1;deferred>=0;deferred--)
 {
  mi355::DeferGradients()=(deferred==1);
  rng_state=0x0123456789ABCDEFull;
  std::vector<std::shared_ptr<INetLayer<type_t> > > owner;
  std::vector<INetLayer<type_t>*> net;
  // gradient descent: Adam would turn the rounding noise of gradients that are zero by construction (the biases in
  // front of a batch normalisation) into steps of the full learning rate
  BuildDiscriminator(batch,owner,net,false);
  CTensor<type_t> image(batch,3,64,64),error(batch,1,1,1);
  FillTensor(image,1.0);
  FillTensor(error,0.5);
  net[0]->SetOutput(image);
  for(uint32_t step=0;step<2;step++)
  {
   for(size_t n=0;n<net.size();n++) net[n]->Forward();
   for(size_t n=0;n<net.size();n++) net[n]->TrainingResetDeltaWeight();
   net[net.size()-1]->SetOutputError(error);
   for(size_t n=net.size()-1;n>=1;n--) net[n]->TrainingBackward(true);
   for(size_t n=1;n<net.size();n++) net[n]->TrainingUpdateWeight(0.05,step+1);
  }
  for(int layer=0;layer<4;layer++)
  {
   CMemoryStream saved;
   net[1+3*layer]->Save(&saved);
   char label[32];
   snprintf(label,sizeof(label),"K.%s.conv%d",deferred==1?"deferred":"eager",layer+1);
   DumpStream(label,saved,8*sizeof(int32_t),2);
  }
  Dump(deferred==1?"K.deferred.out":"K.eager.out",net.back()->GetOutputTensor());
 }
 mi355::DeferGradients()=true;
}

static void ChainC(void)
{
 CNetLayerConvolutionInput<type_t> input(4,5,5,BATCH);
 CNetLayerBatchNormalization<type_t> bn(0.9f,&input,BATCH);
 CNetLayerFunction<type_t> f(NNeuron::NEURON_FUNCTION_RELU,&bn,BATCH);
 CMemoryStream w;
 std::vector<double> beta=Values(100,0.5),gamma=Values(100,1.0);
 w.PutTensor(1,4,5,5,beta);
 w.PutTensor(1,4,5,5,gamma);
 w.PutTensor(1,4,5,5,std::vector<double>(100,0.0));
 w.PutTensor(1,4,5,5,std::vector<double>(100,1.0));
 w.SaveDouble(0.9);
 bn.Load(&w);
 bn.EnableEMA(true);
 CTensor<type_t> x(BATCH,4,5,5);
 FillTensor(x,2.0);
 input.SetOutput(x);
 INetLayer<type_t> *layers[3]={&input,&bn,&f};
 for(int n=0;n<3;n++) {layers[n]->TrainingStart();layers[n]->TrainingResetDeltaWeight();}
 for(int n=0;n<3;n++) layers[n]->Forward();
 Dump("C.input",x);
 CTensor<type_t> tb(1,4,5,5),tg(1,4,5,5);
 for(uint32_t n=0;n<100;n++) {tb.SetElement(0,n/25,(n%25)/5,n%5,static_cast<type_t>(beta[n]));tg.SetElement(0,n/25,(n%25)/5,n%5,static_cast<type_t>(gamma[n]));}
 Dump("C.beta",tb);
 Dump("C.gamma",tg);
 Dump("C.bn",bn.GetOutputTensor());
 Dump("C.relu",f.GetOutputTensor());
 CTensor<type_t> error(BATCH,4,5,5);
 FillTensor(error,0.5);
 Dump("C.error",error);
 f.SetOutputError(error);
 for(int n=2;n>=1;n--) layers[n]->TrainingBackward(true);
 Dump("C.delta_bn",bn.GetDeltaTensor());
 Dump("C.prev_error",input.GetDeltaTensor());   // the input layer hands back its own tensor: unchanged input
 CMemoryStream bn_saved;
 bn.Save(&bn_saved);
 DumpRaw("C.bn_stream",bn_saved);
 // the end of a training step: Mean and Variable take the statistics blended by the forward pass, then a second step
 for(int n=1;n<3;n++) layers[n]->TrainingUpdateWeight(0.05,1);
 CMemoryStream bn_trained;
 bn.Save(&bn_trained);
 DumpRaw("C.bn_trained_stream",bn_trained);
 CMemoryStream bn_ema;
 bn.SaveEMAWeight(&bn_ema);
 DumpRaw("C.bn_ema_stream",bn_ema);
 CTensor<type_t> x2(BATCH,4,5,5);
 FillTensor(x2,1.5);
 input.SetOutput(x2);
 Dump("C.input2",x2);
 for(int n=0;n<3;n++) layers[n]->TrainingResetDeltaWeight();
 for(int n=0;n<3;n++) layers[n]->Forward();
 for(int n=1;n<3;n++) layers[n]->TrainingUpdateWeight(0.0,2);
 CMemoryStream bn_trained2;
 bn.Save(&bn_trained2);
 DumpRaw("C.bn_trained2_stream",bn_trained2);
 // inference mode with the trained statistics
 for(int n=0;n<3;n++) layers[n]->TrainingStop();
 for(int n=0;n<3;n++) layers[n]->Forward();
 Dump("C.bn_inference",bn.GetOutputTensor());
}
#endif

// Chain G: the layers of chain A loaded from a network file that somebody else wrote (every layer's Load() in order,
// as CModelMain::LoadNetLayers does), forward only
static void ChainG(const char *net_file)
{
 CNetLayerConvolutionInput<type_t> input(3,16,16,BATCH);
 CNetLayerConvolution<type_t> conv(8,4,2,2,1,1,&input,BATCH);
 CNetLayerFunction<type_t> f1(NNeuron::NEURON_FUNCTION_SIGMOID,&conv,BATCH);   // the file says leaky ReLU: Load() must take it from there
 CNetLayerLinear<type_t> lin(24,&f1,BATCH);
 CNetLayerFunction<type_t> f2(NNeuron::NEURON_FUNCTION_SIGMOID,&lin,BATCH);
 CMemoryStream net;
 if (net.ReadFile(net_file)==false) throw("network file not found");
 INetLayer<type_t> *layers[5]={&input,&conv,&f1,&lin,&f2};
 for(int n=0;n<5;n++) layers[n]->Load(&net,true);
 CTensor<type_t> image(BATCH,3,16,16);
 FillTensor(image,1.0);
 input.SetOutput(image);
 for(int n=0;n<5;n++) layers[n]->Forward();
 Dump("G.input",image);
 Dump("G.leaky",f1.GetOutputTensor());
 Dump("G.sigmoid",f2.GetOutputTensor());
}

int main(int argc,char **argv)
{
 if (argc<2) {fprintf(stderr,"usage: %s <output file> [network file for chain G]\n",argv[0]);return(2);}
 out_file=fopen(argv[1],"wb");
 if (out_file==NULL) return(2);
 try
 {
#ifndef USE_CPU
  if (argc>2 && strcmp(argv[2],"deferred")==0)   // only the chain that compares deferred and eager weight gradients
  {
   ChainK();
   fclose(out_file);
   return(0);
  }
  if (argc>2 && strcmp(argv[2],"time")==0)   // only the timed chains: time [steps [warm-up [literal | train | vae | diffusion]]]
  {
   const uint32_t steps=(argc>3)?static_cast<uint32_t>(atoi(argv[3])):50,warmup=(argc>4)?static_cast<uint32_t>(atoi(argv[4])):20;
   TimeGenerator(256,warmup,steps);
   TimeDiscriminator(128,warmup,steps);
   TimeGanGenerator(32,warmup,steps);
   if (argc>5 && strcmp(argv[5],"train")==0)   // and the whole training steps (forward, backward, Adam) of the reference's GAN generator and discriminator
   {
    TimeGanGenerator(32,warmup,steps,true);
    TimeGanDiscriminator(32,warmup,steps);
   }
   if (argc>5 && strcmp(argv[5],"vae")==0) TimeVae(32,warmup,steps);   // or the whole training step of the reference's VAE model
   if (argc>5 && strcmp(argv[5],"diffusion")==0) TimeDiffusion(32,warmup,steps);   // or that of its diffusion model
   if (argc>5 && strcmp(argv[5],"literal")==0)   // and the last chain once more with every call run when it is made
   {
    mi355::DeferGradients()=false;
    TimeGanGenerator(32,warmup,steps);
    mi355::DeferGradients()=true;
   }
   fclose(out_file);
   return(0);
  }
#endif
  if (argc>2)   // only the chain that loads the given network file
  {
   ChainG(argv[2]);
   fclose(out_file);
   return(0);
  }
  ChainA();
  ChainB();
  ChainD();
  ChainU();
  ChainH();
#ifndef USE_CPU
  ChainC();
  ChainE();
  ChainF();
#endif
 }
 catch(const char *message)
 {
  fprintf(stderr,"exception: %s\n",message);
  return(1);
 }
 fclose(out_file);
 return(0);
}
