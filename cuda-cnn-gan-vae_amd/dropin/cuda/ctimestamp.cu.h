#ifndef C_TIME_STAMP_CU_H
#define C_TIME_STAMP_CU_H

// Drop-in for the reference's scope timer (cuda/ctimestamp.cu.h:16-34, cuda/ctimestamp.cu:17-32): measures the work
// queued during the object's lifetime and, when enabled, prints "<text><milliseconds> мс." through SYSTEM.
// Header-only: there is no ctimestamp.cu to compile.

#include <stdio.h>
#include <string>

#include "ccudatimespent.cu.h"
#include "../system/system.h"

class CTimeStamp
{
 private:
  std::string Text;
  CCUDATimeSpent cCUDATimeSpent;
  bool Enabled;
 public:
  CTimeStamp(std::string text,bool enabled=false):Text(text),Enabled(enabled) {cCUDATimeSpent.Start();}
  ~CTimeStamp()
  {
   float gpu_time=cCUDATimeSpent.Stop();
   if (Enabled==false) return;
   char str[255];
   snprintf(str,sizeof(str),"%.2f мс.",gpu_time);
   SYSTEM::PutMessageToConsole(Text+str);
  }
};

#endif
