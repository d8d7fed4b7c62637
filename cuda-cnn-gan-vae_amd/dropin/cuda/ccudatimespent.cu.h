#ifndef C_CUDA_TIME_SPENT_CU_H
#define C_CUDA_TIME_SPENT_CU_H

// Drop-in for the reference's interval timer (cuda/ccudatimespent.cu.h:20-40, cuda/ccudatimespent.cu:9-52) over the
// C ABI of libmi355tensor: Start() marks the work stream, Stop() marks it again, waits and returns the milliseconds
// the queued work took in between.  Header-only: there is no ccudatimespent.cu to compile.

#include "mi355_tensor.h"
#include "copqueue.cu.h"

class CCUDATimeSpent
{
 private:
  void *Timer;
  CCUDATimeSpent(const CCUDATimeSpent&);
  CCUDATimeSpent& operator=(const CCUDATimeSpent&);
 public:
  CCUDATimeSpent(void):Timer(0) {mt_timer_create(&Timer);}
  ~CCUDATimeSpent() {mt_timer_destroy(Timer);}
  // calls that the tensor classes have deferred belong to the side of the mark on which they were made
  void Start(void) {mi355::Queue().Flush();if (Timer!=0) mt_timer_start(Timer);}
  float Stop(void)
  {
   float gpu_time=0;
   mi355::Queue().Flush();
   if (Timer!=0) mt_timer_stop(Timer,&gpu_time);
   return(gpu_time);
  }
};

#endif
