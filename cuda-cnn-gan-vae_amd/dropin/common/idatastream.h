// Stream interface CTensor::Save/Load are written against (same names as the reference's common/idatastream.h;
// a build inside the reference tree uses the reference's own header instead, the guard is the same).
#ifndef I_DATA_STREAM_H
#define I_DATA_STREAM_H

#include <stdint.h>
#include <string>

class IDataStream
{
 public:
  virtual ~IDataStream() {}
  virtual int8_t LoadInt8(void)=0;
  virtual int16_t LoadInt16(void)=0;
  virtual int32_t LoadInt32(void)=0;
  virtual uint8_t LoadUInt8(void)=0;
  virtual uint16_t LoadUInt16(void)=0;
  virtual uint32_t LoadUInt32(void)=0;
  virtual float LoadFloat(void)=0;
  virtual double LoadDouble(void)=0;
  virtual void SaveFloat(float value)=0;
  virtual void SaveDouble(double value)=0;
  virtual void SaveInt8(int8_t value)=0;
  virtual void SaveInt16(int16_t value)=0;
  virtual void SaveInt32(int32_t value)=0;
  virtual void SaveUInt8(int8_t value)=0;
  virtual void SaveUInt16(int16_t value)=0;
  virtual void SaveUInt32(int32_t value)=0;
  virtual bool IsFail(void) const=0;
};

#endif
