// The two console helpers the tensor classes use (reference: system/system.h:42-43).
#ifndef SYSTEM_H
#define SYSTEM_H

#include <string>

namespace SYSTEM
{
 void PutMessage(const std::string &message);
 void PutMessageToConsole(const std::string &message);
}

#endif
