#ifndef __NVM_RPC_H__
#define __NVM_RPC_H__
#include "nvm_aq.h"
#endif
