// Umbrella header.
#pragma once
#include "Msnhnet/net/MsnhNetBuilder.h"
