// The kernel library's C ABI, reachable from the host headers' own include directory: a caller of the class API adds
// only msnhnet_amd/host/include to its include path, as it would add the reference's include/ directory.
#include "../../../include/msnh_hip.h"
