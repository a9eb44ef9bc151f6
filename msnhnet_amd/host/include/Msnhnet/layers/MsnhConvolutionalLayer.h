// ConvolutionalLayer is declared in MsnhLayers.h together with the other layers of the convolutional path.
#pragma once
#include "Msnhnet/layers/MsnhLayers.h"
