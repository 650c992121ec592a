// The convolution kernel on float rows with the epilogue (conv_instances.h).
#include "conv_instances.h"

SSC_CONV_INSTANCES(true, 0)
