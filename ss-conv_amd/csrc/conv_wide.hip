// The plain convolution kernel on float rows over a plan of the five-group form (conv_instances.h).
#include "conv_instances.h"

SSC_CONV_INSTANCES(false, 3)
