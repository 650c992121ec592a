// The convolution kernel on float rows in its five-group form (conv_instances.h).
#include "conv_instances.h"

SSC_CONV_INSTANCES(false, 2)
