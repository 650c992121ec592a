// The plain convolution kernel with the epilogue on float rows over a plan of the five-group form (conv_instances.h).
#include "conv_instances.h"

SSC_CONV_INSTANCES(true, 3)
