// The convolution kernel on float rows in its one-column-group form with the epilogue (conv_instances.h).
#include "conv_instances.h"

SSC_CONV_INSTANCES(true, 1)
