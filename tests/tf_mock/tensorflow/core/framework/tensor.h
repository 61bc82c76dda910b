// NOT TensorFlow: see mock_core.h
#include "tensorflow/core/framework/mock_core.h"
