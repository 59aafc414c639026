// Enumerations shared by the host classes; values and order follow the
// reference (types.h:4-21) so that numeric codes written by existing drivers
// keep their meaning.
#pragma once
#include <stdint.h>

enum batchType { TRAINBATCH, TESTBATCH, UNLABELEDBATCH, RESCALEBATCH };
extern const char *batchTypeNames[];

enum ActivationFunction {
  NOSIGMOID,
  RELU,
  VLEAKYRELU,
  LEAKYRELU,
  TANH,
  SOFTMAX,
  PRELU,
  SIGMOID
};
extern const char *sigmoidNames[];

// multiply-accumulate operations of the NiN contractions since the last reset
// (types.h:46-52); processDataset prints it.
extern __int128_t multiplyAddCount;
// (forward passes may be queued from more than one host thread)
void addMultiplyAdds(__int128_t n);
