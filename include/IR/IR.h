#pragma once
// Umbrella include of the IR layer (the reference's include/IR/IR.h pulls in
// the external MLIR tree here; this build carries its own affine IR).
#include "IR/MLIR.h"
