#pragma once
// Enumerations shared by the Frontend, the Optimizer and the Backend; values
// follow the reference (include/enum.h:5-29) because MemorySpace is stored as
// the integer memory space of memref types.

namespace KernelCodeGen {

enum class Target {
  CUDA = 0,
  ROCm = 1,
};

enum class MemorySpace {
  global = 1,
  shared = 2,
  local = 3,
  constant = 4,
  unallocated = 5,
  inplace = 6,
};

enum class Position {
  before = 0,
  after = 1,
  begin = 2,
  end = 3,
};

enum class Layout {
  rowMajor = 0,
  colMajor = 1,
};

}  // namespace KernelCodeGen
