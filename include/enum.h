#pragma once
// Small value sets shared by the Frontend, the Optimizer and the Backend.  Names and numeric values are the
// reference's (include/enum.h:5-29): a program written against it compiles unchanged, and MemorySpace is stored
// as the integer memory space of memref types, so the numbers are part of the IR.

namespace KernelCodeGen {

// Platform a generator emits for.  Only ROCm has a backend here; CUDA is kept so that reference code naming it
// still compiles and gets a clean "unsupported platform" error at codegen().
enum class Target : int { CUDA = 0, ROCm = 1 };

// Where a buffer lives.  `inplace` marks an operand that the operation overwrites with its result.
enum class MemorySpace : int { global = 1, shared = 2, local = 3, constant = 4, unallocated = 5, inplace = 6 };

// Insertion points of the Rewriter primitives relative to an operation (before / after it) or to a region
// (at its begin / end).
enum class Position : int { before = 0, after = 1, begin = 2, end = 3 };

// Storage order of a matrix operand.
enum class Layout : int { rowMajor = 0, colMajor = 1 };

inline const char* toString(MemorySpace space) {
  switch (space) {
    case MemorySpace::global: return "global";
    case MemorySpace::shared: return "shared";
    case MemorySpace::local: return "local";
    case MemorySpace::constant: return "constant";
    case MemorySpace::unallocated: return "unallocated";
    case MemorySpace::inplace: return "inplace";
  }
  return "?";
}

inline const char* toString(Layout layout) { return layout == Layout::rowMajor ? "rowMajor" : "colMajor"; }

}  // namespace KernelCodeGen
