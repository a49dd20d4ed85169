#pragma once
// Two-level log switch (reference: include/log.h:3-11).  Debug dumps the IR
// after every rewrite step and echoes generated source.

enum Log {
  Debug = 0,
  Release = 1,
};

namespace KernelCodeGen {
struct KCGLog {
  static Log level;
};
}  // namespace KernelCodeGen
