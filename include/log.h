#pragma once
// Verbosity switch of the generator (reference: include/log.h:3-11, same names).  At Debug the driver dumps the
// IR after every rewrite step and echoes the generated source; Release prints nothing.  The level is one
// process-wide variable, KCGLog::level, defined in the driver.

enum Log { Debug = 0, Release = 1 };

namespace KernelCodeGen {

struct KCGLog {
  static Log level;
  static bool debug() { return level == Debug; }
};

}  // namespace KernelCodeGen
