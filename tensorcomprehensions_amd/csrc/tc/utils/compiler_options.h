// Front-end behaviour switches (counterpart of tc/utils/compiler_options.h:27-37).
#pragma once
namespace tc {
struct CompilerOptions {
  bool emitWarnings = true;   // print warnings to stderr
  bool throwWarnings = false; // turn warnings into exceptions
};
} // namespace tc
