// <rocwmma/internal/io_layout.hpp> is an implementation detail of the reference library that this
// gfx950-native implementation does not reproduce (fragments are plain register arrays in MFMA
// operand order; there are no cross-lane reorder passes).  Failing here is deliberate: without
// this file the include would silently resolve to the rocWMMA that ships with the toolchain.
#error "rocwmma/internal/io_layout.hpp has no counterpart in this implementation; use the public API in <rocwmma/rocwmma.hpp>"
