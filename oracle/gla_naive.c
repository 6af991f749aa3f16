/* C restatement of the reference's recurrent_gla_naive (gla.py:26-47) and of the two-sweep
 * gradient scheme of its recurrent backward (gla.py:297-359, 263), in fp32 and fp64.
 *
 * TEST INFRASTRUCTURE ONLY.  Loaded through ctypes by oracle/naive_c.py for the parity tests at
 * full benchmark shapes and for bench.py's cpu_baseline leg; the shipped library never links it.
 * Build: make -C oracle   (gcc -O3 -fopenmp).  Pinned against oracle/gla_oracle.py, which is in
 * turn pinned by closed forms and torch.autograd (tests/test_oracle.py). */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define REAL float
#define SUFFIX f32
#define EXP expf
#include "gla_naive_impl.h"
#undef REAL
#undef SUFFIX
#undef EXP

#define REAL double
#define SUFFIX f64
#define EXP exp
#include "gla_naive_impl.h"
#undef REAL
#undef SUFFIX
#undef EXP

int gla_naive_abi_version(void) { return 1; }
