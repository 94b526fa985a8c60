// Named by the API this front end mirrors and not provided by it.  The header exists so that
// including it stops the build here, instead of the compiler picking up a file of the same name
// from another Thrust installation on its include path and mixing two implementations.
#pragma once
#error "thrust::random::linear_feedback_shift_engine is not provided by this Thrust front end (the linear congruential engines and the three distributions are: thrust/random.h)"
