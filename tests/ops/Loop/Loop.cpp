// Test input: a source and a header that include each other (guards on both).
#ifndef TESTS_OPS_LOOP_CPP_
#define TESTS_OPS_LOOP_CPP_

#include "other.h"

const int kLoopAnswer = 1234;

MOBULA_FUNC int loop_answer() { return answer_from_header(); }

#endif  // TESTS_OPS_LOOP_CPP_
