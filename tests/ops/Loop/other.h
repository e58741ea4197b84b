#ifndef TESTS_OPS_LOOP_OTHER_H_
#define TESTS_OPS_LOOP_OTHER_H_

extern const int kLoopAnswer;
#include "Loop.cpp"
inline int answer_from_header() { return kLoopAnswer; }

#endif  // TESTS_OPS_LOOP_OTHER_H_
