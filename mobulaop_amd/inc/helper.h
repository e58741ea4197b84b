// Operator sources written for MobulaOP include this name; everything is in
// mobula_op.h.
#pragma once
#include "mobula_op.h"
