// The reference's include name (include/opfactory.hpp of Graylatzhou/Infer): code written against it
// compiles against this tree unchanged.  Everything lives in infer_kv/operator.hpp.
#pragma once
#include "infer_kv/operator.hpp"
