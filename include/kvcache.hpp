// The reference's include name (include/kvcache.hpp of Graylatzhou/Infer): code written against it
// compiles against this tree unchanged.  Everything lives in infer_kv/kvcache.hpp.
#pragma once
#include "infer_kv/kvcache.hpp"
