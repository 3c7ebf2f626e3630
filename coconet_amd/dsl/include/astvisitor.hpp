// Present so that programs written against the reference, which include <astvisitor.hpp>, compile unchanged.
// This front end walks its IR with plain recursive functions (see src/dsl.cpp), so there is no visitor API.
#ifndef COCONET_AMD_ASTVISITOR_HPP
#define COCONET_AMD_ASTVISITOR_HPP
#include "dsl.hpp"
#endif
