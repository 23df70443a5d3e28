// Constants a PTO kernel source may name (reference: include/pto/common/constants.hpp).
#pragma once
#include "../amd/base.hpp"
