// Device-side scalar helpers shared with the PTO header layer live with it.
#pragma once
#include "../include/pto/amd/device_types.hpp"
