// Forwarding header: keeps the include path of the fbcuda sources working.
#pragma once
#include "../../fbfft_amd.hpp"
