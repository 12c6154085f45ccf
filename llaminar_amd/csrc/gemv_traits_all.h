// All weight-format traits of the decode-GEMV skeleton.
#pragma once
#include "gemv_traits_q4k.h"
#include "gemv_traits_q6k.h"
#include "gemv_traits_iq3s.h"
