// Same include path as the reference's header of this name; everything lives in origin/tensor.h here.
#pragma once
#include "origin/tensor.h"
