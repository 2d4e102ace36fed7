// Same include path as the reference's header of this name; everything lives in origin/nn.h here.
#pragma once
#include "origin/nn.h"
