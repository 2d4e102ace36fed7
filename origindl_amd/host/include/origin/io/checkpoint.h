// Same include path as the reference's header of this name; everything lives in origin/io.h here.
#pragma once
#include "origin/io.h"
#include "origin/nn.h"
