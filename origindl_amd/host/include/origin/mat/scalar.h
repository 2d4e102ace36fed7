// Same include path as the reference's header of this name; everything lives in origin/base.h here.
#pragma once
#include "origin/base.h"
