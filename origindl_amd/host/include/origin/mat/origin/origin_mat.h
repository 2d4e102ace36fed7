// Same include path as the reference's header of this name; everything lives in origin/mat.h here.
#pragma once
#include "origin/mat.h"
