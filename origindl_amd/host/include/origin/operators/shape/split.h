// Same include path as the reference's header of this name; everything lives in origin/functional.h here.
#pragma once
#include "origin/functional.h"
