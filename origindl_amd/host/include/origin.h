// Umbrella header, as the reference's include/origin.h.
#pragma once
#include "origin/base.h"
#include "origin/mat.h"
#include "origin/tensor.h"
#include "origin/functional.h"
#include "origin/nn.h"
#include "origin/pnnx/pnnx_graph.h"
