#pragma once
// Gradient-check helpers for user-defined op logic.
#include <xyz_autodiff/testing/gradient_check.cuh>
