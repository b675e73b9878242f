#pragma once
// Gradient checks for user-defined op logic and whole graphs: the per-case
// functions usable inside kernels (gradient_check.cuh) and the batch testers
// with the reference's class names (UnaryGradientTester, BinaryGradientTester,
// NetworkGradientTester).  None of them needs a test framework.
#include <xyz_autodiff/testing/gradient_check.cuh>
#include <xyz_autodiff/testing/gradient_report.cuh>
#include <xyz_autodiff/testing/unary_gradient_tester.cuh>
#include <xyz_autodiff/testing/binary_gradient_tester.cuh>
#include <xyz_autodiff/testing/network_gradient_tester.cuh>
