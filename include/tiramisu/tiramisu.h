// Umbrella header of the Tiramisu front-end (reference: include/tiramisu/tiramisu.h:1-9).
#ifndef TIRAMISU_AMD_TIRAMISU_H
#define TIRAMISU_AMD_TIRAMISU_H
#include <tiramisu/debug.h>
#include <tiramisu/type.h>
#include <tiramisu/expr.h>
#include <tiramisu/core.h>
#include <tiramisu/block.h>
#include <tiramisu/macros.h>
#endif
