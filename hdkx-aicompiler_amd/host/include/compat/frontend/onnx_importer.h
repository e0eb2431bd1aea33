// Forwarding header: code written against the reference's include/frontend/onnx_importer.h compiles against the host layer
// with -I<host>/include/compat -I<host>/include.
#pragma once
#include "kxc/onnx_importer.h"
