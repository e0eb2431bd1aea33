// Forwarding header: code written against the reference's include/codegen/codegen_c.h compiles against the host layer
// with -I<host>/include/compat -I<host>/include.
#pragma once
#include "kxc/codegen.h"
