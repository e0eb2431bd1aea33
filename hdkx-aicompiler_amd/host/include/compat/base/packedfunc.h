// Forwarding header: code written against the reference's include/base/packedfunc.h compiles against the host layer
// with -I<host>/include/compat -I<host>/include.
#pragma once
#include "kxc/packed_func.h"
