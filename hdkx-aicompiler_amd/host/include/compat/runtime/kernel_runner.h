// Forwarding header: code written against the reference's include/runtime/kernel_runner.h compiles against the host layer
// with -I<host>/include/compat -I<host>/include.
#pragma once
#include "kxc/runtime_session.h"
