// Forwarding header: code written against the reference's include/te/topi/nn.h compiles against the host layer
// with -I<host>/include/compat -I<host>/include.
#pragma once
#include "kxc/topi.h"
