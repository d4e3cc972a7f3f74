// Forwarding header: lets sources written against the reference header name compile against this library unchanged.
#pragma once
#include "../zkrelu.hpp"
