// Raw file <-> device buffer (ioutils.cu:3-45): no header, bytes as they lie in device memory.
#pragma once
#include <string>
using std::string;

void savebin(const string& filename, const void* gpudata, size_t size);
size_t findsize(const string& filename);
void loadbin(const string& filename, void* gpudata, size_t size);
