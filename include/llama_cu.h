// Drop-in name for programs written against eiz/llama.cu's llama_cu.h: the public interface
// (namespace llama_cu) lives in llama_cu_host.hpp, the C ABI of the GPU layer in llama_cu_hip.h.
#pragma once
#include "llama_cu_host.hpp"
