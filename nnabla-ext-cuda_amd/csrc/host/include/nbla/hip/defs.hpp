#pragma once
#define NBLA_HIP_API __attribute__((visibility("default")))
