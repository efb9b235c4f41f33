// Symbol visibility of the host library (the reference's export.h: include/export.h).
#pragma once
#define CS_API __attribute__((visibility("default")))
