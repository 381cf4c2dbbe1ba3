// Shared by the C++ tests of this folder: the PASSED/FAILED line of the reference's tests
// (test/threshold.cpp:9-15) and a GPU-presence gate.
#pragma once
#include <iostream>
#include <comprex_gfx950.h>

inline int print_pass(int errors) {
    if (errors == 0) std::cout << "+++ PASSED +++" << std::endl;
    else {
        std::cout << "--- FAILED ---" << std::endl;
        std::cout << "with " << errors << " errors." << std::endl;
    }
    return errors;
}

inline bool need_gpu() {
    if (cx_device_count() < 1) {
        std::cout << "no GPU: these tests drive the HIP library and cannot run here" << std::endl;
        return false;
    }
    return true;
}
