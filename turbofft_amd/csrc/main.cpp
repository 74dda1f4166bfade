// The `turbofft` executable (the reference's main(), main.cu:137-169).
#include "../../include/turbofft.h"
int main(int argc, char** argv) { return turbofft_main(argc, argv); }
