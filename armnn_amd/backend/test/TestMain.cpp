#include "MiniTest.hpp"
int main(int argc, char** argv) { return minitest::Run(argc, argv); }
