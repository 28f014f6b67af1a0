// command line entry point (the reference's main.cpp:3-7 does the same two lines)
#include "llava_context.h"

int main(int argc, char **argv)
{
    llava_context context;
    return context.run(argc, argv);
}
