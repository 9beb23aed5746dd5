/* Umbrella of the C target: the one public header of the library.  Install
 * include/mi355_qlinear.h on the header search path (or pass -Xcc -I<repo>/include). */
#include <mi355_qlinear.h>
