// lib/acc_compile_worker: the helper process a thread of libacchip's compilation pool keeps, so that the kernels of a
// program compile side by side (hiprtc takes one program at a time per process).  It reads requests from its
// descriptor 0 until that closes; it never touches the device.
extern "C" int acc_compile_worker_main(int fd);
int main() { return acc_compile_worker_main(0); }
