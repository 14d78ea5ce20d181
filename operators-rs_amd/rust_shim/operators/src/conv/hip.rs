im2col!(hip, Hip);
