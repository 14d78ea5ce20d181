impl_op!(hip, Hip);
